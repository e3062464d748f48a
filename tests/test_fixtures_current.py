"""The committed oracle outcomes under tests/golden/ (whole decode horizons, the teacher-forced forward, the
configuration-5 prefill logits) took minutes to an hour of CPU each, so the GPU tests compare against the files and
not against a live oracle run.  These tests tie every one of them to the oracle as it is NOW: the first steps (or
positions) of each file are derived again from the current oracle and the current weight / token generators and
must reproduce the stored ids and logits.  An edit of the oracle or of a generator that changes results fails here
instead of leaving a stale fixture behind.  CPU only.
"""
import os

import numpy as np
import pytest

from conftest import GOLDEN


def _rederive_horizon(orc, w, prompt, g, steps=3, prefix=""):
    """Steps 0..steps-1 of a horizon file through the full recompute over prompt + the file's own ids (the
    files were written by the cached decoder: cached == full recompute is pinned in test_oracle_pins.py)."""
    ids, top_idx, top_val = g[prefix + "ids"], g[prefix + "top_idx"], g[prefix + "top_val"]
    keep = {int(s): i for i, s in enumerate(g[prefix + "full_steps"])}
    for i in range(steps):
        toks = np.concatenate([prompt, ids[:i]]).astype(np.int32)
        lg = orc.forward_full(w, toks, "f64")["logits"][0]
        assert int(np.argmax(lg)) == int(ids[i]), f"step {i}: the oracle now picks another token"
        assert np.array_equal(np.argsort(-lg, kind="stable")[:4], top_idx[i])
        assert np.allclose(lg[top_idx[i]], top_val[i], rtol=1e-10, atol=1e-13)
        if i in keep:
            assert np.allclose(lg, g[prefix + "full_logits"][keep[i]], rtol=1e-5, atol=1e-7)  # rows are stored as float32


def test_horizon_cfg3_file_is_current(pkg, orc):
    g = np.load(os.path.join(GOLDEN, "horizon_cfg3_golden.npz"))
    hp = pkg.config(3)
    prompt = pkg.random_tokens(3, 0, hp.vocabSize, 128)
    assert np.array_equal(prompt, g["prompt"])
    _rederive_horizon(orc, orc.Weights.from_model(pkg.Model.generate(hp, 3)), prompt, g)


def test_horizon_cfg2_flags_file_is_current(pkg, orc):
    g = np.load(os.path.join(GOLDEN, "horizon_cfg2_flags_golden.npz"))
    hp = pkg.config(2, qkRmsNorm=1, queryGating=1)
    prompt = pkg.random_tokens(1, 0, hp.vocabSize, 64)
    assert np.array_equal(prompt, g["prompt"])
    _rederive_horizon(orc, orc.Weights.from_model(pkg.Model.generate(hp, 1)), prompt, g)


def test_horizon_cfg4_file_is_current(pkg, orc):
    g = np.load(os.path.join(GOLDEN, "horizon_cfg4_golden.npz"))
    hp = pkg.config(4)
    lens = np.random.default_rng(44).integers(32, 513, size=hp.maxSeqs)
    assert np.array_equal(lens, g["lens"])
    w = orc.Weights.from_model(pkg.Model.generate(hp, 4))
    for s in g["seqs"]:
        prompt = pkg.random_tokens(44, int(s), hp.vocabSize, int(lens[s]))
        _rederive_horizon(orc, w, prompt, g, prefix=f"s{int(s)}_")


@pytest.fixture(scope="module")
def refdefault(pkg, orc):
    hp = pkg.reference_defaults()
    model = pkg.Model.new(hp)
    model.init_uniform(9, 0.02)
    return hp, orc.Weights.from_model(model)


def test_horizon_refdefault_file_is_current(pkg, orc, refdefault):
    hp, w = refdefault
    g = np.load(os.path.join(GOLDEN, "horizon_refdefault_golden.npz"))
    prompt = pkg.random_tokens(9, 0, hp.vocabSize, 256)
    assert np.array_equal(prompt, g["prompt"])
    _rederive_horizon(orc, w, prompt, g)


def test_forward_refdefault_file_is_current(pkg, orc, refdefault):
    """Positions 0..2 and 63, 64 of the 1280-position teacher-forced forward, from prefixes (causality makes the
    columns of a prefix equal to the same columns of the whole pass)."""
    hp, w = refdefault
    g = np.load(os.path.join(GOLDEN, "forward_refdefault_golden.npz"))
    toks = pkg.random_tokens(91, 0, hp.vocabSize, hp.maxL)
    assert np.array_equal(toks, g["tokens"])
    r = orc.forward_full(w, toks[:65], "f64", last_only=False, want_probs=True)
    lg, pr = r["logits"], r["probs"]
    for p in (0, 1, 2, 63, 64):
        assert np.array_equal(np.argsort(-lg[p], kind="stable")[:2], g["top_idx"][p])
        assert np.allclose(lg[p][g["top_idx"][p]], g["top_val"][p], rtol=1e-10, atol=1e-13)
        assert np.isclose(pr[p].max(), g["p_max"][p], rtol=1e-10)
        if p < 64:
            assert np.isclose(pr[p, toks[p + 1]], g["p_next"][p], rtol=1e-10)
    rows = {int(r_): i for i, r_ in enumerate(g["rows"])}
    for p in (0, 63, 64):
        assert np.allclose(lg[p], g["row_logits"][rows[p]], rtol=1e-5, atol=1e-7)
        assert np.allclose(pr[p], g["row_probs"][rows[p]], rtol=1e-5, atol=1e-10)


def test_cfg5_files_are_current(pkg, orc):
    """Configuration 5 at full size (1.3 G parameters, bf16-rounded): the prefill file at prompts of 1, 64 and 65
    tokens, and step 0 of the decode horizon (one full recompute over its 2048-token prompt: the slow part, a few
    minutes on eight cores)."""
    g = np.load(os.path.join(GOLDEN, "cfg5_prefill_golden.npz"))
    hp = pkg.config(5, maxSeqs=1)
    model = pkg.Model.generate(hp, seed=5)
    assert np.array_equal(model.tensor(0, 0)[:4, :8], g["embedding_head"])
    toks = pkg.random_tokens(5, 0, hp.vocabSize, 2048)
    assert np.array_equal(toks, g["tokens"])
    w = orc.Weights.from_model(model, bf16=True)
    pos = {int(p): i for i, p in enumerate(g["positions"])}
    for p in (0, 63, 64):
        lg = orc.forward_full(w, toks[:p + 1], "f64")["logits"][0]
        assert np.allclose(lg, g["logits"][pos[p]], rtol=1e-5, atol=1e-7)
    h = np.load(os.path.join(GOLDEN, "horizon_cfg5_golden.npz"))
    prompt = pkg.random_tokens(55, 0, hp.vocabSize, 2048)
    assert np.array_equal(prompt, h["prompt"])
    _rederive_horizon(orc, w, prompt, h, steps=1)
