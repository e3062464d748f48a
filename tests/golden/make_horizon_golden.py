#!/usr/bin/env python3
"""Writes horizon_cfg{3,4,5}_golden.npz, horizon_cfg2_flags_golden.npz, horizon_refdefault_golden.npz and forward_refdefault_golden.npz: the FULL decode horizons of configurations
3, 4 and 5 (the benchmark workloads), and a long one at the shape the reference ships compiled in, through the float64 CPU oracle, one token at a time with its cache -- too slow to repeat inside a test
(config 5: half an hour), so the outcome is kept: the oracle's greedy ids, its four best logits at every step, and
complete logit rows (float32) at a few steps.

  config 3  seed 3, 128-token prompt, 1024 greedy steps
  config 4  seed 4, 64 prompts uniform in [32, 512] (numpy default_rng(44)); the shortest, a middle and the longest
            sequence, 256 greedy steps each
  config 5  seed 5, bf16-rounded weights, sequence 0 of the 8 x 2048-token prompts (seed 55), 128 greedy steps
  2         configuration 2 with BOTH architecture flags on (QK-norm, query gating: the reference's shipped setting,
            network_meta.h:19-20), seed 1, 64-token prompt, 512 greedy steps
  1         the reference's compiled-in shape, teacher-forced: one random 1280-token sequence (maxL) through the full
            recompute as the reference's runInference(L) does it -- per position the best two logits, the probability of
            the token that follows (clamped at 1e-4 as training_orchestrator.cu:343-347 does) and complete rows at a few
            positions (forward_refdefault_golden.npz)
  0         the reference's compiled-in shape (network_meta.h:3-20: dim 768, 6 heads x 128, ffn 3072, 16 layers,
            vocabulary 20160, QK-norm and query gating on, maxL 1280), uniform +-0.02 weights from seed 9
            (random_weights.cu:15-25; own generator), a 256-token prompt and 1024 greedy steps: the cache filled to maxL

Run from the repository root: python tests/golden/make_horizon_golden.py 0|1|2|3|4|5"""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def greedy(orc, w, prompt, steps, keep):
    """ids[0] follows the prompt; row i of top_idx / top_val and logits[i] (i in keep) decide ids[i]."""
    dec = orc.Decoder(w, "f64")
    lg = None
    t0 = time.time()
    for k, t in enumerate(prompt):
        _, lg = dec.step(int(t), want_logits=(k == len(prompt) - 1))
    print(f"  prompt of {len(prompt)}: {time.time() - t0:.0f} s", flush=True)
    ids, top_idx, top_val, full = [], [], [], {}
    for i in range(steps + 1):
        order = np.argsort(-lg, kind="stable")[:4]
        top_idx.append(order)
        top_val.append(lg[order])
        if i in keep:
            full[i] = lg.astype(np.float32)
        ids.append(int(order[0]))
        if i < steps:
            _, lg = dec.step(ids[-1])
    dec.close()
    print(f"  {steps} steps: {time.time() - t0:.0f} s, distinct ids {len(set(ids))}", flush=True)
    return dict(ids=np.array(ids, dtype=np.int32), top_idx=np.array(top_idx, dtype=np.int32),
                top_val=np.array(top_val, dtype=np.float64), full_steps=np.array(sorted(keep), dtype=np.int32),
                full_logits=np.stack([full[s] for s in sorted(keep)]))


def main(which):
    m, orc = entry.load_package(), entry.load_oracle()
    if which == 3:
        hp = m.config(3)
        model = m.Model.generate(hp, 3)
        prompt = m.random_tokens(3, 0, hp.vocabSize, 128)
        r = greedy(orc, orc.Weights.from_model(model), prompt, 1024, (0, 1, 255, 256, 511, 767, 1024))
        np.savez_compressed(os.path.join(HERE, "horizon_cfg3_golden.npz"), prompt=prompt.astype(np.int32), **r)
    elif which == 4:
        hp = m.config(4)
        model = m.Model.generate(hp, 4)
        w = orc.Weights.from_model(model)
        lens = np.random.default_rng(44).integers(32, 513, size=hp.maxSeqs)
        order = np.argsort(lens)
        out = {"lens": lens.astype(np.int32)}
        seqs = [int(order[0]), int(order[hp.maxSeqs // 2]), int(order[-1])]
        out["seqs"] = np.array(seqs, dtype=np.int32)
        for s in seqs:
            prompt = m.random_tokens(44, s, hp.vocabSize, int(lens[s]))
            for k, v in greedy(orc, w, prompt, 256, (0, 128, 256)).items():
                out[f"s{s}_{k}"] = v
        np.savez_compressed(os.path.join(HERE, "horizon_cfg4_golden.npz"), **out)
    elif which == 5:
        hp = m.config(5)
        model = m.Model.generate(hp, 5)
        prompt = m.random_tokens(55, 0, hp.vocabSize, 2048)
        r = greedy(orc, orc.Weights.from_model(model, bf16=True), prompt, 128, (0, 64, 128))
        np.savez_compressed(os.path.join(HERE, "horizon_cfg5_golden.npz"), prompt=prompt.astype(np.int32), **r)
    elif which == 2:
        hp = m.config(2, qkRmsNorm=1, queryGating=1)
        model = m.Model.generate(hp, 1)
        prompt = m.random_tokens(1, 0, hp.vocabSize, 64)
        r = greedy(orc, orc.Weights.from_model(model), prompt, 512, (0, 1, 64, 65, 200, 383, 512))
        np.savez_compressed(os.path.join(HERE, "horizon_cfg2_flags_golden.npz"), prompt=prompt.astype(np.int32), **r)
    elif which == 1:
        hp = m.reference_defaults()
        model = m.Model.new(hp)
        model.init_uniform(9, 0.02)
        toks = m.random_tokens(91, 0, hp.vocabSize, hp.maxL)
        t0 = time.time()
        ref = orc.forward_full(orc.Weights.from_model(model), toks, "f64", last_only=False, want_probs=True)
        print(f"  full recompute of {hp.maxL} tokens: {time.time() - t0:.0f} s", flush=True)
        lg, pr = ref["logits"], ref["probs"]
        order = np.argsort(-lg, axis=1, kind="stable")[:, :2]
        rows = (0, 63, 64, 639, hp.maxL - 1)
        np.savez_compressed(os.path.join(HERE, "forward_refdefault_golden.npz"), tokens=toks.astype(np.int32),
                            top_idx=order.astype(np.int32), top_val=np.take_along_axis(lg, order, axis=1),
                            p_next=pr[np.arange(hp.maxL - 1), toks[1:]], p_max=pr.max(axis=1),
                            rows=np.array(rows, dtype=np.int32), row_logits=lg[list(rows)].astype(np.float32),
                            row_probs=pr[list(rows)].astype(np.float32))
    elif which == 0:
        hp = m.reference_defaults()
        model = m.Model.new(hp)
        model.init_uniform(9, 0.02)
        prompt = m.random_tokens(9, 0, hp.vocabSize, 256)
        r = greedy(orc, orc.Weights.from_model(model), prompt, hp.maxL - 256, (0, 1, 255, 256, 700, hp.maxL - 256))
        np.savez_compressed(os.path.join(HERE, "horizon_refdefault_golden.npz"), prompt=prompt.astype(np.int32), **r)
    else:
        raise SystemExit(__doc__)


if __name__ == "__main__":
    main(int(sys.argv[1]) if len(sys.argv) > 1 else -1)
