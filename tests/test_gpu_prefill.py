"""GPU parity of the GEMM prefill path (MFMA GEMMs + tiled causal attention + chunked GDN recurrence)
against the CPU oracle and against the token-by-token path, through the C ABI.

Tolerances as for decode: logits within 1e-3 relative (fp32 weights) and 2e-2 (bf16 weights, where the
GEMM inputs are additionally rounded to bf16).
"""
import numpy as np
import pytest

from conftest import assert_logits_close, check_greedy_against_oracle, rel_diff
from test_gpu_decode import small_cfg, make, FP32_RTOL, BF16_RTOL, GAP_TOL

pytestmark = pytest.mark.gpu


# ---- the GEMM by itself -------------------------------------------------------------------------
@pytest.mark.parametrize("m,n,k", [(128, 128, 32), (1, 1, 32), (17, 300, 96), (130, 257, 704), (64, 1160, 256),
                                   (300, 128, 2048), (257, 4096, 256), (40, 768, 2048), (64, 100, 1024), (24, 1600, 1024)])
def test_gemm_fp32(pkg, m, n, k):
    """C = A.B^T (+R) on the fp32 MFMA path against float64 NumPy; ragged M and N, K a multiple of 32."""
    rng = np.random.default_rng(m * 1000 + n + k)
    a = rng.standard_normal((m, k), dtype=np.float32)
    b = rng.standard_normal((n, k), dtype=np.float32)
    r = rng.standard_normal((m, n), dtype=np.float32)
    for res in (None, r):
        c, _ = pkg.selftest_gemm(a, b, res)
        c2, _ = pkg.selftest_gemm(a, b, res, iters=3)  # repeated launches on one workspace: split-K counters reset themselves
        assert np.array_equal(c, c2)
        want = a.astype(np.float64) @ b.astype(np.float64).T + (0 if res is None else res)
        err = np.max(np.abs(c - want))
        # fp32 products summed in fp32: error grows like sqrt(k) * eps * |a||b|
        assert err <= 4e-6 * np.sqrt(k) * np.max(np.abs(want)) + 1e-5, (m, n, k, err)


@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (1, 1, 64), (17, 300, 128), (130, 257, 704), (300, 128, 2048), (8, 2048, 5632), (33, 96, 512),
                                   (1100, 17000, 192), (300, 600, 64), (2000, 8256, 448)])
def test_gemm_bf16(pkg, orc, m, n, k):
    """bf16 operands (already representable, so the product is exact in fp32) with fp32 accumulation."""
    rng = np.random.default_rng(m * 1000 + n + k + 1)
    a = orc.round_bf16(rng.standard_normal((m, k), dtype=np.float32))
    b = orc.round_bf16(rng.standard_normal((n, k), dtype=np.float32))
    r = rng.standard_normal((m, n), dtype=np.float32)
    for res in (None, r):
        c, _ = pkg.selftest_gemm(a, b, res, bf16=True)
        want = a.astype(np.float64) @ b.astype(np.float64).T + (0 if res is None else res)
        err = np.max(np.abs(c - want))
        assert err <= 4e-6 * np.sqrt(k) * np.max(np.abs(want)) + 1e-5, (m, n, k, err)


@pytest.mark.parametrize("m,n,k", [(8, 2048, 5632), (130, 257, 704), (300, 4096, 2048), (1100, 17000, 192), (300, 600, 64), (2100, 9000, 448), (2048, 8256, 448)])
def test_gemm_f16(pkg, m, n, k):
    """IEEE-half operands (what the MFMA path of bf16 models multiplies) with fp32 accumulation.  The larger shapes
    give a workgroup of the 256 x 256-tile kernel several tiles (more than 256 tiles in all) with an odd and an even
    number of K slices, ragged edges in M and N, and a single-slice K; 8256 columns under 2048 rows is the case where
    the last, quarter-full column of tiles is split off into a launch of its own (8 x 33 tiles on 256 compute units)."""
    rng = np.random.default_rng(m + n + k)
    a = rng.standard_normal((m, k), dtype=np.float32).astype(np.float16).astype(np.float32)
    b = rng.standard_normal((n, k), dtype=np.float32).astype(np.float16).astype(np.float32)
    c, _ = pkg.selftest_gemm(a, b, None, f16=True)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    assert np.max(np.abs(c - want)) <= 4e-6 * np.sqrt(k) * np.max(np.abs(want)) + 1e-5


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("m,n,k", [(300, 512, 256), (257, 1000, 704), (130, 36, 128), (100, 256, 512), (64, 320, 256), (9, 128, 2048),
                                   (1100, 17000, 192)])
def test_gemm_swiglu_epilogue(pkg, orc, kind, m, n, k):
    """The gate/up epilogue (inference.cu:262-281) of all three tile families: columns 2j, 2j+1 of the product are
    gate and up of unit j, the result silu(gate) * up is stored in the operand type; ragged M, N/2 not a multiple
    of the store width."""
    rng = np.random.default_rng(m + 7 * n + k)
    a = (0.5 * rng.standard_normal((m, k))).astype(np.float32)
    b = (0.5 * rng.standard_normal((n, k)) / np.sqrt(k) * 8).astype(np.float32)
    if kind == "bf16":
        a, b = orc.round_bf16(a), orc.round_bf16(b)
    elif kind == "f16":
        a, b = a.astype(np.float16).astype(np.float32), b.astype(np.float16).astype(np.float32)
    c, _ = pkg.selftest_gemm(a, b, None, bf16=(kind == "bf16"), f16=(kind == "f16"), swiglu=True)
    assert c.shape == (m, n // 2)
    p = a.astype(np.float64) @ b.astype(np.float64).T
    want = p[:, 0::2] / (1 + np.exp(-p[:, 0::2])) * p[:, 1::2]
    tol = {"f32": 2e-5, "bf16": 2.0 ** -8, "f16": 2.0 ** -11}[kind]  # the result is rounded to the operand type
    assert np.max(np.abs(c - want)) <= tol * np.max(np.abs(want)) + 2e-5 * np.sqrt(k), (kind, m, n, k)


def test_gemm_rejects_bad_k(pkg):
    a = np.zeros((4, 40), dtype=np.float32)
    with pytest.raises(RuntimeError):
        pkg.selftest_gemm(a, a)


# ---- prefill ------------------------------------------------------------------------------------
@pytest.mark.parametrize("kind,plen", [("attn", 100), ("attn_flags", 77), ("hybrid", 130), ("hybrid_flags", 64),
                                       ("hd128", 150), ("attn_long", 333)])
def test_prefill_logits_vs_oracle_and_tokenwise(pkg, orc, kind, plen):
    """Last-position logits of a GEMM prefill against the float64 oracle's full forward and against the
    token-by-token path; then greedy decoding continues from the prefilled cache."""
    hp = small_cfg(pkg, kind)
    model, dev, w = make(pkg, orc, hp, seed=21)
    prompt = pkg.random_tokens(21, 0, hp.vocabSize, plen)
    want = orc.forward_full(w, prompt, "f64", last_only=True)["logits"][-1]
    dev.prefill(0, prompt)
    assert dev.seq_len(0) == plen
    got = dev.logits(0)
    assert_logits_close(got, want, FP32_RTOL, f"{kind} gemm prefill")
    tok = dev.greedy_token(0)
    ids = [tok]
    for _ in range(11):
        ids.append(int(dev.decode_step([ids[-1]])[0]))
    dec = orc.Decoder(w, "f64")
    exact, tol = check_greedy_against_oracle(dec, prompt, ids, GAP_TOL, what=kind)
    assert exact + tol == len(ids)
    # token-by-token through the decode kernels
    dev.reset()
    dev.set_prefill_mode(1)
    dev.prefill(0, prompt)
    assert_logits_close(dev.logits(0), want, FP32_RTOL, f"{kind} tokenwise prefill")
    assert_logits_close(got, dev.logits(0), FP32_RTOL, f"{kind} gemm vs tokenwise")
    dev.close()


@pytest.mark.parametrize("cfg,plen", [(2, 64), (2, 41), (3, 48)])
def test_prefill_rows_33_to_64_long_k(pkg, orc, cfg, plen):
    """33 to 64 rows take the 16-row fp32 kernel with the RMSNorm fused in and the token rows staged through LDS;
    at d = 768 / F = 2048 a wave of it walks several K chunks (the small shapes above give it one), and the
    down projection splits K over workgroups."""
    hp = pkg.config(cfg, transformers=4 if cfg == 3 else 2, maxL=128)
    if cfg == 3:
        pkg.set_layer_pattern(hp, 1)
    model, dev, w = make(pkg, orc, hp, seed=27)
    prompt = pkg.random_tokens(27, 0, hp.vocabSize, plen)
    want = orc.forward_full(w, prompt, "f64", last_only=True)["logits"][-1]
    dev.prefill(0, prompt)
    got = dev.logits(0)
    assert_logits_close(got, want, FP32_RTOL, f"config {cfg} shape, {plen} rows")
    dev.reset()
    dev.prefill(0, prompt)
    assert np.array_equal(dev.logits(0), got), "a repeated prefill from reset must be bit-identical"
    dev.close()


def test_prefill_in_pieces(pkg, orc):
    """A prompt appended in three calls (GEMM, GEMM, short token-by-token tail) gives the logits of one call."""
    hp = small_cfg(pkg, "hybrid_flags")
    model, dev, w = make(pkg, orc, hp, seed=22)
    prompt = pkg.random_tokens(22, 0, hp.vocabSize, 150)
    want = orc.forward_full(w, prompt, "f64", last_only=True)["logits"][-1]
    dev.prefill(0, prompt[:70])
    dev.prefill(0, prompt[70:141])
    dev.prefill(0, prompt[141:])
    assert dev.seq_len(0) == 150
    assert_logits_close(dev.logits(0), want, FP32_RTOL, "pieces")
    dev.close()


def test_prefill_batch_ragged(pkg, orc):
    """Several sequences of different lengths in one pass: each equals its own single prefill and the
    oracle; decoding the batch afterwards follows the oracle."""
    hp = small_cfg(pkg, "hybrid", maxSeqs=4)
    model, dev, w = make(pkg, orc, hp, seed=23)
    lens = [17, 64, 1, 131]
    prompts = [pkg.random_tokens(100 + i, 0, hp.vocabSize, n) for i, n in enumerate(lens)]
    dev.prefill_batch([2, 0, 3, 1], prompts)
    seqs = [2, 0, 3, 1]
    firsts = {}
    for s, p in zip(seqs, prompts):
        assert dev.seq_len(s) == len(p)
        want = orc.forward_full(w, p, "f64", last_only=True)["logits"][-1]
        assert_logits_close(dev.logits(s), want, FP32_RTOL, f"batch seq {s}")
        firsts[s] = dev.greedy_token(s)
        best = int(np.argmax(want))
        assert firsts[s] == best or want[best] - want[firsts[s]] <= GAP_TOL
    out = dev.decode_loop([firsts[s] for s in range(4)], 6)
    by_seq = {s: p for s, p in zip(seqs, prompts)}
    for s in range(4):
        ids = [firsts[s]] + [int(t) for t in out[:, s]]
        dec = orc.Decoder(w, "f64")
        exact, tol = check_greedy_against_oracle(dec, by_seq[s], ids, GAP_TOL, what=f"batch decode seq {s}")
        assert exact + tol == len(ids)
    dev.close()


def test_prefill_paged(pkg, orc):
    """A permuted page table changes nothing."""
    hp = small_cfg(pkg, "attn_long", maxSeqs=2)
    model, dev, w = make(pkg, orc, hp, seed=24)
    prompt = pkg.random_tokens(24, 0, hp.vocabSize, 200)
    dev.prefill(1, prompt)
    ref = dev.logits(1)
    dev.reset()
    n = ((hp.maxL + 63) // 64) * hp.maxSeqs
    perm = np.random.default_rng(3).permutation(n).astype(np.int32)
    dev.set_page_table(perm)
    dev.prefill(1, prompt)
    assert np.array_equal(ref, dev.logits(1))
    dev.close()


@pytest.mark.parametrize("kind,plen", [("attn_flags", 90), ("hybrid", 100), ("hd128", 199), ("attn_long", 333)])
def test_prefill_bf16(pkg, orc, kind, plen):
    """bf16 weights: the MFMA prefill multiplies exact fp16 mirrors of the bf16-rounded weights with
    activations rounded to fp16: within 2e-2 (stated) and 4e-3 (asserted) of the float64 oracle on the
    bf16-rounded weights, relative to the largest logit; likewise the token-by-token path (fp32 activations)."""
    hp = small_cfg(pkg, kind, weightDtype=pkg.DTYPE_BF16)
    model, dev, w = make(pkg, orc, hp, seed=25, bf16=True)
    prompt = pkg.random_tokens(25, 0, hp.vocabSize, plen)
    want = orc.forward_full(w, prompt, "f64", last_only=True)["logits"][-1]
    dev.prefill(0, prompt)
    got = dev.logits(0)
    floor = 1e-3 * np.max(np.abs(want))
    den = np.maximum(np.maximum(np.abs(got), np.abs(want)), floor)
    worst = float(np.max(np.abs(got - want) / den))
    scale_err = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
    print(f"{kind}: bf16 prefill worst rel {worst:.3e}, max|diff|/max|logit| {scale_err:.3e}")
    assert scale_err <= 4e-3 <= BF16_RTOL
    dev.reset()
    dev.set_prefill_mode(1)
    dev.prefill(0, prompt)
    scale_err2 = float(np.max(np.abs(dev.logits(0) - want)) / np.max(np.abs(want)))
    assert scale_err2 <= BF16_RTOL
    dev.close()


@pytest.mark.parametrize("kind", ["attn_flags", "hd128"])
def test_prefill_bf16_ragged_batch_both_attention_variants(pkg, orc, kind):
    """bf16 weights, several sequences of different lengths in one pass.  A call whose segments all start at position 0
    runs the attention on the half copies of K and V that the RoPE kernel writes (keys = rows of the call); a prompt
    appended in two calls reads the fp32 pages instead.  Both against the float64 oracle, the batch also against each
    sequence prefilled alone (other row offsets, and for the short ones other GEMM tile families)."""
    extra = {"maxL": 200} if kind == "attn_flags" else {}
    hp = small_cfg(pkg, kind, weightDtype=pkg.DTYPE_BF16, maxSeqs=5, **extra)
    model, dev, w = make(pkg, orc, hp, seed=41, bf16=True)
    lens = [37, 128, 1, 199, 65]
    seqs = [3, 0, 4, 1, 2]
    prompts = [pkg.random_tokens(300 + i, 0, hp.vocabSize, n) for i, n in enumerate(lens)]
    wants = [orc.forward_full(w, p, "f64", last_only=True)["logits"][-1] for p in prompts]
    dev.prefill_batch(seqs, prompts)
    batch = {s: dev.logits(s).copy() for s in seqs}
    for s, p, want in zip(seqs, prompts, wants):
        err = float(np.max(np.abs(batch[s] - want)) / np.max(np.abs(want)))
        assert err <= 4e-3 <= BF16_RTOL, ("batch", s, len(p), err)
    dev.reset()
    for s, p, want in zip(seqs, prompts, wants):  # alone
        dev.prefill(s, p)
        assert float(np.max(np.abs(dev.logits(s) - want)) / np.max(np.abs(want))) <= 4e-3, ("alone", s, len(p))
        assert float(np.max(np.abs(dev.logits(s) - batch[s])) / np.max(np.abs(want))) <= 4e-3, ("alone vs batch", s, len(p))
    dev.reset()
    for s, p, want in zip(seqs, prompts, wants):  # in two calls: the second one's keys start in the pages
        if len(p) < 40:
            continue
        cut = len(p) // 2 + 3
        dev.prefill(s, p[:cut])
        dev.prefill(s, p[cut:])
        err = float(np.max(np.abs(dev.logits(s) - want)) / np.max(np.abs(want)))
        assert err <= 4e-3, ("pieces", s, len(p), err)
        assert float(np.max(np.abs(dev.logits(s) - batch[s])) / np.max(np.abs(want))) <= 4e-3
    dev.close()


# ---- batched decode through the skinny GEMM ------------------------------------------------------
@pytest.mark.parametrize("kind,nseq,graph", [("hybrid", 8, 0), ("hybrid_flags", 13, 1), ("hybrid_flags", 20, 0), ("attn_long", 33, 0), ("hd128", 64, 2)])
def test_batched_decode_gemm_path(pkg, orc, kind, nseq, graph):
    """Eight or more sequences per step take the MFMA path (skinny GEMMs + decode attention/GDN kernels):
    ids and final logits against the float64 oracle, per sequence, with ragged prompt lengths; the same
    run through the GEMV kernels (mode 1) must agree within the fp32 tolerance.  From 16 sequences on one attention
    workgroup holds all keys of a (head, sequence) pair and writes the gated output rows itself; below that the
    split-KV partials go through the combine kernel -- the flags case runs both ways."""
    hp = small_cfg(pkg, kind, maxSeqs=nseq)
    model, dev, w = make(pkg, orc, hp, seed=31)
    dev.set_graph(graph)
    rng = np.random.default_rng(nseq)
    lens = rng.integers(1, 90, size=nseq)
    prompts = [pkg.random_tokens(31, s, hp.vocabSize, int(n)) for s, n in enumerate(lens)]
    steps = 10
    res = {}
    for mode in (0, 1):
        dev.reset()
        dev.set_prefill_mode(mode)
        dev.prefill_batch(list(range(nseq)), prompts)
        firsts = [dev.greedy_token(s) for s in range(nseq)]
        out = dev.decode_loop(firsts, steps)
        res[mode] = (firsts, out.copy(), [dev.logits(s) for s in range(nseq)])
    firsts, out, logits = res[0]
    for s in range(0, nseq, max(1, nseq // 8)):  # a spread of sequences keeps the oracle time bounded
        dec = orc.Decoder(w, "f64")
        ids = [firsts[s]] + [int(t) for t in out[:, s]]
        exact, tol = check_greedy_against_oracle(dec, prompts[s], ids, GAP_TOL, what=f"{kind} seq {s}")
        assert exact + tol == len(ids)
        dec.reset()
        for t in list(prompts[s]) + ids[:-1]:
            _, lg = dec.step(int(t))
        assert_logits_close(logits[s], lg, FP32_RTOL, f"{kind} seq {s} final logits")
        assert_logits_close(logits[s], res[1][2][s], FP32_RTOL, f"{kind} seq {s} gemm vs gemv")
    dev.close()


def test_batched_decode_gemm_path_bf16(pkg, orc):
    """bf16 weights, 8 sequences: the MFMA step within 2e-2 (of the largest logit) of the oracle on bf16-rounded weights."""
    hp = small_cfg(pkg, "hybrid", weightDtype=pkg.DTYPE_BF16, maxSeqs=8)
    model, dev, w = make(pkg, orc, hp, seed=32, bf16=True)
    prompts = [pkg.random_tokens(32, s, hp.vocabSize, 20 + 7 * s) for s in range(8)]
    dev.prefill_batch(list(range(8)), prompts)
    firsts = [dev.greedy_token(s) for s in range(8)]
    out = dev.decode_loop(firsts, 6)
    for s in (0, 3, 7):
        dec = orc.Decoder(w, "f64")
        ids = [firsts[s]] + [int(t) for t in out[:, s]]
        for t in list(prompts[s]) + ids[:-1]:
            _, lg = dec.step(int(t))
        err = float(np.max(np.abs(dev.logits(s) - lg)) / np.max(np.abs(lg)))
        assert err <= BF16_RTOL, (s, err)
    dev.close()


# ---- teacher-forced full-sequence forward ----------------------------------------------------------
@pytest.mark.parametrize("kind,n,mode", [("attn_flags", 60, 0), ("hybrid", 97, 0), ("hybrid_flags", 40, 1), ("attn", 9, 0)])
def test_forward_full_all_positions(pkg, orc, kind, n, mode):
    """Logits and probabilities of EVERY position (what the reference's runInference(L) leaves in its
    [V x L] buffers) and the mean next-token loss against the float64 oracle's full recompute."""
    hp = small_cfg(pkg, kind)
    model, dev, w = make(pkg, orc, hp, seed=41)
    ids = pkg.random_tokens(41, 0, hp.vocabSize, n)
    ref = orc.forward_full(w, ids, "f64", last_only=False, want_probs=True)
    dev.set_prefill_mode(mode)
    lg, pr, nll = dev.forward_full(0, ids)
    assert dev.seq_len(0) == n
    for i in range(n):
        assert_logits_close(lg[i], ref["logits"][i], FP32_RTOL, f"{kind} position {i}")
    assert np.max(np.abs(pr - ref["probs"])) <= 1e-6 + FP32_RTOL * np.max(ref["probs"])
    assert np.allclose(pr.sum(axis=1), 1.0, atol=1e-5)
    p_next = np.maximum(ref["probs"][np.arange(n - 1), ids[1:]], 1e-4)  # the reference's clamp
    assert abs(nll - float(np.mean(-np.log(p_next)))) <= 1e-4
    # the cache is filled as by a prefill: decoding continues from it
    assert_logits_close(dev.logits(0), ref["logits"][-1], FP32_RTOL, "last position")
    tok = dev.greedy_token(0)
    nxt = int(dev.decode_step([tok])[0])
    dec = orc.Decoder(w, "f64")
    check_greedy_against_oracle(dec, ids, [tok, nxt], GAP_TOL, what=kind)
    dev.close()


def test_reference_default_architecture(pkg, orc):
    """The shape the reference ships compiled in (network_meta.h:3-20: dim 768, 6 heads x 128, ffn 3072,
    16 layers, vocab 20160, QK-norm and query gating on) with its uniform +-0.02 initialisation
    (random_weights.cu:15-25; own PRNG, cuRAND's stream is not reproducible here): prefill + greedy
    decode against the float64 oracle."""
    hp = pkg.reference_defaults()
    hp.maxL = 128
    model = pkg.Model.new(hp)
    model.init_uniform(9, 0.02)
    model.randomize_gains(9)
    dev = pkg.Device(hp, 0)
    dev.upload(model)
    w = orc.Weights.from_model(model)
    prompt = pkg.random_tokens(9, 0, hp.vocabSize, 24)
    dev.prefill(0, prompt)
    ids = [dev.greedy_token(0)]
    logits = [dev.logits(0)]
    for _ in range(5):
        ids.append(int(dev.decode_step([ids[-1]])[0]))
        logits.append(dev.logits(0))
    dec = orc.Decoder(w, "f64")
    exact, tol = check_greedy_against_oracle(dec, prompt, ids, GAP_TOL, logits, FP32_RTOL, "reference defaults")
    assert exact + tol == len(ids)
    dev.close()
