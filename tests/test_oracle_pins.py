"""Pins every function of the CPU oracle against something that is not the oracle's own formula:
known answers, closed forms, invariants, brute force in NumPy matrix form, and an independent
PyTorch restatement of the reference's pytorch_verification model (oracle/cpu_model.py).

The reference ships no numeric golden vectors; its fixtures (vocab, sample) are covered in
test_host.py.  CPU only.
"""
import ctypes
import os
import sys

import numpy as np
import pytest

from conftest import GOLDEN, ROOT


def _p(a):
    return a.ctypes.data


def _tensors(model):
    hp = model.hparams
    t = {("E",): model.tensor(0, 0), ("gammaF",): model.tensor(0, 1)}
    for l in range(hp.transformers):
        for tid in range(2, 21):
            a = model.tensor(l, tid)
            if a is not None:
                t[(l, tid)] = a
    return t


# --------------------------------------------------------------------------- unit ops
def test_rmsnorm_known_answer_and_invariants(orc):
    x = np.array([3.0, 4.0])
    g = np.array([2.0, 0.5], dtype=np.float32)
    y = np.empty(2)
    orc.lib.orc_rmsnorm_f64(_p(x), _p(g), 2, _p(y))
    r = np.sqrt(12.5 + 1e-8)  # mean(9, 16) = 12.5, eps inside the square root
    assert np.allclose(y, [2 * 3 / r, 0.5 * 4 / r], rtol=1e-12)
    # eps is inside the sqrt: a zero vector maps to zero, not NaN
    z = np.zeros(8)
    out = np.empty(8)
    orc.lib.orc_rmsnorm_f64(_p(z), _p(np.ones(8, np.float32)), 8, _p(out))
    assert np.all(out == 0)
    # with unit gain the output has mean square ms/(ms+eps) and is scale invariant for large inputs
    rng = np.random.default_rng(0)
    x = rng.normal(size=768)
    ones = np.ones(768, np.float32)
    y1, y2 = np.empty(768), np.empty(768)
    orc.lib.orc_rmsnorm_f64(_p(x), _p(ones), 768, _p(y1))
    x2 = x * 1000.0
    orc.lib.orc_rmsnorm_f64(_p(x2), _p(ones), 768, _p(y2))
    ms = np.mean(x * x)
    assert abs(np.mean(y1 * y1) - ms / (ms + 1e-8)) < 1e-12
    assert np.allclose(y1, y2, rtol=1e-7)
    # float version agrees with the double one to float precision
    xf, yf = x.astype(np.float32), np.empty(768, np.float32)
    orc.lib.orc_rmsnorm_f32(_p(xf), _p(ones), 768, _p(yf))
    assert np.allclose(yf, y1, rtol=2e-6, atol=1e-6)


def test_head_rmsnorm_is_per_head_with_per_channel_gain(orc):
    H, hd = 3, 64
    rng = np.random.default_rng(1)
    q = rng.normal(size=H * hd)
    g = (1 + np.arange(H * hd) / 100).astype(np.float32)  # distinct per head AND channel (size dim)
    out = q.copy()
    orc.lib.orc_head_rmsnorm_f64(_p(out), _p(g), H, hd)
    for h in range(H):
        seg = out[h * hd:(h + 1) * hd] / g[h * hd:(h + 1) * hd]
        ms = np.mean(q[h * hd:(h + 1) * hd] ** 2)
        assert abs(np.mean(seg ** 2) - ms / (ms + 1e-8)) < 1e-12  # each head normalised on its own
    q2 = q.copy()
    q2[hd:2 * hd] *= 7.0  # disturbing head 1 leaves heads 0 and 2 untouched
    out2 = q2.copy()
    orc.lib.orc_head_rmsnorm_f64(_p(out2), _p(g), H, hd)
    assert np.array_equal(out2[:hd], out[:hd]) and np.array_equal(out2[2 * hd:], out[2 * hd:])


def test_rope_table_identities(orc, pkg):
    hd, maxL, base = 64, 700, 10000.0
    tab = orc.rope_table(maxL, hd, base)
    assert np.array_equal(tab, pkg.rope_table(maxL, hd, base)), "host table and oracle table differ bitwise"
    assert np.all(tab[0, 0::2] == 1) and np.all(tab[0, 1::2] == 0)          # position 0: no rotation
    assert np.allclose(tab[:, 0::2] ** 2 + tab[:, 1::2] ** 2, 1, atol=3e-7)  # cos^2 + sin^2
    p = np.arange(0, 40)
    assert np.allclose(tab[p, 0], np.cos(p), atol=2e-6) and np.allclose(tab[p, 1], np.sin(p), atol=2e-6)  # pair 0: freq 1
    ang = np.arctan2(tab[1, 1::2].astype(np.float64), tab[1, 0::2].astype(np.float64))
    assert np.allclose(ang, base ** (-2.0 * np.arange(hd // 2) / hd), rtol=3e-6)  # frequency of pair i


def test_rope_is_interleaved_pair_rotation(orc):
    H, hd, pos = 2, 64, 37
    tab = orc.rope_table(64, hd, 10000.0)
    rng = np.random.default_rng(2)
    q = rng.normal(size=H * hd)
    out = q.copy()
    orc.lib.orc_rope_f64(_p(out), _p(tab), pos, H, hd)
    # complex form: (q[2i] + j q[2i+1]) * exp(j * pos * theta_i), adjacent pairs, inside each head
    theta = 10000.0 ** (-2.0 * np.arange(hd // 2) / hd)
    z = (q.reshape(H, hd // 2, 2)[..., 0] + 1j * q.reshape(H, hd // 2, 2)[..., 1]) * np.exp(1j * pos * theta)
    want = np.stack([z.real, z.imag], axis=-1).reshape(-1)
    assert np.allclose(out, want, atol=5e-6)  # table is float32
    # unit vector on coordinate 0 lands on coordinates (0, 1), not (0, hd/2)
    e = np.zeros(H * hd)
    e[0] = 1
    orc.lib.orc_rope_f64(_p(e), _p(tab), 5, H, hd)
    assert abs(e[0] - np.cos(5.0)) < 1e-6 and abs(e[1] - np.sin(5.0)) < 1e-6 and np.all(e[2:] == 0)
    # position 0 is the identity; rotation keeps every pair's norm
    q0 = q.copy()
    orc.lib.orc_rope_f64(_p(q0), _p(tab), 0, H, hd)
    assert np.array_equal(q0, q)
    assert np.allclose(out.reshape(-1, 2).__pow__(2).sum(1), q.reshape(-1, 2).__pow__(2).sum(1), rtol=1e-6)
    # relative-position property: <rope(q,p), rope(k,p')> depends on p - p' only
    k = rng.normal(size=H * hd)
    def dot_at(pq, pk):
        a, b = q.copy(), k.copy()
        orc.lib.orc_rope_f64(_p(a), _p(tab), pq, H, hd)
        orc.lib.orc_rope_f64(_p(b), _p(tab), pk, H, hd)
        return float(a @ b)
    assert abs(dot_at(9, 4) - dot_at(25, 20)) < 1e-4


def test_matvec_row_major(orc):
    rng = np.random.default_rng(3)
    W = rng.normal(size=(37, 96)).astype(np.float32)
    x = rng.normal(size=96)
    y = np.empty(37)
    orc.lib.orc_matvec_f64(_p(W), _p(x), 37, 96, _p(y))
    assert np.allclose(y, W.astype(np.float64) @ x, rtol=1e-12)  # W[o*in + i]: row-major [out, in]
    yf = np.empty(37, np.float32)
    xf = x.astype(np.float32)
    orc.lib.orc_matvec_f32(_p(W), _p(xf), 37, 96, _p(yf))
    assert np.allclose(yf, y, rtol=1e-4, atol=1e-5)


def test_blocked_product_is_bit_identical_to_matvec(orc):
    """The full-sequence forward multiplies all columns at once (blocked over tokens); each element must be
    accumulated exactly as the one-vector routine does it, in float and in double, for ragged shapes."""
    rng = np.random.default_rng(33)
    for rows, cols, L in ((37, 96, 1), (6, 50, 16), (130, 64, 45)):
        W = rng.normal(size=(rows, cols)).astype(np.float32)
        for sfx, real in (("f32", np.float32), ("f64", np.float64)):
            X = np.ascontiguousarray(rng.normal(size=(L, cols + 3)).astype(real))  # rows padded: ldx > cols
            Y = np.full((L, rows + 2), 7.0, dtype=real)
            getattr(orc.lib, f"orc_matmat_{sfx}")(_p(W), _p(X), cols + 3, rows, cols, L, _p(Y), rows + 2)
            for l in range(L):
                y = np.empty(rows, dtype=real)
                x = np.ascontiguousarray(X[l, :cols])
                getattr(orc.lib, f"orc_matvec_{sfx}")(_p(W), _p(x), rows, cols, _p(y))
                assert np.array_equal(Y[l, :rows], y)
            assert np.all(Y[:, rows:] == 7.0)


def test_attend_brute_force_and_special_cases(orc):
    H, hd, T = 3, 64, 29
    d = H * hd
    rng = np.random.default_rng(4)
    q, K, V = rng.normal(size=d), rng.normal(size=(T, d)), rng.normal(size=(T, d))
    out = np.empty(d)
    orc.lib.orc_attend_f64(_p(q), _p(K), _p(V), T, d, H, hd, _p(out))
    for h in range(H):
        sl = slice(h * hd, (h + 1) * hd)
        s = K[:, sl] @ q[sl] / np.sqrt(hd)
        p = np.exp(s - s.max())
        p /= p.sum()
        assert np.allclose(out[sl], p @ V[:, sl], rtol=1e-11)
    # one key: softmax weight 1, the output is that value row
    orc.lib.orc_attend_f64(_p(q), _p(K), _p(V), 1, d, H, hd, _p(out))
    assert np.allclose(out, V[0], rtol=1e-14)
    # identical keys: uniform weights, the output is the mean value
    Ksame = np.tile(K[0], (T, 1))
    orc.lib.orc_attend_f64(_p(q), _p(Ksame), _p(V), T, d, H, hd, _p(out))
    assert np.allclose(out, V.mean(0), rtol=1e-11)
    # large scores do not overflow (max subtraction)
    orc.lib.orc_attend_f64(_p(q * 1e4), _p(K), _p(V), T, d, H, hd, _p(out))
    assert np.all(np.isfinite(out))


def test_gdn_step_closed_forms(orc):
    dk = dv = 64
    rng = np.random.default_rng(5)
    S0 = rng.normal(size=(dv, dk))
    q, k, v = rng.normal(size=dk), rng.normal(size=dk), rng.normal(size=dv)
    k /= np.linalg.norm(k)
    step = orc.lib.orc_gdn_step_f64

    def run(S, alpha, beta):
        S = S.copy()
        o = np.empty(dv)
        step(_p(S), _p(q), _p(k), _p(v), alpha, beta, dk, dv, _p(o))
        return S, o

    S1, o1 = run(S0, 1.0, 0.0)                     # beta = 0, alpha = 1: state unchanged
    assert np.array_equal(S1, S0) and np.allclose(o1, S0 @ q, rtol=1e-12)
    S1, _ = run(np.zeros((dv, dk)), 0.7, 0.3)      # from the zero state: S1 = beta v k^T
    assert np.allclose(S1, 0.3 * np.outer(v, k), rtol=1e-12, atol=1e-15)
    a, b = 0.83, 0.41
    S1, o1 = run(S0, a, b)
    want = a * S0 @ (np.eye(dk) - b * np.outer(k, k)) + b * np.outer(v, k)  # the matrix form of the update
    assert np.allclose(S1, want, rtol=1e-11, atol=1e-13)
    assert np.allclose(S1 @ k, a * (1 - b) * (S0 @ k) + b * v, rtol=1e-10, atol=1e-12)  # |k| = 1 contraction
    assert np.allclose(o1, S1 @ q, rtol=1e-12)     # read-out uses the updated state
    S2, _ = run(S0, a, 1.0)                        # beta = 1 writes v exactly along k
    assert np.allclose(S2 @ k, v, rtol=1e-10, atol=1e-12)


def test_bf16_rounding_matches_library_and_ties_to_even(orc):
    import torch
    rng = np.random.default_rng(6)
    x = (rng.normal(size=20000) * np.exp(rng.normal(size=20000) * 4)).astype(np.float32)
    got = orc.round_bf16(x)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got, want)
    ties = np.array([1 + 2.0 ** -8, 1 + 2.0 ** -7 + 2.0 ** -8, -(1 + 2.0 ** -8)], dtype=np.float32)
    assert np.array_equal(orc.round_bf16(ties), np.array([1.0, 1 + 2.0 ** -6, -1.0], dtype=np.float32))


# --------------------------------------------------------------------------- whole forward
@pytest.fixture(scope="module")
def tiny_attn(pkg, orc):
    hp = pkg.config(1, dim=128, attnHeads=2, headDim=64, ffnDim=192, transformers=3, vocabSize=512, maxL=48)
    model = pkg.Model.generate(hp, seed=9)
    # non-trivial gains so that a missing or misplaced gain would show
    rng = np.random.default_rng(9)
    model.tensor(0, 1)[:] = 1 + 0.1 * rng.normal(size=hp.dim)
    for l in range(hp.transformers):
        model.tensor(l, 2)[:] = 1 + 0.1 * rng.normal(size=hp.dim)
        model.tensor(l, 7)[:] = 1 + 0.1 * rng.normal(size=hp.dim)
    return hp, model, orc.Weights.from_model(model)


def test_full_forward_against_independent_torch_restatement(pkg, orc, tiny_attn):
    """The C oracle (following inference.cu) and oracle/cpu_model.py (following the reference's
    PyTorch script, matrix form, rsqrt) are two separately written statements of the same maths."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import cpu_model
    hp, model, w = tiny_attn
    cm = cpu_model.CpuModel(hp, _tensors(model))
    toks = pkg.random_tokens(9, 0, hp.vocabSize, 23)
    lg = orc.forward_full(w, toks, "f64")["logits"][0]
    lt = cm.forward(toks).numpy()
    assert np.max(np.abs(lg - lt)) < 5e-6 * np.max(np.abs(lg))  # torch side is float32
    lg32 = orc.forward_full(w, toks, "f32")["logits"][0]
    assert np.max(np.abs(lg - lg32)) < 5e-6 * np.max(np.abs(lg))
    # layer order matters and block 0 is the top: reversing the blocks changes the result
    t = _tensors(model)
    rev = {k: v for k, v in t.items() if len(k) == 1}
    for (l, tid), v in [(k, v) for k, v in t.items() if len(k) == 2]:
        rev[(hp.transformers - 1 - l, tid)] = v
    lr = orc.forward_full(orc.Weights(hp, rev), toks, "f64")["logits"][0]
    assert np.max(np.abs(lr - lg)) > 1e-3
    assert np.max(np.abs(cpu_model.CpuModel(hp, rev).forward(toks).numpy() - lr)) < 5e-6 * np.max(np.abs(lr))


def test_probs_are_softmax_of_logits_for_every_column(pkg, orc, tiny_attn):
    hp, model, w = tiny_attn
    toks = pkg.random_tokens(9, 1, hp.vocabSize, 7)
    r = orc.forward_full(w, toks, "f64", last_only=False, want_probs=True)
    lg, pr = r["logits"], r["probs"]
    assert lg.shape == (7, hp.vocabSize)
    e = np.exp(lg - lg.max(1, keepdims=True))
    assert np.allclose(pr, e / e.sum(1, keepdims=True), rtol=1e-12)
    # causality: logits of column j do not depend on later tokens
    r2 = orc.forward_full(w, toks[:4], "f64", last_only=False)
    assert np.array_equal(r2["logits"], lg[:4])


@pytest.mark.parametrize("flags", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_cached_decode_equals_full_recompute(pkg, orc, flags):
    """KV-cache invariant: the logits of step t equal the last column of the reference-style
    recompute over t+1 tokens -- for attention (all flag settings), GDN and PLE layers."""
    hp = pkg.config(3, dim=128, attnHeads=2, headDim=64, ffnDim=192, transformers=4, vocabSize=512, gdnHeads=2,
                    maxL=40, qkRmsNorm=flags[0], queryGating=flags[1])
    pkg.set_layer_pattern(hp, 1)
    model = pkg.Model.generate(hp, seed=13)
    rng = np.random.default_rng(13)
    for l in range(4):  # per-head gains must be indexed by head and channel
        for tid in (11, 12):
            if model.tensor(l, tid) is not None:
                model.tensor(l, tid)[:] = 1 + 0.2 * rng.normal(size=hp.dim)
    w = orc.Weights.from_model(model)
    toks = pkg.random_tokens(13, 0, hp.vocabSize, 30)
    for dt, tol in (("f64", 1e-12), ("f32", 2e-5)):
        dec = orc.Decoder(w, dt)
        for t in range(30):
            nxt, lg = dec.step(int(toks[t]))
            if t in (0, 1, 7, 29):
                full = orc.forward_full(w, toks[:t + 1], dt)["logits"][0]
                assert np.max(np.abs(full - lg)) <= tol * np.max(np.abs(full))
                assert nxt == int(np.argmax(lg))


def test_flags_change_the_result_and_gain_indexing(pkg, orc):
    base = dict(dim=128, attnHeads=2, headDim=64, ffnDim=192, transformers=2, vocabSize=256, maxL=16)
    toks = np.arange(10, dtype=np.int32)
    outs = {}
    for f in ((0, 0), (1, 0), (0, 1)):
        hp = pkg.config(1, qkRmsNorm=f[0], queryGating=f[1], **base)
        outs[f] = orc.forward_full(orc.Weights.from_model(pkg.Model.generate(hp, 3)), toks, "f64")["logits"][0]
    assert np.max(np.abs(outs[(0, 0)] - outs[(1, 0)])) > 1e-4
    assert np.max(np.abs(outs[(0, 0)] - outs[(0, 1)])) > 1e-4
    # zero gating weights: sigmoid(0) = 1/2 scales the attention output by exactly one half before Wo
    hp = pkg.config(1, queryGating=1, **base)
    model = pkg.Model.generate(hp, 3)
    for l in range(2):
        model.tensor(l, 13)[:] = 0
    hid_g = orc.forward_full(orc.Weights.from_model(model), toks, "f64", want_hidden=True)["hidden"]
    hp0 = pkg.config(1, **base)
    model0 = pkg.Model.generate(hp0, 3)
    for l in range(2):
        model0.tensor(l, 6)[:] *= 0.5  # halve Wo instead
    hid_0 = orc.forward_full(orc.Weights.from_model(model0), toks, "f64", want_hidden=True)["hidden"]
    assert np.allclose(hid_g, hid_0, rtol=1e-12, atol=1e-14)


def test_gdn_and_ple_invariants(pkg, orc):
    base = dict(dim=128, attnHeads=2, headDim=64, ffnDim=192, transformers=4, vocabSize=256, gdnHeads=2, maxL=24)
    toks = pkg.random_tokens(4, 0, 256, 18)
    hp = pkg.config(3, **base)
    pkg.set_layer_pattern(hp, 3)
    assert list(hp.layerKinds[:4]) == [0, 1, 1, 1]  # applied first = file index 3 (GDN); top block attention
    model = pkg.Model.generate(hp, 4)
    ref = orc.forward_full(orc.Weights.from_model(model), toks, "f64")["logits"][0]
    # zero per-layer-embedding tables: identical to the same model without PLE
    for l in range(4):
        model.tensor(l, 18)[:] = 0
    z = orc.forward_full(orc.Weights.from_model(model), toks, "f64")["logits"][0]
    hp_np = pkg.config(3, pleDim=0, **base)
    pkg.set_layer_pattern(hp_np, 3)
    m2 = pkg.Model.generate(hp_np, 4)  # same seed and tensor keys: identical non-PLE tensors
    z2 = orc.forward_full(orc.Weights.from_model(m2), toks, "f64")["logits"][0]
    assert np.array_equal(z, z2) and np.max(np.abs(z - ref)) > 1e-7
    # beta -> 0 (bias -60): the state never leaves zero, so the GDN layers add nothing to the residual
    # and the model equals one whose GDN output projections are zero
    m3 = pkg.Model.generate(hp_np, 4)
    m4 = pkg.Model.generate(hp_np, 4)
    for l in (1, 2, 3):
        m3.tensor(l, 17)[:] = -60.0
        m3.tensor(l, 16)[:] = 0
        m4.tensor(l, 6)[:] = 0
    a = orc.forward_full(orc.Weights.from_model(m3), toks, "f64")["logits"][0]
    b = orc.forward_full(orc.Weights.from_model(m4), toks, "f64")["logits"][0]
    assert np.max(np.abs(a - b)) < 1e-20 + 1e-12 * np.max(np.abs(b))


def test_gdn_gates_closed_form(pkg, orc):
    """alpha = exp(-softplus(z)) equals sigmoid(-z); checked through a one-layer model whose gate
    pre-activations are pure biases (zero gate weights) by comparing the first two states."""
    hp = pkg.config(3, dim=64, attnHeads=1, headDim=64, ffnDim=64, transformers=1, vocabSize=32, gdnHeads=1,
                    pleDim=0, maxL=4)
    pkg.set_layer_pattern(hp, 1)
    hp.layerKinds[0] = 1
    model = pkg.Model.generate(hp, 2)
    model.tensor(0, 14)[:] = 0
    model.tensor(0, 16)[:] = 0
    za, zb = float(np.float32(0.37)), float(np.float32(-0.81))  # the model stores float32
    model.tensor(0, 15)[:] = za
    model.tensor(0, 17)[:] = zb
    model.tensor(0, 6)[:] = np.eye(64, dtype=np.float32)   # Wo = I: the mixing output shows in the residual
    model.tensor(0, 8)[:] = 0                               # FFN off
    w = orc.Weights.from_model(model)
    E = model.tensor(0, 0).astype(np.float64)
    Wq, Wk, Wv = (model.tensor(0, t).astype(np.float64) for t in (3, 4, 5))
    alpha, beta = 1 / (1 + np.exp(za)), 1 / (1 + np.exp(-zb))
    toks = [3, 7]
    S = np.zeros((64, 64))
    x_out = None
    for t in toks:
        x = E[t]
        xn = x / np.sqrt(np.mean(x * x) + 1e-8)
        q, k, v = Wq @ xn, Wk @ xn, Wv @ xn
        q, k = q / np.sqrt(q @ q + 1e-6), k / np.sqrt(k @ k + 1e-6)
        S = alpha * S @ (np.eye(64) - beta * np.outer(k, k)) + beta * np.outer(v, k)
        x_out = S @ q + x
    hid = orc.forward_full(w, np.array(toks, np.int32), "f64", want_hidden=True)["hidden"]
    assert np.allclose(hid[-1], x_out, rtol=1e-9, atol=1e-12)


def test_ple_branch_closed_form(pkg, orc):
    """Per-layer embeddings: h1 = Wo a + x + Wpu (silu(Wpg xn) * P[tok]), xn the RMS1-normed input.  One
    attention block with Wo = 0 and the FFN switched off leaves hidden = x + the PLE branch, which is
    compared with an independent NumPy statement; a wrong activation, x in place of xn, a wrong table
    row or a missing gain each fail it."""
    hp = pkg.config(3, dim=64, attnHeads=1, headDim=64, ffnDim=64, transformers=1, vocabSize=32, gdnHeads=1,
                    pleDim=16, maxL=4)
    pkg.set_layer_pattern(hp, 1)
    hp.layerKinds[0] = 0
    model = pkg.Model.generate(hp, 5)
    rng = np.random.default_rng(5)
    model.tensor(0, 6)[:] = 0                                    # Wo = 0: attention adds nothing
    model.tensor(0, 8)[:] = 0                                    # gate rows 0: silu(0) * up = 0, FFN adds nothing
    model.tensor(0, 2)[:] = 1 + 0.3 * rng.normal(size=hp.dim)    # RMS1 gain: xn, not x / rms
    model.tensor(0, 18)[:] = rng.normal(size=(32, 16))           # table rows of visible size
    model.tensor(0, 19)[:] = rng.normal(size=(16, 64))           # gate pre-activations O(1): silu != sigmoid != id
    model.tensor(0, 20)[:] = rng.normal(size=(64, 16))
    E = model.tensor(0, 0).astype(np.float64)
    g1 = model.tensor(0, 2).astype(np.float64)
    P, Wpg, Wpu = (model.tensor(0, t).astype(np.float64) for t in (18, 19, 20))

    def want(tok):
        x = E[tok]
        xn = g1 * (x / np.sqrt(np.mean(x * x) + 1e-8))
        z = Wpg @ xn
        return x + Wpu @ ((z / (1 + np.exp(-z))) * P[tok])

    toks = np.array([3, 7], np.int32)
    hid = orc.forward_full(orc.Weights.from_model(model), toks, "f64", want_hidden=True)["hidden"]
    for i, t in enumerate(toks):
        assert np.allclose(hid[i], want(t), rtol=1e-9, atol=1e-12)
    # the branch is not small here: leaving it out, or using the wrong row, would be far outside the bound
    assert np.max(np.abs(hid[0] - E[3])) > 1e-2 and np.max(np.abs(want(3) - (want(7) - E[7] + E[3]))) > 1e-2
    # row selection: swapping two table rows swaps what the two tokens receive from the table
    model.tensor(0, 18)[[3, 7]] = model.tensor(0, 18)[[7, 3]]
    P[[3, 7]] = P[[7, 3]]
    hid2 = orc.forward_full(orc.Weights.from_model(model), toks, "f64", want_hidden=True)["hidden"]
    for i, t in enumerate(toks):
        assert np.allclose(hid2[i], want(t), rtol=1e-9, atol=1e-12)
    assert np.max(np.abs(hid2 - hid)) > 1e-2
    # the cached decode path uses the same branch: its logits equal the full recompute's
    w = orc.Weights.from_model(model)
    dec = orc.Decoder(w, "f64")
    for t in toks:
        _, lg = dec.step(int(t))
    full = orc.forward_full(w, toks, "f64")["logits"][0]
    assert np.allclose(lg, full, rtol=1e-12, atol=1e-14)
    # and the branch joins the residual with the output projection (before RMS2 / the FFN): with the FFN on,
    # the FFN must see x + branch
    model.tensor(0, 8)[:] = rng.normal(size=(64, 64)) * 0.2
    W1A, W1B, W2 = (model.tensor(0, t).astype(np.float64) for t in (8, 9, 10))
    g2 = model.tensor(0, 7).astype(np.float64)
    hid3 = orc.forward_full(orc.Weights.from_model(model), toks, "f64", want_hidden=True)["hidden"]
    h1 = want(3)
    hn = g2 * (h1 / np.sqrt(np.mean(h1 * h1) + 1e-8))
    a = W1A @ hn
    assert np.allclose(hid3[0], h1 + W2 @ ((a / (1 + np.exp(-a))) * (W1B @ hn)), rtol=1e-9, atol=1e-12)


def test_attention_block_with_both_flags_closed_form(pkg, orc):
    """One attention block with per-head QK RMSNorm and query gating on, random gains (rmsGamma,
    queryRMSGamma, keyRMSGamma), random gate weights, Wo = I and the FFN off, so that hidden = x + gated attention
    output.  Compared with an independent NumPy statement of inference.cu:467-483 (per-head norm with
    gamma[h*hd + i], THEN RoPE) and inference.cu:486-508, 241-250 (gate = sigmoid(Wg xn) from the normed input,
    applied before Wo).  Each plausible mistake is also formed in NumPy and must lie far outside the bound:
    norm after RoPE, a head-shared gain gamma[i % hd], the gate taken from x instead of xn, the gate applied
    after Wo (shown with a non-identity Wo), and a missing RMS1 gain."""
    H, hd = 2, 64
    d = H * hd
    hp = pkg.config(1, dim=d, attnHeads=H, headDim=hd, ffnDim=64, transformers=1, vocabSize=32, maxL=8,
                    qkRmsNorm=1, queryGating=1)
    model = pkg.Model.generate(hp, 21)
    rng = np.random.default_rng(21)
    model.tensor(0, 2)[:] = 1 + 0.3 * rng.uniform(-1, 1, size=d)      # rmsGamma
    model.tensor(0, 11)[:] = 1 + 0.5 * rng.uniform(-1, 1, size=d)     # queryRMSGamma: distinct per head and channel
    model.tensor(0, 12)[:] = 1 + 0.5 * rng.uniform(-1, 1, size=d)     # keyRMSGamma
    for tid in (3, 4, 5):
        model.tensor(0, tid)[:] = rng.normal(size=(d, d)) * 0.3
    model.tensor(0, 13)[:] = rng.normal(size=(d, d)) * 0.2            # gate pre-activations O(1)
    model.tensor(0, 6)[:] = np.eye(d, dtype=np.float32)               # Wo = I
    model.tensor(0, 8)[:] = 0                                         # FFN off
    model.tensor(0, 0)[:] = rng.normal(size=(32, d))                  # embeddings of visible size
    E = model.tensor(0, 0).astype(np.float64)
    g1, gq, gk = (model.tensor(0, t).astype(np.float64) for t in (2, 11, 12))
    Wq, Wk, Wv, Wg = (model.tensor(0, t).astype(np.float64) for t in (3, 4, 5, 13))
    tab = pkg.rope_table(hp.maxL, hd).astype(np.float64)              # the table itself is pinned elsewhere
    toks = np.array([3, 7, 11, 5], np.int32)

    def head_norm(v, gamma, shared=False):
        out = np.empty_like(v)
        for h in range(H):
            s = slice(h * hd, (h + 1) * hd)
            r = np.sqrt(np.mean(v[s] ** 2) + 1e-8)
            out[s] = (gamma[:hd] if shared else gamma[s]) * (v[s] / r)
        return out

    def rope(v, pos):
        out = np.empty_like(v)
        for h in range(H):
            for i in range(hd // 2):
                a, b = v[h * hd + 2 * i], v[h * hd + 2 * i + 1]
                c, s = tab[pos, 2 * i], tab[pos, 2 * i + 1]
                out[h * hd + 2 * i], out[h * hd + 2 * i + 1] = a * c - b * s, a * s + b * c
        return out

    def block(Wo=None, norm_after_rope=False, shared_gain=False, gate_from_x=False, gate_after_wo=False,
              no_rms1_gain=False):
        Ks, Vs, hid = [], [], []
        for pos, t in enumerate(toks):
            x = E[t]
            xn = x / np.sqrt(np.mean(x * x) + 1e-8)
            if not no_rms1_gain:
                xn = g1 * xn
            q, k, v = Wq @ xn, Wk @ xn, Wv @ xn
            if norm_after_rope:
                q, k = head_norm(rope(q, pos), gq, shared_gain), head_norm(rope(k, pos), gk, shared_gain)
            else:
                q, k = rope(head_norm(q, gq, shared_gain), pos), rope(head_norm(k, gk, shared_gain), pos)
            Ks.append(k)
            Vs.append(v)
            a = np.empty(d)
            for h in range(H):
                s = slice(h * hd, (h + 1) * hd)
                sc = np.array([kk[s] @ q[s] for kk in Ks]) / np.sqrt(hd)
                p = np.exp(sc - sc.max())
                p /= p.sum()
                a[s] = sum(pj * vv[s] for pj, vv in zip(p, Vs))
            gate = 1 / (1 + np.exp(-(Wg @ (x if gate_from_x else xn))))
            if Wo is None:
                hid.append(a * gate + x)
            elif gate_after_wo:
                hid.append((Wo @ a) * gate + x)
            else:
                hid.append(Wo @ (a * gate) + x)
        return np.array(hid)

    want = block()
    w = orc.Weights.from_model(model)
    hid = orc.forward_full(w, toks, "f64", want_hidden=True)["hidden"]
    assert np.allclose(hid, want, rtol=1e-9, atol=1e-12)
    # the same block through the cached decode path (logits are a fixed function of hidden)
    dec = orc.Decoder(w, "f64")
    for t in toks:
        _, lg = dec.step(int(t))
    assert np.allclose(lg, orc.forward_full(w, toks, "f64")["logits"][0], rtol=1e-11, atol=1e-13)
    # float32 oracle agrees to float precision
    hid32 = orc.forward_full(w, toks, "f32", want_hidden=True)["hidden"]
    assert np.max(np.abs(hid32 - want)) < 2e-5 * np.max(np.abs(want))
    # each mistake named above is far outside the bound at positions >= 1 (position 0 has RoPE = identity)
    scale = np.max(np.abs(want[1:] - E[toks[1:]]))
    for wrong in (dict(norm_after_rope=True), dict(shared_gain=True), dict(gate_from_x=True),
                  dict(no_rms1_gain=True)):
        assert np.max(np.abs(block(**wrong)[1:] - want[1:])) > 1e-2 * scale, wrong
    # gate before Wo, not after: needs a Wo that is not the identity
    Wo = rng.normal(size=(d, d)) * 0.3
    model.tensor(0, 6)[:] = Wo
    Wo = model.tensor(0, 6).astype(np.float64)
    hid_wo = orc.forward_full(orc.Weights.from_model(model), toks, "f64", want_hidden=True)["hidden"]
    assert np.allclose(hid_wo, block(Wo=Wo), rtol=1e-9, atol=1e-12)
    assert np.max(np.abs(block(Wo=Wo, gate_after_wo=True) - hid_wo)) > 1e-2 * np.max(np.abs(hid_wo))


def test_greedy_pick_takes_lowest_index_on_ties(pkg, orc):
    hp = pkg.config(1, dim=128, attnHeads=2, headDim=64, ffnDim=192, transformers=1, vocabSize=64, maxL=8)
    model = pkg.Model.generate(hp, 1)
    dec = orc.Decoder(orc.Weights.from_model(model), "f64")
    _, lg = dec.step(5)
    top = int(np.argmax(lg))
    E = model.tensor(0, 0)
    lo, hi = (top, 63) if top != 63 else (0, 63)
    E[hi] = E[top]
    E[lo] = E[top]  # two identical embedding rows give identical logits
    dec2 = orc.Decoder(orc.Weights.from_model(model), "f64")
    nxt, lg2 = dec2.step(7)
    best = np.flatnonzero(lg2 == lg2.max())
    assert nxt == best[0]
    if len(best) > 1:
        assert nxt < best[1]


def test_oracle_reproduces_committed_golden(pkg, orc):
    g = np.load(os.path.join(GOLDEN, "cfg1_golden.npz"))
    hp = pkg.config(1)
    model = pkg.Model.generate(hp, seed=0)
    assert np.array_equal(model.tensor(0, 0)[:4, :8], g["embedding_head"])  # generator unchanged
    prompt = pkg.random_tokens(0, 0, hp.vocabSize, 16)
    assert np.array_equal(prompt, g["prompt"])
    dec = orc.Decoder(orc.Weights.from_model(model), "f64")
    for t in prompt:
        nxt, lg = dec.step(int(t))
    keep = {int(s): i for i, s in enumerate(g["full_steps"])}
    for step in range(128):
        assert nxt == g["ids"][step]
        assert np.allclose(lg[g["top_idx"][step]], g["top_val"][step], rtol=1e-9)
        if step in keep:
            assert np.allclose(lg, g["full_logits"][keep[step]], rtol=1e-5, atol=1e-7)
        if step < 127:
            nxt, lg = dec.step(int(nxt))
