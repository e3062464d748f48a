"""PyTorch-CPU restatement of the reference's pytorch_verification model.

TEST INFRASTRUCTURE / CPU BASELINE ONLY (never imported by the product package).

Follows pytorch_verification/pyTorch_gradient_verification.py of the reference, written from
its mathematics and not from its text:
  * activations are [DIM, L] (features x positions)                       (:118-121)
  * layers are applied from index LAYERS-1 down to 0                      (:137)
  * RMSNorm  x * rsqrt(mean(x^2) + 1e-8) * gamma                          (:147-154)
  * RoPE on successive pairs (2i, 2i+1), inv_freq = base^(-2i/head_dim)   (:44-62, 176-192)
  * scores K^T Q * 1/sqrt(head_dim), keys after the query masked, softmax over keys (:199-229)
  * SwiGLU  W2 (silu(W1A x) * (W1B x)), residuals after attention and FFN (:262-291)
  * final RMSNorm and tied-embedding logits                               (:298-314)
Only the attention-only architecture of that script is covered (no QK-norm, gating, GDN, PLE).

Two generation modes, both greedy:
  * generate_full   recomputes all L positions for every new token, which is what the
                    reference's runInferenceLoop does (inference_orchestrator.cu:64-65);
  * generate_cached keeps K and V per layer.
"""
import math
import time

import numpy as np
import torch


class CpuModel:
    def __init__(self, hp, tensors, threads=None):
        """tensors: {("E",): [V,d], ("gammaF",): [d], (layer, tensor_id): array} with the tensor
        ids of include/mlh.h (2 rmsGamma, 3 Wq, 4 Wk, 5 Wv, 6 Wo, 7 rmsGamma2, 8 W1A, 9 W1B, 10 W2)."""
        if threads:
            torch.set_num_threads(int(threads))
        self.d, self.H, self.hd = hp.dim, hp.attnHeads, hp.headDim
        self.NL, self.V, self.maxL = hp.transformers, hp.vocabSize, hp.maxL
        t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
        self.E = t(tensors[("E",)])            # [V, d]
        self.gF = t(tensors[("gammaF",)]).unsqueeze(1)
        self.L = []
        for l in range(self.NL):
            g = lambda tid: t(tensors[(l, tid)])
            self.L.append(dict(g1=g(2).unsqueeze(1), Wq=g(3), Wk=g(4), Wv=g(5), Wo=g(6), g2=g(7).unsqueeze(1),
                               W1A=g(8), W1B=g(9), W2=g(10)))
        idx = torch.arange(0, self.hd, 2, dtype=torch.float32) / self.hd
        inv_freq = 1.0 / (float(hp.ropeDenomBase) ** idx)
        freqs = torch.outer(inv_freq, torch.arange(self.maxL, dtype=torch.float32))  # [hd/2, maxL]
        self.cos, self.sin = freqs.cos(), freqs.sin()
        self.scale = 1.0 / math.sqrt(self.hd)

    @staticmethod
    def _rms(x, gamma):
        return x * torch.rsqrt(x.pow(2).mean(dim=0, keepdim=True) + 1e-8) * gamma

    def _rope(self, v, p0, L):
        pairs = v.view(self.H, self.hd // 2, 2, L)
        a, b = pairs[:, :, 0, :], pairs[:, :, 1, :]
        c, s = self.cos[:, p0:p0 + L].unsqueeze(0), self.sin[:, p0:p0 + L].unsqueeze(0)
        return torch.stack([a * c - b * s, b * c + a * s], dim=2).view(self.H, self.hd, L)

    @torch.no_grad()
    def forward(self, tokens, cache=None):
        """Logits [V] of the last position.  cache: None (all positions recomputed) or a list of
        per-layer [K, V] tensors ([H, hd, T]) that is extended in place."""
        tok = torch.as_tensor(np.asarray(tokens), dtype=torch.long)
        p0 = 0 if cache is None or cache[0] is None else cache[0][0].shape[-1]
        L = tok.numel()
        x = self.E[tok].t().contiguous()  # [d, L]
        for layer in range(self.NL - 1, -1, -1):
            w = self.L[layer]
            xn = self._rms(x, w["g1"])
            q = self._rope((w["Wq"] @ xn).view(self.H, self.hd, L), p0, L)
            k = self._rope((w["Wk"] @ xn).view(self.H, self.hd, L), p0, L)
            v = (w["Wv"] @ xn).view(self.H, self.hd, L)
            if cache is not None:
                if cache[layer] is not None:
                    k = torch.cat([cache[layer][0], k], dim=-1)
                    v = torch.cat([cache[layer][1], v], dim=-1)
                cache[layer] = [k, v]
            T = k.shape[-1]
            scores = torch.matmul(k.transpose(-1, -2), q) * self.scale  # [H, T(keys), L(queries)]
            key_pos = torch.arange(T).unsqueeze(1)
            qry_pos = torch.arange(p0, p0 + L).unsqueeze(0)
            scores = scores.masked_fill((key_pos > qry_pos).unsqueeze(0), float("-inf"))
            probs = torch.softmax(scores, dim=-2)
            a = torch.matmul(v, probs).reshape(self.d, L)
            h1 = w["Wo"] @ a + x
            hn = self._rms(h1, w["g2"])
            g1 = w["W1A"] @ hn
            x = w["W2"] @ (g1 * torch.sigmoid(g1) * (w["W1B"] @ hn)) + h1
        xf = self._rms(x[:, -1:], self.gF)
        return (self.E @ xf).squeeze(1)

    def generate_full(self, prompt, n):
        """Reference-style loop: every token re-runs the forward over the whole sequence."""
        seq = list(int(t) for t in prompt)
        out = []
        for _ in range(n):
            nxt = int(torch.argmax(self.forward(seq)))
            out.append(nxt)
            seq.append(nxt)
        return out

    def generate_cached(self, prompt, n):
        cache = [None] * self.NL
        logits = self.forward(prompt, cache)
        out = []
        for _ in range(n):
            nxt = int(torch.argmax(logits))
            out.append(nxt)
            if len(out) < n:
                logits = self.forward([nxt], cache)
        return out


def time_generation(model, prompt, n, mode):
    t0 = time.perf_counter()
    ids = model.generate_full(prompt, n) if mode == "full" else model.generate_cached(prompt, n)
    dt = time.perf_counter() - t0
    return ids, dt
