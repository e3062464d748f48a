#!/usr/bin/env python3
"""Benchmark of the inference token loop on one MI355X.

Workload (N=1): benchmark configuration 2 -- batch-1 greedy decode of the full-attention decoder
(d_model 768, 12 layers, 12 heads x 64, SwiGLU 2048, vocab 8192, fp32 weights N(0, 0.02) from seed 1),
64-token uniform-random prompt, KV cache up to 576.  A "step" is one decode step (one token through
the whole stack, LM head and argmax included); the token ids never leave the device between steps.

Prints ONE JSON line: decode tok/s (wall clock around K steps, weights and KV resident in HBM), the
roofline of the dominant kernel measured live with HIP events on the context's stream, the whole-step
bytes-per-token roofline, and the CPU baseline (PyTorch restatement of the reference's
pytorch_verification model on this host's cores) timed on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
PROMPT_LEN = 64


def decode_bytes_per_token(hp, T, wbytes=4):
    """Algorithmic bytes one batch-1 decode step must move with T positions in the cache after the
    step: every weight matrix once, K and V rows of the attention layers read once and one row
    written, GDN states read and written.  Gains, activations and partials are left out."""
    d, F, V, NL = hp.dim, hp.ffnDim, hp.vocabSize, hp.transformers
    total = wbytes * V * d
    for t in range(NL):
        if hp.layerKinds[t] == 0:
            total += wbytes * (4 * d * d + 3 * d * F + (d * d if hp.queryGating else 0))
            total += 2 * T * d * 4 + 2 * d * 4
        else:
            qk, vv = hp.gdnHeads * hp.gdnDk, hp.gdnHeads * hp.gdnDv
            total += wbytes * (2 * qk * d + 2 * vv * d + 3 * d * F + 2 * hp.gdnHeads * d)
            total += 2 * hp.gdnHeads * hp.gdnDk * hp.gdnDv * 4
        if hp.pleDim:
            total += wbytes * (2 * hp.pleDim * d + hp.pleDim)
    return total


def cpu_baseline(m, model, hp, prompt, seconds_budget=20.0):
    """Reference-style CPU generation (full recompute per token) on a bounded sample."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import cpu_model

    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    tensors = {("E",): model.tensor(0, 0), ("gammaF",): model.tensor(0, 1)}
    for l in range(hp.transformers):
        for tid in range(2, 11):
            tensors[(l, tid)] = model.tensor(l, tid)
    cm = cpu_model.CpuModel(hp, tensors, threads=threads)
    cm.generate_full(prompt, 1)  # warm-up
    n_full, t_full = 0, 0.0
    ids_full = []
    seq = list(int(t) for t in prompt)
    t0 = time.perf_counter()
    while n_full < 64 and (time.perf_counter() - t0) < seconds_budget * 0.6:
        nxt = int(torch.argmax(cm.forward(seq)))
        seq.append(nxt)
        ids_full.append(nxt)
        n_full += 1
    t_full = time.perf_counter() - t0
    t1 = time.perf_counter()
    ids_cached = cm.generate_cached(prompt, 128)
    t_cached = time.perf_counter() - t1
    return {
        "value": n_full / t_full,
        "unit": "tok/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": (f"config 2, {n_full} greedy tokens after the {len(prompt)}-token prompt, full recompute of all "
                   f"positions per token as the reference's runInferenceLoop does; PyTorch {torch.__version__} CPU fp32"),
        "with_kv_cache_tok_s": 128 / t_cached,
        "host_cpu_count": os.cpu_count(),
        "first_ids": ids_full[:8],
        "first_ids_cached": ids_cached[:8],
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--graph-steps", type=int, default=1,
                    help="decode steps per hipGraph replay; 0 = plain launches (use 0 under rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the token loop runs on a single MI355X); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    m = entry.load_package()
    hp = m.config(2)
    K, W = max(1, args.steps), max(0, args.warmup)
    if PROMPT_LEN + K > hp.maxL:
        hp.maxL = PROMPT_LEN + K
    model = m.Model.generate(hp, seed=1)
    prompt = m.random_tokens(1, 0, hp.vocabSize, PROMPT_LEN)
    dev = m.Device(hp, 0)
    dev.upload(model)
    dev.set_graph(args.graph_steps)

    # warm-up: W untimed steps (this also captures the decode graph)
    dev.prefill(0, prompt)
    first = dev.greedy_token(0)
    if W:
        dev.decode_loop([first], min(W, hp.maxL - PROMPT_LEN))

    # timed region: exactly K decode steps, device idle on both sides
    dev.reset()
    dev.prefill(0, prompt)
    first = dev.greedy_token(0)
    dev.synchronize()
    t0 = time.perf_counter()
    ids = dev.decode_loop([first], K)
    dev.synchronize()
    wall = time.perf_counter() - t0
    tok_s = K / wall

    # the same K steps timed with HIP events on the context's stream
    dev.reset()
    dev.prefill(0, prompt)
    ev_ms = dev.time_decode([first], K)

    mean_bytes = float(np.mean([decode_bytes_per_token(hp, PROMPT_LEN + 1 + i) for i in range(K)]))
    step_gbps = mean_bytes / (wall / K) / 1e9

    # per-kernel durations (HIP events, back-to-back launches) at the mid-run cache length
    dev.reset()
    dev.prefill(0, prompt)
    mid = min(K // 2, hp.maxL - PROMPT_LEN - 1)
    if mid > 0:
        dev.decode_loop([first], mid)
    kernels = {}
    per_token_us = 0.0
    for kid, count in ((m.K_QKV, hp.transformers), (m.K_ATTN, hp.transformers), (m.K_OPROJ, hp.transformers),
                       (m.K_FFN_GATEUP, hp.transformers), (m.K_FFN_DOWN, hp.transformers), (m.K_LMHEAD, 1)):
        us, nbytes = dev.time_kernel(kid, layer=0, nseq=1, iters=200)
        name = m.dev.mlh_kernel_name(kid).decode()
        kernels[name] = {"avg_us": round(us, 3), "algo_bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                         "launches_per_token": count}
        per_token_us += us * count
    copy_us, copy_bytes = dev.time_kernel(m.K_COPY, iters=20)
    dom = max((k for k in kernels), key=lambda k: kernels[k]["avg_us"] * kernels[k]["launches_per_token"])
    roofline = {
        "kernel": dom,
        "bound": "hbm",
        "achieved": kernels[dom]["algo_bytes"] / kernels[dom]["avg_us"] / 1e3,
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": kernels[dom]["algo_bytes"] / kernels[dom]["avg_us"] / 1e3 / HBM_PEAK_GBPS,
        "traffic": None,
        "avg_launch_us": kernels[dom]["avg_us"],
        "algo_bytes_per_launch": kernels[dom]["algo_bytes"],
    }

    cpu = None
    if not args.no_cpu:
        try:
            cpu = cpu_baseline(m, model, hp, prompt)
        except Exception as e:  # the baseline is reported, never required
            cpu = {"value": None, "unit": "tok/s", "cores": 0, "kind": "port", "sample": f"failed: {e!r}"}

    line = {
        "metric": "decode tok/s @ batch 1 (config 2) + % HBM roofline",
        "value": tok_s,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": wall / K * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "config 2: batch-1 greedy decode, d768 x 12 layers x 12 heads x 64, ffn 2048, "
                               "vocab 8192, fp32 weights seed 1, 64-token prompt, KV to %d" % hp.maxL,
                   "prompt_len": PROMPT_LEN, "kv_max": int(hp.maxL), "steps_per_graph": args.graph_steps},
        "roofline": roofline,
        "decode_roofline": {"bound": "hbm", "bytes_per_token": mean_bytes, "achieved": step_gbps,
                            "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": step_gbps / HBM_PEAK_GBPS,
                            "weights_resident_in_infinity_cache": False,
                            "event_ms_per_step": ev_ms / K,
                            "sum_of_kernel_us_per_token": round(per_token_us, 1)},
        "kernels": kernels,
        "copy_kernel": {"avg_us": round(copy_us, 2), "GBps": round(copy_bytes / copy_us / 1e3, 1)},
        "cpu_baseline": cpu,
        "last_ids": [int(x) for x in ids[-4:, 0]],
    }
    print(json.dumps(line))
    dev.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
