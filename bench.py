#!/usr/bin/env python3
"""Benchmark of the inference token loop on one MI355X.

Workload (N=1): benchmark configuration 2 -- batch-1 greedy decode of the full-attention decoder
(d_model 768, 12 layers, 12 heads x 64, SwiGLU 2048, vocab 8192, fp32 weights N(0, 0.02) from seed 1),
64-token uniform-random prompt, KV cache up to 576.  A "step" is one decode step (one token through
the whole stack, LM head and argmax included); the token ids never leave the device between steps.

Prints ONE JSON line: decode tok/s (wall clock around exactly K steps, weights and KV resident in
HBM), the roofline of the dominant kernel measured live with HIP events on the context's stream, the
whole-step bytes-per-token roofline, and the CPU baseline (PyTorch restatement of the reference's
pytorch_verification model on this host's cores) timed on a bounded sample of the same workload.

Three decode paths exist and all are timed; `value` is the one named in config.decode_path:
  xcd         one launch covers all K steps; every XCD is a tensor-parallel rank (its heads, its FFN units),
              exchanges inside an XCD go through its L2, two per layer cross XCDs (default)
  persistent  one launch of the persistent kernel covers all K steps, phases separated by a grid barrier
              built from agent-scope atomics
  kernels     a sequence of per-phase kernels per step (plain launches or hipGraph replays)

Protocol: every figure is the median of REPS (5) timed repetitions of the same work, each with the device idle on
both sides; minimum and maximum are reported beside it.
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
MFMA_BF16_PEAK = 2.5e15  # MI355X dense bf16 MFMA, published peak (flop/s)
PROMPT_LEN = 64
REPS = 5  # timed repetitions per figure; the median is reported


def stats(xs):
    xs = sorted(float(x) for x in xs)
    return {"median": xs[len(xs) // 2], "min": xs[0], "max": xs[-1], "reps": len(xs)}


def physical_cores():
    """Physical cores of this host: distinct (physical id, core id) pairs of /proc/cpuinfo (logical CPUs if absent)."""
    try:
        pairs, phys, core = set(), None, None
        for line in open("/proc/cpuinfo"):
            if line.startswith("physical id"):
                phys = line.split(":")[1].strip()
            elif line.startswith("core id"):
                core = line.split(":")[1].strip()
            elif not line.strip():
                if phys is not None and core is not None:
                    pairs.add((phys, core))
                phys = core = None
        if phys is not None and core is not None:
            pairs.add((phys, core))
        return len(pairs) or (os.cpu_count() or 1)
    except OSError:
        return os.cpu_count() or 1


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


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


def _cpu_model(model, hp):
    import torch
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import cpu_model

    # one thread per physical core, within the share of the host this job has (OMP_NUM_THREADS is set to it on the box)
    share = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    threads = max(1, min(physical_cores(), share))
    tensors = {("E",): model.tensor(0, 0), ("gammaF",): model.tensor(0, 1)}
    for l in range(hp.transformers):
        for tid in range(2, 11):
            tensors[(l, tid)] = model.tensor(l, tid)
    return cpu_model.CpuModel(hp, tensors, threads=threads), cpu_model, torch


def cpu_baseline_one(what, model, hp, prompt, gpu_ids, n_full, n_cached, runs=3):
    """The PyTorch restatement of the reference's pytorch_verification model on this host's cores: after a warm-up,
    `runs` repetitions each of n_full greedy tokens in the reference's algorithmic form (every token recomputes all
    positions, inference_orchestrator.cu:64-65) and of n_cached tokens with a KV cache; medians are reported.  The
    ids are compared with the GPU's for the same prompt (fp32 on both sides: equal unless two logits tie)."""
    cm, cpu_model, torch = _cpu_model(model, hp)
    # before any timing is reported: the restatement's logits for the prompt against the float64 oracle's (the oracle
    # is the checker here, nothing of it is timed)
    orc = entry.load_oracle()
    want = orc.forward_full(orc.Weights.from_model(model), prompt, "f64")["logits"][0]
    got = cm.forward(prompt).numpy().astype(np.float64)
    logit_err = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
    cm.generate_full(prompt, 2)  # warm-up
    full, cached, ids_full, ids_cached = [], [], None, None
    for _ in range(runs):
        ids_full, dt = cpu_model.time_generation(cm, prompt, n_full, "full")
        full.append(n_full / dt)
    for _ in range(runs):
        ids_cached, dt = cpu_model.time_generation(cm, prompt, n_cached, "cached")
        cached.append(n_cached / dt)
    gpu = [int(t) for t in gpu_ids]
    return {
        "value": stats(full)["median"], "unit": "tok/s", "cores": torch.get_num_threads(), "kind": "port",
        "value_stats": stats(full),
        "sample": (f"{what}: {n_full} greedy tokens after the {len(prompt)}-token prompt, full recompute of all positions "
                   f"per token as the reference's runInferenceLoop does, median of {runs} runs after a warm-up; "
                   f"PyTorch {torch.__version__} CPU fp32"),
        "with_kv_cache_tok_s": stats(cached)["median"], "with_kv_cache_stats": stats(cached),
        "with_kv_cache_sample": f"{n_cached} greedy tokens, median of {runs} runs",
        "host_cpu_count": os.cpu_count(), "host_physical_cores": physical_cores(), "host_cpu_model": cpu_model_name(),
        "prompt_logits_vs_float64_oracle": {"max_abs_diff_over_max_logit": logit_err, "within_1e-5": logit_err <= 1e-5},
        "first_ids": ids_full[:8], "first_ids_cached": ids_cached[:8],
        "ids_equal_gpu": (ids_full[:len(gpu)] == gpu[:len(ids_full)] and ids_cached[:len(gpu)] == gpu[:len(ids_cached)]),
        "ids_compared": [min(len(gpu), len(ids_full)), min(len(gpu), len(ids_cached))],
    }


def config1_decode_leg(m, steps=128):
    """Configuration 1 (the pytorch_verification class of model: d256, 4 layers, 4 heads x 64, ffn 704, vocab 4096,
    fp32, seed 0, 16-token prompt, 128 greedy steps) on the GPU.  Its 17 MB of weights stay in the 256 MB Infinity
    Cache (and mostly in the L2s), so no HBM-bandwidth fraction is claimed for it: tok/s only."""
    hp = m.config(1)
    model = m.Model.generate(hp, seed=0)
    prompt = m.random_tokens(0, 0, hp.vocabSize, 16)
    dev = m.Device(hp, 0)
    dev.upload(model)
    walls, ids = [], None
    for i in range(REPS + 1):  # the first repetition is the warm-up
        dev.reset()
        dev.prefill(0, prompt)
        first = dev.greedy_token(0)
        dev.synchronize()
        t0 = time.perf_counter()
        out = dev.decode_loop([first], steps - 1)
        dev.synchronize()
        if i > 0:
            walls.append(time.perf_counter() - t0)
        ids = [first] + [int(t) for t in out[:, 0]]
    wall = stats(walls)["median"]
    path = {0: "kernels", 1: "persistent", 3: "xcd" if dev.xcd_decode_supported() else "persistent"}[dev.get_persistent()]
    dev.close()
    return ({"workload": "config 1: batch-1 greedy decode, d256 x 4 layers x 4 heads x 64, ffn 704, vocab 4096, fp32 weights "
                         "seed 0, 16-token prompt, 128 greedy tokens", "steps": steps - 1, "tok_s": (steps - 1) / wall,
             "ms_per_step": wall / (steps - 1) * 1e3, "ms_per_step_stats": stats([w / (steps - 1) * 1e3 for w in walls]),
             "decode_path": path, "weights_bytes": decode_bytes_per_token(hp, 0) - hp.transformers * 2 * hp.dim * 4,
             "weights_resident_in_infinity_cache": True,
             "note": "17 MB of weights: cache-resident, latency-bound; no bandwidth fraction claimed", "first_ids": ids[:8]},
            model, hp, prompt, ids)


def reference_default_decode_leg(m, steps=256):
    """The shape the reference ships compiled in (network_meta.h:3-20: dim 768, 6 heads x 128, ffn 3072, 16 layers,
    vocabulary 20160, QK-norm and query gating on, maxL 1280) with its uniform +-0.02 init (random_weights.cu:15-25,
    own generator): batch-1 greedy decode after a 256-token prompt -- what a user of the reference's main() runs."""
    hp = m.reference_defaults()
    plen, warm = 256, 16
    model = m.Model.new(hp)
    model.init_uniform(9, 0.02)
    dev = m.Device(hp, 0)
    dev.upload(model)
    dev.prefill(0, m.random_tokens(9, 0, hp.vocabSize, plen))
    out = dev.decode_loop([dev.greedy_token(0)], warm)
    steps = min(steps, (hp.maxL - plen - warm) // REPS)
    walls = []
    for _ in range(REPS):
        dev.synchronize()
        t0 = time.perf_counter()
        out = dev.decode_loop([int(out[-1, 0])], steps)
        dev.synchronize()
        walls.append(time.perf_counter() - t0)
    wall = stats(walls)["median"]
    nbytes = float(np.mean([decode_bytes_per_token(hp, plen + warm + 1 + i) for i in range(REPS * steps)]))
    path = {0: "kernels", 1: "persistent", 3: "xcd" if dev.xcd_decode_supported() else "persistent"}[dev.get_persistent()]
    fell_back = dev.persistent_fallbacks()
    dev.close()
    return {"workload": "reference-default shape: batch-1 greedy decode, d768 x 16 layers x 6 heads x 128, ffn 3072, vocab 20160, "
                        "QK-norm + query gating, fp32 uniform +-0.02, 256-token prompt", "steps": steps,
            "ms_per_step": wall / steps * 1e3, "tok_s": steps / wall, "ms_per_step_stats": stats([w / steps * 1e3 for w in walls]),
            "decode_path": path, "fallbacks": fell_back, "bytes_per_token": nbytes, "achieved_GBps": nbytes / (wall / steps) / 1e9,
            "frac_of_hbm_peak": nbytes / (wall / steps) / 1e9 / HBM_PEAK_GBPS, "last_ids": [int(x) for x in out[-4:, 0]]}


def matrix_params(hp):
    """Weight-matrix elements one token multiplies on its way through the stack (LM head excluded)."""
    d, F, total = hp.dim, hp.ffnDim, 0
    for t in range(hp.transformers):
        if hp.layerKinds[t] == 0:
            total += 4 * d * d + 3 * d * F + (d * d if hp.queryGating else 0)
        else:
            qk, vv = hp.gdnHeads * hp.gdnDk, hp.gdnHeads * hp.gdnDv
            total += 2 * qk * d + 2 * vv * d + 3 * d * F + 2 * hp.gdnHeads * d
        if hp.pleDim:
            total += 2 * hp.pleDim * d
    return total


def batched_decode_leg(m, steps=48):
    """Configuration 4: 64 concurrent sequences of the hybrid architecture, prompt lengths uniform in
    [32, 512] (seeded), greedy decode.  Returns tok/s and the fraction of the bytes-per-step roofline
    (weights once per step + every sequence's K/V rows and GDN states)."""
    hp = m.config(4)
    nseq = hp.maxSeqs
    model = m.Model.generate(hp, seed=4)
    dev = m.Device(hp, 0)
    dev.upload(model)
    lens = np.random.default_rng(4).integers(32, 513, size=nseq)
    prompts = [m.random_tokens(4, s, hp.vocabSize, int(n)) for s, n in enumerate(lens)]
    dev.prefill_batch(list(range(nseq)), prompts)
    firsts = [dev.greedy_token(s) for s in range(nseq)]
    out = dev.decode_loop(firsts, 8)  # warm-up
    walls = []
    for _ in range(REPS):
        dev.synchronize()
        t0 = time.perf_counter()
        out = dev.decode_loop([int(t) for t in out[-1]], steps)
        dev.synchronize()
        walls.append(time.perf_counter() - t0)
    wall = stats(walls)["median"]
    wb = 2 if hp.weightDtype == m.DTYPE_BF16 else 4
    weights = decode_bytes_per_token(hp, 0, wb) - sum(
        (2 * hp.dim * 4 if hp.layerKinds[t] == 0 else 2 * hp.gdnHeads * hp.gdnDk * hp.gdnDv * 4) for t in range(hp.transformers))
    per_seq = [decode_bytes_per_token(hp, int(n) + 8 + (REPS * steps) // 2, wb) - weights for n in lens]
    step_bytes = weights + float(np.sum(per_seq))
    dev.close()
    return {"workload": "config 4: 64 sequences, prompts uniform in [32, 512], hybrid 3 GDN : 1 attention + PLE, fp32",
            "steps": steps, "ms_per_step": wall / steps * 1e3, "tok_s": nseq * steps / wall,
            "ms_per_step_stats": stats([w / steps * 1e3 for w in walls]),
            "bytes_per_step": step_bytes, "achieved_GBps": step_bytes / (wall / steps) / 1e9,
            "frac_of_hbm_peak": step_bytes / (wall / steps) / 1e9 / HBM_PEAK_GBPS,
            "last_ids": [int(x) for x in out[-1, :4]]}


def hybrid_decode_leg(m, steps=192):
    """Configuration 3: batch-1 greedy decode of the hybrid architecture (3 GDN : 1 attention + PLE) after a
    128-token prompt.  Returns tok/s and the fraction of the bytes-per-token roofline (weights, GDN states read and
    written, K/V rows of the attention layers)."""
    hp = m.config(3)
    hp.maxSeqs = 1
    plen, warm = 128, 16
    model = m.Model.generate(hp, seed=3)
    dev = m.Device(hp, 0)
    dev.upload(model)
    dev.prefill(0, m.random_tokens(3, 0, hp.vocabSize, plen))
    out = dev.decode_loop([dev.greedy_token(0)], warm)
    walls = []
    steps = min(steps, (hp.maxL - plen - warm) // REPS)
    for _ in range(REPS):
        dev.synchronize()
        t0 = time.perf_counter()
        out = dev.decode_loop([int(out[-1, 0])], steps)
        dev.synchronize()
        walls.append(time.perf_counter() - t0)
    wall = stats(walls)["median"]
    nbytes = float(np.mean([decode_bytes_per_token(hp, plen + warm + 1 + i) for i in range(REPS * steps)]))
    dev.close()
    return {"workload": "config 3: batch-1 greedy decode, hybrid 3 GDN : 1 attention + PLE at config-2 size, fp32, "
                        "128-token prompt", "steps": steps, "ms_per_step": wall / steps * 1e3, "tok_s": steps / wall,
            "ms_per_step_stats": stats([w / steps * 1e3 for w in walls]),
            "bytes_per_token": nbytes, "achieved_GBps": nbytes / (wall / steps) / 1e9,
            "frac_of_hbm_peak": nbytes / (wall / steps) / 1e9 / HBM_PEAK_GBPS, "last_ids": [int(x) for x in out[-4:, 0]]}


def prefill_leg(m, reps=REPS, with_gemm=True):
    """Configuration 5: 8 prompts of 2048 uniform-random tokens through the bf16 model in one pass.
    MFMA utilisation = algorithmic flops (projections + causal attention, LM head on the last position
    only) / time / the published dense bf16 peak; the GEMM kernel alone is also timed on the pass's own
    gate/up shape (M = 16384 rows)."""
    hp = m.config(5)
    nseq, plen = hp.maxSeqs, 2048
    model = m.Model.generate(hp, seed=5)
    dev = m.Device(hp, 0)
    dev.upload(model)
    prompts = [m.random_tokens(5, s, hp.vocabSize, plen) for s in range(nseq)]
    times = []
    for i in range(reps + 1):  # the first pass allocates the work buffers and is not counted
        dev.reset()
        dev.synchronize()
        t0 = time.perf_counter()
        dev.prefill_batch(list(range(nseq)), prompts)
        dt = time.perf_counter() - t0
        if i > 0:
            times.append(dt)
    med = stats(times)["median"]
    tokens = nseq * plen
    n_attn = sum(1 for t in range(hp.transformers) if hp.layerKinds[t] == 0)
    flops = 2.0 * tokens * matrix_params(hp) + n_attn * nseq * (4.0 * plen * plen * hp.dim) / 2 + 2.0 * nseq * hp.vocabSize * hp.dim
    firsts = [dev.greedy_token(s) for s in range(nseq)]
    decs = []
    for _ in range(REPS):
        dev.synchronize()
        t0 = time.perf_counter()
        firsts = [int(t) for t in dev.decode_loop(firsts, 16)[-1]]
        decs.append((time.perf_counter() - t0) / 16)
    dec = stats(decs)["median"]
    dev.close()
    gemm = gemm_leg(m, iters=10, reps=REPS) if with_gemm else None
    return {"workload": "config 5: 8 x 2048-token prompts, d2048 x 24 layers (3 GDN : 1 attention), 16 heads x 128, "
                        "ffn 5632, vocab 32000, PLE 64, bf16 weights, fp32 accumulation",
            "tokens": tokens, "ms": med * 1e3, "ms_stats": stats([t * 1e3 for t in times]), "tok_s": tokens / med,
            "algo_tflop": flops / 1e12,
            "achieved_TFLOPs": flops / med / 1e12, "mfma_frac_of_bf16_peak": flops / med / MFMA_BF16_PEAK,
            "gemm_kernel": gemm,
            "decode_after_prefill": {"sequences": nseq, "ms_per_step": dec * 1e3, "tok_s": nseq / dec,
                                     "ms_per_step_stats": stats([d * 1e3 for d in decs])}}


def gemm_leg(m, iters=3, reps=1):
    """The gate/up product of one config-5 prefill pass alone (16384 x 11264 x 2048, half operands -- what the bf16
    model's MFMA path multiplies --, N(0,1) data), timed with HIP events: SiLU(gate) * up in the epilogue, half output,
    as the pass runs it.  Top level: ten launches back to back (sustained clock).  Beside it: single launches with the
    device idle in between, the plain fp32 epilogue back to back, the kernel on all-zero operands and the vendor library
    on the same operands.  With reps == 1 (profiler and counter runs) both epilogues are launched `iters` times and
    only the plain timing is reported."""
    hp = m.config(5)
    M = 8 * 2048
    rng = np.random.default_rng(5)
    a = rng.standard_normal((M, hp.dim), dtype=np.float32)
    b = rng.standard_normal((2 * hp.ffnDim, hp.dim), dtype=np.float32)
    flop = 2.0 * M * 2 * hp.ffnDim * hp.dim

    def fig(us_list):
        us = stats(us_list)["median"]
        return {"avg_us": us, "avg_us_stats": stats(us_list), "TFLOPs": flop / us / 1e6, "frac_of_bf16_peak": flop / us / 1e6 * 1e12 / MFMA_BF16_PEAK}

    if reps == 1:
        m.selftest_gemm(a, b, None, f16=True, iters=iters, swiglu=True)
        out = fig([m.selftest_gemm(a, b, None, f16=True, iters=iters)[1]])
        out.update({"shape": [M, 2 * hp.ffnDim, hp.dim], "iters": iters, "epilogue": "plain, fp32 output"})
        return out
    m.selftest_gemm(a, b, None, f16=True, iters=2, swiglu=True)  # warm
    singles = []
    for _ in range(9):
        time.sleep(0.05)
        singles.append(m.selftest_gemm(a, b, None, f16=True, iters=1, swiglu=True)[1])
    # Two protocols, both reported with the same weight.  Sustained: `iters` launches back to back (HIP events around
    # the run, median of `reps` runs) -- the part's clock settles under the load; this is the figure comparable
    # from round to round and with the vendor yardstick below, and the one at the top level of this object.  Single:
    # one launch at a time with 50 ms of idle before it -- the clock has not come down yet; in the prefill pass a
    # GEMM is followed by lighter kernels and runs between the two (the profiler's per-kernel average says where).
    b2b = [m.selftest_gemm(a, b, None, f16=True, iters=iters, swiglu=True)[1] for _ in range(reps)]
    out = fig(b2b)
    out.update({"shape": [M, 2 * hp.ffnDim, hp.dim], "epilogue": "SiLU(gate) * up, half output (as the prefill pass runs this product)",
                "protocol": "%d launches back to back, HIP events around the run, median of %d runs" % (iters, reps)})
    out["back_to_back_%d_launches_swiglu_epilogue" % iters] = fig(b2b)
    out["single_launches_idle_between"] = dict(fig(singles), protocol="median of 9 single launches, 50 ms idle before each, HIP events around the launch")
    plain = fig([m.selftest_gemm(a, b, None, f16=True, iters=iters)[1] for _ in range(reps)])
    out["back_to_back_%d_launches_plain_fp32_epilogue" % iters] = plain
    # Two yardsticks on the same box in the same run, neither on the product path: the same kernel on all-zero
    # operands (no switching activity: what the code alone allows, without the part's power management), and the
    # vendor library's GEMM (torch.matmul -> hipBLASLt) on the same shape, type and data distribution.
    z = np.zeros_like(a), np.zeros_like(b)
    uz = stats([m.selftest_gemm(z[0], z[1], None, f16=True, iters=iters)[1] for _ in range(3)])["median"]
    out["same_kernel_zero_operands_plain_epilogue"] = {"avg_us": uz, "TFLOPs": flop / uz / 1e6}
    try:
        out["vendor_library_yardstick"] = vendor_gemm(a, b, iters, reps, flop)
        out["back_to_back_ratio_to_vendor_library"] = out["vendor_library_yardstick"]["avg_us"] / out["back_to_back_%d_launches_swiglu_epilogue" % iters]["avg_us"]
    except Exception as e:  # a yardstick, never required
        out["vendor_library_yardstick"] = {"failed": repr(e)}
    return out


def vendor_gemm(a, b, iters, reps, flop):
    """torch.matmul (the vendor BLAS library) on the GEMM leg's operands: a yardstick beside the hand-written kernel."""
    import torch
    ta = torch.from_numpy(a).to("cuda:0", dtype=torch.float16)
    tb = torch.from_numpy(b).to("cuda:0", dtype=torch.float16)
    res = {}
    for label, (x, y) in (("normal_data", (ta, tb)), ("zero_operands", (torch.zeros_like(ta), torch.zeros_like(tb)))):
        for _ in range(3):
            x @ y.t()
        torch.cuda.synchronize()
        runs = []
        for _ in range(reps if label == "normal_data" else 3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                x @ y.t()
            e1.record()
            torch.cuda.synchronize()
            runs.append(e0.elapsed_time(e1) * 1e3 / iters)
        res[label] = {"avg_us": stats(runs)["median"], "TFLOPs": flop / stats(runs)["median"] / 1e6}
    return {"what": "torch.matmul, fp16, same shape and N(0,1) data, back-to-back launches", "avg_us": res["normal_data"]["avg_us"],
            "TFLOPs": res["normal_data"]["TFLOPs"], "frac_of_bf16_peak": res["normal_data"]["TFLOPs"] * 1e12 / MFMA_BF16_PEAK,
            "zero_operands": res["zero_operands"]}


def timed_decode(dev, prompt, K, W, persistent, maxL):
    """W untimed warm-up steps, then REPS repetitions of exactly K timed steps from the same starting state (prompt
    prefilled anew each time), the device idle on both sides of each.  Returns (wall seconds per repetition, HIP-event
    milliseconds per repetition of a second series timed on the context's stream, ids)."""
    dev.set_persistent(persistent)
    dev.reset()
    dev.prefill(0, prompt)
    first = dev.greedy_token(0)
    if W:
        dev.decode_loop([first], min(W, maxL - PROMPT_LEN))
    walls, events, ids = [], [], None
    for _ in range(REPS):
        dev.reset()
        dev.prefill(0, prompt)
        first = dev.greedy_token(0)
        dev.synchronize()
        t0 = time.perf_counter()
        ids = dev.decode_loop([first], K)
        dev.synchronize()
        walls.append(time.perf_counter() - t0)
    for _ in range(REPS):
        dev.reset()
        dev.prefill(0, prompt)
        events.append(dev.time_decode([first], K))
    return walls, events, np.concatenate([[first], ids[:, 0]]).astype(np.int32)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--path", choices=["xcd", "persistent", "kernels"], default="xcd",
                    help="decode path reported as `value`")
    ap.add_argument("--no-extras", action="store_true", help="skip the batched-decode (config 4) and prefill (config 5) legs")
    ap.add_argument("--leg", choices=["all", "batched", "prefill", "gemm", "hybrid", "config1", "refdefault"], default="all",
                    help="profiler runs: run only the batched-decode leg, the prefill leg, the big GEMM alone, the "
                         "batch-1 hybrid decode leg, configuration 1 or the reference-default shape and print its JSON object")
    ap.add_argument("--passes", type=int, default=2, help="--leg prefill: timed passes over the 8 x 2048-token batch")
    ap.add_argument("--only-path", action="store_true", help="time only the chosen path (for profiler runs)")
    ap.add_argument("--graph-steps", type=int, default=0,
                    help="kernels path: decode steps per hipGraph replay; 0 = plain launches (use 0 under rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the token loop runs on a single MI355X); "
              "--gpus must be 1", file=sys.stderr)
        return 2

    m = entry.load_package()
    if args.leg != "all":
        leg = {"batched": batched_decode_leg, "prefill": lambda mm: prefill_leg(mm, reps=max(1, args.passes), with_gemm=False),
               "gemm": gemm_leg, "hybrid": hybrid_decode_leg, "config1": lambda mm: config1_decode_leg(mm)[0],
               "refdefault": reference_default_decode_leg}[args.leg]
        print(json.dumps({args.leg: leg(m)}))
        return 0
    hp = m.config(2)
    K, W = max(1, args.steps), max(0, args.warmup)
    if PROMPT_LEN + K > hp.maxL:
        hp.maxL = PROMPT_LEN + K
    model = m.Model.generate(hp, seed=1)
    prompt = m.random_tokens(1, 0, hp.vocabSize, PROMPT_LEN)
    dev = m.Device(hp, 0)
    dev.upload(model)
    dev.set_graph(args.graph_steps)

    paths = {}
    if args.path == "xcd" and not dev.xcd_decode_supported():
        print("bench.py: the XCD-rank kernel does not cover this device; use --path persistent", file=sys.stderr)
        return 4
    order = [args.path] if args.only_path else ["kernels", "persistent", "xcd"]
    ids_by_path = {}
    for name in order:
        walls, events, ids = timed_decode(dev, prompt, K, W, {"kernels": 0, "persistent": 1, "xcd": 3}[name], hp.maxL)
        wall = stats(walls)["median"]
        paths[name] = {"tok_s": K / wall, "ms_per_step": wall / K * 1e3, "ms_per_step_stats": stats([w / K * 1e3 for w in walls]),
                       "event_ms_per_step": stats(events)["median"] / K,
                       "event_ms_per_step_stats": stats([e / K for e in events])}
        ids_by_path[name] = ids  # the token the prefill picked, then the K decoded ones
        if dev.persistent_fallbacks():
            print(f"bench.py: path {name} gave up a wait and fell back to the kernel sequence: {m.dev.mlh_last_error(dev._h).decode()}", file=sys.stderr)
            return 5
    if any(not np.array_equal(v, ids_by_path[args.path]) for v in ids_by_path.values()):
        print("bench.py: the decode paths produced different ids", file=sys.stderr)
        return 3
    chosen = paths[args.path]
    wall_per_step = chosen["ms_per_step"] / 1e3
    ids = ids_by_path[args.path]

    mean_bytes = float(np.mean([decode_bytes_per_token(hp, PROMPT_LEN + 1 + i) for i in range(K)]))
    step_gbps = mean_bytes / wall_per_step / 1e9

    # per-kernel times inside the decode sequence: a HIP event after every launch on the context's
    # stream, over 64 further steps from the middle of the run (run time plus the launch gap before it)
    dev.set_persistent(0)
    dev.reset()
    dev.prefill(0, prompt)
    mid = max(0, min(K // 2, hp.maxL - PROMPT_LEN - 65))
    tok = dev.greedy_token(0)
    if mid > 0:
        tok = int(dev.decode_loop([tok], mid)[-1, 0])
    nprof = min(64, hp.maxL - PROMPT_LEN - mid)
    prof = dev.profile_decode([tok], nprof)
    T_mid = PROMPT_LEN + mid + nprof // 2
    algo = {"k_phaseA": 4.0 * 3 * hp.dim * hp.dim, "k_attn": 2.0 * 4 * hp.dim * (T_mid + 1) + 2.0 * 4 * hp.dim,
            "k_oproj": 4.0 * hp.dim * hp.dim, "k_ffn13": 4.0 * 2 * hp.ffnDim * hp.dim,
            "k_down": 4.0 * hp.dim * hp.ffnDim, "k_lmhead": 4.0 * hp.vocabSize * hp.dim}
    kernels = {}
    for name, (us, n) in prof.items():
        if us <= 0:
            continue
        kernels[name] = {"avg_us_in_sequence": round(us, 3), "launches_per_token": n,
                         "algo_bytes": algo.get(name, 0.0),
                         "GBps": round(algo.get(name, 0.0) / us / 1e3, 1) if us > 0 else None}
    copy_us, copy_bytes = dev.time_kernel(m.K_COPY, iters=20)

    hops = None
    try:
        h = dev.probe_hops(2000)
        # A layer of the XCD-rank kernel is 2 exchanges across XCDs, each followed by a gather inside the XCD, plus 3
        # exchanges inside the XCD, plus its five compute phases: the floor these hop times put under a layer pass.
        hops = {"in_xcd_us": h[0], "cross_xcd_us": h[1], "grid_barrier_us": h[2], "rounds": 2000,
                "what": "one all-to-all of dim tagged words among the 32 workgroups of an XCD / among all 256 / one grid barrier",
                "layer_floor_us_xcd_kernel": 2 * (h[1] + h[0]) + 3 * h[0] if min(h[0], h[1]) > 0 else None,
                "layer_floor_formula": "2 x (cross + in-XCD gather) + 3 x in-XCD, compute phases not counted"}
    except Exception as e:  # a probe, never required
        hops = {"failed": repr(e)}
    try:  # what the matrix cores sustain from registers alone, by instruction form and operand data, and the load path alone
        mfma = {"what": "register-only half-precision MFMA loop on every SIMD, TFLOP/s (nominal dense peak 2500); the part's "
                        "clock follows the power the operand data draws",
                "mfma_32x32x16": {"zeros": dev.probe_mfma(0, 0), "unit_variance": dev.probe_mfma(0, 1)},
                "mfma_16x16x32": {"zeros": dev.probe_mfma(1, 0), "unit_variance": dev.probe_mfma(1, 1)},
                "direct_to_lds_loads_TBps": dev.probe_lds_loads()}
    except Exception as e:
        mfma = {"failed": repr(e)}

    if args.path in ("persistent", "xcd"):
        # the dominant (only) kernel: one launch = K tokens; duration from HIP events around the launch (median of REPS)
        launch_us = chosen["event_ms_per_step"] * K * 1e3
        launch_bytes = mean_bytes * K
        # HBM bytes per launch are not counted in this run: the ratio of counted to algorithmic bytes comes from the
        # tracked profile (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, one run each, scaled by what the same counters read
        # for the 256 MiB copy kernel: reads x 2.0, writes x 1.0), taken on a 16-token launch of the XCD-rank kernel:
        # 381.7 MB read + 3.4 MB written per token against 370.4 MB algorithmic at those lengths.
        traffic_ratio = {"xcd": 1.04}.get(args.path)
        roofline = {"kernel": {"persistent": "k_decode_persistent", "xcd": "k_decode_xcd"}[args.path], "bound": "hbm", "achieved": launch_bytes / launch_us / 1e3,
                    "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": launch_bytes / launch_us / 1e3 / HBM_PEAK_GBPS,
                    "traffic": traffic_ratio * launch_bytes if traffic_ratio else None,
                    "traffic_source": ("profiles/decode_config2_hbm_traffic.md: counter ratio 1.04 from a 16-token launch under "
                                       "rocprofv3 --pmc, applied to this run's algorithmic bytes; not counted in this run") if traffic_ratio else None,
                    "avg_launch_us": launch_us,
                    "avg_launch_us_stats": {k: (v * K * 1e3 if k != "reps" else v) for k, v in chosen["event_ms_per_step_stats"].items()},
                    "algo_bytes_per_launch": launch_bytes, "tokens_per_launch": K}
    else:
        # dominant = the kernel with the largest share of the step's time
        dom = max(kernels, key=lambda k: kernels[k]["avg_us_in_sequence"] * kernels[k]["launches_per_token"])
        kd = kernels[dom]
        gbps = kd["algo_bytes"] / kd["avg_us_in_sequence"] / 1e3
        # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters
        # read for a plain copy of known size (see profiles/); only known for the kernels measured there
        traffic_ratio = {"k_attn": 1.46, "k_ffn13": 1.01, "k_phaseA": 1.02, "k_down": 1.02, "k_oproj": 1.08,
                         "k_lmhead": 1.01}.get(dom)
        traffic = traffic_ratio * kd["algo_bytes"] if traffic_ratio else None
        roofline = {"kernel": dom, "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": gbps / HBM_PEAK_GBPS, "traffic": traffic, "avg_launch_us": kd["avg_us_in_sequence"],
                    "algo_bytes_per_launch": kd["algo_bytes"], "share_of_step_time":
                        kd["avg_us_in_sequence"] * kd["launches_per_token"] / sum(
                            v["avg_us_in_sequence"] * v["launches_per_token"] for v in kernels.values())}

    cpu = None
    if not args.no_cpu:
        try:
            cpu = cpu_baseline_one("config 2", model, hp, prompt, ids, n_full=32, n_cached=96)
        except Exception as e:  # the baseline is reported, never required
            cpu = {"value": None, "unit": "tok/s", "cores": 0, "kind": "port", "sample": f"failed: {e!r}"}

    dev.close()
    extras = {}
    if not args.no_extras and not args.only_path:
        try:  # configuration 1 on the GPU, and the same workload on the host cores beside it
            extras["config1_decode"], model1, hp1, prompt1, ids1 = config1_decode_leg(m)
            if cpu is not None and cpu.get("value"):
                cpu["config1"] = cpu_baseline_one("config 1", model1, hp1, prompt1, ids1, n_full=64, n_cached=127)
            del model1
        except Exception as e:
            extras["config1_decode"] = {"failed": repr(e)}
        for name, leg in (("reference_default_decode", reference_default_decode_leg), ("batched_decode", batched_decode_leg),
                          ("hybrid_decode", hybrid_decode_leg), ("prefill", prefill_leg)):
            try:
                extras[name] = leg(m)
            except Exception as e:  # reported alongside, never required for the headline line
                extras[name] = {"failed": repr(e)}

    line = {
        "metric": "decode tok/s @ batch 1 (config 2) + % HBM roofline",
        "value": chosen["tok_s"],
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": chosen["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "config 2: batch-1 greedy decode, d768 x 12 layers x 12 heads x 64, ffn 2048, "
                               "vocab 8192, fp32 weights seed 1, 64-token prompt, KV to %d" % hp.maxL,
                   "prompt_len": PROMPT_LEN, "kv_max": int(hp.maxL), "decode_path": args.path,
                   "steps_per_graph": args.graph_steps},
        "roofline": roofline,
        "decode_roofline": {"bound": "hbm", "bytes_per_token": mean_bytes, "achieved": step_gbps,
                            "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": step_gbps / HBM_PEAK_GBPS,
                            "weights_resident_in_infinity_cache": False,
                            "note": "365 MB of fp32 weights exceed the 256 MB Infinity Cache"},
        "paths": paths,
        "protocol": f"median of {REPS} timed repetitions per figure (min and max beside it)",
        "exchange_latency": hops,
        "mfma_register_loop": mfma,
        "kernels": kernels,
        "copy_kernel": {"avg_us": round(copy_us, 2), "GBps": round(copy_bytes / copy_us / 1e3, 1)},
        "cpu_baseline": cpu,
        "first_ids": [int(x) for x in ids[:8]],
        "last_ids": [int(x) for x in ids[-4:]],
    }
    line.update(extras)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
