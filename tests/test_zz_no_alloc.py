"""The entry point that allocates nothing (mlh_gemm_device: device pointers, split-K workspace in a static device
array) against the entry point it is a variant of (mlh_selftest_gemm: host arrays, workspace from hipMalloc), through
the C ABI: two calls in a row, the second with a smaller input, then the size limits.  torch only provides the
device memory and the stream here."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F16 = 2  # operand type code of IEEE-half operands (the mirrors a bf16 model's MFMA path multiplies)


def _run(pkg, torch, dtype, M, N, K, seed, with_r):
    rng = np.random.default_rng(seed)
    a = rng.normal(size=(M, K)).astype(np.float32)
    b = rng.normal(size=(N, K)).astype(np.float32)
    r = rng.normal(size=(M, N)).astype(np.float32) if with_r else None
    want, _ = pkg.selftest_gemm(a, b, r, bf16=(dtype == pkg.DTYPE_BF16), f16=(dtype == F16))
    tt = {pkg.DTYPE_F32: torch.float32, pkg.DTYPE_BF16: torch.bfloat16, F16: torch.float16}[dtype]
    da = torch.from_numpy(a).cuda().to(tt).contiguous()
    db = torch.from_numpy(b).cuda().to(tt).contiguous()
    dr = torch.from_numpy(r).cuda() if with_r else None
    dc = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream()
    rc = pkg.dev.mlh_gemm_device(dtype, M, N, K, da.data_ptr(), db.data_ptr(), dr.data_ptr() if with_r else None,
                                 dc.data_ptr(), ctypes.c_void_p(stream.cuda_stream))
    assert rc == 0, pkg.dev.mlh_last_error(None).decode()
    stream.synchronize()
    got = dc.cpu().numpy()
    # same kernels, same deterministic split-K reduction order: the two entry points agree bit for bit
    assert np.array_equal(got, want), f"M {M} N {N} K {K}: max |diff| {np.max(np.abs(got - want))}"
    if dtype == pkg.DTYPE_F32:
        ref = a.astype(np.float64) @ b.astype(np.float64).T + (r if with_r else 0)
        assert np.max(np.abs(got - ref)) <= 1e-5 * np.max(np.abs(ref))  # fp32 product against float64 NumPy
    return got


def test_no_alloc_gemm_matches_allocating_entry_point(pkg):
    import torch
    assert pkg.dev.mlh_gemm_device_init(0) == 0, pkg.dev.mlh_last_error(None).decode()
    # few weight rows, long K: the launch splits K over workgroups, so counters and partial tiles of the static array are in use
    _run(pkg, torch, pkg.DTYPE_F32, 8, 768, 2048, 1, with_r=True)
    _run(pkg, torch, pkg.DTYPE_F32, 4, 256, 1024, 2, with_r=False)   # second call, smaller input, same array
    _run(pkg, torch, pkg.DTYPE_F32, 64, 512, 2048, 3, with_r=True)   # 64 rows: the 16-row fp32 kernel, also split
    _run(pkg, torch, pkg.DTYPE_BF16, 33, 320, 4096, 4, with_r=False)  # half-width operands, ragged M and N
    _run(pkg, torch, pkg.DTYPE_F32, 5, 8192, 768, 5, with_r=False)    # many rows: no split, the array is not touched
    _run(pkg, torch, F16, 8, 256, 5632, 6, with_r=True)               # IEEE-half operands, few rows and long K: split
    _run(pkg, torch, pkg.DTYPE_BF16, 64, 192, 2048, 7, with_r=True)   # 64 rows of bf16: the two-block skinny kernel, split
    # limits and argument checks
    x = torch.zeros(16, dtype=torch.float32, device="cuda")
    p = x.data_ptr()
    for (M, N, K) in ((65, 64, 64), (8, 32769, 64), (8, 64, 65568), (8, 64, 48), (0, 64, 64)):
        assert pkg.dev.mlh_gemm_device(pkg.DTYPE_F32, M, N, K, p, p, None, p, None) == -1
        assert len(pkg.dev.mlh_last_error(None)) > 0
    assert b"M <= 64" in (pkg.dev.mlh_gemm_device(pkg.DTYPE_F32, 65, 64, 64, p, p, None, p, None), pkg.dev.mlh_last_error(None))[1]
    assert pkg.dev.mlh_gemm_device(pkg.DTYPE_F32, 8, 64, 64, None, p, None, p, None) == -1
