// Measurement only: two yardsticks under the prefill GEMM's ceiling, neither on the product path.
//
// mlh_probe_mfma   a register-only MFMA loop: every SIMD of every compute unit issues half-precision MFMAs
//                  back to back on operands that never leave its registers (no LDS, no memory), so the figure is
//                  what the matrix cores sustain under the part's power management for a given instruction form
//                  and operand data.  form 0: v_mfma_f32_32x32x16_f16 (the accumulator block is touched once per 16
//                  products), form 1: v_mfma_f32_16x16x32_f16 (once per 32).  data 0: all-zero operands (no switching
//                  activity: the code's own ceiling), data 1: pseudo-random operands of unit variance (what a
//                  product of activations and weights looks like to the multipliers).
// mlh_probe_lds_loads  the GEMM's global -> LDS load pattern alone: every workgroup streams 64 KB K slices of a
//                  256-row operand pair into LDS with direct loads and multiplies nothing (operands resident in the
//                  XCD's L2, as a GEMM's shared panels are); the figure is the bytes per second the load path delivers
//                  when nothing competes with it.
#include <vector>

#include "mlh_internal.h"

typedef _Float16 pm_f16x8 __attribute__((ext_vector_type(8)));
typedef float pm_f32x16 __attribute__((ext_vector_type(16)));
typedef float pm_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned pm_u32x4 __attribute__((ext_vector_type(4)));

#define PM_WAVES 8   // two per SIMD
#define PM_OPS 4     // distinct operand pairs a wave rotates through, so that operand bits toggle between MFMAs

__device__ __forceinline__ unsigned pm_hash(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

// a half of roughly unit variance: the sum of four uniforms in [-0.87, 0.87] (variance 4 * 0.87^2 / 3 = 1.0)
__device__ __forceinline__ _Float16 pm_value(unsigned seed) {
    float s = 0.f;
    for (int k = 0; k < 4; k++) s += ((float)(pm_hash(seed * 4u + k) & 0xffff) / 32768.f - 1.f) * 0.87f;
    return (_Float16)s;
}

template <int FORM>
__global__ void __launch_bounds__(PM_WAVES * 64) k_probe_mfma(int iters, int data, float* sink) {
    pm_f16x8 a[PM_OPS], b[PM_OPS];
    const unsigned gid = blockIdx.x * blockDim.x + threadIdx.x;
    for (int o = 0; o < PM_OPS; o++)
        for (int e = 0; e < 8; e++) {
            a[o][e] = data ? pm_value((gid * PM_OPS + o) * 16 + e) : (_Float16)0.f;
            b[o][e] = data ? pm_value((gid * PM_OPS + o) * 16 + 8 + e) : (_Float16)0.f;
        }
    float out = 0.f;
    if constexpr (FORM == 0) {
        pm_f32x16 acc[4] = {};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int o = 0; o < PM_OPS; o++)
#pragma unroll
                for (int c = 0; c < 4; c++) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[o], b[(o + c) % PM_OPS], acc[c], 0, 0, 0);
        }
        for (int c = 0; c < 4; c++)
            for (int e = 0; e < 16; e++) out += acc[c][e];
    } else {
        pm_f32x4 acc[8] = {};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int o = 0; o < PM_OPS; o++)
#pragma unroll
                for (int c = 0; c < 8; c++) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[o], b[(o + c) % PM_OPS], acc[c], 0, 0, 0);
        }
        for (int c = 0; c < 8; c++)
            for (int e = 0; e < 4; e++) out += acc[c][e];
    }
    if (out == 12345.678f) sink[gid] = out; // keeps the loop alive; practically never true
}

// flops of one launch: FORM 0: iters * 16 MFMAs of 32*32*16*2; FORM 1: iters * 32 MFMAs of 16*16*32*2 -- per wave
extern "C" int mlh_probe_mfma(mlh_ctx* c, int form, int data, int iters, double* tflops) {
    if (!c || !tflops || iters <= 0 || iters > (1 << 22) || form < 0 || form > 1 || data < 0 || data > 1) { if (c) c->err = "bad argument"; return -1; }
    (void)hipSetDevice(c->device);
    float* sink = nullptr;
    MLH_CHECK(c, hipMalloc((void**)&sink, (size_t)c->numCUs * PM_WAVES * 64 * 4));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = 0;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) rc = -2;
    float ms = 0.f;
    for (int pass = 0; pass < 2 && rc == 0; pass++) { // the first pass warms up
        if (hipEventRecord(e0, c->stream) != hipSuccess) { rc = -2; break; }
        if (form == 0) hipLaunchKernelGGL(k_probe_mfma<0>, dim3(c->numCUs), dim3(PM_WAVES * 64), 0, c->stream, iters, data, sink);
        else hipLaunchKernelGGL(k_probe_mfma<1>, dim3(c->numCUs), dim3(PM_WAVES * 64), 0, c->stream, iters, data, sink);
        if (hipGetLastError() != hipSuccess || hipEventRecord(e1, c->stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
            hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
            rc = -2;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (rc) { c->err = "MFMA probe: a HIP call failed"; return rc; }
    const double flop = (double)c->numCUs * PM_WAVES * iters * 16.0 * 32768.0; // both forms: 524288 flop per wave and iteration
    *tflops = flop / (ms * 1e-3) / 1e12;
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
#define PL_THREADS 256
#define PL_SLICE (512 * 128)            // bytes of one K slice of a 256 + 256 row operand pair (128 bytes of K per row)
#define PL_STAGES 2

__global__ void __launch_bounds__(PL_THREADS) k_probe_lds_loads(const unsigned char* src, size_t bytesPerWg, int slices, float* sink) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pl_lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned char* base = src + (size_t)(blockIdx.x & 63) * bytesPerWg; // four workgroups share a region, as workgroups of a GEMM share panels
    for (int s = 0; s < slices; s++) {
        const unsigned char* g = base + ((size_t)s * PL_SLICE) % bytesPerWg;
        unsigned char* stage = pl_lds + (s % PL_STAGES) * PL_SLICE;
        // 64 KB per slice = 16 loads of 1 KB per wave (64 lanes x 16 bytes), four waves
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const unsigned off = (unsigned)((wave * 16 + k) * 1024);
            __builtin_amdgcn_global_load_lds(g + off + lane * 16, stage + off, 16, 0, 0);
        }
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); // the slice before this one has landed; this one stays in flight
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const float v = *(const float*)(pl_lds + threadIdx.x * 4);
    if (v == 12345.678f) sink[blockIdx.x] = v;
}

extern "C" int mlh_probe_lds_loads(mlh_ctx* c, int slices, double* tbPerSec) {
    if (!c || !tbPerSec || slices <= 0 || slices > (1 << 20)) { if (c) c->err = "bad argument"; return -1; }
    (void)hipSetDevice(c->device);
    const size_t bytesPerWg = (size_t)2 * PL_SLICE; // 64 regions of 128 KiB, walked round and round: 1 MiB per XCD, resident in its L2 as the panels of a GEMM are
    unsigned char* src = nullptr;
    float* sink = nullptr;
    MLH_CHECK(c, hipMalloc((void**)&src, bytesPerWg * 64));
    if (hipMalloc((void**)&sink, (size_t)c->numCUs * 4) != hipSuccess) { (void)hipFree(src); c->err = "load probe: allocation failed"; return -2; }
    int rc = 0;
    if (hipMemsetAsync(src, 1, bytesPerWg * 64, c->stream) != hipSuccess) rc = -2;
    if (rc == 0 && hipFuncSetAttribute(reinterpret_cast<const void*>(&k_probe_lds_loads), hipFuncAttributeMaxDynamicSharedMemorySize, PL_STAGES * PL_SLICE) != hipSuccess) rc = -2;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (rc == 0 && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) rc = -2;
    float ms = 0.f;
    for (int pass = 0; pass < 2 && rc == 0; pass++) {
        if (hipEventRecord(e0, c->stream) != hipSuccess) { rc = -2; break; }
        hipLaunchKernelGGL(k_probe_lds_loads, dim3(c->numCUs), dim3(PL_THREADS), PL_STAGES * PL_SLICE, c->stream, (const unsigned char*)src, bytesPerWg, slices, sink);
        if (hipGetLastError() != hipSuccess || hipEventRecord(e1, c->stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
            hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
            rc = -2;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(src);
    (void)hipFree(sink);
    if (rc) { c->err = "load probe: a HIP call failed"; return rc; }
    *tbPerSec = (double)c->numCUs * slices * PL_SLICE / (ms * 1e-3) / 1e12;
    return 0;
}
