// Measurement only: how long one dependent exchange between workgroups takes on this device -- the quantity that
// bounds batch-1 decode, where a token is a chain of ~60 all-to-all exchanges.  Three probes, each `iters` dependent
// rounds inside ONE launch of one workgroup per compute unit, timed with HIP events on the context's stream:
//   [0] all-to-all of `dim` tagged words among the workgroups of one XCD, through that XCD's L2 (store written
//       through the L1, non-temporal load) -- the exchange the XCD-rank decode kernel uses inside an XCD
//   [1] the same words among ALL workgroups through the memory side (agent-scope atomics) -- its cross-XCD exchange
//   [2] a two-level grid barrier of relaxed agent-scope atomics -- what separates the phases of the barrier kernel
// Every wait is bounded; a probe whose wait expires reports -1 for its figure.
#include <vector>

#include "mlh_internal.h"

typedef unsigned long long u64;
#define HP_XCDS 8
#define HP_SPIN (1u << 18)
#define HP_BUFS 5

struct HopArgs {
    u64* words;        // [HP_BUFS][HP_XCDS][maxWords]
    unsigned* ctl;     // [0] abort flag, [1 + x] arrival counters per XCD, [16 + 64 * k] barrier words
    int maxWords, iters, perWg, mode;
};

__device__ __forceinline__ unsigned hp_ald(const unsigned* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void hp_ast(unsigned* p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__global__ void __launch_bounds__(256) k_hop_probe(HopArgs P) {
    __shared__ unsigned s_x, s_r, s_bad;
    const unsigned n = gridDim.x, per = n / HP_XCDS;
    if (threadIdx.x == 0) {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        xcc &= 15u;
        unsigned rank = per;
        if (xcc < HP_XCDS) rank = __hip_atomic_fetch_add(P.ctl + 1 + xcc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_bad = rank >= per;
        if (s_bad) hp_ast(P.ctl, 2u);
        s_x = xcc;
        s_r = rank;
    }
    __syncthreads();
    if (s_bad) return;
    const unsigned X = s_x, r = s_r;
    if (P.mode == 2) { // grid barrier: group word per XCD, top word, one release word per XCD
        for (int it = 0; it < P.iters; it++) {
            const unsigned ep = (unsigned)it + 1;
            if (threadIdx.x == 0) {
                const unsigned prev = __hip_atomic_fetch_add(P.ctl + 16 + 64 * (1 + X), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (prev == ep * per - 1) {
                    const unsigned p2 = __hip_atomic_fetch_add(P.ctl + 16, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (p2 == ep * HP_XCDS - 1)
                        for (unsigned k = 0; k < HP_XCDS; k++) hp_ast(P.ctl + 16 + 64 * (9 + k), ep);
                }
                unsigned spins = 0;
                while (hp_ald(P.ctl + 16 + 64 * (9 + X)) < ep)
                    if (++spins > HP_SPIN || ((spins & 255) == 0 && hp_ald(P.ctl))) { hp_ast(P.ctl, 1u); break; }
            }
            __syncthreads();
            if (hp_ald(P.ctl)) return;
        }
        return;
    }
    const bool cross = P.mode == 1;
    const unsigned group = cross ? 0 : X, members = cross ? n : per, me = cross ? X * per + r : r;
    const unsigned perWg = (unsigned)P.perWg / (cross ? HP_XCDS : 1); // the same vector, dealt to 8 times as many writers
    const unsigned total = members * perWg;
    for (int it = 0; it < P.iters; it++) {
        const unsigned ep = (unsigned)it + 1;
        u64* buf = P.words + ((size_t)(it % HP_BUFS) * HP_XCDS + group) * P.maxWords;
        if (threadIdx.x < perWg) {
            const u64 w = ((u64)ep << 32) | (me * perWg + threadIdx.x);
            if (cross) __hip_atomic_store(buf + me * perWg + threadIdx.x, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else __hip_atomic_store(buf + me * perWg + threadIdx.x, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        bool giveUp = false;
        for (unsigned i = threadIdx.x; i < total && !giveUp; i += blockDim.x) {
            unsigned spins = 0;
            for (;;) {
                const u64 w = cross ? __hip_atomic_load(buf + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : __builtin_nontemporal_load(buf + i);
                if ((unsigned)(w >> 32) == ep) break;
                if (++spins > HP_SPIN || ((spins & 255) == 0 && hp_ald(P.ctl))) { giveUp = true; break; }
            }
        }
        if (giveUp) hp_ast(P.ctl, 1u);
        __syncthreads();
        if (hp_ald(P.ctl)) return;
    }
}

__global__ void k_hop_clear(unsigned* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

extern "C" int mlh_probe_hops(mlh_ctx* c, int iters, double* us) {
    if (!c || !us || iters <= 0 || iters > 100000) { if (c) c->err = "bad argument"; return -1; }
    (void)hipSetDevice(c->device);
    if (c->numCUs % HP_XCDS || c->numCUs < HP_XCDS) { c->err = "hop probe: the compute units do not split into 8 XCDs"; return -1; }
    const int per = c->numCUs / HP_XCDS;
    const int perWg = std::max(1, c->hp.dim / per); // words a workgroup contributes inside its XCD (cross-XCD: an eighth of it)
    if (perWg > 256 || perWg % HP_XCDS) { c->err = "hop probe: dim / workgroups per XCD must be a multiple of 8, at most 256"; return -1; }
    const int maxWords = per * perWg;
    const size_t wordBytes = (size_t)HP_BUFS * HP_XCDS * maxWords * 8, ctlWords = 16 + 64 * 20;
    u64* words = nullptr;
    unsigned* ctl = nullptr;
    MLH_CHECK(c, hipMalloc((void**)&words, wordBytes));
    hipError_t e = hipMalloc((void**)&ctl, ctlWords * 4);
    if (e != hipSuccess) { (void)hipFree(words); c->err = "hop probe: allocation failed"; return -2; }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = 0;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) rc = -2;
    for (int mode = 0; mode < 3 && rc == 0; mode++) {
        us[mode] = -1.0;
        for (int pass = 0; pass < 2 && rc == 0; pass++) { // the first pass warms up
            hipLaunchKernelGGL(k_hop_clear, dim3((unsigned)((wordBytes / 4 + 255) / 256)), dim3(256), 0, c->stream, (unsigned*)words, wordBytes / 4);
            hipLaunchKernelGGL(k_hop_clear, dim3((unsigned)((ctlWords + 255) / 256)), dim3(256), 0, c->stream, ctl, ctlWords);
            HopArgs P{words, ctl, maxWords, pass == 0 ? std::min(iters, 50) : iters, perWg, mode};
            if (hipEventRecord(e0, c->stream) != hipSuccess) { rc = -2; break; }
            hipLaunchKernelGGL(k_hop_probe, dim3(c->numCUs), dim3(256), 0, c->stream, P);
            if (hipGetLastError() != hipSuccess || hipEventRecord(e1, c->stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) { rc = -2; break; }
            float ms = 0.f;
            unsigned flag = 1;
            if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess || hipMemcpy(&flag, ctl, 4, hipMemcpyDeviceToHost) != hipSuccess) { rc = -2; break; }
            if (pass == 1 && flag == 0) us[mode] = (double)ms * 1000.0 / iters;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(words);
    (void)hipFree(ctl);
    if (rc) c->err = "hop probe: a HIP call failed";
    return rc;
}
