// Batch-1 decode with every XCD of the MI355X acting as a tensor-parallel rank (gfx950, wave64).
//
// The chip is eight XCDs of 32 compute units, each XCD with its own L2.  An exchange between
// workgroups of ONE XCD can go through that L2 (about 0.7 us per hop: the producer's store is written
// through its L1, the consumer reads with non-temporal loads that do not stay in its L1); an exchange
// ACROSS XCDs has to go through the memory side (about 2.2 us).  The barrier-per-phase decode kernel
// pays five chip-wide exchanges per layer; this one pays two, plus five inside the XCDs:
//
//   XCD X owns the attention heads h = X, X+8, ... and the FFN units [X F/8, (X+1) F/8).
//   A  RMSNorm(x) and the q|k|v|gate rows of the XCD's heads           -> inside the XCD  (inference.cu:388-465)
//   B  attention of those heads, split over 32-key tiles               -> inside the XCD  (inference.cu:467-573)
//   C  combine + gate, then the Wo product over the XCD's COLUMNS      -> partial h1, across XCDs
//      (inference.cu:241-250, 582-610)
//      every workgroup adds the eight partials of its 1/32 slice, publishes the slice inside the XCD
//   D  RMSNorm(h1) and gate/up rows of the XCD's FFN units, SiLU*up    -> inside the XCD  (inference.cu:612-672)
//   E  W2 product over the XCD's F/8 columns                           -> partial x, across XCDs (inference.cu:675-699)
//   LM head rows over all workgroups, argmax across XCDs                                  (inference.cu:705-743)
//
// Hybrid models (template flag HYB; these layer kinds have no counterpart in inference.cu, they follow the kernel
// sequence's k_gdn and k_oproj): a gated-delta-net layer keeps the five phases; A also yields the two gate scalars
// of each of the XCD's heads, B is the delta rule on state rows (one row per wave, lane = column, the row resident
// in LDS for the whole launch) followed by a gather of the 64 read-outs of a head inside the XCD.  The PLE gate
// rows are split over the XCDs in A, e = silu(gate) * P[tok] is formed in B, and C adds the XCD's pleUp columns.
//
// Every exchanged value is one 64-bit word (value, tag): the tag is the number of the layer pass that
// produced it, the buffers start at zero, and a consumer reads until the tag is there, so data arrival is
// the synchronisation and a late or stale read only costs another read.  Every exchange is all-to-all
// within its group, so no workgroup can run more than one exchange ahead of another one of its group and
// each buffer is rewritten a whole layer later.  Waits are bounded: an expired wait raises the abort
// flag and every workgroup leaves.
//
// A workgroup is 7 worker waves and one communicator wave (two waves per SIMD: 256 registers each).  Workers never wait on global memory except
// for their own weights: each holds the weight rows of its next two phases in registers, issued two
// phases ahead, so that HBM latency is off the critical path (loads return in issue order on this ISA:
// a wave that polled would see its poll answered only after its prefetches).  The communicator does all
// the polling, the small reductions, q/k norm + RoPE and the softmax-partials combine, puts the result
// in LDS and meets the workers at a workgroup barrier.  K/V tiles of a wave's first attention unit are
// fetched global -> LDS directly (no registers) a whole layer ahead.
#include <stdlib.h>

#include <algorithm>

#include "mlh_internal.h"
#include "persist_common.h"

#define XWORK 7                 // worker waves per workgroup
#define XS1 4                   // full-width rows a worker keeps in its first register set
#define XWG ((XWORK + 1) * 64)  // + the communicator wave
#define XCDS 8
#define XPER 32                 // workgroups per XCD: the grid is exactly XCDS * XPER
#define XLW (XWORK * XPER)      // worker waves per XCD
#define XNH 4                   // heads per XCD at most
#define XAW 2                   // worker waves of a workgroup that take attention units
#define XCB 24                  // softmax partials the communicator fetches per round
#define XSPIN (1u << 20)
#define XHD 64
#define XQX 16                  // extra first-phase rows per XCD in hybrid models: two gate scalars per GDN head + PLE gate rows
#define XTK 32                  // keys per attention unit (half a KV page)
#define XTILE (XTK * XHD)       // floats of a K or V tile

typedef unsigned long long u64;

struct XcdArgs {
    StepArgs a;
    const LayerDev* layers;
    int NL, steps, seq;
    int abortAtStep;        // test hook: > 0 makes workgroup 0 give up when it reaches this step of the launch
    unsigned* abortFlag;
    unsigned* tagCounter;   // tags already used by earlier launches (advanced by workgroup 0 at the end)
    unsigned* xcdCount;     // [XCDS] zero at launch: workgroups that have arrived on each XCD
    int fs;                 // FFN units per XCD
    // exchange words: L = read inside the XCD that wrote them ([XCDS] regions), P = partials read by every XCD
    u64* qkvL; int qkvStride;   // [XCDS][4 * XNH * 64 + XQX]
    u64* partL; int partStride; // [XCDS][XNH * (32-key tiles of the longest sequence) * 66]; GDN layers: the read-outs [64 nh]
    u64* h1P;                   // [XCDS][d]
    u64* h1L;                   // [XCDS][d]
    u64* uL;                    // [XCDS][fs]
    u64* xP;                    // [XCDS][d]
    u64* xL;                    // [XCDS][d]
    u64* amax;                  // [grid][2]
    u64* timing;                // optional: communicator of workgroup 0, last step, 8 stamps per layer
    int wide;                   // slices of 64 elements (d / 64 readers per XCD) instead of d / 32 elements (32 readers)
    int napRound;               // 64-cycle units between two reads of the partial sums from other XCDs
    int nap[5];                 // 64-cycle units a consumer stays away before its first read of: partial sums from other
                                // XCDs, the gathered slices, q|k|v rows, FFN activations, softmax partials
};

__device__ __forceinline__ u64 xpack(float v, unsigned tag) { return ((u64)tag << 32) | __float_as_uint(v); }
// across XCDs: write-through store, load served by the memory side
__device__ __forceinline__ void xst(u64* p, float v, unsigned tag) { __hip_atomic_store(p, xpack(v, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ u64 xld(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// inside one XCD: the store leaves the L1 (which is write-through) for the XCD's L2; the load is non-temporal, so
// the line is not kept in the reader's L1 and the next read fetches it from the L2 again
__device__ __forceinline__ void lst(u64* p, float v, unsigned tag) { __hip_atomic_store(p, xpack(v, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
__device__ __forceinline__ u64 lld(const u64* p) { return __builtin_nontemporal_load(p); }

// Values that are the same in every lane of a wave, said so to the compiler: address arithmetic on them is then
// done once per wave on the scalar unit, and loads take the form scalar base + 32-bit lane offset.
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename T>
__device__ __forceinline__ T* uni_ptr(T* p) { // p points into global memory (the layer table holds it as a generic pointer)
    const u64 v = (u64)p;
    const u64 u = ((u64)(unsigned)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) | (u64)(unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v);
    return (T*)(__attribute__((address_space(1))) T*)u;
}

// Pins a wave-uniform pointer in scalar registers as an opaque value: without this the optimiser re-associates
// (base + row offset) + lane offset into (base + lane offset) + row offset, hoists the per-lane part out of the loops
// and ends up with one 64-bit vector address per load site, held in registers across the whole kernel.
template <typename T>
__device__ __forceinline__ const T* pin_uniform(const T* p) { // p: wave-uniform, into global memory
    u64 v = (u64)p;
    asm("" : "+s"(v));
    return (const T*)(__attribute__((address_space(1))) const T*)v;
}

// One tagged word at (wave-uniform base) + lane offset + constant, both in bytes (scalar base, one offset register).
template <bool CROSS>
__device__ __forceinline__ u64 ldw(const u64* base, unsigned laneBytes, unsigned constBytes) {
    asm volatile("" : "+v"(laneBytes));
    const u64* p = reinterpret_cast<const u64*>(reinterpret_cast<const char*>(base) + (size_t)laneBytes + constBytes);
    return CROSS ? xld(p) : lld(p);
}

// Keeps this wave off the memory system for about n x 64 cycles.  Reading before anything can have arrived only
// competes with the producers' stores: a first read delayed by the known minimum latency arrives just as early.
__device__ __forceinline__ void nap64(int n) {
    for (; n >= 16; n -= 16) __builtin_amdgcn_s_sleep(16);
    for (; n >= 4; n -= 4) __builtin_amdgcn_s_sleep(4);
    for (; n > 0; n--) __builtin_amdgcn_s_sleep(1);
}

// One wave fetches n tagged words into LDS, NB loads per lane and round, reading again until every tag is there.
// With PIPE two rounds are in flight, a fraction of a round trip apart: the answer to a round that just missed the
// data is followed closely by the next one instead of by a whole new round trip.  All 64 lanes take part.
template <bool CROSS, int NB, bool PIPE>
__device__ __forceinline__ void poll_vec(const u64* src, int n, unsigned tag, float* dst, const unsigned* abortFlag, bool& ok, int nap = 0) {
    const int lane = threadIdx.x & 63;
    nap64(nap);
    for (int base = 0; base < n; base += 64 * NB) {
        u64 wA[NB], wB[NB];
        auto issue = [&](u64 (&w)[NB]) {
            asm volatile("" ::: "memory"); // the loads are repeated every round
#pragma unroll
            for (int k = 0; k < NB; k++) {
                const int i0 = base + k * 64; // wave-uniform
                if (i0 < n) w[k] = ldw<CROSS>(pin_uniform(src + i0), (unsigned)min(lane, n - 1 - i0) * 8u, 0u);
                else w[k] = (u64)tag << 32;
            }
        };
        auto good = [&](const u64 (&w)[NB]) {
            bool all = true;
#pragma unroll
            for (int k = 0; k < NB; k++) all = all && (unsigned)(w[k] >> 32) == tag;
            return __all(all) != 0;
        };
        auto keep = [&](const u64 (&w)[NB]) {
#pragma unroll
            for (int k = 0; k < NB; k++) {
                const int i = base + k * 64 + lane;
                if (i < n) dst[i] = __uint_as_float((unsigned)w[k]);
            }
        };
        issue(wA);
        for (unsigned spins = 0;; spins++) {
            if (PIPE) {
                __builtin_amdgcn_s_sleep(CROSS ? 8 : 3);
                issue(wB);
            }
            if (good(wA)) { keep(wA); break; }
            if (PIPE) __builtin_amdgcn_s_sleep(CROSS ? 8 : 3);
            issue(wA);
            if (PIPE && good(wB)) { keep(wB); break; }
            if (!ok || spins > XSPIN || ((spins & 127) == 127 && aldu(abortFlag))) { ok = false; break; }
        }
    }
}

// A vector that every workgroup needs, out of the eight XCDs' partial sums: workgroup `rank` of every XCD adds the
// eight partials of slice [rank sl, (rank + 1) sl) (sl = d / 32 <= 64) and the residual and publishes the slice inside
// the XCD; then every workgroup fetches the whole vector from its XCD's 32 slices.  haveMask bit X' clear: that XCD
// contributes nothing.  Reads across XCDs disturb the stores they wait for, so the first one comes late (napCross).
__device__ __forceinline__ void reduce_publish_fetch(const u64* part, int d, int rank, unsigned tag, unsigned haveMask,
                                                     const float* resid, u64* pub, float* dst, const unsigned* abortFlag, bool& ok,
                                                     int napCross, int napGather, int napRound, bool wide, u64* stamp = nullptr) {
    const int lane = threadIdx.x & 63;
    const int sl = wide ? 64 : d / XPER, s0 = rank * sl;
    if (s0 >= d) { // (wide slices: only d / 64 workgroups of the XCD read the other XCDs' partial sums)
        nap64(napCross + 24);
        poll_vec<false, 16, false>(pub, d, tag, dst, abortFlag, ok, napGather);
        return;
    }
    const unsigned lb = (unsigned)min(lane, sl - 1) * 8u;
    u64 wA[XCDS], wB[XCDS];
    auto issue = [&](u64 (&w)[XCDS]) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int xc = 0; xc < XCDS; xc++) {
            if ((haveMask >> xc) & 1u) w[xc] = ldw<true>(pin_uniform(part + (size_t)xc * d + s0), lb, 0u);
            else w[xc] = (u64)tag << 32;
        }
    };
    auto good = [&](const u64 (&w)[XCDS]) {
        bool all = true;
#pragma unroll
        for (int xc = 0; xc < XCDS; xc++) all = all && (unsigned)(w[xc] >> 32) == tag;
        return __all(all) != 0;
    };
    auto total = [&](const u64 (&w)[XCDS]) { // fixed order: the result does not depend on timing
        float t = 0.f;
#pragma unroll
        for (int xc = 0; xc < XCDS; xc++) t += __uint_as_float((unsigned)w[xc]);
        return t;
    };
    float sum = 0.f;
    nap64(napCross);
    issue(wA);
    for (unsigned spins = 0;; spins++) {
        nap64(napRound);
        issue(wB);
        if (good(wA)) { sum = total(wA); break; }
        nap64(napRound);
        issue(wA);
        if (good(wB)) { sum = total(wB); break; }
        if (!ok || spins > XSPIN || ((spins & 127) == 127 && aldu(abortFlag))) { ok = false; break; }
    }
    if (stamp && lane == 0) stamp[0] = wall_clock64();
    if (lane < sl) lst(pub + s0 + lane, sum + resid[s0 + lane], tag);
    poll_vec<false, 16, false>(pub, d, tag, dst, abortFlag, ok, napGather);
}

// NCH (template parameter of the kernel): 16-byte chunks per lane of a full-width row, dim / (64 N)
template <typename WT, int NR, int NCH> struct XRows { typename PVec<WT>::Raw r[NR * NCH]; }; // NR full-width rows
template <typename WT> struct XPf { typename PVec<WT>::Raw r[8]; };
template <typename WT, int NCH> struct XGain { f32x4 g[NCH][PVec<WT>::N / 4]; };

// weights (16 bytes) times N activations in registers
template <typename WT>
__device__ __forceinline__ float chunk_dot_reg(const typename PVec<WT>::Raw& w, const float (&x)[PVec<WT>::N], float acc) {
    constexpr int N = PVec<WT>::N;
    float f[N];
    PVec<WT>::unpack(w, f);
#pragma unroll
    for (int i = 0; i < N; i++) acc = fmaf(f[i], x[i], acc);
    return acc;
}
// weights (16 bytes) times N activations in LDS
template <typename WT>
__device__ __forceinline__ float chunk_dot_lds(const typename PVec<WT>::Raw& w, const float* xs, float acc) {
    constexpr int N = PVec<WT>::N;
    float f[N];
    PVec<WT>::unpack(w, f);
#pragma unroll
    for (int i = 0; i < N; i += 4) {
        const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + i);
        acc = fmaf(f[i], xv.x, acc); acc = fmaf(f[i + 1], xv.y, acc);
        acc = fmaf(f[i + 2], xv.z, acc); acc = fmaf(f[i + 3], xv.w, acc);
    }
    return acc;
}

// 16 bytes at (wave-uniform base) + (32-bit lane offset in bytes) + constant: the addressing mode that needs no
// 64-bit arithmetic per lane (scalar base register + one offset register + immediate).
// (The empty statement keeps the widening of the lane offset next to the load: instruction selection works block by
// block and only then sees that the offset is a 32-bit value.)
template <typename WT>
__device__ __forceinline__ typename PVec<WT>::Raw load16(const void* base, unsigned laneBytes, unsigned constBytes) {
    asm volatile("" : "+v"(laneBytes));
    return *reinterpret_cast<const typename PVec<WT>::Raw*>(reinterpret_cast<const char*>(base) + (size_t)laneBytes + constBytes);
}
__device__ __forceinline__ f32x4 load16f(const void* base, unsigned laneBytes, unsigned constBytes) {
    asm volatile("" : "+v"(laneBytes));
    return *reinterpret_cast<const f32x4*>(reinterpret_cast<const char*>(base) + (size_t)laneBytes + constBytes);
}

// NR full-width rows (wave-uniform, valid indices) of the wave-uniform matrix W go into registers: lane l holds
// columns (ch 64 + l) N .. + N of every row.  Every register is assigned on every call (callers clamp indices
// instead of skipping loads), so nothing of an earlier phase stays live in them.
template <typename WT, int NR, int NCH>
__device__ __forceinline__ void issue_rows(typename PVec<WT>::Raw (&dst)[NR * NCH], const WT* W, size_t ld, const int (&rows)[NR]) {
    const unsigned lb = (threadIdx.x & 63u) * 16u;
#pragma unroll
    for (int k = 0; k < NR; k++) {
        const WT* rp = pin_uniform(W + (size_t)rows[k] * ld);
#pragma unroll
        for (int ch = 0; ch < NCH; ch++) dst[k * NCH + ch] = load16<WT>(rp, lb, ch * 1024u);
    }
}
template <typename WT, int NCH>
__device__ __forceinline__ void issue_gain(XGain<WT, NCH>& gn, const float* gain) {
    constexpr int N = PVec<WT>::N;
    const unsigned lb = (threadIdx.x & 63u) * (N * 4u);
    gain = pin_uniform(gain);
#pragma unroll
    for (int ch = 0; ch < NCH; ch++)
#pragma unroll
        for (int q = 0; q < N / 4; q++) gn.g[ch][q] = load16f(gain, lb, ch * 64u * N * 4u + q * 16u);
}

// xn = gain * (src / sqrt(mean(src^2) + 1e-8)) for this lane's columns (inference.cu:24-50, 83-95); every wave
// computes the mean itself from the vector in LDS, so no workgroup reduction is needed.
template <typename WT, int NCH>
__device__ __forceinline__ void normed_columns(const float* src, const XGain<WT, NCH>& gn, int d, float (&xn)[NCH][PVec<WT>::N]) {
    constexpr int N = PVec<WT>::N;
    const int c0 = (threadIdx.x & 63) * N;
    float ss = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ch++)
#pragma unroll
        for (int q = 0; q < N / 4; q++) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(src + ch * 64 * N + c0 + 4 * q);
            xn[ch][4 * q] = v.x; xn[ch][4 * q + 1] = v.y; xn[ch][4 * q + 2] = v.z; xn[ch][4 * q + 3] = v.w;
            ss = fmaf(v.x, v.x, ss); ss = fmaf(v.y, v.y, ss); ss = fmaf(v.z, v.z, ss); ss = fmaf(v.w, v.w, ss);
        }
    ss = pwave_sum(ss);
    const float ri = 1.0f / sqrtf(ss / (float)d + 1e-8f); // one division per wave; the elements are multiplied
#pragma unroll
    for (int ch = 0; ch < NCH; ch++)
#pragma unroll
        for (int q = 0; q < N / 4; q++) {
            const f32x4 g = gn.g[ch][q];
            xn[ch][4 * q] = g.x * (xn[ch][4 * q] * ri); xn[ch][4 * q + 1] = g.y * (xn[ch][4 * q + 1] * ri);
            xn[ch][4 * q + 2] = g.z * (xn[ch][4 * q + 2] * ri); xn[ch][4 * q + 3] = g.w * (xn[ch][4 * q + 3] * ri);
        }
}

template <typename WT, int NCH, int NRAW>
__device__ __forceinline__ float row_dot_reg(const typename PVec<WT>::Raw (&r)[NRAW], int which, const float (&xn)[NCH][PVec<WT>::N]) {
    float acc = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ch++) acc = chunk_dot_reg<WT>(r[which * NCH + ch], xn[ch], acc);
    return acc;
}
template <typename WT, int NCH>
__device__ __forceinline__ float row_dot_stream(const WT* W, size_t ld, int row, const float (&xn)[NCH][PVec<WT>::N]) {
    const WT* rp = pin_uniform(W + (size_t)row * ld);
    const unsigned lb = (threadIdx.x & 63u) * 16u;
    float acc = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCH; ch++) acc = chunk_dot_reg<WT>(load16<WT>(rp, lb, ch * 1024u), xn[ch], acc);
    return acc;
}

// The kernel works on 64-wide SLICES of the model dimension: a head of size 64 is one slice, a head of size 128 two
// (template parameter G = slices per head).  XCD X owns the heads X, X + 8, ... and with them their slices; everything
// that is linear in the head dimension (the q | k | v | gate rows, the Wo columns, the softmax-partials combine, the
// gate) runs per slice, only the attention unit itself -- per-head norm, scores, softmax -- sees the G slices of a head
// together.  Slice number (64-column block of the model dimension) of the j-th slice XCD X owns:
template <int G>
__device__ __forceinline__ int slice_of(int X, int j) {
    return G == 1 ? X + XCDS * j : G * (X + XCDS * (j / G)) + (j % G);
}

// Row of the fused first-phase matrix behind local index rho of XCD X: parts q, k, v, gate; nh slices of 64 rows each.
template <int G = 1>
__device__ __forceinline__ int rowA_of(int offK, int offV, int offG, int X, int nh, int rho) {
    const int per = nh * XHD, p = rho / per, rem = rho - p * per, j = rem >> 6, i = rem & 63;
    const int off = p == 0 ? 0 : p == 1 ? offK : p == 2 ? offV : offG;
    return off + slice_of<G>(X, j) * XHD + i;
}

// The same for models with gated-delta-net layers and per-layer embeddings: behind the q | k | v | gate rows come
// the two gate scalars of every GDN head of the XCD (alpha rows, then beta rows) and the XCD's share (pleX) of the
// PLE gate rows.
__device__ __forceinline__ int rowA_hyb(const LayerDev& L, int X, int nh, int np, int pleX, int rho) {
    const int rq = np * nh * XHD;
    if (rho < rq) return rowA_of(uni(L.offK), uni(L.offV), uni(L.offG), X, nh, rho);
    int e = rho - rq;
    if (uni(L.kind) != MLH_KIND_ATTENTION) {
        if (e < nh) return uni(L.offGa) + X + XCDS * e;
        if (e < 2 * nh) return uni(L.offGb) + X + XCDS * (e - nh);
        e -= 2 * nh;
    }
    return uni(L.offPle) + X * pleX + e;
}

// Wo columns of the XCD's heads: a pass covers N rows per wave (64/N lanes per 64-column head segment).  Rows
// and heads beyond the end are clamped to the last valid one (loaded, never used).
template <typename WT, int G = 1>
__device__ __forceinline__ void issue_wo(XPf<WT>& pf, const WT* Wo, int ad, int X, int nh, int heads, int lw, int d) {
    constexpr int N = PVec<WT>::N, CPS = XHD / N;
    const unsigned lane = threadIdx.x & 63u;
    const unsigned lb = ((lane / CPS) * (unsigned)ad + (lane % CPS) * N) * (unsigned)sizeof(WT); // row within the pass, chunk within the head segment
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const int rb = min((p * XLW + lw) * N, d - N);
#pragma unroll
        for (int j = 0; j < XNH; j++) {
            const int h = min(slice_of<G>(X, min(j, max(nh, 1) - 1)), G * heads - 1); // slice, clamped to the last one
            pf.r[p * XNH + j] = load16<WT>(pin_uniform(Wo + (size_t)rb * ad + h * XHD), lb, 0u);
        }
    }
}
// W2 columns [X fs, (X+1) fs): a wave takes blocks of four consecutive rows (block wb first); the first block, two
// chunks per lane, is prefetched (clamped likewise).
template <typename WT>
__device__ __forceinline__ void issue_w2(XPf<WT>& pf, const WT* W2, int X, int fs, int F, int wb, int d) {
    constexpr int N = PVec<WT>::N;
    const int lane = threadIdx.x & 63, CR = fs / N;
    const unsigned lb0 = (unsigned)min(lane, CR - 1) * 16u, lb1 = (unsigned)min(lane + 64, CR - 1) * 16u;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const WT* rp = pin_uniform(W2 + (size_t)min(wb * 4 + k, d - 1) * F + (size_t)X * fs);
        pf.r[k * 2] = load16<WT>(rp, lb0, 0u);
        pf.r[k * 2 + 1] = load16<WT>(rp, lb1, 0u);
    }
}

// K and V tile (XTK rows x 64 floats each) of one head, rows below `lim`, global -> LDS without registers.  An
// instruction moves 1 KB: lane i's 16 bytes land at base + 16 i, i.e. row 4q + i/16, slot i%16; the lane fetches the
// piece that belongs there: for K under the swizzle slot = piece ^ (row & 15), which makes the per-lane row reads of
// the score loop conflict-free; V stays row-major (the P.V loop reads a row across the lanes).  Kh, Vh: wave-uniform
// pointers to row 0 of the head's slice of the page.
__device__ __forceinline__ void issue_kv_tile(const float* Kh, const float* Vh, int d, int lim, float* tK, float* tV) {
    const unsigned lane = threadIdx.x & 63u;
#pragma unroll
    for (int q = 0; q < XTK / 4; q++) {
        const unsigned row = 4 * q + (lane >> 4), piece = (lane & 15) ^ (row & 15);
        // row 4q of the tile is the wave-uniform part of the address, the lane adds (lane / 16) rows and its piece
        const char* Kq = pin_uniform(reinterpret_cast<const char*>(Kh + (size_t)(4 * q) * d));
        const char* Vq = pin_uniform(reinterpret_cast<const char*>(Vh + (size_t)(4 * q) * d));
        unsigned lbK = ((lane >> 4) * (unsigned)d + piece * 4u) * 4u, lbV = ((lane >> 4) * (unsigned)d + (lane & 15) * 4u) * 4u;
        if ((int)row < lim) {
            asm volatile("" : "+v"(lbK), "+v"(lbV));
            __builtin_amdgcn_global_load_lds(Kq + (size_t)lbK, tK + q * 256, 16, 0, 0);
            __builtin_amdgcn_global_load_lds(Vq + (size_t)lbV, tV + q * 256, 16, 0, 0);
        }
    }
}

struct XShared {
    float *xs, *h1s, *qkvs, *as, *us, *scratch, *bestv, *tiles;
    float *es, *gst; // hybrid models: the XCD's PLE values of the layer; this workgroup's GDN state rows [layer][4][64]
    int *besti, *ctl;
    LayerDev* Ls;
};

#define X_STAMP(slot)                                                                                   \
    do {                                                                                                \
        if (P.timing && wg == 0 && lane == 0 && step == P.steps - 1) P.timing[(slot)] = wall_clock64(); \
    } while (0)
#define X_BARRIER()                  \
    do {                             \
        lds_barrier();               \
        if (uni(S.ctl[0])) return;   \
    } while (0)

// ------------------------------------------------------------------------------------------------ communicator
template <typename WT, bool HYB, int G>
__device__ __forceinline__ void xcd_communicator(const XcdArgs& P, const XShared& S, int tok, int pos, unsigned tagBase, int X, int r) {
    const StepArgs& a = P.a;
    const int d = a.dim, V = a.vocab;
    const int lane = threadIdx.x & 63, wg = blockIdx.x;
    const int nh = a.heads > X ? G * ((a.heads - X + XCDS - 1) / XCDS) : 0; // slices of this XCD
    const int np = 3 + (a.gating ? 1 : 0);
    const int RA = np * nh * XHD;
    unsigned headMask = 0; // XCDs that own at least one head
    for (int xc = 0; xc < XCDS; xc++) headMask |= (a.heads > xc ? 1u : 0u) << xc;
    u64* qkvL = P.qkvL + (size_t)X * P.qkvStride;
    u64* partL = P.partL + (size_t)X * P.partStride;
    bool ok = true;

    for (int step = 0; step < P.steps; step++) {
        // embedding gather (inference.cu:9-22): every workgroup keeps its own copy of the residual stream
        for (int i = lane; i < d; i += 64) S.xs[i] = PVec<WT>::one((const WT*)a.E + (size_t)tok * d + i);
        if (P.abortAtStep > 0 && step == P.abortAtStep && wg == 0) ok = false; // test hook: a wait given up in mid-launch

        for (int t = P.NL - 1; t >= 0; t--) { // file block 0 is the top of the stack (inference.cu:384-385)
            const LayerDev& L = S.Ls[t];
            const unsigned lt = tagBase + (unsigned)(step * P.NL + (P.NL - 1 - t) + 1);
            const int ts = (P.NL - 1 - t) * 16;
            X_STAMP(ts + 0);
            if (t != P.NL - 1) // partial x of the layer below, all XCDs, + its residual h1
                reduce_publish_fetch(P.xP, d, r, lt - 1, 0xffu, S.h1s, P.xL + (size_t)X * d, S.xs, P.abortFlag, ok, P.nap[0], P.nap[1], P.napRound, P.wide != 0,
                                     (P.timing && wg == 0 && step == P.steps - 1) ? P.timing + ts + 6 : nullptr);
            if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
            X_STAMP(ts + 1);
            X_BARRIER(); // 1: x in LDS

            // q | k | v | gate rows of the XCD's heads, as the workers produced them; the attention waves take it from there
            int RAL = RA;
            if constexpr (HYB) {
                const bool gdnL = uni(L.kind) != MLH_KIND_ATTENTION;
                RAL = (gdnL ? 3 : np) * nh * XHD + (gdnL ? 2 * nh : 0) + a.ple / XCDS;
            }
            poll_vec<false, 8, false>(qkvL, RAL, lt, S.qkvs, P.abortFlag, ok, P.nap[2]);
            if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
            X_STAMP(ts + 2);
            X_BARRIER(); // 2: q, k, v, gate in LDS

            // (softmax partials are combined by the attention waves, one head per wave)
            X_STAMP(ts + 3);
            X_BARRIER(); // 3: mixing output of the XCD's heads in LDS

            // h1 = x + sum of the XCDs' Wo partials (inference.cu:252-260)
            reduce_publish_fetch(P.h1P, d, r, lt, headMask, S.xs, P.h1L + (size_t)X * d, S.h1s, P.abortFlag, ok, P.nap[0], P.nap[1], P.napRound, P.wide != 0,
                                 (P.timing && wg == 0 && step == P.steps - 1) ? P.timing + ts + 8 : nullptr);
            if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
            X_STAMP(ts + 4);
            X_BARRIER(); // 4: h1 in LDS

            poll_vec<false, 8, false>(P.uL + (size_t)X * P.fs, P.fs, lt, S.us, P.abortFlag, ok, P.nap[3]);
            if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
            X_STAMP(ts + 5);
            X_BARRIER(); // 5: the XCD's FFN activations in LDS
        }

        // ---------------------------------------------------------------------- LM head + argmax
        const unsigned ltLast = tagBase + (unsigned)(step * P.NL + P.NL);
        reduce_publish_fetch(P.xP, d, r, ltLast, 0xffu, S.h1s, P.xL + (size_t)X * d, S.xs, P.abortFlag, ok, P.nap[0], P.nap[1], P.napRound, P.wide != 0);
        if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
        X_BARRIER(); // final x in LDS
        X_BARRIER(); // the workers' best logits in LDS
        {
            float v = lane < XWORK ? S.bestv[lane] : -3.0e38f;
            int i = lane < XWORK ? S.besti[lane] : 0x7fffffff;
#pragma unroll
            for (int o = 4; o > 0; o >>= 1) {
                const float v2 = __shfl_xor(v, o, MLH_WAVE);
                const int i2 = __shfl_xor(i, o, MLH_WAVE);
                if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
            }
            if (lane == 0) {
                xst(P.amax + 2 * wg, v, tagBase + (unsigned)step + 1);
                xst(P.amax + 2 * wg + 1, __uint_as_float((unsigned)i), tagBase + (unsigned)step + 1);
            }
            poll_vec<true, 8, true>(P.amax, 2 * (int)gridDim.x, tagBase + (unsigned)step + 1, S.scratch, P.abortFlag, ok, P.nap[0] / 2);
            v = -3.0e38f; i = 0x7fffffff;
            for (int k = lane; k < (int)gridDim.x; k += 64) {
                const float v2 = S.scratch[2 * k];
                const int i2 = (int)__float_as_uint(S.scratch[2 * k + 1]);
                if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float v2 = __shfl_xor(v, o, MLH_WAVE);
                const int i2 = __shfl_xor(i, o, MLH_WAVE);
                if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
            }
            if (i < 0 || i >= V) i = 0; // only reachable with non-finite logits
            tok = i;
            if (lane == 0) S.ctl[1] = tok;
            if (wg == 0 && lane == 0) { // the append of inference_orchestrator.cu:149-151, kept on the device
                const int sc = *a.stepCounter;
                if (sc + step < a.outCapacity) a.outIds[sc + step] = tok;
            }
        }
        if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
        pos += 1;
        X_BARRIER(); // next token in LDS
    }
    if (wg == 0 && lane == 0) {
        // every workgroup read the counter before it could contribute to the first exchange, and this point lies
        // behind the last one
        *P.tagCounter = tagBase + (unsigned)(P.steps * P.NL + 1);
        *a.stepCounter += P.steps;
        a.pos[P.seq] = pos;
        ((int*)a.tok)[0] = tok;
        a.nextTok[P.seq] = tok;
    }
}

// ------------------------------------------------------------------------------------------------ workers
template <typename WT, int NCH, bool HYB, int G>
__device__ __forceinline__ void xcd_worker(const XcdArgs& P, const XShared& S, int tok, int pos, unsigned tagBase, int X, int r) {
    static_assert(G == 1 || !HYB, "heads of two slices: attention-only models");
    constexpr int HD = G * XHD; // head size
    constexpr int N = PVec<WT>::N, CPS = XHD / N;
    const StepArgs& a = P.a;
    const int d = a.dim, F = a.ffn, V = a.vocab, fs = P.fs;
    const int lane = threadIdx.x & 63, wave = uni(threadIdx.x >> 6), wg = blockIdx.x;
    const int lw = wave * XPER + r;             // worker wave within the XCD: consecutive rows land on different workgroups
    const int wbE = r * XWORK + wave;           // first block of four W2 rows of this wave
    const int lwF = (XWORK - 1 - wave) * XPER + r; // the same in reverse wave order, for the FFN units: a second unit, where
                                                   // there is one, goes to the last waves, not to the attention waves
    const int gwl = wave * (int)gridDim.x + wg; // worker wave within the grid (LM head)
    const int TWL = XWORK * (int)gridDim.x;
    const int nhh = a.heads > X ? (a.heads - X + XCDS - 1) / XCDS : 0; // heads of this XCD
    const int nh = G * nhh;                                            // and their slices
    const int np = 3 + (a.gating ? 1 : 0);
    const int RA = np * nh * XHD;
    const int pleX = HYB ? a.ple / XCDS : 0; // PLE columns of this XCD
    // rows of the first phase in layer Lx (hybrid models: fewer parts and two gate scalars per head in a GDN layer,
    // the PLE gate rows in every layer)
    auto rowsA = [&](const LayerDev& Lx) {
        if constexpr (!HYB) return RA;
        const bool g = uni(Lx.kind) != MLH_KIND_ATTENTION;
        return (g ? 3 : np) * nh * XHD + (g ? 2 * nh : 0) + pleX;
    };
    auto rowA = [&](const LayerDev& Lx, int rho) {
        if constexpr (HYB) return rowA_hyb(Lx, X, nh, uni(Lx.kind) != MLH_KIND_ATTENTION ? 3 : np, pleX, rho);
        else return rowA_of<G>(uni(Lx.offK), uni(Lx.offV), uni(Lx.offG), X, nh, rho);
    };
    u64* qkvL = P.qkvL + (size_t)X * P.qkvStride;
    u64* partL = P.partL + (size_t)X * P.partStride;
    float* tK = S.tiles + (wave < XAW ? wave : 0) * (G * 2 * XTILE); // slice g of the head: K tile at + g 2 XTILE, V tile behind it
    float* tV = tK + XTILE;
    const int aslot = wave * XPER + r; // attention unit slot of this wave (waves below XAW only)
    const WT* E = (const WT*)a.E;

    XRows<WT, XS1, NCH> s1; // rows of phases A / D / LM head
    XPf<WT> s2;      // rows of phases C / E / LM head
    XGain<WT, NCH> gn;
    // first-phase rows lw, lw + XLW, ... of layer Lx and its first gain vector
    auto issueA = [&](const LayerDev& Lx) {
        const int ra = rowsA(Lx);
        int rows[XS1];
#pragma unroll
        for (int k = 0; k < XS1; k++) rows[k] = nh > 0 ? rowA(Lx, min(lw + XLW * k, ra - 1)) : 0;
        issue_rows<WT, XS1, NCH>(s1.r, uni_ptr((const WT*)Lx.Wa), d, rows);
        issue_gain<WT, NCH>(gn, uni_ptr(Lx.g1));
    };
    // first K/V tile of this wave in layer Lx when the sequence holds npos rows, and the q/k gains of its head
    float gqv[G], gkv[G];
#pragma unroll
    for (int g = 0; g < G; g++) { gqv[g] = 1.f; gkv[g] = 1.f; }
    // (the tile index of a wave's first unit never changes, so its page is looked up once)
    const int pageFirst = (wave < XAW && nhh > 0 && aslot / nhh < 2 * a.pagesPerSeq) ? uni(a.pageTable[P.seq * a.pagesPerSeq + ((aslot / nhh) >> 1)]) : 0;
    // gains of head h's slices for this lane, and the K/V tiles of its slices from the page rows at `base`
    auto loadGains = [&](const LayerDev& Lx, int h) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            gqv[g] = uni_ptr(Lx.gq)[h * HD + g * XHD + lane];
            gkv[g] = uni_ptr(Lx.gk)[h * HD + g * XHD + lane];
        }
    };
    auto issueTiles = [&](const LayerDev& Lx, size_t base, int lim) {
#pragma unroll
        for (int g = 0; g < G; g++)
            issue_kv_tile(uni_ptr((const float*)Lx.K) + base + g * XHD, uni_ptr((const float*)Lx.V) + base + g * XHD, d, lim, tK + g * 2 * XTILE, tV + g * 2 * XTILE);
    };
    auto issueKV = [&](const LayerDev& Lx, int npos) {
        const int nt = (npos + XTK) / XTK;
        if (aslot < nhh * nt) {
            const int j = aslot % nhh, tl = aslot / nhh, h = X + XCDS * j;
            if (a.qkNorm) loadGains(Lx, h);
            issueTiles(Lx, ((size_t)pageFirst * MLH_KV_PAGE + (tl & 1) * XTK) * d + h * HD, npos - tl * XTK);
        }
    };
    if (wave < XAW) { // the tiles must never hold anything but finite numbers (rows beyond the sequence get weight zero)
        for (int i = lane * 4; i < G * 2 * XTILE; i += 256) *reinterpret_cast<f32x4*>(tK + i) = (f32x4)(0.f);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    // hybrid models: the PLE up-projection columns of this XCD for the first two passes of the output projection
    // (lane c of a row group holds column X pleX + c), fetched together with the Wo columns
    float plw[2] = {0.f, 0.f};
    float plv = 0.f; // wave 0, lane c < pleX: the token's PLE table value for the coming layer
    auto issuePlw = [&](const LayerDev& Lx) {
        if constexpr (HYB) {
            if (pleX > 0) {
                const int rs = lane / CPS, c = min(lane % CPS, pleX - 1);
                const WT* up = uni_ptr((const WT*)Lx.pleUp);
#pragma unroll
                for (int p = 0; p < 2; p++) plw[p] = PVec<WT>::one(up + (size_t)min((p * XLW + lw) * N + rs, d - 1) * a.ple + X * pleX + c);
            }
        }
    };
    auto issuePlv = [&](const LayerDev& Lx, int token) {
        if constexpr (HYB) {
            if (pleX > 0 && wave == 0) plv = PVec<WT>::one(uni_ptr((const WT*)Lx.pleTable) + (size_t)token * a.ple + X * pleX + min(lane, pleX - 1));
        }
    };
    // hybrid models: wave w < 2 nh owns state row r 2nh + w of the XCD's GDN heads in every GDN layer; the rows stay
    // in LDS for the whole launch (lane = column) and go back to memory at its end
    const int grow = r * 2 * nh + wave;         // row among the 64 nh state rows of the XCD
    const bool gwave = HYB && wave < 2 * nh;
    float* gst = S.gst + (size_t)wave * XHD + lane; // + layer * 4 * XHD
    auto stateRow = [&](const LayerDev& Lx) {
        return uni_ptr(Lx.S) + (((size_t)P.seq * a.gdnHeads + (X + XCDS * (grow >> 6))) * XHD + (grow & 63)) * XHD + lane;
    };
    if constexpr (HYB) {
        if (gwave)
            for (int t = 0; t < P.NL; t++)
                if (uni(S.Ls[t].kind) != MLH_KIND_ATTENTION) gst[(size_t)t * 4 * XHD] = *stateRow(S.Ls[t]);
    }
    {
        const LayerDev& L0 = S.Ls[P.NL - 1];
        issueA(L0);
        issue_wo<WT, G>(s2, uni_ptr((const WT*)L0.Wo), uni(L0.ad), X, nh, a.heads, lw, d);
        issuePlw(L0);
        if (wave < XAW && (!HYB || uni(L0.kind) == MLH_KIND_ATTENTION)) issueKV(L0, pos);
    }

    float* qh = S.tiles + XAW * G * 2 * XTILE + (wave < XAW ? wave : 0) * HD; // this wave's query after norm and RoPE
    bool ok = true; // attention waves poll the softmax partials (bounded)

    for (int step = 0; step < P.steps; step++) {
        const int T = pos + 1, ntiles = (T + XTK - 1) / XTK, newTile = pos / XTK;
        float rc[G], rsn[G]; // RoPE of this step's position: lanes (2i, 2i+1) of slice g hold the pair 32 g + i (inference.cu:113-134)
#pragma unroll
        for (int g = 0; g < G; g++) { rc[g] = 1.f; rsn[g] = 0.f; }
        int pageNew = 0; // page that receives this step's K/V row
        if (wave < XAW) {
#pragma unroll
            for (int g = 0; g < G; g++) {
                rc[g] = a.rope[(size_t)pos * HD + g * XHD + (lane & ~1)];
                rsn[g] = a.rope[(size_t)pos * HD + g * XHD + (lane | 1)];
            }
            pageNew = uni(a.pageTable[P.seq * a.pagesPerSeq + (pos >> 6)]);
        }
        issuePlv(S.Ls[P.NL - 1], tok);
        for (int t = P.NL - 1; t >= 0; t--) {
            const LayerDev& L = S.Ls[t];
            const unsigned lt = tagBase + (unsigned)(step * P.NL + (P.NL - 1 - t) + 1);
            const bool lastLayer = t == 0;
            const bool gdnL = HYB && uni(L.kind) != MLH_KIND_ATTENTION;
            const int RAL = rowsA(L);                       // rows of the first phase in this layer
            const int RAq = (gdnL ? 3 : np) * nh * XHD;     // of which q | k | v | gate
            const LayerDev& Ln = S.Ls[lastLayer ? P.NL - 1 : t - 1];
            X_BARRIER(); // 1
            const int ts = (P.NL - 1 - t) * 16;
            const bool stampW = P.timing && wg == 0 && wave == 0 && lane == 0 && step == P.steps - 1;
#define W_STAMP(slot) do { if (stampW) P.timing[ts + (slot)] = wall_clock64(); } while (0)
            W_STAMP(10);
            // ------------------------------------------------------------------ phase A
            {
                float xn[NCH][N];
                normed_columns<WT, NCH>(S.xs, gn, d, xn);
#pragma unroll
                for (int k = 0; k < XS1; k++) {
                    const int rho = lw + XLW * k;
                    if (rho < RAL) {
                        const float acc = pwave_sum(row_dot_reg<WT, NCH>(s1.r, k, xn));
                        if (lane == 0) lst(qkvL + rho, acc, lt);
                    }
                }
                if (lw + XS1 * XLW < RAL) {
                    const WT* Wa = uni_ptr((const WT*)L.Wa);
                    for (int rho = lw + XS1 * XLW; rho < RAL; rho += XLW) {
                        const float acc = pwave_sum(row_dot_stream<WT, NCH>(Wa, d, rowA(L, rho), xn));
                        if (lane == 0) lst(qkvL + rho, acc, lt);
                    }
                }
            }
            W_STAMP(11);
            X_BARRIER(); // 2
            // ------------------------------------------------------------------ phase B
            if constexpr (HYB) {
                if (pleX > 0 && wave == 0) { // e = silu(gate) * P[tok] for the XCD's PLE columns (inference-side PLE rule of k_oproj)
                    if (lane < pleX) S.es[lane] = psilu(S.qkvs[RAL - pleX + lane]) * plv;
                    if (!(lastLayer)) issuePlv(Ln, tok); // the last layer's successor belongs to the next token
                }
                if (gdnL) {
                    // gated delta rule on this wave's state row (k_gdn of the kernel sequence, one row per wave, lane = column):
                    //   u = S k ; S <- alpha (S - beta u k^T) + beta v k^T ; o = S q   with q, k L2-normalised
                    if (gwave) {
                        const int j = grow >> 6, i = grow & 63, h = X + XCDS * j;
                        const float* qsA = S.qkvs;
                        const float qc = qsA[j * XHD + lane], kc = qsA[nh * XHD + j * XHD + lane];
                        const float vr = qsA[2 * nh * XHD + j * XHD + i];
                        const float rq = sqrtf(pwave_sum(qc * qc) + 1e-6f), rk = sqrtf(pwave_sum(kc * kc) + 1e-6f);
                        const float za = qsA[RAq + j] + uni_ptr(L.gdnBa)[h], zb = qsA[RAq + nh + j] + uni_ptr(L.gdnBb)[h];
                        const float sp = fmaxf(za, 0.f) + log1pf(expf(-fabsf(za)));
                        const float alpha = expf(-sp), beta = psigmoid(zb);
                        const float kn = kc / rk, qn = qc / rq;
                        float* sp_ = gst + (size_t)t * 4 * XHD;
                        float sv = *sp_;
                        const float u = pwave_sum(sv * kn);
                        sv = alpha * (sv - beta * u * kn) + beta * vr * kn;
                        const float o = pwave_sum(sv * qn);
                        *sp_ = sv;
                        if (lane == 0) lst(partL + grow, o, lt);
                    }
                    // the read-outs of a head's 64 rows come from 32 / nh workgroups: one head per wave gathers them
                    for (int j = wave; j < nh; j += XAW) {
                        if (wave >= XAW) break;
                        const u64* ub = pin_uniform(partL + (size_t)j * XHD);
                        u64 w = 0;
                        for (unsigned spins = 0;; spins++) {
                            asm volatile("" ::: "memory");
                            w = ldw<false>(ub, (unsigned)lane * 8u, 0u);
                            if (__all((unsigned)(w >> 32) == lt)) break;
                            if (!ok || spins > XSPIN || ((spins & 255) == 255 && aldu(P.abortFlag))) { ok = false; break; }
                        }
                        S.as[j * XHD + lane] = __uint_as_float((unsigned)w);
                    }
                    if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
                    if (wave < XAW && !(lastLayer && step == P.steps - 1) && uni(Ln.kind) == MLH_KIND_ATTENTION)
                        issueKV(Ln, lastLayer ? pos + 1 : pos);
                }
            }
            if (wave < XAW && !gdnL) {
                const int U = nhh * ntiles;
                const float* qsAll = S.qkvs; // rows as the first phase produced them
                const float* ksAll = qsAll + nh * XHD;
                const float* vsAll = ksAll + nh * XHD;
                const float* gsAll = vsAll + nh * XHD;
                // per-head RMSNorm (inference.cu:52-81, 97-111) and RoPE of a head's vector held one element per lane and slice
                auto norm_rope = [&](float (&v)[G], const float (&gain)[G]) {
                    if (a.qkNorm) {
                        float ss = 0.f;
#pragma unroll
                        for (int g = 0; g < G; g++) ss = fmaf(v[g], v[g], ss);
                        const float rr = sqrtf(pwave_sum(ss) / (float)HD + 1e-8f);
#pragma unroll
                        for (int g = 0; g < G; g++) v[g] = gain[g] * (v[g] / rr);
                    }
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        const float o = dpp_move<0xB1, 0xf>(v[g], 0.f); // the other element of the pair
                        v[g] = (lane & 1) ? rsn[g] * o + rc[g] * v[g] : rc[g] * v[g] - rsn[g] * o;
                    }
                };
                const bool dbg = P.timing && t == 0 && step == P.steps - 1 && lane == 0 && wave == 0;
                if (dbg) P.timing[16 * (P.NL + 1) + 4 * wg + 1] = aslot < U ? wall_clock64() : 0;
                for (int u = aslot; u < U; u += XAW * XPER) {
                    const int j = u % nhh, tl = u / nhh, j0 = tl * XTK, h = X + XCDS * j; // j: head among the XCD's, its slices G j + g
                    if (u != aslot) { // tiles beyond the first one were not fetched ahead
                        const int page = uni(a.pageTable[P.seq * a.pagesPerSeq + (tl >> 1)]);
                        issueTiles(L, ((size_t)page * MLH_KV_PAGE + (tl & 1) * XTK) * d + h * HD, pos - j0);
                        if (a.qkNorm) loadGains(L, h);
                    }
                    {
                        float qv[G];
#pragma unroll
                        for (int g = 0; g < G; g++) qv[g] = qsAll[(G * j + g) * XHD + lane];
                        norm_rope(qv, gqv);
#pragma unroll
                        for (int g = 0; g < G; g++) qh[g * XHD + lane] = qv[g];
                    }
                    // The tile has landed in LDS.  A tile fetched a layer ahead is older than the dozens of weight loads
                    // issued since (loads and stores retire in issue order): the few stores of the first phase may stay
                    // in flight.
                    if (u == aslot) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    if (dbg) P.timing[16 * (P.NL + 1) + 4 * wg + 3] = wall_clock64();
                    const int nv = T - j0 < XTK ? T - j0 : XTK;     // keys of this tile, the new one included
                    if (tl == newTile) { // this step's row comes from the first phase, not from the cache; it is appended here
                        const int rn = pos - j0;
                        float kn[G];
#pragma unroll
                        for (int g = 0; g < G; g++) kn[g] = ksAll[(G * j + g) * XHD + lane];
                        norm_rope(kn, gkv);
#pragma unroll
                        for (int g = 0; g < G; g++) {
                            const float vn = vsAll[(G * j + g) * XHD + lane];
                            tK[g * 2 * XTILE + rn * 64 + ((((lane >> 2) ^ (rn & 15)) << 2) | (lane & 3))] = kn[g];
                            tV[g * 2 * XTILE + rn * 64 + lane] = vn;
                            // write-through: read from the next step on, by whichever workgroup of this XCD takes the tile
                            const size_t o = ((size_t)pageNew * MLH_KV_PAGE + (pos & 63)) * d + h * HD + g * XHD + lane;
                            ast(uni_ptr(L.K) + o, kn[g]);
                            ast(uni_ptr(L.V) + o, vn);
                        }
                    }
                    __builtin_amdgcn_wave_barrier();
                    // scores: lanes l and l + 32 share key l % 32, each takes half of the 64 dimensions of every slice
                    const int key = lane & 31, dh = lane >> 5;
                    float s = 0.f;
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        const float* kr = tK + g * 2 * XTILE + key * 64;
#pragma unroll
                        for (int p = 0; p < 8; p++) {
                            const int pp = p + 8 * dh;
                            const f32x4 kk = *reinterpret_cast<const f32x4*>(kr + ((pp ^ (key & 15)) << 2));
                            const f32x4 qq = *reinterpret_cast<const f32x4*>(qh + g * XHD + pp * 4);
                            s = fmaf(kk.x, qq.x, s); s = fmaf(kk.y, qq.y, s); s = fmaf(kk.z, qq.z, s); s = fmaf(kk.w, qq.w, s);
                        }
                    }
                    s += __shfl_xor(s, 32, MLH_WAVE);
                    const bool valid = key < nv;
                    s = valid ? s / sqrtf((float)HD) : -1.0e30f; // inference.cu:154
                    const float m = pwave_max(s);
                    const float e = (valid && dh == 0) ? expf(s - m) : 0.f; // lanes 0..31 carry the weights
                    const float l = pwave_sum(e);
                    // all XTK rows: rows from nv on hold older K/V rows or the zeros of the start of the kernel, and
                    // their weights are zero.  Sixteen rows are fetched before they are used, so that the LDS latency
                    // is paid twice, not once per row.
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        float acc = 0.f;
                        const float* vcol = tV + g * 2 * XTILE + lane;
#pragma unroll
                        for (int jj0 = 0; jj0 < XTK; jj0 += 16) {
                            float vr[16];
#pragma unroll
                            for (int i = 0; i < 16; i++) vr[i] = vcol[(jj0 + i) * 64];
#pragma unroll
                            for (int i = 0; i < 16; i++)
                                acc = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(e), jj0 + i)), vr[i], acc);
                        }
                        // a slice's tiles one after the other, as the combine reads them; every slice of the head carries the
                        // head's maximum and sum, so the combine runs slice by slice
                        u64* out = partL + ((size_t)(G * j + g) * ntiles + tl) * (XHD + 2);
                        lst(out + lane, acc, lt);
                        if (lane == 0) { lst(out + XHD, m, lt); lst(out + XHD + 1, l, lt); }
                    }
                    __builtin_amdgcn_wave_barrier();
                }
                if (P.timing && t == 0 && step == P.steps - 1 && lane == 0)
                    P.timing[16 * (P.NL + 1) + 4 * wg + wave] = aslot < U ? wall_clock64() : 0;
                W_STAMP(12);
                // Softmax partials of the XCD's heads -> mixing output (lane = dimension), gate (inference.cu:241-250):
                // every workgroup needs it, so its attention waves take one head each.  A single wave issues one
                // instruction every four cycles whatever its kind: the weights exp(m - M) of a batch of tiles are
                // formed at once (lane = tile), per tile only a broadcast and a multiply-add remain.
                if (wave < nh) nap64(P.nap[4]);
                for (int j = wave; j < nh; j += XAW) {
                    float M = -1.0e30f, num = 0.f, den = 0.f;
                    for (int t0 = 0; t0 < ntiles; t0 += XCB) {
                        const int nb = ntiles - t0 < XCB ? ntiles - t0 : XCB;
                        u64 wa[XCB], wm, wl;
                        const u64* ub = pin_uniform(partL + ((size_t)j * ntiles + t0) * (XHD + 2));
                        const unsigned uOff = (unsigned)min(lane & 31, nb - 1) * ((XHD + 2) * 8u);
                        for (unsigned spins = 0;; spins++) {
                            asm volatile("" ::: "memory");
                            bool all = true;
#pragma unroll
                            for (int k = 0; k < XCB; k++) {
                                if (k < nb) wa[k] = ldw<false>(ub, (unsigned)lane * 8u, k * ((XHD + 2) * 8u));
                                else wa[k] = (u64)lt << 32;
                                all = all && (unsigned)(wa[k] >> 32) == lt;
                            }
                            wm = ldw<false>(ub, uOff, XHD * 8u);       // lane k < 32: running maximum of tile t0 + k
                            wl = ldw<false>(ub, uOff, (XHD + 1) * 8u); //              and its sum of exponentials
                            all = all && (unsigned)(wm >> 32) == lt && (unsigned)(wl >> 32) == lt;
                            if (__all(all)) break;
                            if (!ok || spins > XSPIN || ((spins & 255) == 255 && aldu(P.abortFlag))) { ok = false; break; }
                        }
                        const float mk = __uint_as_float((unsigned)wm), lk = __uint_as_float((unsigned)wl);
                        const bool mine = lane < nb;
                        const float Mn = fmaxf(M, pwave_max(mine ? mk : -1.0e30f));
                        const float corr = __expf(M - Mn);
                        const float w = mine ? __expf(mk - Mn) : 0.f;
                        den = fmaf(den, corr, pwave_sum(w * lk));
                        num *= corr;
#pragma unroll
                        for (int k8 = 0; k8 < XCB; k8 += 8)
                            if (k8 < nb) {
#pragma unroll
                                for (int k = k8; k < k8 + 8; k++)
                                    num = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), k)), __uint_as_float((unsigned)wa[k]), num);
                            }
                        M = Mn;
                    }
                    float v = num * __builtin_amdgcn_rcpf(den);
                    if (a.gating) v = v * __builtin_amdgcn_rcpf(1.0f + __expf(-gsAll[j * XHD + lane])); // inference.cu:248
                    S.as[j * XHD + lane] = v;
                }
                if (dbg) P.timing[16 * (P.NL + 1) + 4 * wg + 2] = wave < nh ? wall_clock64() : 0;
                W_STAMP(15);
                if (!ok) { S.ctl[0] = 1; astu(P.abortFlag, 1u); }
                // first tile of this wave for the next layer pass (the next step's first layer sees one more row)
                if (!(lastLayer && step == P.steps - 1) && (!HYB || uni(Ln.kind) == MLH_KIND_ATTENTION)) issueKV(Ln, lastLayer ? pos + 1 : pos);
            }
            // gate/up rows of this wave's first two FFN units, and the second gain vector
            {
                int rows[XS1];
#pragma unroll
                for (int k = 0; k < XS1 / 2; k++) {
                    const int q = min(lwF + XLW * k, fs - 1);
                    rows[2 * k] = 2 * (X * fs + q);
                    rows[2 * k + 1] = 2 * (X * fs + q) + 1;
                }
                issue_rows<WT, XS1, NCH>(s1.r, uni_ptr((const WT*)L.W13), d, rows);
                issue_gain<WT, NCH>(gn, uni_ptr(L.g2));
            }
            X_BARRIER(); // 3
            W_STAMP(13);
            // ------------------------------------------------------------------ phase C
            if (nh > 0) {
                const int rs = lane / CPS, c = lane % CPS;
                const int ad = uni(L.ad);
                for (int p = 0; (p * XLW + lw) * N < d; p++) {
                    const int row = (p * XLW + lw) * N + rs;
                    float acc = 0.f;
#pragma unroll
                    for (int j = 0; j < XNH; j++)
                        if (j < nh) {
                            const typename PVec<WT>::Raw w = p == 0 ? s2.r[j] : p == 1 ? s2.r[XNH + j]
                                : PVec<WT>::load(uni_ptr((const WT*)L.Wo) + (size_t)row * ad + slice_of<G>(X, j) * XHD + c * N);
                            acc = chunk_dot_lds<WT>(w, S.as + j * XHD + c * N, acc);
                        }
                    if constexpr (HYB) { // + pleUp . e over the XCD's PLE columns (one column per lane of the row group)
                        if (pleX > 0) {
                            const float w = p == 0 ? plw[0] : p == 1 ? plw[1]
                                                  : PVec<WT>::one(uni_ptr((const WT*)L.pleUp) + (size_t)row * a.ple + X * pleX + min(c, pleX - 1));
                            if (c < pleX) acc = fmaf(w, S.es[c], acc);
                        }
                    }
                    acc = pgroup_sum<CPS>(acc);
                    if (c == 0) xst(P.h1P + (size_t)X * d + row, acc, lt);
                }
            }
            W_STAMP(14);
            issue_w2<WT>(s2, uni_ptr((const WT*)L.W2), X, fs, F, wbE, d);
            X_BARRIER(); // 4
            // ------------------------------------------------------------------ phase D
            {
                float xn[NCH][N];
                normed_columns<WT, NCH>(S.h1s, gn, d, xn);
#pragma unroll
                for (int k = 0; k < XS1 / 2; k++) {
                    const int q = lwF + XLW * k;
                    if (q < fs) {
                        const float g = pwave_sum(row_dot_reg<WT, NCH>(s1.r, 2 * k, xn)), up = pwave_sum(row_dot_reg<WT, NCH>(s1.r, 2 * k + 1, xn));
                        if (lane == 0) lst(P.uL + (size_t)X * fs + q, psilu(g) * up, lt); // inference.cu:262-281
                    }
                }
                if (lwF + (XS1 / 2) * XLW < fs) {
                    const WT* W13 = uni_ptr((const WT*)L.W13);
                    for (int q = lwF + (XS1 / 2) * XLW; q < fs; q += XLW) {
                        const int pr = X * fs + q;
                        const float g = pwave_sum(row_dot_stream<WT, NCH>(W13, d, 2 * pr, xn));
                        const float up = pwave_sum(row_dot_stream<WT, NCH>(W13, d, 2 * pr + 1, xn));
                        if (lane == 0) lst(P.uL + (size_t)X * fs + q, psilu(g) * up, lt);
                    }
                }
            }
            W_STAMP(7);
            if (!lastLayer) {
                issueA(Ln);
            } else { // LM-head rows gwl, gwl + TWL, ... and the final gain
                int rows[XS1];
#pragma unroll
                for (int k = 0; k < XS1; k++) rows[k] = min(gwl + TWL * k, V - 1);
                issue_rows<WT, XS1, NCH>(s1.r, E, d, rows);
                issue_gain<WT, NCH>(gn, a.gF);
            }
            X_BARRIER(); // 5
            // ------------------------------------------------------------------ phase E
            {
                // four consecutive rows per wave, written with one store: 32 contiguous bytes towards the memory side
                // instead of four separate words
                const int CR = fs / N;
                const WT* W2x = uni_ptr((const WT*)L.W2) + (size_t)X * fs;
                if (wbE * 4 < d) {
                    float val = 0.f;
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const int row = min(wbE * 4 + k, d - 1);
                        float acc = 0.f;
#pragma unroll
                        for (int c0 = 0; c0 < 2; c0++) {
                            const int cc = lane + 64 * c0;
                            if (cc < CR) acc = chunk_dot_lds<WT>(s2.r[k * 2 + c0], S.us + cc * N, acc);
                        }
                        for (int cc = lane + 128; cc < CR; cc += 64)
                            acc = chunk_dot_lds<WT>(PVec<WT>::load(W2x + (size_t)row * F + cc * N), S.us + cc * N, acc);
                        acc = pwave_sum(acc);
                        val = lane == k ? acc : val;
                    }
                    if (lane < 4 && wbE * 4 + lane < d) xst(P.xP + (size_t)X * d + wbE * 4 + lane, val, lt); // inference.cu:283-291 (the readers add the residual)
                }
                for (int b = wbE + XLW; b * 4 < d; b += XLW) {
                    float val = 0.f;
                    for (int k = 0; k < 4; k++) {
                        const int row = min(b * 4 + k, d - 1);
                        float acc = 0.f;
                        for (int cc = lane; cc < CR; cc += 64)
                            acc = chunk_dot_lds<WT>(PVec<WT>::load(W2x + (size_t)row * F + cc * N), S.us + cc * N, acc);
                        acc = pwave_sum(acc);
                        val = lane == k ? acc : val;
                    }
                    if (lane < 4 && b * 4 + lane < d) xst(P.xP + (size_t)X * d + b * 4 + lane, val, lt);
                }
            }
            W_STAMP(9);
            if (!lastLayer) {
                issue_wo<WT, G>(s2, uni_ptr((const WT*)Ln.Wo), uni(Ln.ad), X, nh, a.heads, lw, d);
                issuePlw(Ln);
            } else {
                // two more LM-head rows; the second register set has room for them when a row has at most 4 chunks
                const int rows[2] = {min(gwl + XS1 * TWL, V - 1), min(gwl + (XS1 + 1) * TWL, V - 1)};
                typename PVec<WT>::Raw (&lm)[2 * NCH] = reinterpret_cast<typename PVec<WT>::Raw (&)[2 * NCH]>(s2.r);
                issue_rows<WT, 2, NCH>(lm, E, d, rows);
            }
        }

        // ---------------------------------------------------------------------- LM head + argmax
        X_BARRIER(); // final x in LDS
        {
            float xn[NCH][N];
            normed_columns<WT, NCH>(S.xs, gn, d, xn); // inference.cu:705-715
            float best = -3.0e38f;
            int bidx = 0x7fffffff;
            auto take = [&](int row, float acc) { // rows ascend per wave: ties keep the lower index
                acc = pwave_sum(acc);
                if (lane == 0) a.logits[(size_t)P.seq * V + row] = acc;
                if (acc > best) { best = acc; bidx = row; }
            };
#pragma unroll
            for (int k = 0; k < XS1; k++)
                if (gwl + TWL * k < V) take(gwl + TWL * k, row_dot_reg<WT, NCH>(s1.r, k, xn));
#pragma unroll
            for (int k = 0; k < 2; k++)
                if (gwl + TWL * (XS1 + k) < V) take(gwl + TWL * (XS1 + k), row_dot_reg<WT, NCH>(reinterpret_cast<const typename PVec<WT>::Raw (&)[2 * NCH]>(s2.r), k, xn));
            // a large vocabulary leaves rows beyond the prefetched ones: XS1 at a time through the first register set (its
            // rows are used up), so that a wave pays one memory round trip per XS1 rows instead of one per row
            for (int row0 = gwl + (XS1 + 2) * TWL; row0 < V; row0 += XS1 * TWL) {
                int rows[XS1];
#pragma unroll
                for (int k = 0; k < XS1; k++) rows[k] = min(row0 + TWL * k, V - 1);
                issue_rows<WT, XS1, NCH>(s1.r, E, d, rows);
#pragma unroll
                for (int k = 0; k < XS1; k++)
                    if (row0 + TWL * k < V) take(row0 + TWL * k, row_dot_reg<WT, NCH>(s1.r, k, xn));
            }
            if (lane == 0) { S.bestv[wave] = best; S.besti[wave] = bidx; }
        }
        if (step + 1 < P.steps) { // first layer of the next step
            const LayerDev& L0 = S.Ls[P.NL - 1];
            issueA(L0);
            issue_wo<WT, G>(s2, uni_ptr((const WT*)L0.Wo), uni(L0.ad), X, nh, a.heads, lw, d);
            issuePlw(L0);
        }
        X_BARRIER(); // best logits in LDS
        X_BARRIER(); // next token in LDS
        tok = S.ctl[1];
        pos += 1;
    }
    if constexpr (HYB) {
        if (gwave)
            for (int t = 0; t < P.NL; t++)
                if (uni(S.Ls[t].kind) != MLH_KIND_ATTENTION) *const_cast<float*>(stateRow(S.Ls[t])) = gst[(size_t)t * 4 * XHD];
    }
    (void)tok;
}

template <typename WT, int NCH, bool HYB, int G>
__global__ void __launch_bounds__(XWG) k_decode_xcd(XcdArgs P) {
    extern __shared__ float lds[];
    const StepArgs& a = P.a;
    const int d = a.dim, wave = uni(threadIdx.x >> 6);
    XShared S;
    S.xs = lds;
    S.h1s = S.xs + d;
    S.qkvs = S.h1s + d;                 // [4][nh * 64] q | k | v | gate of the XCD's heads
    S.as = S.qkvs + 4 * XNH * XHD + XQX; // [nh * 64] mixing output (XQX: room for the extra first-phase rows of hybrid models)
    S.us = S.as + XNH * XHD;            // [fs]
    S.scratch = S.us + ((P.fs + 3) & ~3); // [max(d / 4, 2 * grid)]
    S.bestv = S.scratch + 512;
    S.besti = reinterpret_cast<int*>(S.bestv + 16);
    S.ctl = S.besti + 16;               // [0] a wait expired, [1] next token
    S.tiles = reinterpret_cast<float*>(S.ctl + 16); // [XAW][K tile | V tile]
    S.Ls = reinterpret_cast<LayerDev*>(S.tiles + XAW * G * 2 * XTILE + XAW * G * 64); // (after the tiles: one query vector per attention wave)
    S.es = reinterpret_cast<float*>(S.Ls + P.NL);
    S.gst = S.es + 16;                  // hybrid models only: [NL][4][64]
    for (int i = threadIdx.x; i < P.NL * (int)(sizeof(LayerDev) / 4); i += XWG)
        reinterpret_cast<uint32_t*>(S.Ls)[i] = reinterpret_cast<const uint32_t*>(P.layers)[i];
    if (threadIdx.x == 0) {
        // The exchange inside an XCD needs to know which workgroups share an L2: the XCD is read from the hardware
        // register, the rank inside it is the order of arrival.  256 workgroups of this size on 256 compute units
        // put exactly XPER on every XCD; anything else is reported instead of trusted.
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        xcc &= 15u;
        unsigned rank = XPER;
        if (xcc < XCDS && gridDim.x == XCDS * XPER) rank = __hip_atomic_fetch_add(P.xcdCount + xcc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool bad = rank >= XPER;
        S.ctl[0] = bad ? 1 : 0;
        S.ctl[1] = 0;
        S.ctl[2] = (int)xcc;
        S.ctl[3] = (int)rank;
        if (bad) astu(P.abortFlag, 2u);
    }
    lds_barrier();
    if (uni(S.ctl[0])) return;
    const int X = uni(S.ctl[2]), r = uni(S.ctl[3]);
    const int tok = uni(a.tok[0]), pos = uni(a.pos[P.seq]);
    const unsigned tagBase = *P.tagCounter; // tags do not repeat from launch to launch (the host clears everything before the count wraps)
    if (wave == XWORK) xcd_communicator<WT, HYB, G>(P, S, tok, pos, tagBase, X, r);
    else xcd_worker<WT, NCH, HYB, G>(P, S, tok, pos, tagBase, X, r);
}

// before every launch: abort flag and per-XCD arrival counters
__global__ void k_xcd_prep(unsigned* abortFlag, unsigned* xcdCount, unsigned startCount) {
    if (threadIdx.x == 0) *abortFlag = 0u;
    if (threadIdx.x < XCDS) xcdCount[threadIdx.x] = startCount;
}

__global__ void k_xcd_zero(unsigned* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
// hybrid model: gated-delta-net layers or per-layer embeddings (the HYB instantiation of the kernel)
static bool xcd_hybrid(const mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    if (hp.pleDim > 0) return true;
    for (int t = 0; t < hp.transformers; t++)
        if (hp.layerKinds[t] != MLH_KIND_ATTENTION) return true;
    return false;
}

static size_t xcd_lds_bytes(const mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    const int fs = hp.ffnDim / XCDS;
    const int G = hp.headDim / XHD; // slices per head
    return ((size_t)2 * hp.dim + 5 * XNH * XHD + XQX + ((fs + 3) & ~3) + 512 + 48 + XAW * G * 2 * XTILE + XAW * G * 64 + 16 +
            (xcd_hybrid(c) ? (size_t)hp.transformers * 4 * XHD : 0)) * 4 + (size_t)hp.transformers * sizeof(LayerDev);
}

// Exchange words (64-bit) the kernel needs for this model.
size_t mlh_xcd_words(const mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    return (size_t)XCDS * (4 * XNH * XHD + XQX) + (size_t)XCDS * XNH * (MLH_KV_PAGE / XTK) * c->pagesPerSeq * (XHD + 2) + (size_t)4 * XCDS * hp.dim + hp.ffnDim +
           2 * (size_t)XCDS * XPER + 64;
}

// True when the XCD-rank kernel supports this context's shape: head size 64 (attention heads, and GDN heads with
// 64 x 64 states, as many as attention heads) or, for attention-only models without per-layer embeddings, 128 (the
// shape the reference ships: network_meta.h:3-20); PLE columns that split evenly over the XCDs, a 256-unit chip, rows
// that fit the register sets.
bool mlh_xcd_supported(const mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    if (c->numCUs != XCDS * XPER || !c->xcdWords) return false;
    const int N = hp.weightDtype == MLH_DTYPE_BF16 ? 8 : 4;
    bool gdn = false;
    for (int t = 0; t < hp.transformers; t++) gdn = gdn || hp.layerKinds[t] != MLH_KIND_ATTENTION;
    if (gdn && (hp.gdnDk != XHD || hp.gdnDv != XHD || hp.gdnHeads != hp.attnHeads || hp.attnHeads < XCDS || hp.attnHeads > 2 * XCDS)) return false; // (four state rows per workgroup and layer)
    if (hp.pleDim % XCDS || hp.pleDim / XCDS > XHD / N || 2 * XNH + hp.pleDim / XCDS > XQX) return false;
    if (hp.pleDim > 0 && hp.attnHeads < XCDS) return false;
    if (hp.headDim != XHD && !(hp.headDim == 2 * XHD && !gdn && hp.pleDim == 0)) return false;
    const int G = hp.headDim / XHD;
    if (hp.dim != hp.attnHeads * hp.headDim || hp.dim > 4 * 64 * N || hp.dim % (64 * N) || hp.dim % XPER) return false;
    if (G * ((hp.attnHeads + XCDS - 1) / XCDS) > XNH) return false; // slices per XCD
    if (hp.ffnDim % (XCDS * N)) return false;
    if (hp.dim / 4 > 512 || hp.dim % N) return false;
    return xcd_lds_bytes(c) <= 160 * 1024;
}

template <typename WT, int NCH, bool HYB, int G>
static int launch_xcd_as(mlh_ctx* c, XcdArgs& P, size_t ldsBytes) {
    if (!c->xcdPrepared) { // once per context (mlh_finalize does it; a context has one model, hence one instantiation)
        MLH_CHECK(c, hipFuncSetAttribute(reinterpret_cast<const void*>(&k_decode_xcd<WT, NCH, HYB, G>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
        int perCu = 0;
        MLH_CHECK(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, k_decode_xcd<WT, NCH, HYB, G>, XWG, ldsBytes));
        if (perCu < 1) { c->err = "XCD-rank decode kernel does not fit on a compute unit"; return -1; }
        c->xcdPrepared = true;
    }
    if (P.steps <= 0) return 0; // preparation only
    // one workgroup per compute unit, all resident at once (the occupancy query says each unit can hold one); waits are bounded
    hipLaunchKernelGGL((k_decode_xcd<WT, NCH, HYB, G>), dim3(XCDS * XPER), dim3(XWG), ldsBytes, c->stream, P);
    MLH_CHECK(c, hipGetLastError());
    return 0;
}
template <typename WT, int NCH>
static int launch_xcd(mlh_ctx* c, XcdArgs& P, size_t ldsBytes) {
    if (c->hp.headDim == 2 * XHD) return launch_xcd_as<WT, NCH, false, 2>(c, P, ldsBytes); // (attention-only: mlh_xcd_supported)
    return xcd_hybrid(c) ? launch_xcd_as<WT, NCH, true, 1>(c, P, ldsBytes) : launch_xcd_as<WT, NCH, false, 1>(c, P, ldsBytes);
}

// Puts the exchange words and the tag counter back to zero (after a launch that gave up a wait, and before the
// 32-bit tags would wrap).
int mlh_xcd_reset(mlh_ctx* c) {
    if (!c->xcdBuf) return 0;
    c->xcdTagNext = 0;
    const size_t words32 = c->xcdWords * 2;
    hipLaunchKernelGGL(k_xcd_zero, dim3((unsigned)((words32 + 255) / 256)), dim3(256), 0, c->stream, (unsigned*)c->xcdBuf, words32);
    hipLaunchKernelGGL(k_xcd_zero, dim3(1), dim3(64), 0, c->stream, c->d_sync + 64 * 21, (size_t)1);
    MLH_CHECK(c, hipGetLastError());
    return 0;
}

// Enqueues `steps` decode steps of sequence 0 (slot 0) in one launch of the XCD-rank kernel.
int mlh_launch_xcd(mlh_ctx* c, int steps) {
    const mlh_hparams& hp = c->hp;
    XcdArgs P;
    mlh_fill_args(c, P.a, 1, c->d_tok);
    P.layers = c->d_layers;
    P.NL = hp.transformers;
    P.steps = steps;
    P.seq = 0;
    P.abortAtStep = 0;
    P.abortFlag = c->d_sync + 64 * 20;
    P.tagCounter = c->d_sync + 64 * 21;
    P.xcdCount = c->d_sync + 64 * 22;
    P.fs = hp.ffnDim / XCDS;
    P.timing = c->d_timing;
    P.wide = c->xcdWide;
    P.napRound = c->xcdNapRound;
    for (int k = 0; k < 5; k++) P.nap[k] = c->xcdNap[k];
    u64* t = c->xcdBuf;
    P.qkvStride = 4 * XNH * XHD + XQX;
    P.qkvL = t; t += (size_t)XCDS * P.qkvStride;
    P.partStride = XNH * (MLH_KV_PAGE / XTK) * c->pagesPerSeq * (XHD + 2);
    P.partL = t; t += (size_t)XCDS * P.partStride;
    P.h1P = t; t += (size_t)XCDS * hp.dim;
    P.h1L = t; t += (size_t)XCDS * hp.dim;
    P.xP = t; t += (size_t)XCDS * hp.dim;
    P.xL = t; t += (size_t)XCDS * hp.dim;
    P.uL = t; t += hp.ffnDim;
    P.amax = t;
    const size_t ldsBytes = xcd_lds_bytes(c);
    if (steps > 0) {
        // Tags are a 32-bit running count of layer passes and a word whose tag matches is taken as fresh: before the
        // count could wrap (and meet tag 0 of cleared words, or a stale word), everything goes back to zero.
        const unsigned long long need = (unsigned long long)steps * hp.transformers + 1;
        if (c->xcdTagNext + need >= 0xFFFFFFFFull) {
            int rc = mlh_xcd_reset(c);
            if (rc) return rc;
        }
        c->xcdTagNext += need; // (a launch that gives up is followed by mlh_xcd_reset, which puts this back to zero)
        // test hook: arrival counters that start full make every workgroup give up before it touches anything
        const unsigned startCount = c->injectAbort > 0 ? (unsigned)XPER : 0u;
        if (c->injectAbort > 0) c->injectAbort--;
        P.abortAtStep = c->injectAbortStep;
        c->injectAbortStep = 0;
        hipLaunchKernelGGL(k_xcd_prep, dim3(1), dim3(64), 0, c->stream, P.abortFlag, P.xcdCount, startCount);
    }
    if (hp.weightDtype == MLH_DTYPE_BF16) {
        switch (hp.dim / 512) { // chunks of 8 values per lane and row
            case 1: return launch_xcd<bf16_t, 1>(c, P, ldsBytes);
            case 2: return launch_xcd<bf16_t, 2>(c, P, ldsBytes);
            case 3: return launch_xcd<bf16_t, 3>(c, P, ldsBytes);
            default: return launch_xcd<bf16_t, 4>(c, P, ldsBytes);
        }
    }
    switch (hp.dim / 256) { // chunks of 4 values per lane and row
        case 1: return launch_xcd<float, 1>(c, P, ldsBytes);
        case 2: return launch_xcd<float, 2>(c, P, ldsBytes);
        case 3: return launch_xcd<float, 3>(c, P, ldsBytes);
        default: return launch_xcd<float, 4>(c, P, ldsBytes);
    }
}
