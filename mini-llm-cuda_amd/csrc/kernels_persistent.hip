// Persistent batch-1 decode kernel for gfx950.
//
// One cooperative launch decodes `steps` tokens of one sequence.  The grid is one
// workgroup of 512 threads per compute unit; every workgroup walks the same
// sequence of phases and meets the others at a grid barrier between phases:
//
//   per layer:  A  RMSNorm + fused q|k|v|gate|ple|gdn rows          (inference.cu:388-465,487-507)
//               B  attention over 64-key tiles, or the GDN state update  (inference.cu:467-573)
//               C  partials combine + gate + Wo rows + PLE + residual    (inference.cu:241-250,582-610)
//               D  RMSNorm + gate/up rows + SiLU*up                      (inference.cu:612-672)
//               E  W2 rows + residual                                    (inference.cu:675-699)
//   per token:  final RMSNorm + LM-head rows + argmax                    (inference.cu:705-743)
//
// Why this shape on MI355X: a dependent kernel launch costs 6-10 us here and a batch-1 token of a
// small model needs ~60 dependent steps, so launches (or graph nodes) dominate.  Inside one kernel a
// step boundary is a grid barrier built from agent-scope relaxed atomics (about 2 us across the
// eight XCDs).  Agent-scope fences are avoided on purpose: on this part they write back and
// invalidate the L2 and cost tens of microseconds.  Instead every value that another workgroup
// reads is written with an agent-scope atomic store (write-through) and read with an agent-scope
// atomic load (served from the memory side), with workgroup-scope fences for ordering.  Weights are
// read-only and use ordinary cached loads; each wave issues the loads of its next phase's weight
// rows before it enters the barrier, so HBM latency overlaps the synchronisation.
#include <stdlib.h>

#include "mlh_internal.h"
#include "persist_common.h"

#define PWG 512
#define PWAVES (PWG / MLH_WAVE)
#define P_SPIN_LIMIT (1u << 21)
#define PPF 8 // 16-byte chunks per lane and row held in registers across a barrier

template <typename WT>
struct RowPf {
    typename PVec<WT>::Raw r[2][PPF];
};

// Issue the loads of up to two rows (row, row2; row2 < 0: none) of W for this wave.
template <typename WT>
__device__ __forceinline__ void pf_rows(RowPf<WT>& pf, const WT* __restrict__ W, size_t ld, int row, int row2, int cols) {
    constexpr int N = PVec<WT>::N;
    const int lane = threadIdx.x & 63;
    typedef typename PVec<WT>::Raw Raw;
    // every element is (re)assigned, so nothing of the previous phase stays live in these registers
#pragma unroll
    for (int ch = 0; ch < PPF; ch++) {
        const int c = (ch * 64 + lane) * N;
        const bool in = row >= 0 && c < cols;
        pf.r[0][ch] = in ? PVec<WT>::load(W + (size_t)row * ld + c) : (Raw)(0);
        pf.r[1][ch] = (in && row2 >= 0) ? PVec<WT>::load(W + (size_t)row2 * ld + c) : (Raw)(0);
    }
}

// Dot products of the prefetched rows (and their streamed tails) with a vector in LDS.
template <typename WT, bool TWO>
__device__ __forceinline__ void dot_pf(const RowPf<WT>& pf, const WT* __restrict__ W, size_t ld, int row, int row2,
                                       int cols, const float* xs, float& acc0, float& acc1) {
    constexpr int N = PVec<WT>::N;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int ch = 0; ch < PPF; ch++) {
        const int c = (ch * 64 + lane) * N;
        if (c < cols) {
            float w0[N], w1[N];
            PVec<WT>::unpack(pf.r[0][ch], w0);
            if (TWO) PVec<WT>::unpack(pf.r[1][ch], w1);
#pragma unroll
            for (int j = 0; j < N; j += 4) {
                const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + c + j);
                acc0 = fmaf(w0[j], xv.x, acc0); acc0 = fmaf(w0[j + 1], xv.y, acc0);
                acc0 = fmaf(w0[j + 2], xv.z, acc0); acc0 = fmaf(w0[j + 3], xv.w, acc0);
                if (TWO) {
                    acc1 = fmaf(w1[j], xv.x, acc1); acc1 = fmaf(w1[j + 1], xv.y, acc1);
                    acc1 = fmaf(w1[j + 2], xv.z, acc1); acc1 = fmaf(w1[j + 3], xv.w, acc1);
                }
            }
        }
    }
    for (int c = (PPF * 64 + lane) * N; c < cols; c += 64 * N) {
        float w0[N], w1[N];
        PVec<WT>::unpack(PVec<WT>::load(W + (size_t)row * ld + c), w0);
        if (TWO) PVec<WT>::unpack(PVec<WT>::load(W + (size_t)row2 * ld + c), w1);
#pragma unroll
        for (int j = 0; j < N; j += 4) {
            const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + c + j);
            acc0 = fmaf(w0[j], xv.x, acc0); acc0 = fmaf(w0[j + 1], xv.y, acc0);
            acc0 = fmaf(w0[j + 2], xv.z, acc0); acc0 = fmaf(w0[j + 3], xv.w, acc0);
            if (TWO) {
                acc1 = fmaf(w1[j], xv.x, acc1); acc1 = fmaf(w1[j + 1], xv.y, acc1);
                acc1 = fmaf(w1[j + 2], xv.z, acc1); acc1 = fmaf(w1[j + 3], xv.w, acc1);
            }
        }
    }
}

// One row streamed from memory (rows beyond a wave's first).
template <typename WT>
__device__ __forceinline__ float dot_stream(const WT* __restrict__ W, size_t ld, int row, int cols, const float* xs) {
    constexpr int N = PVec<WT>::N;
    const int lane = threadIdx.x & 63;
    float acc = 0.f;
    for (int c = lane * N; c < cols; c += 64 * N) {
        float w[N];
        PVec<WT>::unpack(PVec<WT>::load(W + (size_t)row * ld + c), w);
#pragma unroll
        for (int j = 0; j < N; j += 4) {
            const f32x4 xv = *reinterpret_cast<const f32x4*>(xs + c + j);
            acc = fmaf(w[j], xv.x, acc); acc = fmaf(w[j + 1], xv.y, acc);
            acc = fmaf(w[j + 2], xv.z, acc); acc = fmaf(w[j + 3], xv.w, acc);
        }
    }
    return acc;
}

// This wave's rows of a phase: gw, gw + TW, gw + 2 TW, ...  The first two are prefetched.
template <typename WT>
__device__ __forceinline__ void pf_first(RowPf<WT>& pf, const WT* __restrict__ W, size_t ld, int nrows, int cols, int gw, int TW) {
    pf_rows<WT>(pf, W, ld, gw < nrows ? gw : -1, gw + TW < nrows ? gw + TW : -1, cols);
}

// out(row, W[row] . xs (+ Wb[row] . xb)) for every row of this wave.
template <typename WT, typename Epi>
__device__ __forceinline__ void rows_phase(const RowPf<WT>& pf, const WT* __restrict__ W, size_t ld, int nrows, int cols,
                                           const float* xs, const WT* __restrict__ Wb, int colsb, const float* xb,
                                           int gw, int TW, Epi epi) {
    const int lane = threadIdx.x & 63;
    for (int row = gw; row < nrows; row += 2 * TW) {
        const int row2 = row + TW < nrows ? row + TW : -1;
        float a0 = 0.f, a1 = 0.f;
        if (row == gw) {
            if (row2 >= 0) dot_pf<WT, true>(pf, W, ld, row, row2, cols, xs, a0, a1);
            else dot_pf<WT, false>(pf, W, ld, row, -1, cols, xs, a0, a1);
        } else {
            a0 = dot_stream<WT>(W, ld, row, cols, xs);
            if (row2 >= 0) a1 = dot_stream<WT>(W, ld, row2, cols, xs);
        }
        if (colsb > 0) {
            a0 += dot_stream<WT>(Wb, colsb, row, colsb, xb);
            if (row2 >= 0) a1 += dot_stream<WT>(Wb, colsb, row2, colsb, xb);
        }
        a0 = pwave_sum(a0);
        if (lane == 0) epi(row, a0);
        if (row2 >= 0) {
            a1 = pwave_sum(a1);
            if (lane == 0) epi(row2, a1);
        }
    }
}

struct PersistArgs {
    StepArgs a;
    const LayerDev* layers; // device copy of the per-layer table
    int NL;
    int steps;
    int seq;
    unsigned* sync;      // barrier words, zero at launch: [0] top, [64*(1+g)] group g, [64*(9+g)] release g
    unsigned* abortFlag; // set when a bounded wait expires; every workgroup then leaves
    float* pamaxVal;     // [grid] per-workgroup best logit
    int* pamaxIdx;
    float* kvPart;       // attention partials [heads * maxTiles * (hd + 2)]
    int maxTiles;
    int stageFloats;     // LDS staging vector length
    int abortAtStep;     // test hook: > 0 makes workgroup 0 raise the abort flag when it reaches this step of the launch
    unsigned long long* timing; // optional (may be null): phase timestamps of workgroup 0 during the last step
};

// Diagnostic: workgroup 0 records the constant-rate clock at phase boundaries of the last step.
#define P_STAMP(slot)                                                                             \
    do {                                                                                          \
        if (P.timing && wg == 0 && tid == 0 && step == P.steps - 1) P.timing[(slot)] = wall_clock64(); \
    } while (0)

// Grid barrier in two halves, so that loads issued between them overlap the wait.  Workgroups of one
// XCD (blockIdx % 8) arrive on their group word, the last of a group arrives on the top word, the
// last there publishes the epoch to the eight release words.
__device__ __forceinline__ void grid_arrive(const PersistArgs& P, unsigned& epoch) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup"); // this thread's write-through stores have completed
    lds_barrier();
    epoch++;
    if (threadIdx.x == 0) {
        const unsigned n = gridDim.x, g = blockIdx.x & 7, gsize = (n + 7 - g) >> 3;
        unsigned* gc = P.sync + 64 * (1 + g);
        const unsigned prev = __hip_atomic_fetch_add(gc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == epoch * gsize - 1) {
            const unsigned ngroups = n < 8 ? n : 8;
            const unsigned p2 = __hip_atomic_fetch_add(P.sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (p2 == epoch * ngroups - 1)
                for (unsigned k = 0; k < ngroups; k++) astu(P.sync + 64 * (9 + k), epoch);
        }
    }
}

// Returns false when the wait was abandoned (the abort flag is then set for everyone).
__device__ __forceinline__ bool grid_wait(const PersistArgs& P, unsigned epoch) {
    __shared__ unsigned s_ok;
    if (threadIdx.x == 0) {
        const unsigned* rel = P.sync + 64 * (9 + (blockIdx.x & 7));
        unsigned spins = 0, ok = 1;
        // the first look takes the abort flag along (both loads are in flight together): a launch whose flag is already
        // raised is left by every workgroup at its first wait, before anything of the sequence has been written
        const unsigned r0 = aldu(rel), ab0 = aldu(P.abortFlag);
        if (ab0) ok = 0;
        else if (r0 < epoch)
            while (aldu(rel) < epoch) {
                if (++spins > P_SPIN_LIMIT || ((spins & 1023) == 0 && aldu(P.abortFlag))) { astu(P.abortFlag, 1u); ok = 0; break; }
            }
        s_ok = ok;
    }
    lds_barrier();
    return s_ok != 0;
}

// Block-wide sum over PWAVES waves (red: PWAVES floats of LDS).
__device__ __forceinline__ float block_sum(float v, float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v = pwave_sum(v);
    lds_barrier();
    if (lane == 0) red[wave] = v;
    lds_barrier();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < PWAVES; w++) t += red[w];
    return t;
}

// dst = gamma * (src / sqrt(mean(src^2) + 1e-8)) over LDS vectors (inference.cu:24-50, 83-95).
__device__ __forceinline__ void lds_rmsnorm(const float* src, const float* __restrict__ gamma, int n, float* dst, float* red) {
    float part = 0.f;
    for (int i = threadIdx.x; i < n; i += PWG) part = fmaf(src[i], src[i], part);
    const float tot = block_sum(part, red);
    const float r = sqrtf(tot / (float)n + 1e-8f);
    for (int i = threadIdx.x; i < n; i += PWG) dst[i] = gamma[i] * (src[i] / r);
    lds_barrier();
}

template <int HD> struct PAttn {
    static constexpr int NW = (HD <= 64) ? 4 : 2; // waves of a workgroup that take attention tiles
    static constexpr int LDK = HD + 4;
    static constexpr int EPL = HD / 64;
    static constexpr int TILE_FLOATS = 64 * LDK + 4 * HD; // K/V tile + q, k, v, spare rows
};

template <typename WT, int HD, int GDK>
__global__ void __launch_bounds__(PWG) k_decode_persistent(PersistArgs P) {
    extern __shared__ float lds[];
    const StepArgs& a = P.a;
    const int d = a.dim, F = a.ffn, V = a.vocab;
    float* xres = lds;                 // [d] residual stream entering the layer
    float* h1res = xres + d;           // [d] residual after the mixing block
    float* stage = h1res + d;          // [stageFloats] normed input / mixing output / FFN activations
    float* red = stage + P.stageFloats; // [PWAVES + 2*PWAVES] reductions and argmax scratch
    float* g1s = red + 4 * PWAVES;     // [d] rms1 gain of the current layer (final gain during the LM head)
    float* g2s = g1s + d;              // [d] rms2 gain
    float* gqs = g2s + d;              // [d] per-head q gain
    float* gks = gqs + d;              // [d] per-head k gain
    float* tiles = gks + d;            // attention tiles, PAttn<HD>::NW x TILE_FLOATS
    LayerDev* Ls = reinterpret_cast<LayerDev*>(tiles + PAttn<HD>::NW * PAttn<HD>::TILE_FLOATS); // the layer table (8-byte aligned: all lengths above are even)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < P.NL * (int)(sizeof(LayerDev) / 4); i += PWG)
        reinterpret_cast<uint32_t*>(Ls)[i] = reinterpret_cast<const uint32_t*>(P.layers)[i];
    lds_barrier();
    const int G = gridDim.x, wg = blockIdx.x;
    const int TW = G * PWAVES;         // waves in the grid
    const int gw = wave * G + wg;      // consecutive rows land on different workgroups
    const int seq = P.seq;
    unsigned epoch = 0;
    int tok = a.tok[0];
    int pos = a.pos[seq];
    RowPf<WT> pf;

    for (int step = 0; step < P.steps; step++) {
        if (P.abortAtStep > 0 && step == P.abortAtStep && wg == 0 && tid == 0) astu(P.abortFlag, 1u); // test hook: given up in mid-launch
        // embedding gather (inference.cu:9-22): every workgroup keeps its own copy of the residual stream
        for (int i = tid; i < d; i += PWG) xres[i] = PVec<WT>::one((const WT*)a.E + (size_t)tok * d + i);
        pf_first<WT>(pf, (const WT*)Ls[P.NL - 1].Wa, d, Ls[P.NL - 1].rowsA, d, gw, TW);

        for (int t = P.NL - 1; t >= 0; t--) { // file block 0 is the top of the stack (inference.cu:384-385)
            // The layer table sits in LDS (copied once at kernel start): no dependent global loads for the
            // pointers, and no registers held for them; gains and the residual stream arrive in one round of loads.
            const LayerDev& L = Ls[t];
            const LayerDev& Lnext = Ls[t > 0 ? t - 1 : P.NL - 1];
            const int ts = (P.NL - 1 - t) * 16;
            P_STAMP(ts + 0);
            {
                const bool qk = a.qkNorm && L.kind == MLH_KIND_ATTENTION;
                for (int i = tid; i < d; i += PWG) {
                    if (t != P.NL - 1) xres[i] = ald(a.x + i);
                    g1s[i] = L.g1[i];
                    g2s[i] = L.g2[i];
                    if (qk) { gqs[i] = L.gq[i]; gks[i] = L.gk[i]; }
                }
                lds_barrier();
            }
            // ------------------------------------------------------------------ phase A
            lds_rmsnorm(xres, g1s, d, stage, red);
            P_STAMP(ts + 1);
            rows_phase<WT>(pf, (const WT*)L.Wa, d, L.rowsA, d, stage, (const WT*)nullptr, 0, nullptr, gw, TW,
                           [&](int row, float v) { ast(a.qkv + row, v); });
            P_STAMP(ts + 2);
            grid_arrive(P, epoch);
            if (!grid_wait(P, epoch)) return;
            P_STAMP(ts + 3);

            // ------------------------------------------------------------------ phase B
            if (L.kind == MLH_KIND_ATTENTION) {
                constexpr int NW = PAttn<HD>::NW, LDK = PAttn<HD>::LDK, EPL = PAttn<HD>::EPL;
                constexpr int LPR = HD / 4, RPI = 64 / LPR, NLD = 64 / RPI;
                const int T = pos + 1, ntiles = (T + 63) >> 6, newTile = pos >> 6;
                const int nunits = a.heads * ntiles;
                if (wave < NW) {
                    float* tile = tiles + wave * PAttn<HD>::TILE_FLOATS;
                    float* qs = tile + 64 * LDK;
                    float* ks = qs + HD;
                    float* vn = ks + HD;
                    const int lrow = lane / LPR, c4 = (lane % LPR) * 4;
                    for (int u = wave * G + wg; u < nunits; u += NW * G) {
                        const int h = u % a.heads, tl = u / a.heads, j0 = tl << 6;
                        const int page = a.pageTable[seq * a.pagesPerSeq + tl];
                        const size_t base = ((size_t)page * MLH_KV_PAGE) * d + h * HD;
                        // One staging set of registers, at most 16 loads of 16 bytes per lane at a time (a 128-wide head's
                        // tile in two batches: 32 at once left no registers for the prefetched weight rows and spilled
                        // ~250 of them): K tile first, reused for the V tile once K sits in LDS.  The loads are
                        // unconditional (every row of a page is mapped; rows at or behind this step's position are
                        // replaced on the way into LDS): a load under a per-row condition becomes a branch with a wait.
                        constexpr int BL = NLD > 16 ? 16 : NLD, NB = NLD / BL;
                        f32x4 kreg[BL];
                        auto issue = [&](const float* src, int b) {
#pragma unroll
                            for (int it = 0; it < BL; it++)
                                kreg[it] = *reinterpret_cast<const f32x4*>(src + base + (size_t)((b * BL + it) * RPI + lrow) * d + c4);
                        };
                        auto put = [&](int b, const float* newRow) { // rows before this step's from the registers, this step's from LDS, later ones zero
#pragma unroll
                            for (int it = 0; it < BL; it++) {
                                const int row = (b * BL + it) * RPI + lrow;
                                f32x4 v = (j0 + row < pos) ? kreg[it] : (f32x4)(0.f);
                                if (j0 + row == pos) v = *reinterpret_cast<const f32x4*>(newRow + c4);
                                *reinterpret_cast<f32x4*>(tile + row * LDK + c4) = v;
                            }
                        };
                        issue(L.K, 0);
                        const float rc0 = a.rope[(size_t)pos * HD + (EPL == 1 ? (lane & ~1) : 2 * lane)];
                        const float rs0 = a.rope[(size_t)pos * HD + (EPL == 1 ? (lane | 1) : 2 * lane + 1)];
                        // q (and, for the tile that receives this step's row, k and v): per-head RMSNorm
                        // (inference.cu:52-81, 97-111) then RoPE on adjacent pairs (inference.cu:113-134)
                        const bool own = tl == newTile;
                        float qv[EPL], kv[EPL], vv[EPL];
#pragma unroll
                        for (int e = 0; e < EPL; e++) {
                            const int i = lane * EPL + e;
                            qv[e] = ald(a.qkv + h * HD + i);
                            kv[e] = own ? ald(a.qkv + L.offK + h * HD + i) : 0.f;
                            vv[e] = own ? ald(a.qkv + L.offV + h * HD + i) : 0.f;
                        }
                        if (a.qkNorm) {
                            float sq = 0.f, sk = 0.f;
#pragma unroll
                            for (int e = 0; e < EPL; e++) { sq = fmaf(qv[e], qv[e], sq); sk = fmaf(kv[e], kv[e], sk); }
                            sq = pwave_sum(sq); sk = pwave_sum(sk);
                            const float rq = sqrtf(sq / (float)HD + 1e-8f), rk = sqrtf(sk / (float)HD + 1e-8f);
#pragma unroll
                            for (int e = 0; e < EPL; e++) {
                                const int i = lane * EPL + e;
                                qv[e] = gqs[h * HD + i] * (qv[e] / rq);
                                kv[e] = gks[h * HD + i] * (kv[e] / rk);
                            }
                        }
                        if (EPL == 1) { // pair (2i, 2i+1) sits in lanes (2i, 2i+1)
                            const float c = rc0, s = rs0;
                            const float qo = __shfl_xor(qv[0], 1, MLH_WAVE), ko = __shfl_xor(kv[0], 1, MLH_WAVE);
                            if (lane & 1) { qv[0] = s * qo + c * qv[0]; kv[0] = s * ko + c * kv[0]; }
                            else { qv[0] = c * qv[0] - s * qo; kv[0] = c * kv[0] - s * ko; }
                        } else { // the lane holds the pair (2*lane, 2*lane+1)
                            const float c = rc0, s = rs0;
                            const float q0 = qv[0], q1 = qv[EPL - 1], k0 = kv[0], k1 = kv[EPL - 1];
                            qv[0] = c * q0 - s * q1; qv[EPL - 1] = s * q0 + c * q1;
                            kv[0] = c * k0 - s * k1; kv[EPL - 1] = s * k0 + c * k1;
                        }
#pragma unroll
                        for (int e = 0; e < EPL; e++) {
                            const int i = lane * EPL + e;
                            qs[i] = qv[e]; ks[i] = kv[e]; vn[i] = vv[e];
                            if (own) { // append this step's row to the cache (write-through: read next step by any XCD)
                                const size_t o = base + (size_t)(pos - j0) * d + i;
                                ast(L.K + o, kv[e]);
                                ast(L.V + o, vv[e]);
                            }
                        }
                        __builtin_amdgcn_wave_barrier();
                        put(0, ks);
#pragma unroll
                        for (int b = 1; b < NB; b++) { issue(L.K, b); put(b, ks); }
                        // V tile loads go out now, into the same registers, and fly during the score computation
                        issue(L.V, 0);
                        __builtin_amdgcn_wave_barrier();
                        float s = 0.f;
                        {
                            const float* kr = tile + lane * LDK;
#pragma unroll
                            for (int i = 0; i < HD; i += 4) {
                                const f32x4 kk = *reinterpret_cast<const f32x4*>(kr + i);
                                const f32x4 qq = *reinterpret_cast<const f32x4*>(qs + i);
                                s = fmaf(kk.x, qq.x, s); s = fmaf(kk.y, qq.y, s); s = fmaf(kk.z, qq.z, s); s = fmaf(kk.w, qq.w, s);
                            }
                        }
                        const bool valid = j0 + lane < T;
                        s = valid ? s / sqrtf((float)HD) : -1.0e30f; // inference.cu:154
                        const float m = pwave_max(s);
                        const float e = valid ? expf(s - m) : 0.f;
                        const float l = pwave_sum(e);
                        __builtin_amdgcn_wave_barrier();
                        put(0, vn);
#pragma unroll
                        for (int b = 1; b < NB; b++) { issue(L.V, b); put(b, vn); }
                        __builtin_amdgcn_wave_barrier();
                        float acc[EPL];
#pragma unroll
                        for (int ee = 0; ee < EPL; ee++) acc[ee] = 0.f;
#pragma unroll
                        for (int j = 0; j < 64; j++) {
                            const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(e), j));
#pragma unroll
                            for (int ee = 0; ee < EPL; ee++) acc[ee] = fmaf(pj, tile[j * LDK + lane + 64 * ee], acc[ee]);
                        }
                        float* out = P.kvPart + ((size_t)h * P.maxTiles + tl) * (HD + 2);
#pragma unroll
                        for (int ee = 0; ee < EPL; ee++) ast(out + lane + 64 * ee, acc[ee]);
                        if (lane == 0) { ast(out + HD, m); ast(out + HD + 1, l); }
                        __builtin_amdgcn_wave_barrier();
                    }
                }
            } else if (GDK > 0) {
                // gated-delta-net: one head's state per workgroup; S <- alpha (S - beta (S k) k^T) + beta v k^T ; o = S q
                constexpr int DK = GDK > 0 ? GDK : 64, DV = DK;
                constexpr int EPT = DK * DV / PWG; // state elements per thread, contiguous in a row
                constexpr int TPR = DK / EPT;      // threads per state row
                float* qs = stage;                 // the normed input in `stage` is no longer needed
                float* ks = stage + DK;
                for (int h = wg; h < a.gdnHeads; h += G) {
                    lds_barrier();
                    for (int i = tid; i < DK; i += PWG) { qs[i] = ald(a.qkv + h * DK + i); ks[i] = ald(a.qkv + L.offK + h * DK + i); }
                    lds_barrier();
                    float sq = 0.f, sk = 0.f;
#pragma unroll 8
                    for (int i = 0; i < DK; i++) { sq = fmaf(qs[i], qs[i], sq); sk = fmaf(ks[i], ks[i], sk); }
                    const float rq = sqrtf(sq + 1e-6f), rk = sqrtf(sk + 1e-6f);
                    const float za = ald(a.qkv + L.offGa + h) + L.gdnBa[h];
                    const float zb = ald(a.qkv + L.offGb + h) + L.gdnBb[h];
                    const float alpha = expf(-(fmaxf(za, 0.f) + log1pf(expf(-fabsf(za)))));
                    const float beta = psigmoid(zb);
                    const int r = tid / TPR, c0 = (tid % TPR) * EPT;
                    const float vr = ald(a.qkv + L.offV + h * DV + r);
                    float* Srow = L.S + (((size_t)seq * a.gdnHeads + h) * DV + r) * DK + c0;
                    float S[EPT];
#pragma unroll
                    for (int c = 0; c < EPT; c += 4) {
                        const f32x4 v = *reinterpret_cast<const f32x4*>(Srow + c);
                        S[c] = v.x; S[c + 1] = v.y; S[c + 2] = v.z; S[c + 3] = v.w;
                    }
                    float u = 0.f;
#pragma unroll
                    for (int c = 0; c < EPT; c++) u = fmaf(S[c], ks[c0 + c] / rk, u);
#pragma unroll
                    for (int o = TPR / 2; o > 0; o >>= 1) u += __shfl_xor(u, o, MLH_WAVE);
                    float oacc = 0.f;
#pragma unroll
                    for (int c = 0; c < EPT; c++) {
                        const float kn = ks[c0 + c] / rk;
                        S[c] = alpha * (S[c] - beta * u * kn) + beta * vr * kn;
                        oacc = fmaf(S[c], qs[c0 + c] / rq, oacc);
                    }
#pragma unroll
                    for (int o = TPR / 2; o > 0; o >>= 1) oacc += __shfl_xor(oacc, o, MLH_WAVE);
                    // the state of a head is always handled by the same workgroup, so ordinary stores do:
                    // the only other readers come after the end of the kernel
#pragma unroll
                    for (int c = 0; c < EPT; c += 4) {
                        f32x4 v; v.x = S[c]; v.y = S[c + 1]; v.z = S[c + 2]; v.w = S[c + 3];
                        *reinterpret_cast<f32x4*>(Srow + c) = v;
                    }
                    if ((tid % TPR) == 0) ast(a.mix + h * DV + r, oacc);
                }
            }
            P_STAMP(ts + 4);
            grid_arrive(P, epoch);
            pf_first<WT>(pf, (const WT*)L.Wo, L.ad, d, L.ad, gw, TW);
            if (!grid_wait(P, epoch)) return;
            P_STAMP(ts + 5);

            // ------------------------------------------------------------------ phase C
            {
                const int ad = L.ad, pl = a.ple;
                float* as = stage;
                float* es = stage + ad;
                if (L.kind == MLH_KIND_ATTENTION) {
                    const int ntiles = (pos + 64) >> 6;
                    for (int i = tid; i < ad; i += PWG) {
                        const int h = i / HD, e = i - h * HD;
                        const float* pp = P.kvPart + ((size_t)h * P.maxTiles) * (HD + 2);
                        // partials are fetched eight tiles at a time, all loads of a batch in flight together
                        float M = -1.0e30f, num = 0.f, den = 0.f;
                        for (int t0 = 0; t0 < ntiles; t0 += 8) {
                            float pm[8], pl_[8], pa[8];
#pragma unroll
                            for (int k = 0; k < 8; k++) {
                                const bool in = t0 + k < ntiles;
                                const float* q = pp + (in ? t0 + k : 0) * (HD + 2);
                                pm[k] = in ? ald(q + HD) : -1.0e30f;
                                pl_[k] = in ? ald(q + HD + 1) : 0.f;
                                pa[k] = in ? ald(q + e) : 0.f;
                            }
                            float Mb = M;
#pragma unroll
                            for (int k = 0; k < 8; k++) Mb = fmaxf(Mb, pm[k]);
                            const float corr = expf(M - Mb);
                            num *= corr; den *= corr;
#pragma unroll
                            for (int k = 0; k < 8; k++) {
                                const float w = expf(pm[k] - Mb);
                                num = fmaf(w, pa[k], num);
                                den = fmaf(w, pl_[k], den);
                            }
                            M = Mb;
                        }
                        float v = num / den;
                        if (a.gating) v = v * psigmoid(ald(a.qkv + L.offG + i)); // inference.cu:241-250
                        as[i] = v;
                    }
                } else {
                    for (int i = tid; i < ad; i += PWG) as[i] = ald(a.mix + i);
                }
                for (int j = tid; j < pl; j += PWG)
                    es[j] = psilu(ald(a.qkv + L.offPle + j)) * PVec<WT>::one((const WT*)L.pleTable + (size_t)tok * pl + j);
                lds_barrier();
                P_STAMP(ts + 6);
                rows_phase<WT>(pf, (const WT*)L.Wo, ad, d, ad, as, (const WT*)L.pleUp, pl, es, gw, TW,
                               [&](int row, float v) { ast(a.h1 + row, v + xres[row]); }); // inference.cu:252-260
            }
            P_STAMP(ts + 7);
            grid_arrive(P, epoch);
            {
                const int pr = gw < F ? gw : -1;
                pf_rows<WT>(pf, (const WT*)L.W13, d, pr < 0 ? -1 : 2 * pr, pr < 0 ? -1 : 2 * pr + 1, d);
            }
            if (!grid_wait(P, epoch)) return;
            P_STAMP(ts + 8);

            // ------------------------------------------------------------------ phase D
            for (int i = tid; i < d; i += PWG) h1res[i] = ald(a.h1 + i);
            lds_barrier();
            lds_rmsnorm(h1res, g2s, d, stage, red);
            P_STAMP(ts + 9);
            for (int pr = gw; pr < F; pr += TW) {
                float g = 0.f, up = 0.f;
                if (pr == gw) dot_pf<WT, true>(pf, (const WT*)L.W13, d, 2 * pr, 2 * pr + 1, d, stage, g, up);
                else { g = dot_stream<WT>((const WT*)L.W13, d, 2 * pr, d, stage); up = dot_stream<WT>((const WT*)L.W13, d, 2 * pr + 1, d, stage); }
                g = pwave_sum(g); up = pwave_sum(up);
                if (lane == 0) ast(a.u + pr, psilu(g) * up); // inference.cu:262-281
            }
            P_STAMP(ts + 10);
            grid_arrive(P, epoch);
            pf_first<WT>(pf, (const WT*)L.W2, F, d, F, gw, TW);
            if (!grid_wait(P, epoch)) return;
            P_STAMP(ts + 11);

            // ------------------------------------------------------------------ phase E
            lds_barrier();
            for (int i = tid; i < F; i += PWG) stage[i] = ald(a.u + i);
            lds_barrier();
            P_STAMP(ts + 12);
            rows_phase<WT>(pf, (const WT*)L.W2, F, d, F, stage, (const WT*)nullptr, 0, nullptr, gw, TW,
                           [&](int row, float v) { ast(a.x + row, v + h1res[row]); }); // inference.cu:283-291
            P_STAMP(ts + 13);
            grid_arrive(P, epoch);
            if (t > 0) pf_first<WT>(pf, (const WT*)Lnext.Wa, d, Lnext.rowsA, d, gw, TW);
            else pf_first<WT>(pf, (const WT*)a.E, d, V, d, gw, TW);
            if (!grid_wait(P, epoch)) return;
            P_STAMP(ts + 14);
            P_STAMP(ts + 15);
        }

        // ---------------------------------------------------------------------- LM head + argmax
        for (int i = tid; i < d; i += PWG) { xres[i] = ald(a.x + i); g1s[i] = a.gF[i]; }
        lds_barrier();
        lds_rmsnorm(xres, g1s, d, stage, red); // inference.cu:705-715
        float best = -3.0e38f;
        int bidx = 0x7fffffff;
        for (int row = gw; row < V; row += 2 * TW) { // rows ascend per wave: ties keep the lower index
            const int row2 = row + TW < V ? row + TW : -1;
            float a0 = 0.f, a1 = 0.f;
            if (row == gw) {
                if (row2 >= 0) dot_pf<WT, true>(pf, (const WT*)a.E, d, row, row2, d, stage, a0, a1);
                else dot_pf<WT, false>(pf, (const WT*)a.E, d, row, -1, d, stage, a0, a1);
            } else {
                a0 = dot_stream<WT>((const WT*)a.E, d, row, d, stage);
                if (row2 >= 0) a1 = dot_stream<WT>((const WT*)a.E, d, row2, d, stage);
            }
            a0 = pwave_sum(a0);
            if (lane == 0) a.logits[(size_t)seq * V + row] = a0;
            if (a0 > best) { best = a0; bidx = row; }
            if (row2 >= 0) {
                a1 = pwave_sum(a1);
                if (lane == 0) a.logits[(size_t)seq * V + row2] = a1;
                if (a1 > best) { best = a1; bidx = row2; }
            }
        }
        {
            float* bv = red + PWAVES;
            int* bi = (int*)(red + 2 * PWAVES);
            lds_barrier();
            if (lane == 0) { bv[wave] = best; bi[wave] = bidx; }
            lds_barrier();
            if (tid == 0) {
                float v = bv[0];
                int i = bi[0];
                for (int w = 1; w < PWAVES; w++)
                    if (bv[w] > v || (bv[w] == v && bi[w] < i)) { v = bv[w]; i = bi[w]; }
                ast(P.pamaxVal + wg, v);
                astu((unsigned*)P.pamaxIdx + wg, (unsigned)i);
            }
        }
        grid_arrive(P, epoch);
        if (!grid_wait(P, epoch)) return;
        {
            float v = -3.0e38f;
            int i = 0x7fffffff;
            for (int k = tid; k < G; k += PWG) {
                const float v2 = ald(P.pamaxVal + k);
                const int i2 = (int)aldu((const unsigned*)P.pamaxIdx + k);
                if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
            }
            // reduce (v, i) over the block: value max, lowest index on ties
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float v2 = __shfl_xor(v, o, MLH_WAVE);
                const int i2 = __shfl_xor(i, o, MLH_WAVE);
                if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
            }
            float* bv = red + PWAVES;
            int* bi = (int*)(red + 2 * PWAVES);
            lds_barrier();
            if (lane == 0) { bv[wave] = v; bi[wave] = i; }
            lds_barrier();
            v = bv[0]; i = bi[0];
#pragma unroll
            for (int w = 1; w < PWAVES; w++)
                if (bv[w] > v || (bv[w] == v && bi[w] < i)) { v = bv[w]; i = bi[w]; }
            if (i < 0 || i >= V) i = 0; // only reachable with non-finite logits
            tok = i;
            pos += 1;
            if (wg == 0 && tid == 0) { // the append of inference_orchestrator.cu:149-151, kept on the device
                const int sc = *a.stepCounter;
                if (sc + step < a.outCapacity) a.outIds[sc + step] = tok;
            }
            lds_barrier();
        }
    }
    if (wg == 0 && tid == 0) {
        *a.stepCounter += P.steps;
        a.pos[seq] = pos;
        ((int*)a.tok)[0] = tok;
        a.nextTok[seq] = tok;
    }
}

__global__ void k_set_word(unsigned* p, unsigned v) { *p = v; }

// The barrier kernel stores the updated gated-delta-net state of every GDN layer at every step, so a launch that
// gives up in mid-run has advanced the states of the steps it finished.  Before the launch the states of the
// sequence are copied aside (blockIdx.y = layer, n floats per layer), and put back before the steps are redone.
__global__ void k_gdn_snapshot(const LayerDev* layers, int seq, int n, float* snap, int restore) {
    const LayerDev& L = layers[blockIdx.y];
    if (L.kind != MLH_KIND_GDN) return;
    f32x4* state = reinterpret_cast<f32x4*>(L.S + (size_t)seq * n);
    f32x4* keep = reinterpret_cast<f32x4*>(snap + (size_t)blockIdx.y * n);
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n / 4; i += gridDim.x * blockDim.x) {
        if (restore) state[i] = keep[i];
        else keep[i] = state[i];
    }
}

__global__ void k_zero_words(unsigned* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
template <typename WT, int HD, int GDK>
static int launch_persistent(mlh_ctx* c, PersistArgs& P, size_t ldsBytes) {
    void* fn = reinterpret_cast<void*>(&k_decode_persistent<WT, HD, GDK>);
    if (!c->persistentPrepared) { // once per context
        MLH_CHECK(c, hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes));
        int perCu = 0;
        MLH_CHECK(c, hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, fn, PWG, ldsBytes));
        if (perCu < 1) { c->err = "persistent decode kernel does not fit on a compute unit"; return -1; }
        if (GDK > 0 && !c->gdnSnapshot) {
            int rc = mlh_dev_alloc_bytes(c, (void**)&c->gdnSnapshot, (size_t)c->hp.transformers * c->hp.gdnHeads * c->hp.gdnDk * c->hp.gdnDv * 4);
            if (rc) return rc;
        }
        c->persistentPrepared = true;
    }
    if (P.steps <= 0) return 0; // preparation only
    void* args[] = {&P};
    // All workgroups must be resident at once: the grid is one workgroup per compute unit and the
    // occupancy query above says each unit can hold one.  A plain launch then behaves like a
    // cooperative one (and, unlike it, is visible to rocprofv3 and capturable in a graph); if some
    // unit were busy with other work the bounded barrier wait gives up and the call reports it.
    if (GDK > 0) { // sequence 0's states as they are before the launch (see k_gdn_snapshot)
        const int n = c->hp.gdnHeads * c->hp.gdnDk * c->hp.gdnDv;
        hipLaunchKernelGGL(k_gdn_snapshot, dim3(std::min(64, (n / 4 + 255) / 256), c->hp.transformers), dim3(256), 0, c->stream,
                           (const LayerDev*)c->d_layers, P.seq, n, c->gdnSnapshot, 0);
    }
    if (c->persistCooperative) {
        MLH_CHECK(c, hipLaunchCooperativeKernel(fn, dim3(c->numCUs), dim3(PWG), args, (unsigned)ldsBytes, c->stream));
    } else {
        hipLaunchKernelGGL((k_decode_persistent<WT, HD, GDK>), dim3(c->numCUs), dim3(PWG), ldsBytes, c->stream, P);
        MLH_CHECK(c, hipGetLastError());
    }
    return 0;
}

// After a barrier-kernel launch that gave up: sequence 0's gated-delta-net states go back to what they were before it.
int mlh_persistent_restore_states(mlh_ctx* c) {
    if (!c->gdnSnapshot) return 0; // no GDN layers
    const int n = c->hp.gdnHeads * c->hp.gdnDk * c->hp.gdnDv;
    hipLaunchKernelGGL(k_gdn_snapshot, dim3(std::min(64, (n / 4 + 255) / 256), c->hp.transformers), dim3(256), 0, c->stream,
                       (const LayerDev*)c->d_layers, 0, n, c->gdnSnapshot, 1);
    MLH_CHECK(c, hipGetLastError());
    return 0;
}

// True when the persistent kernel supports this context's shape.
bool mlh_persistent_supported(const mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    bool gdn = false;
    for (int t = 0; t < hp.transformers; t++) gdn = gdn || hp.layerKinds[t] == MLH_KIND_GDN;
    if (hp.headDim != 64 && hp.headDim != 128) return false;
    if (gdn && !(hp.gdnDk == hp.headDim && hp.gdnDv == hp.headDim)) return false;
    if (gdn && hp.gdnHeads > c->numCUs) return false;
    return c->numCUs >= 8;
}

// Enqueues `steps` decode steps of sequence 0 (slot 0) in one cooperative launch.
int mlh_launch_persistent(mlh_ctx* c, int steps) {
    const mlh_hparams& hp = c->hp;
    PersistArgs P;
    mlh_fill_args(c, P.a, 1, c->d_tok);
    P.layers = c->d_layers;
    P.NL = hp.transformers;
    P.steps = steps;
    P.seq = 0;
    P.sync = c->d_sync;
    P.abortFlag = c->d_sync + 64 * 20;
    P.pamaxVal = c->pamaxVal;
    P.pamaxIdx = c->pamaxIdx;
    P.kvPart = c->kvPart;
    P.maxTiles = c->pagesPerSeq;
    P.timing = c->d_timing;
    P.abortAtStep = 0;
    int stage = std::max(std::max(hp.dim, hp.ffnDim), c->maxAd + hp.pleDim);
    stage = (stage + 3) & ~3;
    P.stageFloats = stage;
    bool gdn = false;
    for (int t = 0; t < hp.transformers; t++) gdn = gdn || hp.layerKinds[t] == MLH_KIND_GDN;
    const int hd = hp.headDim;
    const size_t tileFloats = hd == 64 ? (size_t)PAttn<64>::NW * PAttn<64>::TILE_FLOATS : (size_t)PAttn<128>::NW * PAttn<128>::TILE_FLOATS;
    const size_t ldsBytes = ((size_t)6 * hp.dim + stage + 4 * PWAVES + tileFloats) * 4 + (size_t)hp.transformers * sizeof(LayerDev);
    if (ldsBytes > 160 * 1024) { c->err = "model too wide for the persistent decode kernel"; return -1; }
    if (steps > 0) {
        hipLaunchKernelGGL(k_zero_words, dim3(5), dim3(256), 0, c->stream, c->d_sync, 64 * 20); // barrier words
        // abort flag; test hook: a flag that starts raised makes every workgroup leave at its first wait
        hipLaunchKernelGGL(k_set_word, dim3(1), dim3(1), 0, c->stream, P.abortFlag, c->injectAbort > 0 ? 1u : 0u);
        if (c->injectAbort > 0) c->injectAbort--;
        P.abortAtStep = c->injectAbortStep;
        c->injectAbortStep = 0;
    }
    const bool bf = hp.weightDtype == MLH_DTYPE_BF16;
    if (hd == 64) {
        if (gdn) return bf ? launch_persistent<bf16_t, 64, 64>(c, P, ldsBytes) : launch_persistent<float, 64, 64>(c, P, ldsBytes);
        return bf ? launch_persistent<bf16_t, 64, 0>(c, P, ldsBytes) : launch_persistent<float, 64, 0>(c, P, ldsBytes);
    }
    if (gdn) return bf ? launch_persistent<bf16_t, 128, 128>(c, P, ldsBytes) : launch_persistent<float, 128, 128>(c, P, ldsBytes);
    return bf ? launch_persistent<bf16_t, 128, 0>(c, P, ldsBytes) : launch_persistent<float, 128, 0>(c, P, ldsBytes);
}
