// Decode-step kernels for gfx950 (wave64).  One decode step for `nseq` slots is
//
//   embed -> per layer { phaseA (RMSNorm + fused q|k|v|gate|ple|gdn GEMV)
//                        attention (QK-norm, RoPE, KV append, register-resident blocks of keys, running softmax)
//                          or gated-delta-net state update
//                        oproj (partials combine + gating + Wo GEMV + PLE + residual)
//                        ffn13 (RMSNorm + gate/up GEMV + SiLU*up)
//                        down  (W2 GEMV + residual) }
//         -> lmhead (final RMSNorm + tied-embedding GEMV + per-workgroup argmax) -> finish
//
// All GEMVs stream the weight matrix once in its file order (row-major
// [out, in]): one wavefront per output row, 16-byte loads per lane, the
// activation vector staged in LDS, butterfly reduction across the 64 lanes.
// The arithmetic follows inference.cu of the reference op for op (citations at
// each kernel); the reduction order inside a dot product is this file's own.
#include <type_traits>
#include "mlh_internal.h"
#include "persist_common.h"
#include "sample.h"

#define WG 256
#define WAVES (WG / MLH_WAVE)
#define RROWS 2 // rows one wave accumulates at a time

// ----------------------------------------------------------------------------
// small device helpers
// ----------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, MLH_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MLH_WAVE));
    return v;
}

template <typename WT>
struct WVec;
template <>
struct WVec<float> {
    static constexpr int N = 4;
    typedef float4 Raw;
    static __device__ __forceinline__ Raw loadRaw(const float* p) { return *reinterpret_cast<const float4*>(p); }
    static __device__ __forceinline__ void unpack(const Raw& v, float (&o)[4]) {
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
    static __device__ __forceinline__ void load(const float* p, float (&o)[4]) { unpack(loadRaw(p), o); }
    static __device__ __forceinline__ float one(const float* p) { return *p; }
};
template <>
struct WVec<bf16_t> {
    static constexpr int N = 8;
    typedef uint4 Raw;
    static __device__ __forceinline__ Raw loadRaw(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
    static __device__ __forceinline__ void unpack(const Raw& v, float (&o)[8]) {
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[8]) { unpack(loadRaw(p), o); }
    static __device__ __forceinline__ float one(const bf16_t* p) {
        return __uint_as_float(((uint32_t)*p) << 16);
    }
};

// Partial dot products of RROWS consecutive rows of W (row-major, leading dimension ldw)
// against NB vectors held in LDS (xs[b*xstride + c]).  Rows past nrows are clamped
// (their results are discarded by the caller).  Not yet reduced across lanes.
template <typename WT, int NB>
__device__ __forceinline__ void rows_dot(const WT* __restrict__ W, size_t ldw, int row0, int nrows,
                                         int cols, const float* xs, int xstride,
                                         float (&acc)[RROWS][NB]) {
    constexpr int N = WVec<WT>::N;
    const int lane = threadIdx.x & (MLH_WAVE - 1);
    const WT* rp[RROWS];
#pragma unroll
    for (int r = 0; r < RROWS; r++) {
        int row = row0 + r;
        if (row > nrows - 1) row = nrows - 1;
        rp[r] = W + (size_t)row * ldw;
    }
    for (int c = lane * N; c < cols; c += MLH_WAVE * N) {
        float w[RROWS][N];
#pragma unroll
        for (int r = 0; r < RROWS; r++) WVec<WT>::load(rp[r] + c, w[r]);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            float xv[N];
#pragma unroll
            for (int j = 0; j < N; j += 4) {
                float4 t = *reinterpret_cast<const float4*>(xs + b * xstride + c + j);
                xv[j] = t.x; xv[j + 1] = t.y; xv[j + 2] = t.z; xv[j + 3] = t.w;
            }
#pragma unroll
            for (int r = 0; r < RROWS; r++)
#pragma unroll
                for (int j = 0; j < N; j++) acc[r][b] = fmaf(w[r][j], xv[j], acc[r][b]);
        }
    }
}

// The first PF_CHUNKS 16-byte vectors per lane of each of a wave's RROWS rows, loaded ahead of the
// kernel's prologue: the weights do not depend on the activations, so their HBM latency overlaps
// the activation load, the RMSNorm reduction and the LDS staging.
#define PF_CHUNKS 8
template <typename WT>
struct Prefetched {
    typename WVec<WT>::Raw raw[RROWS][PF_CHUNKS];
};

template <typename WT>
__device__ __forceinline__ void prefetch_rows(Prefetched<WT>& pf, const WT* __restrict__ W, size_t ldw,
                                              int row0, int nrows, int cols) {
    constexpr int N = WVec<WT>::N;
    const int lane = threadIdx.x & (MLH_WAVE - 1);
#pragma unroll
    for (int r = 0; r < RROWS; r++) {
        int row = row0 + r;
        if (row > nrows - 1) row = nrows - 1;
        const WT* rp = W + (size_t)row * ldw;
#pragma unroll
        for (int ch = 0; ch < PF_CHUNKS; ch++) {
            const int c = (ch * MLH_WAVE + lane) * N;
            if (c < cols) pf.raw[r][ch] = WVec<WT>::loadRaw(rp + c);
        }
    }
}

// rows_dot for rows whose leading chunks were prefetched; columns beyond the prefetched span are streamed.
template <typename WT, int NB>
__device__ __forceinline__ void rows_dot_pf(const Prefetched<WT>& pf, const WT* __restrict__ W, size_t ldw,
                                            int row0, int nrows, int cols, const float* xs, int xstride,
                                            float (&acc)[RROWS][NB]) {
    constexpr int N = WVec<WT>::N;
    const int lane = threadIdx.x & (MLH_WAVE - 1);
#pragma unroll
    for (int ch = 0; ch < PF_CHUNKS; ch++) {
        const int c = (ch * MLH_WAVE + lane) * N;
        if (c < cols) {
            float w[RROWS][N];
#pragma unroll
            for (int r = 0; r < RROWS; r++) WVec<WT>::unpack(pf.raw[r][ch], w[r]);
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float xv[N];
#pragma unroll
                for (int j = 0; j < N; j += 4) {
                    float4 t = *reinterpret_cast<const float4*>(xs + b * xstride + c + j);
                    xv[j] = t.x; xv[j + 1] = t.y; xv[j + 2] = t.z; xv[j + 3] = t.w;
                }
#pragma unroll
                for (int r = 0; r < RROWS; r++)
#pragma unroll
                    for (int j = 0; j < N; j++) acc[r][b] = fmaf(w[r][j], xv[j], acc[r][b]);
            }
        }
    }
    if (cols > PF_CHUNKS * MLH_WAVE * N) {
        const WT* rp[RROWS];
#pragma unroll
        for (int r = 0; r < RROWS; r++) {
            int row = row0 + r;
            if (row > nrows - 1) row = nrows - 1;
            rp[r] = W + (size_t)row * ldw;
        }
        for (int c = (PF_CHUNKS * MLH_WAVE + lane) * N; c < cols; c += MLH_WAVE * N) {
            float w[RROWS][N];
#pragma unroll
            for (int r = 0; r < RROWS; r++) WVec<WT>::load(rp[r] + c, w[r]);
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float xv[N];
#pragma unroll
                for (int j = 0; j < N; j += 4) {
                    float4 t = *reinterpret_cast<const float4*>(xs + b * xstride + c + j);
                    xv[j] = t.x; xv[j + 1] = t.y; xv[j + 2] = t.z; xv[j + 3] = t.w;
                }
#pragma unroll
                for (int r = 0; r < RROWS; r++)
#pragma unroll
                    for (int j = 0; j < N; j++) acc[r][b] = fmaf(w[r][j], xv[j], acc[r][b]);
            }
        }
    }
}

// RMSNorm of NB vectors into LDS (inference.cu:24-50 + 83-95):
//   r = sqrtf(sum(x^2)/n + 1e-8f);  xs = gamma * (x / r)      (divide first, then the gain)
// red: LDS scratch of WAVES floats.  Slots >= nseq are zero-filled.
template <int NB>
__device__ __forceinline__ void rmsnorm_to_lds(const float* __restrict__ x, int xld, int slot0,
                                               int nseq, const float* __restrict__ gamma, int n,
                                               float* xs, int xstride, float* red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int slot = slot0 + b;
        const bool valid = slot < nseq;
        float part = 0.f;
        if (valid)
            for (int i = tid; i < n; i += WG) {
                float v = x[(size_t)slot * xld + i];
                part = fmaf(v, v, part);
            }
        part = wave_sum(part);
        __syncthreads();
        if (lane == 0) red[wave] = part;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) tot += red[w];
        const float r = sqrtf(tot / (float)n + 1e-8f);
        for (int i = tid; i < n; i += WG)
            xs[b * xstride + i] = valid ? gamma[i] * (x[(size_t)slot * xld + i] / r) : 0.f;
    }
    __syncthreads();
}

__device__ __forceinline__ float sigmoidf_ref(float v) { return 1.0f / (1.0f + expf(-v)); } // inference.cu:248
__device__ __forceinline__ float siluf_ref(float v) { return v / (1.0f + expf(-v)); }       // inference.cu:270

// ----------------------------------------------------------------------------
// embedding gather (inference.cu:9-22): x[slot] = E[tok[slot]]
// ----------------------------------------------------------------------------
template <typename WT>
__global__ void k_embed(StepArgs a) {
    const int slot = blockIdx.y;
    const int i = blockIdx.x * WG + threadIdx.x;
    if (slot >= a.nseq || i >= a.dim) return;
    const int t = a.tok[slot];
    a.x[(size_t)slot * a.dim + i] = WVec<WT>::one((const WT*)a.E + (size_t)t * a.dim + i);
}

// ----------------------------------------------------------------------------
// phase A: xn = RMSNorm(x, g1); qkv[slot] = Wa . xn
// replaces getRMSColSums + applyRMSNorm + the Q/K/V(/gate) cublasGemmEx calls
// (inference.cu:388-465, 487-507); the PLE gate rows and GDN alpha/beta rows ride along.
// ----------------------------------------------------------------------------
template <typename WT, int NB>
__global__ void __launch_bounds__(WG) k_phaseA(StepArgs a, LayerDev L, int rowsPerWg) {
    extern __shared__ float lds[];
    float* xs = lds;
    float* red = lds + NB * a.dim;
    const int slot0 = blockIdx.y * NB;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int rowBase = blockIdx.x * rowsPerWg;
    Prefetched<WT> pf;
    prefetch_rows<WT>(pf, (const WT*)L.Wa, a.dim, rowBase + wave * RROWS, L.rowsA, a.dim);
    rmsnorm_to_lds<NB>(a.x, a.dim, slot0, a.nseq, L.g1, a.dim, xs, a.dim, red);
    for (int r0 = wave * RROWS; r0 < rowsPerWg; r0 += WAVES * RROWS) {
        const int row0 = rowBase + r0;
        if (row0 >= L.rowsA) break;
        float acc[RROWS][NB] = {};
        if (r0 == wave * RROWS) rows_dot_pf<WT, NB>(pf, (const WT*)L.Wa, a.dim, row0, L.rowsA, a.dim, xs, a.dim, acc);
        else rows_dot<WT, NB>((const WT*)L.Wa, a.dim, row0, L.rowsA, a.dim, xs, a.dim, acc);
#pragma unroll
        for (int r = 0; r < RROWS; r++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float v = wave_sum(acc[r][b]);
                if (lane == 0 && row0 + r < L.rowsA && slot0 + b < a.nseq)
                    a.qkv[(size_t)(slot0 + b) * a.qkvStride + row0 + r] = v;
            }
    }
}

// ----------------------------------------------------------------------------
// attention: per (head, slot, split).  Replaces, for the newest column only,
// the per-head RMSNorm (inference.cu:52-81, 97-111), RoPE (113-134), the KtQ GEMM
// + scale/mask (511-539, 136-155), the three softmax kernels (157-239) and the
// V.P GEMM (549-573).  K and V of earlier positions come from the paged cache;
// this step's K/V row is written to it.  The sequence is cut into blocks of BR
// keys that go round the waves and never leave the registers: LPR lanes cover a
// key row with 16-byte pieces (the wave holds RPI rows per load instruction),
// a score is the 4-element partial product summed over the row's lanes on the
// vector ALU's lane-permute path, every lane of a row then knows the row's
// probability and scales its own piece of the V row with it.  Each of the RPI
// row groups keeps its own running (max, sum, output piece); they are merged
// once at the end.  The loads of the next block (K and V) are in flight while a
// block is worked on.  Partial (acc, m, l) per workgroup goes to a.part.
// ----------------------------------------------------------------------------
template <int HD>
struct AttnCfg {
    static constexpr int NW = (HD <= 64) ? 4 : 2; // waves per workgroup
    static constexpr int LPR = HD / 4;            // lanes per key row
    static constexpr int RPI = 64 / LPR;          // rows per load instruction = row groups of a wave
    static constexpr int BLD = 4;                 // load instructions per operand and block
    static constexpr int BR = BLD * RPI;          // key rows per block
    static constexpr int NBP = 64 / BR;           // blocks per page
};

// sum over the aligned group of W = 16 or 32 lanes; every lane of the group receives it
template <int W>
__device__ __forceinline__ float attn_row_sum(float v) {
    static_assert(W == 16 || W == 32, "a key row spans 16 or 32 lanes");
    v = pgroup_sum<16>(v);
    if (W == 32) v += __shfl_xor(v, 16, MLH_WAVE);
    return v;
}

template <int HD>
__global__ void __launch_bounds__(AttnCfg<HD>::NW * 64) k_attn(StepArgs a, LayerDev L) {
    constexpr int NW = AttnCfg<HD>::NW, LPR = AttnCfg<HD>::LPR, RPI = AttnCfg<HD>::RPI, BLD = AttnCfg<HD>::BLD, BR = AttnCfg<HD>::BR,
                  NBP = AttnCfg<HD>::NBP;
    extern __shared__ float lds[];
    float* qs = lds;                // [HD]
    float* ks = qs + HD;            // [HD]
    float* vn = ks + HD;            // [HD]
    float* comb = vn + HD;          // [NW][HD + 2]

    const int h = blockIdx.x, slot = blockIdx.y, sp = blockIdx.z;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int seq = a.sidx[slot];
    const int p = a.pos[seq];
    const int T = p + 1;
    const int dim = a.dim;
    const float* qkv = a.qkv + (size_t)slot * a.qkvStride;

    const int lrow = lane / LPR, c4 = (lane % LPR) * 4;
    const unsigned loff = (unsigned)(lrow * dim + c4); // this lane's offset inside a group of RPI rows: the rest of an address is uniform
    // blocks of BR keys go round the waves of the (head, slot)'s workgroups, so that a short sequence still
    // occupies every wave
    const int nblocks = (T + BR - 1) / BR;
    const int newBlock = p / BR;
    const int bstep = a.nsplit * NW;
    int b = sp * NW + wave;

    // Two register sets of one block each.  Every row of a block is loaded, also those at and beyond position p (the
    // page is allocated as a whole; what they hold is replaced below): a load that depends on a comparison would put
    // the compiler's wait for it in front of the next block's loads.
    f32x4 kb[2][BLD], vb[2][BLD];
    // first element of key row 0 of block b (blocks are numbered along the sequence; NBP of them share a page)
    auto block_base = [&](int b) {
        return ((size_t)a.pageTable[seq * a.pagesPerSeq + b / NBP] * MLH_KV_PAGE + (size_t)(b % NBP) * BR) * dim + h * HD;
    };
    auto issue = [&](size_t bbase, int set) {
#pragma unroll
        for (int it = 0; it < BLD; it++) {
            const size_t o = bbase + (size_t)(it * RPI) * dim;
            kb[set][it] = *reinterpret_cast<const f32x4*>(L.K + o + loff);
            vb[set][it] = *reinterpret_cast<const f32x4*>(L.V + o + loff);
        }
    };
    // this wave's first block: issued before anything else, nothing below depends on it
    size_t base = 0;
    if (b < nblocks) {
        base = block_base(b);
        issue(base, 0);
    }

    for (int i = tid; i < HD; i += NW * 64) {
        qs[i] = qkv[h * HD + i];
        ks[i] = qkv[L.offK + h * HD + i];
        vn[i] = qkv[L.offV + h * HD + i];
    }
    __syncthreads();
    if (a.qkNorm && wave < 2) { // wave 0: q, wave 1: k
        float* v = wave == 0 ? qs : ks;
        const float* g = (wave == 0 ? L.gq : L.gk) + h * HD;
        float s = 0.f;
        for (int i = lane; i < HD; i += 64) s = fmaf(v[i], v[i], s);
        s = wave_sum(s);
        const float r = sqrtf(s / (float)HD + 1e-8f);
        for (int i = lane; i < HD; i += 64) v[i] = g[i] * (v[i] / r);
    }
    __syncthreads();
    if (wave < 2 && lane < HD / 2) { // RoPE on adjacent pairs (inference.cu:127-133)
        float* v = wave == 0 ? qs : ks;
        const float c = a.rope[(size_t)p * HD + 2 * lane];
        const float s = a.rope[(size_t)p * HD + 2 * lane + 1];
        const float f = v[2 * lane], g = v[2 * lane + 1];
        v[2 * lane] = c * f - s * g;
        v[2 * lane + 1] = s * f + c * g;
    }
    __syncthreads();

    const f32x4 q4 = *reinterpret_cast<const f32x4*>(qs + c4);
    const float scale = sqrtf((float)HD);
    float m_run = -1.0e30f, l_run = 0.f; // of this lane's row group
    f32x4 acc = (f32x4)(0.f);             // output dims c4 .. c4 + 3, keys of this lane's row group

    // TAIL: the block holds the newest position or rows beyond it (row p comes from this step, later rows count as absent)
    auto block = [&](int j, int set, auto tailTag) { // keys j .. j + BR - 1 out of register set `set`
        constexpr bool TAIL = decltype(tailTag)::value;
        float s[BLD];
#pragma unroll
        for (int it = 0; it < BLD; it++) {
            f32x4 k = kb[set][it];
            if (TAIL) {
                const int r = j + it * RPI + lrow;
                const f32x4 alt = r == p ? *reinterpret_cast<const f32x4*>(ks + c4) : (f32x4)(0.f);
                k.x = r < p ? k.x : alt.x; k.y = r < p ? k.y : alt.y; k.z = r < p ? k.z : alt.z; k.w = r < p ? k.w : alt.w;
            }
            float d = k.x * q4.x;
            d = fmaf(k.y, q4.y, d); d = fmaf(k.z, q4.z, d); d = fmaf(k.w, q4.w, d);
            s[it] = d;
        }
#pragma unroll
        for (int it = 0; it < BLD; it++) {
            s[it] = attn_row_sum<LPR>(s[it]) / scale;
            if (TAIL) s[it] = j + it * RPI + lrow < T ? s[it] : -1.0e30f;
        }
        float mb = s[0];
#pragma unroll
        for (int it = 1; it < BLD; it++) mb = fmaxf(mb, s[it]);
        const float m_new = fmaxf(m_run, mb);
        const float corr = expf(m_run - m_new);
        float ls = 0.f;
#pragma unroll
        for (int it = 0; it < BLD; it++) {
            float e = expf(s[it] - m_new);
            if (TAIL) e = j + it * RPI + lrow < T ? e : 0.f;
            s[it] = e;
            ls += e;
        }
        l_run = l_run * corr + ls;
        m_run = m_new;
        acc *= corr;
#pragma unroll
        for (int it = 0; it < BLD; it++) {
            f32x4 v = vb[set][it];
            if (TAIL) {
                const int r = j + it * RPI + lrow;
                const f32x4 alt = r == p ? *reinterpret_cast<const f32x4*>(vn + c4) : (f32x4)(0.f);
                v.x = r < p ? v.x : alt.x; v.y = r < p ? v.y : alt.y; v.z = r < p ? v.z : alt.z; v.w = r < p ? v.w : alt.w;
            }
            acc.x = fmaf(s[it], v.x, acc.x); acc.y = fmaf(s[it], v.y, acc.y);
            acc.z = fmaf(s[it], v.z, acc.z); acc.w = fmaf(s[it], v.w, acc.w);
        }
    };

    // Two blocks per trip: the block in register set 0, then the one in set 1; while one is worked on the loads of
    // the wave's next block go out into the other set (no next block: the same loads are repeated and dropped, they
    // hit the cache -- a conditional issue would make the compiler wait for every load in front of each block).
    auto step = [&](int bb, int set, size_t& cur) -> bool { // returns whether the wave has a further block
        if (bb == newBlock) { // append this step's K/V row (only the owning wave writes it)
            const size_t o = cur + (size_t)(p - bb * BR) * dim;
            for (int i = lane; i < HD; i += 64) {
                L.K[o + i] = ks[i];
                L.V[o + i] = vn[i];
            }
        }
        const bool more = bb + bstep < nblocks;
        const size_t nxt = more ? block_base(bb + bstep) : cur;
        issue(nxt, set ^ 1);
        __builtin_amdgcn_sched_barrier(0); // one block ahead and no more
        if ((bb + 1) * BR > p) block(bb * BR, set, std::true_type());
        else block(bb * BR, set, std::false_type());
        __builtin_amdgcn_sched_barrier(0);
        cur = nxt;
        return more;
    };
    if (b < nblocks)
        for (;;) {
            if (!step(b, 0, base)) break;
            b += bstep;
            if (!step(b, 1, base)) break;
            b += bstep;
        }
    // merge the row groups of the wave (lanes LPR, 2 LPR, ... apart hold the same output dims)
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) {
        const float mo = __shfl_xor(m_run, o, MLH_WAVE), lo = __shfl_xor(l_run, o, MLH_WAVE);
        f32x4 ao;
        ao.x = __shfl_xor(acc.x, o, MLH_WAVE); ao.y = __shfl_xor(acc.y, o, MLH_WAVE);
        ao.z = __shfl_xor(acc.z, o, MLH_WAVE); ao.w = __shfl_xor(acc.w, o, MLH_WAVE);
        const float mm = fmaxf(m_run, mo);
        const float ca = expf(m_run - mm), cb = expf(mo - mm);
        l_run = l_run * ca + lo * cb;
        acc = acc * ca + ao * cb;
        m_run = mm;
    }

    // ---- combine the NW waves of this workgroup, write one partial ----
    float* cw = comb + wave * (HD + 2);
    if (lane < LPR) *reinterpret_cast<f32x4*>(cw + c4) = acc;
    if (lane == 0) { cw[HD] = m_run; cw[HD + 1] = l_run; }
    __syncthreads();
    float* out = a.part + (((size_t)slot * a.nsplit + sp) * a.heads + h) * (HD + 2);
    float M = -1.0e30f;
#pragma unroll
    for (int w = 0; w < NW; w++) M = fmaxf(M, comb[w * (HD + 2) + HD]);
    if (a.mixRows && a.nsplit == 1) {
        // batched step, one workgroup per (head, sequence): the finished mixing output (inference.cu:549-573), gated
        // (inference.cu:241-250), goes straight into the output-projection GEMM's input row; the workgroup of head 0
        // appends the PLE columns e = silu(gate) * P[tok]
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) l += expf(comb[w * (HD + 2) + HD] - M) * comb[w * (HD + 2) + HD + 1];
        const size_t row = (size_t)slot * a.mixRowsLd;
        auto put_row = [&](size_t col, float v) {
            if (a.mixRowsHalf) ((_Float16*)a.mixRows)[row + col] = (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f); // saturating
            else ((float*)a.mixRows)[row + col] = v;
        };
        for (int i = tid; i < HD; i += NW * 64) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) s += expf(comb[w * (HD + 2) + HD] - M) * comb[w * (HD + 2) + i];
            float v = s / l;
            if (a.gating) v = v * sigmoidf_ref(qkv[L.offG + h * HD + i]);
            put_row((size_t)h * HD + i, v);
        }
        if (h == 0)
            for (int j = tid; j < a.ple; j += NW * 64) {
                const size_t e = (size_t)a.tok[slot] * a.ple + j;
                const float pv = a.wbytes == 2 ? __uint_as_float(((uint32_t)((const uint16_t*)L.pleTable)[e]) << 16) : ((const float*)L.pleTable)[e];
                put_row((size_t)a.heads * HD + j, siluf_ref(qkv[L.offPle + j]) * pv);
            }
        return;
    }
    for (int i = tid; i < HD; i += NW * 64) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) s += expf(comb[w * (HD + 2) + HD] - M) * comb[w * (HD + 2) + i];
        out[i] = s;
    }
    if (tid == 0) {
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) l += expf(comb[w * (HD + 2) + HD] - M) * comb[w * (HD + 2) + HD + 1];
        out[HD] = M;
        out[HD + 1] = l;
    }
}

// ----------------------------------------------------------------------------
// gated-delta-net state update, one head's state per RS workgroups (rows of the state are independent):
//   q,k L2-normalised; alpha = exp(-softplus(za + ba)); beta = sigmoid(zb + bb)
//   u = S k ; S <- alpha (S - beta u k^T) + beta v k^T ; o = S q
// S is [DV, DK] row-major, held in registers for the step; workgroup z of a head takes rows [z DV/RS, (z+1) DV/RS).
// The normalised q and k are formed once per workgroup in LDS.
// ----------------------------------------------------------------------------
template <int DK, int DV, int RS>
__global__ void __launch_bounds__(WG) k_gdn(StepArgs a, LayerDev L) {
    constexpr int TPR = WG * RS / DV; // threads per state row
    constexpr int CPT = DK / TPR;     // columns per thread
    static_assert(TPR >= 1 && TPR <= 64 && (TPR & (TPR - 1)) == 0 && CPT % 4 == 0 && DK % 64 == 0, "unsupported GDN shape");
    __shared__ float qn[DK], kn[DK];
    const int h = blockIdx.x, slot = blockIdx.y, tid = threadIdx.x;
    const int seq = a.sidx[slot];
    const float* qkv = a.qkv + (size_t)slot * a.qkvStride;
    const int r = (int)blockIdx.z * (DV / RS) + tid / TPR, cg = tid % TPR, c0 = cg * CPT;
    // the state row's loads go out first: nothing below depends on them until the products
    float* Srow = L.S + (((size_t)seq * a.gdnHeads + h) * DV + r) * DK + c0;
    float S[CPT];
#pragma unroll
    for (int c = 0; c < CPT; c += 4) {
        float4 t = *reinterpret_cast<const float4*>(Srow + c);
        S[c] = t.x; S[c + 1] = t.y; S[c + 2] = t.z; S[c + 3] = t.w;
    }
    const float vr = qkv[L.offV + h * DV + r];
    float qv[DK / 64], kv[DK / 64];
    if (tid < 64) { // wave 0: the two norms
        float sq = 0.f, sk = 0.f;
#pragma unroll
        for (int i = 0; i < DK / 64; i++) {
            qv[i] = qkv[h * DK + tid + 64 * i];
            kv[i] = qkv[L.offK + h * DK + tid + 64 * i];
            sq = fmaf(qv[i], qv[i], sq);
            sk = fmaf(kv[i], kv[i], sk);
        }
        sq = wave_sum(sq);
        sk = wave_sum(sk);
        const float rq = sqrtf(sq + 1e-6f), rk = sqrtf(sk + 1e-6f);
#pragma unroll
        for (int i = 0; i < DK / 64; i++) {
            qn[tid + 64 * i] = qv[i] / rq;
            kn[tid + 64 * i] = kv[i] / rk;
        }
    }
    const float za = qkv[L.offGa + h] + L.gdnBa[h];
    const float zb = qkv[L.offGb + h] + L.gdnBb[h];
    const float sp = fmaxf(za, 0.f) + log1pf(expf(-fabsf(za)));
    const float alpha = expf(-sp);
    const float beta = sigmoidf_ref(zb);
    __syncthreads();

    float u = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; c++) u = fmaf(S[c], kn[c0 + c], u);
#pragma unroll
    for (int o = TPR / 2; o > 0; o >>= 1) u += __shfl_xor(u, o, MLH_WAVE);
    float oacc = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; c++) {
        const float k1 = kn[c0 + c];
        S[c] = alpha * (S[c] - beta * u * k1) + beta * vr * k1;
        oacc = fmaf(S[c], qn[c0 + c], oacc);
    }
#pragma unroll
    for (int o = TPR / 2; o > 0; o >>= 1) oacc += __shfl_xor(oacc, o, MLH_WAVE);
#pragma unroll
    for (int c = 0; c < CPT; c += 4)
        *reinterpret_cast<float4*>(Srow + c) = make_float4(S[c], S[c + 1], S[c + 2], S[c + 3]);
    if (!a.mixRows) {
        if (cg == 0) a.mix[(size_t)slot * (a.gdnHeads * DV) + h * DV + r] = oacc;
        return;
    }
    // batched step: the read-out is a row segment of the output-projection GEMM's input; the workgroup of head 0 also
    // appends the PLE columns e = silu(gate) * P[tok] behind the gdnHeads * DV read-out columns
    const size_t row = (size_t)slot * a.mixRowsLd;
    auto put_row = [&](size_t col, float v) {
        if (a.mixRowsHalf) ((_Float16*)a.mixRows)[row + col] = (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f); // saturating
        else ((float*)a.mixRows)[row + col] = v;
    };
    if (cg == 0) put_row((size_t)h * DV + r, oacc);
    if (h == 0 && blockIdx.z == 0)
        for (int j = tid; j < a.ple; j += WG) {
            const size_t e = (size_t)a.tok[slot] * a.ple + j;
            const float p = a.wbytes == 2 ? __uint_as_float(((uint32_t)((const uint16_t*)L.pleTable)[e]) << 16) : ((const float*)L.pleTable)[e];
            put_row((size_t)a.gdnHeads * DV + j, siluf_ref(qkv[L.offPle + j]) * p);
        }
}

// ----------------------------------------------------------------------------
// output projection: builds the mixing output in LDS (attention: combine the
// split partials, apply the sigmoid query gate, inference.cu:241-250; GDN: copy),
// then h1 = Wo . a + x (+ Wpu . (silu(ple gate) * P[tok]))   (inference.cu:582-610)
// ----------------------------------------------------------------------------
template <typename WT, int NB>
__global__ void __launch_bounds__(WG) k_oproj(StepArgs a, LayerDev L, int rowsPerWg) {
    extern __shared__ float lds[];
    const int ad = L.ad, pl = a.ple;
    float* as = lds;             // [NB][ad]
    float* es = lds + NB * ad;   // [NB][pl]
    const int slot0 = blockIdx.y * NB, tid = threadIdx.x;
    Prefetched<WT> pf;
    prefetch_rows<WT>(pf, (const WT*)L.Wo, ad, blockIdx.x * rowsPerWg + (tid >> 6) * RROWS, a.dim, ad);
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int slot = slot0 + b;
        const bool valid = slot < a.nseq;
        const float* qkv = a.qkv + (size_t)(valid ? slot : 0) * a.qkvStride;
        if (L.kind == MLH_KIND_ATTENTION) {
            const int hd = a.hd;
            for (int i = tid; i < ad; i += WG) {
                float v = 0.f;
                if (valid) {
                    const int h = i / hd, e = i - h * hd;
                    const float* pp = a.part + (((size_t)slot * a.nsplit) * a.heads + h) * (hd + 2);
                    const size_t sstride = (size_t)a.heads * (hd + 2);
                    float M = -1.0e30f;
                    for (int s = 0; s < a.nsplit; s++) M = fmaxf(M, pp[s * sstride + hd]);
                    float num = 0.f, den = 0.f;
                    for (int s = 0; s < a.nsplit; s++) {
                        const float w = expf(pp[s * sstride + hd] - M);
                        num = fmaf(w, pp[s * sstride + e], num);
                        den = fmaf(w, pp[s * sstride + hd + 1], den);
                    }
                    v = num / den;
                    if (a.gating) v = v * sigmoidf_ref(qkv[L.offG + i]);
                }
                as[b * ad + i] = v;
            }
        } else {
            for (int i = tid; i < ad; i += WG) as[b * ad + i] = valid ? a.mix[(size_t)slot * ad + i] : 0.f;
        }
        if (pl > 0) {
            for (int j = tid; j < pl; j += WG) {
                float v = 0.f;
                if (valid) {
                    const int t = a.tok[slot];
                    v = siluf_ref(qkv[L.offPle + j]) * WVec<WT>::one((const WT*)L.pleTable + (size_t)t * pl + j);
                }
                es[b * pl + j] = v;
            }
        }
    }
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63;
    const int rowBase = blockIdx.x * rowsPerWg;
    for (int r0 = wave * RROWS; r0 < rowsPerWg; r0 += WAVES * RROWS) {
        const int row0 = rowBase + r0;
        if (row0 >= a.dim) break;
        float acc[RROWS][NB] = {};
        if (r0 == wave * RROWS) rows_dot_pf<WT, NB>(pf, (const WT*)L.Wo, ad, row0, a.dim, ad, as, ad, acc);
        else rows_dot<WT, NB>((const WT*)L.Wo, ad, row0, a.dim, ad, as, ad, acc);
        if (pl > 0) rows_dot<WT, NB>((const WT*)L.pleUp, pl, row0, a.dim, pl, es, pl, acc);
#pragma unroll
        for (int r = 0; r < RROWS; r++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float v = wave_sum(acc[r][b]);
                if (lane == 0 && row0 + r < a.dim && slot0 + b < a.nseq) {
                    const size_t o = (size_t)(slot0 + b) * a.dim + row0 + r;
                    a.h1[o] = v + a.x[o];
                }
            }
    }
}

// ----------------------------------------------------------------------------
// FFN first half: hn = RMSNorm(h1, g2); u = silu(W1A . hn) * (W1B . hn)
// (inference.cu:612-672).  W13 interleaves gate and up rows so that one wave
// produces both values of an output element.
// ----------------------------------------------------------------------------
template <typename WT, int NB>
__global__ void __launch_bounds__(WG) k_ffn13(StepArgs a, LayerDev L, int pairsPerWg) {
    extern __shared__ float lds[];
    float* xs = lds;
    float* red = lds + NB * a.dim;
    const int slot0 = blockIdx.y * NB;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pairBase = blockIdx.x * pairsPerWg;
    Prefetched<WT> pf;
    prefetch_rows<WT>(pf, (const WT*)L.W13, a.dim, 2 * (pairBase + wave), 2 * a.ffn, a.dim);
    rmsnorm_to_lds<NB>(a.h1, a.dim, slot0, a.nseq, L.g2, a.dim, xs, a.dim, red);
    static_assert(RROWS == 2, "one wave handles one gate/up pair per pass");
    for (int p0 = wave; p0 < pairsPerWg; p0 += WAVES) {
        const int pr = pairBase + p0;
        if (pr >= a.ffn) break;
        float acc[RROWS][NB] = {};
        if (p0 == wave) rows_dot_pf<WT, NB>(pf, (const WT*)L.W13, a.dim, 2 * pr, 2 * a.ffn, a.dim, xs, a.dim, acc);
        else rows_dot<WT, NB>((const WT*)L.W13, a.dim, 2 * pr, 2 * a.ffn, a.dim, xs, a.dim, acc);
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float g = wave_sum(acc[0][b]);
            const float up = wave_sum(acc[1][b]);
            if (lane == 0 && slot0 + b < a.nseq) a.u[(size_t)(slot0 + b) * a.ffn + pr] = siluf_ref(g) * up;
        }
    }
}

// ----------------------------------------------------------------------------
// FFN second half: x_next = W2 . u + h1 (inference.cu:675-699)
// ----------------------------------------------------------------------------
template <typename WT, int NB>
__global__ void __launch_bounds__(WG) k_down(StepArgs a, LayerDev L, int rowsPerWg) {
    extern __shared__ float lds[];
    float* us = lds;
    const int slot0 = blockIdx.y * NB, tid = threadIdx.x;
    Prefetched<WT> pf;
    prefetch_rows<WT>(pf, (const WT*)L.W2, a.ffn, blockIdx.x * rowsPerWg + (tid >> 6) * RROWS, a.dim, a.ffn);
#pragma unroll
    for (int b = 0; b < NB; b++)
        for (int i = tid; i < a.ffn; i += WG)
            us[b * a.ffn + i] = (slot0 + b < a.nseq) ? a.u[(size_t)(slot0 + b) * a.ffn + i] : 0.f;
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63;
    const int rowBase = blockIdx.x * rowsPerWg;
    for (int r0 = wave * RROWS; r0 < rowsPerWg; r0 += WAVES * RROWS) {
        const int row0 = rowBase + r0;
        if (row0 >= a.dim) break;
        float acc[RROWS][NB] = {};
        if (r0 == wave * RROWS) rows_dot_pf<WT, NB>(pf, (const WT*)L.W2, a.ffn, row0, a.dim, a.ffn, us, a.ffn, acc);
        else rows_dot<WT, NB>((const WT*)L.W2, a.ffn, row0, a.dim, a.ffn, us, a.ffn, acc);
#pragma unroll
        for (int r = 0; r < RROWS; r++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float v = wave_sum(acc[r][b]);
                if (lane == 0 && row0 + r < a.dim && slot0 + b < a.nseq) {
                    const size_t o = (size_t)(slot0 + b) * a.dim + row0 + r;
                    a.x[o] = v + a.h1[o];
                }
            }
    }
}

// ----------------------------------------------------------------------------
// LM head: xf = RMSNorm(x, gF) (inference.cu:705-715); logits = E . xf (tied
// embedding, inference.cu:723-743); per-workgroup (max, lowest index) for the
// greedy pick that the reference does with a host qsort
// (inference_orchestrator.cu:77-84,112).
// ----------------------------------------------------------------------------
template <typename WT, int NB>
__global__ void __launch_bounds__(WG) k_lmhead(StepArgs a, int rowsPerWg) {
    extern __shared__ float lds[];
    float* xs = lds;
    float* red = lds + NB * a.dim;           // [WAVES]
    float* bv = red + WAVES;                 // [WAVES][NB]
    int* bi = (int*)(bv + WAVES * NB);       // [WAVES][NB]
    const int slot0 = blockIdx.y * NB;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int rowBase = blockIdx.x * rowsPerWg;
    Prefetched<WT> pf;
    prefetch_rows<WT>(pf, (const WT*)a.E, a.dim, rowBase + wave * RROWS, a.vocab, a.dim);
    rmsnorm_to_lds<NB>(a.x, a.dim, slot0, a.nseq, a.gF, a.dim, xs, a.dim, red);
    float best[NB];
    int bidx[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) { best[b] = -3.0e38f; bidx[b] = 0x7fffffff; }
    for (int r0 = wave * RROWS; r0 < rowsPerWg; r0 += WAVES * RROWS) {
        const int row0 = rowBase + r0;
        if (row0 >= a.vocab) break;
        float acc[RROWS][NB] = {};
        if (r0 == wave * RROWS) rows_dot_pf<WT, NB>(pf, (const WT*)a.E, a.dim, row0, a.vocab, a.dim, xs, a.dim, acc);
        else rows_dot<WT, NB>((const WT*)a.E, a.dim, row0, a.vocab, a.dim, xs, a.dim, acc);
#pragma unroll
        for (int r = 0; r < RROWS; r++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
                float v = wave_sum(acc[r][b]);
                if (row0 + r < a.vocab && slot0 + b < a.nseq) {
                    if (lane == 0) a.logits[(size_t)a.sidx[slot0 + b] * a.vocab + row0 + r] = v;
                    if (v > best[b]) { best[b] = v; bidx[b] = row0 + r; } // rows ascend: ties keep the lower index
                }
            }
    }
    if (lane == 0)
#pragma unroll
        for (int b = 0; b < NB; b++) { bv[wave * NB + b] = best[b]; bi[wave * NB + b] = bidx[b]; }
    __syncthreads();
    if (threadIdx.x < NB && slot0 + threadIdx.x < a.nseq) {
        const int b = threadIdx.x;
        float v = bv[b];
        int i = bi[b];
        for (int w = 1; w < WAVES; w++) {
            const float v2 = bv[w * NB + b];
            const int i2 = bi[w * NB + b];
            if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
        }
        a.amaxVal[(size_t)(slot0 + b) * a.amaxParts + blockIdx.x] = v;
        a.amaxIdx[(size_t)(slot0 + b) * a.amaxParts + blockIdx.x] = i;
    }
}

// Final argmax reduce + bookkeeping: next token -> tokOut[slot] and the id log,
// pos[seq]++ (the append of inference_orchestrator.cu:149-151, kept on the device).
__global__ void __launch_bounds__(WG) k_finish(StepArgs a, int* tokOut, int nparts) {
    __shared__ float sv[WG];
    __shared__ int si[WG];
    __shared__ double sd[WG + 1];
    const int tid = threadIdx.x;
    const int step = *a.stepCounter;
    for (int slot = 0; slot < a.nseq; slot++) {
        if (a.temperature > 0.f) { // draw instead of argmax: the row of logits is complete (k_lmhead wrote it)
            const int seq = a.sidx[slot];
            const int nxt = mlh_sample_row<WG>(a.logits + (size_t)seq * a.vocab, a.vocab, a.temperature,
                                               mlh_sample_uniform(a.sampleSeed, seq, a.pos[seq] + 1), sd, si);
            __syncthreads();
            if (tid == 0) {
                tokOut[slot] = nxt;
                a.nextTok[seq] = nxt;
                if (step < a.outCapacity) a.outIds[(size_t)step * a.nseq + slot] = nxt;
                a.pos[seq] += 1;
            }
            __syncthreads();
            continue;
        }
        float v = -3.0e38f;
        int idx = 0x7fffffff;
        for (int i = tid; i < nparts; i += WG) {
            const float v2 = a.amaxVal[(size_t)slot * a.amaxParts + i];
            const int i2 = a.amaxIdx[(size_t)slot * a.amaxParts + i];
            if (v2 > v || (v2 == v && i2 < idx)) { v = v2; idx = i2; }
        }
        sv[tid] = v;
        si[tid] = idx;
        __syncthreads();
        for (int s = WG / 2; s > 0; s >>= 1) {
            if (tid < s) {
                const float v2 = sv[tid + s];
                const int i2 = si[tid + s];
                if (v2 > sv[tid] || (v2 == sv[tid] && i2 < si[tid])) { sv[tid] = v2; si[tid] = i2; }
            }
            __syncthreads();
        }
        if (tid == 0) {
            int nxt = si[0];
            if (nxt < 0 || nxt >= a.vocab) nxt = 0; // only reachable with non-finite logits
            tokOut[slot] = nxt;
            a.nextTok[a.sidx[slot]] = nxt;
            if (step < a.outCapacity) a.outIds[(size_t)step * a.nseq + slot] = nxt;
            a.pos[a.sidx[slot]] += 1;
        }
        __syncthreads();
    }
    if (tid == 0) *a.stepCounter = step + 1;
}

// Prefill bookkeeping when the LM head is skipped: pos[seq]++ only.
__global__ void k_advance(StepArgs a) {
    const int slot = blockIdx.x * blockDim.x + threadIdx.x;
    if (slot < a.nseq) a.pos[a.sidx[slot]] += 1;
}

// Softmax over the vocabulary for one sequence (inference.cu:293-362).
__global__ void __launch_bounds__(WG) k_probs(const float* logits, float* probs, int n) {
    __shared__ float red[WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float m = -1.0e20f;
    for (int i = tid; i < n; i += WG) m = fmaxf(m, logits[i]);
    m = wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = red[0];
    for (int w = 1; w < WAVES; w++) m = fmaxf(m, red[w]);
    __syncthreads();
    float s = 0.f;
    for (int i = tid; i < n; i += WG) {
        const float e = expf(logits[i] - m);
        probs[i] = e;
        s += e;
    }
    s = wave_sum(s);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    s = 0.f;
    for (int w = 0; w < WAVES; w++) s += red[w];
    for (int i = tid; i < n; i += WG) probs[i] = probs[i] / s;
}

__global__ void k_copy(const float4* __restrict__ src, float4* __restrict__ dst, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

// ----------------------------------------------------------------------------
// host-side launch logic
// ----------------------------------------------------------------------------
static int pick_nb(int nseq, int cols) {
    int nb = nseq >= 8 ? 8 : nseq >= 4 ? 4 : nseq >= 2 ? 2 : 1;
    while (nb > 1 && (size_t)nb * cols * 4 > 48 * 1024) nb >>= 1;
    return nb;
}
static int ceil_div(int a, int b) { return (a + b - 1) / b; }

void mlh_fill_args(mlh_ctx* c, StepArgs& a, int nseq, const int* tokPtr) {
    const mlh_hparams& hp = c->hp;
    a.dim = hp.dim; a.heads = hp.attnHeads; a.hd = hp.headDim; a.ffn = hp.ffnDim;
    a.vocab = hp.vocabSize; a.maxL = hp.maxL; a.ple = hp.pleDim;
    a.gdnHeads = hp.gdnHeads; a.gdnDk = hp.gdnDk; a.gdnDv = hp.gdnDv;
    a.qkNorm = hp.qkRmsNorm; a.gating = hp.queryGating;
    a.nseq = nseq; a.sidx = c->d_sidx; a.tok = tokPtr; a.pos = c->d_pos;
    a.pageTable = c->d_pageTable; a.pagesPerSeq = c->pagesPerSeq; a.nsplit = c->nsplit;
    a.x = c->x; a.qkv = c->qkv; a.qkvStride = c->maxRowsA; a.part = c->part; a.mix = c->mix;
    a.mixRows = c->mixRows; a.mixRowsLd = c->mixRowsLd; a.mixRowsHalf = c->mixRowsHalf; a.wbytes = c->wbytes;
    a.temperature = c->temperature; a.sampleSeed = c->sampleSeed;
    a.h1 = c->h1; a.u = c->u; a.logits = c->logits; a.amaxVal = c->amaxVal; a.amaxIdx = c->amaxIdx;
    a.amaxParts = c->amaxParts; a.rope = c->rope; a.E = c->E; a.gF = c->gF;
    a.nextTok = c->d_next; a.outIds = c->d_outIds; a.stepCounter = c->d_stepCounter; a.outCapacity = c->outCapacity;
}

#define LMHEAD_ROWS_PER_WG 16
#define GEMV_ROWS_PER_WG 8

template <typename WT, int NB>
static void launch_gemv_kernel(mlh_ctx* c, int kernel, const StepArgs& a, const LayerDev& L) {
    hipStream_t st = c->stream;
    const int gy = ceil_div(a.nseq, NB);
    switch (kernel) {
        case MLH_K_QKV: {
            size_t lds = ((size_t)NB * a.dim + WAVES) * 4;
            hipLaunchKernelGGL((k_phaseA<WT, NB>), dim3(ceil_div(L.rowsA, GEMV_ROWS_PER_WG), gy), dim3(WG),
                               lds, st, a, L, GEMV_ROWS_PER_WG);
            break;
        }
        case MLH_K_OPROJ: {
            size_t lds = ((size_t)NB * (L.ad + a.ple)) * 4;
            hipLaunchKernelGGL((k_oproj<WT, NB>), dim3(ceil_div(a.dim, GEMV_ROWS_PER_WG), gy), dim3(WG), lds,
                               st, a, L, GEMV_ROWS_PER_WG);
            break;
        }
        case MLH_K_FFN_GATEUP: {
            size_t lds = ((size_t)NB * a.dim + WAVES) * 4;
            hipLaunchKernelGGL((k_ffn13<WT, NB>), dim3(ceil_div(a.ffn, GEMV_ROWS_PER_WG / 2), gy), dim3(WG),
                               lds, st, a, L, GEMV_ROWS_PER_WG / 2);
            break;
        }
        case MLH_K_FFN_DOWN: {
            size_t lds = ((size_t)NB * a.ffn) * 4;
            hipLaunchKernelGGL((k_down<WT, NB>), dim3(ceil_div(a.dim, GEMV_ROWS_PER_WG), gy), dim3(WG), lds, st,
                               a, L, GEMV_ROWS_PER_WG);
            break;
        }
        case MLH_K_LMHEAD: {
            size_t lds = ((size_t)NB * a.dim + WAVES + 2 * WAVES * NB) * 4;
            hipLaunchKernelGGL((k_lmhead<WT, NB>), dim3(ceil_div(a.vocab, LMHEAD_ROWS_PER_WG), gy), dim3(WG),
                               lds, st, a, LMHEAD_ROWS_PER_WG);
            break;
        }
        default: break;
    }
}

template <typename WT>
static void launch_gemv_nb(mlh_ctx* c, int kernel, const StepArgs& a, const LayerDev& L, int cols) {
    switch (pick_nb(a.nseq, cols)) {
        case 8: launch_gemv_kernel<WT, 8>(c, kernel, a, L); break;
        case 4: launch_gemv_kernel<WT, 4>(c, kernel, a, L); break;
        case 2: launch_gemv_kernel<WT, 2>(c, kernel, a, L); break;
        default: launch_gemv_kernel<WT, 1>(c, kernel, a, L); break;
    }
}

static void launch_gemv(mlh_ctx* c, int kernel, const StepArgs& a, const LayerDev& L) {
    int cols = a.dim;
    if (kernel == MLH_K_OPROJ) cols = L.ad + a.ple;
    if (kernel == MLH_K_FFN_DOWN) cols = a.ffn;
    if (c->hp.weightDtype == MLH_DTYPE_BF16) launch_gemv_nb<bf16_t>(c, kernel, a, L, cols);
    else launch_gemv_nb<float>(c, kernel, a, L, cols);
}

static size_t attn_lds_bytes(int hd) {
    return hd == 64 ? (3 * 64 + AttnCfg<64>::NW * 66) * 4 : (3 * 128 + AttnCfg<128>::NW * 130) * 4;
}

// Nothing to set up: no decode kernel needs more LDS than a launch may use without opting in.
int mlh_init_kernels(mlh_ctx*) { return 0; }

static int launch_mix(mlh_ctx* c, const StepArgs& a, const LayerDev& L) {
    hipStream_t st = c->stream;
    if (L.kind == MLH_KIND_ATTENTION) {
        if (a.hd == 64) {
            size_t lds = attn_lds_bytes(64);
            hipLaunchKernelGGL((k_attn<64>), dim3(a.heads, a.nseq, a.nsplit), dim3(256), lds, st, a, L);
        } else if (a.hd == 128) {
            size_t lds = attn_lds_bytes(128);
            hipLaunchKernelGGL((k_attn<128>), dim3(a.heads, a.nseq, a.nsplit), dim3(128), lds, st, a, L);
        } else {
            c->err = "attention kernel supports headDim 64 or 128";
            return -1;
        }
    } else {
        // few (head, sequence) pairs: a head's rows are split over four workgroups so that every compute unit has work
        const bool split = a.gdnHeads * a.nseq <= 256;
        if (a.gdnDk == 64 && a.gdnDv == 64) {
            if (split) hipLaunchKernelGGL((k_gdn<64, 64, 4>), dim3(a.gdnHeads, a.nseq, 4), dim3(WG), 0, st, a, L);
            else hipLaunchKernelGGL((k_gdn<64, 64, 1>), dim3(a.gdnHeads, a.nseq), dim3(WG), 0, st, a, L);
        } else if (a.gdnDk == 128 && a.gdnDv == 128) {
            if (split) hipLaunchKernelGGL((k_gdn<128, 128, 4>), dim3(a.gdnHeads, a.nseq, 4), dim3(WG), 0, st, a, L);
            else hipLaunchKernelGGL((k_gdn<128, 128, 1>), dim3(a.gdnHeads, a.nseq), dim3(WG), 0, st, a, L);
        }
        else {
            c->err = "GDN kernel supports dk = dv = 64 or 128";
            return -1;
        }
    }
    return 0;
}

// Enqueues one decode step on the context's stream (no synchronisation).
int mlh_launch_step(mlh_ctx* c, int nseq, const int* tokPtr, bool lmHead) {
    if (lmHead && !c->profEvents && mlh_batch_step_applicable(c, nseq)) return mlh_launch_batch_step(c, nseq, tokPtr);
    StepArgs a;
    mlh_fill_args(c, a, nseq, tokPtr);
    hipStream_t st = c->stream;
    // measurement hook: an event after every launch, tagged with the kernel id
    auto mark = [&](int id) {
        if (!c->profEvents) return;
        hipEvent_t ev;
        if (hipEventCreate(&ev) != hipSuccess) return;
        (void)hipEventRecord(ev, st);
        c->profEvents->push_back(ev);
        c->profIds->push_back(id);
    };
    if (c->hp.weightDtype == MLH_DTYPE_BF16)
        hipLaunchKernelGGL((k_embed<bf16_t>), dim3(ceil_div(a.dim, WG), nseq), dim3(WG), 0, st, a);
    else
        hipLaunchKernelGGL((k_embed<float>), dim3(ceil_div(a.dim, WG), nseq), dim3(WG), 0, st, a);
    mark(MLH_K_EMBED);
    for (int t = c->hp.transformers - 1; t >= 0; t--) { // file block 0 is the top (inference.cu:384-385)
        const LayerDev& L = c->layers[t];
        launch_gemv(c, MLH_K_QKV, a, L);
        mark(MLH_K_QKV);
        if (launch_mix(c, a, L) != 0) return -1;
        mark(L.kind == MLH_KIND_ATTENTION ? MLH_K_ATTN : MLH_K_GDN);
        launch_gemv(c, MLH_K_OPROJ, a, L);
        mark(MLH_K_OPROJ);
        launch_gemv(c, MLH_K_FFN_GATEUP, a, L);
        mark(MLH_K_FFN_GATEUP);
        launch_gemv(c, MLH_K_FFN_DOWN, a, L);
        mark(MLH_K_FFN_DOWN);
    }
    if (lmHead) {
        launch_gemv(c, MLH_K_LMHEAD, a, c->layers[0]);
        mark(MLH_K_LMHEAD);
        hipLaunchKernelGGL(k_finish, dim3(1), dim3(WG), 0, st, a, c->d_tok,
                           ceil_div(a.vocab, LMHEAD_ROWS_PER_WG));
        mark(MLH_K_FINISH);
    } else {
        hipLaunchKernelGGL(k_advance, dim3(ceil_div(nseq, 64)), dim3(64), 0, st, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        c->err = std::string("kernel launch: ") + hipGetErrorString(e);
        return -2;
    }
    return 0;
}

// Launches a single kernel of the step (measurement support).  The attention and
// GDN kernels mutate the cache/state in place, which is harmless for timing.
int mlh_launch_one(mlh_ctx* c, int kernel, int layer, int nseq) {
    StepArgs a;
    mlh_fill_args(c, a, nseq, c->d_tok);
    const LayerDev& L = c->layers[layer];
    switch (kernel) {
        case MLH_K_QKV: case MLH_K_OPROJ: case MLH_K_FFN_GATEUP: case MLH_K_FFN_DOWN: case MLH_K_LMHEAD:
            launch_gemv(c, kernel, a, L);
            break;
        case MLH_K_ATTN:
            if (L.kind != MLH_KIND_ATTENTION) { c->err = "layer is not an attention layer"; return -1; }
            if (launch_mix(c, a, L) != 0) return -1;
            break;
        case MLH_K_GDN:
            if (L.kind != MLH_KIND_GDN) { c->err = "layer is not a GDN layer"; return -1; }
            if (launch_mix(c, a, L) != 0) return -1;
            break;
        case MLH_K_COPY:
            return mlh_launch_copy(c);
        default:
            c->err = "unknown kernel id";
            return -1;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { c->err = std::string("kernel launch: ") + hipGetErrorString(e); return -2; }
    return 0;
}

int mlh_launch_copy(mlh_ctx* c) {
    if (!c->copySrc) { // the calibration buffers exist only once the copy has been asked for
        int rc;
        if ((rc = mlh_dev_alloc_bytes(c, &c->copySrc, c->copyBytes)) || (rc = mlh_dev_alloc_bytes(c, &c->copyDst, c->copyBytes))) return rc;
        MLH_CHECK(c, hipMemsetAsync(c->copySrc, 0, c->copyBytes, c->stream));
    }
    hipLaunchKernelGGL(k_copy, dim3(2048), dim3(256), 0, c->stream, (const float4*)c->copySrc,
                       (float4*)c->copyDst, c->copyBytes / 16);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { c->err = std::string("kernel launch: ") + hipGetErrorString(e); return -2; }
    return 0;
}

int mlh_launch_probs(mlh_ctx* c, int seq) {
    hipLaunchKernelGGL(k_probs, dim3(1), dim3(WG), 0, c->stream,
                       c->logits + (size_t)seq * c->hp.vocabSize, c->probs, c->hp.vocabSize);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { c->err = std::string("kernel launch: ") + hipGetErrorString(e); return -2; }
    return 0;
}

// Algorithmic bytes one launch of `kernel` must move: the weight matrix once,
// plus (attention) the K/V rows of the current lengths, (GDN) the states read
// and written.  Activations, gains and partials are left out.
double mlh_kernel_bytes(mlh_ctx* c, int kernel, int layer, int nseq) {
    const mlh_hparams& hp = c->hp;
    const LayerDev& L = c->layers[layer];
    const double wb = c->wbytes;
    switch (kernel) {
        case MLH_K_QKV: return wb * L.rowsA * hp.dim;
        case MLH_K_OPROJ: return wb * ((double)hp.dim * L.ad + (double)hp.dim * hp.pleDim);
        case MLH_K_FFN_GATEUP: return wb * 2.0 * hp.ffnDim * hp.dim;
        case MLH_K_FFN_DOWN: return wb * (double)hp.dim * hp.ffnDim;
        case MLH_K_LMHEAD: return wb * (double)hp.vocabSize * hp.dim;
        case MLH_K_ATTN: {
            double b = 0;
            for (int s = 0; s < nseq; s++) b += 2.0 * 4.0 * hp.dim * (c->h_len[s] + 1) + 2.0 * 4.0 * hp.dim;
            return b;
        }
        case MLH_K_GDN: return 2.0 * 4.0 * nseq * hp.gdnHeads * hp.gdnDk * hp.gdnDv;
        case MLH_K_COPY: return 2.0 * c->copyBytes;
        default: return 0;
    }
}
