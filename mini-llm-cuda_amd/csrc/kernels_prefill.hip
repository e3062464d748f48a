// Prefill: many tokens of one or more sequences through the stack at once.
//
// Rows of the activation matrices are tokens (all segments concatenated); the projections are MFMA
// GEMMs (kernels_gemm.hip) against the same weight buffers the decode path streams; per layer
//
//   rmsnorm rows -> GEMM Wa -> attention: per-head QK-norm + RoPE + KV-page write, tiled causal attention
//                              GDN:       chunked recurrence, one head of one sequence per workgroup
//                -> (PLE rows) -> GEMM Wo (+ residual) (+ GEMM pleUp accumulate)
//                -> rmsnorm rows -> GEMM W13 with SiLU(gate)*up epilogue -> GEMM W2 (+ residual)
//
// and at the end the LM head runs for the last row of every segment only (the reference computes
// logits for all L columns, inference.cu:723-743, and uses the last one).  With bf16 weights the GEMM
// inputs (normed activations, mixing output, FFN activations) are rounded to bf16; accumulation, the
// residual stream, K/V and GDN states stay fp32.  This is what runInference(L) (inference.cu:376-751)
// does for L columns, minus the columns that are already in the cache.
#include <algorithm>

#include "mlh_internal.h"
#include "sample.h"

#define PWG 256
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct PfArgs {
    StepArgs a;        // model dimensions and shared pointers (rope, page table, E, gains ...)
    int n;             // rows (tokens) in this call
    int nseg;
    const int* ids;    // [n]
    const int* rowSeq; // [n] sequence of the row
    const int* rowPos; // [n] position of the row's token in its sequence
    const int* segStart;
    const int* segLen;
    const int* segSeq;
    const int* segPos0;
    const int* blkSeg; // attention query blocks: segment and first query of the block
    const int* blkQ0;
    float* X;          // [n, dim] residual stream
    void* Xn;          // [n, dim] GEMM input (weight dtype)
    float* QKV;        // [n, qkvLd]
    int qkvLd;
    void* Amix;        // [n, aLd] GEMM input of the output projection: mixing output, then (at column L.ad) the PLE row
    int aLd;
    float* H1;         // [n, dim]
    void* U;           // [n, ffn]
    uint16_t* Kh;      // [n, dim] IEEE-half copies of this call's K and V rows (after norm and RoPE), or null: what the MFMA
    uint16_t* Vh;      //          attention reads when every segment starts at position 0 (all of its keys are rows of the call)
};

__device__ __forceinline__ float pf_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float pf_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float pf_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); } // inference.cu:248
__device__ __forceinline__ float pf_silu(float v) { return v / (1.0f + expf(-v)); }       // inference.cu:270

// store a float as the GEMM input type (fp32; IEEE half for bf16 models, whose MFMA path runs in fp16; bf16)
template <typename AT> __device__ __forceinline__ void put(AT* p, float v);
template <> __device__ __forceinline__ void put<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void put<bf16_t>(bf16_t* p, float v) {
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) u |= 0x00400000u;
    else u += 0x7fffu + ((u >> 16) & 1u);
    *p = (bf16_t)(u >> 16);
}
template <> __device__ __forceinline__ void put<f16_t>(f16_t* p, float v) { // saturating: an overflow must not become inf
    const _Float16 h = (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f);
    p->bits = __builtin_bit_cast(uint16_t, h);
}
template <typename WT> __device__ __forceinline__ float getw(const WT* p);
template <> __device__ __forceinline__ float getw<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float getw<bf16_t>(const bf16_t* p) { return __uint_as_float(((uint32_t)*p) << 16); }

// inference.cu:9-22
template <typename WT>
__global__ void k_pf_embed(PfArgs P) {
    const int row = blockIdx.y, i = blockIdx.x * PWG + threadIdx.x;
    if (i >= P.a.dim) return;
    P.X[(size_t)row * P.a.dim + i] = getw<WT>((const WT*)P.a.E + (size_t)P.ids[row] * P.a.dim + i);
}

// inference.cu:24-50 + 83-95, one wave per row (d is a multiple of 8 on this path: 16-byte loads).  Rows of up to
// 4096 elements stay in registers between the sum of squares and the scaling (one pass over memory), and a lane's
// four results leave as one store.
template <typename AT> __device__ __forceinline__ void put4(AT* o, float a, float b, float c, float d);
template <> __device__ __forceinline__ void put4<float>(float* o, float a, float b, float c, float d) {
    f32x4 v; v.x = a; v.y = b; v.z = c; v.w = d;
    *reinterpret_cast<f32x4*>(o) = v;
}
template <> __device__ __forceinline__ void put4<bf16_t>(bf16_t* o, float a, float b, float c, float d) {
    put<bf16_t>(o, a); put<bf16_t>(o + 1, b); put<bf16_t>(o + 2, c); put<bf16_t>(o + 3, d);
}
template <> __device__ __forceinline__ void put4<f16_t>(f16_t* o, float a, float b, float c, float d) { // saturating like put<f16_t>
    auto h = [](float v) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f)); };
    uint2 w;
    w.x = h(a) | (h(b) << 16); w.y = h(c) | (h(d) << 16);
    *reinterpret_cast<uint2*>(o) = w;
}

template <typename AT>
__global__ void __launch_bounds__(PWG) k_pf_rmsnorm(const float* __restrict__ X, const float* __restrict__ gamma, AT* out, int n, int d) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= n) return;
    const float* x = X + (size_t)row * d;
    constexpr int KEEP = 16; // 16-byte pieces a lane keeps: rows of up to 64 * 4 * 16 = 4096 elements
    f32x4 keep[KEEP];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        const int i = lane * 4 + k * 256;
        keep[k] = i < d ? *reinterpret_cast<const f32x4*>(x + i) : (f32x4)(0.f);
        s = fmaf(keep[k].x, keep[k].x, s); s = fmaf(keep[k].y, keep[k].y, s); s = fmaf(keep[k].z, keep[k].z, s); s = fmaf(keep[k].w, keep[k].w, s);
    }
    for (int i = lane * 4 + KEEP * 256; i < d; i += 256) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(x + i);
        s = fmaf(v.x, v.x, s); s = fmaf(v.y, v.y, s); s = fmaf(v.z, v.z, s); s = fmaf(v.w, v.w, s);
    }
    s = pf_wave_sum(s);
    const float r = sqrtf(s / (float)d + 1e-8f);
#pragma unroll
    for (int k = 0; k < KEEP; k++) {
        const int i = lane * 4 + k * 256;
        if (i < d) {
            const f32x4 v = keep[k], g = *reinterpret_cast<const f32x4*>(gamma + i);
            put4<AT>(out + (size_t)row * d + i, g.x * (v.x / r), g.y * (v.y / r), g.z * (v.z / r), g.w * (v.w / r));
        }
    }
    for (int i = lane * 4 + KEEP * 256; i < d; i += 256) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(x + i), g = *reinterpret_cast<const f32x4*>(gamma + i);
        put4<AT>(out + (size_t)row * d + i, g.x * (v.x / r), g.y * (v.y / r), g.z * (v.z / r), g.w * (v.w / r));
    }
}

// Per (head, row): per-head RMSNorm of q and k (inference.cu:52-81, 97-111), RoPE on adjacent pairs at the
// row's position (inference.cu:113-134), q written back in place, k and v written to the KV pages.
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) { // two floats -> two IEEE halves (round to nearest even)
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
}

template <int HD>
__global__ void __launch_bounds__(64) k_pf_qk_rope_kv(PfArgs P, LayerDev L) {
    constexpr int EPL = HD / 64;
    const StepArgs& a = P.a;
    const int h = blockIdx.x, row = blockIdx.y, lane = threadIdx.x;
    const int seq = P.rowSeq[row], pos = P.rowPos[row];
    float* qkv = P.QKV + (size_t)row * P.qkvLd;
    float qv[EPL], kv[EPL], vv[EPL];
#pragma unroll
    for (int e = 0; e < EPL; e++) {
        const int i = lane * EPL + e;
        qv[e] = qkv[h * HD + i]; kv[e] = qkv[L.offK + h * HD + i]; vv[e] = qkv[L.offV + h * HD + i];
    }
    if (a.qkNorm) {
        float sq = 0.f, sk = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; e++) { sq = fmaf(qv[e], qv[e], sq); sk = fmaf(kv[e], kv[e], sk); }
        sq = pf_wave_sum(sq); sk = pf_wave_sum(sk);
        const float rq = sqrtf(sq / (float)HD + 1e-8f), rk = sqrtf(sk / (float)HD + 1e-8f);
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            const int i = lane * EPL + e;
            qv[e] = L.gq[h * HD + i] * (qv[e] / rq);
            kv[e] = L.gk[h * HD + i] * (kv[e] / rk);
        }
    }
    if (EPL == 1) {
        const float c = a.rope[(size_t)pos * HD + (lane & ~1)], s = a.rope[(size_t)pos * HD + (lane | 1)];
        const float qo = __shfl_xor(qv[0], 1, 64), ko = __shfl_xor(kv[0], 1, 64);
        if (lane & 1) { qv[0] = s * qo + c * qv[0]; kv[0] = s * ko + c * kv[0]; }
        else { qv[0] = c * qv[0] - s * qo; kv[0] = c * kv[0] - s * ko; }
    } else {
        const float c = a.rope[(size_t)pos * HD + 2 * lane], s = a.rope[(size_t)pos * HD + 2 * lane + 1];
        const float q0 = qv[0], q1 = qv[EPL - 1], k0 = kv[0], k1 = kv[EPL - 1];
        qv[0] = c * q0 - s * q1; qv[EPL - 1] = s * q0 + c * q1;
        kv[0] = c * k0 - s * k1; kv[EPL - 1] = s * k0 + c * k1;
    }
    const int page = a.pageTable[seq * a.pagesPerSeq + (pos >> 6)];
    const size_t o = ((size_t)page * MLH_KV_PAGE + (pos & 63)) * a.dim + h * HD;
#pragma unroll
    for (int e = 0; e < EPL; e++) {
        const int i = lane * EPL + e;
        qkv[h * HD + i] = qv[e];
        L.K[o + i] = kv[e];
        L.V[o + i] = vv[e];
    }
    if (P.Kh) { // the half copies, rounded exactly as the attention kernel rounds the fp32 rows on its way into LDS
        const size_t ho = (size_t)row * a.dim + h * HD + lane * EPL;
        if (EPL == 2) {
            *reinterpret_cast<uint32_t*>(P.Kh + ho) = pack_f16(kv[0], kv[1]);
            *reinterpret_cast<uint32_t*>(P.Vh + ho) = pack_f16(vv[0], vv[1]);
        } else {
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                P.Kh[ho + e] = __builtin_bit_cast(uint16_t, (_Float16)kv[e]);
                P.Vh[ho + e] = __builtin_bit_cast(uint16_t, (_Float16)vv[e]);
            }
        }
    }
}

// Tiled causal attention for 16 queries of one head: K and V of 64 positions at a time in LDS, online
// softmax per query (inference.cu:136-239, 511-573 for these columns), optional sigmoid gate (:241-250).
#define PF_QB 16
template <int HD, typename AT>
__global__ void __launch_bounds__(PWG) k_pf_attn(PfArgs P, LayerDev L) {
    constexpr int LDK = HD + 4, EPL = HD / 64, QPW = PF_QB / 4;
    extern __shared__ float lds[];
    float* Kt = lds;              // [64][LDK]
    float* Vt = Kt + 64 * LDK;    // [64][LDK]
    float* qs = Vt + 64 * LDK;    // [PF_QB][HD]
    const StepArgs& a = P.a;
    const int h = blockIdx.x, blk = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int seg = P.blkSeg[blk], q0 = P.blkQ0[blk];
    const int seq = P.segSeq[seg], pos0 = P.segPos0[seg], len = P.segLen[seg], row0 = P.segStart[seg] + q0;
    const int nq = min(PF_QB, len - q0);
    const int maxPos = pos0 + q0 + nq - 1;
    for (int i = tid; i < PF_QB * HD; i += PWG) {
        const int q = i / HD, e = i - q * HD;
        qs[i] = q < nq ? P.QKV[(size_t)(row0 + q) * P.qkvLd + h * HD + e] : 0.f;
    }
    float m[QPW], l[QPW], acc[QPW][EPL];
#pragma unroll
    for (int q = 0; q < QPW; q++) {
        m[q] = -1.0e30f; l[q] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; e++) acc[q][e] = 0.f;
    }
    const float scale = sqrtf((float)HD);
    const int ntiles = (maxPos >> 6) + 1;
    for (int t = 0; t < ntiles; t++) {
        const int j0 = t << 6;
        const int page = a.pageTable[seq * a.pagesPerSeq + t];
        const size_t base = ((size_t)page * MLH_KV_PAGE) * a.dim + h * HD;
        __syncthreads();
        for (int i = tid; i < 64 * (HD / 4); i += PWG) {
            const int r = i / (HD / 4), c4 = (i % (HD / 4)) * 4;
            f32x4 kk = (f32x4)(0.f), vv = (f32x4)(0.f);
            if (j0 + r <= maxPos) {
                kk = *reinterpret_cast<const f32x4*>(L.K + base + (size_t)r * a.dim + c4);
                vv = *reinterpret_cast<const f32x4*>(L.V + base + (size_t)r * a.dim + c4);
            }
            *reinterpret_cast<f32x4*>(Kt + r * LDK + c4) = kk;
            *reinterpret_cast<f32x4*>(Vt + r * LDK + c4) = vv;
        }
        __syncthreads();
#pragma unroll
        for (int qq = 0; qq < QPW; qq++) {
            const int q = wave * QPW + qq;
            const int qpos = pos0 + q0 + q;
            if (q >= nq || j0 > qpos) continue; // wave-uniform
            float s = 0.f;
            const float* kr = Kt + lane * LDK;
            const float* qr = qs + q * HD;
#pragma unroll
            for (int i = 0; i < HD; i += 4) {
                const f32x4 kk = *reinterpret_cast<const f32x4*>(kr + i);
                const f32x4 qv = *reinterpret_cast<const f32x4*>(qr + i);
                s = fmaf(kk.x, qv.x, s); s = fmaf(kk.y, qv.y, s); s = fmaf(kk.z, qv.z, s); s = fmaf(kk.w, qv.w, s);
            }
            const bool valid = j0 + lane <= qpos;
            s = valid ? s / scale : -1.0e30f;
            const float mn = fmaxf(m[qq], pf_wave_max(s));
            const float e = valid ? expf(s - mn) : 0.f;
            const float corr = expf(m[qq] - mn);
            l[qq] = l[qq] * corr + pf_wave_sum(e);
            m[qq] = mn;
#pragma unroll
            for (int ee = 0; ee < EPL; ee++) acc[qq][ee] *= corr;
#pragma unroll 16
            for (int j = 0; j < 64; j++) {
                const float pj = __shfl(e, j, 64);
#pragma unroll
                for (int ee = 0; ee < EPL; ee++) acc[qq][ee] = fmaf(pj, Vt[j * LDK + lane + 64 * ee], acc[qq][ee]);
            }
        }
    }
#pragma unroll
    for (int qq = 0; qq < QPW; qq++) {
        const int q = wave * QPW + qq;
        if (q >= nq) continue;
        const size_t row = (size_t)(row0 + q);
#pragma unroll
        for (int ee = 0; ee < EPL; ee++) {
            const int dcol = h * HD + lane + 64 * ee;
            float v = acc[qq][ee] / l[qq];
            if (a.gating) v = v * pf_sigmoid(P.QKV[row * P.qkvLd + L.offG + dcol]);
            put<AT>((AT*)P.Amix + row * P.aLd + dcol, v);
        }
    }
}

// ----------------------------------------------------------------------------
// fp16 MFMA causal attention (bf16-weight models; their MFMA path computes in IEEE half, see the host section).  A workgroup owns one head and 128 consecutive
// queries of one segment, a wave 32 of them.  Per 64-key page:
//   S^T[key, query] = K . Q^T      (A = K tile from LDS, B = Q^T held in registers)
//   online softmax down the key axis -- with the transposed product every lane owns ONE query column
//   (accumulator element i of lane l is row 8(i/4) + 4(l/32) + i%4, column l%32), so the running max,
//   the running sum and the rescale of the output are in-lane, plus one exchange between lane halves
//   O^T[hd, query] += V^T . P^T    (B = the lane's own P values, A = V transposed in LDS)
// The contraction index of the second product may be permuted freely as long as A and B agree: slot
// (half, e) of 16-key step t is the key the accumulator layout puts there, and the V tile is written
// to LDS transposed in exactly that order, so P never leaves its registers.
// K and V come from the fp32 pages and are rounded to fp16 on the way into LDS; scores, softmax
// statistics and the output accumulate in fp32.
// ----------------------------------------------------------------------------
#define PF_MQB 128
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));


// position of key k (0..63) of a page along the permuted contraction axis of O^T += V^T . P^T
__device__ __forceinline__ int pv_slot(int k) {
    const int b = k >> 5, k32 = k & 31;
    const int i = 4 * (k32 >> 3) + (k32 & 3), hh = (k32 >> 2) & 1;
    return 16 * (2 * b + (i >> 3)) + 8 * hh + (i & 7);
}

template <int HD, bool H16>
__global__ void __launch_bounds__(PWG, H16 ? 2 : 1) k_pf_attn_mfma(PfArgs P, LayerDev L) {
    constexpr int KP = HD + 8;   // K tile row pitch (16-bit elements): 16-byte reads, rows 4 banks apart
    constexpr int VP = 64 + 8;   // V^T row pitch
    constexpr int KS = HD / 16;  // 16-wide contraction steps of K . Q^T
    constexpr int MB = HD / 32;  // 32-row blocks of O^T
    __shared__ __attribute__((aligned(16))) uint16_t Kt[64 * KP];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[HD * VP];
    const StepArgs& a = P.a;
    const int h = blockIdx.x, blk = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int seg = P.blkSeg[blk], q0 = P.blkQ0[blk];
    const int seq = P.segSeq[seg], pos0 = P.segPos0[seg], len = P.segLen[seg];
    const int n32 = lane & 31, half = lane >> 5;
    const int qi = q0 + wave * 32 + n32;              // this lane's query within the segment
    const int qrow = P.segStart[seg] + min(qi, len - 1);
    const int qpos = pos0 + qi;
    const int waveMaxPos = pos0 + min(q0 + wave * 32 + 31, len - 1);
    const int maxPos = pos0 + min(q0 + PF_MQB, len) - 1;
    const bool waveActive = q0 + wave * 32 < len;

    // Q^T operand (fp16): for step s the lane holds q[16 s + 8 half .. +7] of its query, times log2(e) / sqrt(HD): the
    // scores come out of the MFMA ready for exp2
    u32x4 qop[KS];
    {
        const float* q = P.QKV + (size_t)qrow * P.qkvLd + h * HD + 8 * half;
        const float qs = 1.44269504088896341f / sqrtf((float)HD);
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(q + 16 * s) * qs, hi = *reinterpret_cast<const f32x4*>(q + 16 * s + 4) * qs;
            qop[s].x = pack_f16(lo.x, lo.y); qop[s].y = pack_f16(lo.z, lo.w);
            qop[s].z = pack_f16(hi.x, hi.y); qop[s].w = pack_f16(hi.z, hi.w);
        }
    }
    f32x16 oacc[MB];
#pragma unroll
    for (int b = 0; b < MB; b++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[b][i] = 0.f;
    float m_run = -1.0e30f, l_run = 0.f;
    const int waveMinPos = pos0 + q0 + wave * 32; // the lowest query position of the wave
    const int ntiles = (maxPos >> 6) + 1;

    // A tile's K and V rows travel global -> registers -> LDS; the loads of tile t + 1 are issued before tile t is
    // multiplied, so their latency runs under the MFMAs.  Rows beyond the last position any query of the workgroup
    // may see are read from a clamped row and zeroed (every load unconditional: all of them in flight at once).
    // H16: every segment of the call starts at position 0, so key j of the segment is row segStart + j of the call and
    // its K and V rows exist as halves (written by the QK-norm / RoPE kernel): half the bytes, no conversion, and few
    // enough registers for two workgroups per compute unit -- one multiplies while the other does its softmax.
    constexpr int NK = 64 * (HD / 4) / PWG, NV = 32 * (HD / 4) / PWG;
    constexpr int NK16 = 64 * (HD / 8) / PWG, NV16 = 32 * (HD / 8) / PWG;
    f32x4 kreg[H16 ? 1 : NK], vreg[H16 ? 1 : NV][2];
    u32x4 kreg16[H16 ? NK16 : 1], vreg16[H16 ? NV16 : 1][2];
    auto fetch = [&](int t) {
        const int j0 = t << 6;
        const int rmax = maxPos - j0; // >= 0
        if (H16) {
            const size_t base = ((size_t)P.segStart[seg] + j0) * a.dim + h * HD; // pos0 == 0: key position == row within the segment
#pragma unroll
            for (int n = 0; n < NK16; n++) {
                const int i = tid + n * PWG, r = i / (HD / 8), c8 = (i % (HD / 8)) * 8;
                kreg16[n] = *reinterpret_cast<const u32x4*>(P.Kh + base + (size_t)min(r, rmax) * a.dim + c8);
            }
#pragma unroll
            for (int n = 0; n < NV16; n++) {
                const int i = tid + n * PWG, kp = i & 7, g = (i >> 3) % (HD / 8), ko = (i >> 3) / (HD / 8);
                const int k = 16 * ko + 2 * kp, c8 = 8 * g;
                vreg16[n][0] = *reinterpret_cast<const u32x4*>(P.Vh + base + (size_t)min(k, rmax) * a.dim + c8);
                vreg16[n][1] = *reinterpret_cast<const u32x4*>(P.Vh + base + (size_t)min(k + 1, rmax) * a.dim + c8);
            }
            return;
        }
        const int page = a.pageTable[seq * a.pagesPerSeq + t];
        const size_t base = ((size_t)page * MLH_KV_PAGE) * a.dim + h * HD;
#pragma unroll
        for (int n = 0; n < NK; n++) {
            const int i = tid + n * PWG, r = i / (HD / 4), c4 = (i % (HD / 4)) * 4;
            kreg[n] = *reinterpret_cast<const f32x4*>(L.K + base + (size_t)min(r, rmax) * a.dim + c4);
        }
#pragma unroll
        for (int n = 0; n < NV; n++) {
            const int i = tid + n * PWG, kp = i & 7, g = (i >> 3) % (HD / 4), ko = (i >> 3) / (HD / 4);
            const int k = 16 * ko + 2 * kp, c4 = 4 * g;
            vreg[n][0] = *reinterpret_cast<const f32x4*>(L.V + base + (size_t)min(k, rmax) * a.dim + c4);
            vreg[n][1] = *reinterpret_cast<const f32x4*>(L.V + base + (size_t)min(k + 1, rmax) * a.dim + c4);
        }
    };
    fetch(0);
    for (int t = 0; t < ntiles; t++) {
        const int j0 = t << 6;
        const int rmax = maxPos - j0;
        __syncthreads(); // the previous tile has been consumed
        if (H16) {
            // ---- K tile: natural layout, sixteen bytes per store ----
#pragma unroll
            for (int n = 0; n < NK16; n++) {
                const int i = tid + n * PWG, r = i / (HD / 8), c8 = (i % (HD / 8)) * 8;
                *reinterpret_cast<u32x4*>(Kt + r * KP + c8) = r <= rmax ? kreg16[n] : (u32x4)(0u);
            }
            // ---- V tile: transposed, keys in contraction-slot order; a lane carries two keys that are neighbours there:
            // for every column the halves of both keys go into one 32-bit word (v_perm picks the two 16-bit pieces) ----
#pragma unroll
            for (int n = 0; n < NV16; n++) {
                const int i = tid + n * PWG, kp = i & 7, g = (i >> 3) % (HD / 8), ko = (i >> 3) / (HD / 8);
                const int k = 16 * ko + 2 * kp, c8 = 8 * g;
                const u32x4 v0 = k <= rmax ? vreg16[n][0] : (u32x4)(0u), v1 = k + 1 <= rmax ? vreg16[n][1] : (u32x4)(0u);
                const int slot = pv_slot(k); // even, and pv_slot(k + 1) == slot + 1
#pragma unroll
                for (int w = 0; w < 4; w++) { // word w holds columns c8 + 2 w (low half) and c8 + 2 w + 1 (high half)
                    *reinterpret_cast<uint32_t*>(Vt + (c8 + 2 * w + 0) * VP + slot) = __builtin_amdgcn_perm(v1[w], v0[w], 0x05040100u);
                    *reinterpret_cast<uint32_t*>(Vt + (c8 + 2 * w + 1) * VP + slot) = __builtin_amdgcn_perm(v1[w], v0[w], 0x07060302u);
                }
            }
        } else {
        // ---- K tile: natural layout ----
#pragma unroll
            for (int n = 0; n < NK; n++) {
                const int i = tid + n * PWG, r = i / (HD / 4), c4 = (i % (HD / 4)) * 4;
                const f32x4 kk = r <= rmax ? kreg[n] : (f32x4)(0.f);
                u32x2 w; w.x = pack_f16(kk.x, kk.y); w.y = pack_f16(kk.z, kk.w);
                *reinterpret_cast<u32x2*>(Kt + r * KP + c4) = w;
            }
            // ---- V tile: transposed, keys in contraction-slot order; a lane carries two keys that are neighbours there ----
#pragma unroll
            for (int n = 0; n < NV; n++) {
                const int i = tid + n * PWG, kp = i & 7, g = (i >> 3) % (HD / 4), ko = (i >> 3) / (HD / 4); // key pair, column chunk, group of 8 pairs
                const int k = 16 * ko + 2 * kp, c4 = 4 * g;
                const f32x4 v0 = k <= rmax ? vreg[n][0] : (f32x4)(0.f), v1 = k + 1 <= rmax ? vreg[n][1] : (f32x4)(0.f);
                const int slot = pv_slot(k); // even, and pv_slot(k + 1) == slot + 1
                *reinterpret_cast<uint32_t*>(Vt + (c4 + 0) * VP + slot) = pack_f16(v0.x, v1.x);
                *reinterpret_cast<uint32_t*>(Vt + (c4 + 1) * VP + slot) = pack_f16(v0.y, v1.y);
                *reinterpret_cast<uint32_t*>(Vt + (c4 + 2) * VP + slot) = pack_f16(v0.z, v1.z);
                *reinterpret_cast<uint32_t*>(Vt + (c4 + 3) * VP + slot) = pack_f16(v0.w, v1.w);
            }
        }
        __syncthreads();
        if (t + 1 < ntiles) fetch(t + 1);
        if (!waveActive || j0 > waveMaxPos) continue; // wave-uniform; the barriers above are still reached by every wave
        // ---- S^T = K . Q^T for the two 32-key blocks ----
        f32x16 sacc[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[b][i] = 0.f;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const u32x4 kop = *reinterpret_cast<const u32x4*>(Kt + (32 * b + n32) * KP + 16 * s + 8 * half);
                sacc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kop), __builtin_bit_cast(f16x8, qop[s]), sacc[b], 0, 0, 0);
            }
        }
        // ---- causal mask, online softmax down the key axis (base 2: the scores carry log2(e) / sqrt(HD)) ----
        // A tile that lies entirely at or below the wave's lowest query position needs no mask (all but the last one or
        // two tiles of a wave), and the output is only rescaled when some query's running maximum moved.
        float mx = -1.0e30f;
        const bool fullTile = j0 + 63 <= waveMinPos; // wave-uniform
        if (fullTile) {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i += 2) mx = fmaxf(mx, fmaxf(sacc[b][i], sacc[b][i + 1]));
        } else {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = j0 + 32 * b + 8 * (i >> 2) + 4 * half + (i & 3);
                    const float sv = key <= qpos ? sacc[b][i] : -1.0e30f;
                    sacc[b][i] = sv;
                    mx = fmaxf(mx, sv);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(m_run, mx);
        float ls = 0.f;
        if (fullTile) {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const float pv = __builtin_amdgcn_exp2f(sacc[b][i] - mn);
                    sacc[b][i] = pv;
                    ls += pv;
                }
        } else {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const float pv = sacc[b][i] > -1.0e29f ? __builtin_amdgcn_exp2f(sacc[b][i] - mn) : 0.f;
                    sacc[b][i] = pv;
                    ls += pv;
                }
        }
        ls += __shfl_xor(ls, 32, 64);
        if (__any(mn > m_run)) { // wave-uniform
            const float corr = __builtin_amdgcn_exp2f(m_run - mn);
            l_run *= corr;
#pragma unroll
            for (int b = 0; b < MB; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) oacc[b][i] *= corr;
        }
        l_run += ls;
        m_run = mn;
        // ---- O^T += V^T . P^T ----
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const int b = st >> 1, e0 = 8 * (st & 1);
            u32x4 pop;
            pop.x = pack_f16(sacc[b][e0 + 0], sacc[b][e0 + 1]); pop.y = pack_f16(sacc[b][e0 + 2], sacc[b][e0 + 3]);
            pop.z = pack_f16(sacc[b][e0 + 4], sacc[b][e0 + 5]); pop.w = pack_f16(sacc[b][e0 + 6], sacc[b][e0 + 7]);
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const u32x4 vop = *reinterpret_cast<const u32x4*>(Vt + (32 * mb + n32) * VP + 16 * st + 8 * half);
                oacc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, vop), __builtin_bit_cast(f16x8, pop), oacc[mb], 0, 0, 0);
            }
        }
    }
    if (qi >= len) return;
    const float inv_l = 1.0f / l_run;
    const size_t row = (size_t)qrow;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
            const int dcol = h * HD + 32 * mb + 8 * i4 + 4 * half;
            f32x4 o;
            o.x = oacc[mb][4 * i4] * inv_l; o.y = oacc[mb][4 * i4 + 1] * inv_l; o.z = oacc[mb][4 * i4 + 2] * inv_l; o.w = oacc[mb][4 * i4 + 3] * inv_l;
            if (a.gating) {
                const f32x4 gt = *reinterpret_cast<const f32x4*>(P.QKV + row * P.qkvLd + L.offG + dcol);
                o.x *= pf_sigmoid(gt.x); o.y *= pf_sigmoid(gt.y); o.z *= pf_sigmoid(gt.z); o.w *= pf_sigmoid(gt.w);
            }
            u32x2 w; w.x = pack_f16(o.x, o.y); w.y = pack_f16(o.z, o.w);
            *reinterpret_cast<u32x2*>((bf16_t*)P.Amix + row * P.aLd + dcol) = w;
        }
}

// Gated-delta-net prefill.  The rows of a head's state evolve independently of each other
//   S[r,:] <- alpha S[r,:] + beta (v_r - alpha u_r) k^T,  u_r = S[r,:].k,   o_r = S_new[r,:].q
// (the decode kernel's update, regrouped; k, q L2-normalised), so one workgroup carries PF_GR rows of
// one head of one segment in registers across the whole segment: 4 lanes per row, each with DK/4
// columns.  The decay is kept out of the element loop: the registers hold S / a for a running scalar a
// (the product of the alphas since the last renormalisation), so a token costs three FMAs per element
// -- S.k, S.q and the rank-1 update -- instead of four.  Sixteen tokens of q, k, v and gate inputs are staged in LDS at a time, the next sixteen
// being loaded into registers meanwhile.  With p = S_old[r,:].q the read-out needs no second pass:
// o_r = (alpha p + w (k.q)) / |q|,  w = beta (v_r - alpha u_r) / |k|.
#define PF_GC 16
#define PF_GR 64
// Workgroup barrier that orders LDS traffic only: __syncthreads() also waits for every outstanding global
// load (loads and stores share one counter), which would put the next chunk's prefetch on the critical path.
__device__ __forceinline__ void pf_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
template <int CTRL> __device__ __forceinline__ float quad_swap(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
template <int DK, typename AT>
__global__ void __launch_bounds__(PWG) k_pf_gdn(PfArgs P, LayerDev L, int skipFrom) {
    constexpr int DV = DK, TPR = PWG / PF_GR, CPT = DK / TPR;
    static_assert(TPR == 4, "the row sum below is a quad reduction");
    constexpr int NQK = PF_GC * DK / 4 / PWG; // f32x4 loads per thread for each of q and k
    __shared__ __attribute__((aligned(16))) float qs[PF_GC][DK];
    __shared__ __attribute__((aligned(16))) float ks[PF_GC][DK];
    __shared__ float vs[PF_GC][PF_GR];
    __shared__ float zs[PF_GC][2];
    __shared__ float gate[PF_GC][6]; // alpha, beta, 1/|q|, 1/|k|, k.q, 1/alpha
    const StepArgs& a = P.a;
    const int h = blockIdx.x, seg = blockIdx.y, r0 = blockIdx.z * PF_GR, tid = threadIdx.x;
    const int seq = P.segSeq[seg], len = P.segLen[seg], row0 = P.segStart[seg];
    if (len >= skipFrom) return; // taken by the chunk-parallel kernels
    const int r = tid / TPR, cg = tid % TPR, c0 = cg * CPT;
    float* Srow = L.S + (((size_t)seq * a.gdnHeads + h) * DV + r0 + r) * DK + c0;
    float S[CPT];
#pragma unroll
    for (int c = 0; c < CPT; c += 4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(Srow + c);
        S[c] = v.x; S[c + 1] = v.y; S[c + 2] = v.z; S[c + 3] = v.w;
    }
    float ascale = 1.0f, ainv = 1.0f; // S (true state) = ascale * S[] (registers); ainv = 1 / ascale
    f32x4 qreg[NQK], kreg[NQK];
    float vreg[PF_GC * PF_GR / PWG], zreg = 0.f;
    auto fetch = [&](int t0) {
        const int last = len - 1 - t0; // >= 0
#pragma unroll
        for (int it = 0; it < NQK; it++) {
            const int i = it * PWG + tid, c = i / (DK / 4), e4 = (i % (DK / 4)) * 4;
            const float* qkv = P.QKV + (size_t)(row0 + t0 + min(c, last)) * P.qkvLd;
            qreg[it] = *reinterpret_cast<const f32x4*>(qkv + h * DK + e4);
            kreg[it] = *reinterpret_cast<const f32x4*>(qkv + L.offK + h * DK + e4);
        }
#pragma unroll
        for (int it = 0; it < PF_GC * PF_GR / PWG; it++) {
            const int i = it * PWG + tid, c = i / PF_GR, e = i % PF_GR;
            vreg[it] = P.QKV[(size_t)(row0 + t0 + min(c, last)) * P.qkvLd + L.offV + h * DV + r0 + e];
        }
        if (tid < 2 * PF_GC) {
            const int c = tid >> 1;
            zreg = P.QKV[(size_t)(row0 + t0 + min(c, last)) * P.qkvLd + ((tid & 1) ? L.offGb : L.offGa) + h];
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < len; t0 += PF_GC) {
        const int nt = min(PF_GC, len - t0);
        pf_lds_barrier(); // the previous chunk has been consumed
#pragma unroll
        for (int it = 0; it < NQK; it++) {
            const int i = it * PWG + tid, c = i / (DK / 4), e4 = (i % (DK / 4)) * 4;
            *reinterpret_cast<f32x4*>(&qs[c][e4]) = qreg[it];
            *reinterpret_cast<f32x4*>(&ks[c][e4]) = kreg[it];
        }
#pragma unroll
        for (int it = 0; it < PF_GC * PF_GR / PWG; it++) {
            const int i = it * PWG + tid;
            vs[i / PF_GR][i % PF_GR] = vreg[it];
        }
        if (tid < 2 * PF_GC) zs[tid >> 1][tid & 1] = zreg;
        pf_lds_barrier();
        if (t0 + PF_GC < len) fetch(t0 + PF_GC); // in flight during this chunk's arithmetic
        { // per token: |q|, |k|, k.q and the gates -- 16 threads per token
            const int c = tid >> 4, sub = tid & 15;
            float sq = 0.f, sk = 0.f, kq = 0.f;
            for (int e = sub; e < DK; e += 16) {
                const float qv = qs[c][e], kv = ks[c][e];
                sq = fmaf(qv, qv, sq); sk = fmaf(kv, kv, sk); kq = fmaf(kv, qv, kq);
            }
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) { sq += __shfl_xor(sq, o, 64); sk += __shfl_xor(sk, o, 64); kq += __shfl_xor(kq, o, 64); }
            if (sub == 0) {
                const float za = zs[c][0] + L.gdnBa[h], zb = zs[c][1] + L.gdnBb[h];
                const float rq = 1.0f / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
                const float sp = fmaxf(za, 0.f) + log1pf(expf(-fabsf(za)));
                gate[c][0] = expf(-sp);
                gate[c][5] = expf(sp);
                gate[c][1] = pf_sigmoid(zb);
                gate[c][2] = rq; gate[c][3] = rk; gate[c][4] = kq * rq * rk; // k.q of the normalised vectors
            }
        }
        pf_lds_barrier();
#pragma unroll 4
        for (int c = 0; c < nt; c++) {
            const float alpha = gate[c][0], beta = gate[c][1], rq = gate[c][2], rk = gate[c][3], kqn = gate[c][4];
            float kk[CPT];
            float ua[4] = {0.f, 0.f, 0.f, 0.f}, pa[4] = {0.f, 0.f, 0.f, 0.f}; // four independent chains each
#pragma unroll
            for (int e = 0; e < CPT; e += 4) {
                const f32x4 k4 = *reinterpret_cast<const f32x4*>(&ks[c][c0 + e]);
                const f32x4 q4 = *reinterpret_cast<const f32x4*>(&qs[c][c0 + e]);
                kk[e] = k4.x; kk[e + 1] = k4.y; kk[e + 2] = k4.z; kk[e + 3] = k4.w;
                ua[0] = fmaf(S[e], k4.x, ua[0]); ua[1] = fmaf(S[e + 1], k4.y, ua[1]); ua[2] = fmaf(S[e + 2], k4.z, ua[2]); ua[3] = fmaf(S[e + 3], k4.w, ua[3]);
                pa[0] = fmaf(S[e], q4.x, pa[0]); pa[1] = fmaf(S[e + 1], q4.y, pa[1]); pa[2] = fmaf(S[e + 2], q4.z, pa[2]); pa[3] = fmaf(S[e + 3], q4.w, pa[3]);
            }
            float u = (ua[0] + ua[1]) + (ua[2] + ua[3]), p = (pa[0] + pa[1]) + (pa[2] + pa[3]);
            // sum over the 4 lanes of a row: quad permutes in the VALU (a cross-lane shuffle through LDS costs
            // ~100 cycles each, and this is the serial path from one token to the next)
            u += quad_swap<0xB1>(u); p += quad_swap<0xB1>(p);   // lanes 0<->1, 2<->3
            u += quad_swap<0x4E>(u); p += quad_swap<0x4E>(p);   // lanes 0<->2, 1<->3
            u *= rk * ascale; p *= rq * ascale;                // against the normalised k and q, with the decay put back
            const float wn = beta * (vs[c][r] - alpha * u);    // coefficient of the normalised k
            ascale *= alpha; ainv *= gate[c][5];               // gate[c][5] = 1 / alpha
            if (ascale < 1.0e-12f) {                           // workgroup-uniform (one head): fold the decay into the registers
#pragma unroll
                for (int e = 0; e < CPT; e++) S[e] *= ascale;
                ascale = 1.0f; ainv = 1.0f;
            }
            const float w = wn * rk * ainv;
#pragma unroll
            for (int e = 0; e < CPT; e++) S[e] = fmaf(w, kk[e], S[e]);
            if (cg == 0) put<AT>((AT*)P.Amix + (size_t)(row0 + t0 + c) * P.aLd + h * DV + r0 + r, alpha * p + wn * kqn);
        }
    }
#pragma unroll
    for (int e = 0; e < CPT; e++) S[e] *= ascale;
#pragma unroll
    for (int c = 0; c < CPT; c += 4) {
        f32x4 v; v.x = S[c]; v.y = S[c + 1]; v.z = S[c + 2]; v.w = S[c + 3];
        *reinterpret_cast<f32x4*>(Srow + c) = v;
    }
}

// ----------------------------------------------------------------------------
// Chunk-parallel gated-delta-net prefill on the MFMA units (bf16 models, segments of 64 tokens or more).
//
// Over a chunk of C = 64 tokens starting from state S0, with g_t = sum_{j<=t} log(alpha_j):
//   S_t = e^{g_t} S0 + sum_{i<=t} e^{g_t - g_i} w_i k_i^T,      w_t = beta_t (v_t - alpha_t S_{t-1} k_t)
// (k, q L2-normalised).  Substituting S_{t-1} gives a unit-lower-triangular system for the w_t:
//   (I + A) W^T = beta (.) V - diag(beta e^{g}) K S0^T,   A[t,i] = beta_t e^{g_t - g_i} (k_i . k_t), i < t
// so W^T = Vt - Kt S0^T with Vt = (I+A)^{-1} (beta (.) V) and Kt = (I+A)^{-1} diag(beta e^{g}) K, both free
// of S0.  The outputs and the next state are then plain products:
//   O   = diag(e^{g}) Q S0^T + M W^T,      M[t,i] = e^{g_t - g_i} (k_i . q_t), i <= t
//   S_C = e^{g_C} S0 + W Kh,               Kh[i,:] = e^{g_C - g_i} k_i
// k_gdn_prep builds Vt, Kt, diag(e^g) Q, M, Kh for every chunk of every head in parallel (forward
// substitution, 64 steps, one column per thread); k_gdn_scan walks the chunks of one head of one
// segment in order with the state -- transposed, S^T[dk, dv] -- in MFMA accumulators, 56 MFMAs per
// chunk and wave.  Operands are IEEE half, accumulation and the state fp32.  Every contraction index
// (dk in Kt S0^T and Q S0^T, the chunk's token index in M W^T and Kh^T W^T) is stored in the order
// the accumulator layout holds it (slot_of below), so S0^T and W^T are used as MFMA B operands straight
// from the accumulator registers, without a transpose through LDS.
// ----------------------------------------------------------------------------
#define GD_C 64
// accumulator element i of lane (n, half) of a 32x32 tile is row 8(i/4) + 4 half + i%4; a 16-wide MFMA step
// st takes elements 8 st .. 8 st + 7 of both halves.  slot_of(x) = position of row x of a (multi-tile)
// contraction axis in that order: tile x/32, then step, half, element.
__host__ __device__ __forceinline__ int slot_of(int x) {
    const int x32 = x & 31;
    const int i = 4 * (x32 >> 3) + (x32 & 3), hh = (x32 >> 2) & 1;
    return (x & ~31) + 16 * (i >> 3) + 8 * hh + (i & 7);
}
template <int DK> struct GdLayout { // one chunk's operand image (bytes), rows padded by 16 bytes against LDS bank conflicts
    static constexpr int KP = (DK + 8) * 2, TP = (GD_C + 8) * 2; // row pitches of [*, DK] and [*, 64] half matrices
    static constexpr int oKt = 0, oQh = oKt + GD_C * KP, oM = oQh + GD_C * KP, oKhT = oM + GD_C * TP;
    static constexpr int oVt = oKhT + DK * TP;                    // half [DV, 64]: a column's 64 tokens contiguous
    static constexpr int image = oVt + DK * TP;                   // 80896 (DK 128), 46080 (DK 64): multiples of 1024
    static constexpr int total = image;
};
__device__ __forceinline__ uint16_t f16_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }

template <int DK>
__global__ void __launch_bounds__(2 * DK, 2) k_gdn_prep(PfArgs P, LayerDev L, const int* __restrict__ chunkSeg, const int* __restrict__ chunkT0,
                                                      unsigned char* __restrict__ ws, float* __restrict__ gCexp) {
    constexpr int DV = DK, NT = 2 * DK;
    typedef GdLayout<DK> Lay;
    extern __shared__ __attribute__((aligned(16))) unsigned char pls[];
    float* Am = reinterpret_cast<float*>(pls);            // [64][64]
    float* gs = Am + GD_C * GD_C;                         // g[64], beta[64], sp[64], 1/|k|[64], 1/|q|[64], partial sums [4][64]
    uint16_t* k16 = reinterpret_cast<uint16_t*>(gs + 12 * GD_C); // [64][DK + 8] normalised k, half
    uint16_t* q16 = k16 + GD_C * (DK + 8);
    const StepArgs& a = P.a;
    const int chunk = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int seg = chunkSeg[chunk], t0 = chunkT0[chunk];
    const int nv = min(GD_C, P.segLen[seg] - t0), row0 = P.segStart[seg] + t0;
    unsigned char* img = ws + ((size_t)chunk * a.gdnHeads + h) * Lay::total;
    float* g = gs; float* beta = gs + GD_C; float* sp = gs + 2 * GD_C; float* rk = gs + 3 * GD_C; float* rq = gs + 4 * GD_C;
    float* part = gs + 5 * GD_C;
    float* eg = gs + 9 * GD_C;   // e^{g_t}
    float* egc = gs + 10 * GD_C; // e^{g_C - g_t}

    // Thread (sel, cidx) keeps column cidx of q (sel 0: threads [0, DK)) or k (sel 1: threads [DK, 2 DK)) for the 64
    // tokens of the chunk in registers (tokens past the segment end: zero).
    const int sel = tid / DK, cidx = tid % DK;
    float colv[GD_C];
    {
        const float* src = P.QKV + (size_t)row0 * P.qkvLd + (sel ? L.offK : 0) + h * DK + cidx;
#pragma unroll
        for (int t = 0; t < GD_C; t++) { // unconditional loads of clamped rows: 64 loads in flight, no branch per row
            const float v = src[(size_t)min(t, nv - 1) * P.qkvLd];
            colv[t] = t < nv ? v : 0.f;
        }
    }
    if (tid < GD_C) { // gates
        const int t = tid;
        float s_ = 0.f, b_ = 0.f;
        if (t < nv) {
            const float* qkv = P.QKV + (size_t)(row0 + t) * P.qkvLd;
            const float za = qkv[L.offGa + h] + L.gdnBa[h], zb = qkv[L.offGb + h] + L.gdnBb[h];
            s_ = fmaxf(za, 0.f) + log1pf(expf(-fabsf(za))); // -log(alpha)
            b_ = pf_sigmoid(zb);
        }
        sp[t] = s_; beta[t] = b_;
        float v = -s_; // inclusive prefix sum over the 64 tokens (one wave)
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const float u = __shfl_up(v, o, 64); if (tid >= o) v += u; }
        g[t] = v;
    }
    { // squared norms per token: reduce-scatter over the 64 lanes of a wave (lane t ends up with token t), then over waves
        float r[GD_C];
#pragma unroll
        for (int t = 0; t < GD_C; t++) r[t] = colv[t] * colv[t];
#pragma unroll
        for (int o = 32, n = 32; o > 0; o >>= 1, n >>= 1) {
            const bool up = (lane & o) != 0;
#pragma unroll
            for (int i = 0; i < n; i++) {
                const float keep = up ? r[i + n] : r[i], send = up ? r[i] : r[i + n];
                r[i] = keep + __shfl_xor(send, o, 64);
            }
        }
        part[wave * GD_C + lane] = r[0];
    }
    __syncthreads();
    if (tid < 2 * GD_C) { // 1 / norm of q (threads 0..63) and k (64..127)
        const int t = tid & 63, m = tid >> 6; // m 0: q, 1: k
        constexpr int WPM = DK / 64;          // waves per matrix
        float ss = 0.f;
#pragma unroll
        for (int w = 0; w < WPM; w++) ss += part[(m * WPM + w) * GD_C + t];
        (m ? rk : rq)[t] = 1.0f / sqrtf(ss + 1e-6f);
        if (m == 0) { eg[t] = expf(g[t]); egc[t] = expf(g[GD_C - 1] - g[t]); }
    }
    __syncthreads();
    { // normalise the register column, publish the half copy for the MFMAs
        const float* rr = sel ? rk : rq;
        uint16_t* d16 = sel ? k16 : q16;
#pragma unroll
        for (int t = 0; t < GD_C; t++) {
            colv[t] *= rr[t];
            d16[t * (DK + 8) + cidx] = f16_bits(colv[t]);
        }
    }
    __syncthreads();
    { // K K^T and Q K^T on the MFMA units: 2 x 2 tiles each
        const int n32 = lane & 31, half = lane >> 5;
        for (int tix = wave; tix < 8; tix += NT / 64) {
            const int which = tix >> 2, tt = (tix >> 1) & 1, ti = tix & 1;
            const uint16_t* Aop = (which ? q16 : k16) + (32 * tt + n32) * (DK + 8) + 8 * half;
            const uint16_t* Bop = k16 + (32 * ti + n32) * (DK + 8) + 8 * half;
            f32x16 acc;
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] = 0.f;
#pragma unroll
            for (int s_ = 0; s_ < DK / 16; s_++)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(Aop + 16 * s_)),
                                                             __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(Bop + 16 * s_)), acc, 0, 0, 0);
            const int i_ = 32 * ti + n32;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int t = 32 * tt + 8 * (e >> 2) + 4 * half + (e & 3);
                const float dec = expf(g[t] - g[i_]); // <= 1 where it is used (i <= t)
                if (which == 0) Am[t * GD_C + i_] = i_ < t ? beta[t] * dec * acc[e] : 0.f;
                else *reinterpret_cast<uint16_t*>(img + Lay::oM + t * Lay::TP + 2 * slot_of(i_)) = f16_bits(i_ <= t ? dec * acc[e] : 0.f);
            }
        }
    }
    __syncthreads();
    // forward substitution, one column per thread: threads [0, DV) solve beta (.) V, threads [DV, 2 DV) -- the ones
    // that hold the k columns -- solve diag(beta e^g) K
    float X[GD_C];
    const int col = cidx;
    if (tid < DV) {
        const float* vsrc = P.QKV + (size_t)row0 * P.qkvLd + L.offV + h * DV + col;
#pragma unroll
        for (int t = 0; t < GD_C; t++) X[t] = vsrc[(size_t)min(t, nv - 1) * P.qkvLd]; // all 64 loads in flight at once
#pragma unroll
        for (int t = 0; t < GD_C; t++) X[t] *= beta[t]; // beta is zero for tokens past the segment end
    } else {
#pragma unroll
        for (int t = 0; t < GD_C; t++) X[t] = beta[t] * eg[t] * colv[t];
    }
    // Blocked forward substitution.  The 64 rows go in four blocks of 16: inside a block a thread solves its column in
    // fp32 as before (the block's own triangle, 120 multiply-adds); what the solved block contributes to all later rows,
    // A[later rows, block] X[block], is a matrix product and runs on the MFMA units with half operands -- a wave takes
    // its own 64 columns (two column tiles), so nothing here needs a workgroup barrier: LDS instructions of a wave
    // execute in order.  Per wave 8 MFMAs replace three quarters of the 2016 multiply-adds a thread had on its chain.
    {
        constexpr int AHP = GD_C + 8;                       // pitch of the half copy of A (elements): 16-byte reads, rows 4 banks apart
        uint16_t* Ah = k16;                                 // [64][AHP]; k16 / q16 are free: their MFMAs are done (barrier above)
        unsigned char* wsc = reinterpret_cast<unsigned char*>(Ah + GD_C * AHP) + wave * (64 * 80); // this wave's exchange area
        // X of the solved block as halves, [column][16] with pitch 48 bytes (B operand); the update of the next block's
        // rows, [column][16] floats with pitch 80 bytes -- both conflict-free for 16-byte accesses, and they may share
        // the area: the MFMAs have read the one before the other is written (same wave, in order)
        for (int i = tid; i < GD_C * GD_C / 2; i += NT) { // half copy of A, two elements per thread and trip
            const int t = i / (GD_C / 2), i2 = (i % (GD_C / 2)) * 2;
            *reinterpret_cast<uint32_t*>(Ah + t * AHP + i2) = pack_f16(Am[t * GD_C + i2], Am[t * GD_C + i2 + 1]);
        }
        __syncthreads();
        const int n32 = lane & 31, half = lane >> 5;
        f32x16 upd[2]; // [column tile of the wave]: what the solved blocks contribute to rows 32 .. 63
#pragma unroll
        for (int ct = 0; ct < 2; ct++)
#pragma unroll
            for (int e = 0; e < 16; e++) upd[ct][e] = 0.f;
        auto hand_over = [&](const f32x16& u, int ct, int e0) { // elements e0 .. e0 + 7 = 16 rows of a tile, to the owners of the columns
#pragma unroll
            for (int j = 0; j < 2; j++) {
                f32x4 v;
                v.x = u[e0 + 4 * j]; v.y = u[e0 + 4 * j + 1]; v.z = u[e0 + 4 * j + 2]; v.w = u[e0 + 4 * j + 3];
                *reinterpret_cast<f32x4*>(wsc + (32 * ct + n32) * 80 + (8 * j + 4 * half) * 4) = v; // rows 8 j + 4 half + 0..3 of the block
            }
        };
#pragma unroll
        for (int b = 0; b < 4; b++) {
            if (b > 1) { // rows 16 b .. 16 b + 15: elements 8 (b & 1) .. + 7 of the tile of rows 32 .. 63 (block 1's were handed over by block 0)
                hand_over(upd[0], 0, 8 * (b & 1));
                hand_over(upd[1], 1, 8 * (b & 1));
            }
            if (b > 0) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const f32x4 u = *reinterpret_cast<const f32x4*>(wsc + lane * 80 + q * 16);
                    X[16 * b + 4 * q] -= u.x; X[16 * b + 4 * q + 1] -= u.y; X[16 * b + 4 * q + 2] -= u.z; X[16 * b + 4 * q + 3] -= u.w;
                }
            }
#pragma unroll
            for (int tt = 1; tt < 16; tt++) { // the block's own triangle
                const int t = 16 * b + tt;
                float acc0 = X[t], acc1 = 0.f, acc2 = 0.f, acc3 = 0.f; // four chains: the row's dot product is on the serial path
#pragma unroll
                for (int i4 = 0; i4 < tt; i4 += 4) {
                    const f32x4 a4 = *reinterpret_cast<const f32x4*>(Am + t * GD_C + 16 * b + i4); // zero at and beyond the diagonal
                    acc0 = fmaf(-a4.x, X[16 * b + i4], acc0);
                    if (i4 + 1 < tt) acc1 = fmaf(-a4.y, X[16 * b + i4 + 1], acc1);
                    if (i4 + 2 < tt) acc2 = fmaf(-a4.z, X[16 * b + i4 + 2], acc2);
                    if (i4 + 3 < tt) acc3 = fmaf(-a4.w, X[16 * b + i4 + 3], acc3);
                }
                X[t] = (acc0 + acc1) + (acc2 + acc3);
            }
            if (b < 3) { // publish the block as halves and add its contribution to the later rows
                u32x4 w0, w1;
                w0.x = pack_f16(X[16 * b + 0], X[16 * b + 1]); w0.y = pack_f16(X[16 * b + 2], X[16 * b + 3]);
                w0.z = pack_f16(X[16 * b + 4], X[16 * b + 5]); w0.w = pack_f16(X[16 * b + 6], X[16 * b + 7]);
                w1.x = pack_f16(X[16 * b + 8], X[16 * b + 9]); w1.y = pack_f16(X[16 * b + 10], X[16 * b + 11]);
                w1.z = pack_f16(X[16 * b + 12], X[16 * b + 13]); w1.w = pack_f16(X[16 * b + 14], X[16 * b + 15]);
                *reinterpret_cast<u32x4*>(wsc + lane * 48) = w0;
                *reinterpret_cast<u32x4*>(wsc + lane * 48 + 16) = w1;
                u32x4 xop[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) xop[ct] = *reinterpret_cast<const u32x4*>(wsc + (32 * ct + n32) * 48 + 16 * half);
                const u32x4 aop1 = *reinterpret_cast<const u32x4*>(Ah + (32 + n32) * AHP + 16 * b + 8 * half);
#pragma unroll
                for (int ct = 0; ct < 2; ct++)
                    upd[ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, aop1), __builtin_bit_cast(f16x8, xop[ct]), upd[ct], 0, 0, 0);
                if (b == 0) { // rows 16 .. 31 are fed by block 0 alone: their tile lives only until it is handed over
                    const u32x4 aop0 = *reinterpret_cast<const u32x4*>(Ah + n32 * AHP + 8 * half);
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {
                        f32x16 u0;
#pragma unroll
                        for (int e = 0; e < 16; e++) u0[e] = 0.f;
                        u0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, aop0), __builtin_bit_cast(f16x8, xop[ct]), u0, 0, 0, 0);
                        hand_over(u0, ct, 8); // (the exchange area is free: both column tiles' operands are in registers)
                    }
                }
            }
        }
    }
    const float gC = g[GD_C - 1];
    const int sl = slot_of(col);
    // Kt, diag(e^g) Q and Kh^T are assembled in LDS in the image layout (the half copies of k and q are no longer
    // needed: the MFMAs are done) and leave as 16-byte rows; element-wise 2-byte stores to global would touch a
    // different cache line per lane.
    uint16_t* khs = q16 + GD_C * (DK + 8); // [DK][64 + 8]
    __syncthreads();                       // every column is solved: the triangular matrix has been read for the last time
    uint16_t* vts = reinterpret_cast<uint16_t*>(Am); // V^T [DV][64] takes its place (the same 64 * DV * 2 bytes)
    if (tid < DV) { // holds the q column
#pragma unroll
        for (int t = 0; t < GD_C; t += 8) { // this column's 64 tokens in a row: the scan reads four at a time
            u32x4 w;
            w.x = pack_f16(X[t], X[t + 1]); w.y = pack_f16(X[t + 2], X[t + 3]); w.z = pack_f16(X[t + 4], X[t + 5]); w.w = pack_f16(X[t + 6], X[t + 7]);
            *reinterpret_cast<u32x4*>(vts + col * GD_C + t) = w;
        }
#pragma unroll
        for (int t = 0; t < GD_C; t++) q16[t * (DK + 8) + sl] = f16_bits(eg[t] * colv[t]);
    } else { // holds the k column
#pragma unroll
        for (int t = 0; t < GD_C; t++) {
            k16[t * (DK + 8) + sl] = f16_bits(X[t]);
            khs[col * (GD_C + 8) + slot_of(t)] = f16_bits(egc[t] * colv[t]); // e^{g_C - g_t} k_t, token axis in slot order
        }
    }
    __syncthreads();
    {
        const u32x4* s1 = reinterpret_cast<const u32x4*>(k16);
        u32x4* d1 = reinterpret_cast<u32x4*>(img + Lay::oKt);
        for (int i = tid; i < 2 * GD_C * Lay::KP / 16; i += NT) d1[i] = s1[i];
        const u32x4* s2 = reinterpret_cast<const u32x4*>(khs);
        u32x4* d2 = reinterpret_cast<u32x4*>(img + Lay::oKhT);
        for (int i = tid; i < DK * Lay::TP / 16; i += NT) d2[i] = s2[i];
        const u32x4* s3 = reinterpret_cast<const u32x4*>(vts); // rows of eight 16-byte pieces to rows of pitch TP
        for (int i = tid; i < DV * 8; i += NT) *reinterpret_cast<u32x4*>(img + Lay::oVt + (i >> 3) * Lay::TP + (i & 7) * 16) = s3[i];
    }
    if (tid == 0) gCexp[(size_t)chunk * a.gdnHeads + h] = expf(gC);
}

// Copies one chunk's operand image (IMG bytes, a multiple of 1 KB) from global memory straight into LDS, 1 KB per
// instruction, the NW waves of the workgroup taking instructions in turn.
template <int IMG, int NW>
__device__ __forceinline__ void gd_issue_image(const unsigned char* src, unsigned char* dst, int wave, int lane) {
    for (int q = wave; q < IMG / 1024; q += NW) __builtin_amdgcn_global_load_lds(src + q * 1024 + lane * 16, dst + q * 1024, 16, 0, 0);
}

// The same, one instruction at a time: load k of this wave (k < ceil(IMG / 1024 / NW)), to be spread over other work.
template <int IMG, int NW>
__device__ __forceinline__ void gd_issue_image_one(const unsigned char* src, unsigned char* dst, int wave, int lane, int k) {
    const int q = wave + k * NW;
    if (q < IMG / 1024) __builtin_amdgcn_global_load_lds(src + q * 1024 + lane * 16, dst + q * 1024, 16, 0, 0);
}

template <int DK>
__global__ void __launch_bounds__(2 * DK) k_gdn_scan(PfArgs P, LayerDev L, const int* __restrict__ chunkBase, const unsigned char* __restrict__ ws,
                                                      const float* __restrict__ gCexp) {
    constexpr int DV = DK, NW = DV / 32, JT = DK / 32; // waves (one per 32 state columns dv), dk tiles
    typedef GdLayout<DK> Lay;
    extern __shared__ __attribute__((aligned(16))) unsigned char sls[]; // two operand images
    const StepArgs& a = P.a;
    const int h = blockIdx.x, seg = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int len = P.segLen[seg];
    if (len < GD_C) return; // short segments take the recurrent kernel
    const int seq = P.segSeq[seg], row0 = P.segStart[seg], nch = (len + GD_C - 1) / GD_C, cb = chunkBase[seg];
    const int n32 = lane & 31, half = lane >> 5, dv = 32 * wave + n32;
    float* Sg = L.S + ((size_t)seq * a.gdnHeads + h) * DV * DK;
    f32x16 St[JT]; // S^T tile j: rows dk = 32 j + 8(i/4) + 4 half + i%4, column dv
#pragma unroll
    for (int j = 0; j < JT; j++)
#pragma unroll
        for (int i = 0; i < 16; i++) St[j][i] = Sg[(size_t)dv * DK + 32 * j + 8 * (i >> 2) + 4 * half + (i & 3)];
    auto image_of = [&](int c) { return ws + ((size_t)(cb + c) * a.gdnHeads + h) * Lay::total; };
    auto issue = [&](int c, int stage) { gd_issue_image<Lay::image, NW>(image_of(c), sls + stage * Lay::image, wave, lane); };
    constexpr int NIMG = (Lay::image / 1024 + NW - 1) / NW; // loads per wave and image
    auto issue_one = [&](int c, int stage, int k) { gd_issue_image_one<Lay::image, NW>(image_of(c), sls + stage * Lay::image, wave, lane, k); };
    // V^T - (what the state predicts) needs tokens 8 g + 4 half + e, e = 0..3, of column dv: eight bytes of the image
    auto vt_of = [&](const unsigned char* im, int tt, int st, float (&v)[8]) { // elements 8 st .. 8 st + 7 of tile tt
        const unsigned char* p = im + Lay::oVt + dv * Lay::TP + (32 * tt + 16 * st + 4 * half) * 2;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            const u32x2 w = *reinterpret_cast<const u32x2*>(p + 16 * g);
            v[4 * g + 0] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w.x & 0xffff));
            v[4 * g + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w.x >> 16));
            v[4 * g + 2] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w.y & 0xffff));
            v[4 * g + 3] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w.y >> 16));
        }
    };
    issue(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
    asm volatile("" ::: "memory");
    __syncthreads();
    for (int c = 0; c < nch; c++) {
        const unsigned char* im = sls + (c & 1) * Lay::image;
        const bool more = c + 1 < nch;
        const float gC = gCexp[(size_t)(cb + c) * a.gdnHeads + h];
        // S0^T as B operands: step (j, st) = elements 8 st .. 8 st + 7 of tile j, rounded to half
        u32x4 sop[JT][2];
#pragma unroll
        for (int j = 0; j < JT; j++)
#pragma unroll
            for (int st = 0; st < 2; st++) {
                sop[j][st].x = pack_f16(St[j][8 * st + 0], St[j][8 * st + 1]); sop[j][st].y = pack_f16(St[j][8 * st + 2], St[j][8 * st + 3]);
                sop[j][st].z = pack_f16(St[j][8 * st + 4], St[j][8 * st + 5]); sop[j][st].w = pack_f16(St[j][8 * st + 6], St[j][8 * st + 7]);
            }
        // X = Kt S0^T : [64 tokens, 32 dv] (lane = dv), Y^T = S0 (diag(e^g) Q)^T : [32 dv, 64 tokens] (lane = token: the
        // operands swapped), so that an output row leaves as four neighbouring columns per store.  The next image's
        // loads go out between the MFMAs, one per pair: issued in one go they hold the wave for a microsecond.
        f32x16 X[2], Y[2];
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
#pragma unroll
            for (int i = 0; i < 16; i++) { X[tt][i] = 0.f; Y[tt][i] = 0.f; }
            const unsigned char* kr = im + Lay::oKt + (32 * tt + n32) * Lay::KP + 16 * half;
            const unsigned char* qr = im + Lay::oQh + (32 * tt + n32) * Lay::KP + 16 * half;
#pragma unroll
            for (int j = 0; j < JT; j++)
#pragma unroll
                for (int st = 0; st < 2; st++) {
                    const u32x4 ka = *reinterpret_cast<const u32x4*>(kr + 32 * (2 * j + st));
                    const u32x4 qa = *reinterpret_cast<const u32x4*>(qr + 32 * (2 * j + st));
                    X[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, ka), __builtin_bit_cast(f16x8, sop[j][st]), X[tt], 0, 0, 0);
                    Y[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, sop[j][st]), __builtin_bit_cast(f16x8, qa), Y[tt], 0, 0, 0);
                    if (more && (tt * JT + j) * 2 + st < NIMG) issue_one(c + 1, (c + 1) & 1, (tt * JT + j) * 2 + st);
                }
        }
#pragma unroll
        for (int k = 2 * JT * 2; k < NIMG; k++) // (more loads than MFMA pairs: the rest goes out here)
            if (more) issue_one(c + 1, (c + 1) & 1, k);
        // W^T = Vt - X, as B operands (token axis in slot order by construction)
        u32x4 wop[2][2];
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int st = 0; st < 2; st++) {
                float w[8];
                vt_of(im, tt, st, w);
#pragma unroll
                for (int e = 0; e < 8; e++) w[e] -= X[tt][8 * st + e];
                wop[tt][st].x = pack_f16(w[0], w[1]); wop[tt][st].y = pack_f16(w[2], w[3]);
                wop[tt][st].z = pack_f16(w[4], w[5]); wop[tt][st].w = pack_f16(w[6], w[7]);
            }
        // O = Y + M W^T (M is lower triangular: tokens of tile 0 see only tile 0)
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            const unsigned char* mr = im + Lay::oM + (32 * tt + n32) * Lay::TP + 16 * half;
#pragma unroll
            for (int t2 = 0; t2 <= tt; t2++)
#pragma unroll
                for (int st = 0; st < 2; st++) {
                    const u32x4 ma = *reinterpret_cast<const u32x4*>(mr + 32 * (2 * t2 + st));
                    Y[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, wop[t2][st]), __builtin_bit_cast(f16x8, ma), Y[tt], 0, 0, 0);
                }
            // lane = token n32 of this tile; element i = column 32 wave + 8 (i / 4) + 4 half + i % 4.  The two lanes of a
            // token (half 0 and 1) swap two of their four 8-byte pieces so that each holds two whole 16-byte pieces:
            // half as many store instructions, and the address unit works through a store per lane and instruction.
            {
                u32x2 w[4];
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float o[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) o[e] = fminf(fmaxf(Y[tt][4 * g + e], -65504.0f), 65504.0f); // saturating: an overflow must not become inf
                    w[g].x = pack_f16(o[0], o[1]); w[g].y = pack_f16(o[2], o[3]);
                }
                // half 0 keeps pieces g = 0, 2 (and gets the partner's upper halves of them), half 1 keeps g = 1, 3
                u32x2 give[2], got[2];
                give[0] = half ? w[0] : w[1]; give[1] = half ? w[2] : w[3];
#pragma unroll
                for (int k = 0; k < 2; k++) {
                    got[k].x = (uint32_t)__shfl_xor((int)give[k].x, 32, 64);
                    got[k].y = (uint32_t)__shfl_xor((int)give[k].y, 32, 64);
                }
                if (n32 < len - (c * GD_C + 32 * tt)) {
                    f16_t* orow = (f16_t*)P.Amix + (size_t)(row0 + c * GD_C + 32 * tt + n32) * P.aLd + h * DV + 32 * wave + 8 * half;
#pragma unroll
                    for (int k = 0; k < 2; k++) { // columns 16 k + 8 half .. + 7: lower four from the half-0 lane, upper four from the half-1 lane
                        const u32x2 mine = w[2 * k + half];
                        u32x4 v;
                        v.x = half ? got[k].x : mine.x; v.y = half ? got[k].y : mine.y;
                        v.z = half ? mine.x : got[k].x; v.w = half ? mine.y : got[k].y;
                        *reinterpret_cast<u32x4*>(orow + 16 * k) = v;
                    }
                }
            }
        }
        // S^T <- e^{g_C} S^T + Kh^T W^T
#pragma unroll
        for (int j = 0; j < JT; j++) {
#pragma unroll
            for (int i = 0; i < 16; i++) St[j][i] *= gC;
            const unsigned char* hr = im + Lay::oKhT + (32 * j + n32) * Lay::TP + 16 * half;
#pragma unroll
            for (int t2 = 0; t2 < 2; t2++)
#pragma unroll
                for (int st = 0; st < 2; st++) {
                    const u32x4 ha = *reinterpret_cast<const u32x4*>(hr + 32 * (2 * t2 + st));
                    St[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, ha), __builtin_bit_cast(f16x8, wop[t2][st]), St[j], 0, 0, 0);
                }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);              // vmcnt(0): the next chunk's image has landed -- as a builtin, so that
        asm volatile("" ::: "memory");                   // the compiler knows and does not wait again among the next loads
        __syncthreads();                                  // ... for every wave; everyone is done with this image
    }
#pragma unroll
    for (int j = 0; j < JT; j++)
#pragma unroll
        for (int i = 0; i < 16; i++) Sg[(size_t)dv * DK + 32 * j + 8 * (i >> 2) + 4 * half + (i & 3)] = St[j][i];
}

// e[row][j] = silu(ple gate output) * P[tok][j], appended to the row of the mixing output
template <typename WT, typename AT>
__global__ void k_pf_ple(PfArgs P, LayerDev L) {
    const int row = blockIdx.x, j = threadIdx.x;
    if (j >= P.a.ple) return;
    const float g = P.QKV[(size_t)row * P.qkvLd + L.offPle + j];
    put<AT>((AT*)P.Amix + (size_t)row * P.aLd + L.ad + j, pf_silu(g) * getw<WT>((const WT*)L.pleTable + (size_t)P.ids[row] * P.a.ple + j));
}

// residual of the last row of every segment -> decode slot buffer x[slot]
__global__ void k_pf_gather_last(PfArgs P) {
    const int seg = blockIdx.y, i = blockIdx.x * PWG + threadIdx.x;
    if (i >= P.a.dim) return;
    const int row = P.segStart[seg] + P.segLen[seg] - 1;
    P.a.x[(size_t)seg * P.a.dim + i] = P.X[(size_t)row * P.a.dim + i];
}

// argmax over the LM-head partials of every segment's last row; sequence lengths advance by the segment length
__global__ void __launch_bounds__(PWG) k_pf_finish(PfArgs P, int nparts, int* tokOut) {
    __shared__ float sv[PWG];
    __shared__ int si[PWG];
    const StepArgs& a = P.a;
    const int tid = threadIdx.x;
    for (int seg = 0; seg < P.nseg; seg++) {
        float v = -3.0e38f;
        int idx = 0x7fffffff;
        for (int i = tid; i < nparts; i += PWG) {
            const float v2 = a.amaxVal[(size_t)seg * a.amaxParts + i];
            const int i2 = a.amaxIdx[(size_t)seg * a.amaxParts + i];
            if (v2 > v || (v2 == v && i2 < idx)) { v = v2; idx = i2; }
        }
        sv[tid] = v; si[tid] = idx;
        __syncthreads();
        for (int s = PWG / 2; s > 0; s >>= 1) {
            if (tid < s && (sv[tid + s] > sv[tid] || (sv[tid + s] == sv[tid] && si[tid + s] < si[tid]))) { sv[tid] = sv[tid + s]; si[tid] = si[tid + s]; }
            __syncthreads();
        }
        if (tid == 0) {
            int nxt = si[0];
            if (nxt < 0 || nxt >= a.vocab) nxt = 0;
            const int seq = P.segSeq[seg];
            tokOut[seg] = nxt;
            a.nextTok[seq] = nxt;
            a.pos[seq] += P.segLen[seg];
        }
        __syncthreads();
    }
}

// Row-wise softmax over the vocabulary (inference.cu:293-362) and the cross-entropy of the next token:
// probs[row] = softmax(logits[row]); nll[row] = -log max(probs[row][target[row]], 1e-4), the clamp of
// training_orchestrator.cu:343-347 (target < 0: none).
__global__ void __launch_bounds__(PWG) k_pf_softmax_rows(const float* logits, float* probs, const int* target, float* nll, int V) {
    __shared__ float red[PWG / 64];
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* lg = logits + (size_t)row * V;
    float m = -3.0e38f;
    for (int i = tid; i < V; i += PWG) m = fmaxf(m, lg[i]);
    m = pf_wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float sum = 0.f;
    for (int i = tid; i < V; i += PWG) sum += expf(lg[i] - m);
    sum = pf_wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    sum = (red[0] + red[1]) + (red[2] + red[3]);
    if (probs) {
        float* pr = probs + (size_t)row * V;
        for (int i = tid; i < V; i += PWG) pr[i] = expf(lg[i] - m) / sum;
    }
    if (nll && tid == 0) {
        const int t = target[row];
        nll[row] = t >= 0 ? -logf(fmaxf(expf(lg[t] - m) / sum, 0.0001f)) : 0.f;
    }
}

int mlh_launch_softmax_rows(mlh_ctx* c, const float* logits, float* probs, const int* target, float* nll, int rows) {
    hipLaunchKernelGGL(k_pf_softmax_rows, dim3(rows), dim3(PWG), 0, c->stream, logits, probs, target, nll, c->hp.vocabSize);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { c->err = std::string("softmax launch: ") + hipGetErrorString(e); return -2; }
    return 0;
}

// ----------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------
static int cdiv(int a, int b) { return (a + b - 1) / b; }

bool mlh_prefill_gemm_supported(const mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    const int esz = c->wbytes, kmul = 128 / esz;
    if (hp.dim % kmul || hp.ffnDim % kmul || (hp.pleDim && hp.pleDim % kmul)) return false;
    for (const LayerDev& L : c->layers)
        if (L.ad % kmul) return false;
    return true;
}

// ---- fp16 operands of the MFMA path for bf16 models ----
// A bf16 value has 8 significand bits, an IEEE half 11: scaled by a power of two that brings the
// matrix's largest magnitude just under the half range, every weight down to 2^-29 of that maximum
// converts exactly, so the MFMA path multiplies the very bf16-rounded weights the GEMV path reads --
// but against activations that keep 11 significand bits instead of 8.  (Accumulation is fp32 either way.)
__global__ void k_absmax_bf16(const bf16_t* __restrict__ w, size_t n, unsigned* out) {
    unsigned m = 0;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) m = max(m, (unsigned)(w[i] & 0x7fffu));
    for (int o = 32; o > 0; o >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, o, 64));
    if ((threadIdx.x & 63) == 0 && m) atomicMax(out, m);
}
__global__ void k_bf16_to_f16(const bf16_t* __restrict__ w, f16_t* __restrict__ out, size_t n, float scale, unsigned* inexact) {
    unsigned bad = 0;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float v = __uint_as_float(((uint32_t)w[i]) << 16) * scale;
        const _Float16 h = (_Float16)v;
        out[i].bits = __builtin_bit_cast(uint16_t, h);
        bad += ((float)h != v);
    }
    if (bad) atomicAdd(inexact, bad);
}

static int build_mirror(mlh_ctx* c, const void* src, size_t n, const void** dst, float* alpha, unsigned* d_scratch) {
    void* buf = nullptr;
    MLH_CHECK(c, hipMalloc(&buf, n * 2));
    c->mirrorAllocs.push_back(buf);
    MLH_CHECK(c, hipMemsetAsync(d_scratch, 0, 8, c->stream));
    hipLaunchKernelGGL(k_absmax_bf16, dim3(1024), dim3(256), 0, c->stream, (const bf16_t*)src, n, d_scratch);
    unsigned h[2] = {0, 0};
    MLH_CHECK(c, hipMemcpyAsync(h, d_scratch, 4, hipMemcpyDeviceToHost, c->stream));
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    // largest magnitude = bf16 bits h[0]; its exponent e (unbiased): scale 2^(14 - e) puts it in [2^14, 2^15)
    const int e = (int)((h[0] >> 7) & 0xff) - 127;
    const int k = h[0] ? 14 - e : 0;
    const float scale = ldexpf(1.0f, k);
    hipLaunchKernelGGL(k_bf16_to_f16, dim3(1024), dim3(256), 0, c->stream, (const bf16_t*)src, (f16_t*)buf, n, scale, d_scratch + 1);
    MLH_CHECK(c, hipMemcpyAsync(h, d_scratch, 8, hipMemcpyDeviceToHost, c->stream));
    MLH_CHECK(c, hipStreamSynchronize(c->stream));
    c->f16Inexact += h[1];
    *dst = buf;
    *alpha = ldexpf(1.0f, -k);
    return 0;
}

int mlh_build_gemm_operands(mlh_ctx* c) {
    const mlh_hparams& hp = c->hp;
    const bool mirror = hp.weightDtype == MLH_DTYPE_BF16 && mlh_prefill_gemm_supported(c);
    c->gemmDtype = mirror ? MLH_GEMM_F16 : hp.weightDtype;
    c->f16Inexact = 0;
    for (void* p : c->mirrorAllocs) (void)hipFree(p); // a repeated finalize rebuilds them
    c->mirrorAllocs.clear();
    unsigned* d_scratch = nullptr;
    if (mirror) { MLH_CHECK(c, hipMalloc((void**)&d_scratch, 8)); }
    int rc = 0;
    const size_t d = hp.dim, F = hp.ffnDim, pl = hp.pleDim, wb = c->wbytes;
    for (LayerDev& L : c->layers) {
        L.WaG = L.Wa; L.WoG = L.Wo; L.W13G = L.W13; L.W2G = L.W2;
        L.sWa = L.sWo = L.sW13 = L.sW2 = 1.0f;
        const void* wo = L.Wo;
        if (pl > 0) { // [Wo | pleUp] along K, in the storage type
            void* cat = nullptr;
            MLH_CHECK(c, hipMalloc(&cat, d * (L.ad + pl) * wb));
            c->mirrorAllocs.push_back(cat);
            MLH_CHECK(c, hipMemcpy2D(cat, (L.ad + pl) * wb, L.Wo, L.ad * wb, L.ad * wb, d, hipMemcpyDeviceToDevice));
            MLH_CHECK(c, hipMemcpy2D((char*)cat + L.ad * wb, (L.ad + pl) * wb, L.pleUp, pl * wb, pl * wb, d, hipMemcpyDeviceToDevice));
            wo = cat;
            L.WoG = cat;
        }
        if (!mirror) continue;
        if ((rc = build_mirror(c, L.Wa, (size_t)L.rowsA * d, &L.WaG, &L.sWa, d_scratch)) ||
            (rc = build_mirror(c, wo, d * (L.ad + pl), &L.WoG, &L.sWo, d_scratch)) ||
            (rc = build_mirror(c, L.W13, 2 * F * d, &L.W13G, &L.sW13, d_scratch)) ||
            (rc = build_mirror(c, L.W2, d * F, &L.W2G, &L.sW2, d_scratch)))
            break;
    }
    c->EG = c->E; c->sE = 1.0f;
    if (rc == 0 && mirror) rc = build_mirror(c, c->E, (size_t)hp.vocabSize * hp.dim, &c->EG, &c->sE, d_scratch);
    if (d_scratch) (void)hipFree(d_scratch);
    return rc;
}

// The headDim-128 attention tiles exceed the 64 KB a launch may use without opting in.
static size_t gdn_prep_lds(int dk) { return ((size_t)GD_C * GD_C + 12 * GD_C) * 4 + (size_t)2 * GD_C * (dk + 8) * 2 + (size_t)dk * (GD_C + 8) * 2; }

int mlh_init_prefill_kernels(mlh_ctx* c) {
    MLH_CHECK(c, hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gdn_prep<64>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)gdn_prep_lds(64)));
    MLH_CHECK(c, hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gdn_prep<128>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)gdn_prep_lds(128)));
    MLH_CHECK(c, hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gdn_scan<64>), hipFuncAttributeMaxDynamicSharedMemorySize, 2 * GdLayout<64>::image));
    MLH_CHECK(c, hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gdn_scan<128>), hipFuncAttributeMaxDynamicSharedMemorySize, 2 * GdLayout<128>::image));
    const int lds = (2 * 64 * 132 + PF_QB * 128) * 4;
    MLH_CHECK(c, hipFuncSetAttribute(reinterpret_cast<const void*>(&k_pf_attn<128, float>), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    return 0;
}

static int ensure_prefill_buffers(mlh_ctx* c, int rows) {
    if (rows <= c->pfRows) return 0;
    const mlh_hparams& hp = c->hp;
    (void)hipStreamSynchronize(c->stream);
    for (void* p : c->pfAllocs) (void)hipFree(p);
    c->pfAllocs.clear();
    c->pfRows = 0;
    for (int g = 0; g < 2; g++) // captured batched steps hold the old buffer addresses
        if (c->graphExec[g]) { (void)hipGraphExecDestroy(c->graphExec[g]); c->graphExec[g] = nullptr; }
    const size_t n = (size_t)rows, wb = c->wbytes;
    auto alloc = [&](void** p, size_t bytes) -> int {
        MLH_CHECK(c, hipMalloc(p, std::max<size_t>(bytes, 16)));
        c->pfAllocs.push_back(*p);
        return 0;
    };
    int rc;
    const int nblk = cdiv(rows, PF_QB) + hp.maxSeqs, nchunk = cdiv(rows, GD_C) + hp.maxSeqs;
    if ((rc = alloc((void**)&c->pfX, n * hp.dim * 4)) || (rc = alloc(&c->pfXn, n * hp.dim * wb)) ||
        (rc = alloc((void**)&c->pfQKV, n * c->maxRowsA * 4)) || (rc = alloc(&c->pfA, n * (c->maxAd + hp.pleDim) * wb)) ||
        (rc = alloc((void**)&c->pfH1, n * hp.dim * 4)) ||
        (rc = alloc(&c->pfU, n * hp.ffnDim * wb)) ||
        (hp.weightDtype == MLH_DTYPE_BF16 && ((rc = alloc((void**)&c->pfKh, n * hp.dim * 2)) || (rc = alloc((void**)&c->pfVh, n * hp.dim * 2)))) ||
        (rc = alloc((void**)&c->pfMeta, (3 * n + 4 * (size_t)hp.maxSeqs + 2 * (size_t)nblk + 2 * (size_t)nchunk + hp.maxSeqs) * 4)))
        return rc;
    c->pfRows = rows;
    c->pfBlkCap = nblk;
    c->pfChunkCap = nchunk;
    return 0;
}

#define PF_DISPATCH_WT(c, expr_f32, expr_bf16) do { if ((c)->hp.weightDtype == MLH_DTYPE_BF16) { expr_bf16; } else { expr_f32; } } while (0)

// Appends lens[s] tokens to sequence seqs[s] for every segment s (token ids concatenated in `ids`).
// allLogits: null, or a device buffer [rows, vocab] that receives the logits of every position.
int mlh_run_prefill_gemm(mlh_ctx* c, int nseg, const int32_t* seqs, const int32_t* ids, const int32_t* lens, float* allLogits) {
    const mlh_hparams& hp = c->hp;
    int n = 0;
    for (int s = 0; s < nseg; s++) n += lens[s];
    int rc = ensure_prefill_buffers(c, n);
    if (rc) return rc;
    // ---- metadata ----
    const bool mfmaAttn = hp.weightDtype == MLH_DTYPE_BF16; // bf16 models: bf16 MFMA attention, 128 queries per workgroup
    const int qb = mfmaAttn ? PF_MQB : PF_QB;
    std::vector<int> rowSeq(n), rowPos(n), segStart(nseg), segPos0(nseg), blkSeg, blkQ0, chunkSeg, chunkT0, chunkBase(nseg, 0);
    bool anyGdn = false;
    for (const LayerDev& L : c->layers) anyGdn = anyGdn || L.kind == MLH_KIND_GDN;
    const bool gdnChunked = anyGdn && c->gemmDtype == MLH_GEMM_F16; // segments of 64 tokens or more: chunk-parallel MFMA path
    int r = 0;
    for (int s = 0; s < nseg; s++) {
        segStart[s] = r;
        segPos0[s] = c->h_len[seqs[s]];
        for (int i = 0; i < lens[s]; i++, r++) { rowSeq[r] = seqs[s]; rowPos[r] = segPos0[s] + i; }
        for (int q0 = 0; q0 < lens[s]; q0 += qb) { blkSeg.push_back(s); blkQ0.push_back(q0); }
        chunkBase[s] = (int)chunkSeg.size();
        if (gdnChunked && lens[s] >= GD_C)
            for (int t0 = 0; t0 < lens[s]; t0 += GD_C) { chunkSeg.push_back(s); chunkT0.push_back(t0); }
    }
    const int nblk = (int)blkSeg.size(), nchunk = (int)chunkSeg.size();
    if (nblk > c->pfBlkCap) { c->err = "prefill: too many attention blocks"; return -1; }
    if (nchunk > 0) {
        const size_t per = (size_t)hp.gdnHeads * (hp.gdnDk == 64 ? GdLayout<64>::total : GdLayout<128>::total);
        if ((size_t)nchunk > c->pfGdnChunks) {
            MLH_CHECK(c, hipStreamSynchronize(c->stream));
            if (c->pfGdnWs) { (void)hipFree(c->pfGdnWs); (void)hipFree(c->pfGdnG); c->pfGdnWs = nullptr; c->pfGdnG = nullptr; c->pfGdnChunks = 0; }
            MLH_CHECK(c, hipMalloc(&c->pfGdnWs, (size_t)nchunk * per));
            MLH_CHECK(c, hipMalloc((void**)&c->pfGdnG, (size_t)nchunk * hp.gdnHeads * 4));
            c->pfGdnChunks = nchunk;
        }
    }
    int* d = c->pfMeta;
    int* d_ids = d; int* d_rowSeq = d + n; int* d_rowPos = d + 2 * n;
    int* d_seg = d + 3 * n; // segStart, segLen, segSeq, segPos0 (maxSeqs each)
    int* d_blk = d_seg + 4 * hp.maxSeqs;
    int* d_chunk = d_blk + 2 * c->pfBlkCap; // chunkSeg, chunkT0 (pfChunkCap each), chunkBase (maxSeqs)
    hipStream_t st = c->stream;
    MLH_CHECK(c, hipMemcpyAsync(d_ids, ids, (size_t)n * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_rowSeq, rowSeq.data(), (size_t)n * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_rowPos, rowPos.data(), (size_t)n * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_seg, segStart.data(), (size_t)nseg * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_seg + hp.maxSeqs, lens, (size_t)nseg * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_seg + 2 * hp.maxSeqs, seqs, (size_t)nseg * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_seg + 3 * hp.maxSeqs, segPos0.data(), (size_t)nseg * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_blk, blkSeg.data(), (size_t)nblk * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipMemcpyAsync(d_blk + c->pfBlkCap, blkQ0.data(), (size_t)nblk * 4, hipMemcpyHostToDevice, st));
    if (nchunk > 0) {
        if (nchunk > c->pfChunkCap) { c->err = "prefill: too many GDN chunks"; return -1; }
        MLH_CHECK(c, hipMemcpyAsync(d_chunk, chunkSeg.data(), (size_t)nchunk * 4, hipMemcpyHostToDevice, st));
        MLH_CHECK(c, hipMemcpyAsync(d_chunk + c->pfChunkCap, chunkT0.data(), (size_t)nchunk * 4, hipMemcpyHostToDevice, st));
        MLH_CHECK(c, hipMemcpyAsync(d_chunk + 2 * c->pfChunkCap, chunkBase.data(), (size_t)nseg * 4, hipMemcpyHostToDevice, st));
    }
    MLH_CHECK(c, hipMemcpyAsync(c->d_sidx, seqs, (size_t)nseg * 4, hipMemcpyHostToDevice, st));
    MLH_CHECK(c, hipStreamSynchronize(st)); // the host vectors above go out of scope
    c->identityNseq = 0;

    PfArgs P;
    mlh_fill_args(c, P.a, nseg, c->d_tok);
    P.n = n; P.nseg = nseg; P.ids = d_ids; P.rowSeq = d_rowSeq; P.rowPos = d_rowPos;
    P.segStart = d_seg; P.segLen = d_seg + hp.maxSeqs; P.segSeq = d_seg + 2 * hp.maxSeqs; P.segPos0 = d_seg + 3 * hp.maxSeqs;
    P.blkSeg = d_blk; P.blkQ0 = d_blk + c->pfBlkCap;
    P.X = c->pfX; P.Xn = c->pfXn; P.QKV = c->pfQKV; P.qkvLd = c->maxRowsA; P.Amix = c->pfA; P.aLd = c->maxAd + hp.pleDim;
    P.H1 = c->pfH1; P.U = c->pfU;
    bool fresh = true; // every segment starts its sequence: all keys of the call are rows of the call
    for (int s = 0; s < nseg; s++) fresh = fresh && segPos0[s] == 0;
    P.Kh = mfmaAttn && fresh ? c->pfKh : nullptr;
    P.Vh = mfmaAttn && fresh ? c->pfVh : nullptr;
    const int d_ = hp.dim, F = hp.ffnDim, dt = c->gemmDtype;
#define GEMM(A, lda, B, alpha, ldb, C, ldc, R, ldr, M, N, K)                                                \
    do {                                                                                                    \
        hipError_t e_ = mlh_gemm_tn_epi(st, dt, 0, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, nullptr, alpha); \
        if (e_ != hipSuccess) { c->err = std::string("prefill GEMM: ") + hipGetErrorString(e_); return -2; } \
    } while (0)

    PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_embed<float>), dim3(cdiv(d_, PWG), n), dim3(PWG), 0, st, P),
                   hipLaunchKernelGGL((k_pf_embed<bf16_t>), dim3(cdiv(d_, PWG), n), dim3(PWG), 0, st, P));
    for (int t = hp.transformers - 1; t >= 0; t--) { // file block 0 is the top (inference.cu:384-385)
        const LayerDev& L = c->layers[t];
        PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_rmsnorm<float>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, P.X, L.g1, (float*)P.Xn, n, d_),
                       hipLaunchKernelGGL((k_pf_rmsnorm<f16_t>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, P.X, L.g1, (f16_t*)P.Xn, n, d_));
        GEMM(P.Xn, d_, L.WaG, L.sWa, d_, P.QKV, P.qkvLd, nullptr, 0, n, L.rowsA, d_);
        if (L.kind == MLH_KIND_ATTENTION) {
            if (hp.headDim == 64) {
                hipLaunchKernelGGL((k_pf_qk_rope_kv<64>), dim3(hp.attnHeads, n), dim3(64), 0, st, P, L);
                if (mfmaAttn && P.Kh) hipLaunchKernelGGL((k_pf_attn_mfma<64, true>), dim3(hp.attnHeads, nblk), dim3(PWG), 0, st, P, L);
                else if (mfmaAttn) hipLaunchKernelGGL((k_pf_attn_mfma<64, false>), dim3(hp.attnHeads, nblk), dim3(PWG), 0, st, P, L);
                else hipLaunchKernelGGL((k_pf_attn<64, float>), dim3(hp.attnHeads, nblk), dim3(PWG), (size_t)(2 * 64 * 68 + PF_QB * 64) * 4, st, P, L);
            } else {
                hipLaunchKernelGGL((k_pf_qk_rope_kv<128>), dim3(hp.attnHeads, n), dim3(64), 0, st, P, L);
                if (mfmaAttn && P.Kh) hipLaunchKernelGGL((k_pf_attn_mfma<128, true>), dim3(hp.attnHeads, nblk), dim3(PWG), 0, st, P, L);
                else if (mfmaAttn) hipLaunchKernelGGL((k_pf_attn_mfma<128, false>), dim3(hp.attnHeads, nblk), dim3(PWG), 0, st, P, L);
                else hipLaunchKernelGGL((k_pf_attn<128, float>), dim3(hp.attnHeads, nblk), dim3(PWG), (size_t)(2 * 64 * 132 + PF_QB * 128) * 4, st, P, L);
            }
        } else {
            const int skipFrom = nchunk > 0 ? GD_C : 0x7fffffff;
            const dim3 gr(hp.gdnHeads, nseg, hp.gdnDv / PF_GR);
            if (hp.gdnDk == 64) {
                PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_gdn<64, float>), gr, dim3(PWG), 0, st, P, L, skipFrom),
                               hipLaunchKernelGGL((k_pf_gdn<64, f16_t>), gr, dim3(PWG), 0, st, P, L, skipFrom));
            } else {
                PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_gdn<128, float>), gr, dim3(PWG), 0, st, P, L, skipFrom),
                               hipLaunchKernelGGL((k_pf_gdn<128, f16_t>), gr, dim3(PWG), 0, st, P, L, skipFrom));
            }
            if (nchunk > 0) {
                const int* dcs = d_chunk; const int* dct = d_chunk + c->pfChunkCap; const int* dcb = d_chunk + 2 * c->pfChunkCap;
                if (hp.gdnDk == 64) {
                    hipLaunchKernelGGL((k_gdn_prep<64>), dim3(nchunk, hp.gdnHeads), dim3(128), gdn_prep_lds(64), st, P, L, dcs, dct, (unsigned char*)c->pfGdnWs, c->pfGdnG);
                    hipLaunchKernelGGL((k_gdn_scan<64>), dim3(hp.gdnHeads, nseg), dim3(128), (size_t)2 * GdLayout<64>::image, st, P, L, dcb, (const unsigned char*)c->pfGdnWs, c->pfGdnG);
                } else {
                    hipLaunchKernelGGL((k_gdn_prep<128>), dim3(nchunk, hp.gdnHeads), dim3(256), gdn_prep_lds(128), st, P, L, dcs, dct, (unsigned char*)c->pfGdnWs, c->pfGdnG);
                    hipLaunchKernelGGL((k_gdn_scan<128>), dim3(hp.gdnHeads, nseg), dim3(256), (size_t)2 * GdLayout<128>::image, st, P, L, dcb, (const unsigned char*)c->pfGdnWs, c->pfGdnG);
                }
            }
        }
        if (hp.pleDim > 0)
            PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_ple<float, float>), dim3(n), dim3(std::max(64, hp.pleDim)), 0, st, P, L),
                           hipLaunchKernelGGL((k_pf_ple<bf16_t, f16_t>), dim3(n), dim3(std::max(64, hp.pleDim)), 0, st, P, L));
        GEMM(P.Amix, P.aLd, L.WoG, L.sWo, L.ad + hp.pleDim, P.H1, d_, P.X, d_, n, d_, L.ad + hp.pleDim); // Wo . a + pleUp . e + x
        PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_rmsnorm<float>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, P.H1, L.g2, (float*)P.Xn, n, d_),
                       hipLaunchKernelGGL((k_pf_rmsnorm<f16_t>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, P.H1, L.g2, (f16_t*)P.Xn, n, d_));
        { // gate/up projection with SiLU(gate) * up in the epilogue (inference.cu:262-281): U comes out in the GEMM input type
            hipError_t e_ = mlh_gemm_tn_epi(st, dt, 1, P.Xn, d_, L.W13G, d_, P.U, F, nullptr, 0, n, 2 * F, d_, nullptr, L.sW13);
            if (e_ != hipSuccess) { c->err = std::string("prefill GEMM: ") + hipGetErrorString(e_); return -2; }
        }
        GEMM(P.U, F, L.W2G, L.sW2, F, P.X, d_, P.H1, d_, n, d_, F);
    }
#undef GEMM
    if (allLogits) { // final RMSNorm + tied LM head for every row (inference.cu:705-743 computes all L columns)
        PF_DISPATCH_WT(c, hipLaunchKernelGGL((k_pf_rmsnorm<float>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, P.X, c->gF, (float*)P.Xn, n, d_),
                       hipLaunchKernelGGL((k_pf_rmsnorm<f16_t>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, P.X, c->gF, (f16_t*)P.Xn, n, d_));
        hipError_t e_ = mlh_gemm_tn_epi(st, dt, 0, P.Xn, d_, c->EG, d_, allLogits, hp.vocabSize, nullptr, 0, n, hp.vocabSize, d_, nullptr, c->sE);
        if (e_ != hipSuccess) { c->err = std::string("prefill GEMM: ") + hipGetErrorString(e_); return -2; }
    }
    hipLaunchKernelGGL(k_pf_gather_last, dim3(cdiv(d_, PWG), nseg), dim3(PWG), 0, st, P);
    if ((rc = mlh_launch_one(c, MLH_K_LMHEAD, 0, nseg))) return rc;
    hipLaunchKernelGGL(k_pf_finish, dim3(1), dim3(PWG), 0, st, P, c->amaxParts, c->d_tok);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { c->err = std::string("prefill launch: ") + hipGetErrorString(e); return -2; }
    MLH_CHECK(c, hipStreamSynchronize(st));
    for (int s = 0; s < nseg; s++) c->h_len[seqs[s]] += lens[s];
    return 0;
}

// ----------------------------------------------------------------------------
// Batched decode step (8 or more sequences, one new token each): the same row pipeline with the
// skinny MFMA GEMM -- every weight matrix is streamed once per step whatever the batch size -- and
// the decode path's own attention / GDN kernels, whose split-KV partials are combined here.
// Everything stays on the device and on the stream (no allocation, no host round trip), so a
// step can be captured into a graph like the GEMV step.
// ----------------------------------------------------------------------------
#define MLH_BATCH_GEMM_MIN_SEQS 8

template <typename WT>
__global__ void k_bd_embed(StepArgs a) {
    const int slot = blockIdx.y, i = blockIdx.x * PWG + threadIdx.x;
    if (slot == 0 && i == 0) *a.stepCounter += 1; // steps started; k_bd_finish logs into row (counter - 1)
    if (i >= a.dim) return;
    a.x[(size_t)slot * a.dim + i] = getw<WT>((const WT*)a.E + (size_t)a.tok[slot] * a.dim + i);
}

// Mixing output rows in the GEMM input type: attention layers combine the split-KV partials of the decode
// attention kernel and apply the sigmoid gate (inference.cu:241-250); GDN layers convert the read-out.
// PLE rows e = silu(gate) * P[tok] are appended to the row (column L.ad on).
template <typename WT, typename AT>
__global__ void __launch_bounds__(PWG) k_bd_mix(StepArgs a, LayerDev L, AT* Amix, int aLd) {
    const int slot = blockIdx.x, tid = threadIdx.x;
    const float* qkv = a.qkv + (size_t)slot * a.qkvStride;
    // the row is dealt to the gridDim.y workgroups of the slot in contiguous pieces (one workgroup per slot would
    // walk every head's partials alone)
    const int piece = (L.ad + (int)gridDim.y - 1) / (int)gridDim.y, i0 = (int)blockIdx.y * piece, i1 = min(L.ad, i0 + piece);
    if (L.kind == MLH_KIND_ATTENTION) {
        const int hd = a.hd;
        for (int i = i0 + tid; i < i1; i += PWG) {
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
            float v = num / den;
            if (a.gating) v = v * pf_sigmoid(qkv[L.offG + i]);
            put<AT>(Amix + (size_t)slot * aLd + i, v);
        }
    } else {
        for (int i = i0 + tid; i < i1; i += PWG) put<AT>(Amix + (size_t)slot * aLd + i, a.mix[(size_t)slot * L.ad + i]);
    }
    if (blockIdx.y == 0)
        for (int j = tid; j < a.ple; j += PWG)
        put<AT>(Amix + (size_t)slot * aLd + L.ad + j, pf_silu(qkv[L.offPle + j]) * getw<WT>((const WT*)L.pleTable + (size_t)a.tok[slot] * a.ple + j));
}

// One workgroup per slot: argmax of the slot's logits (lowest index on ties), logits copied to the
// sequence's row, bookkeeping of k_finish (next token, id log, position).
__global__ void __launch_bounds__(PWG) k_bd_finish(StepArgs a, const float* lg, int* tokOut) {
    __shared__ float sv[PWG];
    __shared__ int si[PWG];
    __shared__ double sd[PWG + 1];
    const int slot = blockIdx.x, tid = threadIdx.x, seq = a.sidx[slot];
    const float* row = lg + (size_t)slot * a.vocab;
    float* dst = a.logits + (size_t)seq * a.vocab;
    if (a.temperature > 0.f) { // draw instead of argmax
        for (int i = tid; i < a.vocab; i += PWG) dst[i] = row[i];
        const int nxt = mlh_sample_row<PWG>(row, a.vocab, a.temperature, mlh_sample_uniform(a.sampleSeed, seq, a.pos[seq] + 1), sd, si);
        __syncthreads();
        if (tid == 0) {
            const int step = *a.stepCounter - 1;
            tokOut[slot] = nxt;
            a.nextTok[seq] = nxt;
            if (step >= 0 && step < a.outCapacity) a.outIds[(size_t)step * a.nseq + slot] = nxt;
            a.pos[seq] += 1;
        }
        return;
    }
    float v = -3.0e38f;
    int idx = 0x7fffffff;
    if ((a.vocab & 3) == 0) { // 16 bytes per lane, four loads in flight before the first store (row and dst do not overlap)
        const f32x4* row4 = reinterpret_cast<const f32x4*>(row);
        f32x4* dst4 = reinterpret_cast<f32x4*>(dst);
        const int n4 = a.vocab >> 2;
        for (int i0 = tid; i0 < n4; i0 += 4 * PWG) {
            f32x4 x[4];
#pragma unroll
            for (int k = 0; k < 4; k++) x[k] = row4[min(i0 + k * PWG, n4 - 1)];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int i = i0 + k * PWG;
                if (i < n4) {
                    dst4[i] = x[k];
                    // i ascends per thread and the four elements are taken in order: ties keep the lower index
                    if (x[k].x > v) { v = x[k].x; idx = 4 * i; }
                    if (x[k].y > v) { v = x[k].y; idx = 4 * i + 1; }
                    if (x[k].z > v) { v = x[k].z; idx = 4 * i + 2; }
                    if (x[k].w > v) { v = x[k].w; idx = 4 * i + 3; }
                }
            }
        }
    } else {
        for (int i = tid; i < a.vocab; i += PWG) {
            const float x = row[i];
            dst[i] = x;
            if (x > v) { v = x; idx = i; } // i ascends: ties keep the lower index
        }
    }
    sv[tid] = v; si[tid] = idx;
    __syncthreads();
    for (int s = PWG / 2; s > 0; s >>= 1) {
        if (tid < s && (sv[tid + s] > sv[tid] || (sv[tid + s] == sv[tid] && si[tid + s] < si[tid]))) { sv[tid] = sv[tid + s]; si[tid] = si[tid + s]; }
        __syncthreads();
    }
    if (tid == 0) {
        int nxt = si[0];
        if (nxt < 0 || nxt >= a.vocab) nxt = 0;
        const int step = *a.stepCounter - 1;
        tokOut[slot] = nxt;
        a.nextTok[seq] = nxt;
        if (step >= 0 && step < a.outCapacity) a.outIds[(size_t)step * a.nseq + slot] = nxt;
        a.pos[seq] += 1;
    }
}

bool mlh_batch_step_applicable(const mlh_ctx* c, int nseq) {
    return c->prefillMode == 0 && nseq >= MLH_BATCH_GEMM_MIN_SEQS && nseq <= 64 && mlh_prefill_gemm_supported(c);
}

// Allocations the batched step needs; call outside graph capture.
int mlh_prepare_batch_step(mlh_ctx* c, int nseq) {
    if (!mlh_batch_step_applicable(c, nseq)) return 0;
    int rc = ensure_prefill_buffers(c, std::max(nseq, 64));
    if (rc) return rc;
    if (!c->gemmWs) {
        MLH_CHECK(c, hipMalloc(&c->gemmWs, mlh_gemm_workspace_bytes()));
        c->allocs.push_back(c->gemmWs);
        MLH_CHECK(c, hipMemset(c->gemmWs, 0, mlh_gemm_workspace_bytes()));
    }
    if (!c->pfLogits) {
        MLH_CHECK(c, hipMalloc((void**)&c->pfLogits, (size_t)64 * c->hp.vocabSize * 4));
        c->allocs.push_back(c->pfLogits);
    }
    return 0;
}

int mlh_launch_batch_step(mlh_ctx* c, int nseq, const int* tokPtr) {
    const mlh_hparams& hp = c->hp;
    if (c->pfRows < nseq || !c->pfLogits) { c->err = "batched step buffers not prepared"; return -1; }
    StepArgs a;
    mlh_fill_args(c, a, nseq, tokPtr);
    hipStream_t st = c->stream;
    const int d_ = hp.dim, F = hp.ffnDim, dt = c->gemmDtype, n = nseq;
    const bool bf = hp.weightDtype == MLH_DTYPE_BF16;
#define GEMMN(epi, A, lda, B, alpha, ldb, C, ldc, R, ldr, M, N, K, G)                                                 \
    do {                                                                                                            \
        hipError_t e_ = mlh_gemm_tn_epi(st, dt, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, c->gemmWs, alpha, G);  \
        if (e_ != hipSuccess) { c->err = std::string("batched step GEMM: ") + hipGetErrorString(e_); return -2; }    \
    } while (0)
#define GEMM(epi, A, lda, B, alpha, ldb, C, ldc, R, ldr, M, N, K) GEMMN(epi, A, lda, B, alpha, ldb, C, ldc, R, ldr, M, N, K, nullptr)
    if (bf) hipLaunchKernelGGL((k_bd_embed<bf16_t>), dim3(cdiv(d_, PWG), n), dim3(PWG), 0, st, a);
    else hipLaunchKernelGGL((k_bd_embed<float>), dim3(cdiv(d_, PWG), n), dim3(PWG), 0, st, a);
    for (int t = hp.transformers - 1; t >= 0; t--) {
        const LayerDev& L = c->layers[t];
        // (fp32, 33..64 sequences: the RMSNorm rides in the product, see mlh_gemm_norm_fusable)
        if (mlh_gemm_norm_fusable(dt, n, L.rowsA, d_)) {
            GEMMN(0, c->x, d_, L.WaG, L.sWa, d_, c->qkv, c->maxRowsA, nullptr, 0, n, L.rowsA, d_, L.g1);
        } else {
            if (bf) hipLaunchKernelGGL((k_pf_rmsnorm<f16_t>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, c->x, L.g1, (f16_t*)c->pfXn, n, d_);
            else hipLaunchKernelGGL((k_pf_rmsnorm<float>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, c->x, L.g1, (float*)c->pfXn, n, d_);
            GEMM(0, c->pfXn, d_, L.WaG, L.sWa, d_, c->qkv, c->maxRowsA, nullptr, 0, n, L.rowsA, d_);
        }
        const bool gdn = L.kind != MLH_KIND_ATTENTION;
        // The GDN kernel writes its read-out and the PLE columns straight into the GEMM's input rows (mlh_launch_one
        // reads the step's tokens from the context's own buffer, hence the second condition).
        // The attention kernel does the same when one workgroup holds all keys of a (head, sequence) pair.
        const bool direct = (gdn || c->nsplit == 1) && tokPtr == c->d_tok;
        if (direct) { c->mixRows = c->pfA; c->mixRowsLd = c->maxAd + hp.pleDim; c->mixRowsHalf = bf ? 1 : 0; }
        int rc = mlh_launch_one(c, gdn ? MLH_K_GDN : MLH_K_ATTN, t, nseq);
        c->mixRows = nullptr;
        if (rc) return rc;
        if (!direct) { // attention: combine the split-KV partials, gate; PLE columns
            const dim3 mg(n, std::max(1, (L.ad + PWG - 1) / PWG * (n <= 16 ? 4 : 1))); // few slots: more workgroups per row
            if (bf) hipLaunchKernelGGL((k_bd_mix<bf16_t, f16_t>), mg, dim3(PWG), 0, st, a, L, (f16_t*)c->pfA, c->maxAd + hp.pleDim);
            else hipLaunchKernelGGL((k_bd_mix<float, float>), mg, dim3(PWG), 0, st, a, L, (float*)c->pfA, c->maxAd + hp.pleDim);
        }
        GEMM(0, c->pfA, c->maxAd + hp.pleDim, L.WoG, L.sWo, L.ad + hp.pleDim, c->h1, d_, c->x, d_, n, d_, L.ad + hp.pleDim);
        if (mlh_gemm_norm_fusable(dt, n, 2 * F, d_)) {
            GEMMN(1, c->h1, d_, L.W13G, L.sW13, d_, c->pfU, F, nullptr, 0, n, 2 * F, d_, L.g2);
        } else {
            if (bf) hipLaunchKernelGGL((k_pf_rmsnorm<f16_t>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, c->h1, L.g2, (f16_t*)c->pfXn, n, d_);
            else hipLaunchKernelGGL((k_pf_rmsnorm<float>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, c->h1, L.g2, (float*)c->pfXn, n, d_);
            GEMM(1, c->pfXn, d_, L.W13G, L.sW13, d_, c->pfU, F, nullptr, 0, n, 2 * F, d_);
        }
        GEMM(0, c->pfU, F, L.W2G, L.sW2, F, c->x, d_, c->h1, d_, n, d_, F);
    }
    if (bf) hipLaunchKernelGGL((k_pf_rmsnorm<f16_t>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, c->x, c->gF, (f16_t*)c->pfXn, n, d_);
    else hipLaunchKernelGGL((k_pf_rmsnorm<float>), dim3(cdiv(n, 4)), dim3(PWG), 0, st, c->x, c->gF, (float*)c->pfXn, n, d_);
    GEMM(0, c->pfXn, d_, c->EG, c->sE, d_, c->pfLogits, hp.vocabSize, nullptr, 0, n, hp.vocabSize, d_);
#undef GEMM
#undef GEMMN
    hipLaunchKernelGGL(k_bd_finish, dim3(n), dim3(PWG), 0, st, a, c->pfLogits, c->d_tok);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { c->err = std::string("batched step launch: ") + hipGetErrorString(e); return -2; }
    return 0;
}
