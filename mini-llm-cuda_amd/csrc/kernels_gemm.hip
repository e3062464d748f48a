// MFMA GEMM for prefill and batched decode on gfx950:
//
//     C[M, N] = A[M, K] . B[N, K]^T  (+ R[M, N])        C, R fp32;  A and B both fp32 or both bf16
//
// A holds activations (one token per row), B a weight matrix in the checkpoint's row-major [out, in]
// order -- both operands are K-contiguous, which is what the MFMA operand layout wants: for the
// 32x32 tiles used here lane l supplies row (l % 32) and the K elements of half (l / 32), so a
// 16-byte piece of a row is one operand (eight bf16 for v_mfma_f32_32x32x16_bf16, or four floats
// feeding four v_mfma_f32_32x32x2_f32 steps).  This replaces the cublasGemmEx calls of
// inference.cu:401-465, 487-507, 582-602, 624-695 and 723-743 for L > 1 columns.
//
// Tiling: 128 x 128 output tile per 256-thread workgroup (2 x 2 waves of 64 x 64), K in slices of
// 128 bytes per row.  Slices go global -> registers -> LDS (rows padded to 144 bytes: conflict-free
// 16-byte reads), the next slice's global loads fly while the current one is multiplied.
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <string>

#include "mlh_internal.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define GKB 128           // bytes of K per row and slice
#define GLD 144           // padded LDS row pitch in bytes
#define GTHREADS 256

template <typename T> struct GemmTraits;
template <> struct GemmTraits<float> {
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x16& c) {
        // lanes of half 0 hold k = 8j..8j+3, half 1 holds k = 8j+4..8j+7: step s pairs k = 8j+s with 8j+4+s,
        // the same pairing in A and B, so every k is multiplied with itself exactly once
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
    }
    static __device__ __forceinline__ void put(float* p, float v) { *p = v; }
    static __device__ __forceinline__ uint32_t bits(float v) { return __float_as_uint(v); }
};
template <> struct GemmTraits<bf16_t> {
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t bits(float v) {
        const uint32_t u = __float_as_uint(v);
        return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    }
    static __device__ __forceinline__ void put(bf16_t* p, float v) { *p = (bf16_t)bits(v); }
};

template <> struct GemmTraits<f16_t> {
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t bits(float v) { // saturating: an overflow must not become inf
        const _Float16 h = (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f);
        return __builtin_bit_cast(uint16_t, h);
    }
    static __device__ __forceinline__ void put(f16_t* p, float v) { p->bits = (uint16_t)bits(v); }
};

// Workgroups that run at the same time on one XCD (ids congruent mod 8 go to the same XCD and share its
// L2) get tiles that are neighbours: every XCD takes a contiguous eighth of the tile sequence, and
// the sequence walks panels of four N tiles top to bottom, so ~32 resident workgroups cover about
// 8 M tiles x 4 N tiles and re-read each other's A rows and B rows from L2.
__device__ __forceinline__ void gemm_tile_of(int id, int tilesM, int tilesN, int& tm, int& tn) {
    const int total = tilesM * tilesN;
    const int per = (total + 7) / 8;
    int t = (id & 7) * per + (id >> 3);
    if ((id >> 3) >= per || t >= total) { tm = -1; tn = -1; return; } // (ids past an XCD's share would walk into the next XCD's)
    const int panel = t / (4 * tilesM);
    const int pw = min(4, tilesN - 4 * panel);
    const int r = t - panel * 4 * tilesM;
    tm = r / pw;
    tn = 4 * panel + r % pw;
}

#define GEMM_EPI_PLAIN 0  // C = acc (+ R), fp32
#define GEMM_EPI_SWIGLU 1 // columns 2j, 2j+1 are gate and up of unit j: U[m, j] = silu(gate) * up, stored as T

// lda/ldb in elements; K * sizeof(T) must be a multiple of 128.  R may be null, and may alias C.
// BM x BN 32x32 blocks per wave, waves arranged 2 x 2: the workgroup tile is 64 BM x 64 BN.
template <typename T, int BM, int BN, int EPI>
__global__ void __launch_bounds__(GTHREADS) k_gemm_tn(const T* __restrict__ A, int lda, const T* __restrict__ B, int ldb,
                                                      void* Cv, int ldc, const float* R, int ldr, int M, int N, int K, int tilesM, int tilesN, float alpha) {
    constexpr int TM = 64 * BM, TN = 64 * BN;
    constexpr int PA = TM / 32, PB = TN / 32; // 16-byte pieces per thread and slice
    extern __shared__ __attribute__((aligned(16))) unsigned char gsm[];
    unsigned char* As = gsm;
    unsigned char* Bs = gsm + TM * GLD;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tm, tn;
    gemm_tile_of(blockIdx.x, tilesM, tilesN, tm, tn);
    if (tm < 0) return;
    const int m0 = tm * TM, n0 = tn * TN;
    const int nslices = (int)(((size_t)K * sizeof(T)) / GKB);
    const unsigned char* Ab = reinterpret_cast<const unsigned char*>(A);
    const unsigned char* Bb = reinterpret_cast<const unsigned char*>(B);
    const size_t ldaB = (size_t)lda * sizeof(T), ldbB = (size_t)ldb * sizeof(T);

    // global -> register staging; rows past the edge repeat the last row, their results are never stored
    const int piece = tid & 7, srow = tid >> 3; // piece i of a thread is row srow + 32 i
    u32x4 ra[PA], rb[PB];
    auto load_slice = [&](int s) {
#pragma unroll
        for (int i = 0; i < PA; i++)
            ra[i] = *reinterpret_cast<const u32x4*>(Ab + (size_t)min(m0 + srow + 32 * i, M - 1) * ldaB + (size_t)s * GKB + piece * 16);
#pragma unroll
        for (int i = 0; i < PB; i++)
            rb[i] = *reinterpret_cast<const u32x4*>(Bb + (size_t)min(n0 + srow + 32 * i, N - 1) * ldbB + (size_t)s * GKB + piece * 16);
    };
    auto store_slice = [&]() {
#pragma unroll
        for (int i = 0; i < PA; i++) *reinterpret_cast<u32x4*>(As + (srow + 32 * i) * GLD + piece * 16) = ra[i];
#pragma unroll
        for (int i = 0; i < PB; i++) *reinterpret_cast<u32x4*>(Bs + (srow + 32 * i) * GLD + piece * 16) = rb[i];
    };

    f32x16 acc[BM][BN];
#pragma unroll
    for (int i = 0; i < BM; i++)
#pragma unroll
        for (int j = 0; j < BN; j++) acc[i][j] = (f32x16)(0.f);

    load_slice(0);
    store_slice();
    __syncthreads();
    const int half = lane >> 5, lrow = lane & 31;
    for (int s = 0; s < nslices; s++) {
        if (s + 1 < nslices) load_slice(s + 1);
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            u32x4 fa[BM], fb[BN];
#pragma unroll
            for (int b = 0; b < BM; b++) fa[b] = *reinterpret_cast<const u32x4*>(As + (wm * 32 * BM + b * 32 + lrow) * GLD + (2 * jj + half) * 16);
#pragma unroll
            for (int b = 0; b < BN; b++) fb[b] = *reinterpret_cast<const u32x4*>(Bs + (wn * 32 * BN + b * 32 + lrow) * GLD + (2 * jj + half) * 16);
#pragma unroll
            for (int bm = 0; bm < BM; bm++)
#pragma unroll
                for (int bn = 0; bn < BN; bn++) GemmTraits<T>::mma(fa[bm], fb[bn], acc[bm][bn]);
        }
        __syncthreads();
        if (s + 1 < nslices) {
            store_slice();
            __syncthreads();
        }
    }

    // accumulator layout of the 32x32 tile: element i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32
#pragma unroll
    for (int bm = 0; bm < BM; bm++)
#pragma unroll
        for (int bn = 0; bn < BN; bn++) {
            const int col = n0 + wn * 32 * BN + bn * 32 + lrow;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = m0 + wm * 32 * BM + bm * 32 + 8 * (i >> 2) + 4 * half + (i & 3);
                float v = acc[bm][bn][i] * alpha;
                if (EPI == GEMM_EPI_SWIGLU) {
                    const float o = __shfl_xor(v, 1, 64); // the up value sits in the odd neighbour lane
                    if (!(lane & 1) && row < M && col < N) GemmTraits<T>::put((T*)Cv + (size_t)row * ldc + (col >> 1), (v / (1.0f + expf(-v))) * o);
                } else if (row < M && col < N) {
                    if (R) v += R[(size_t)row * ldr + col];
                    ((float*)Cv)[(size_t)row * ldc + col] = v;
                }
            }
        }
}

// ----------------------------------------------------------------------------
// Large-tile variant for long M (prefill): 256 x 256 output tile per 512-thread workgroup, each of the
// 2 x 4 waves owning 128 x 64 (eight 32x32 accumulators).  K slices of 128 bytes per row go from global
// memory straight into LDS (no register staging), two stages deep: the loads of slice s+1 are in
// flight while slice s is multiplied, and one barrier per slice separates the stages.
//
// A direct load puts lane i's 16 bytes at (wave-uniform base) + 16 i, so rows cannot be padded.  The
// 8 pieces of a 128-byte row are stored permuted instead: slot j of row r holds piece j ^ ((r >> 1) & 7)
// -- the lane picks which piece it fetches, not where it lands.  The LDS serves 256 bytes (64 banks) per
// cycle, i.e. sixteen lanes of a 16-byte read; two consecutive rows fill the 64 banks once, so sixteen
// consecutive rows reading the same piece touch sixteen different 16-byte bank groups: even and odd rows
// lie in different halves of the banks, and rows of equal parity differ in (r >> 1) & 7.
// ----------------------------------------------------------------------------
#define GB_T 256
#define GB_STAGE (2 * GB_T * GKB) // bytes per stage: A rows then B rows

#define GB_THREADS 512 // 8 waves: 2 along M x 4 along N, each 128 x 64 (two waves per SIMD keep LDS and MFMA busy in turn)
#define GB_BN 2        // 32-wide column blocks per wave

template <typename T, int EPI>
__global__ void __launch_bounds__(GB_THREADS) k_gemm_tn_big(const T* __restrict__ A, int lda, const T* __restrict__ B, int ldb,
                                                            void* Cv, int ldc, const float* R, int ldr, int M, int N, int K, int tilesM, int tilesN, float alpha) {
    extern __shared__ __attribute__((aligned(16))) unsigned char gsm[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    // A workgroup walks the tiles id, id + gridDim.x, ... (one workgroup per compute unit): the first slice of the next
    // tile is fetched during the last slice of the current one and the epilogue's stores drain under the next tile's
    // first slices, so a tile boundary costs the epilogue's issue time, not a kernel launch, a cold start and a drain.
    int id = blockIdx.x, tm, tn;
    gemm_tile_of(id, tilesM, tilesN, tm, tn);
    if (tm < 0) return;
    const int nslices = (int)(((size_t)K * sizeof(T)) / GKB);
    const size_t ldaB = (size_t)lda * sizeof(T), ldbB = (size_t)ldb * sizeof(T);

    // A loading wave fills 64 rows of A and of B, eight rows per load instruction.  A load's address is
    // a scalar base (the tile's first row, advanced by one slice per trip on the scalar unit) plus a 32-bit lane offset
    // that changes only from tile to tile, and its LDS target is scalar too: issuing a slice's loads takes no vector-ALU
    // instruction, so it does not queue behind the MFMAs of the other wave on the SIMD.
    // Only the first wave of every SIMD (waves 0..3) loads, for its own rows and for those of the SIMD's second wave:
    // the load path takes an instruction every ~50 ns per SIMD and a wave starts its MFMAs only when its loads are
    // out, so the second wave multiplies while the first one feeds the load path.  (Spreading the loads between the
    // MFMAs instead, by quarters or one per MFMA pair, measured 5-9 % slower.)
    unsigned goffA[8], goffB[8];
    auto uniform_base = [](const void* p) { // wave-uniform pointer into global memory, kept in scalar registers
        unsigned long long v = (unsigned long long)p;
        asm("" : "+s"(v));
        return (const unsigned char*)(__attribute__((address_space(1))) const unsigned char*)v;
    };
    const unsigned char *baseA, *baseB;
    auto aim = [&](int tm_, int tn_) { // lane offsets and scalar bases of tile (tm_, tn_)
        const int m0_ = tm_ * GB_T, n0_ = tn_ * GB_T;
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int r = (wave & 3) * 64 + q * 8 + (lane >> 3);
            const int pc = (lane & 7) ^ ((r >> 1) & 7);
            goffA[q] = (unsigned)((size_t)(min(m0_ + r, M - 1) - m0_) * ldaB) + pc * 16; // rows past the end: the last row again
            goffB[q] = (unsigned)((size_t)(min(n0_ + r, N - 1) - n0_) * ldbB) + pc * 16;
        }
        baseA = uniform_base(reinterpret_cast<const unsigned char*>(A) + (size_t)m0_ * ldaB);
        baseB = uniform_base(reinterpret_cast<const unsigned char*>(B) + (size_t)n0_ * ldbB);
    };
    // (written as the instruction itself: through the builtin the compiler either re-forms 64-bit lane addresses or
    // copies the offsets, one vector-ALU instruction per load either way)
    auto dma16 = [](unsigned long long sbase, unsigned laneOff, unsigned ldsAddr) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(ldsAddr), "v"(laneOff), "s"(sbase) : "memory", "m0");
    };
    const unsigned ldsBase = (unsigned)(unsigned long long)gsm + (unsigned)((wave & 3) * 64 * GKB);
    auto issue = [&](int s, int stage) {
        if (wave >= 4) return;
        const unsigned dst = ldsBase + (unsigned)(stage * GB_STAGE);
        const unsigned long long sa = (unsigned long long)baseA + (unsigned long long)s * GKB, sb = (unsigned long long)baseB + (unsigned long long)s * GKB;
#pragma unroll
        for (int q = 0; q < 8; q++) {
            dma16(sa, goffA[q], dst + q * 8 * GKB);
            dma16(sb, goffB[q], dst + GB_T * GKB + q * 8 * GKB);
        }
    };

    const int half = lane >> 5, lrow = lane & 31;
    // row offsets and swizzle keys of this lane's operand rows ((row >> 1) & 7 does not depend on the 32-row block)
    const int keyA = ((wm * 128 + lrow) >> 1) & 7, keyB = ((wn * 32 * GB_BN + lrow) >> 1) & 7;
    const int offA = (wm * 128 + lrow) * GKB, offB = GB_T * GKB + (wn * 32 * GB_BN + lrow) * GKB;

    aim(tm, tn);
    issue(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int gs = 0; // slices consumed so far, over all tiles: slice gs sits in stage gs & 1
  for (;;) {
    const int m0 = tm * GB_T, n0 = tn * GB_T;
    int tmN, tnN;
    gemm_tile_of(id + (int)gridDim.x, tilesM, tilesN, tmN, tnN);
    const bool more = tmN >= 0;
    f32x16 acc[4][GB_BN];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < GB_BN; j++) acc[i][j] = (f32x16)(0.f);
    for (int s = 0; s < nslices; s++, gs++) {
        const int stage = gs & 1;
        const unsigned char* base = gsm + stage * GB_STAGE;
        // operand fragments one 16-wide step ahead of the MFMAs that use them
        u32x4 fa[2][4], fb[2][GB_BN];
        auto frags = [&](int jj, int buf) {
            const int pa = ((2 * jj + half) ^ keyA) * 16, pb = ((2 * jj + half) ^ keyB) * 16;
#pragma unroll
            for (int b = 0; b < 4; b++) fa[buf][b] = *reinterpret_cast<const u32x4*>(base + offA + b * 32 * GKB + pa);
#pragma unroll
            for (int b = 0; b < GB_BN; b++) fb[buf][b] = *reinterpret_cast<const u32x4*>(base + offB + b * 32 * GKB + pb);
        };
        frags(0, 0); // before the loads: the first operands cross the LDS latency while the loads go out
        __builtin_amdgcn_sched_barrier(0);
        if (s + 1 < nslices) issue(s + 1, stage ^ 1);
        else if (more) { aim(tmN, tnN); issue(0, stage ^ 1); } // the tile's own slices are all out: the next tile's first one
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            // the reads of step jj+1 go out in the middle of step jj's MFMAs: early enough to have landed when
            // they are needed, late enough that waiting for step jj's operands does not wait for them too.
            // The scheduling barriers pin that order (the scheduler would sink every read to its first use).
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int bm = 0; bm < 2; bm++)
#pragma unroll
                for (int bn = 0; bn < GB_BN; bn++) GemmTraits<T>::mma(fb[jj & 1][bn], fa[jj & 1][bm], acc[bm][bn]);
            __builtin_amdgcn_sched_barrier(0);
            if (jj < 3) frags(jj + 1, (jj + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int bm = 2; bm < 4; bm++)
#pragma unroll
                for (int bn = 0; bn < GB_BN; bn++) GemmTraits<T>::mma(fb[jj & 1][bn], fa[jj & 1][bm], acc[bm][bn]);
        }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the slice after this one has landed
        __syncthreads();                                  // ... for every wave, and everyone is done with this one
    }
    unsigned char* const freeStage = gsm + ((gs - 1) & 1) * GB_STAGE; // the stage consumed last: the epilogue's patches live there

    // Epilogue.  The product was formed transposed (weights as the first MFMA operand), so lane (lrow, half) holds, for
    // every 32 x 32 block, row lrow of C and the columns 8 g + 4 half + 0..3 in acc[..][4 g + 0..3]: the gate and up value
    // of a SwiGLU pair sit in one lane.  A block then goes through a patch of LDS of the wave's own (the stages are free:
    // the loop ended with a barrier) and is read back with several lanes per row, so that a store instruction writes whole
    // rows of 64 or 128 bytes instead of 64 scattered pieces; the residual is read the same way.
    {
        constexpr int EP = 144;                                  // patch row pitch in bytes (16-byte aligned, rows 4 banks apart)
        typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
        typedef __attribute__((address_space(3))) uint32_t lds_u32;
        typedef __attribute__((address_space(3))) float lds_f32;
        const unsigned patch = (unsigned)(unsigned long long)freeStage + wave * (32 * EP); // 8 x 4.5 KB inside the 64 KB stage
        const int mW = m0 + wm * 128, nW = n0 + wn * 32 * GB_BN;
        if (EPI == GEMM_EPI_PLAIN) {
            const bool vec = ((ldc & 3) == 0) && (!R || (ldr & 3) == 0) && (((unsigned long long)Cv & 15) == 0) && (((unsigned long long)R & 15) == 0);
            const unsigned wr = patch + lrow * EP + half * 16, rd = patch + (lane >> 3) * EP + (lane & 7) * 16;
#pragma unroll
            for (int bm = 0; bm < 4; bm++)
#pragma unroll
                for (int bn = 0; bn < GB_BN; bn++) {
                    const unsigned pb = 0;
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        f32x4 v;
                        v.x = acc[bm][bn][4 * g] * alpha; v.y = acc[bm][bn][4 * g + 1] * alpha; v.z = acc[bm][bn][4 * g + 2] * alpha; v.w = acc[bm][bn][4 * g + 3] * alpha;
                        *(lds_f32x4*)(wr + pb + g * 32) = v;
                    }
                    const int rowb = mW + bm * 32 + (lane >> 3), col = nW + bn * 32 + (lane & 7) * 4;
                    f32x4 v[4];
#pragma unroll
                    for (int k = 0; k < 4; k++) v[k] = *(const lds_f32x4*)(rd + pb + k * 8 * EP);
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const int row = rowb + 8 * k;
                        if (row >= M || col >= N) continue;
                        float* cp = (float*)Cv + (size_t)row * ldc + col;
                        if (vec && col + 3 < N) {
                            if (R) v[k] += *reinterpret_cast<const f32x4*>(R + (size_t)row * ldr + col);
                            *reinterpret_cast<f32x4*>(cp) = v[k];
                        } else {
                            const float* rp = R ? R + (size_t)row * ldr + col : nullptr;
                            cp[0] = v[k].x + (rp ? rp[0] : 0.f);
                            if (col + 1 < N) cp[1] = v[k].y + (rp ? rp[1] : 0.f);
                            if (col + 2 < N) cp[2] = v[k].z + (rp ? rp[2] : 0.f);
                            if (col + 3 < N) cp[3] = v[k].w + (rp ? rp[3] : 0.f);
                        }
                    }
                }
        } else { // SwiGLU: columns 2 j, 2 j + 1 of the product are gate and up of unit j; U[m, j] = silu(gate) * up in the operand type
            constexpr int ES = (int)sizeof(T);                   // 2 or 4
            constexpr int OUTW = 16 * GB_BN;                     // units per row of the wave's tile
            constexpr int LPR = OUTW * ES / 16;                  // lanes per row when reading back 16 bytes each
            constexpr int RPP = 64 / LPR;                        // rows per pass
            const bool vec = (((size_t)ldc * ES) & 15) == 0 && (((unsigned long long)Cv & 15) == 0);
            const int jW = nW >> 1, NU = N >> 1;
#pragma unroll
            for (int bm = 0; bm < 4; bm++) {
                const unsigned pb = 0;
#pragma unroll
                for (int bn = 0; bn < GB_BN; bn++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float g0 = acc[bm][bn][4 * g] * alpha, u0 = acc[bm][bn][4 * g + 1] * alpha;
                        const float g1 = acc[bm][bn][4 * g + 2] * alpha, u1 = acc[bm][bn][4 * g + 3] * alpha;
                        const float o0 = (g0 / (1.0f + expf(-g0))) * u0, o1 = (g1 / (1.0f + expf(-g1))) * u1;
                        const unsigned at = patch + pb + lrow * EP + (bn * 16 + 4 * g + 2 * half) * ES;
                        if (ES == 2) {
                            *(lds_u32*)at = GemmTraits<T>::bits(o0) | (GemmTraits<T>::bits(o1) << 16);
                        } else {
                            *(lds_f32*)at = o0;
                            *(lds_f32*)(at + 4) = o1;
                        }
                    }
#pragma unroll
                for (int k = 0; k < 32 / RPP; k++) {
                    const int rl = (lane / LPR) + RPP * k, piece = lane % LPR;
                    const f32x4 v = *(const lds_f32x4*)(patch + pb + rl * EP + piece * 16);
                    const int row = mW + bm * 32 + rl, j = jW + piece * (16 / ES);
                    if (row >= M || j >= NU) continue;
                    T* up = (T*)Cv + (size_t)row * ldc + j;
                    if (vec && j + 16 / ES - 1 < NU) {
                        *reinterpret_cast<f32x4*>(up) = v;
                    } else {
                        const uint32_t w[4] = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
#pragma unroll
                        for (int e = 0; e < 16 / ES; e++)
                            if (j + e < NU) {
                                if (ES == 2) reinterpret_cast<uint16_t*>(up)[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
                                else reinterpret_cast<uint32_t*>(up)[e] = w[e];
                            }
                    }
                }
            }
        }
    }
    if (!more) break;
    __syncthreads(); // every wave is done with its patch: the stage may be fetched into again
    id += (int)gridDim.x; tm = tmN; tn = tnN;
  }
}

template <typename T>
static hipError_t launch_gemm_big(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                                  const float* R, int ldr, int M, int N, int K, float alpha) {
    const int tilesM = (M + GB_T - 1) / GB_T, tilesN = (N + GB_T - 1) / GB_T;
    static int numCUs = 0;
    if (!numCUs) {
        hipDeviceProp_t prop;
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return hipErrorInvalidDevice;
        numCUs = std::max(8, (prop.multiProcessorCount / 8) * 8);
    }
    const unsigned grid = (unsigned)std::min(numCUs, ((tilesM * tilesN + 7) / 8) * 8); // one workgroup per compute unit walks its tiles
    const size_t lds = 2 * GB_STAGE;
    static std::atomic<bool> attr{false}; // set-up is idempotent: two threads that race here both do it
    if (!attr) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_tn_big<T, GEMM_EPI_PLAIN>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_tn_big<T, GEMM_EPI_SWIGLU>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr = true;
    }
    if (epi == GEMM_EPI_SWIGLU)
        hipLaunchKernelGGL((k_gemm_tn_big<T, GEMM_EPI_SWIGLU>), dim3(grid), dim3(GB_THREADS), lds, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, tilesM, tilesN, alpha);
    else
        hipLaunchKernelGGL((k_gemm_tn_big<T, GEMM_EPI_PLAIN>), dim3(grid), dim3(GB_THREADS), lds, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, tilesM, tilesN, alpha);
    return hipGetLastError();
}

// ----------------------------------------------------------------------------
// Large-tile kernel for two-byte operands (the prefill path of a bf16 model): the same 256 x 256 tile, K slices and
// LDS layout as k_gemm_tn_big, but FOUR waves per workgroup, one per SIMD, each owning 128 x 128 of the tile in 256
// accumulator registers, multiplied with v_mfma_f32_16x16x32 (64 blocks of 16 x 16 per wave, two 32-wide steps per
// slice).  On operand data that toggles the multipliers the part is limited by power, not by issue slots, and the
// 16 x 16 x 32 form does a given product on less of it than 32 x 32 x 16 (an accumulator is read and written once per
// 32 products instead of once per 16): a register-only loop of either form sustains 1.95 against 1.70 PFLOP/s on
// N(0, s) data and the same 2.4-2.5 on zeros.
// With one instruction stream per SIMD nothing takes turns: every wave issues its own 16 loads of a slice between its
// own MFMAs (one load per GW_LR MFMAs), reads an operand fragment behind every other MFMA while there are any to read,
// and the MFMA pipe only stands still at two points per slice:
//   F  the wave has read the second (last) step's operands of the slice it is multiplying -- they are read during the
//      first quarter of the slice -- so after a barrier the stage is free and the loads of the slice after next start
//      flowing into it, more than a slice and a half before they are needed;
//   R  the loads of the next slice have landed for every wave (vmcnt counts in issue order: the loads already out for
//      the slice after next may stay in flight), so after a barrier its first step's operands are read under the last
//      quarter of the current slice's MFMAs.
// The load cursor runs ahead of the multiply position and crosses tile boundaries by itself: a workgroup walks its
// tiles in one launch and the next tile's first two slices are in flight while the epilogue runs.  The epilogue uses a
// patch of LDS per wave outside the two stages.  Per slice and wave: 128 MFMAs, 32 LDS reads, 16 loads -- a third fewer
// LDS bytes per flop than the 8-wave kernel (128 x 128 per wave instead of 128 x 64).
// ----------------------------------------------------------------------------
#define GW_THREADS 256
#define GW_FPOS 40     // MFMA index within a slice (0..127) in front of which F sits
#define GW_RPOS 96     // ... and R
#define GW_LR 6        // one load per this many MFMAs, starting at F
#define GW_NOUT ((GW_RPOS - GW_FPOS + GW_LR - 1) / GW_LR) // loads of the slice after next that are out when R is reached
#define GW_EP 144      // row pitch of a wave's epilogue patch in bytes (rows 4 banks apart)
#define GW_PATCH (16 * GW_EP) // one epilogue patch: 16 rows; every wave has two and alternates between them
#define GW_LDS (2 * GB_STAGE + 4 * 2 * GW_PATCH)
#define GW_LOADK(p_) (((p_) - GW_FPOS) / GW_LR)
#define GW_ISLOAD(p_) ((p_) >= GW_FPOS && ((p_) - GW_FPOS) % GW_LR == 0 && GW_LOADK(p_) < 16)

template <typename T> struct GemmMma16;
// (written as the instruction: with 64 accumulator tuples the register allocator otherwise shuffles them between
// MFMAs; the "a" constraint keeps every tuple in its accumulator registers from the first slice to the epilogue)
template <> struct GemmMma16<f16_t> {
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};
template <> struct GemmMma16<bf16_t> {
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};

template <typename T, int EPI>
__global__ void __launch_bounds__(GW_THREADS) k_gemm_tn_w4(const T* __restrict__ A, int lda, const T* __restrict__ B, int ldb,
                                                           void* Cv, int ldc, const float* R, int ldr, int M, int N, int K, int tilesM, int tilesN, float alpha) {
    static_assert(sizeof(T) == 2, "two-byte operands only");
    extern __shared__ __attribute__((aligned(16))) unsigned char gsm[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int id = blockIdx.x, tm, tn;
    gemm_tile_of(id, tilesM, tilesN, tm, tn);
    if (tm < 0) return;
    const int nslices = (int)(((size_t)K * sizeof(T)) / GKB);
    const size_t ldaB = (size_t)lda * sizeof(T), ldbB = (size_t)ldb * sizeof(T);
    const unsigned lds0 = (unsigned)(unsigned long long)gsm;
    typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
    typedef __attribute__((address_space(3))) f32x4 lds_f32x4;
    typedef __attribute__((address_space(3))) uint32_t lds_u32;
    auto lds_rd = [](unsigned addr, int imm) -> u32x4 { return *(const lds_u32x4*)(addr + (unsigned)imm); };

    // ---- load side: wave w fetches rows 64 w .. 64 w + 63 of the A rows and of the B rows of the cursor's tile, eight rows
    // per instruction; address = scalar base (advanced slice by slice) + a lane offset that only changes from tile to tile,
    // LDS target scalar: no vector-ALU instruction per load.  Rows past the end of a matrix fetch its last row again.
    unsigned goffA[8], goffB[8];
    unsigned long long baseA, baseB;
    // (the same in every lane; read out of lane 0 so that it is a scalar for the compiler too, wherever it kept the value)
    auto uniform64 = [](unsigned long long v) {
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
        return ((unsigned long long)hi << 32) | lo;
    };
    auto aim = [&](int tm_, int tn_) {
        const int m0_ = tm_ * GB_T, n0_ = tn_ * GB_T;
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int r = wave * 64 + q * 8 + (lane >> 3);
            const int pc = (lane & 7) ^ ((r >> 1) & 7);
            goffA[q] = (unsigned)((size_t)(min(m0_ + r, M - 1) - m0_) * ldaB) + pc * 16;
            goffB[q] = (unsigned)((size_t)(min(n0_ + r, N - 1) - n0_) * ldbB) + pc * 16;
        }
        baseA = uniform64((unsigned long long)A + (size_t)m0_ * ldaB);
        baseB = uniform64((unsigned long long)B + (size_t)n0_ * ldbB);
    };
    auto dma16 = [&](unsigned long long sbase, unsigned laneOff, unsigned ldsAddr) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(__builtin_amdgcn_readfirstlane(ldsAddr)), "v"(laneOff), "s"(uniform64(sbase)) : "memory", "m0");
    };
    const unsigned ldsLoad = lds0 + (unsigned)(wave * 64 * GKB);
    // load i (0..15) of the cursor's slice into the stage at byte offset SOFF: even i -> A rows, odd i -> B rows
#define GW_LOAD1(i, SOFF)                                                                                                \
    do {                                                                                                                 \
        if (((i) & 1) == 0) dma16(baseA, goffA[(i) >> 1], ldsLoad + (SOFF) + ((i) >> 1) * 8 * GKB);                       \
        else dma16(baseB, goffB[(i) >> 1], ldsLoad + (SOFF) + GB_T * GKB + ((i) >> 1) * 8 * GKB);                         \
    } while (0)
    int curId = id, curS = 0;
    aim(tm, tn);
    auto advance = [&]() { // the cursor's slice is out: on to the next one, of the next tile when this one is through
        curS++;
        baseA += GKB; baseB += GKB;
        if (curS == nslices) {
            curS = 0;
            curId += (int)gridDim.x;
            int a, b;
            gemm_tile_of(curId, tilesM, tilesN, a, b);
            if (a >= 0) aim(a, b);
            else { baseA -= (unsigned long long)nslices * GKB; baseB -= (unsigned long long)nslices * GKB; } // past the last tile: the same rows again, never multiplied
        }
    };

    // ---- operand side: lane (r16 = lane & 15, kq = lane >> 4) supplies row r16 of a 16-row block and the eight K elements
    // 8 kq .. 8 kq + 7 of a 32-wide step kk: piece 4 kk + kq of the row's 128-byte slice, read from the slot the fetching
    // lane put it in.  Block b of the wave's A rows at + b * 16 rows (an immediate), the B rows behind the stage's A rows.
    // The stage of the slice being multiplied alternates: its offset is kept in the addresses themselves and flipped
    // after every slice, so there is one copy of the slice's code.
    const int r16 = lane & 15, kq = lane >> 4;
    const int key = (r16 >> 1) & 7;
    unsigned rdA[2], rdB[2], rdNextA, rdNextB; // this stage, steps 0 and 1; the other stage, step 0
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
        rdA[kk] = lds0 + wm * 128 * GKB + r16 * GKB + ((4 * kk + kq) ^ key) * 16;
        rdB[kk] = rdA[kk] - wm * 128 * GKB + GB_T * GKB + wn * 128 * GKB;
    }
    rdNextA = rdA[0] + GB_STAGE;
    rdNextB = rdB[0] + GB_STAGE;
    unsigned stageOff = 0; // scalar: byte offset of the stage being multiplied

    f32x4 acc[8][8];
    u32x4 fa[2][8], fb[2][8];
    // prologue: slice 0 whole, then the loads of slice 1 that a slice in front of it would have issued after its F
#pragma unroll
    for (int i = 0; i < 16; i++) GW_LOAD1(i, 0u);
    advance();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int b = 0; b < 8; b++) {
        fb[0][b] = lds_rd(rdB[0], b * 16 * GKB);
        fa[0][b] = lds_rd(rdA[0], b * 16 * GKB);
    }
#pragma unroll
    for (int p = GW_FPOS; p < 128; p++)
        if (GW_ISLOAD(p)) { GW_LOAD1(GW_LOADK(p), (unsigned)GB_STAGE); if (GW_LOADK(p) == 15) advance(); }

    // One slice; p = 64 kk + 8 bn + bm is the MFMA's index within it.  On entry fa[0] / fb[0] hold the first step's operands.
    // Reads (behind MFMAs with an odd index, the loads go behind even ones): the second step's during p = 1..31, the next
    // slice's first step (other stage) from R on, in the order the MFMAs need them (B block 0, the eight A blocks, B 1..7).
    // Loads: the slice after next from F on (into this stage), its tail during the first MFMAs of the next slice.
    // The product is formed transposed (weights as the first operand): see the epilogue.  firstOfTile: R also has the
    // epilogue's stores of the previous tile in front of it and waits for everything.
#define GW_SLICE(firstOfTile)                                                                                                \
    {                                                                                                                        \
        const unsigned otherOff = stageOff ^ (unsigned)GB_STAGE;                                                             \
        _Pragma("unroll") for (int kk = 0; kk < 2; kk++) {                                                                   \
            _Pragma("unroll") for (int bn = 0; bn < 8; bn++)                                                                 \
            _Pragma("unroll") for (int bm = 0; bm < 8; bm++) {                                                               \
                const int i = 8 * bn + bm, p = 64 * kk + i;                                                                  \
                if (p == GW_FPOS) {                                                                                          \
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                       \
                    __builtin_amdgcn_s_barrier();                                                                            \
                    __builtin_amdgcn_sched_barrier(0);                                                                       \
                }                                                                                                            \
                if (p == GW_RPOS) {                                                                                          \
                    if (firstOfTile) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                        \
                    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(GW_NOUT) : "memory");                                      \
                    __builtin_amdgcn_s_barrier();                                                                            \
                    __builtin_amdgcn_sched_barrier(0);                                                                       \
                }                                                                                                            \
                GemmMma16<T>::mma(fb[kk][bn], fa[kk][bm], acc[bm][bn]);                                                      \
                {                                                                                                            \
                    int q = -1;                                                                                              \
                    if (kk == 0 && i < 32 && (i & 1)) q = i >> 1;                                                            \
                    if (kk == 1 && p > GW_RPOS && ((p - GW_RPOS) & 1) && (p - GW_RPOS) / 2 < 16) q = (p - GW_RPOS) / 2;       \
                    if (q >= 0) {                                                                                            \
                        const int nb = kk ^ 1;                                                                               \
                        const unsigned raA = kk == 0 ? rdA[1] : rdNextA, raB = kk == 0 ? rdB[1] : rdNextB;                    \
                        if (q == 0) fb[nb][0] = lds_rd(raB, 0);                                                              \
                        else if (q < 9) fa[nb][q - 1] = lds_rd(raA, (q - 1) * 16 * GKB);                                     \
                        else fb[nb][q - 8] = lds_rd(raB, (q - 8) * 16 * GKB);                                                \
                    }                                                                                                        \
                }                                                                                                            \
                if (GW_ISLOAD(p)) { GW_LOAD1(GW_LOADK(p), stageOff); if (GW_LOADK(p) == 15) advance(); }                     \
                if (GW_ISLOAD(p + 128)) { GW_LOAD1(GW_LOADK(p + 128), otherOff); if (GW_LOADK(p + 128) == 15) advance(); }   \
                __builtin_amdgcn_sched_barrier(0);                                                                           \
            }                                                                                                                \
        }                                                                                                                    \
        stageOff = otherOff;                                                                                                 \
        rdA[0] ^= (unsigned)GB_STAGE; rdA[1] ^= (unsigned)GB_STAGE; rdB[0] ^= (unsigned)GB_STAGE; rdB[1] ^= (unsigned)GB_STAGE; \
        rdNextA ^= (unsigned)GB_STAGE; rdNextB ^= (unsigned)GB_STAGE;                                                        \
    }

    for (bool firstTile = true;; firstTile = false) {
        const int m0 = tm * GB_T, n0 = tn * GB_T;
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) acc[i][j] = (f32x4)(0.f);
        for (int s = 0; s < nslices; s++) GW_SLICE(s == 0 && !firstTile)

        // Epilogue.  Lane (r16, kq) holds, for every 16 x 16 block, row r16 of C and the columns 4 kq .. 4 kq + 3: a SwiGLU
        // lane has two (gate, up) pairs.  Blocks go through the wave's patch of LDS (16 rows of 128 bytes) and are read back
        // with eight lanes per row, so that a store instruction writes whole 128-byte lines; the residual is read the same
        // way.  LDS instructions of a wave execute in order: the next writes need not wait for this read-back.
        {
            const unsigned patch = lds0 + 2 * GB_STAGE + wave * (2 * GW_PATCH);
            const unsigned rdp = patch + (lane >> 3) * GW_EP + (lane & 7) * 16;
            const int mW = m0 + wm * 128, nW = n0 + wn * 128;
            if (EPI == GEMM_EPI_PLAIN) {
                const bool vec = ((ldc & 3) == 0) && (!R || (ldr & 3) == 0) && (((unsigned long long)Cv & 15) == 0) && (((unsigned long long)R & 15) == 0);
                // the wave's whole 128 x 128 lies inside C: no per-element tests (the same for every lane; said so explicitly)
                const bool inside = __builtin_amdgcn_readfirstlane((int)(vec && mW + 128 <= M && nW + 128 <= N)) != 0;
                const unsigned wr = patch + r16 * GW_EP + kq * 16;
                // The residual of the interior path is fetched GW_RPF iterations ahead: an iteration is two stores' worth of
                // time and a load's latency is several of those, so waited for on the spot (32 times per tile) it would cost
                // more than the stores themselves.
                constexpr int GW_RPF = 6;
                f32x4 rpre[GW_RPF][2];
                const bool resid = inside && R != nullptr;
                auto rfetch = [&](int it, int slot) { // iteration it = 4 bm + bp
                    const int bm = it >> 2, bp = it & 3;
                    const float* rp = R + (size_t)(mW + bm * 16 + (lane >> 3)) * ldr + nW + bp * 32 + (lane & 7) * 4;
#pragma unroll
                    for (int k2 = 0; k2 < 2; k2++) rpre[slot][k2] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(rp + (size_t)(8 * k2) * ldr));
                };
                if (resid) {
#pragma unroll
                    for (int it = 0; it < GW_RPF; it++) rfetch(it, it);
                }
                if (inside) {
                    // Interior tile: no per-element tests, and the iterations overlap -- block pair it + 1 is written into
                    // the wave's other patch while pair it is on its way back (LDS instructions of a wave execute in order,
                    // so the write cannot overtake the read of pair it - 1 out of that patch), which takes the LDS round
                    // trip off every iteration.
                    auto put = [&](int it) {
                        const int bm = it >> 2, bp = it & 3;
                        const unsigned w = wr + (unsigned)(it & 1) * GW_PATCH;
                        *(lds_f32x4*)(w) = acc[bm][2 * bp] * alpha;
                        *(lds_f32x4*)(w + 64) = acc[bm][2 * bp + 1] * alpha;
                    };
                    put(0);
#pragma unroll
                    for (int it = 0; it < 32; it++) {
                        const int bm = it >> 2, bp = it & 3;
                        f32x4 v[2];
#pragma unroll
                        for (int k = 0; k < 2; k++) v[k] = *(const lds_f32x4*)(rdp + (unsigned)(it & 1) * GW_PATCH + k * 8 * GW_EP);
                        if (it + 1 < 32) put(it + 1);
                        float* cp = (float*)Cv + (size_t)(mW + bm * 16 + (lane >> 3)) * ldc + nW + bp * 32 + (lane & 7) * 4;
                        if (resid) {
#pragma unroll
                            for (int k = 0; k < 2; k++) v[k] += rpre[it % GW_RPF][k];
                            if (it + GW_RPF < 32) rfetch(it + GW_RPF, it % GW_RPF);
                        }
                        // (streaming stores: the output is far larger than the caches and is read by a later kernel,
                        // keeping it out of the L2 leaves the operand panels there and drains 5-8 % faster)
#pragma unroll
                        for (int k = 0; k < 2; k++) __builtin_nontemporal_store(v[k], reinterpret_cast<f32x4*>(cp + (size_t)(8 * k) * ldc));
                    }
                } else {
#pragma unroll
                    for (int bm = 0; bm < 8; bm++)
#pragma unroll
                        for (int bp = 0; bp < 4; bp++) { // two column blocks side by side: 32 columns = one 128-byte line per row
                            *(lds_f32x4*)(wr) = acc[bm][2 * bp] * alpha;
                            *(lds_f32x4*)(wr + 64) = acc[bm][2 * bp + 1] * alpha;
                            const int rowb = mW + bm * 16 + (lane >> 3), col = nW + bp * 32 + (lane & 7) * 4;
                            f32x4 v[2];
#pragma unroll
                            for (int k = 0; k < 2; k++) v[k] = *(const lds_f32x4*)(rdp + k * 8 * GW_EP);
#pragma unroll
                            for (int k = 0; k < 2; k++) {
                                const int row = rowb + 8 * k;
                                if (row >= M || col >= N) continue;
                                float* cp = (float*)Cv + (size_t)row * ldc + col;
                                if (vec && col + 3 < N) {
                                    if (R) v[k] += *reinterpret_cast<const f32x4*>(R + (size_t)row * ldr + col);
                                    *reinterpret_cast<f32x4*>(cp) = v[k];
                                } else {
                                    const float* rp = R ? R + (size_t)row * ldr + col : nullptr;
                                    cp[0] = v[k].x + (rp ? rp[0] : 0.f);
                                    if (col + 1 < N) cp[1] = v[k].y + (rp ? rp[1] : 0.f);
                                    if (col + 2 < N) cp[2] = v[k].z + (rp ? rp[2] : 0.f);
                                    if (col + 3 < N) cp[3] = v[k].w + (rp ? rp[3] : 0.f);
                                }
                            }
                        }
                }
            } else { // SwiGLU: columns 2 j, 2 j + 1 of the product are gate and up of unit j; U[m, j] = silu(gate) * up in the operand type
                const bool vec = (((size_t)ldc * 2) & 15) == 0 && (((unsigned long long)Cv & 15) == 0);
                const int jW = nW >> 1, NU = N >> 1; // the wave's 128 columns are 64 units: 128 bytes per row, eight lanes a row
                const bool inside = __builtin_amdgcn_readfirstlane((int)(vec && mW + 128 <= M && nW + 128 <= N)) != 0;
                // one 16-row block of the wave's tile -> silu(gate) * up in the operand type -> the given patch
                auto put = [&](int bm, unsigned pp) {
#pragma unroll
                    for (int bn = 0; bn < 8; bn++) {
                        const float g0 = acc[bm][bn].x * alpha, u0 = acc[bm][bn].y * alpha;
                        const float g1 = acc[bm][bn].z * alpha, u1 = acc[bm][bn].w * alpha;
                        // silu(g) u = g u / (1 + e^-g) on the hardware's exp2 and reciprocal (1 ulp each: far inside the rounding
                        // of the two-byte result); e^-g = inf gives 0, as the limit does
                        const float o0 = g0 * u0 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * g0));
                        const float o1 = g1 * u1 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * g1));
                        *(lds_u32*)(pp + r16 * GW_EP + (bn * 8 + 2 * kq) * 2) = GemmTraits<T>::bits(o0) | (GemmTraits<T>::bits(o1) << 16);
                    }
                };
                if (inside) { // interior tile: block bm + 1 is formed and written into the other patch while block bm comes back
                    put(0, patch);
#pragma unroll
                    for (int bm = 0; bm < 8; bm++) {
                        f32x4 v[2];
#pragma unroll
                        for (int k = 0; k < 2; k++) v[k] = *(const lds_f32x4*)(rdp + (unsigned)(bm & 1) * GW_PATCH + k * 8 * GW_EP);
                        if (bm + 1 < 8) put(bm + 1, patch + (unsigned)((bm + 1) & 1) * GW_PATCH);
#pragma unroll
                        for (int k = 0; k < 2; k++) {
                            T* up = (T*)Cv + (size_t)(mW + bm * 16 + (lane >> 3) + 8 * k) * ldc + jW + (lane & 7) * 8;
                            __builtin_nontemporal_store(v[k], reinterpret_cast<f32x4*>(up));
                        }
                    }
                } else {
#pragma unroll
                    for (int bm = 0; bm < 8; bm++) {
                        put(bm, patch);
#pragma unroll
                        for (int k = 0; k < 2; k++) {
                            const int rl = (lane >> 3) + 8 * k, piece = lane & 7;
                            const f32x4 v = *(const lds_f32x4*)(rdp + k * 8 * GW_EP);
                            const int row = mW + bm * 16 + rl, j = jW + piece * 8;
                            T* up = (T*)Cv + (size_t)row * ldc + j;
                            if (row >= M || j >= NU) continue;
                            if (vec && j + 7 < NU) {
                                *reinterpret_cast<f32x4*>(up) = v;
                            } else {
                                const uint32_t w[4] = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
#pragma unroll
                                for (int e = 0; e < 8; e++)
                                    if (j + e < NU) reinterpret_cast<uint16_t*>(up)[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
                            }
                        }
                    }
                }
            }
        }
        id += (int)gridDim.x;
        gemm_tile_of(id, tilesM, tilesN, tm, tn);
        if (tm < 0) break;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the cursor's last loads target this workgroup's LDS: let them land before it is given up
#undef GW_SLICE
#undef GW_LOAD1
}

// Compute units of the current device, rounded down to a multiple of eight (one workgroup per unit, the same number
// on every XCD); 0 when the device cannot be asked.
static int gemm_num_cus() {
    static std::atomic<int> numCUs{0};
    if (!numCUs) {
        hipDeviceProp_t prop;
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
        numCUs = std::max(8, (prop.multiProcessorCount / 8) * 8);
    }
    return numCUs;
}

template <typename T>
static hipError_t launch_gemm_w4(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                                 const float* R, int ldr, int M, int N, int K, float alpha) {
    const int tilesM = (M + GB_T - 1) / GB_T, tilesN = (N + GB_T - 1) / GB_T;
    const int numCUs = gemm_num_cus();
    if (!numCUs) return hipErrorInvalidDevice;
    const unsigned grid = (unsigned)std::min(numCUs, ((tilesM * tilesN + 7) / 8) * 8); // one workgroup per compute unit walks its tiles
    const size_t lds = GW_LDS;
    static std::atomic<bool> attr{false}; // set-up is idempotent: two threads that race here both do it
    if (!attr) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_tn_w4<T, GEMM_EPI_PLAIN>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_tn_w4<T, GEMM_EPI_SWIGLU>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        // the kernel flips stages by XOR on absolute LDS addresses, which is an add/subtract of a stage only while
        // its dynamic LDS starts at address 0, i.e. while it declares no static __shared__ storage
        for (const void* f : {reinterpret_cast<const void*>(&k_gemm_tn_w4<T, GEMM_EPI_PLAIN>), reinterpret_cast<const void*>(&k_gemm_tn_w4<T, GEMM_EPI_SWIGLU>)}) {
            hipFuncAttributes fa;
            if ((e = hipFuncGetAttributes(&fa, f)) != hipSuccess) return e;
            if (fa.sharedSizeBytes != 0) return hipErrorInvalidConfiguration;
        }
        attr = true;
    }
    if (epi == GEMM_EPI_SWIGLU)
        hipLaunchKernelGGL((k_gemm_tn_w4<T, GEMM_EPI_SWIGLU>), dim3(grid), dim3(GW_THREADS), lds, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, tilesM, tilesN, alpha);
    else
        hipLaunchKernelGGL((k_gemm_tn_w4<T, GEMM_EPI_PLAIN>), dim3(grid), dim3(GW_THREADS), lds, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, tilesM, tilesN, alpha);
    return hipGetLastError();
}

template <typename T, int BM, int BN>
static hipError_t launch_gemm(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                              const float* R, int ldr, int M, int N, int K, float alpha) {
    constexpr int TM = 64 * BM, TN = 64 * BN;
    const int tilesM = (M + TM - 1) / TM, tilesN = (N + TN - 1) / TN;
    const int total = tilesM * tilesN;
    const unsigned grid = (unsigned)(((total + 7) / 8) * 8);
    const size_t lds = (size_t)(TM + TN) * GLD;
    static std::atomic<bool> attr[2] = {{false}, {false}};
    if (lds > 64 * 1024 && !attr[epi]) {
        hipError_t e = hipFuncSetAttribute(epi ? reinterpret_cast<const void*>(&k_gemm_tn<T, BM, BN, GEMM_EPI_SWIGLU>)
                                               : reinterpret_cast<const void*>(&k_gemm_tn<T, BM, BN, GEMM_EPI_PLAIN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr[epi] = true;
    }
    if (epi == GEMM_EPI_SWIGLU)
        hipLaunchKernelGGL((k_gemm_tn<T, BM, BN, GEMM_EPI_SWIGLU>), dim3(grid), dim3(GTHREADS), lds, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, tilesM, tilesN, alpha);
    else
        hipLaunchKernelGGL((k_gemm_tn<T, BM, BN, GEMM_EPI_PLAIN>), dim3(grid), dim3(GTHREADS), lds, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, tilesM, tilesN, alpha);
    return hipGetLastError();
}

// ----------------------------------------------------------------------------
// Skinny variant for M <= 64 (batched decode: one row per sequence).  The weight matrix is the big
// operand and is read exactly once: a workgroup owns 32 weight rows and (with split-K) one slice of
// K, its four waves take 128-byte chunks of that slice in turn and multiply straight out of global
// memory -- the MFMA operand layout (lane = row, 16 bytes of K) is also a reasonable load pattern:
// the four 16-byte loads of a lane cover 64 contiguous bytes of its row.  The next chunk's loads are
// issued before the current chunk is multiplied.  The product is formed transposed, D[n, m] = B . A^T,
// so a lane ends up with four consecutive n for one m.  The four waves' partial sums meet in LDS and
// are added in a fixed order.
//
// Split-K over workgroups (matrices with few rows would otherwise occupy a fraction of the CUs):
// every workgroup writes its partial tile to a workspace and bumps the tile's counter; whichever
// arrives last adds the partials in slice order -- the result does not depend on arrival order --
// applies the epilogue and resets the counter.  Partials and counters move with agent-scope atomics
// (memory-side), which is all the ordering this needs: no cache write-back or invalidate.
// ----------------------------------------------------------------------------
__device__ __forceinline__ float g_ald(const float* p) {
    return __uint_as_float(__hip_atomic_load(reinterpret_cast<const unsigned*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ void g_ast(float* p, float v) {
    __hip_atomic_store(reinterpret_cast<unsigned*>(p), __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

#define GSK_COUNTERS 1024 // tiles a split-K launch may have (N <= 32768)
#define GSK_WAVES 8       // waves of a skinny-GEMM workgroup: they split K, and each keeps two chunks of loads in flight --
                          // with few waves the kernel waits on memory latency chunk after chunk, not on bandwidth

// Sum of the waves' partial accumulators, in a fixed order.
template <int MB>
__device__ __forceinline__ float red_sum(const float (&red)[GSK_WAVES][MB][16][64], int mb, int i, int lane) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < GSK_WAVES; w += 2) t += red[w][mb][i][lane] + red[w + 1][mb][i][lane];
    return t;
}

template <typename T, int MB, int EPI>
__global__ void __launch_bounds__(GSK_WAVES * 64) k_gemm_skinny(const T* __restrict__ A, int lda, const T* __restrict__ B, int ldb,
                                                          void* Cv, int ldc, const float* R, int ldr, int M, int N, int K,
                                                          unsigned* counters, float* partials, float alpha) {
    __shared__ float red[GSK_WAVES][MB][16][64];
    __shared__ int lastFlag;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * 32, n32 = lane & 31, half = lane >> 5;
    const int ks = gridDim.y, kslice = blockIdx.y;
    const int nchunks = (int)(((size_t)K * sizeof(T)) / GKB);
    // (32-bit and skipped without split-K: a 64-bit division is some 130 instructions in front of every wave's first load)
    const int cbeg = ks == 1 ? 0 : (int)((unsigned)nchunks * (unsigned)kslice / (unsigned)ks);
    const int cend = ks == 1 ? nchunks : (int)((unsigned)nchunks * (unsigned)(kslice + 1) / (unsigned)ks);
    const unsigned char* brow = reinterpret_cast<const unsigned char*>(B) + (size_t)min(n0 + n32, N - 1) * ldb * sizeof(T) + half * 64;
    const unsigned char* arow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
        arow[mb] = reinterpret_cast<const unsigned char*>(A) + (size_t)min(mb * 32 + n32, M - 1) * lda * sizeof(T) + half * 64;
    f32x16 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) acc[mb] = (f32x16)(0.f);
    u32x4 fb[2][4], fa[2][MB][4];
    auto load = [&](int c, int buf) {
#pragma unroll
        for (int p = 0; p < 4; p++) fb[buf][p] = *reinterpret_cast<const u32x4*>(brow + (size_t)c * GKB + p * 16);
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int p = 0; p < 4; p++) fa[buf][mb][p] = *reinterpret_cast<const u32x4*>(arow[mb] + (size_t)c * GKB + p * 16);
    };
    auto mul = [&](int buf) {
        // both operands put the same K elements in the same (half, position) slots, so every k meets itself
#pragma unroll
        for (int p = 0; p < 4; p++)
#pragma unroll
            for (int mb = 0; mb < MB; mb++) GemmTraits<T>::mma(fb[buf][p], fa[buf][mb][p], acc[mb]);
    };
    // (The product itself bounds this kernel at M = 64 in fp32: 32 rows x 64 tokens x K on one compute unit's matrix
    // cores is 5.8 us at K = 768, whatever the number of waves or of loads in flight.)
    int c = cbeg + wave;
    if (c < cend) load(c, 0);
    for (; c < cend; c += 2 * GSK_WAVES) { // two chunks per trip so the buffers are addressed statically
        if (c + GSK_WAVES < cend) load(c + GSK_WAVES, 1);
        mul(0);
        if (c + GSK_WAVES < cend) {
            if (c + 2 * GSK_WAVES < cend) load(c + 2 * GSK_WAVES, 0);
            mul(1);
        }
    }
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int i = 0; i < 16; i++) red[wave][mb][i][lane] = acc[mb][i];
    __syncthreads();
    // the workgroup's tile: MB x 4 groups of four accumulator elements per lane, wave w takes groups w, w + GSK_WAVES, ...
    const size_t tileFloats = (size_t)MB * 16 * 64;
    float* myPart = partials + ((size_t)blockIdx.x * ks + kslice) * tileFloats;
    if (ks > 1) {
        for (int g = wave; g < MB * 4; g += GSK_WAVES) {
            const int mb = g >> 2, i4 = g & 3;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = 4 * i4 + j;
                g_ast(myPart + ((size_t)mb * 16 + i) * 64 + lane, red_sum(red, mb, i, lane));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup"); // the stores above have been acknowledged ...
        __syncthreads();                                        // ... for every wave of the workgroup
        if (tid == 0) {
            const unsigned prev = __hip_atomic_fetch_add(counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lastFlag = prev == (unsigned)(ks - 1);
            if (lastFlag) __hip_atomic_store(counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!lastFlag) return;
    }
    for (int g = wave; g < MB * 4; g += GSK_WAVES) {
        const int mb = g >> 2, i4 = g & 3;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = 4 * i4 + j;
            if (ks > 1) {
                float sum = 0.f;
                for (int q = 0; q < ks; q++) sum += g_ald(partials + ((size_t)blockIdx.x * ks + q) * tileFloats + ((size_t)mb * 16 + i) * 64 + lane);
                v[j] = sum;
            } else {
                v[j] = red_sum(red, mb, i, lane);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] *= alpha;
        const int m = mb * 32 + n32, n = n0 + 8 * i4 + 4 * half; // accumulator element i: weight row 8 (i / 4) + 4 half + i % 4, column m
        if (m >= M) continue;
        if (EPI == GEMM_EPI_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; j += 2)
                if (n + j + 1 < N) GemmTraits<T>::put((T*)Cv + (size_t)m * ldc + ((n + j) >> 1), (v[j] / (1.0f + expf(-v[j]))) * v[j + 1]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (n + j < N) {
                    float o = v[j];
                    if (R) o += R[(size_t)m * ldr + n + j];
                    ((float*)Cv)[(size_t)m * ldc + n + j] = o;
                }
        }
    }
}

// The same for 32 < M <= 64 in fp32 with 16 weight rows per workgroup (v_mfma_f32_16x16x4f32, four token blocks of
// 16).  At this size the product is bound by the matrix cores of the compute units it runs on -- 32 rows x 64 tokens
// x K = 768 take one unit 5.8 us -- and a matrix of a few thousand rows in 32-row tiles occupies a third of the chip:
// tiles of 16 rows double the units at work.  Lane l holds weight row l % 16 (token l % 16 of a block) and the
// 16 bytes at K offset (l / 16) * 16 of each 64-byte half chunk; element e of those vectors meets element e.
// With NORM the rows of A are RMS-normalised on the way in (inference.cu:24-50): C = (gain * A / rms(A)) . B^T.  The gain
// multiplies the elements as they are loaded, the sum of squares of a row is gathered from the same loads, and
// 1 / rms scales the finished product, so the normalised activations are never written to memory (gridDim.y = 1).
// The activation rows take the way through LDS: the operand layout wants 16 different rows in 16 neighbouring lanes,
// and a load of that shape touches 16 cache lines for 64 bytes each -- the L1 then fills at 36 GB/s per compute unit
// instead of 112 GB/s with eight lanes per 128-byte line (measured with a load-only probe), and at 64 tokens the
// activation matrix is four fifths of what a workgroup reads.  So a wave fetches its chunk of A global -> LDS with
// line-shaped loads (8 token rows per instruction, the 16-byte piece order XOR-swizzled by the fetching lane) into a
// private buffer and reads the operands from there; only the 16 weight rows still load row per lane.
#define SK16_ABUF (64 * GKB)                          // one chunk of A: 64 token rows x 128 bytes
#define SK16_LDS (GSK_WAVES * SK16_ABUF)              // bytes of dynamic LDS per workgroup
template <int EPI, bool NORM>
__global__ void __launch_bounds__(GSK_WAVES * 64) k_gemm_skinny16(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb,
                                                                   void* Cv, int ldc, const float* R, int ldr, int M, int N, int K,
                                                                   unsigned* counters, float* partials, float alpha,
                                                                   const float* __restrict__ gain) {
    extern __shared__ __attribute__((aligned(16))) unsigned char sk16_lds[];
    float (*red)[4][4][64] = reinterpret_cast<float (*)[4][4][64]>(sk16_lds); // [GSK_WAVES], over the A buffers once they are done
    __shared__ float ssred[GSK_WAVES][4][16];
    __shared__ int lastFlag;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.x * 16, n16 = lane & 15, kq = lane >> 4;
    const int ks = gridDim.y, kslice = blockIdx.y;
    const int nchunks = (int)(((size_t)K * 4) / GKB);
    // (32-bit and skipped without split-K: a 64-bit division is some 130 instructions in front of every wave's first load)
    const int cbeg = ks == 1 ? 0 : (int)((unsigned)nchunks * (unsigned)kslice / (unsigned)ks);
    const int cend = ks == 1 ? nchunks : (int)((unsigned)nchunks * (unsigned)(kslice + 1) / (unsigned)ks);
    const unsigned char* brow = reinterpret_cast<const unsigned char*>(B) + (size_t)min(n0 + n16, N - 1) * ldb * 4 + kq * 16;
    // fetch side: instruction j of a chunk brings token rows 8 j + lane / 8, this lane the piece that belongs into
    // slot lane % 8 of its row; read side: row tb * 16 + n16, pieces kq and kq + 4 (their slots: XOR with the same key)
    unsigned aoff[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int r = j * 8 + (lane >> 3);
        aoff[j] = (unsigned)((size_t)min(r, M - 1) * lda * 4) + (unsigned)(((lane & 7) ^ ((r >> 1) & 7)) * 16);
    }
    const unsigned char* abase = reinterpret_cast<const unsigned char*>(A);
    unsigned char* const wbuf = sk16_lds + wave * SK16_ABUF;
    const int akey = (n16 >> 1) & 7;
    const int ardoff = n16 * GKB;
    f32x4 acc[4];
#pragma unroll
    for (int tb = 0; tb < 4; tb++) acc[tb] = (f32x4)(0.f);
    f32x4 fb[2][2], fa[4][2], fg[2][2];
    float ss[4] = {0.f, 0.f, 0.f, 0.f}; // NORM: this lane's share of the sums of squares of its four tokens
    const unsigned char* grow = reinterpret_cast<const unsigned char*>(gain) + kq * 16;
    auto load = [&](int c, int buf) { // buf names the registers of the weight rows and the gain; A has one LDS buffer
#pragma unroll
        for (int p = 0; p < 2; p++) fb[buf][p] = *reinterpret_cast<const f32x4*>(brow + (size_t)c * GKB + p * 64);
        if (NORM) {
#pragma unroll
            for (int p = 0; p < 2; p++) fg[buf][p] = *reinterpret_cast<const f32x4*>(grow + (size_t)c * GKB + p * 64);
        }
        const unsigned char* src = abase + (size_t)c * GKB;
#pragma unroll
        for (int j = 0; j < 8; j++) __builtin_amdgcn_global_load_lds(src + aoff[j], wbuf + j * 8 * GKB, 16, 0, 0);
    };
    // One chunk per wave is in flight at a time and every wait is for all of the wave's loads; the overlap comes from
    // the registers: a chunk's operands are read out of LDS, then the next chunk's loads go out into the same buffer,
    // then this chunk is multiplied.  (Two chunks in flight with a counted wait do not work: with register loads and
    // direct-to-LDS loads mixed the compiler waits for all of them anyway, and loads written as instructions behind
    // its back get their target registers copied before the data has landed.)
    auto mul = [&](int buf, int cnext) { // cnext < 0: nothing more to fetch
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this chunk's weight rows, gain and A rows have landed
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        const unsigned char* rd = wbuf + ardoff;
#pragma unroll
        for (int tb = 0; tb < 4; tb++)
#pragma unroll
            for (int p = 0; p < 2; p++) fa[tb][p] = *reinterpret_cast<const f32x4*>(rd + tb * 16 * GKB + (((kq + 4 * p) ^ akey) * 16));
        // the operands must be in registers before the buffer is fetched into again
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[1][0]), "+v"(fa[1][1]), "+v"(fa[2][0]), "+v"(fa[2][1]), "+v"(fa[3][0]), "+v"(fa[3][1]) : : "memory");
        __builtin_amdgcn_sched_barrier(0);
        if (cnext >= 0) load(cnext, buf ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        if (NORM) {
#pragma unroll
            for (int tb = 0; tb < 4; tb++)
#pragma unroll
                for (int p = 0; p < 2; p++) {
                    const f32x4 x = fa[tb][p];
                    ss[tb] = fmaf(x.x, x.x, ss[tb]); ss[tb] = fmaf(x.y, x.y, ss[tb]); ss[tb] = fmaf(x.z, x.z, ss[tb]); ss[tb] = fmaf(x.w, x.w, ss[tb]);
                    fa[tb][p] = x * fg[buf][p];
                }
        }
#pragma unroll
        for (int p = 0; p < 2; p++)
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int tb = 0; tb < 4; tb++) acc[tb] = __builtin_amdgcn_mfma_f32_16x16x4f32(fb[buf][p][e], fa[tb][p][e], acc[tb], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    int c = cbeg + wave;
    if (c < cend) {
        load(c, 0);
        for (;;) {
            if (c + GSK_WAVES < cend) mul(0, c + GSK_WAVES); else { mul(0, -1); break; }
            c += GSK_WAVES;
            if (c + GSK_WAVES < cend) mul(1, c + GSK_WAVES); else { mul(1, -1); break; }
            c += GSK_WAVES;
        }
    }
    __syncthreads(); // every wave is done with its A buffers: red lies over them
#pragma unroll
    for (int tb = 0; tb < 4; tb++)
#pragma unroll
        for (int r = 0; r < 4; r++) red[wave][tb][r][lane] = acc[tb][r];
    if (NORM) { // lanes n16, n16 + 16, + 32, + 48 hold the four K quarters of token n16
#pragma unroll
        for (int tb = 0; tb < 4; tb++) {
            float t = ss[tb];
            t += __shfl_xor(t, 16, 64);
            t += __shfl_xor(t, 32, 64);
            if (lane < 16) ssred[wave][tb][lane] = t;
        }
    }
    __syncthreads();
    auto wsum = [&](int tb, int r) { // fixed order
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < GSK_WAVES; w += 2) t += red[w][tb][r][lane] + red[w + 1][tb][r][lane];
        return t;
    };
    const size_t tileFloats = 4 * 4 * 64;
    float* myPart = partials + ((size_t)blockIdx.x * ks + kslice) * tileFloats;
    if (ks > 1) {
        if (wave < 4) {
#pragma unroll
            for (int r = 0; r < 4; r++) g_ast(myPart + ((size_t)wave * 4 + r) * 64 + lane, wsum(wave, r));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0) {
            const unsigned prev = __hip_atomic_fetch_add(counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lastFlag = prev == (unsigned)(ks - 1);
            if (lastFlag) __hip_atomic_store(counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!lastFlag) return;
    }
    if (wave >= 4) return;
    const int tb = wave; // one token block per wave
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (ks > 1) {
            float sum = 0.f;
            for (int q = 0; q < ks; q++) sum += g_ald(partials + ((size_t)blockIdx.x * ks + q) * tileFloats + ((size_t)tb * 4 + r) * 64 + lane);
            v[r] = sum * alpha;
        } else {
            v[r] = wsum(tb, r) * alpha;
        }
    }
    const int m = tb * 16 + n16, n = n0 + 4 * kq; // accumulator element r: weight row 4 (lane / 16) + r, token lane % 16
    if (NORM) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < GSK_WAVES; w++) t += ssred[w][tb][n16];
        const float ri = 1.0f / sqrtf(t / (float)K + 1e-8f);
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] *= ri;
    }
    if (m >= M) return;
    if (EPI == GEMM_EPI_SWIGLU) {
#pragma unroll
        for (int j = 0; j < 4; j += 2)
            if (n + j + 1 < N) ((float*)Cv)[(size_t)m * ldc + ((n + j) >> 1)] = (v[j] / (1.0f + expf(-v[j]))) * v[j + 1];
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (n + j < N) {
                float o = v[j];
                if (R) o += R[(size_t)m * ldr + n + j];
                ((float*)Cv)[(size_t)m * ldc + n + j] = o;
            }
    }
}

// The weight-streaming kernel for M <= 32 with the RMSNorm of the activation rows fused in (one 32-row tile, no split
// over K): A holds the fp32 residual rows; a lane multiplies its elements by the gain on the way into the operand
// registers (rounded to half for half weights), adds up their squares, and 1 / rms scales the result:
//   W . (g (.) x / rms(x)) = (W . (g (.) x)) / rms(x),   rms(x) = sqrt(sum x^2 / K + 1e-8)   (inference.cu:24-50, 83-95)
// T is the weight operand type (float, or f16_t for the half mirrors of a bf16 model).
template <typename T, int EPI>
__global__ void __launch_bounds__(GSK_WAVES * 64) k_gemm_skinny_norm(const float* __restrict__ A, int lda, const T* __restrict__ B, int ldb,
                                                               void* Cv, int ldc, const float* R, int ldr, int M, int N, int K,
                                                               float alpha, const float* __restrict__ gain) {
    constexpr int EPC = GKB / (int)sizeof(T), HPC = EPC / 2, NV = HPC / 4; // elements per chunk, per lane half, 16-byte loads of fp32
    __shared__ float red[GSK_WAVES][1][16][64];
    __shared__ float ssq[GSK_WAVES][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * 32, n32 = lane & 31, half = lane >> 5;
    const int nchunks = (int)(((size_t)K * sizeof(T)) / GKB);
    const unsigned char* brow = reinterpret_cast<const unsigned char*>(B) + (size_t)min(n0 + n32, N - 1) * ldb * sizeof(T) + half * 64;
    const float* arow = A + (size_t)min(n32, M - 1) * lda + half * HPC;
    const float* grow = gain + half * HPC;
    f32x16 acc = (f32x16)(0.f);
    float ss = 0.f;
    u32x4 fb[2][4];
    f32x4 xa[2][NV], ga[2][NV];
    auto load = [&](int c, int buf) {
#pragma unroll
        for (int p = 0; p < 4; p++) fb[buf][p] = *reinterpret_cast<const u32x4*>(brow + (size_t)c * GKB + p * 16);
#pragma unroll
        for (int q = 0; q < NV; q++) {
            xa[buf][q] = *reinterpret_cast<const f32x4*>(arow + (size_t)c * EPC + 4 * q);
            ga[buf][q] = *reinterpret_cast<const f32x4*>(grow + (size_t)c * EPC + 4 * q);
        }
    };
    auto half2 = [](float lo, float hi) { // two floats -> two IEEE halves, saturating
        const _Float16 a = (_Float16)fminf(fmaxf(lo, -65504.0f), 65504.0f), b = (_Float16)fminf(fmaxf(hi, -65504.0f), 65504.0f);
        return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
    };
    auto mul = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            u32x4 fa;
            if constexpr (sizeof(T) == 4) {
                const f32x4 x = xa[buf][p], g = ga[buf][p];
                ss = fmaf(x.x, x.x, ss); ss = fmaf(x.y, x.y, ss); ss = fmaf(x.z, x.z, ss); ss = fmaf(x.w, x.w, ss);
                fa.x = __float_as_uint(g.x * x.x); fa.y = __float_as_uint(g.y * x.y); fa.z = __float_as_uint(g.z * x.z); fa.w = __float_as_uint(g.w * x.w);
            } else {
                const f32x4 x0 = xa[buf][2 * p], x1 = xa[buf][2 * p + 1], g0 = ga[buf][2 * p], g1 = ga[buf][2 * p + 1];
                ss = fmaf(x0.x, x0.x, ss); ss = fmaf(x0.y, x0.y, ss); ss = fmaf(x0.z, x0.z, ss); ss = fmaf(x0.w, x0.w, ss);
                ss = fmaf(x1.x, x1.x, ss); ss = fmaf(x1.y, x1.y, ss); ss = fmaf(x1.z, x1.z, ss); ss = fmaf(x1.w, x1.w, ss);
                fa.x = half2(g0.x * x0.x, g0.y * x0.y); fa.y = half2(g0.z * x0.z, g0.w * x0.w);
                fa.z = half2(g1.x * x1.x, g1.y * x1.y); fa.w = half2(g1.z * x1.z, g1.w * x1.w);
            }
            GemmTraits<T>::mma(fb[buf][p], fa, acc);
        }
    };
    int c = wave;
    if (c < nchunks) load(c, 0);
    for (; c < nchunks; c += 2 * GSK_WAVES) { // two chunks per trip so the buffers are addressed statically
        if (c + GSK_WAVES < nchunks) load(c + GSK_WAVES, 1);
        mul(0);
        if (c + GSK_WAVES < nchunks) {
            if (c + 2 * GSK_WAVES < nchunks) load(c + 2 * GSK_WAVES, 0);
            mul(1);
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) red[wave][0][i][lane] = acc[i];
    ssq[wave][lane] = ss;
    __syncthreads();
    // token m = n32: the squares of its row are spread over the waves and the two lane halves (fixed summation order)
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < GSK_WAVES; w++) tot += ssq[w][n32] + ssq[w][n32 + 32];
    const float scale = alpha / sqrtf(tot / (float)K + 1e-8f);
    for (int g = wave; g < 4; g += GSK_WAVES) {
        const int i4 = g;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = red_sum(red, 0, 4 * i4 + j, lane) * scale;
        const int m = n32, n = n0 + 8 * i4 + 4 * half; // accumulator element i: weight row 8 (i / 4) + 4 half + i % 4, column m
        if (m >= M) continue;
        if (EPI == GEMM_EPI_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; j += 2)
                if (n + j + 1 < N) GemmTraits<T>::put((T*)Cv + (size_t)m * ldc + ((n + j) >> 1), (v[j] / (1.0f + expf(-v[j]))) * v[j + 1]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (n + j < N) {
                    float o = v[j];
                    if (R) o += R[(size_t)m * ldr + n + j];
                    ((float*)Cv)[(size_t)m * ldc + n + j] = o;
                }
        }
    }
}

// The same for at most GSK_WAVES rows and half weights, with the normalised-up-to-1/rms rows staged in LDS: wave w
// turns row w into halves of g (.) x once (sum of squares from the same pass), the product then reads its token
// operand from LDS instead of holding fp32 rows and gains in registers -- this keeps the register need of the plain
// kernel, so two workgroups share a compute unit and a matrix of several hundred row blocks still takes one round.
// LDS rows are K halves + 16 bytes apart (rows four banks apart: the eight rows a read touches do not collide).
template <int EPI>
__global__ void __launch_bounds__(GSK_WAVES * 64) k_gemm_skinny_norm8(const float* __restrict__ A, int lda, const f16_t* __restrict__ B, int ldb,
                                                                void* Cv, int ldc, const float* R, int ldr, int M, int N, int K,
                                                                float alpha, const float* __restrict__ gain) {
    extern __shared__ __attribute__((aligned(16))) unsigned char a16[]; // [M][2 K + 16] bytes
    __shared__ float red[GSK_WAVES][1][16][64];
    __shared__ float rinv[GSK_WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * 32, n32 = lane & 31, half = lane >> 5;
    const int nchunks = (int)(((size_t)K * 2) / GKB);
    const int pitch = 2 * K + 16;
    const unsigned char* brow = reinterpret_cast<const unsigned char*>(B) + (size_t)min(n0 + n32, N - 1) * ldb * 2 + half * 64;
    f32x16 acc = (f32x16)(0.f);
    u32x4 fb[2][4];
    auto loadw = [&](int c, int buf) {
#pragma unroll
        for (int p = 0; p < 4; p++) fb[buf][p] = *reinterpret_cast<const u32x4*>(brow + (size_t)c * GKB + p * 16);
    };
    int c = wave;
    if (c < nchunks) loadw(c, 0); // the first weights are on their way while the rows are staged
    if (wave < M) {
        const float* xr = A + (size_t)wave * lda;
        float ss = 0.f;
        for (int k = lane * 8; k < K; k += 64 * 8) {
            const f32x4 x0 = *reinterpret_cast<const f32x4*>(xr + k), x1 = *reinterpret_cast<const f32x4*>(xr + k + 4);
            const f32x4 g0 = *reinterpret_cast<const f32x4*>(gain + k), g1 = *reinterpret_cast<const f32x4*>(gain + k + 4);
            ss = fmaf(x0.x, x0.x, ss); ss = fmaf(x0.y, x0.y, ss); ss = fmaf(x0.z, x0.z, ss); ss = fmaf(x0.w, x0.w, ss);
            ss = fmaf(x1.x, x1.x, ss); ss = fmaf(x1.y, x1.y, ss); ss = fmaf(x1.z, x1.z, ss); ss = fmaf(x1.w, x1.w, ss);
            auto h2 = [](float lo, float hi) {
                const _Float16 a = (_Float16)fminf(fmaxf(lo, -65504.0f), 65504.0f), b = (_Float16)fminf(fmaxf(hi, -65504.0f), 65504.0f);
                return (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
            };
            u32x4 w;
            w.x = h2(g0.x * x0.x, g0.y * x0.y); w.y = h2(g0.z * x0.z, g0.w * x0.w);
            w.z = h2(g1.x * x1.x, g1.y * x1.y); w.w = h2(g1.z * x1.z, g1.w * x1.w);
            *reinterpret_cast<u32x4*>(a16 + (size_t)wave * pitch + 2 * k) = w;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        if (lane == 0) rinv[wave] = 1.0f / sqrtf(ss / (float)K + 1e-8f);
    }
    __syncthreads();
    const unsigned char* arow = a16 + (size_t)min(n32, M - 1) * pitch + half * 64;
    auto mul = [&](int cc, int buf) {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const u32x4 fa = *reinterpret_cast<const u32x4*>(arow + (size_t)cc * GKB + p * 16);
            GemmTraits<f16_t>::mma(fb[buf][p], fa, acc);
        }
    };
    for (; c < nchunks; c += 2 * GSK_WAVES) { // two chunks per trip so the buffers are addressed statically
        if (c + GSK_WAVES < nchunks) loadw(c + GSK_WAVES, 1);
        mul(c, 0);
        if (c + GSK_WAVES < nchunks) {
            if (c + 2 * GSK_WAVES < nchunks) loadw(c + 2 * GSK_WAVES, 0);
            mul(c + GSK_WAVES, 1);
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i++) red[wave][0][i][lane] = acc[i];
    __syncthreads();
    const float scale = alpha * rinv[min(n32, M - 1)];
    for (int g = wave; g < 4; g += GSK_WAVES) {
        const int i4 = g;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = red_sum(red, 0, 4 * i4 + j, lane) * scale;
        const int m = n32, n = n0 + 8 * i4 + 4 * half; // accumulator element i: weight row 8 (i / 4) + 4 half + i % 4, column m
        if (m >= M) continue;
        if (EPI == GEMM_EPI_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; j += 2)
                if (n + j + 1 < N) GemmTraits<f16_t>::put((f16_t*)Cv + (size_t)m * ldc + ((n + j) >> 1), (v[j] / (1.0f + expf(-v[j]))) * v[j + 1]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (n + j < N) {
                    float o = v[j];
                    if (R) o += R[(size_t)m * ldr + n + j];
                    ((float*)Cv)[(size_t)m * ldc + n + j] = o;
                }
        }
    }
}

// rows that k_gemm_skinny_norm8 can stage: at most one per wave, and 40 KB of LDS beside the reduction buffer (two workgroups per unit)
static bool skinny_norm8_fits(int M, int K) { return M <= GSK_WAVES && (size_t)M * (2 * (size_t)K + 16) <= 40 * 1024 && K % 512 == 0; }

static hipError_t launch_gemm_skinny_norm8(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                                           const float* R, int ldr, int M, int N, int K, float alpha, const float* normGain) {
    const dim3 grid((N + 31) / 32);
    const size_t lds = (size_t)M * (2 * (size_t)K + 16);
    static std::atomic<bool> attr{false}; // set-up is idempotent: two threads that race here both do it // static + dynamic LDS pass 64 KB
    if (!attr) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_skinny_norm8<GEMM_EPI_PLAIN>), hipFuncAttributeMaxDynamicSharedMemorySize, 40 * 1024);
        if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_skinny_norm8<GEMM_EPI_SWIGLU>), hipFuncAttributeMaxDynamicSharedMemorySize, 40 * 1024);
        if (e != hipSuccess) return e;
        attr = true;
    }
    if (epi == GEMM_EPI_SWIGLU)
        hipLaunchKernelGGL((k_gemm_skinny_norm8<GEMM_EPI_SWIGLU>), grid, dim3(GSK_WAVES * 64), lds, stream, (const float*)A, lda, (const f16_t*)B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain);
    else
        hipLaunchKernelGGL((k_gemm_skinny_norm8<GEMM_EPI_PLAIN>), grid, dim3(GSK_WAVES * 64), lds, stream, (const float*)A, lda, (const f16_t*)B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_gemm_skinny_norm(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                                          const float* R, int ldr, int M, int N, int K, float alpha, const float* normGain) {
    const dim3 grid((N + 31) / 32);
    if (epi == GEMM_EPI_SWIGLU)
        hipLaunchKernelGGL((k_gemm_skinny_norm<T, GEMM_EPI_SWIGLU>), grid, dim3(GSK_WAVES * 64), 0, stream, (const float*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain);
    else
        hipLaunchKernelGGL((k_gemm_skinny_norm<T, GEMM_EPI_PLAIN>), grid, dim3(GSK_WAVES * 64), 0, stream, (const float*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain);
    return hipGetLastError();
}

static hipError_t launch_gemm_skinny16(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                                       const float* R, int ldr, int M, int N, int K, void* ws, float alpha, const float* normGain) {
    const int nblocks = (N + 15) / 16;
    const int nchunks = (int)(((size_t)K * 4) / GKB);
    int ks = 1;
    if (ws && !normGain && nblocks <= 64 && nchunks >= 32) { // few rows, long K: also split K over workgroups (see launch_gemm_skinny)
        ks = std::min(std::min(8, 256 / nblocks), std::max(1, nchunks / GSK_WAVES));
        if ((size_t)nblocks * ks > 256 * 8) ks = 1;
    }
    const dim3 grid(nblocks, ks);
    unsigned* counters = (unsigned*)ws;
    float* partials = ws ? (float*)((unsigned char*)ws + (size_t)GSK_COUNTERS * 4) : nullptr;
    static std::atomic<bool> attr{false}; // set-up is idempotent: two threads that race here both do it
    if (!attr) {
        const void* fns[4] = {reinterpret_cast<const void*>(&k_gemm_skinny16<GEMM_EPI_PLAIN, false>), reinterpret_cast<const void*>(&k_gemm_skinny16<GEMM_EPI_PLAIN, true>),
                              reinterpret_cast<const void*>(&k_gemm_skinny16<GEMM_EPI_SWIGLU, false>), reinterpret_cast<const void*>(&k_gemm_skinny16<GEMM_EPI_SWIGLU, true>)};
        for (const void* f : fns) {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, SK16_LDS);
            if (e != hipSuccess) return e;
        }
        attr = true;
    }
#define SK16(EPI_, NORM_)                                                                                                     \
    hipLaunchKernelGGL((k_gemm_skinny16<EPI_, NORM_>), grid, dim3(GSK_WAVES * 64), SK16_LDS, stream, (const float*)A, lda, (const float*)B, ldb, \
                       C, ldc, R, ldr, M, N, K, counters, partials, alpha, normGain)
    if (epi == GEMM_EPI_SWIGLU) { if (normGain) SK16(GEMM_EPI_SWIGLU, true); else SK16(GEMM_EPI_SWIGLU, false); }
    else { if (normGain) SK16(GEMM_EPI_PLAIN, true); else SK16(GEMM_EPI_PLAIN, false); }
#undef SK16
    return hipGetLastError();
}

// Workspace for split-K: GSK_COUNTERS zeroed counters, then the partial tiles.
size_t mlh_gemm_workspace_bytes(void) { return (size_t)GSK_COUNTERS * 4 + (size_t)256 * 8 * 2 * 16 * 64 * 4; }

template <typename T, int MB>
static hipError_t launch_gemm_skinny(hipStream_t stream, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                                     const float* R, int ldr, int M, int N, int K, void* ws, float alpha) {
    const int nblocks = (N + 31) / 32;
    const int nchunks = (int)(((size_t)K * sizeof(T)) / GKB);
    int ks = 1;
    // The exchange costs about three memory round trips (~5 us): only worth it when a wave would otherwise
    // grind through many chunks on a handful of CUs (few rows, long K).
    if (ws && nblocks <= 64 && nchunks >= 32) { // aim at ~256 workgroups, every wave with at least one chunk, workspace bounds respected
        ks = std::min(std::min(8, 256 / nblocks), std::max(1, nchunks / 4));
        if (nblocks > GSK_COUNTERS || (size_t)nblocks * ks > 256 * 8) ks = 1;
    }
    const dim3 grid(nblocks, ks);
    unsigned* counters = (unsigned*)ws;
    float* partials = ws ? (float*)((unsigned char*)ws + (size_t)GSK_COUNTERS * 4) : nullptr;
    if (epi == GEMM_EPI_SWIGLU)
        hipLaunchKernelGGL((k_gemm_skinny<T, MB, GEMM_EPI_SWIGLU>), grid, dim3(GSK_WAVES * 64), 0, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, counters, partials, alpha);
    else
        hipLaunchKernelGGL((k_gemm_skinny<T, MB, GEMM_EPI_PLAIN>), grid, dim3(GSK_WAVES * 64), 0, stream, (const T*)A, lda, (const T*)B, ldb, C, ldc, R, ldr, M, N, K, counters, partials, alpha);
    return hipGetLastError();
}

// Enqueues the GEMM on `stream`.  Returns hipSuccess, or an error when the shape is not supported.
// epi = GEMM_EPI_PLAIN: C fp32 [M, N] (+ R).  epi = GEMM_EPI_SWIGLU: C is [M, N/2] in the operand type.
// ws: optional zero-initialised workspace of mlh_gemm_workspace_bytes() (enables split-K for M <= 64); launches that
// share a workspace must be ordered on one stream.
// True when mlh_gemm_tn_epi can take `normGain` for this shape (the RMSNorm of A's rows fused into the product).
bool mlh_gemm_norm_fusable(int dtype, int M, int N, int K) {
    // k_gemm_skinny_norm (A is the fp32 residual for both operand types).  With half weights its register need allows
    // one workgroup per compute unit, where the plain kernel runs two: a matrix of more than 256 row blocks would
    // take two rounds and lose more than the saved RMSNorm launch brings -- unless the rows fit k_gemm_skinny_norm8's LDS.
    if (M <= 32) return dtype == MLH_DTYPE_F32 || (dtype == MLH_GEMM_F16 && ((N + 31) / 32 <= 256 || skinny_norm8_fits(M, K)));
    return dtype == MLH_DTYPE_F32 && M > 32 && M <= 64 && N <= 16 * GSK_COUNTERS && (N + 31) / 32 < 200;
}

hipError_t mlh_gemm_tn_epi(hipStream_t stream, int dtype, int epi, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                           const float* R, int ldr, int M, int N, int K, void* ws, float alpha, const float* normGain) {
    const size_t esz = dtype == MLH_DTYPE_F32 ? 4 : 2;
    if (M <= 0 || N <= 0 || K <= 0 || ((size_t)K * esz) % GKB != 0 || ((size_t)lda * esz) % 16 != 0 || ((size_t)ldb * esz) % 16 != 0)
        return hipErrorInvalidValue;
    if (epi == GEMM_EPI_SWIGLU && (N & 1)) return hipErrorInvalidValue;
    if (normGain && !mlh_gemm_norm_fusable(dtype, M, N, K)) return hipErrorInvalidValue;
    // M <= 64 (one row per sequence of a decode batch): weight-streaming skinny kernel; long M: 256 x 256 tiles
    // fed by direct-to-LDS loads; in between: 128 x 128 tiles
#define GEMM_BY_TYPE(call_f32, call_bf16, call_f16) \
    return dtype == MLH_DTYPE_BF16 ? (call_bf16) : dtype == MLH_GEMM_F16 ? (call_f16) : (call_f32)
    if (M <= 32 && normGain && dtype == MLH_GEMM_F16 && skinny_norm8_fits(M, K))
        return launch_gemm_skinny_norm8(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain);
    if (M <= 32 && normGain)
        return dtype == MLH_GEMM_F16 ? launch_gemm_skinny_norm<f16_t>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain)
                                     : launch_gemm_skinny_norm<float>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha, normGain);
    if (M <= 32)
        GEMM_BY_TYPE((launch_gemm_skinny<float, 1>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha)),
                     (launch_gemm_skinny<bf16_t, 1>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha)),
                     (launch_gemm_skinny<f16_t, 1>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha)));
    if (M > 32 && M <= 64 && dtype == MLH_DTYPE_F32 && N <= 16 * GSK_COUNTERS && (N + 31) / 32 < 200) // the 32-row tiles would leave compute units idle
        return launch_gemm_skinny16(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha, normGain);
    if (M <= 64)
        GEMM_BY_TYPE((launch_gemm_skinny<float, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha)),
                     (launch_gemm_skinny<bf16_t, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha)),
                     (launch_gemm_skinny<f16_t, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, ws, alpha)));
    if (M > 128 && N <= 128 && dtype != MLH_DTYPE_F32 && epi == GEMM_EPI_PLAIN) { // a narrow strip of columns: 64-row tiles put every compute unit to work
        if (dtype == MLH_GEMM_F16) return launch_gemm<f16_t, 1, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha);
        return launch_gemm<bf16_t, 1, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha);
    }
    if (M > 128 && dtype != MLH_DTYPE_F32 && epi == GEMM_EPI_PLAIN && N > GB_T && N % GB_T != 0 && N % GB_T <= 128) {
        // A last column of tiles that is less than half full: when taking it away saves the tile walkers a whole round
        // (every compute unit one 256 x 256 tile: K x 31 ns) and the strip kernel does those columns in less than that
        // (5 us + 180 TFLOP/s, measured), the product runs as two launches.
        const int rem = N % GB_T, cus = gemm_num_cus(), tilesM = (M + GB_T - 1) / GB_T;
        if (!cus) return hipErrorInvalidDevice;
        const int roundsAll = (tilesM * (N / GB_T + 1) + cus - 1) / cus, roundsMain = (tilesM * (N / GB_T) + cus - 1) / cus;
        if (roundsMain < roundsAll && 5.0 + 2.0 * M * rem * K / 180e6 < 0.031 * K) {
            const int Nm = N - rem;
            const hipError_t e = mlh_gemm_tn_epi(stream, dtype, epi, A, lda, B, ldb, C, ldc, R, ldr, M, Nm, K, ws, alpha, nullptr);
            if (e != hipSuccess) return e;
            return mlh_gemm_tn_epi(stream, dtype, epi, A, lda, (const unsigned char*)B + (size_t)Nm * ldb * esz, ldb, (float*)C + Nm, ldc,
                                   R ? R + Nm : nullptr, ldr, M, rem, K, ws, alpha, nullptr);
        }
    }
    if (M > 128)
        GEMM_BY_TYPE((launch_gemm_big<float>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha)),
                     (launch_gemm_w4<bf16_t>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha)),
                     (launch_gemm_w4<f16_t>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha)));
    GEMM_BY_TYPE((launch_gemm<float, 2, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha)),
                 (launch_gemm<bf16_t, 2, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha)),
                 (launch_gemm<f16_t, 2, 2>(stream, epi, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, alpha)));
#undef GEMM_BY_TYPE
}

hipError_t mlh_gemm_tn(hipStream_t stream, int dtype, const void* A, int lda, const void* B, int ldb, float* C, int ldc,
                       const float* R, int ldr, int M, int N, int K) {
    return mlh_gemm_tn_epi(stream, dtype, GEMM_EPI_PLAIN, A, lda, B, ldb, C, ldc, R, ldr, M, N, K, nullptr, 1.0f);
}

static void host_to_bf16(const float* src, bf16_t* dst, size_t n) {
    for (size_t i = 0; i < n; i++) {
        uint32_t u;
        memcpy(&u, &src[i], 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) u |= 0x00400000u;
        else u += 0x7fffu + ((u >> 16) & 1u);
        dst[i] = (bf16_t)(u >> 16);
    }
}

static void host_to_f16(const float* src, f16_t* dst, size_t n) {
    for (size_t i = 0; i < n; i++) {
        const _Float16 h = (_Float16)src[i];
        memcpy(&dst[i].bits, &h, 2);
    }
}

// Stand-alone check and timing of the GEMM kernel: host fp32 inputs (rounded to bf16 first when
// dtype says so), result back on the host, mean launch time over `iters` launches from HIP events.
extern "C" int mlh_selftest_gemm(int dtypeAndEpilogue, int M, int N, int K, const float* A, const float* B, const float* R, float* C,
                                 int iters, double* avgUs) {
    const int dtype = dtypeAndEpilogue & 0xff;
    const bool swiglu = (dtypeAndEpilogue & MLH_SELFTEST_SWIGLU) != 0; // C is then [M, N / 2]: silu(gate) * up of the column pairs
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0 || (swiglu && (R || (N & 1)))) return -1;
    if (mlh_device_count() <= 0) return -1;
    const size_t esz = dtype == MLH_DTYPE_F32 ? 4 : 2;
    const int NC = swiglu ? N / 2 : N;
    const size_t csz = swiglu ? esz : 4; // the SwiGLU epilogue writes the operand type
    void *dA = nullptr, *dB = nullptr, *dW = nullptr, *dC = nullptr;
    float* dR = nullptr;
    int rc = 0;
    std::vector<bf16_t> ha, hb;
    std::vector<uint16_t> hc;
    const void *srcA = A, *srcB = B;
    if (dtype == MLH_DTYPE_BF16) {
        ha.resize((size_t)M * K); hb.resize((size_t)N * K);
        host_to_bf16(A, ha.data(), ha.size()); host_to_bf16(B, hb.data(), hb.size());
        srcA = ha.data(); srcB = hb.data();
    } else if (dtype == MLH_GEMM_F16) {
        ha.resize((size_t)M * K); hb.resize((size_t)N * K);
        host_to_f16(A, (f16_t*)ha.data(), ha.size()); host_to_f16(B, (f16_t*)hb.data(), hb.size());
        srcA = ha.data(); srcB = hb.data();
    }
    const int epi = swiglu ? GEMM_EPI_SWIGLU : GEMM_EPI_PLAIN;
    hipEvent_t e0 = nullptr, e1 = nullptr;
#define ST(x) do { if ((x) != hipSuccess) { rc = -2; goto done; } } while (0)
    ST(hipMalloc(&dA, (size_t)M * K * esz)); ST(hipMalloc(&dB, (size_t)N * K * esz));
    ST(hipMalloc(&dC, (size_t)M * NC * csz));
    if (R) { ST(hipMalloc((void**)&dR, (size_t)M * N * 4)); ST(hipMemcpy(dR, R, (size_t)M * N * 4, hipMemcpyHostToDevice)); }
    ST(hipMemcpy(dA, srcA, (size_t)M * K * esz, hipMemcpyHostToDevice));
    ST(hipMemcpy(dB, srcB, (size_t)N * K * esz, hipMemcpyHostToDevice));
    ST(hipMalloc(&dW, mlh_gemm_workspace_bytes()));
    ST(hipMemset(dW, 0, mlh_gemm_workspace_bytes()));
    ST(mlh_gemm_tn_epi(nullptr, dtype, epi, dA, K, dB, K, dC, NC, dR, N, M, N, K, dW));
    ST(hipDeviceSynchronize());
    if (iters > 0 && avgUs) {
        ST(hipEventCreate(&e0)); ST(hipEventCreate(&e1));
        ST(hipEventRecord(e0, nullptr));
        for (int i = 0; i < iters; i++) ST(mlh_gemm_tn_epi(nullptr, dtype, epi, dA, K, dB, K, dC, NC, dR, N, M, N, K, dW));
        ST(hipEventRecord(e1, nullptr));
        ST(hipEventSynchronize(e1));
        float ms = 0.f;
        ST(hipEventElapsedTime(&ms, e0, e1));
        *avgUs = (double)ms * 1000.0 / iters;
    }
    if (csz == 4) {
        ST(hipMemcpy(C, dC, (size_t)M * NC * 4, hipMemcpyDeviceToHost));
    } else { // half or bf16 results back as floats
        hc.resize((size_t)M * NC);
        ST(hipMemcpy(hc.data(), dC, hc.size() * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < hc.size(); i++) {
            if (dtype == MLH_DTYPE_BF16) { const uint32_t u = (uint32_t)hc[i] << 16; memcpy(&C[i], &u, 4); }
            else { _Float16 h; memcpy(&h, &hc[i], 2); C[i] = (float)h; }
        }
    }
#undef ST
done:
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(dA); (void)hipFree(dB); (void)hipFree(dC); (void)hipFree(dR); (void)hipFree(dW);
    return rc;
}

// ----------------------------------------------------------------------------
// The same product for callers that cannot allocate (code under graph capture, serving loops that forbid
// hipMalloc): device pointers in and out, the launch enqueued on the caller's stream, and the split-K workspace
// (tile counters + partial tiles) in a file-scope device array instead of a hipMalloc'ed buffer.  Every GPU holds
// its own copy of the array at its own address; the address is looked up once per device and kept.  All calls on
// one GPU share the array: calls that overlap on one GPU (two streams, two threads) race on it.
// ----------------------------------------------------------------------------
#define NOALLOC_MAX_M 64           // rows of A (one per sequence of a decode batch): the skinny kernels' range
#define NOALLOC_MAX_N 32768        // rows of B
#define NOALLOC_MAX_K 65536        // contraction length
#define NOALLOC_MAX_TILES 256      // partial tiles of a split-K launch (launch_gemm_skinny*: nblocks * ks <= 256)
#define NOALLOC_TILE_BYTES (2 * 16 * 64 * 4) // largest partial tile: 64 activation rows x 32 weight rows, fp32
#define NOALLOC_SCRATCH_BYTES (GSK_COUNTERS * 4 + NOALLOC_MAX_TILES * NOALLOC_TILE_BYTES) // 4 KiB + 2 MiB
#define NOALLOC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
static void* g_scratchPtr[NOALLOC_MAX_DEVICES]; // per device: the device address of that GPU's copy of `scratch`
static std::mutex g_scratchMutex;

__global__ void k_fill_u32(unsigned* p, unsigned v, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// Looks up the address of this device's copy of the scratch array (once per device, that device current).
static int noalloc_setup(int device, void** out) {
    if (device < 0 || device >= NOALLOC_MAX_DEVICES) { mlh_set_thread_error("device index out of range"); return -1; }
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (!g_scratchPtr[device]) {
        int cur = -1;
        hipError_t e = hipGetDevice(&cur);
        if (e == hipSuccess && cur != device) e = hipSetDevice(device);
        void* p = nullptr;
        if (e == hipSuccess) e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (cur >= 0 && cur != device) (void)hipSetDevice(cur);
        if (e != hipSuccess || !p) {
            mlh_set_thread_error(std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
            return -2;
        }
        g_scratchPtr[device] = p;
    }
    *out = g_scratchPtr[device];
    return 0;
}

extern "C" int mlh_gemm_device_init(int device) {
    void* p;
    return noalloc_setup(device, &p);
}

extern "C" int mlh_gemm_device(int dtype, int M, int N, int K, const void* dA, const void* dB, const float* dR, float* dC,
                               void* stream) {
    if (!dA || !dB || !dC) { mlh_set_thread_error("null operand pointer"); return -1; }
    if (dtype != MLH_DTYPE_F32 && dtype != MLH_DTYPE_BF16 && dtype != MLH_GEMM_F16) { mlh_set_thread_error("unknown operand type"); return -1; }
    if (M <= 0 || N <= 0 || K <= 0) { mlh_set_thread_error("M, N and K must be positive"); return -1; }
    if (M > NOALLOC_MAX_M || N > NOALLOC_MAX_N || K > NOALLOC_MAX_K) {
        mlh_set_thread_error("shape beyond the static workspace: this entry point takes M <= 64, N <= 32768, K <= 65536 "
                         "(got M " + std::to_string(M) + ", N " + std::to_string(N) + ", K " + std::to_string(K) + ")");
        return -1;
    }
    const size_t esz = dtype == MLH_DTYPE_F32 ? 4 : 2;
    if (((size_t)K * esz) % GKB != 0) { mlh_set_thread_error("K * element size must be a multiple of 128 bytes"); return -1; }
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) { mlh_set_thread_error("hipGetDevice failed"); return -2; }
    void* ws = nullptr;
    int rc = noalloc_setup(device, &ws);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    // The counters must start at zero.  A finished launch leaves them at zero, a launch that was cut short may not;
    // a fill kernel rather than hipMemsetAsync, so that the call can be recorded into a graph.
    hipLaunchKernelGGL(k_fill_u32, dim3((GSK_COUNTERS + 255) / 256), dim3(256), 0, st, (unsigned*)ws, 0u, GSK_COUNTERS);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = mlh_gemm_tn_epi(st, dtype, GEMM_EPI_PLAIN, dA, K, dB, K, dC, N, dR, N, M, N, K, ws, 1.0f);
    if (e != hipSuccess) { mlh_set_thread_error(std::string("launch failed: ") + hipGetErrorString(e)); return -2; }
    return 0;
}
