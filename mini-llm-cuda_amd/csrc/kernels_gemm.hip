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

#include "mlh_internal.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define GT 128            // tile rows (M) and columns (N)
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
};
template <> struct GemmTraits<bf16_t> {
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};

// lda/ldb in elements; K * sizeof(T) must be a multiple of 128.  R may be null, and may alias C.
template <typename T>
__global__ void __launch_bounds__(GTHREADS) k_gemm_tn(const T* __restrict__ A, int lda, const T* __restrict__ B, int ldb,
                                                      float* C, int ldc, const float* R, int ldr, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) unsigned char As[GT * GLD];
    __shared__ __attribute__((aligned(16))) unsigned char Bs[GT * GLD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    const int nslices = (int)(((size_t)K * sizeof(T)) / GKB);
    const unsigned char* Ab = reinterpret_cast<const unsigned char*>(A);
    const unsigned char* Bb = reinterpret_cast<const unsigned char*>(B);
    const size_t ldaB = (size_t)lda * sizeof(T), ldbB = (size_t)ldb * sizeof(T);

    // global -> register staging: 128 rows x 8 pieces of 16 bytes per operand, 4 pieces per thread each
    int rowA[4], rowB[4], piece[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int id = tid + GTHREADS * i;
        const int r = id >> 3;
        piece[i] = id & 7;
        rowA[i] = min(m0 + r, M - 1); // rows past the edge repeat the last row; their results are never stored
        rowB[i] = min(n0 + r, N - 1);
    }
    u32x4 ra[4], rb[4];
    auto load_slice = [&](int s) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            ra[i] = *reinterpret_cast<const u32x4*>(Ab + (size_t)rowA[i] * ldaB + (size_t)s * GKB + piece[i] * 16);
            rb[i] = *reinterpret_cast<const u32x4*>(Bb + (size_t)rowB[i] * ldbB + (size_t)s * GKB + piece[i] * 16);
        }
    };
    auto store_slice = [&]() {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int id = tid + GTHREADS * i;
            *reinterpret_cast<u32x4*>(As + (id >> 3) * GLD + piece[i] * 16) = ra[i];
            *reinterpret_cast<u32x4*>(Bs + (id >> 3) * GLD + piece[i] * 16) = rb[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = (f32x16)(0.f);

    load_slice(0);
    store_slice();
    __syncthreads();
    const int half = lane >> 5, lrow = lane & 31;
    for (int s = 0; s < nslices; s++) {
        if (s + 1 < nslices) load_slice(s + 1);
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            u32x4 fa[2], fb[2];
#pragma unroll
            for (int b = 0; b < 2; b++) {
                fa[b] = *reinterpret_cast<const u32x4*>(As + (wm * 64 + b * 32 + lrow) * GLD + (2 * jj + half) * 16);
                fb[b] = *reinterpret_cast<const u32x4*>(Bs + (wn * 64 + b * 32 + lrow) * GLD + (2 * jj + half) * 16);
            }
#pragma unroll
            for (int bm = 0; bm < 2; bm++)
#pragma unroll
                for (int bn = 0; bn < 2; bn++) GemmTraits<T>::mma(fa[bm], fb[bn], acc[bm][bn]);
        }
        __syncthreads();
        if (s + 1 < nslices) {
            store_slice();
            __syncthreads();
        }
    }

    // accumulator layout of the 32x32 tile: element i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32
#pragma unroll
    for (int bm = 0; bm < 2; bm++)
#pragma unroll
        for (int bn = 0; bn < 2; bn++) {
            const int col = n0 + wn * 64 + bn * 32 + lrow;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = m0 + wm * 64 + bm * 32 + 8 * (i >> 2) + 4 * half + (i & 3);
                if (row < M && col < N) {
                    float v = acc[bm][bn][i];
                    if (R) v += R[(size_t)row * ldr + col];
                    C[(size_t)row * ldc + col] = v;
                }
            }
        }
}

// Enqueues the GEMM on `stream`.  Returns hipSuccess, or an error when the shape is not supported.
hipError_t mlh_gemm_tn(hipStream_t stream, int dtype, const void* A, int lda, const void* B, int ldb, float* C, int ldc,
                       const float* R, int ldr, int M, int N, int K) {
    const size_t esz = dtype == MLH_DTYPE_BF16 ? 2 : 4;
    if (M <= 0 || N <= 0 || K <= 0 || ((size_t)K * esz) % GKB != 0 || ((size_t)lda * esz) % 16 != 0 || ((size_t)ldb * esz) % 16 != 0)
        return hipErrorInvalidValue;
    const dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
    if (dtype == MLH_DTYPE_BF16)
        hipLaunchKernelGGL((k_gemm_tn<bf16_t>), grid, dim3(GTHREADS), 0, stream, (const bf16_t*)A, lda, (const bf16_t*)B, ldb, C, ldc, R, ldr, M, N, K);
    else
        hipLaunchKernelGGL((k_gemm_tn<float>), grid, dim3(GTHREADS), 0, stream, (const float*)A, lda, (const float*)B, ldb, C, ldc, R, ldr, M, N, K);
    return hipGetLastError();
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

// Stand-alone check and timing of the GEMM kernel: host fp32 inputs (rounded to bf16 first when
// dtype says so), result back on the host, mean launch time over `iters` launches from HIP events.
extern "C" int mlh_selftest_gemm(int dtype, int M, int N, int K, const float* A, const float* B, const float* R, float* C,
                                 int iters, double* avgUs) {
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return -1;
    if (mlh_device_count() <= 0) return -1;
    const size_t esz = dtype == MLH_DTYPE_BF16 ? 2 : 4;
    void *dA = nullptr, *dB = nullptr;
    float *dC = nullptr, *dR = nullptr;
    int rc = 0;
    std::vector<bf16_t> ha, hb;
    const void *srcA = A, *srcB = B;
    if (dtype == MLH_DTYPE_BF16) {
        ha.resize((size_t)M * K); hb.resize((size_t)N * K);
        host_to_bf16(A, ha.data(), ha.size()); host_to_bf16(B, hb.data(), hb.size());
        srcA = ha.data(); srcB = hb.data();
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
#define ST(x) do { if ((x) != hipSuccess) { rc = -2; goto done; } } while (0)
    ST(hipMalloc(&dA, (size_t)M * K * esz)); ST(hipMalloc(&dB, (size_t)N * K * esz));
    ST(hipMalloc((void**)&dC, (size_t)M * N * 4));
    if (R) { ST(hipMalloc((void**)&dR, (size_t)M * N * 4)); ST(hipMemcpy(dR, R, (size_t)M * N * 4, hipMemcpyHostToDevice)); }
    ST(hipMemcpy(dA, srcA, (size_t)M * K * esz, hipMemcpyHostToDevice));
    ST(hipMemcpy(dB, srcB, (size_t)N * K * esz, hipMemcpyHostToDevice));
    ST(mlh_gemm_tn(nullptr, dtype, dA, K, dB, K, dC, N, dR, N, M, N, K));
    ST(hipDeviceSynchronize());
    if (iters > 0 && avgUs) {
        ST(hipEventCreate(&e0)); ST(hipEventCreate(&e1));
        ST(hipEventRecord(e0, nullptr));
        for (int i = 0; i < iters; i++) ST(mlh_gemm_tn(nullptr, dtype, dA, K, dB, K, dC, N, dR, N, M, N, K));
        ST(hipEventRecord(e1, nullptr));
        ST(hipEventSynchronize(e1));
        float ms = 0.f;
        ST(hipEventElapsedTime(&ms, e0, e1));
        *avgUs = (double)ms * 1000.0 / iters;
    }
    ST(hipMemcpy(C, dC, (size_t)M * N * 4, hipMemcpyDeviceToHost));
#undef ST
done:
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(dA); (void)hipFree(dB); (void)hipFree(dC); (void)hipFree(dR);
    return rc;
}
