// Device helpers shared by the persistent batch-1 decode kernels (not part of the C ABI).
#pragma once

#include "mlh_internal.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float ald(const float* p) {
    return __uint_as_float(__hip_atomic_load(reinterpret_cast<const unsigned*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ void ast(float* p, float v) {
    __hip_atomic_store(reinterpret_cast<unsigned*>(p), __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned aldu(const unsigned* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void astu(unsigned* p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load (loads and stores share one counter on this ISA), which would serialise the weight
// prefetch with each barrier; inside this kernel threads of a workgroup exchange data through LDS only.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Wave-wide reductions on the data-parallel-primitive path of the vector ALU (a handful of cycles per step) instead of
// LDS-crossbar shuffles (a hundred-odd cycles each): within rows of 16 lanes by quad permutes and mirrors, across the
// four rows by row broadcasts; lane 63 then holds the result and every lane receives it through a scalar register.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v, float fill) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float pwave_sum(float v) {
    v += dpp_move<0xB1, 0xf>(v, 0.f);  // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xf>(v, 0.f);  // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xf>(v, 0.f); // row_half_mirror
    v += dpp_move<0x140, 0xf>(v, 0.f); // row_mirror: every lane holds the sum of its row
    v += dpp_move<0x142, 0xa>(v, 0.f); // row_bcast15 into rows 1 and 3
    v += dpp_move<0x143, 0xc>(v, 0.f); // row_bcast31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
// Sum within aligned groups of W = 8 or 16 lanes; every lane of a group receives it.
template <int W>
__device__ __forceinline__ float pgroup_sum(float v) {
    static_assert(W == 8 || W == 16, "group of 8 or 16 lanes");
    v += dpp_move<0xB1, 0xf>(v, 0.f);
    v += dpp_move<0x4E, 0xf>(v, 0.f);
    v += dpp_move<0x141, 0xf>(v, 0.f);
    if (W == 16) v += dpp_move<0x140, 0xf>(v, 0.f);
    return v;
}
__device__ __forceinline__ float pwave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x4E, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x141, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x140, 0xf>(v, v));
    v = fmaxf(v, dpp_move<0x142, 0xa>(v, v));
    v = fmaxf(v, dpp_move<0x143, 0xc>(v, v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float psigmoid(float v) { return 1.0f / (1.0f + expf(-v)); } // inference.cu:248
__device__ __forceinline__ float psilu(float v) { return v / (1.0f + expf(-v)); }       // inference.cu:270

// Weight element access: 16-byte vectors, fp32 (4 values) or bf16 (8 values).
template <typename WT> struct PVec;
template <> struct PVec<float> {
    static constexpr int N = 4;
    typedef f32x4 Raw;
    static __device__ __forceinline__ Raw load(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
    static __device__ __forceinline__ void unpack(const Raw& v, float (&o)[4]) { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
    static __device__ __forceinline__ float one(const float* p) { return *p; }
};
template <> struct PVec<bf16_t> {
    static constexpr int N = 8;
    typedef u32x4 Raw;
    static __device__ __forceinline__ Raw load(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
    static __device__ __forceinline__ void unpack(const Raw& v, float (&o)[8]) {
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    static __device__ __forceinline__ float one(const bf16_t* p) { return __uint_as_float(((uint32_t)*p) << 16); }
};

