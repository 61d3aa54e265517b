// Device-side helpers shared by the kernels: element conversion, wavefront reductions, DPP moves.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fhip {

typedef _Float16 half_t;
struct bf16_t {
    uint16_t bits;
};

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(half_t x) { return (float)x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float((uint32_t)x.bits << 16); }

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) {
    return x;
}
template <>
__device__ __forceinline__ half_t from_float<half_t>(float x) {
    return (half_t)x;  // round to nearest even
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
    uint32_t u = __float_as_uint(x);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r.bits = (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
        r.bits = (uint16_t)(u >> 16);
    }
    return r;
}

// Orders this wavefront's LDS writes before its later LDS reads (no workgroup barrier).
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the vector-memory
// counter, i.e. it waits for every global load in flight, which would serialise a tile prefetch
// with the math it is meant to overlap.
// The scheduling fences keep register-only work (e.g. a softmax tail) from drifting across the
// barrier into the neighbouring phase.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// value of `x` in lane `l`, l uniform across the wavefront
__device__ __forceinline__ float read_lane(float x, int l) {
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), l));
}

// DPP move: returns x from the lane selected by `ctrl` within the row of 16 lanes
template <int ctrl>
__device__ __forceinline__ float dpp_mov(float x) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), ctrl, 0xf, 0xf, true));
}
constexpr int DPP_QUAD_XOR1 = 0xB1;    // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;    // quad_perm [2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// sum over each aligned group of 4 / 8 / 16 / 32 lanes, result in every lane of the group
__device__ __forceinline__ float group_sum4(float x) {
    x += dpp_mov<DPP_QUAD_XOR1>(x);
    x += dpp_mov<DPP_QUAD_XOR2>(x);
    return x;
}
__device__ __forceinline__ float group_sum8(float x) {
    x = group_sum4(x);
    x += dpp_mov<DPP_ROW_HALF_MIRROR>(x);
    return x;
}
__device__ __forceinline__ float group_sum16(float x) {
    x = group_sum8(x);
    x += dpp_mov<DPP_ROW_MIRROR>(x);
    return x;
}
__device__ __forceinline__ float group_sum32(float x) {
    x = group_sum16(x);
    x += __shfl_xor(x, 16, 64);
    return x;
}

template <int ctrl>
__device__ __forceinline__ int dpp_mov_i(int x) {
    return (int)__builtin_amdgcn_update_dpp(0u, (uint32_t)x, ctrl, 0xf, 0xf, true);
}
// reduction over the 64 lanes of a wavefront, result in every lane: four DPP steps inside the rows of 16 lanes, two
// swaps across them (no LDS traffic, unlike __shfl_xor)
template <typename OP>
__device__ __forceinline__ int wave_reduce_i(int x, OP op) {
    x = op(x, dpp_mov_i<DPP_QUAD_XOR1>(x));
    x = op(x, dpp_mov_i<DPP_QUAD_XOR2>(x));
    x = op(x, dpp_mov_i<DPP_ROW_HALF_MIRROR>(x));
    x = op(x, dpp_mov_i<DPP_ROW_MIRROR>(x));
    auto a = __builtin_amdgcn_permlane16_swap((uint32_t)x, (uint32_t)x, false, false);
    x = op((int)a[0], (int)a[1]);
    auto b = __builtin_amdgcn_permlane32_swap((uint32_t)x, (uint32_t)x, false, false);
    return op((int)b[0], (int)b[1]);
}

}  // namespace fhip
