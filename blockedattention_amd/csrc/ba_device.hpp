// Device helpers shared by the gfx950 kernels: 16-bit element traits, MFMA
// wrappers, cross-lane reductions, prefix search.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ba_plan.hpp"

namespace ba {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;

// ---------------------------------------------------------------- elements
// DT 0 = fp16, 1 = bf16.  Storage is always uint16_t; the traits turn bits
// into floats and back (round to nearest even) and issue the MFMA.
template <int DT> struct Elem;

template <> struct Elem<0> {
    static __device__ __forceinline__ float to_float(uint16_t b) {
        return (float)__builtin_bit_cast(_Float16, b);
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    // D[m][n] += sum_k a[m][k] * b[n][k] with a-lane (m = lane%16, k = 8*(lane/16)..+8),
    // b-lane (n = lane%16, same k); the lane then holds D[4*(lane/16)+i][lane%16].
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                      0, 0, 0);
    }
};

template <> struct Elem<1> {
    static __device__ __forceinline__ float to_float(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        b2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
    }
};

// --------------------------------------------------------------- cross-lane
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63); }

// Values of the four lanes that share lane%16 (lane, lane^16, lane^32, lane^48).
__device__ __forceinline__ float quad_column_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ __forceinline__ float quad_column_sum(float v) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

// Full-wave reductions (all 64 lanes end with the result).
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// Values that are the same in every lane of the wavefront by construction
// (derived from the work-item index) are pinned into scalar registers, so that
// buffer descriptors and scalar offsets built from them need no per-lane handling.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Largest g in [0, n) with pfx[g] <= i, for an exclusive prefix array with
// pfx[n] = total and 0 <= i < total.  Segments with no items are skipped.
__device__ __forceinline__ int prefix_search(const int32_t *__restrict__ pfx, int n, int i) {
    int lo = 0, hi = n;  // invariant: pfx[lo] <= i < pfx[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (pfx[mid] <= i) lo = mid; else hi = mid;
    }
    return lo;
}

}  // namespace ba
