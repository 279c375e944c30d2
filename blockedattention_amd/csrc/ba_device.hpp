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
// The same through the two half-swaps of the register file (lanes 32.. of one register against lanes ..31 of
// another, then odd rows of 16 against even rows): after each, the two registers hold both partners' values
// in every lane.  No LDS round trip; the s_nop covers the distance a swap needs from the write of its operands.
__device__ __forceinline__ float quad_column_max_swap(float v) {
    float w;
    asm volatile("v_mov_b32 %1, %0\n\ts_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_max_f32 %0, %0, %1\n\t"
                 "v_mov_b32 %1, %0\n\ts_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_max_f32 %0, %0, %1"
                 : "+v"(v), "=&v"(w));
    return v;
}
__device__ __forceinline__ float quad_column_sum(float v) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

// Full-wave reductions (all 64 lanes end with the result): data-parallel-primitive row shifts and row
// broadcasts accumulate into lane 63, which is then read back as a scalar.  No LDS round trips.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_or(float v, float identity) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity),
                                                                 __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf,
                                                                 false));
}
__device__ __forceinline__ float wave_max(float v) {
    const float lowest = -INFINITY;
    v = fmaxf(v, dpp_or<0x111, 0xf>(v, lowest));   // row_shr:1
    v = fmaxf(v, dpp_or<0x112, 0xf>(v, lowest));   // row_shr:2
    v = fmaxf(v, dpp_or<0x114, 0xf>(v, lowest));   // row_shr:4
    v = fmaxf(v, dpp_or<0x118, 0xf>(v, lowest));   // row_shr:8
    v = fmaxf(v, dpp_or<0x142, 0xa>(v, lowest));   // row_bcast:15 into rows 1 and 3
    v = fmaxf(v, dpp_or<0x143, 0xc>(v, lowest));   // row_bcast:31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_or<0x111, 0xf>(v, 0.f);
    v += dpp_or<0x112, 0xf>(v, 0.f);
    v += dpp_or<0x114, 0xf>(v, 0.f);
    v += dpp_or<0x118, 0xf>(v, 0.f);
    v += dpp_or<0x142, 0xa>(v, 0.f);
    v += dpp_or<0x143, 0xc>(v, 0.f);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
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

// ------------------------------------------------------------ plan access
// The plan is read-only while the compute kernels run, so it is read through
// the constant address space: the loads become scalar loads (one per
// wavefront, no vector registers, low latency).
typedef const __attribute__((address_space(4))) int32_t *ConstI32;
typedef const __attribute__((address_space(4))) int64_t *ConstI64;
typedef const __attribute__((address_space(4))) SegRec *ConstSeg;
typedef const __attribute__((address_space(4))) PlanHeader *ConstHdr;

struct PlanRO {
    ConstHdr hdr;
    ConstSeg recs;
    ConstSeg list[kNumLists];
};

__device__ __forceinline__ PlanRO plan_ro(const void *buf, int nseg) {
    PlanRO v;
    const size_t cap = (size_t)plan_cap(nseg);
    uintptr_t p = (uintptr_t)buf;
    v.hdr = (ConstHdr)p; p += sizeof(PlanHeader);
    v.recs = (ConstSeg)p; p += cap * sizeof(SegRec);
    for (int i = 0; i < kNumLists; ++i) { v.list[i] = (ConstSeg)p; p += cap * sizeof(SegRec); }
    return v;
}

// One segment record, field by field (scalar loads when g is wave-uniform).
__device__ __forceinline__ SegRec load_rec(ConstSeg recs, int g) {
    const ConstI64 q = (ConstI64)(recs + g);
    const ConstI32 w = (ConstI32)(recs + g);
    SegRec r;
    r.off1 = q[0]; r.off2 = q[1]; r.offO = q[2];
    r.M = w[6]; r.N = w[7]; r.K = w[8]; r.packLen = w[9]; r.kind = w[10]; r.index = w[11];
    return r;
}

// Largest g in [0, n) with pfx[g] <= i, for an exclusive prefix array with
// pfx[n] = total and 0 <= i < total (segments with no items are skipped).
// 64-ary search: every lane tests one pivot per round, so 4096 segments take
// two dependent loads instead of twelve.  The result is wave-uniform.
template <typename PfxPtr> __device__ __forceinline__ int prefix_search(PfxPtr pfx, int n, int i) {
    const int lane = lane_id();
    int lo = 0, len = n;   // the answer lies in [lo, lo + len)
    while (len > 1) {
        const int step = (len + 63) >> 6;
        const int idx = lo + (lane + 1) * step;
        const bool le = idx < lo + len && pfx[idx] <= i;
        const int cnt = __builtin_popcountll(__ballot(le));
        const int end = lo + len;
        lo += cnt * step;
        len = min(step, end - lo);
    }
    return uniform(lo);
}

// ---------------------------------------------------------------- DPP scans
// Inclusive prefix sum across the 64 lanes with data-parallel-primitive moves
// (row shifts inside each 16-lane row, then two row broadcasts); no LDS traffic.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ int dpp_or_zero(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ int wave_inclusive_scan(int v) {
    v += dpp_or_zero<0x111, 0xf>(v);   // row_shr:1
    v += dpp_or_zero<0x112, 0xf>(v);   // row_shr:2
    v += dpp_or_zero<0x114, 0xf>(v);   // row_shr:4
    v += dpp_or_zero<0x118, 0xf>(v);   // row_shr:8
    v += dpp_or_zero<0x142, 0xa>(v);   // row_bcast:15 into rows 1 and 3
    v += dpp_or_zero<0x143, 0xc>(v);   // row_bcast:31 into rows 2 and 3
    return v;
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ int64_t dpp64_or_zero(int64_t v) {
    const uint32_t lo = (uint32_t)dpp_or_zero<CTRL, ROW_MASK>((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)dpp_or_zero<CTRL, ROW_MASK>((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int64_t wave_inclusive_scan(int64_t v) {
    v += dpp64_or_zero<0x111, 0xf>(v);
    v += dpp64_or_zero<0x112, 0xf>(v);
    v += dpp64_or_zero<0x114, 0xf>(v);
    v += dpp64_or_zero<0x118, 0xf>(v);
    v += dpp64_or_zero<0x142, 0xa>(v);
    v += dpp64_or_zero<0x143, 0xc>(v);
    return v;
}
// Inclusive scan inside every row of 16 lanes (four independent scans per wavefront).
__device__ __forceinline__ int row16_inclusive_scan(int v) {
    v += dpp_or_zero<0x111, 0xf>(v);
    v += dpp_or_zero<0x112, 0xf>(v);
    v += dpp_or_zero<0x114, 0xf>(v);
    v += dpp_or_zero<0x118, 0xf>(v);
    return v;
}
__device__ __forceinline__ int64_t row16_inclusive_scan(int64_t v) {
    v += dpp64_or_zero<0x111, 0xf>(v);
    v += dpp64_or_zero<0x112, 0xf>(v);
    v += dpp64_or_zero<0x114, 0xf>(v);
    v += dpp64_or_zero<0x118, 0xf>(v);
    return v;
}
// Maximum of non-negative ints over the wavefront (result in every lane).
__device__ __forceinline__ int wave_max_nonneg(int v) {
    v = max(v, dpp_or_zero<0x111, 0xf>(v));
    v = max(v, dpp_or_zero<0x112, 0xf>(v));
    v = max(v, dpp_or_zero<0x114, 0xf>(v));
    v = max(v, dpp_or_zero<0x118, 0xf>(v));
    v = max(v, dpp_or_zero<0x142, 0xa>(v));
    v = max(v, dpp_or_zero<0x143, 0xc>(v));
    return __builtin_amdgcn_readlane(v, 63);
}

}  // namespace ba
