// Device code shared by the MFMA kernels (strip, segment and tile kernels):
// segment views, buffer descriptors, plan checks, cross-lane reductions.
#pragma once
#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

struct Seg {
    int M, N, K;
    int kind, index, packLen;   // SegKind, segment index g, pack length (leaders)
    int64_t a, b, o;  // element offsets of the segment inside A, B, out (head included)
};

// Buffer resources of one segment.  Operand loads go through a raw buffer
// descriptor whose range is exactly the segment: the address is one 32-bit lane
// offset plus a scalar offset, and anything past the segment's end (rows >= M
// of a ragged strip, columns >= N of a ragged tile) reads as zero instead of
// being clamped in code.
struct SegRes {
    __amdgpu_buffer_rsrc_t a, b;
};

constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family)

__device__ __forceinline__ SegRes make_res(const Seg &s, const void *A, const void *B) {
    SegRes r;
    r.a = __builtin_amdgcn_make_buffer_rsrc((void *)((const uint16_t *)A + s.a), 0, s.M * s.K * 2, kRsrcFlags);
    r.b = __builtin_amdgcn_make_buffer_rsrc((void *)((const uint16_t *)B + s.b), 0, s.N * s.K * 2, kRsrcFlags);
    return r;
}

// The compiler pads the distance between a matrix instruction and ITS OWN vector instructions that
// read the result registers; instructions inside inline assembly (max3 below, the DPP reductions) get
// no such padding, and one that reads an accumulator too soon after the last MFMA sees what the
// register held before.  Call this between the MFMAs and the first inline-assembly read of acc: the
// accumulators pass through 24 idle cycles (the longest write-back distance of these MFMAs is 18).
template <int N>
__device__ __forceinline__ void settle_mfma(f32x4 (&acc)[N]) {
#pragma unroll
    for (int g = 0; g < N; g += 8) {
        if constexpr (N >= 8) {
            const int b = g + 8 <= N ? g : N - 8;           // the last group may overlap the one before
            asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7"
                         : "+v"(acc[b]), "+v"(acc[b + 1]), "+v"(acc[b + 2]), "+v"(acc[b + 3]), "+v"(acc[b + 4]),
                           "+v"(acc[b + 5]), "+v"(acc[b + 6]), "+v"(acc[b + 7]));
        } else {
#pragma unroll
            for (int k = 0; k + 1 < N; ++k) asm volatile("" : "+v"(acc[k]));
            asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(acc[N - 1]));
        }
    }
}

__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;   // one instruction for two new elements; fmaxf() would add a canonicalising max per operand
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}


typedef u32x2 __attribute__((aligned(2))) u32x2_unaligned;
typedef f32x4 __attribute__((aligned(4))) f32x4_unaligned;
typedef u32x4 __attribute__((aligned(2))) u32x4_unaligned;
typedef uint32_t __attribute__((aligned(2))) u32_unaligned;
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef f32x2 __attribute__((aligned(4))) f32x2_unaligned;

// Results are written once and not read again by the kernel that writes them.  As ordinary stores they delay the
// kernel's own reads (the operand fills of a large-segment kernel wait behind its write stream: 2500 cycles per
// chunk against 540 with the stores compiled out); as NON-TEMPORAL stores they do so much less -- where
// a kernel writes whole lines.  Measured per kernel, non-temporal against ordinary stores: pipelined row-block
// kernel 1365 / 1478 us and the product alone 1000 / 1206 us (16 x 16 pairs of 1024..4096 rows), lane-run softmax
// 12.2 / 13.4 us (256 x 8 heads); but the any-layout GEMM 2226 / 1663 us (its 8- and 16-byte pieces end in partial
// lines, which ordinary stores merge in L2), the tile kernel 2320 / 1940 us (rows at any 2-byte phase, 16-byte pieces)
// and the softmax row kernel 1620 / 1549 us: those keep ordinary stores.  The strip kernel's runs of 4 N values per
// instruction: 512 segments of 16..256 rows and columns 17.05 / 17.45 us, the other batches equal.
// kResultAux is the policy bit for the buffer-store builtins.
constexpr int kResultAux = 2;
template <bool NT, typename P, typename V> __device__ __forceinline__ void store_result(P *p, V v) {
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}
// Reductions over the 16 lanes of a row group (lanes 16*rg .. 16*rg+15) with
// data-parallel-primitive row rotations: x = op(rotate(x), x) for rotations by 8,
// 4, 2, 1, after which every lane holds the result.  Four independent values go
// through the steps side by side, which also keeps a rotation three instructions
// away from the write of its source (the hardware needs two).
#define BA_ROT_STEP(OP, ROT)                                                   \
    OP " %0, %0, %0 row_ror:" #ROT " row_mask:0xf bank_mask:0xf\n"            \
    OP " %1, %1, %1 row_ror:" #ROT " row_mask:0xf bank_mask:0xf\n"            \
    OP " %2, %2, %2 row_ror:" #ROT " row_mask:0xf bank_mask:0xf\n"            \
    OP " %3, %3, %3 row_ror:" #ROT " row_mask:0xf bank_mask:0xf\n"
#define BA_ROT_REDUCE(OP)                                                                      \
    asm("s_nop 1\n" BA_ROT_STEP(OP, 8) BA_ROT_STEP(OP, 4) BA_ROT_STEP(OP, 2) BA_ROT_STEP(OP, 1) \
        : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]))
__device__ __forceinline__ void row16_max4(float (&x)[4]) { BA_ROT_REDUCE("v_max_f32_dpp"); }
__device__ __forceinline__ void row16_sum4(float (&x)[4]) { BA_ROT_REDUCE("v_add_f32_dpp"); }
#undef BA_ROT_REDUCE
#undef BA_ROT_STEP

// Row softmax over values laid out as "lane runs": lane (j = lane%16, rg = lane/16) holds G
// consecutive columns (index g) of four rows (index e) in acc[g][e]; the sixteen lanes of a row group
// together hold whole rows.  In: scores, c >= 0 (scale * log2 e), w[g] in {0, 1} = whether the
// column counts in the row sum (0 for columns a neighbouring lane also holds, or that do not exist;
// such columns must hold a value that does not exceed the row maximum).  Out: probabilities.
// FROM_MFMA: acc comes straight out of matrix instructions (see settle_mfma).
template <int G, bool FROM_MFMA = true>
__device__ __forceinline__ void softmax_lane_runs(f32x4 (&acc)[G], const float (&w)[G], float c) {
    if constexpr (FROM_MFMA) settle_mfma(acc);
    float ext[4], sum[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        ext[e] = acc[0][e];
#pragma unroll
        for (int g = 1; g + 1 < G; g += 2) ext[e] = max3(ext[e], acc[g][e], acc[g + 1][e]);
        ext[e] = max3(ext[e], acc[G - 1][e], acc[G - 1][e]);
    }
    row16_max4(ext);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float bias = -((__builtin_fabsf(ext[e]) == INFINITY) ? 0.f : ext[e]) * c;
        sum[e] = 0.f;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float pr = __builtin_amdgcn_exp2f(fmaf(acc[g][e], c, bias));
            acc[g][e] = pr;
            sum[e] = fmaf(pr, w[g], sum[e]);
        }
    }
    row16_sum4(sum);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float inv = __builtin_amdgcn_rcpf(sum[e]);
#pragma unroll
        for (int g = 0; g < G; ++g) acc[g][e] *= inv;
    }
}

// One row (register index e) of a lane's run of G values to memory as the widest stores; the address
// may have any element alignment.
template <int DT, int G, bool F32OUT, bool NT>
__device__ __forceinline__ void store_run(char *dst, const f32x4 (&acc)[G], int e) {
    if constexpr (!F32OUT) {
        uint32_t w[G / 2];
#pragma unroll
        for (int k = 0; k < G / 2; ++k) w[k] = Elem<DT>::pack2(acc[2 * k][e], acc[2 * k + 1][e]);
#pragma unroll
        for (int k = 0; k + 4 <= G / 2; k += 4)
            store_result<NT>(reinterpret_cast<u32x4_unaligned *>(dst + 4 * k), u32x4{w[k], w[k + 1], w[k + 2], w[k + 3]});
        constexpr int kDone = (G / 2) & ~3;
        if constexpr (((G / 2) & 2) != 0)
            store_result<NT>(reinterpret_cast<u32x2_unaligned *>(dst + 4 * kDone), u32x2{w[kDone], w[kDone + 1]});
        if constexpr (((G / 2) & 1) != 0) store_result<NT>(reinterpret_cast<u32_unaligned *>(dst + 4 * (G / 2 - 1)), w[G / 2 - 1]);
    } else {
#pragma unroll
        for (int k = 0; k + 4 <= G; k += 4)
            store_result<NT>(reinterpret_cast<f32x4_unaligned *>(dst + 4 * k),
                         f32x4{acc[k][e], acc[k + 1][e], acc[k + 2][e], acc[k + 3][e]});
        if constexpr ((G & 2) != 0)
            store_result<NT>(reinterpret_cast<f32x2_unaligned *>(dst + 4 * (G - 2)), f32x2{acc[G - 2][e], acc[G - 1][e]});
    }
}

// The same through a buffer descriptor: `off` is a byte offset inside the descriptor's range, or any value outside
// it for a lane that has nothing to store (the hardware drops the store): no branch around the stores, so a loop that
// loads at its top and stores at its bottom stays one block of straight-line code and the wait in front of the first
// use of what it loaded counts the stores as still in flight instead of waiting for them.
template <int DT, int G, bool F32OUT>
__device__ __forceinline__ void store_run_buf(__amdgpu_buffer_rsrc_t res, uint32_t off, const f32x4 (&acc)[G], int e) {
    if constexpr (!F32OUT) {
        uint32_t w[G / 2];
#pragma unroll
        for (int k = 0; k < G / 2; ++k) w[k] = Elem<DT>::pack2(acc[2 * k][e], acc[2 * k + 1][e]);
#pragma unroll
        for (int k = 0; k + 4 <= G / 2; k += 4)
            __builtin_amdgcn_raw_buffer_store_b128(u32x4{w[k], w[k + 1], w[k + 2], w[k + 3]}, res, off + 4 * k, 0, kResultAux);
        constexpr int kDone = (G / 2) & ~3;
        if constexpr (((G / 2) & 2) != 0)
            __builtin_amdgcn_raw_buffer_store_b64(u32x2{w[kDone], w[kDone + 1]}, res, off + 4 * kDone, 0, kResultAux);
        if constexpr (((G / 2) & 1) != 0) __builtin_amdgcn_raw_buffer_store_b32(w[G / 2 - 1], res, off + 4 * (G / 2 - 1), 0, kResultAux);
    } else {
#pragma unroll
        for (int k = 0; k + 4 <= G; k += 4)
            __builtin_amdgcn_raw_buffer_store_b128(
                __builtin_bit_cast(u32x4, f32x4{acc[k][e], acc[k + 1][e], acc[k + 2][e], acc[k + 3][e]}), res, off + 4 * k, 0, kResultAux);
        if constexpr ((G & 2) != 0)
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, f32x2{acc[G - 2][e], acc[G - 1][e]}), res,
                                                  off + 4 * (G - 2), 0, kResultAux);
    }
}

__device__ __forceinline__ Seg load_seg(const PlanRO &pv, int g, int64_t h, const RunArgs &a) {
    const SegRec r = load_rec(pv.recs, g);   // scalar loads
    Seg s;
    s.M = r.M; s.N = r.N; s.K = r.K;
    s.kind = r.kind; s.index = r.index; s.packLen = r.packLen;
    s.a = h * a.Dm1 + r.off1;
    s.b = h * a.Dm2 + r.off2;
    s.o = h * a.Dout + r.offO;
    return s;
}

// Segment of a workgroup: entry `slot` of the launch's work list (a compacted copy of the records), or
// segment `slot` itself when the launch walks every segment.  The record load does not wait for the list
// length: slots never exceed the arrays.  valid = false past the end of the list.
__device__ __forceinline__ Seg load_listed(const PlanRO &pv, int slot, int64_t h, const RunArgs &a, bool &valid) {
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const int count = a.list < 0 ? a.nseg : (int)hdr->totals[a.list < 0 ? 0 : a.list];
    // the lists follow the per-segment records back to back, cap records each: list -1 is the records themselves
    const SegRec r = load_rec(pv.recs + (int64_t)(a.list + 1) * plan_cap(a.nseg), slot);
    valid = slot < count;
    Seg s;
    s.M = r.M; s.N = r.N; s.K = r.K;
    s.kind = r.kind; s.index = r.index; s.packLen = r.packLen;
    s.a = h * a.Dm1 + r.off1;
    s.b = h * a.Dm2 + r.off2;
    s.o = h * a.Dout + r.offO;
    return s;
}

// The header fields every kernel checks, fetched as one batch of scalar loads
// (no branch between them).  The segment count comes with the launch, so the
// addresses of the plan's arrays do not wait for the header either.
__device__ __forceinline__ bool header_ok(const RunArgs &a) {
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const uint32_t magic = hdr->magic;
    const int nseg = hdr->nseg, kind = hdr->kind, bad = hdr->bad_segments;
    const int64_t d1 = hdr->Dm1, d2 = hdr->Dm2, dO = hdr->Dout;
    return (magic == kPlanMagic) & (nseg == a.nseg) & (kind == 0) & (bad == 0) & (d1 == a.Dm1) & (d2 == a.Dm2) &
           (dO == a.Dout);
}
__device__ __forceinline__ void report_mismatch(const RunArgs &a) {
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
        atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
}

}  // namespace ba
