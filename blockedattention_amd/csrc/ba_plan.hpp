// Plan: the device-resident result of the segment scheduler.  One contiguous
// buffer; every compute kernel takes only this pointer plus the data pointers.
//
//   PlanHeader                    (256 bytes)
//   SegRec recs[cap]              one 48-byte record per segment: offsets and shape
//   int32 prefix arrays, each [cap+4]   scanned work-item counts, one array per kind
//
// cap = nseg rounded up so that every array starts 16-byte aligned.  The
// compute kernels read the plan through scalar loads (it is never written
// while they run, except the run_errors counter nobody reads back on the device).
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace ba {

constexpr uint32_t kPlanMagic = 0xB10CA77Eu;
constexpr int kStripRows = 16;    // rows of one work item (one MFMA tile high)
constexpr int kWaveCols = 256;    // columns one wavefront keeps in registers (16 MFMA tiles)
constexpr int kWavesPerGroup = 16;
constexpr int kSplitCols = kWaveCols * kWavesPerGroup;  // 4096: columns one workgroup keeps in registers
constexpr int kPackDim = 16;      // a pack of tiny segments fits one 16x16 MFMA tile

// Strip-class segments whose whole B_g fits the strip kernel's LDS window: G =
// the even tile count covering N, G * ceil(K/32) operand blocks of 1 KiB.
constexpr int kFastBlocks = 32;
constexpr int kFastSteps = 4;     // k-steps of 32 whose A fragments a wavefront holds
__host__ __device__ inline int fast_strip_tiles(int N) { return 2 * ((N + 31) >> 5); }
__host__ __device__ inline bool fast_strip_shape(int N, int K) {
    const int nks = (K + 31) >> 5;
    return N >= 2 && N <= kWaveCols && nks >= 1 && nks <= kFastSteps && fast_strip_tiles(N) * nks <= kFastBlocks;
}

// Kinds of scanned work-item counts.  Every kind except kPfxRows and kPfxSlow
// counts aligned segments only (see below).
enum PrefixKind {
    kPfxGemm = 0,   // GEMM only, N > 256: ceil(M/16) * ceil(N/256) per segment
    kPfxStrip = 1,  // fused, N <= 256 and not packed: ceil(M/16)
    kPfxSplit = 2,  // fused, 256 < N <= 4096: ceil(M/16)
    kPfxWide = 3,   // fused, N > 4096: ceil(M/16)
    kPfxRows = 4,   // softmax: M rows
    kPfxPack = 5,   // 1 for the first segment of a pack of tiny segments, else 0
    kPfxSlow = 6,   // ceil(M/16) for segments the 16-byte operand loads cannot serve
    kNumPrefix = 7
};

// A segment is "aligned" when K % 8 == 0 and its A and B offsets are multiples
// of 8 elements: every operand row then starts on a 16-byte boundary (given
// 16-byte aligned base pointers and per-head strides that are multiples of 8).
// Only aligned segments are counted in kPfxGemm/Strip/Split/Wide/Pack; the
// others are counted in kPfxSlow and take the element-wise path.

struct PlanHeader {
    uint32_t magic;
    int32_t nseg;
    int32_t cap;
    int32_t kind;            // 0 = GEMM plan, 1 = softmax plan
    int64_t Dm1, Dm2, Dout;
    int64_t total_rows;
    int64_t totals[8];       // last entry of each prefix array
    int32_t max_M, max_N, max_K;
    int32_t bad_segments;
    int32_t run_errors;      // bumped by kernels that refuse to run
    int32_t strip_rest;      // strip-class segments that do not fit the strip kernel's LDS window
    int32_t pad_[30];
};
static_assert(sizeof(PlanHeader) == 256, "PlanHeader must stay 256 bytes");

__host__ __device__ inline int64_t plan_cap(int64_t nseg) { return (nseg + 4) & ~int64_t(3); }

// How a segment is processed.
enum SegKind : int32_t {
    kSegEmpty = 0,       // no rows or no columns: no work
    kSegStrip = 1,       // aligned, N <= 256: one wavefront per 16-row strip, scores in registers
    kSegPackLead = 2,    // first segment of a pack of tiny segments sharing one MFMA tile
    kSegPackFollow = 3,  // later member of a pack (processed with its leader)
    kSegSplit = 4,       // aligned, 256 < N <= 4096
    kSegWide = 5,        // aligned, N > 4096
    kSegSlow = 6         // not 16-byte aligned (K % 8, odd offsets) or too large for 32-bit offsets
};

// Segments the tile kernel takes: N > 256, or strip-class segments too large for the strip
// kernel's LDS window that have at least one full chunk of columns.
constexpr int kTileCols = 128;
__host__ __device__ inline bool tile_segment(int kind, int N, int K) {
    if (kind == kSegSplit || kind == kSegWide) return true;
    return kind == kSegStrip && !fast_strip_shape(N, K) && N >= kTileCols;
}

// Everything a kernel needs to know about one segment, in one aligned record
// (three 16-byte scalar loads).
struct alignas(16) SegRec {
    int64_t off1, off2, offO;   // element offsets of the segment in A, B and out (per head)
    int32_t M, N, K;
    int32_t packLen;            // > 0: first segment of a pack of this many segments
    int32_t kind;               // SegKind
    int32_t pad_;
};
static_assert(sizeof(SegRec) == 48, "SegRec must stay 48 bytes");

struct PlanView {
    PlanHeader *hdr;
    SegRec *recs;
    int32_t *pfx[kNumPrefix];
};

__host__ __device__ inline size_t plan_bytes_for(int64_t nseg) {
    const size_t cap = (size_t)plan_cap(nseg);
    return sizeof(PlanHeader) + cap * sizeof(SegRec) + kNumPrefix * (cap + 4) * sizeof(int32_t);
}

__host__ __device__ inline PlanView plan_view(void *buf, int64_t nseg) {
    PlanView v;
    const size_t cap = (size_t)plan_cap(nseg);
    char *p = (char *)buf;
    v.hdr = (PlanHeader *)p; p += sizeof(PlanHeader);
    v.recs = (SegRec *)p; p += cap * sizeof(SegRec);
    for (int i = 0; i < kNumPrefix; ++i) { v.pfx[i] = (int32_t *)p; p += (cap + 4) * sizeof(int32_t); }
    return v;
}

}  // namespace ba
