// Plan: the device-resident result of the segment scheduler.  One contiguous
// buffer; every compute kernel takes only this pointer plus the data pointers.
//
//   PlanHeader                    (256 bytes)
//   SegRec recs[cap]              one 48-byte record per segment: offsets and shape
//   SegRec lists[5][cap]          the records of each launch class once more, compacted (work lists)
//   int32  rowblocks[2][cap + 4]  GEMM plans: exclusive prefix over the segments of their row blocks of 64 and of
//                                 128 rows (the one-pass attention's work items); entry nseg = all of them
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

// Strip-class segments whose whole B_g fits the strip kernel's LDS window: G = the
// even tile count covering N, G * ceil(K/32) operand blocks of 1 KiB.  Segments
// needing up to kFastBlocks blocks run in the main launch; those needing up to
// kBigBlocks run in a second launch with a larger window (fewer resident
// workgroups, so it is kept apart from the many small segments).
constexpr int kFastBlocks = 32;
constexpr int kBigBlocks = 64;
constexpr int kFastSteps = 4;     // k-steps of 32 whose A fragments a wavefront holds
__host__ __device__ inline int fast_strip_tiles(int N) { return 2 * ((N + 31) >> 5); }
// LDS blocks the strip kernel needs for an N x K operand, or 0 if the shape is not its kind.
__host__ __device__ inline int strip_blocks(int N, int K) {
    const int nks = (K + 31) >> 5;
    if (N < 2 || N > kWaveCols || nks < 1 || nks > kFastSteps) return 0;
    return fast_strip_tiles(N) * nks;
}
__host__ __device__ inline bool fast_strip_shape(int N, int K) {
    const int b = strip_blocks(N, K);
    return b >= 1 && b <= kBigBlocks;
}

// What the scheduler scans per segment.  The first five are 0/1 class flags whose
// scan compacts the segment indices into one work list per launch (the arrays of
// the plan hold those lists); the others are work-item counts of which only the
// totals are kept (plan summary).
constexpr int kRunCols = 256;     // widest row of the softmax lane-run kernel; wider rows take the row kernel

enum PrefixKind {
    kListSmall = 0,  // strip-class segments for the strip kernel's main launch (<= kFastBlocks LDS blocks)
    kListBig = 1,    // strip-class segments for its second launch (<= kBigBlocks)
    kListTile = 2,   // segments of the tile kernel
    kListRest = 3,   // everything else that has work: pack leaders, element-wise class, leftovers
    kListRows = 4,   // segments of the softmax row kernel: N > kRunCols, any plan kind (independent of the four above)
    kNumLists = 5,
    kPfxGemm = 5,   // GEMM only, N > 256: ceil(M/16) * ceil(N/256) per segment
    kPfxStrip = 6,  // fused, N <= 256 and not packed: ceil(M/16)
    kPfxSplit = 7,  // fused, 256 < N <= 4096: ceil(M/16)
    kPfxWide = 8,   // fused, N > 4096: ceil(M/16)
    kPfxRows = 9,   // softmax: M rows
    kPfxPack = 10,  // 1 for the first segment of a pack of tiny segments, else 0
    kPfxSlow = 11,  // ceil(M/16) for segments the 16-byte operand loads cannot serve
    kPfxAtt64 = 12,   // GEMM plans: ceil(M/64) for every segment with rows (one-pass attention, any-layout GEMM)
    kPfxAtt128 = 13,  // the same in row blocks of 128
    kPfxMini = 14,    // 1 for a segment of the strip kernel's main list that is small enough for one wavefront
    kPfxPipe = 15,    // 1 for a segment of the tile list that the pipelined row-block kernel can take (fused call)
    kNumPrefix = 16
};

// "Mini" segments: strip-class segments of at most 64 rows whose B_g needs at most kMiniBlocks LDS blocks and at most
// eight column tiles.  One wavefront can take such a segment on its own (a quarter of a 64 KiB window), so four of
// them share a workgroup where the launch has that window.  They belong to the main strip list, but are kept
// apart from its other entries: entry k of them sits at position cap - 1 - k of that list's array (from the end
// backwards), totals[kListSmall] counts the others, PlanHeader::mini_count these.
constexpr int kMiniBlocks = 16;
constexpr int kMiniRows = 64;
__host__ __device__ inline bool mini_shape(int M, int N, int K) {
    const int b = strip_blocks(N, K);
    return M >= 1 && M <= kMiniRows && b >= 1 && b <= kMiniBlocks && fast_strip_tiles(N) <= 8;
}
constexpr int kMailboxTicket = 256;   // byte offset of the ticket word in a scheduler mailbox (behind the header copy)
constexpr int kAttBlockRows = 64;   // kPfxAtt64 counts blocks of this many rows, kPfxAtt128 of twice as many

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
    int64_t totals[12];      // totals of the scanned quantities (PrefixKind)
    int32_t max_M, max_N, max_K;
    int32_t bad_segments;
    int32_t run_errors;      // bumped by kernels that refuse to run
    int32_t small_max_N, small_max_M;   // maxima over the segments of the strip kernel's main launch
    int32_t att_blocks64, att_blocks128;   // totals of kPfxAtt64 / kPfxAtt128: the one-pass attention's row blocks per head
    int32_t mini_count;      // total of kPfxMini
    int32_t pipe_count;      // total of kPfxPipe
    int32_t pipe_groups;     // bumped by every workgroup of the pipelined row-block kernel that found work in this plan
    int32_t min_N, min_K;    // smallest N and K over the segments that have rows and columns (0: there is none)
    int32_t ring_groups;     // bumped by every workgroup of the any-layout GEMM that wrote its rows through the LDS ring
    int32_t wide_groups;     // bumped by every workgroup of the row-block kernel's build for 128 < K <= 256 that found work
    int32_t pad_[12];
};
static_assert(sizeof(PlanHeader) == 256, "PlanHeader must stay 256 bytes");

__host__ __device__ constexpr int64_t plan_cap(int64_t nseg) { return (nseg + 4) & ~int64_t(3); }

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

// Segments of the tile list that the pipelined row-block kernel takes in a fused call with 16-bit results: the A
// fragments of a wavefront's 64 rows stay in registers (K <= 128) and the chunk pipeline is five chunks of 64
// columns deep.
__host__ __device__ inline bool pipe_segment(int kind, int N, int K) {
    return tile_segment(kind, N, K) && K <= 128 && N > 4 * 64;
}
// Segments of the tile list that the row-block kernel's build for 128 < K <= 256 takes (16-bit results) where the
// call launches it.
__host__ __device__ inline bool wide_k_segment(int kind, int N, int K) {
    return tile_segment(kind, N, K) && K > 128 && K <= 256;
}

// Launch class (work list) of a segment of a GEMM plan, or -1 for none.
__host__ __device__ inline int launch_class(int kind, int M, int N, int K) {
    if (kind == kSegEmpty || kind == kSegPackFollow || M < 1 || N < 1) return -1;
    if (kind == kSegStrip) {
        const int b = strip_blocks(N, K);
        if (b >= 1 && b <= kFastBlocks) return kListSmall;
        if (b > kFastBlocks && b <= kBigBlocks) return kListBig;
    }
    if (tile_segment(kind, N, K)) return kListTile;
    return kListRest;
}

// Everything a kernel needs to know about one segment, in one aligned record
// (three 16-byte scalar loads).
struct alignas(16) SegRec {
    int64_t off1, off2, offO;   // element offsets of the segment in A, B and out (per head)
    int32_t M, N, K;
    int32_t packLen;            // > 0: first segment of a pack of this many segments
    int32_t kind;               // SegKind
    int32_t index;              // the segment's index g (records are also kept compacted per launch class)
};
static_assert(sizeof(SegRec) == 48, "SegRec must stay 48 bytes");

struct PlanView {
    PlanHeader *hdr;
    SegRec *recs;
    SegRec *list[kNumLists];    // records of one launch class, compacted, in segment order
};

__host__ __device__ constexpr size_t plan_lists_end(int64_t nseg) {
    return sizeof(PlanHeader) + (1 + kNumLists) * (size_t)plan_cap(nseg) * sizeof(SegRec);
}
__host__ __device__ constexpr size_t plan_bytes_for(int64_t nseg) {
    return plan_lists_end(nseg) + 2 * ((size_t)plan_cap(nseg) + 4) * sizeof(int32_t);     // cap is a multiple of 4
}
// Row-block prefix `which` (0: blocks of 64 rows, 1: of 128): entry g = blocks of the segments before g,
// entry nseg = all.
__host__ __device__ inline int32_t *plan_rowblocks(void *buf, int64_t nseg, int which) {
    return (int32_t *)((char *)buf + plan_lists_end(nseg)) + (size_t)which * ((size_t)plan_cap(nseg) + 4);
}

__host__ __device__ inline PlanView plan_view(void *buf, int64_t nseg) {
    PlanView v;
    const size_t cap = (size_t)plan_cap(nseg);
    char *p = (char *)buf;
    v.hdr = (PlanHeader *)p; p += sizeof(PlanHeader);
    v.recs = (SegRec *)p; p += cap * sizeof(SegRec);
    for (int i = 0; i < kNumLists; ++i) { v.list[i] = (SegRec *)p; p += cap * sizeof(SegRec); }
    return v;
}

}  // namespace ba
