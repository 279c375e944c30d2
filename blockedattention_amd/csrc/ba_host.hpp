// Host-side declarations shared by the translation units of libblockedattn_hip.so.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/blocked_attention.h"
#include "ba_plan.hpp"

namespace ba {

// Flags passed to the compute kernels.
enum RunFlags : int {
    kFlagTranspose1 = 1,   // A segments stored K x M
    kFlagTranspose2 = 2,   // B segments stored K x N
    kFlagMfmaOk = 4,       // layouts, base pointers and head strides allow 16-byte operand loads
    kFlagOutF32 = 8,       // fused path writes fp32 probabilities
    kFlagPacksToo = 16,    // strip kernel: the blocks behind its own list walk the pack leaders of the rest list
    kFlagTilesToo = 32,    // strip kernel, 64 KiB launch: further blocks run the tile kernel's workgroups (tile_zdim, tile_groups)
    kFlagQuiet = 64,       // an earlier launch of the same call reports a plan that does not match
    kFlagSmallToo = 128,   // strip kernel, 64 KiB launch: the slots from both_split on walk the main launch's list
    kFlagHeadFast = 256,   // strip kernel: grid (head, slot, z) instead of (slot, head, z)
    kFlagPipeToo = 512,    // tile kernel: the pipelined row-block kernel runs in the same call and takes its segments
    kFlagRingToo = 1024,   // any-layout GEMM: the ring kernel runs in the same call and takes its segments
    kFlagWideKToo = 2048,  // tile and row-block kernel: the row-block kernel's build for 128 < K <= 256 runs in the same call and takes its segments
    kFlagRowsToo = 4096    // tile kernel: the row-block kernel runs in the same call and takes the large segments with K <= 128
};

struct RunArgs {
    void *plan;
    const void *A;
    const void *B;
    void *out;
    int64_t H, Dm1, Dm2, Dout;
    float scale;
    int flags;
    int lds_blocks;   // 1 KiB operand blocks of dynamic LDS given to the segment / strip kernel
    int list;         // work list the launch walks (PrefixKind), or -1: every segment, by block index
    int nseg;         // segment count the plan was built for (checked against the plan)
    int lds_extra;    // bytes of dynamic LDS behind the operand blocks (strip kernel: copy of the ragged run)
    int tile_zdim;    // with kFlagTilesToo: row-block dimension and number of workgroups of the tile kernel,
    int tile_groups;  // which take the first tile_groups blocks of a flat grid; the strip part then has
    int ride_slots;   // ride_slots x H x ride_z workgroups, slot fastest
    int ride_z;
    int both_split;   // with kFlagSmallToo: length of the launch's own list; slot s >= both_split is entry s - both_split of the small list
    int mini_first;   // strip kernel: first slot of the mini entries of the main list (0: the launch carries none) ...
    int mini_solo;    // ... 1: four to a workgroup, one wavefront each (64 KiB window); 0: one workgroup each
};

int launch_schedule(void *plan, size_t plan_bytes, int64_t nseg, int mode, int kind, int64_t *M, int64_t *N,
                    int64_t *K, int64_t *a1, int64_t *a2, int64_t *aO, hipStream_t stream, void *mailbox = nullptr,
                    uint32_t ticket = 0);

// mode 0 = GEMM only, 1 = fused GEMM + softmax.  dtype BA_F16 / BA_BF16.
// info: optional host copy of the plan summary (from ba_plan_read), or nullptr.
int launch_strips(int dtype, int fused, const RunArgs &args, int64_t nseg, const ba_plan_info *info,
                  hipStream_t stream);
// The tile kernel over the large segments (see tile_segment()); slots = length of its work list (or nseg).
int launch_tiles(int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                 hipStream_t stream);
// The row-block kernel over the same list (large segments, K <= 128, 16-bit output): whole-line stores.
// BA_ERR_UNSUPPORTED when the plan summary is missing or does not fit; the caller then takes launch_tiles.
int launch_rowblocks(int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                     hipStream_t stream);
// Its build for 128 < K <= 256 over the same list; workgroups of other segments leave at once.
int launch_rowblocks_wide_k(int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                            hipStream_t stream);
// The pipelined row-block kernel (rowpipe_kernel.hip): the fused pair over the same list, two sweeps of adjacent
// row blocks sharing one stream of B_g.  Same conditions as launch_rowblocks.
int launch_rowpipe(int dtype, const RunArgs &args, int64_t slots, const ba_plan_info *info, hipStream_t stream);
// fp16 / bf16 in any layout and alignment (gemm_any16.hip: both operands staged through LDS, MFMA)
// Fused GEMM + softmax of a batch of at most kOneCallMaxSegments segments in one launch that reads the metadata
// itself (mode 0: sizes given, prefix sums written; mode 2: both given); no plan.  Every workgroup redoes the
// scheduler's sums and runs with the widest build's registers and LDS window, so it only pays while the batch has
// few (segment, head) pairs: measured against scheduler + plan-driven kernels, 64 segments x 1 head 4.5 against
// 8.3 us, 256 x 2 heads 9.2 against 12.9, 256 x 4 equal (16.5 / 16.2), 256 x 8 30.5 against 21.0.
constexpr int kOneCallMaxSegments = 512;
constexpr int kOneCallMaxPairs = 1024;
// ... and while the call is short enough for a launch to matter: with more than 2^24 results or operand values
// (32 MiB of 16-bit data, at least some 10 us of kernel) the plan-driven kernels' better fit to the batch (work
// order, row-block kernels for large segments, the lean build) is worth more than the launch saved.
constexpr int64_t kOneCallMaxElements = int64_t(1) << 24;
int launch_onecall(int dtype, const RunArgs &args, int mode, const int64_t *M, const int64_t *N, const int64_t *K,
                   int64_t *a1, int64_t *a2, int64_t *aO, hipStream_t stream);
int launch_gemm_any16(int dtype, const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream);
// Two such calls with the layouts of the backward pass (a: B operand k-major; b: both operands k-major) as ONE launch
// where both take the 64 x 64 build; BA_ERR_UNSUPPORTED (nothing launched) otherwise.
int launch_gemm_any16_two(int dtype, const RunArgs &a, const ba_plan_info *info_a, const RunArgs &b, const ba_plan_info *info_b,
                          hipStream_t stream);
// fp32, fp64 and the integer types (gemm_generic.hip); dtype: ba_dtype
int launch_gemm_generic(int dtype, const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream);
int launch_softmax(int dtype, void *plan, int64_t nseg, const void *src, void *dst, int64_t H, int64_t Dsrc,
                   float scale, const ba_plan_info *info, hipStream_t stream);

int launch_softmax_backward(int dtype, void *plan, int64_t nseg, const void *y, const void *dy, void *dx, int64_t H,
                            int64_t Dsrc, float scale, const ba_plan_info *info, hipStream_t stream);

// Varlen attention O = softmax(scale Q K^T) V without the probabilities in memory (see attention.hip).
// args.A = Q, args.B = K, args.out = O ([H, Dm1]); V has K's layout.
int launch_attention(int dtype, const RunArgs &args, const void *V, int64_t nseg, const ba_plan_info *info,
                     hipStream_t stream);

// Number of compute units of the current device (cached per device).
int device_cu_count();

}  // namespace ba
