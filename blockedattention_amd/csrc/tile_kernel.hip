// The tile kernel (large segments) as a launch of its own; the workgroup body is tile_body.hpp.
#include <algorithm>

#include "tile_body.hpp"

namespace ba {

template <int DT, bool FUSED, bool F32OUT>
__global__ __launch_bounds__(kTileThreads, 2) void tile_kernel(RunArgs a, int zdim) {
    __shared__ __attribute__((aligned(1024))) unsigned char lds[kStages * kTileChunkBytes];
    tile_block<DT, FUSED, F32OUT>(a, zdim, blockIdx.x, lds);
}

template <int DT, bool FUSED, bool F32OUT>
static void launch_one(const RunArgs &args, unsigned groups, int zdim, hipStream_t stream) {
    hipLaunchKernelGGL((tile_kernel<DT, FUSED, F32OUT>), dim3(groups), dim3(kTileThreads), 0, stream, args, zdim);
}

// Launches the tile kernel over (segment, head, row block).  With a plan summary the row-block
// dimension covers the tallest segment; without it the workgroups loop over row blocks.
int launch_tiles(int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                 hipStream_t stream) {
    static const int use_rowblocks = [] { const char *e = getenv("BLOCKEDATTN_ROWBLOCK"); return e ? atoi(e) : 1; }();
    if (slots <= 0) return BA_OK;
    RunArgs targs = args;
    static const int use_pipe = [] { const char *e = getenv("BLOCKEDATTN_ROWPIPE"); return e ? atoi(e) : 1; }();
    static const int use_wide_k = [] { const char *e = getenv("BLOCKEDATTN_ROWBLOCK_WIDE_K"); return e ? atoi(e) : 1; }();
    const bool rows_ok = use_rowblocks && !(args.flags & kFlagOutF32);      // 16-bit results: the row-block kernels
    // Large segments with 128 < K <= 256: the row-block kernel's build for them, where the summary says the batch may
    // hold some; the kernels launched beside it pass over them.
    const bool wide_ok = rows_ok && use_wide_k && info && info->max_K > 128;
    // nothing left for the tile kernel: every large segment has 128 < K <= 256 (the product alone: see below)
    bool all_taken = wide_ok && info->min_K > 128 && info->max_K <= 256;
    if (rows_ok && fused && !use_pipe && info && info->max_K <= 128)
        return launch_rowblocks(dtype, fused, args, slots, info, stream);     // the kernel before the pipelined one
    if (rows_ok && fused && use_pipe) {
        // The fused pair with 16-bit results: every segment with K <= 128 goes to the pipelined row-block kernel,
        // the others stay here.  The plan counts the former (list_pipe); without the summary both kernels are
        // launched over the whole list and each workgroup keeps to its own kind of segment.
        const int64_t pipe = info ? info->list_pipe : slots;
        if (pipe > 0) {
            const int st = launch_rowpipe(dtype, args, slots, info, stream);
            if (st == BA_OK) {
                if (info && pipe >= slots) return BA_OK;          // nothing left for the tile kernel
                targs.flags |= kFlagPipeToo | kFlagQuiet;
            } else if (st != BA_ERR_UNSUPPORTED) {
                return st;
            }
        }
    } else if (rows_ok && !fused && info) {
        // The product alone: the row-block kernel for K <= 128, its wide build for K <= 256, the tile kernel beyond.
        if (info->max_K <= 128) return launch_rowblocks(dtype, fused, args, slots, info, stream);
        if (wide_ok) {
            all_taken = info->max_K <= 256;
            if (info->min_K <= 128) {
                RunArgs na = args;
                na.flags |= kFlagWideKToo;
                const int st = launch_rowblocks(dtype, fused, na, slots, info, stream);
                if (st == BA_OK) targs.flags |= kFlagRowsToo | kFlagQuiet;
                else if (st != BA_ERR_UNSUPPORTED) return st;
                else all_taken = false;
            }
        }
    }
    if (wide_ok) {
        const int st = launch_rowblocks_wide_k(dtype, fused, targs, slots, info, stream);
        if (st == BA_OK) {
            if (all_taken) return BA_OK;
            targs.flags |= kFlagWideKToo | kFlagQuiet;
        } else if (st != BA_ERR_UNSUPPORTED) {
            return st;
        }
    }
    int64_t z = 4;
    if (info)
        z = std::max<int64_t>(1, std::min<int64_t>(64, (std::max<int64_t>(info->max_M, 1) + kTileRows - 1) / kTileRows));
    const int64_t pairs = (slots + kDies - 1) / kDies * kDies * args.H;   // entries padded to whole dies
    const int64_t groups = pairs * z;
    if (pairs > (int64_t(1) << 30) || groups > (int64_t(1) << 31) - 1) return BA_ERR_UNSUPPORTED;
    const bool f32out = args.flags & kFlagOutF32;
    if (dtype == BA_F16) {
        if (!fused) launch_one<0, false, false>(targs, (unsigned)groups, (int)z, stream);
        else if (f32out) launch_one<0, true, true>(targs, (unsigned)groups, (int)z, stream);
        else launch_one<0, true, false>(targs, (unsigned)groups, (int)z, stream);
    } else if (dtype == BA_BF16) {
        if (!fused) launch_one<1, false, false>(targs, (unsigned)groups, (int)z, stream);
        else if (f32out) launch_one<1, true, true>(targs, (unsigned)groups, (int)z, stream);
        else launch_one<1, true, false>(targs, (unsigned)groups, (int)z, stream);
    } else {
        return BA_ERR_UNSUPPORTED;
    }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
