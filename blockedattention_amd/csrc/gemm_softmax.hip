// Varlen GEMM (S_g = A_g B_g^T) and the fused GEMM + row softmax for fp16/bf16
// on gfx950: MFMA 16x16x32 with fp32 accumulation, scores kept in registers.
// This file holds the two kernels for segments of up to 256 columns and the
// launcher of a whole call; large segments are tile_kernel.hip.
//
//   strip_kernel    strip-class segments whose B_g fits an LDS window: B_g is
//                   copied to LDS once per workgroup, each wavefront computes
//                   16-row strips with code specialised for the exact tile count
//                   and with lane order following memory order (strips_exact).
//   segment_kernel  everything that needs care instead of speed: packs of tiny
//                   segments sharing one MFMA tile (wave_pack), segments that
//                   break the 16-byte operand alignment (K % 8 != 0, odd segment
//                   starts, transposed layouts: element-wise generic_rows),
//                   strip-class leftovers whose B_g is walked in K slabs
//                   (strips_from_lds).
//
// Both operands are K-contiguous (A_g is M x K, B_g is N x K), so a lane's
// eight k-values are one 16-byte load straight into an MFMA operand register;
// no transposition is ever needed.
#include "strip_body.hpp"

namespace ba {

// ------------------------------------------------------------------ kernels
// segment_kernel   grid (segment, head, z): one workgroup per segment and head;
//                  its wavefronts take the segment's 16-row strips (N <= 256),
//                  the pack it leads, or its rows on the element-wise path.
//                  No search: the block index is the segment.
// gemm_large_kernel  GEMM only, N > 256: one wavefront per 16 x 256 piece, found
//                  by a search in the scanned piece counts.
// split_kernel / wide_kernel  fused, N > 256: one 16-wave workgroup per strip.
// The list kernels loop `for (item = first; item < total; item += stride)` with
// the total read from the plan, so any grid size is correct.

// MAXNT = 8 is the build for batches whose widest segment has N <= 128: half the
// accumulator registers, half again as many resident wavefronts.  The host picks it from
// the plan summary; without a summary the 16-tile build runs.
template <int DT, bool FUSED, bool F32OUT, int MAXNT>
__global__ __launch_bounds__(kSegThreads, MAXNT <= 8 ? 6 : 4) void segment_kernel(RunArgs a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const int64_t h = blockIdx.y;
    const bool ok = header_ok(a);
    bool valid;
    const Seg s = load_listed(pv, blockIdx.x, h, a, valid);
    if (!ok) {
        if (!(a.flags & kFlagQuiet)) report_mismatch(a);
        return;
    }
    if (!valid) return;
    const int g = s.index;
    const int kind = s.kind;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int first = blockIdx.z * kSegWaves + wave, stride = gridDim.z * kSegWaves;
    const bool mfma_ok = (a.flags & kFlagMfmaOk) != 0;
    if (kind == kSegEmpty) return;
    if (mfma_ok && a.list < 0 && launch_class(kind, s.M, s.N, s.K) != kListRest) return;   // another kernel's
    if (!mfma_ok || kind == kSegSlow) {
        // Element-wise path.  With MFMA ruled out for the whole launch this also
        // covers the segments the list kernels would have taken.
        for (int r = first; r < s.M; r += stride) generic_seg_rows<DT, FUSED>(s, a, r, r + 1, 0, s.N);
        return;
    }
    if (kind == kSegStrip) {
        // One strip per wavefront; blockIdx.z selects the group of kSegWaves strips.
        const int strips = (s.M + kStripRows - 1) / kStripRows;
        const int nt = (s.N + 15) >> 4;
        for (int base = blockIdx.z * kSegWaves; base < strips; base += gridDim.z * kSegWaves) {
            if (base != (int)blockIdx.z * kSegWaves) __syncthreads();    // LDS is refilled for the next group
            const int strip = base + wave;
            strips_from_lds_dispatch<DT, FUSED, F32OUT, MAXNT>(nt, s, a, lds, a.lds_blocks, strip * kStripRows,
                                                        strip < strips, wave, kSegWaves);
        }
    } else if (kind == kSegPackLead) {
        if (first == 0) wave_pack<DT, FUSED, F32OUT>(pv, g, s.packLen, h, a);
    }
}

// strip_kernel: the strip-class segments whose B_g fits the LDS window, nothing else.
// Grid (segment, head, z); the workgroups with the same (segment, head) share the
// segment's strips round-robin.
// RIDE: the build whose launch also carries the tile kernel's workgroups.  Its grid is flat: the first
// a.tile_groups blocks are tile workgroups (they run longest, so they start first), the rest decode to
// (slot, head, z) with the slot fastest.  Two launches that each fill half the machine become one.
template <int DT, bool FUSED, bool F32OUT, int MAXNT, bool RIDE = false>
__global__ __launch_bounds__(kSegThreads, MAXNT <= 8 ? 4 : 2) void strip_kernel(RunArgs a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    unsigned bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z, gz = gridDim.z;
    if (!RIDE && (a.flags & kFlagHeadFast)) { bx = blockIdx.y; by = blockIdx.x; }
    if constexpr (RIDE) {
        if (bx < (unsigned)a.tile_groups) {
            RunArgs ta = a;
            ta.list = kListTile;
            ta.flags |= kFlagQuiet;
            tile_block<DT, FUSED, F32OUT>(ta, a.tile_zdim, bx, lds);
            return;
        }
        const unsigned lin = bx - (unsigned)a.tile_groups;
        if (a.flags & kFlagHeadFast) {
            by = lin % (unsigned)a.H;
            bx = (lin / (unsigned)a.H) % (unsigned)a.ride_slots;
        } else {
            bx = lin % (unsigned)a.ride_slots;
            by = (lin / (unsigned)a.ride_slots) % (unsigned)a.H;
        }
        bz = lin / ((unsigned)a.ride_slots * (unsigned)a.H);
        gz = (unsigned)a.ride_z;
    }
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const int64_t h = by;
    if (a.mini_first > 0 && bx >= (unsigned)a.mini_first) {
        // The mini entries of the main list (kept at the end of its array, backwards): four to a workgroup, one
        // wavefront and a quarter of the 64 KiB window each, or one workgroup each where the window is smaller.
        const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
        const int count = hdr->mini_count;
        const bool ok = header_ok(a);
        const int wave = uniform((int)(threadIdx.x >> 6));
        const int k = a.mini_solo ? 4 * (int)(bx - (unsigned)a.mini_first) + wave : (int)(bx - (unsigned)a.mini_first);
        // header, count and record are fetched together (the record from a position that exists whatever k is)
        const int64_t cap = plan_cap(a.nseg);
        const SegRec r = load_rec(pv.recs + (int64_t)(kListSmall + 1) * cap, (int)(cap - 1 - min((int64_t)k, cap - 1)));
        if (!ok || k >= count || bz != 0) return;       // (a plan that does not match is reported by the launch's other blocks)
        Seg s;
        s.M = r.M; s.N = r.N; s.K = r.K;
        s.kind = r.kind; s.index = r.index; s.packLen = r.packLen;
        s.a = h * a.Dm1 + r.off1; s.b = h * a.Dm2 + r.off2; s.o = h * a.Dout + r.offO;
        const int tiles = fast_strip_tiles(s.N);
        if (s.kind != kSegStrip || !mini_shape(s.M, s.N, s.K) || tiles > MAXNT) return;
        if (a.mini_solo) strips_solo_dispatch<DT, FUSED, F32OUT>(tiles, s, a, lds + wave * (kMiniBlocks * kLdsBlockBytes));
        else if (strip_blocks(s.N, s.K) <= a.lds_blocks)
            strips_exact_dispatch<DT, FUSED, F32OUT, MAXNT>(tiles, s, a, lds, wave, wave, kSegWaves);
        return;
    }
    if ((a.flags & kFlagSmallToo) && bx >= (unsigned)a.both_split) {
        bx -= (unsigned)a.both_split;
        a.list = kListSmall;
    }
    // header and record are fetched together; nothing waits on the header alone
    const bool ok = header_ok(a);
    bool valid;
    const Seg s = load_listed(pv, bx, h, a, valid);
    if (!ok) {
        if (!(a.flags & kFlagQuiet)) report_mismatch(a);
        return;
    }
    if (!valid) {
        // Blocks behind the kernel's own list: with kFlagPacksToo they take the packs of tiny segments
        // (the rest list then holds nothing but pack leaders), which saves the call a launch.
        if (a.flags & kFlagPacksToo) {
            const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
            const int slot = (int)bx - (int)hdr->totals[a.list], packs = (int)hdr->totals[kListRest];
            if (slot >= 0 && slot < packs && bz == 0 && threadIdx.x < 64) {
                const SegRec r = load_rec(pv.recs + (int64_t)(kListRest + 1) * plan_cap(a.nseg), slot);
                if (r.kind == kSegPackLead) wave_pack<DT, FUSED, F32OUT>(pv, r.index, r.packLen, h, a);
            }
        }
        return;
    }
    const int tiles = fast_strip_tiles(s.N);
    const int need = strip_blocks(s.N, s.K);
    // the lists hold only segments of this kernel; the checks guard against a launch that does not match
    if ((s.kind != kSegStrip) | (need < 1) | (need > a.lds_blocks) | (tiles > MAXNT)) return;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int first = bz * kSegWaves + wave, step = gz * kSegWaves;
    if ((int)bz * kSegWaves * kStripRows >= s.M) return;   // no strip for this workgroup
    strips_exact_dispatch<DT, FUSED, F32OUT, MAXNT>(tiles, s, a, lds, wave, first, step);
}

// --------------------------------------------------------------------- host
// With a host copy of the plan summary the grids cover the work exactly and
// kernels with nothing to do are not launched; without it every kernel is
// launched with a generous grid and reads the counts from the plan.
static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// One call = up to four launches, each walking its own work list of the plan:
//   strip kernel    strip-class segments whose B_g fits its LDS window (main launch: up to 32 KiB;
//                   second launch: up to 64 KiB, fewer resident workgroups)
//   tile kernel     large segments (see tile_segment())
//   segment kernel  packs, the element-wise class, and what the others leave
// With a host copy of the plan summary the grids are exactly the list lengths, empty lists are not
// launched, and launches are merged where that saves one: the packs ride in the first strip launch
// when the rest list holds nothing else, and a modest amount of tile-kernel work rides in the 64 KiB
// strip launch.  Without the summary every kernel is launched over nseg slots and reads its list
// length from the plan.
// The first launch reports a plan that does not match the call; the later ones stay quiet.
template <int DT, bool FUSED, bool F32OUT>
static int launch_set(int dtype, const RunArgs &args_in, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args_in.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    const int cus = device_cu_count();
    const bool mfma_ok = args_in.flags & kFlagMfmaOk;
    const unsigned H = (unsigned)args_in.H;
    if (info) nseg = info->nseg;
    if (nseg <= 0) return BA_OK;
    RunArgs args = args_in;
    const int64_t n_small = !mfma_ok ? 0 : info ? info->list_small : nseg;
    const int64_t n_big = !mfma_ok ? 0 : info ? info->list_big : nseg;
    const int64_t n_tile = !mfma_ok ? 0 : info ? info->list_tile : nseg;
    const int64_t n_rest = !mfma_ok ? nseg : info ? info->list_rest : nseg;
    const int64_t n_mini = !mfma_ok ? 0 : info ? info->list_mini : nseg;    // part of the main strip list, kept apart
    const bool lean = info && info->max_N <= 128;
    // z: enough workgroups to fill the machine, at most one per kSegWaves strips of the tallest segment.  The
    // narrow build (up to eight column tiles, four to five workgroups resident per compute unit) aims at eight
    // workgroups per compute unit; the wide build holds two (64 KiB window) or three (registers), and one round of
    // resident workgroups that loop over their strips beats several rounds of short ones (non-square 512-segment
    // batch: 17.9 us with one workgroup per segment, 19.7 us with four).
    static const int z_env = [] { const char *e = getenv("BLOCKEDATTN_STRIP_Z"); return e ? atoi(e) : 0; }();
    auto strip_z = [&](int64_t slots, int64_t tallest, int per_cu) {
        if (z_env > 0) return (int64_t)z_env;
        if (!info) return (int64_t)2;
        const int64_t groups = ceil_div(ceil_div(std::max<int64_t>(tallest, 1), kStripRows), kSegWaves);
        const int64_t want = ceil_div((int64_t)cus * per_cu, std::max<int64_t>(1, slots * (int64_t)H));
        return std::max<int64_t>(1, std::min<int64_t>(groups, std::min<int64_t>(want, 64)));
    };
    // the rest list is nothing but pack leaders: the first strip launch takes them along
    const bool packs_ride = info && mfma_ok && n_rest > 0 && n_rest == info->pack_items && info->slow_items == 0 &&
                            (n_small > 0 || n_big > 0 || n_mini > 0);
    bool packs_taken = false;
    // a modest amount of tile-kernel work rides in the strip kernel's 64 KiB launch (same LDS, same
    // residency) instead of following it; large tile work keeps its own die-aware launch
    const int64_t tile_z = !info ? 1 : std::max<int64_t>(1, std::min<int64_t>(64, ceil_div(std::max<int64_t>(info->max_M, 1), kTileRows)));
    const int64_t tile_groups = ceil_div(n_tile, kDies) * kDies * (int64_t)H * tile_z;
    const bool tiles_ride = info && n_big > 0 && n_tile > 0 && tile_groups <= 4096 && (dtype == BA_F16 || dtype == BA_BF16);
    bool tiles_taken = false;
    // Both strip lists go in ONE launch with the 64 KiB window, the 64 KiB segments first, where two launches
    // would each be bound by the life of a workgroup rather than by how many are resident: when the main
    // launch's list holds wide segments (more than eight column tiles: three workgroups per compute unit by
    // registers, against two in the 64 KiB launch), or when the batch is small (measured: the non-square
    // 512-segment batch 23.6 -> 19.4 us, the power-law batch 51.2 -> 49.9 us).
    static const int merge_env = [] { const char *e = getenv("BLOCKEDATTN_MERGE_STRIPS"); return e ? atoi(e) : -1; }();
    const bool merge = info && n_small > 0 && n_big > 0 &&
                       (merge_env >= 0 ? merge_env != 0 : info->small_max_N > 128 || (n_small + n_big) * (int64_t)H <= 4096);
    // The mini entries ride in ONE of the strip launches: the merged one, else the main launch if it has entries
    // of its own, else the 64 KiB launch, else a main launch for them alone.
    const int mini_pass = n_mini <= 0 ? -1 : merge ? 1 : n_small > 0 ? 0 : n_big > 0 ? 1 : 0;
    static const int solo_env = [] { const char *e = getenv("BLOCKEDATTN_MINI_SOLO"); return e ? atoi(e) : 1; }();
    for (int pass = 0; pass < 2; ++pass) {
        int64_t slots = pass == 0 ? n_small : n_big;
        if ((slots <= 0 && pass != mini_pass) || (merge && pass == 0)) continue;
        RunArgs fa = args;
        if (merge) {
            fa.flags |= kFlagSmallToo;
            fa.both_split = (int)n_big;
            slots += n_small;
        }
        if (packs_ride && !packs_taken) {
            fa.flags |= kFlagPacksToo;
            slots += n_rest;
            packs_taken = true;
        }
        const bool ride = pass == 1 && tiles_ride;
        if (ride) {
            fa.flags |= kFlagTilesToo;
            fa.tile_zdim = (int)tile_z;
            fa.tile_groups = (int)tile_groups;
            fa.ride_slots = (int)slots;
            fa.ride_z = (int)strip_z(slots, info->max_M, 2);
            tiles_taken = true;
        }
        fa.list = pass == 0 ? kListSmall : kListBig;
        fa.lds_blocks = pass == 0 ? kFastBlocks : kBigBlocks;
        bool lean_pass = lean;
        if (info && pass == 0 && !merge) {
            // the main launch is sized by ITS widest and tallest segment, not the batch's
            const int64_t nt = fast_strip_tiles((int)std::max(info->small_max_N, 1));
            const int64_t nks = ceil_div(std::max<int64_t>(info->max_K, 1), 32);
            fa.lds_blocks = (int)std::min<int64_t>(kFastBlocks, nt * nks);
            lean_pass = info->small_max_N <= 128;
        }
        if (pass == mini_pass) {
            // four mini segments to a workgroup where the window has a quarter for each of them
            fa.mini_first = (int)std::max<int64_t>(slots, 1);
            fa.mini_solo = solo_env && info && fa.lds_blocks >= 4 * kMiniBlocks ? 1 : 0;
            slots = fa.mini_first + (fa.mini_solo ? ceil_div(n_mini, kSegWaves) : n_mini);
            if (ride) fa.ride_slots = (int)slots;
        }
        const int64_t tallest = !info ? 0 : pass == 0 ? info->small_max_M : info->max_M;
        const dim3 grid((unsigned)slots, H, (unsigned)strip_z(slots, tallest, lean_pass ? 8 : pass == 0 ? 3 : 2));
        // room for the copy of the ragged run behind the image of B_g, while the total stays within 64 KiB
        fa.lds_extra = fa.lds_blocks * kLdsBlockBytes + kRaggedCopyBytes <= 65536 ? kRaggedCopyBytes : 0;
        const size_t lds_bytes = (size_t)fa.lds_blocks * kLdsBlockBytes + fa.lds_extra;
        // Head as the fastest index of the grid: consecutive workgroups are the heads of one list entry, so
        // workgroups that start together have one shape and take equally long, and (with the list in work
        // buckets) the longest start first.  Measured against entry-fastest order: 256 x 8 heads fused 15.6 ->
        // 14.9 us, GEMM only 15.5 -> 13.6 us; power-law batch fused 49.3 -> 46.7 us.
        static const int hf = [] { const char *e = getenv("BLOCKEDATTN_HEAD_FAST"); return e ? atoi(e) : 1; }();
        const bool head_fast = hf && (ride || slots <= 65535);      // heads on gridDim.x, entries on gridDim.y
        if (head_fast) fa.flags |= kFlagHeadFast;
        const dim3 grid_hf(H, (unsigned)slots, grid.z);
        if (ride)
            hipLaunchKernelGGL((strip_kernel<DT, FUSED, F32OUT, 16, true>),
                               dim3((unsigned)(tile_groups + slots * (int64_t)H * fa.ride_z)), dim3(kSegThreads), lds_bytes,
                               stream, fa);
        else if (lean_pass)
            hipLaunchKernelGGL((strip_kernel<DT, FUSED, F32OUT, 8>), head_fast ? grid_hf : grid, dim3(kSegThreads), lds_bytes,
                               stream, fa);
        else
            hipLaunchKernelGGL((strip_kernel<DT, FUSED, F32OUT, 16>), head_fast ? grid_hf : grid, dim3(kSegThreads), lds_bytes,
                               stream, fa);
        args.flags |= kFlagQuiet;
    }
    if (n_tile > 0 && !tiles_taken) {
        RunArgs ta = args;
        ta.list = kListTile;
        const int st = launch_tiles(dtype, FUSED ? 1 : 0, ta, n_tile, info, stream);
        if (st != BA_OK) return st;
        args.flags |= kFlagQuiet;
    }
    if (n_rest > 0 && !packs_taken) {
        // z spreads the 16-row strips (or rows) of the largest segment over workgroups
        int64_t z = 4, blocks = 32;
        if (info) {
            const int64_t units = mfma_ok && info->slow_items == 0 ? ceil_div(std::min<int64_t>(info->max_M, 256), kStripRows)
                                                                     : std::min<int64_t>(info->max_M, 4096);
            z = std::max<int64_t>(1, std::min<int64_t>(64, ceil_div(units, kSegWaves)));
            // LDS window for B_g: whole B_g of the largest strip-class segment if it fits 64 KiB
            const int64_t nt = ceil_div(std::min<int64_t>(std::max<int64_t>(info->max_N, 1), kWaveCols), 16);
            const int64_t nks = ceil_div(std::max<int64_t>(info->max_K, 1), 32);
            blocks = std::max<int64_t>(nt, std::min<int64_t>(nt * nks, 64));
        }
        RunArgs seg_args = args;
        seg_args.list = mfma_ok ? kListRest : -1;
        seg_args.lds_blocks = (int)blocks;
        const dim3 grid((unsigned)n_rest, H, (unsigned)z);
        const size_t lds_bytes = (size_t)blocks * kLdsBlockBytes;
        if (lean)
            hipLaunchKernelGGL((segment_kernel<DT, FUSED, F32OUT, 8>), grid, dim3(kSegThreads), lds_bytes, stream,
                               seg_args);
        else
            hipLaunchKernelGGL((segment_kernel<DT, FUSED, F32OUT, 16>), grid, dim3(kSegThreads), lds_bytes, stream,
                               seg_args);
    }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_strips(int dtype, int fused, const RunArgs &args, int64_t nseg, const ba_plan_info *info,
                  hipStream_t stream) {
    const bool f32out = args.flags & kFlagOutF32;
    if (dtype == BA_F16) {
        if (!fused) return launch_set<0, false, false>(dtype, args, nseg, info, stream);
        return f32out ? launch_set<0, true, true>(dtype, args, nseg, info, stream)
                      : launch_set<0, true, false>(dtype, args, nseg, info, stream);
    }
    if (dtype == BA_BF16) {
        if (!fused) return launch_set<1, false, false>(dtype, args, nseg, info, stream);
        return f32out ? launch_set<1, true, true>(dtype, args, nseg, info, stream)
                      : launch_set<1, true, false>(dtype, args, nseg, info, stream);
    }
    return BA_ERR_UNSUPPORTED;
}

}  // namespace ba
