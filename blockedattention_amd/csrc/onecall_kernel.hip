// Fused GEMM + softmax of a small batch (at most 512 segments) in ONE launch, without a plan: every
// workgroup derives its own segment's offsets and class from the metadata arrays in registers, then runs
// the same device bodies as the plan-driven kernels (strip, tile, leftover-strip or element-wise).
//
// Grid (head, segment, z).  The first wavefront of a workgroup reads the whole metadata (one entry per lane
// and round of 64 segments, every load issued before the first is used), applies the scheduler's acceptance
// rules, and reduces what the workgroup needs across the lanes: the segment's three offsets (sums over the
// segments before it), the three totals, the scan weight and whether any segment was rejected; the other
// wavefronts take the result from LDS.  That is the work of the scheduler's one workgroup redone by every
// workgroup: a few hundred instructions, against a launch of its own plus a round trip through memory.  It pays
// while the batch has few workgroups; the host falls back to scheduler + plan-driven kernels beyond that.
// Workgroup (0, 0, 0) also writes the prefix-sum arrays the scheduler would have written.  The differences
// from a plan-driven call: tiny segments are not joined into packs (each is a strip-class segment of its
// own), the segments run in index order, not in work order, and every workgroup has the 64 KiB window and the
// 16-tile build's registers, whatever the widest segment is (the host does not know it).
#include "strip_body.hpp"

namespace ba {

struct MetaArgs {
    const int64_t *M, *N, *K;
    int64_t *a1, *a2, *aO;
    int mode;     // ba_meta_mode: 0 sizes given, offsets produced; 2 both given
    int rounds;   // 64-segment rounds walked: 1 up to 64 segments, 4 up to 256, else 8 (the scheduler's thread counts)
};

__device__ __forceinline__ int64_t readlane64(int64_t v, int l) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, l);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), l);
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int64_t wave_total(int64_t v) { return readlane64(wave_inclusive_scan(v), 63); }

template <int DT, bool F32OUT>
__global__ __launch_bounds__(kSegThreads, 2) void onecall_kernel(RunArgs a, MetaArgs m) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const int64_t h = blockIdx.x;
    const int g0 = blockIdx.y, bz = blockIdx.z, gz = gridDim.z;
    const int lane = lane_id();
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int nseg = a.nseg;
    const bool offsets_given = m.mode != 0;
    int64_t *box = reinterpret_cast<int64_t *>(lds);      // wavefront 0 -> the others: offsets, sizes, verdict
    if (wave == 0) {
        const bool writer = blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && !offsets_given;
        constexpr int kRounds = kOneCallMaxSegments / 64;
        // every load first (one round trip), then the arithmetic
        int64_t mm[kRounds], nn[kRounds], kk[kRounds], s1[kRounds], s2[kRounds], sO[kRounds], e1[kRounds], e2[kRounds],
            eO[kRounds];
#pragma unroll
        for (int q = 0; q < kRounds; ++q) {
            const int g = 64 * q + lane;
            const bool live = q < m.rounds && g < nseg;
            mm[q] = live ? m.M[g] : 0; nn[q] = live ? m.N[g] : 0; kk[q] = live ? m.K[g] : 0;
            s1[q] = s2[q] = sO[q] = e1[q] = e2[q] = eO[q] = 0;
            if (offsets_given && live) {
                s1[q] = m.a1[g]; s2[q] = m.a2[g]; sO[q] = m.aO[g];
                e1[q] = m.a1[g + 1]; e2[q] = m.a2[g + 1]; eO[q] = m.aO[g + 1];
            }
        }
        int64_t pre1 = 0, pre2 = 0, preO = 0, tot1 = 0, tot2 = 0, totO = 0, weight = 0;
        int64_t my_m = 0, my_n = 0, my_k = 0;
        bool any_bad = false;
        int nbad = 0;
#pragma unroll
        for (int q = 0; q < kRounds; ++q) {
            if (q >= m.rounds) break;
            const int g = 64 * q + lane;
            const bool live = g < nseg;
            bool bad = false;
            if (live) {
                if (offsets_given)
                    bad = sO[q] < 0 || eO[q] - sO[q] < mm[q] * nn[q] || s1[q] < 0 || s2[q] < 0 ||
                          e1[q] - s1[q] < mm[q] * kk[q] || e2[q] - s2[q] < nn[q] * kk[q];
                // the scheduler's limits: every dimension and every area of a segment below 2^30
                const int64_t lim = int64_t(1) << 30;
                bad = bad || mm[q] < 0 || nn[q] < 0 || kk[q] < 0 || mm[q] >= lim || nn[q] >= lim || kk[q] >= lim;
                bad = bad || mm[q] * kk[q] >= lim || nn[q] * kk[q] >= lim || mm[q] * nn[q] >= lim;
                if (bad) { mm[q] = nn[q] = kk[q] = 0; }
            }
            nbad += __builtin_popcountll(__ballot(bad));
            any_bad = nbad != 0;
            const int64_t v1 = mm[q] * kk[q], v2 = nn[q] * kk[q], vO = mm[q] * nn[q];
            const int32_t mi = (int32_t)mm[q], ni = (int32_t)nn[q];
            const int32_t strips = ni >= 1 ? (mi + kStripRows - 1) / kStripRows : 0;
            const int32_t chunks = (ni + kWaveCols - 1) / kWaveCols;
            weight += max((int64_t)mi, (int64_t)strips * chunks) + 1;     // every lane of every round, as in the scheduler
            if (!offsets_given) {
                if (writer) {
                    // the scheduler's outputs: exclusive prefix sums of the three areas
                    const int64_t i1 = wave_inclusive_scan(v1), i2 = wave_inclusive_scan(v2), iO = wave_inclusive_scan(vO);
                    if (live) {
                        if (m.a1) m.a1[g] = tot1 + i1 - v1;
                        if (m.a2) m.a2[g] = tot2 + i2 - v2;
                        if (m.aO) m.aO[g] = totO + iO - vO;
                    }
                    tot1 += readlane64(i1, 63); tot2 += readlane64(i2, 63); totO += readlane64(iO, 63);
                } else {
                    tot1 += v1; tot2 += v2; totO += vO;      // per lane; reduced after the loop
                }
                if (g < g0) { pre1 += v1; pre2 += v2; preO += vO; }
            }
            if (q == (g0 >> 6)) {
                my_m = readlane64(mm[q], g0 & 63); my_n = readlane64(nn[q], g0 & 63); my_k = readlane64(kk[q], g0 & 63);
            }
        }
        weight = wave_total(weight);
        int64_t D1, D2, DO, o1, o2, oO;
        if (offsets_given) {
            D1 = m.a1[nseg]; D2 = m.a2[nseg]; DO = m.aO[nseg];
            o1 = m.a1[g0]; o2 = m.a2[g0]; oO = m.aO[g0];
        } else {
            o1 = wave_total(pre1); o2 = wave_total(pre2); oO = wave_total(preO);
            if (writer) {
                D1 = tot1; D2 = tot2; DO = totO;
                if (lane == 0) {
                    if (m.a1) m.a1[nseg] = D1;
                    if (m.a2) m.a2[nseg] = D2;
                    if (m.aO) m.aO[nseg] = DO;
                }
            } else {
                D1 = wave_total(tot1); D2 = wave_total(tot2); DO = wave_total(totO);
            }
        }
        // what the scheduler would have rejected, or a plan that would not match the call: nothing is written
        const bool ok = !any_bad && D1 >= 0 && D2 >= 0 && DO >= 0 && weight < (int64_t(1) << 31) && D1 == a.Dm1 &&
                        D2 == a.Dm2 && DO == a.Dout;
        if (lane == 0) {
            box[0] = o1; box[1] = o2; box[2] = oO; box[3] = my_m; box[4] = my_n; box[5] = my_k; box[6] = ok ? 1 : 0;
        }
        // The verdict, where the caller gave a place for it: a plan header without lists, with what the scheduler
        // would have reported (rejected segments, or totals that do not match the call as a run error).
        if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && lane == 0 && a.plan) {
            PlanHeader hd = {};
            hd.magic = kPlanMagic;
            hd.nseg = nseg;
            hd.cap = (int32_t)plan_cap(nseg);
            hd.Dm1 = D1; hd.Dm2 = D2; hd.Dout = DO;
            hd.bad_segments = nbad + ((D1 < 0 || D2 < 0 || DO < 0) ? 1 : 0) + (weight >= (int64_t(1) << 31) ? 1 : 0);
            hd.run_errors = hd.bad_segments == 0 && !ok ? 1 : 0;
            *reinterpret_cast<PlanHeader *>(a.plan) = hd;
        }
    }
    __syncthreads();
    int64_t o1 = box[0], o2 = box[1], oO = box[2];
    const int64_t my_m = box[3], my_n = box[4], my_k = box[5];
    const bool ok = box[6] != 0;
    __syncthreads();                                       // the window is the bodies' from here on
    if (!ok) return;

    Seg s;
    s.M = uniform((int)my_m); s.N = uniform((int)my_n); s.K = uniform((int)my_k);
    s.index = g0; s.packLen = 0;
    o1 = uniform64(o1); o2 = uniform64(o2); oO = uniform64(oO);
    s.a = h * a.Dm1 + o1; s.b = h * a.Dm2 + o2; s.o = h * a.Dout + oO;
    if (s.M < 1 || s.N < 1) return;
    const int64_t lim31 = int64_t(1) << 31;
    const bool aligned = ((s.K | o1 | o2) & 7) == 0 && (int64_t)s.M * s.K < lim31 && (int64_t)s.N * s.K < lim31 &&
                         (int64_t)s.M * s.N < lim31 / 2;
    const int first = bz * kSegWaves + wave, stride = gz * kSegWaves;
    if (!(a.flags & kFlagMfmaOk) || !aligned) {
        s.kind = kSegSlow;
        for (int r = first; r < s.M; r += stride) generic_seg_rows<DT, true>(s, a, r, r + 1, 0, s.N);
        return;
    }
    s.kind = s.N <= kWaveCols ? kSegStrip : s.N <= kSplitCols ? kSegSplit : kSegWide;
    if (fast_strip_shape(s.N, s.K)) {
        if (bz * kSegWaves * kStripRows >= s.M) return;       // no strip for this workgroup
        strips_exact_dispatch<DT, true, F32OUT, 16>(fast_strip_tiles(s.N), s, a, lds, wave, first, stride);
    } else if (tile_segment(s.kind, s.N, s.K)) {
        if (bz * kTileRows >= s.M) return;
        tile_rows<DT, true, F32OUT>(a, s, bz, gz, lds);
    } else {
        // strip-class leftovers (one column, or a long K with few columns): B_g walked in K slabs
        const int strips = (s.M + kStripRows - 1) / kStripRows;
        const int nt = (s.N + 15) >> 4;
        for (int base = bz * kSegWaves; base < strips; base += stride) {
            if (base != bz * kSegWaves) __syncthreads();
            const int strip = base + wave;
            strips_from_lds_dispatch<DT, true, F32OUT, 16>(nt, s, a, lds, a.lds_blocks, strip * kStripRows, strip < strips,
                                                           wave, kSegWaves);
        }
    }
}

template <int DT, bool F32OUT>
static int launch_oc(const RunArgs &args_in, const MetaArgs &meta, hipStream_t stream) {
    RunArgs args = args_in;
    args.lds_blocks = kBigBlocks;
    args.lds_extra = 0;
    args.list = -1;
    const size_t lds_bytes = (size_t)kBigBlocks * kLdsBlockBytes;
    static_assert(kBigBlocks * kLdsBlockBytes >= kStages * kTileChunkBytes, "the tile body's stages fit the window");
    // two workgroups per compute unit's worth of (segment, head) pairs where the batch has that few; a z
    // beyond a segment's strips or row blocks costs a workgroup that reads the metadata and leaves
    const int64_t pairs = (int64_t)args.nseg * args.H;
    const int64_t z = std::max<int64_t>(1, std::min<int64_t>(8, (2 * (int64_t)device_cu_count() + pairs - 1) / pairs));
    hipLaunchKernelGGL((onecall_kernel<DT, F32OUT>), dim3((unsigned)args.H, (unsigned)args.nseg, (unsigned)z),
                       dim3(kSegThreads), lds_bytes, stream, args, meta);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_onecall(int dtype, const RunArgs &args, int mode, const int64_t *M, const int64_t *N, const int64_t *K,
                   int64_t *a1, int64_t *a2, int64_t *aO, hipStream_t stream) {
    if (args.nseg < 1 || args.nseg > kOneCallMaxSegments || (mode != 0 && mode != 2)) return BA_ERR_UNSUPPORTED;
    static_assert(kOneCallMaxSegments == 512, "the rounds below follow the scheduler's 64-, 256- and 512-thread builds");
    if (args.H < 1 || args.H > 0x7fffffff) return BA_ERR_UNSUPPORTED;
    if (!M || !N || !K) return BA_ERR_INVALID_ARG;
    if (mode == 2 && (!a1 || !a2 || !aO)) return BA_ERR_INVALID_ARG;
    const MetaArgs meta{M, N, K, a1, a2, aO, mode, args.nseg <= 64 ? 1 : args.nseg <= 256 ? 4 : 8};
    const bool f32out = args.flags & kFlagOutF32;
    if (dtype == BA_F16) return f32out ? launch_oc<0, true>(args, meta, stream) : launch_oc<0, false>(args, meta, stream);
    if (dtype == BA_BF16) return f32out ? launch_oc<1, true>(args, meta, stream) : launch_oc<1, false>(args, meta, stream);
    return BA_ERR_UNSUPPORTED;
}

}  // namespace ba
