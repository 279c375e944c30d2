// Device-side segment scheduler: one 1024-thread workgroup turns the segment
// shapes into exclusive prefix-sum offsets, exact (M,N,K) lists, packs of tiny
// segments and the scanned work-item counts the compute kernels search.
// Replaces the reference's host-side metadata and tile list construction
// (csrc/sparseBlockedAttention.cpp:17-44, 85-91; csrc/cuda/spBlkGEMM.cu:943-983;
// csrc/cuda/spBlkSoftmax.cu:358-373) without any device-to-host round trip.
#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

__device__ __forceinline__ int32_t readlane_t(int32_t v, int l) { return __builtin_amdgcn_readlane(v, l); }
__device__ __forceinline__ int64_t readlane_t(int64_t v, int l) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, l);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), l);
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

constexpr int kSchedThreadsMax = 1024;   // one workgroup; batches of up to 256 segments use a 256-thread build

struct SchedArgs {
    void *plan;
    int64_t nseg;
    int mode;   // ba_meta_mode
    int kind;   // 0 GEMM plan, 1 softmax plan
    int64_t *M, *N, *K;
    int64_t *a1, *a2, *aO;
    void *mailbox;      // host memory the GPU can write, or nullptr: receives a copy of the header, then the ticket
    uint32_t ticket;
};

// Exclusive scan of NQ quantities over the workgroup.  Wavefront-level DPP
// scans; the totals of the (up to 16) wavefronts go to LDS as lds[16 q + wavefront] and are scanned four
// quantities at a time: lane l of every wavefront takes entry 64 b + l of batch b, i.e. quantity 4 b + l / 16 of
// wavefront l % 16, and one scan inside the rows of 16 lanes serves all four.  lds holds 16 * NQ entries and is
// free for reuse after the next __syncthreads().  One barrier (none in the one-wavefront build).
template <typename T, int NQ, int kSchedWaves>
__device__ __forceinline__ void block_exclusive_scan(T (&v)[NQ], T (&total)[NQ], T *lds) {
    static_assert(kSchedWaves <= 16, "one row of 16 lanes scans the wavefront totals");
    const int wave = uniform((int)(threadIdx.x >> 6)), lane = lane_id();
    T incl[NQ];
    if constexpr (kSchedWaves == 1) {
        // one wavefront: its own scan is the workgroup's (callers still place their barrier before reusing lds)
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            incl[q] = wave_inclusive_scan(v[q]);
            total[q] = readlane_t(incl[q], 63);
            v[q] = incl[q] - v[q];
        }
        return;
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        incl[q] = wave_inclusive_scan(v[q]);
        if (lane == 63) lds[q * 16 + wave] = incl[q];
    }
    __syncthreads();
    constexpr int kBatches = (NQ + 3) / 4;
    const bool mine = (lane & 15) < kSchedWaves;
#pragma unroll
    for (int b = 0; b < kBatches; ++b) {
        T t = (mine && 64 * b + lane < 16 * NQ) ? lds[64 * b + lane] : T(0);
        t = row16_inclusive_scan(t);                   // lanes 16 r .. 16 r + 15: scan over wavefronts of quantity 4 b + r
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int q = 4 * b + r;
            if (q < NQ) {
                const T upto = readlane_t(t, 16 * r + kSchedWaves - 1);
                const T before = wave == 0 ? T(0) : readlane_t(t, 16 * r + wave - 1);
                v[q] = before + incl[q] - v[q];
                total[q] = upto;
            }
        }
    }
}

__device__ __forceinline__ int64_t isqrt64(int64_t v) {
    if (v <= 0) return 0;
    int64_t r = (int64_t)sqrt((double)v);
    while (r * r > v) --r;
    while ((r + 1) * (r + 1) <= v) ++r;
    return r;
}

// Exact (M,N,K) from the three areas mk = M*K, nk = N*K, mn = M*N.
// M^2 = mk*mn/nk needs more than 64 bits in general, so divide out
// g = gcd(mk, nk) first: M^2 = (mk/g) * mn / (nk/g) and nk/g divides mn.
__device__ __forceinline__ bool derive_lists(int64_t mk, int64_t nk, int64_t mn, int64_t &m, int64_t &n,
                                             int64_t &k) {
    if (mk == 0 && nk == 0 && mn == 0) { m = n = k = 0; return true; }
    // one empty dimension leaves one area: the product of the other two dimensions, whose split changes no
    // result; it goes to the first of them whole
    if (mk == 0 && mn == 0 && nk > 0) { m = 0; n = nk; k = 1; return true; }
    if (nk == 0 && mn == 0 && mk > 0) { m = mk; n = 0; k = 1; return true; }
    if (mk == 0 && nk == 0 && mn > 0) { m = mn; n = 1; k = 0; return true; }
    if (mk <= 0 || nk <= 0 || mn <= 0) return false;
    int64_t a = mk, b = nk;
    while (b) { const int64_t t = a % b; a = b; b = t; }
    const int64_t p = mk / a, q = nk / a;  // M/N in lowest terms is p/q
    if (mn % q) return false;
    const int64_t r = mn / q;              // M^2 = p * r
    // p * r < 2^63 is checked through the quotient to stay inside 64 bits.
    if (r != 0 && p > INT64_MAX / r) return false;
    const int64_t m2 = p * r;
    m = isqrt64(m2);
    if (m <= 0 || m * m != m2 || mn % m || mk % m) return false;
    n = mn / m;
    k = mk / m;
    return n * k == nk;
}

constexpr int kSmallBuckets = 8;                          // work buckets of the main strip launch's list

template <int kSchedThreads>
__global__ __launch_bounds__(kSchedThreads) void schedule_kernel(SchedArgs a) {
    constexpr int kSchedWaves = kSchedThreads / 64;
    // Only the 256-thread build (65 to 256 segments) orders its list by work: smaller batches are resident at
    // once whatever their order, and in the larger builds, which are bound by instruction issue, the four more
    // scans cost more than the order gains (1024 segments: scheduler +0.8 us, kernels unchanged).
    constexpr bool kBucketed = kSchedThreads == 256;
    constexpr int kNumScan = kNumPrefix + (kBucketed ? kSmallBuckets / 2 : 0);   // scanned words
    __shared__ int64_t sScan64[16 * 3];
    __shared__ int32_t sScan32[16 * kNumScan];
    __shared__ int32_t sRed[kSchedWaves][8];
    __shared__ int64_t sWeight[kSchedWaves];

    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6), lane = lane_id();
    const int64_t nseg = a.nseg;
    PlanView pv = plan_view(a.plan, nseg);

    int64_t base64[3] = {0, 0, 0};
    int32_t base32[kNumPrefix] = {};
    int32_t maxM = 0, maxN = 0, maxK = 0, nbad = 0;
    int32_t maxSmallN = 0, maxSmallM = 0;       // widest / tallest segment of the strip kernel's main launch
    int32_t maxInvN = 0, maxInvK = 0;           // INT32_MAX - the smallest N and K of the segments that have rows and columns
    // Every scanned count of a segment is at most max(rows, strips x chunks): while the sum of these weights stays
    // below 2^31, none of the int32 scans can overflow; a batch beyond that is rejected as a whole.
    int64_t weight = 0;
    const bool offsets_given = a.mode != 0;   // prefix sums are inputs

    for (int64_t chunk = 0; chunk < nseg || chunk == 0; chunk += kSchedThreads) {
        const int64_t g = chunk + tid;
        const bool live = g < nseg;
        int64_t m = 0, n = 0, k = 0, o1 = 0, o2 = 0, oO = 0;
        bool bad = false;
        if (live) {
            if (a.mode == 1) {               // prefix sums -> lists
                o1 = a.a1[g]; o2 = a.a2[g]; oO = a.aO[g];
                const int64_t mk = a.a1[g + 1] - o1, nk = a.a2[g + 1] - o2, mn = a.aO[g + 1] - oO;
                bad = !derive_lists(mk, nk, mn, m, n, k) || o1 < 0 || o2 < 0 || oO < 0;
            } else {
                m = a.M[g]; n = a.N[g]; k = a.kind == 0 ? a.K[g] : 0;
                if (offsets_given) {
                    oO = a.aO[g];
                    bad = oO < 0 || a.aO[g + 1] - oO < m * n;
                    if (a.kind == 0) {
                        o1 = a.a1[g]; o2 = a.a2[g];
                        bad = bad || o1 < 0 || o2 < 0 || a.a1[g + 1] - o1 < m * k || a.a2[g + 1] - o2 < n * k;
                    }
                }
            }
            // every dimension and every area of a segment below 2^30: the kernels address a segment with 32-bit byte
            // offsets (the products below cannot overflow: each factor is below 2^30 when they are formed)
            const int64_t lim = int64_t(1) << 30;
            bad = bad || m < 0 || n < 0 || k < 0 || m >= lim || n >= lim || k >= lim;
            bad = bad || m * k >= lim || n * k >= lim || m * n >= lim;
            if (bad) { m = n = k = 0; }
        }
        const int32_t mi = (int32_t)m, ni = (int32_t)n, ki = (int32_t)k;
        // Offsets first: alignment decides which path a segment takes.
        int64_t v64[3] = {m * k, n * k, m * n}, t64[3] = {0, 0, 0};
        if (!offsets_given) {
            block_exclusive_scan<int64_t, 3, kSchedWaves>(v64, t64, sScan64);
            o1 = base64[0] + v64[0]; o2 = base64[1] + v64[1]; oO = base64[2] + v64[2];
        }
        // 16-byte operand rows, and segment areas that fit the 32-bit byte
        // offsets of the buffer instructions.
        const int64_t lim31 = int64_t(1) << 31;
        const bool aligned = ((k | o1 | o2) & 7) == 0 && m * k < lim31 && n * k < lim31 && m * n < lim31 / 2;

        // Packs: inside each aligned window of 16 segments, greedily join
        // consecutive tiny aligned segments (same K, sum M <= 16, sum N <= 16).
        // The first lane of every window walks its 16 entries in registers.
        int32_t pack = 0;
        // Only batches that contain segments small enough to pack pay for the window walk.
        const bool packable = aligned && mi >= 1 && ni >= 1 && ki >= 1 && mi < kPackDim && ni < kPackDim;
        if (a.kind == 0 && __ballot(packable) != 0) {          // per wavefront: the windows are rows of 16 lanes
            // A window is the 16 lanes of one DPP row.  The greedy walk runs along the row: lane j takes the
            // state that lane j-1 holds (rows sum, columns sum, members so far, K of the open pack), decides
            // whether its segment joins that pack, and holds the state after it.  After step t lanes 0..t
            // are final; every lane recomputes in every step, so nothing diverges and nothing leaves the
            // registers.  Sizes enter clamped to 17 ("does not fit whatever follows").
            const bool ok = mi >= 1 && ni >= 1 && ki >= 1 && aligned;
            const uint32_t mc = (uint32_t)min(mi, kPackDim + 1), nc = (uint32_t)min(ni, kPackDim + 1);
            const uint32_t alone = mc | (nc << 8) | ((ok ? 1u : 0u) << 16);   // a pack opened by this segment
            uint32_t st = alone;
            int32_t kopen = ki;
            bool joins = false;
#pragma unroll
            for (int t = 1; t < 16; ++t) {
                const uint32_t pst = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)st, 0x111, 0xf, 0xf, false);
                const int32_t pk = __builtin_amdgcn_update_dpp(0, kopen, 0x111, 0xf, 0xf, false);
                const uint32_t sm = (pst & 0xff) + mc, sn = ((pst >> 8) & 0xff) + nc, len = pst >> 16;
                joins = ok && len > 0 && pk == ki && sm <= (uint32_t)kPackDim && sn <= (uint32_t)kPackDim;
                st = joins ? (sm | (sn << 8) | ((len + 1) << 16)) : alone;
                kopen = ki;                                   // a joining segment has the pack's K anyway
            }
            // members of a pack = this leader plus the run of joining lanes right after it
            const uint64_t jb = __ballot(joins);
            const int j = lane & 15;
            const uint32_t row = (uint32_t)(jb >> (lane & 48)) & 0xffffu;
            const uint32_t after = (~row & 0xffffu) >> (j + 1);              // bit i: lane j+1+i does not join
            const int run = j == 15 ? 0 : min((int)__builtin_ctz(after | (1u << (15 - j))), 15 - j);
            pack = joins ? -1 : (ok && run >= 1) ? run + 1 : 0;
        }

        const int32_t strips = (ni >= 1) ? (mi + kStripRows - 1) / kStripRows : 0;
        const int32_t chunks = (ni + kWaveCols - 1) / kWaveCols;
        const bool packed = pack != 0;
        const bool mfma_ok = aligned && !packed;
        const int32_t seg_kind = strips == 0 ? kSegEmpty
                                 : !aligned ? kSegSlow
                                 : pack > 0 ? kSegPackLead
                                 : pack < 0 ? kSegPackFollow
                                 : ni <= kWaveCols ? kSegStrip
                                 : ni <= kSplitCols ? kSegSplit : kSegWide;
        const int cls = a.kind == 0 ? launch_class(seg_kind, mi, ni, ki) : -1;
        const bool mini = cls == kListSmall && mini_shape(mi, ni, ki);     // kept apart from the list's other entries
        int32_t v32[kNumScan], t32[kNumScan];
#pragma unroll
        for (int q = 0; q < kNumLists; ++q) v32[q] = (cls == q && !mini) ? 1 : 0;
        v32[kPfxMini] = mini ? 1 : 0;
        v32[kPfxPipe] = (cls == kListTile && pipe_segment(seg_kind, ni, ki)) ? 1 : 0;
        const bool wide_rows = mi >= 1 && ni > kRunCols;      // the softmax row kernel's, whatever the plan kind
        v32[kListRows] = wide_rows ? 1 : 0;
        weight += max((int64_t)mi, (int64_t)strips * chunks) + 1;
        v32[kPfxGemm] = (mfma_ok && ni > kWaveCols) ? strips * chunks : 0;
        v32[kPfxStrip] = (mfma_ok && ni <= kWaveCols) ? strips : 0;
        v32[kPfxSplit] = (mfma_ok && ni > kWaveCols && ni <= kSplitCols) ? strips : 0;
        v32[kPfxWide] = (mfma_ok && ni > kSplitCols) ? strips : 0;
        v32[kPfxRows] = ni >= 1 ? mi : 0;
        v32[kPfxPack] = pack > 0 ? 1 : 0;
        v32[kPfxSlow] = aligned ? 0 : strips;
        const bool att_rows = mi >= 1;                         // row blocks of every segment with rows, whatever N and K are
        v32[kPfxAtt64] = att_rows ? (mi + kAttBlockRows - 1) / kAttBlockRows : 0;
        v32[kPfxAtt128] = att_rows ? (mi + 2 * kAttBlockRows - 1) / (2 * kAttBlockRows) : 0;
        if (a.kind == 1) {
#pragma unroll
            for (int q = 0; q < kNumPrefix; ++q)
                if (q >= kNumLists && q != kPfxRows) v32[q] = 0;
        }
        // The main strip launch's list is kept in eight buckets of decreasing work (16-row strips x column
        // tiles / 8, clipped): workgroups that start together then take about equally long and the longest
        // start first (256 segments x 8 heads of 32..128 rows: fused kernel 16.1 -> 15.4 us).  One counter of
        // 16 bits per bucket (a pass holds at most 1024 segments), two to a scanned word.
        const int bucket = (cls == kListSmall && !mini) ? min(kSmallBuckets - 1, min(strips, 64) * fast_strip_tiles(min(ni, 256)) / 8) : -1;
        if constexpr (kBucketed) {
#pragma unroll
            for (int wd = 0; wd < kSmallBuckets / 2; ++wd)
                v32[kNumPrefix + wd] = (bucket >> 1) == wd ? 1 << (16 * (bucket & 1)) : 0;
        }
        block_exclusive_scan<int32_t, kNumScan, kSchedWaves>(v32, t32, sScan32);
        int32_t small_pos = v32[kListSmall];                  // position in the list among this pass's entries
        if constexpr (kBucketed) {
            small_pos = 0;
#pragma unroll
            for (int b = 0; b < kSmallBuckets; ++b) {
                const int32_t count = (t32[kNumPrefix + (b >> 1)] >> (16 * (b & 1))) & 0xffff;
                const int32_t rank = (v32[kNumPrefix + (b >> 1)] >> (16 * (b & 1))) & 0xffff;
                small_pos += b > bucket ? count : b == bucket ? rank : 0;
            }
        }

        if (live) {
            SegRec rec;
            rec.off1 = o1; rec.off2 = o2; rec.offO = oO;
            rec.M = mi; rec.N = ni; rec.K = ki; rec.packLen = pack > 0 ? pack : 0;
            rec.kind = seg_kind;
            rec.index = (int32_t)g;
            pv.recs[g] = rec;
#pragma unroll
            for (int q = 0; q < kNumLists; ++q)          // v32 now holds the exclusive scans
                if (cls == q && !mini) pv.list[q][base32[q] + (q == kListSmall ? small_pos : v32[q])] = rec;
            if (mini) pv.list[kListSmall][plan_cap(nseg) - 1 - (base32[kPfxMini] + v32[kPfxMini])] = rec;
            if (wide_rows) pv.list[kListRows][base32[kListRows] + v32[kListRows]] = rec;
            if (a.kind == 0) {
                plan_rowblocks(a.plan, nseg, 0)[g] = base32[kPfxAtt64] + v32[kPfxAtt64];
                plan_rowblocks(a.plan, nseg, 1)[g] = base32[kPfxAtt128] + v32[kPfxAtt128];
            }
            if (!offsets_given) {
                if (a.a1) a.a1[g] = o1;
                if (a.a2) a.a2[g] = o2;
                if (a.aO) a.aO[g] = oO;
            }
            if (a.mode == 1) {
                if (a.M) a.M[g] = bad ? -1 : m;
                if (a.N) a.N[g] = bad ? -1 : n;
                if (a.K) a.K[g] = bad ? -1 : k;
            }
        }
        maxM = max(maxM, mi); maxN = max(maxN, ni); maxK = max(maxK, ki); nbad += bad ? 1 : 0;
        if (cls == kListSmall) { maxSmallN = max(maxSmallN, ni); maxSmallM = max(maxSmallM, mi); }
        if (mi >= 1 && ni >= 1) { maxInvN = max(maxInvN, INT32_MAX - ni); maxInvK = max(maxInvK, INT32_MAX - ki); }
#pragma unroll
        for (int q = 0; q < kNumPrefix; ++q) base32[q] += t32[q];
        if (!offsets_given) {
#pragma unroll
            for (int q = 0; q < 3; ++q) base64[q] += t64[q];
        }
        if (chunk + kSchedThreads >= nseg) break;
        __syncthreads();   // the scan scratch is rewritten by the next pass
    }

    // Shape maxima and the count of rejected segments: DPP reduction per
    // wavefront, then thread 0 folds the 16 partial results.
    maxM = wave_max_nonneg(maxM); maxN = wave_max_nonneg(maxN); maxK = wave_max_nonneg(maxK);
    maxSmallN = wave_max_nonneg(maxSmallN); maxSmallM = wave_max_nonneg(maxSmallM);
    maxInvN = wave_max_nonneg(maxInvN); maxInvK = wave_max_nonneg(maxInvK);
    nbad = __builtin_amdgcn_readlane(wave_inclusive_scan(nbad), 63);
#pragma unroll
    for (int msk = 32; msk >= 1; msk >>= 1) weight += __shfl_xor(weight, msk);
    if (lane == 0) sWeight[wave] = weight;
    if (lane == 0) { sRed[wave][0] = maxM; sRed[wave][1] = maxN; sRed[wave][2] = maxK; sRed[wave][3] = nbad; sRed[wave][4] = maxSmallN; sRed[wave][5] = maxSmallM; sRed[wave][6] = maxInvN; sRed[wave][7] = maxInvK; }
    __syncthreads();

    if (tid == 0) {
        int64_t D1, D2, DO;
        if (offsets_given) {
            DO = a.aO[nseg];
            D1 = a.kind == 0 ? a.a1[nseg] : 0;
            D2 = a.kind == 0 ? a.a2[nseg] : 0;
        } else {
            D1 = base64[0]; D2 = base64[1]; DO = base64[2];
            if (a.a1) a.a1[nseg] = D1;
            if (a.a2) a.a2[nseg] = D2;
            if (a.aO) a.aO[nseg] = DO;
        }
        int32_t rM = 0, rN = 0, rK = 0, rBad = 0, rSN = 0, rSM = 0, rInvN = 0, rInvK = 0;
        int64_t total_weight = 0;
        for (int w = 0; w < kSchedWaves; ++w) {
            rM = max(rM, sRed[w][0]); rN = max(rN, sRed[w][1]); rK = max(rK, sRed[w][2]); rBad += sRed[w][3];
            total_weight += sWeight[w];
            rSN = max(rSN, sRed[w][4]); rSM = max(rSM, sRed[w][5]); rInvN = max(rInvN, sRed[w][6]); rInvK = max(rInvK, sRed[w][7]);
        }
        PlanHeader *h = pv.hdr;
        h->magic = kPlanMagic;
        h->nseg = (int32_t)nseg;
        h->cap = (int32_t)plan_cap(nseg);
        h->kind = a.kind;
        h->Dm1 = D1; h->Dm2 = D2; h->Dout = DO;
        h->total_rows = base32[kPfxRows];
        for (int q = 0; q < 12; ++q) h->totals[q] = q < kNumPrefix ? base32[q] : 0;
        h->max_M = rM; h->max_N = rN; h->max_K = rK;
        h->small_max_N = rSN; h->small_max_M = rSM;
        h->bad_segments = rBad + ((D1 < 0 || D2 < 0 || DO < 0) ? 1 : 0) + (total_weight >= (int64_t(1) << 31) ? 1 : 0);
        h->run_errors = 0;
        h->att_blocks64 = base32[kPfxAtt64];
        h->att_blocks128 = base32[kPfxAtt128];
        h->mini_count = base32[kPfxMini];
        h->pipe_count = base32[kPfxPipe];
        h->pipe_groups = 0;
        h->min_N = rInvN ? INT32_MAX - rInvN : 0;
        h->min_K = rInvK ? INT32_MAX - rInvK : 0;
        h->ring_groups = 0;
        h->wide_groups = 0;
        plan_rowblocks(a.plan, nseg, 0)[nseg] = base32[kPfxAtt64];     // zero for softmax plans
        plan_rowblocks(a.plan, nseg, 1)[nseg] = base32[kPfxAtt128];
        if (a.mailbox) {
            // the summary for a host that waits on the ticket instead of copying and synchronising: the header
            // first, visible system-wide, then the ticket behind it
            __builtin_memcpy(a.mailbox, h, sizeof(PlanHeader));
            __threadfence_system();
            __hip_atomic_store(reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(a.mailbox) + kMailboxTicket), a.ticket,
                               __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

int launch_schedule(void *plan, size_t plan_bytes, int64_t nseg, int mode, int kind, int64_t *M, int64_t *N,
                    int64_t *K, int64_t *a1, int64_t *a2, int64_t *aO, hipStream_t stream, void *mailbox,
                    uint32_t ticket) {
    if (!plan || nseg < 0 || nseg > (int64_t(1) << 30)) return BA_ERR_INVALID_ARG;
    if (plan_bytes < plan_bytes_for(nseg) || ((uintptr_t)plan & 15)) return BA_ERR_WORKSPACE;
    if (mode < 0 || mode > 2) return BA_ERR_INVALID_ARG;
    const bool need_lists = mode != BA_META_FROM_ACCUM;
    const bool need_accum = mode != BA_META_FROM_LISTS;
    if (nseg > 0) {
        if (need_lists && (!M || !N || (kind == 0 && !K))) return BA_ERR_INVALID_ARG;
        if (need_accum && (!aO || (kind == 0 && (!a1 || !a2)))) return BA_ERR_INVALID_ARG;
    } else if (need_accum && (!aO || (kind == 0 && (!a1 || !a2)))) {
        return BA_ERR_INVALID_ARG;
    }
    if (mailbox && ((uintptr_t)mailbox & 15)) return BA_ERR_INVALID_ARG;
    SchedArgs args{plan, nseg, mode, kind, M, N, K, a1, a2, aO, mailbox, ticket};
    if (nseg <= 64) hipLaunchKernelGGL(schedule_kernel<64>, dim3(1), dim3(64), 0, stream, args);
    else if (nseg <= 256) hipLaunchKernelGGL(schedule_kernel<256>, dim3(1), dim3(256), 0, stream, args);
    else if (nseg <= 512) hipLaunchKernelGGL(schedule_kernel<512>, dim3(1), dim3(512), 0, stream, args);
    else hipLaunchKernelGGL(schedule_kernel<kSchedThreadsMax>, dim3(1), dim3(kSchedThreadsMax), 0, stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
