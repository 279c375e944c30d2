// Device-side segment scheduler: one 1024-thread workgroup turns the segment
// shapes into exclusive prefix-sum offsets, exact (M,N,K) lists, packs of tiny
// segments and the scanned work-item counts the compute kernels search.
// Replaces the reference's host-side metadata and tile list construction
// (csrc/sparseBlockedAttention.cpp:17-44, 85-91; csrc/cuda/spBlkGEMM.cu:943-983;
// csrc/cuda/spBlkSoftmax.cu:358-373) without any device-to-host round trip.
#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kSchedThreads = 1024;
constexpr int kSchedWaves = kSchedThreads / 64;

struct SchedArgs {
    void *plan;
    int64_t nseg;
    int mode;   // ba_meta_mode
    int kind;   // 0 GEMM plan, 1 softmax plan
    int64_t *M, *N, *K;
    int64_t *a1, *a2, *aO;
};

// Inclusive scan inside one wavefront.
template <typename T> __device__ __forceinline__ T wave_inclusive_scan(T v) {
    const int lane = lane_id();
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        T u = __shfl_up(v, o);
        if (lane >= o) v += u;
    }
    return v;
}

// Exclusive scan of NQ quantities over the workgroup; total[] receives the sums.
// lds must hold kSchedWaves * NQ entries.  Ends with a barrier-free state in
// which lds may be reused after the next __syncthreads().
template <typename T, int NQ>
__device__ __forceinline__ void block_exclusive_scan(T (&v)[NQ], T (&total)[NQ], T *lds) {
    const int wave = threadIdx.x >> 6, lane = lane_id();
    T incl[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        incl[q] = wave_inclusive_scan(v[q]);
        if (lane == 63) lds[wave * NQ + q] = incl[q];
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        T base = 0, tot = 0;
        for (int w = 0; w < kSchedWaves; ++w) {
            const T s = lds[w * NQ + q];
            if (w < wave) base += s;
            tot += s;
        }
        v[q] = base + incl[q] - v[q];
        total[q] = tot;
    }
    __syncthreads();
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

__global__ __launch_bounds__(kSchedThreads) void schedule_kernel(SchedArgs a) {
    __shared__ int64_t sScan64[kSchedWaves * 3];
    __shared__ int32_t sScan32[kSchedWaves * kNumPrefix];
    __shared__ int32_t sM[kSchedThreads], sN[kSchedThreads], sK[kSchedThreads], sPack[kSchedThreads];
    __shared__ int32_t sMax[3], sBad;

    const int tid = threadIdx.x;
    const int64_t nseg = a.nseg;
    PlanView pv = plan_view(a.plan, nseg);
    if (tid == 0) { sMax[0] = sMax[1] = sMax[2] = 0; sBad = 0; }
    __syncthreads();

    int64_t base64[3] = {0, 0, 0};
    int32_t base32[kNumPrefix] = {0, 0, 0, 0, 0, 0, 0};
    int64_t rows_total = 0;
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
            const int64_t lim = int64_t(1) << 30;
            bad = bad || m < 0 || n < 0 || k < 0 || m >= lim || n >= lim || k >= lim;
            if (bad) { m = n = k = 0; atomicAdd(&sBad, 1); }
        }
        // Offsets first: alignment decides which path a segment takes.
        int64_t v64[3] = {m * k, n * k, m * n}, t64[3] = {0, 0, 0};
        if (!offsets_given) {
            block_exclusive_scan<int64_t, 3>(v64, t64, sScan64);
            o1 = base64[0] + v64[0]; o2 = base64[1] + v64[1]; oO = base64[2] + v64[2];
        }
        // 16-byte operand rows, and segment areas that fit the 32-bit byte
        // offsets of the buffer instructions.
        const int64_t lim31 = int64_t(1) << 31;
        const bool aligned = ((k | o1 | o2) & 7) == 0 && m * k < lim31 && n * k < lim31 && m * n < lim31 / 2;
        sM[tid] = (int32_t)m; sN[tid] = (int32_t)n; sK[tid] = aligned ? (int32_t)k : -1; sPack[tid] = 0;
        __syncthreads();

        // Packs: inside each aligned window of 16 segments, greedily join
        // consecutive tiny aligned segments (same K, sum M <= 16, sum N <= 16).
        if (a.kind == 0 && (tid & 15) == 0) {
            int i = 0;
            while (i < 16) {
                const int s = tid + i;
                int len = 0, sumM = 0, sumN = 0;
                const int k0 = sK[s];
                while (i + len < 16) {
                    const int mm = sM[s + len], nn = sN[s + len];
                    if (mm < 1 || nn < 1 || sK[s + len] != k0 || k0 < 1) break;
                    if (sumM + mm > kPackDim || sumN + nn > kPackDim) break;
                    sumM += mm; sumN += nn; ++len;
                }
                if (len >= 2) {
                    sPack[s] = len;
                    for (int j = 1; j < len; ++j) sPack[s + j] = -1;
                    i += len;
                } else {
                    i += 1;
                }
            }
        }
        __syncthreads();

        const int32_t pack = sPack[tid];
        const int32_t strips = (n >= 1) ? (int32_t)((m + kStripRows - 1) / kStripRows) : 0;
        const int64_t chunks = (n + kWaveCols - 1) / kWaveCols;
        const bool packed = pack != 0;
        const bool mfma_ok = aligned && !packed;
        int32_t v32[kNumPrefix], t32[kNumPrefix];
        v32[kPfxGemm] = mfma_ok ? (int32_t)(strips * chunks) : 0;
        v32[kPfxStrip] = (mfma_ok && n <= kWaveCols) ? strips : 0;
        v32[kPfxSplit] = (mfma_ok && n > kWaveCols && n <= kSplitCols) ? strips : 0;
        v32[kPfxWide] = (mfma_ok && n > kSplitCols) ? strips : 0;
        v32[kPfxRows] = n >= 1 ? (int32_t)m : 0;
        v32[kPfxPack] = pack > 0 ? 1 : 0;
        v32[kPfxSlow] = aligned ? 0 : strips;
        if (a.kind == 1) {
#pragma unroll
            for (int q = 0; q < kNumPrefix; ++q)
                if (q != kPfxRows) v32[q] = 0;
        }
        block_exclusive_scan<int32_t, kNumPrefix>(v32, t32, sScan32);

        if (live) {
            pv.off1[g] = o1; pv.off2[g] = o2; pv.offO[g] = oO;
            pv.M[g] = (int32_t)m; pv.N[g] = (int32_t)n; pv.K[g] = (int32_t)k;
            pv.packLen[g] = pack > 0 ? pack : 0;
#pragma unroll
            for (int q = 0; q < kNumPrefix; ++q) pv.pfx[q][g] = base32[q] + v32[q];
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
            atomicMax(&sMax[0], (int32_t)m); atomicMax(&sMax[1], (int32_t)n); atomicMax(&sMax[2], (int32_t)k);
        }
        rows_total += t32[kPfxRows];
#pragma unroll
        for (int q = 0; q < kNumPrefix; ++q) base32[q] += t32[q];
        if (!offsets_given) {
#pragma unroll
            for (int q = 0; q < 3; ++q) base64[q] += t64[q];
        }
        if (nseg == 0) break;
    }
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
        pv.off1[nseg] = D1; pv.off2[nseg] = D2; pv.offO[nseg] = DO;
        for (int q = 0; q < kNumPrefix; ++q) pv.pfx[q][nseg] = base32[q];
        PlanHeader *h = pv.hdr;
        h->magic = kPlanMagic;
        h->nseg = (int32_t)nseg;
        h->cap = (int32_t)plan_cap(nseg);
        h->kind = a.kind;
        h->Dm1 = D1; h->Dm2 = D2; h->Dout = DO;
        h->total_rows = rows_total;
        for (int q = 0; q < 8; ++q) h->totals[q] = q < kNumPrefix ? base32[q] : 0;
        h->max_M = sMax[0]; h->max_N = sMax[1]; h->max_K = sMax[2];
        h->bad_segments = sBad + ((D1 < 0 || D2 < 0 || DO < 0) ? 1 : 0);
        h->run_errors = 0;
    }
}

int launch_schedule(void *plan, size_t plan_bytes, int64_t nseg, int mode, int kind, int64_t *M, int64_t *N,
                    int64_t *K, int64_t *a1, int64_t *a2, int64_t *aO, hipStream_t stream) {
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
    SchedArgs args{plan, nseg, mode, kind, M, N, K, a1, a2, aO};
    hipLaunchKernelGGL(schedule_kernel, dim3(1), dim3(kSchedThreads), 0, stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
