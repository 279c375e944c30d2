// Standalone blocked row softmax: dst row = softmax(scale * src row) for every
// row of every segment (csrc/cuda/spBlkSoftmax.cu:88-138, 182-269 restated for
// wave64), and its backward.  fp32 arithmetic for fp16, bf16 and fp32, one rounding at
// the store, no column limit; fp64 has a plain kernel of its own at the end of the file.
//
// A segment is a contiguous run of rows x cols elements, rows back to back.  The
// memory pipeline works per lane access, so both kernels move 16 bytes per lane
// with adjacent lanes on adjacent addresses, at whatever element alignment the
// rows happen to have:
//   lane-run kernel  cols <= 256.  Sixteen lanes share a row: lane j owns the G
//                    consecutive columns [G*j, G*j + G) (G = even tile count
//                    covering cols), a wavefront takes 16 rows at a time, four per
//                    instruction -- the layout of the fused strip kernel, with the
//                    scores loaded instead of computed.  Ragged cols: the lane
//                    holding the row's end takes the run [cols - G, cols), which
//                    overlaps its neighbour (both load and store identical values,
//                    the overlap counts once in the row sum); there are no partial
//                    loads or stores.
//   row kernel       cols > 256 (and cols < 2).  One wavefront per row, lane l owns
//                    the eight columns 8*l + 512*k; rows of up to 4096 columns stay
//                    in registers, longer rows are re-read in three passes.
#include <algorithm>
#include <cstdlib>

#include "ba_gemm_common.hpp"

namespace ba {

constexpr int kSoftmaxThreads = 256;
constexpr int kSoftmaxWaves = kSoftmaxThreads / 64;
constexpr int kRowSteps = 8;      // 512-column steps a row keeps in registers (4096 columns)

template <int DT> struct Io;
template <> struct Io<BA_F16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const T *p) { return Elem<0>::to_float(*p); }
    static __device__ __forceinline__ void st(T *p, float v) { *p = Elem<0>::from_float(v); }
    static __device__ __forceinline__ float lo(uint32_t w) { return Elem<0>::to_float((uint16_t)w); }
    static __device__ __forceinline__ float hi(uint32_t w) { return Elem<0>::to_float((uint16_t)(w >> 16)); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) { return Elem<0>::pack2(a, b); }
};
template <> struct Io<BA_BF16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const T *p) { return Elem<1>::to_float(*p); }
    static __device__ __forceinline__ void st(T *p, float v) { *p = Elem<1>::from_float(v); }
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
    static __device__ __forceinline__ uint32_t pack(float a, float b) { return Elem<1>::pack2(a, b); }
};
template <> struct Io<BA_F32> {
    typedef float T;
    static __device__ __forceinline__ float ld(const T *p) { return *p; }
    static __device__ __forceinline__ void st(T *p, float v) { *p = v; }
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w); }   // unused
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w); }   // unused
    static __device__ __forceinline__ uint32_t pack(float a, float) { return __builtin_bit_cast(uint32_t, a); }
};

struct SoftmaxArgs {
    void *plan;
    const void *src;     // forward: x            backward: y (saved forward output)
    const void *aux;     // forward: unused       backward: dy
    void *dst;           // forward: y            backward: dx
    int64_t H, Dsrc;
    float scale;
    int head_fast;       // lane-run kernel: grid (head, segment, z) instead of (segment, head, z)
};

// Plan checks shared by both kernels, fetched as one batch of scalar loads.
__device__ __forceinline__ int softmax_plan_nseg(const SoftmaxArgs &a) {
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const uint32_t magic = hdr->magic;
    const int nseg = hdr->nseg, bad = hdr->bad_segments;
    const int64_t d = hdr->Dout;
    if ((magic == kPlanMagic) & (bad == 0) & (d == a.Dsrc)) return nseg;
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
        atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
    return -1;
}

// ---------------------------------------------------------------- lane runs
// G consecutive elements of one row from memory into x[g][e] (any element alignment).
// G consecutive elements of one row as they come from memory (any element alignment); unpacked later,
// so that the loads of a whole strip are in flight together.
template <int DT, int G> struct RawRun {
    typedef typename Io<DT>::T T;
    uint32_t w[G / 2];
    __device__ __forceinline__ void load(const T *p) {
        const char *q = reinterpret_cast<const char *>(p);
#pragma unroll
        for (int k = 0; k + 4 <= G / 2; k += 4) {
            const u32x4 v = *reinterpret_cast<const u32x4_unaligned *>(q + 4 * k);
            w[k] = v[0]; w[k + 1] = v[1]; w[k + 2] = v[2]; w[k + 3] = v[3];
        }
        constexpr int kDone = (G / 2) & ~3;
        if constexpr (((G / 2) & 2) != 0) {
            const u32x2 v = *reinterpret_cast<const u32x2_unaligned *>(q + 4 * kDone);
            w[kDone] = v[0]; w[kDone + 1] = v[1];
        }
        if constexpr (((G / 2) & 1) != 0) w[G / 2 - 1] = *reinterpret_cast<const u32_unaligned *>(q + 4 * (G / 2 - 1));
    }
    __device__ __forceinline__ void unpack(f32x4 (&x)[G], int e) const {
#pragma unroll
        for (int k = 0; k < G / 2; ++k) { x[2 * k][e] = Io<DT>::lo(w[k]); x[2 * k + 1][e] = Io<DT>::hi(w[k]); }
    }
};
template <int G> struct RawRun<BA_F32, G> {
    typedef float T;
    float w[G];
    __device__ __forceinline__ void load(const T *q) {
#pragma unroll
        for (int k = 0; k + 4 <= G; k += 4) {
            const f32x4 v = *reinterpret_cast<const f32x4_unaligned *>(q + k);
            w[k] = v[0]; w[k + 1] = v[1]; w[k + 2] = v[2]; w[k + 3] = v[3];
        }
        if constexpr ((G & 2) != 0) {
            const f32x2 v = *reinterpret_cast<const f32x2_unaligned *>(q + (G - 2));
            w[G - 2] = v[0]; w[G - 1] = v[1];
        }
    }
    __device__ __forceinline__ void unpack(f32x4 (&x)[G], int e) const {
#pragma unroll
        for (int k = 0; k < G; ++k) x[k][e] = w[k];
    }
};

// The 16-row strips first, first + step, ... of one segment with 2 <= cols <= 16 * G.  Every lane loads
// in every step: lanes past the row end hold the run [cols-G, cols) once more (weight 0), rows past the
// segment's end repeat its last row (computed, not stored), so no load sits behind a branch; the loads
// of the next strip are issued before the arithmetic of the current one.
template <int DT, int G, bool BACKWARD>
__device__ __forceinline__ void softmax_runs(const SoftmaxArgs &a, int64_t seg0, int rows, int cols, int first_strip,
                                             int strip_step) {
    typedef typename Io<DT>::T T;
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int J = cols / G, v = cols - G * J;
    const bool owner = j < J || (j == J && v > 0);
    const int col0 = j < J ? G * j : cols - G;
    float w[G];
#pragma unroll
    for (int g = 0; g < G; ++g) w[g] = (j < J || (j == J && g >= G - v)) ? 1.f : 0.f;
    const T *src = reinterpret_cast<const T *>(a.src) + seg0 + col0;
    const T *aux = reinterpret_cast<const T *>(a.aux) + seg0 + col0;
    T *dst = reinterpret_cast<T *>(a.dst) + seg0 + col0;
    const float c_signed = a.scale * kLog2e;
    const float sgn = c_signed < 0.f ? -1.f : 1.f;   // forward works on sgn * x so that the multiplier is >= 0
    const float c = c_signed * sgn;
    const int strips = (rows + 15) >> 4;
    RawRun<DT, G> rx[4], rd[BACKWARD ? 4 : 1];
    auto issue = [&](int strip) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // register e of row group rg is row 16*strip + 4*e + rg: an instruction covers four consecutive rows
            const int64_t row = min(16 * strip + rg + 4 * e, rows - 1);
            rx[e].load(src + row * cols);
            if (BACKWARD) rd[BACKWARD ? e : 0].load(aux + row * cols);
        }
    };
    if (first_strip < strips) issue(first_strip);
    for (int strip = first_strip; strip < strips; strip += strip_step) {
        const int r0 = 16 * strip + rg;
        f32x4 x[G], dy[BACKWARD ? G : 1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            rx[e].unpack(x, e);
            if constexpr (BACKWARD) rd[e].unpack(dy, e);
        }
        if (strip + strip_step < strips) issue(strip + strip_step);
        if constexpr (!BACKWARD) {
            if (sgn < 0.f) {
#pragma unroll
                for (int g = 0; g < G; ++g) x[g] = -x[g];
            }
            softmax_lane_runs<G, false>(x, w, c);
        } else {
            // dx = scale * (dy - sum(y * dy)) * y; src is the saved forward output here
            float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int g = 0; g < G; ++g) dot[e] = fmaf(x[g][e] * dy[g][e], w[g], dot[e]);
            row16_sum4(dot);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int g = 0; g < G; ++g) x[g][e] = a.scale * (dy[g][e] - dot[e]) * x[g][e];
        }
        if (owner) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (r0 + 4 * e < rows)
                    store_run<DT == BA_BF16 ? 1 : 0, G, DT == BA_F32, true>(
                        reinterpret_cast<char *>(dst + (int64_t)(r0 + 4 * e) * cols), x, e);
        }
    }
}

// grid (segment, head, z): the wavefronts of the workgroups with the same (segment, head) share the
// segment's 16-row strips round-robin.
// MAXG = 8 is the build for batches whose widest row has 128 columns or fewer: half the registers,
// twice the resident wavefronts.
template <int DT, bool BACKWARD, int MAXG>
__device__ __forceinline__ void softmax_runs_body(const SoftmaxArgs &a, unsigned bx, unsigned by, unsigned bz, unsigned gz) {
    typedef typename Io<DT>::T T;
    const int nseg = softmax_plan_nseg(a);
    const int g = bx;
    if (g >= nseg) return;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int rows = rec.M, cols = rec.N;
    if (cols < 1 || cols > kRunCols || cols > 16 * MAXG || rows < 1) return;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int first = bz * kSoftmaxWaves + wave, step = gz * kSoftmaxWaves;
    const int64_t seg0 = (int64_t)by * a.Dsrc + rec.offO;
    if (cols == 1) {
        // one column: softmax is 1 (NaN where the input is not finite); backward is 0 * (...) likewise
        const T *src = reinterpret_cast<const T *>(a.src) + seg0;
        const T *aux = reinterpret_cast<const T *>(a.aux) + seg0;
        T *dst = reinterpret_cast<T *>(a.dst) + seg0;
        for (int r = first * 64 + lane_id(); r < rows; r += step * 64) {
            const float x = Io<DT>::ld(src + r);
            if (!BACKWARD) {
                Io<DT>::st(dst + r, fmaf(x, 0.f, 1.f));
            } else {
                const float dy = Io<DT>::ld(aux + r);
                Io<DT>::st(dst + r, a.scale * (dy - x * dy) * x);
            }
        }
        return;
    }
    const int tiles = fast_strip_tiles(cols);
#define BA_RUNS(G_) case G_: softmax_runs<DT, G_, BACKWARD>(a, seg0, rows, cols, first, step); break;
    switch (tiles) {
        BA_RUNS(2) BA_RUNS(4) BA_RUNS(6) BA_RUNS(8)
        default:
            if (MAXG > 8) {
                switch (tiles) {
                    BA_RUNS(10) BA_RUNS(12) BA_RUNS(14) BA_RUNS(16)
                    default: break;
                }
            }
            break;
    }
#undef BA_RUNS
}

// --------------------------------------------------------------------- rows
// One wavefront per row; lane l owns columns 8*l .. 8*l+7 of every 512-column step.
// Eight consecutive elements as they come from memory (any element alignment).
template <int DT> struct Raw8 {
    typedef typename Io<DT>::T T;
    u32x4 a;
    __device__ __forceinline__ void load(const T *p) { a = *reinterpret_cast<const u32x4_unaligned *>(p); }
    __device__ __forceinline__ void unpack(float (&x)[8]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) { x[2 * i] = Io<DT>::lo(a[i]); x[2 * i + 1] = Io<DT>::hi(a[i]); }
    }
    static __device__ __forceinline__ void store(T *p, const float (&x)[8]) {
        store_result<false>(reinterpret_cast<u32x4_unaligned *>(p), u32x4{Io<DT>::pack(x[0], x[1]), Io<DT>::pack(x[2], x[3]),
                                                                   Io<DT>::pack(x[4], x[5]), Io<DT>::pack(x[6], x[7])});
    }
};
template <> struct Raw8<BA_F32> {
    typedef float T;
    f32x4 a, b;
    __device__ __forceinline__ void load(const T *p) {
        a = *reinterpret_cast<const f32x4_unaligned *>(p);
        b = *reinterpret_cast<const f32x4_unaligned *>(p + 4);
    }
    __device__ __forceinline__ void unpack(float (&x)[8]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) { x[i] = a[i]; x[4 + i] = b[i]; }
    }
    static __device__ __forceinline__ void store(T *p, const float (&x)[8]) {
        store_result<false>(reinterpret_cast<f32x4_unaligned *>(p), f32x4{x[0], x[1], x[2], x[3]});
        store_result<false>(reinterpret_cast<f32x4_unaligned *>(p + 4), f32x4{x[4], x[5], x[6], x[7]});
    }
};
// Forward softmax of rows first, first + stride, ... of one segment whose rows take STEPS 512-column
// steps (256 < cols <= 512 * STEPS); one wavefront per row, the whole row in registers.
// Every step is one unconditional 8-element load per lane: a lane whose run would pass the end of the
// row reads the eight elements ENDING at the row's end instead; the elements it shares with the lane
// before get weight 0 in the sum and are stored again with the same value (lanes wholly past the end
// repeat that last run).  Straight-line code: the loads of the next row are issued before the
// arithmetic of the current one, and nothing waits for stores.
template <int DT, int STEPS>
__device__ __forceinline__ void softmax_rows_forward(const typename Io<DT>::T *src, typename Io<DT>::T *dst, int rows,
                                                     int cols, int first, int stride, float c, float sgn) {
    const int lane = lane_id();
    int at[STEPS];                                       // first column of the lane's run in step k
#pragma unroll
    for (int k = 0; k < STEPS; ++k) at[k] = min(512 * k + 8 * lane, cols - 8);
    // elements of the last step's run that belong to the lanes before (8 or more: none are ours)
    const int own = 512 * (STEPS - 1) + 8 * lane - at[STEPS - 1];
    float w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = (i >= own && own < 8) ? 1.f : 0.f;
    Raw8<DT> raw[STEPS];
    if (first < rows) {
#pragma unroll
        for (int k = 0; k < STEPS; ++k) raw[k].load(src + (int64_t)first * cols + at[k]);
    }
    for (int r = first; r < rows; r += stride) {
        float v[STEPS][8];
#pragma unroll
        for (int k = 0; k < STEPS; ++k) raw[k].unpack(v[k]);
        if (r + stride < rows) {
#pragma unroll
            for (int k = 0; k < STEPS; ++k) raw[k].load(src + (int64_t)(r + stride) * cols + at[k]);
        }
        float mx = -3.0e38f;
#pragma unroll
        for (int k = 0; k < STEPS; ++k)
#pragma unroll
            for (int i = 0; i < 8; i += 2) mx = max3(mx, sgn * v[k][i], sgn * v[k][i + 1]);
        mx = wave_max(mx);
        const float bias = -((__builtin_fabsf(mx) == INFINITY) ? 0.f : mx) * c;
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < STEPS; ++k)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[k][i] = __builtin_amdgcn_exp2f(fmaf(sgn * v[k][i], c, bias));
                sum = k < STEPS - 1 ? sum + v[k][i] : fmaf(v[k][i], w[i], sum);
            }
        sum = wave_sum(sum);
        const float inv = __builtin_amdgcn_rcpf(sum);
        typename Io<DT>::T *y = dst + (int64_t)r * cols;
#pragma unroll
        for (int k = 0; k < STEPS; ++k) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[k][i] *= inv;
            Raw8<DT>::store(y + at[k], v[k]);
        }
    }
}

// Backward of rows first, first + stride, ... with the row's y and dy in registers (as they were loaded: 16-bit types
// stay packed), so that both are read from memory ONCE: dx = scale * (dy - sum(y * dy)) * y needs the row's sum before
// its first result.  The same runs, weights and re-stored overlap as in the forward above; the next row's loads are
// issued before the arithmetic of the current one, whose stores come after all of its loads (dst may alias y or dy).
template <int DT, int STEPS>
__device__ __forceinline__ void softmax_rows_backward(const typename Io<DT>::T *ysrc, const typename Io<DT>::T *gsrc,
                                                      typename Io<DT>::T *dst, int rows, int cols, int first, int stride,
                                                      float scale) {
    const int lane = lane_id();
    int at[STEPS];
#pragma unroll
    for (int k = 0; k < STEPS; ++k) at[k] = min(512 * k + 8 * lane, cols - 8);
    const int own = 512 * (STEPS - 1) + 8 * lane - at[STEPS - 1];
    float w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = (i >= own && own < 8) ? 1.f : 0.f;
    // up to 2048 columns two rows fit the registers of a wavefront at four wavefronts per SIMD; wider rows are loaded
    // when their turn comes, and the other wavefronts of the SIMD cover the wait
    constexpr bool kAhead = STEPS * (DT == BA_F32 ? 2 : 1) <= 4;
    Raw8<DT> ry[STEPS], rg[STEPS];
    if (kAhead && first < rows) {
#pragma unroll
        for (int k = 0; k < STEPS; ++k) {
            ry[k].load(ysrc + (int64_t)first * cols + at[k]);
            rg[k].load(gsrc + (int64_t)first * cols + at[k]);
        }
    }
    for (int r = first; r < rows; r += stride) {
        Raw8<DT> cy[STEPS], cg[STEPS];
        if constexpr (kAhead) {
#pragma unroll
            for (int k = 0; k < STEPS; ++k) { cy[k] = ry[k]; cg[k] = rg[k]; }
            if (r + stride < rows) {
#pragma unroll
                for (int k = 0; k < STEPS; ++k) {
                    ry[k].load(ysrc + (int64_t)(r + stride) * cols + at[k]);
                    rg[k].load(gsrc + (int64_t)(r + stride) * cols + at[k]);
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < STEPS; ++k) {
                cy[k].load(ysrc + (int64_t)r * cols + at[k]);
                cg[k].load(gsrc + (int64_t)r * cols + at[k]);
            }
        }
        float dot = 0.f;
#pragma unroll
        for (int k = 0; k < STEPS; ++k) {
            float yv[8], gv[8];
            cy[k].unpack(yv);
            cg[k].unpack(gv);
#pragma unroll
            for (int i = 0; i < 8; ++i) dot = k < STEPS - 1 ? fmaf(yv[i], gv[i], dot) : fmaf(yv[i] * gv[i], w[i], dot);
        }
        dot = wave_sum(dot);
        typename Io<DT>::T *dx = dst + (int64_t)r * cols;
#pragma unroll
        for (int k = 0; k < STEPS; ++k) {
            float yv[8], gv[8], dv[8];
            cy[k].unpack(yv);
            cg[k].unpack(gv);
#pragma unroll
            for (int i = 0; i < 8; ++i) dv[i] = scale * (gv[i] - dot) * yv[i];
            Raw8<DT>::store(dx + at[k], dv);
        }
    }
}

template <int DT, bool BACKWARD, int MAXG>
__global__ __launch_bounds__(kSoftmaxThreads, MAXG <= 8 ? 3 : 1) void softmax_runs_kernel(SoftmaxArgs a) {
    if (a.head_fast) softmax_runs_body<DT, BACKWARD, MAXG>(a, blockIdx.y, blockIdx.x, blockIdx.z, gridDim.z);
    else softmax_runs_body<DT, BACKWARD, MAXG>(a, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.z);
}

// lin = linear index of the workgroup in a grid of (list entries, gy heads, gz row groups)
template <int DT, bool BACKWARD>
__device__ __forceinline__ void softmax_rows_body(const SoftmaxArgs &a, uint64_t lin, unsigned gy, unsigned gz) {
    typedef typename Io<DT>::T T;
    // walks the plan's list of wide segments: the grid is as long as the list (or longer, without a host
    // copy of the plan summary)
    const int nseg = softmax_plan_nseg(a);
    if (nseg < 0) return;
    const int count = (int)((ConstHdr)(uintptr_t)a.plan)->totals[kListRows];
    const PlanRO pv = plan_ro(a.plan, nseg);
    // Workgroups start in the order of their linear index.  Taking the row group from its fastest digits,
    // then the head, then the list entry makes the machine work through one (segment, head) after the
    // other, each as one stream of consecutive rows; with the entry fastest it would read and write
    // hundreds of segments of unequal row lengths at once, which costs a third of the bandwidth.
    const unsigned group = (unsigned)(lin % gz), head = (unsigned)((lin / gz) % gy);
    const unsigned entry = (unsigned)(lin / ((uint64_t)gz * gy));
    const SegRec rec = load_rec(pv.recs + (int64_t)(kListRows + 1) * plan_cap(nseg), entry);
    if ((int)entry >= count) return;
    const int rows = rec.M, cols = rec.N;
    if (cols <= kRunCols) return;                       // the lane-run kernel's
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int lane = lane_id();
    const int first = group * kSoftmaxWaves + wave, stride = gz * kSoftmaxWaves;
    const int64_t seg0 = (int64_t)head * a.Dsrc + rec.offO;
    const T *src = reinterpret_cast<const T *>(a.src) + seg0;
    const T *aux = reinterpret_cast<const T *>(a.aux) + seg0;
    T *dst = reinterpret_cast<T *>(a.dst) + seg0;
    const float c_signed = a.scale * kLog2e;
    const float sgn = c_signed < 0.f ? -1.f : 1.f;
    const float c = c_signed * sgn;
    const int steps = (cols + 511) >> 9;

    if (!BACKWARD && steps <= kRowSteps) {
#define BA_ROWS(S_) case S_: softmax_rows_forward<DT, S_>(src, dst, rows, cols, first, stride, c, sgn); break;
        switch (steps) {
            BA_ROWS(1) BA_ROWS(2) BA_ROWS(3) BA_ROWS(4) BA_ROWS(5) BA_ROWS(6) BA_ROWS(7) BA_ROWS(8)
            default: break;
        }
#undef BA_ROWS
        return;
    }
    if (BACKWARD && steps <= (DT == BA_F32 ? kRowSteps / 2 : kRowSteps)) {
#define BA_ROWS(S_) case S_: softmax_rows_backward<DT, S_>(src, aux, dst, rows, cols, first, stride, a.scale); break;
        switch (steps) {
            BA_ROWS(1) BA_ROWS(2) BA_ROWS(3) BA_ROWS(4)
            default:
                if constexpr (DT != BA_F32) {
                    switch (steps) {
                        BA_ROWS(5) BA_ROWS(6) BA_ROWS(7) BA_ROWS(8)
                        default: break;
                    }
                }
                break;
        }
#undef BA_ROWS
        return;
    }
    // Rows wider than the register path holds (forward and backward): the row is streamed in 512-column steps,
    // four steps of loads in flight, once per pass.  A lane reads the run of eight elements that starts
    // at its column, or the run ENDING at the row's end when that would pass it; `own` is the number of
    // leading elements of the run that belong to the lanes before (8 or more: none are this lane's).
    // A lane writes only its own elements, so dst may alias src (or dy).
    auto run_at = [&](int k, int &own) {
        const int col = 512 * k + 8 * lane;
        const int at = min(col, cols - 8);
        own = col - at;
        return at;
    };
    auto store_own = [&](T *p, const float (&v)[8], int own) {
        if (own == 0) {
            Raw8<DT>::store(p, v);
        } else {
#pragma unroll
            for (int i = 1; i < 8; ++i)
                if (i >= own) Io<DT>::st(p + i, v[i]);
        }
    };
    // fn(k, at, own, x[8]) or, with a second source, fn(k, at, own, x[8], g[8]) for every step of the row
    auto sweep = [&](const T *x, const T *g, auto &&fn) {
        for (int k0 = 0; k0 < steps; k0 += 4) {
            Raw8<DT> rx[4], rg[4];
            int at[4], own[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (k0 + u < steps) {
                    at[u] = run_at(k0 + u, own[u]);
                    rx[u].load(x + at[u]);
                    if (BACKWARD) rg[u].load(g + at[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (k0 + u < steps) {
                    float xv[8], gv[8];
                    rx[u].unpack(xv);
                    if (BACKWARD) rg[u].unpack(gv);
                    fn(at[u], own[u], xv, gv);
                }
            }
        }
    };
    for (int r = first; r < rows; r += stride) {
        const int64_t e0 = (int64_t)r * cols;
        const T *x = src + e0;
        T *y = dst + e0;
        if (!BACKWARD) {
            float mx = -3.0e38f;
            sweep(x, x, [&](int, int, const float (&xv)[8], const float (&)[8]) {
#pragma unroll
                for (int i = 0; i < 8; i += 2) mx = max3(mx, sgn * xv[i], sgn * xv[i + 1]);
            });
            mx = wave_max(mx);
            const float bias = -((__builtin_fabsf(mx) == INFINITY) ? 0.f : mx) * c;
            float sum = 0.f;
            sweep(x, x, [&](int, int own, const float (&xv)[8], const float (&)[8]) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sgn * xv[i], c, bias));
                    sum += i >= own ? p : 0.f;
                }
            });
            sum = wave_sum(sum);
            const float inv = __builtin_amdgcn_rcpf(sum);
            sweep(x, x, [&](int at, int own, const float (&xv)[8], const float (&)[8]) {
                float pv[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) pv[i] = __builtin_amdgcn_exp2f(fmaf(sgn * xv[i], c, bias)) * inv;
                store_own(y + at, pv, own);
            });
        } else {
            // dx = scale * (dy - sum(y * dy)) * y; x is the saved forward output here.
            const T *dy = aux + e0;
            float dot = 0.f;
            sweep(x, dy, [&](int, int own, const float (&yv)[8], const float (&gv)[8]) {
#pragma unroll
                for (int i = 0; i < 8; ++i) dot += i >= own ? yv[i] * gv[i] : 0.f;
            });
            dot = wave_sum(dot);
            sweep(x, dy, [&](int at, int own, const float (&yv)[8], const float (&gv)[8]) {
                float dv[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) dv[i] = a.scale * (gv[i] - dot) * yv[i];
                store_own(y + at, dv, own);
            });
        }
    }
}

template <int DT, bool BACKWARD>
__global__ __launch_bounds__(kSoftmaxThreads) void softmax_rows_kernel(SoftmaxArgs a) {
    const uint64_t lin = blockIdx.x + (uint64_t)gridDim.x * (blockIdx.y + (uint64_t)gridDim.y * blockIdx.z);
    softmax_rows_body<DT, BACKWARD>(a, lin, gridDim.y, gridDim.z);
}

// Both kernels in one launch (flat grid): the first both.rows_blocks workgroups are the row kernel's (wide
// rows run longest, so they start first), the rest decode to the lane-run kernel's (segment, head, row group),
// segment fastest.  Two launches that would each leave part of the machine idle become one.
struct BothGrid {
    unsigned rows_blocks, rows_z, runs_slots, runs_z;
};
template <int DT>
__global__ __launch_bounds__(kSoftmaxThreads, DT == 2 ? 2 : 3) void softmax_both_kernel(SoftmaxArgs a, BothGrid both) {
    const unsigned id = blockIdx.x;
    if (id < both.rows_blocks) {
        softmax_rows_body<DT, false>(a, id, (unsigned)a.H, both.rows_z);
        return;
    }
    const unsigned r = id - both.rows_blocks;
    const unsigned bx = a.head_fast ? (r / (unsigned)a.H) % both.runs_slots : r % both.runs_slots;
    const unsigned by = a.head_fast ? r % (unsigned)a.H : (r / both.runs_slots) % (unsigned)a.H;
    softmax_runs_body<DT, false, 16>(a, bx, by, r / (both.runs_slots * (unsigned)a.H), both.runs_z);
}

template <int DT, bool BACKWARD>
static int launch_softmax_t(const SoftmaxArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    const int cus = device_cu_count();
    // lane-run kernel: z spreads the 16-row strips over workgroups when there are few (segment, head) pairs
    int64_t z_runs = 4, z_rows = 8;
    bool rows_work = true;
    int64_t n_rows = nseg;                               // length of the row kernel's list (grid)
    if (info) {
        nseg = info->nseg;
        const int64_t groups = (((int64_t)info->max_M + 15) / 16 + kSoftmaxWaves - 1) / kSoftmaxWaves;
        // sixteen workgroups per compute unit: with one 16-row strip per wavefront the segments of a batch finish
        // together (256 segments x 8 heads of 32..128 rows: 14.4 us with two workgroups per segment, 15.6 with one)
        const int64_t want = ((int64_t)cus * 16 + nseg * args.H - 1) / std::max<int64_t>(1, nseg * args.H);
        z_runs = std::max<int64_t>(1, std::min<int64_t>(groups, std::min<int64_t>(want, 64)));
        n_rows = info->list_rows;
        rows_work = n_rows > 0;
        // row kernel: about four workgroups' worth of rows in flight per compute unit over ITS segments,
        // never more than one wavefront per row
        const int64_t pairs = std::max<int64_t>(1, n_rows * args.H);
        const int64_t want_rows = ((int64_t)cus * 32 + pairs - 1) / pairs;
        z_rows = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want_rows, 4096),
                                                        (info->max_M + kSoftmaxWaves - 1) / kSoftmaxWaves));
    }
    if (nseg <= 0) return BA_OK;
    // head as the fastest grid index of the lane-run kernel: workgroups that start together are the heads of one
    // segment and take equally long
    static const int hf = [] { const char *e = getenv("BLOCKEDATTN_HEAD_FAST"); return e ? atoi(e) : 1; }();
    SoftmaxArgs run = args;
    run.head_fast = hf && nseg <= 65535 ? 1 : 0;
    const dim3 grid_runs = run.head_fast ? dim3((unsigned)args.H, (unsigned)nseg, (unsigned)z_runs)
                                         : dim3((unsigned)nseg, (unsigned)args.H, (unsigned)z_runs);
    if constexpr (!BACKWARD) {
        // a modest row-kernel launch (it would not fill the machine for long) rides with the lane-run kernel
        static const int both_env = [] { const char *e = getenv("BLOCKEDATTN_SOFTMAX_BOTH"); return e ? atoi(e) : -1; }();
        const int64_t rows_blocks = n_rows * args.H * z_rows, runs_blocks = nseg * args.H * z_runs;
        const bool both = info && rows_work && n_rows < nseg && info->max_N > 128 &&
                          rows_blocks + runs_blocks < (int64_t(1) << 31) &&
                          (both_env >= 0 ? both_env != 0 : rows_blocks <= (int64_t)cus * 64);
        if (both) {
            const BothGrid bg{(unsigned)rows_blocks, (unsigned)z_rows, (unsigned)nseg, (unsigned)z_runs};
            hipLaunchKernelGGL((softmax_both_kernel<DT>), dim3((unsigned)(rows_blocks + runs_blocks)), dim3(kSoftmaxThreads), 0,
                               stream, run, bg);
            return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
        }
    }
    if (info && info->max_N <= 128)
        hipLaunchKernelGGL((softmax_runs_kernel<DT, BACKWARD, 8>), grid_runs, dim3(kSoftmaxThreads), 0, stream, run);
    else
        hipLaunchKernelGGL((softmax_runs_kernel<DT, BACKWARD, 16>), grid_runs, dim3(kSoftmaxThreads), 0, stream, run);
    if (rows_work)
        hipLaunchKernelGGL((softmax_rows_kernel<DT, BACKWARD>),
                           dim3((unsigned)n_rows, (unsigned)args.H, (unsigned)z_rows), dim3(kSoftmaxThreads), 0, stream,
                           args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

// ---------------------------------------------------------------- fp64
// The reference instantiates its softmax for double as well (csrc/cuda/spBlkSoftmax.cu:400).  One wavefront per
// row, arithmetic in double, the row read again for each of the three steps (maximum, sum, result); grid
// (segment, head, z), wavefront w of workgroup z takes rows 4 z + w, then on in steps of 4 gridDim.z.
__device__ __forceinline__ double wave_max_f64(double v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmax(v, __shfl_xor(v, m));
    return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m);
    return v;
}

template <bool BACKWARD>
__global__ __launch_bounds__(kSoftmaxThreads) void softmax_f64_kernel(SoftmaxArgs a) {
    const int nseg = softmax_plan_nseg(a);
    const int g = blockIdx.x;
    if (g >= nseg) return;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int rows = rec.M, cols = rec.N;
    if (rows < 1 || cols < 1) return;
    const int wave = uniform((int)(threadIdx.x >> 6)), lane = lane_id();
    const int64_t seg0 = (int64_t)blockIdx.y * a.Dsrc + rec.offO;
    const double *src = reinterpret_cast<const double *>(a.src) + seg0;
    const double *aux = reinterpret_cast<const double *>(a.aux) + seg0;
    double *dst = reinterpret_cast<double *>(a.dst) + seg0;
    const double scale = (double)a.scale;
    for (int r = blockIdx.z * kSoftmaxWaves + wave; r < rows; r += gridDim.z * kSoftmaxWaves) {
        const double *x = src + (int64_t)r * cols;
        double *y = dst + (int64_t)r * cols;
        if constexpr (!BACKWARD) {
            double m = -INFINITY;
            for (int c = lane; c < cols; c += 64) m = fmax(m, x[c] * scale);
            m = wave_max_f64(m);
            double sum = 0.0;
            for (int c = lane; c < cols; c += 64) sum += exp(x[c] * scale - m);
            sum = wave_sum_f64(sum);
            for (int c = lane; c < cols; c += 64) y[c] = exp(x[c] * scale - m) / sum;       // a row of -inf: NaN, like torch
        } else {
            const double *dy = aux + (int64_t)r * cols;
            double dot = 0.0;
            for (int c = lane; c < cols; c += 64) dot += x[c] * dy[c];
            dot = wave_sum_f64(dot);
            for (int c = lane; c < cols; c += 64) y[c] = scale * (dy[c] - dot) * x[c];
        }
    }
}

template <bool BACKWARD>
static int launch_softmax_f64(const SoftmaxArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;
    int64_t z = 8;
    if (info) {
        nseg = info->nseg;
        const int64_t pairs = std::max<int64_t>(1, nseg * args.H);
        const int64_t want = ((int64_t)device_cu_count() * 16 + pairs - 1) / pairs;
        z = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, 4096),
                                                   (info->max_M + kSoftmaxWaves - 1) / kSoftmaxWaves));
    }
    if (nseg <= 0) return BA_OK;
    if (nseg > 2147483647) return BA_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((softmax_f64_kernel<BACKWARD>), dim3((unsigned)nseg, (unsigned)args.H, (unsigned)z),
                       dim3(kSoftmaxThreads), 0, stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_softmax(int dtype, void *plan, int64_t nseg, const void *src, void *dst, int64_t H, int64_t Dsrc,
                   float scale, const ba_plan_info *info, hipStream_t stream) {
    SoftmaxArgs args{plan, src, nullptr, dst, H, Dsrc, scale};
    switch (dtype) {
        case BA_F16: return launch_softmax_t<BA_F16, false>(args, nseg, info, stream);
        case BA_BF16: return launch_softmax_t<BA_BF16, false>(args, nseg, info, stream);
        case BA_F32: return launch_softmax_t<BA_F32, false>(args, nseg, info, stream);
        case BA_F64: return launch_softmax_f64<false>(args, nseg, info, stream);
        default: return BA_ERR_UNSUPPORTED;
    }
}

// Backward of the blocked softmax: dx = scale * (dy - sum(y * dy)) * y per row
// (csrc/cuda/spBlkSoftmax.cu:140-180, 271-332; the reference has scale = 1).
int launch_softmax_backward(int dtype, void *plan, int64_t nseg, const void *y, const void *dy, void *dx, int64_t H,
                            int64_t Dsrc, float scale, const ba_plan_info *info, hipStream_t stream) {
    SoftmaxArgs args{plan, y, dy, dx, H, Dsrc, scale};
    switch (dtype) {
        case BA_F16: return launch_softmax_t<BA_F16, true>(args, nseg, info, stream);
        case BA_BF16: return launch_softmax_t<BA_BF16, true>(args, nseg, info, stream);
        case BA_F32: return launch_softmax_t<BA_F32, true>(args, nseg, info, stream);
        case BA_F64: return launch_softmax_f64<true>(args, nseg, info, stream);
        default: return BA_ERR_UNSUPPORTED;
    }
}

}  // namespace ba
