// Standalone blocked row softmax: dst row = softmax(scale * src row) for every
// row of every segment (csrc/cuda/spBlkSoftmax.cu:88-138, 182-269 restated for
// wave64).  fp32 arithmetic for every dtype, one rounding at the store, no
// column limit.
//
// A row is a contiguous run of `cols` elements, and consecutive rows of a
// segment are contiguous too.  Rows of up to 64*kRegs elements are held in
// registers by one wavefront (lane-strided, so every load and store of the
// wavefront is one contiguous 128/256-byte run); longer rows are re-read from
// the cache hierarchy in three passes.
#include <algorithm>

#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kSoftmaxThreads = 256;
constexpr int kSoftmaxWaves = kSoftmaxThreads / 64;
constexpr int kRegs = 16;  // elements per lane kept in registers: rows up to 1024 columns

template <int DT> struct Io;
template <> struct Io<BA_F16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const T *p) { return Elem<0>::to_float(*p); }
    static __device__ __forceinline__ void st(T *p, float v) { *p = Elem<0>::from_float(v); }
};
template <> struct Io<BA_BF16> {
    typedef uint16_t T;
    static __device__ __forceinline__ float ld(const T *p) { return Elem<1>::to_float(*p); }
    static __device__ __forceinline__ void st(T *p, float v) { *p = Elem<1>::from_float(v); }
};
template <> struct Io<BA_F32> {
    typedef float T;
    static __device__ __forceinline__ float ld(const T *p) { return *p; }
    static __device__ __forceinline__ void st(T *p, float v) { *p = v; }
};

struct SoftmaxArgs {
    void *plan;
    const void *src;
    void *dst;
    int64_t H, Dsrc;
    float scale;
};

template <int DT> __global__ __launch_bounds__(kSoftmaxThreads) void softmax_rows_kernel(SoftmaxArgs a) {
    typedef typename Io<DT>::T T;
    PlanHeader *hdr = reinterpret_cast<PlanHeader *>(a.plan);
    if (hdr->magic != kPlanMagic || hdr->bad_segments != 0 || hdr->Dout != a.Dsrc) {
        if (blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&hdr->run_errors, 1);
        return;
    }
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const ConstI32 pfx = pv.pfx[kPfxRows];
    const int64_t per_head = hdr->totals[kPfxRows];
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int lane = lane_id();
    float c = a.scale * kLog2e;
    const float sgn = c < 0.f ? -1.f : 1.f;  // work on sgn*x so the multiplier is >= 0
    c *= sgn;
    const T *src = reinterpret_cast<const T *>(a.src);
    T *dst = reinterpret_cast<T *>(a.dst);

    const int64_t gw = (int64_t)blockIdx.x * kSoftmaxWaves + wave, nw = (int64_t)gridDim.x * kSoftmaxWaves;
    for (int64_t it = gw; it < per_head * a.H; it += nw) {
        const int64_t h = it / per_head;
        const int i = (int)(it - h * per_head);
        const int g = prefix_search(pfx, nseg, i);
        const int r = i - pfx[g];
        const SegRec rec = load_rec(pv.recs, g);
        const int cols = rec.N;
        const int64_t e0 = h * a.Dsrc + rec.offO + (int64_t)r * cols;
        const T *x = src + e0;
        T *y = dst + e0;
        if (cols <= 64 * kRegs) {
            float v[kRegs];
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int col = lane + 64 * j;
                v[j] = (col < cols) ? sgn * Io<DT>::ld(x + col) : -INFINITY;
                mx = fmaxf(mx, v[j]);
            }
            mx = wave_max(mx);
            const float bias = -((mx == -INFINITY) ? 0.f : mx) * c;
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int col = lane + 64 * j;
                v[j] = (col < cols) ? __builtin_amdgcn_exp2f(fmaf(v[j], c, bias)) : 0.f;
                sum += v[j];
            }
            sum = wave_sum(sum);
            const float inv = 1.f / sum;
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int col = lane + 64 * j;
                if (col < cols) Io<DT>::st(y + col, v[j] * inv);
            }
        } else {
            float mx = -INFINITY;
            for (int col = lane; col < cols; col += 64) mx = fmaxf(mx, sgn * Io<DT>::ld(x + col));
            mx = wave_max(mx);
            const float bias = -((mx == -INFINITY) ? 0.f : mx) * c;
            float sum = 0.f;
            for (int col = lane; col < cols; col += 64)
                sum += __builtin_amdgcn_exp2f(fmaf(sgn * Io<DT>::ld(x + col), c, bias));
            sum = wave_sum(sum);
            const float inv = 1.f / sum;
            // src may alias dst: every lane re-reads only the elements it writes.
            for (int col = lane; col < cols; col += 64)
                Io<DT>::st(y + col, __builtin_amdgcn_exp2f(fmaf(sgn * Io<DT>::ld(x + col), c, bias)) * inv);
        }
    }
}

template <int DT> static int launch_softmax_t(const SoftmaxArgs &args, const ba_plan_info *info, hipStream_t stream) {
    // Resident-size grid; with the row count known, no more groups than rows need.
    int64_t grid = (int64_t)device_cu_count() * 8;
    if (info) grid = std::min(grid * 4, (info->total_rows * args.H + kSoftmaxWaves - 1) / kSoftmaxWaves);
    if (grid <= 0) return BA_OK;
    hipLaunchKernelGGL(softmax_rows_kernel<DT>, dim3((unsigned)grid), dim3(kSoftmaxThreads), 0, stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_softmax(int dtype, void *plan, const void *src, void *dst, int64_t H, int64_t Dsrc, float scale,
                   const ba_plan_info *info, hipStream_t stream) {
    SoftmaxArgs args{plan, src, dst, H, Dsrc, scale};
    switch (dtype) {
        case BA_F16: return launch_softmax_t<BA_F16>(args, info, stream);
        case BA_BF16: return launch_softmax_t<BA_BF16>(args, info, stream);
        case BA_F32: return launch_softmax_t<BA_F32>(args, info, stream);
        default: return BA_ERR_UNSUPPORTED;
    }
}

// Backward of the blocked softmax: dx = scale * (dy - sum(y * dy)) * y per row
// (csrc/cuda/spBlkSoftmax.cu:140-180, 271-332; the reference has scale = 1).
// y is the saved forward output.  Same row mapping as the forward kernel;
// products and the row sum are fp32 for every dtype.
struct SoftmaxBwdArgs {
    void *plan;
    const void *y;
    const void *dy;
    void *dx;
    int64_t H, Dsrc;
    float scale;
};

template <int DT> __global__ __launch_bounds__(kSoftmaxThreads) void softmax_rows_backward_kernel(SoftmaxBwdArgs a) {
    typedef typename Io<DT>::T T;
    PlanHeader *hdr = reinterpret_cast<PlanHeader *>(a.plan);
    if (hdr->magic != kPlanMagic || hdr->bad_segments != 0 || hdr->Dout != a.Dsrc) {
        if (blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&hdr->run_errors, 1);
        return;
    }
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const ConstI32 pfx = pv.pfx[kPfxRows];
    const int64_t per_head = hdr->totals[kPfxRows];
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int lane = lane_id();
    const T *ys = reinterpret_cast<const T *>(a.y), *dys = reinterpret_cast<const T *>(a.dy);
    T *dxs = reinterpret_cast<T *>(a.dx);
    const int64_t gw = (int64_t)blockIdx.x * kSoftmaxWaves + wave, nw = (int64_t)gridDim.x * kSoftmaxWaves;
    for (int64_t it = gw; it < per_head * a.H; it += nw) {
        const int64_t h = it / per_head;
        const int i = (int)(it - h * per_head);
        const int g = prefix_search(pfx, nseg, i);
        const int r = i - pfx[g];
        const SegRec rec = load_rec(pv.recs, g);
        const int cols = rec.N;
        const int64_t e0 = h * a.Dsrc + rec.offO + (int64_t)r * cols;
        const T *y = ys + e0, *dy = dys + e0;
        T *dx = dxs + e0;
        if (cols <= 64 * kRegs) {
            float yv[kRegs], gv[kRegs];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int col = lane + 64 * j;
                yv[j] = (col < cols) ? Io<DT>::ld(y + col) : 0.f;
                gv[j] = (col < cols) ? Io<DT>::ld(dy + col) : 0.f;
                dot = fmaf(yv[j], gv[j], dot);
            }
            dot = wave_sum(dot);
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int col = lane + 64 * j;
                if (col < cols) Io<DT>::st(dx + col, a.scale * (gv[j] - dot) * yv[j]);
            }
        } else {
            float dot = 0.f;
            for (int col = lane; col < cols; col += 64) dot = fmaf(Io<DT>::ld(y + col), Io<DT>::ld(dy + col), dot);
            dot = wave_sum(dot);
            for (int col = lane; col < cols; col += 64)
                Io<DT>::st(dx + col, a.scale * (Io<DT>::ld(dy + col) - dot) * Io<DT>::ld(y + col));
        }
    }
}

template <int DT>
static int launch_softmax_bwd_t(const SoftmaxBwdArgs &args, const ba_plan_info *info, hipStream_t stream) {
    int64_t grid = (int64_t)device_cu_count() * 8;
    if (info) grid = std::min(grid * 4, (info->total_rows * args.H + kSoftmaxWaves - 1) / kSoftmaxWaves);
    if (grid <= 0) return BA_OK;
    hipLaunchKernelGGL(softmax_rows_backward_kernel<DT>, dim3((unsigned)grid), dim3(kSoftmaxThreads), 0, stream,
                       args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_softmax_backward(int dtype, void *plan, const void *y, const void *dy, void *dx, int64_t H, int64_t Dsrc,
                            float scale, const ba_plan_info *info, hipStream_t stream) {
    SoftmaxBwdArgs args{plan, y, dy, dx, H, Dsrc, scale};
    switch (dtype) {
        case BA_F16: return launch_softmax_bwd_t<BA_F16>(args, info, stream);
        case BA_BF16: return launch_softmax_bwd_t<BA_BF16>(args, info, stream);
        case BA_F32: return launch_softmax_bwd_t<BA_F32>(args, info, stream);
        default: return BA_ERR_UNSUPPORTED;
    }
}

}  // namespace ba
