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
    const void *src;     // forward: x            backward: y (saved forward output)
    const void *aux;     // forward: unused       backward: dy
    void *dst;           // forward: y            backward: dx
    int64_t H, Dsrc;
    float scale;
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

// grid (segment, head, z): the workgroup's wavefronts walk the rows of one
// segment of one head, row r going to wavefront r mod (4 * gridDim.z).
template <int DT, bool BACKWARD>
__global__ __launch_bounds__(kSoftmaxThreads) void softmax_rows_kernel(SoftmaxArgs a) {
    typedef typename Io<DT>::T T;
    const int nseg = softmax_plan_nseg(a);
    const int g = blockIdx.x;
    if (g >= nseg) return;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int rows = rec.M, cols = rec.N;
    if (cols < 1) return;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int lane = lane_id();
    const int first = blockIdx.z * kSoftmaxWaves + wave, stride = gridDim.z * kSoftmaxWaves;
    const int64_t seg0 = (int64_t)blockIdx.y * a.Dsrc + rec.offO;
    const T *src = reinterpret_cast<const T *>(a.src) + seg0;
    const T *aux = reinterpret_cast<const T *>(a.aux) + seg0;
    T *dst = reinterpret_cast<T *>(a.dst) + seg0;
    float c = a.scale * kLog2e;
    const float sgn = c < 0.f ? -1.f : 1.f;  // forward works on sgn*x so the multiplier is >= 0
    c *= sgn;

    for (int r = first; r < rows; r += stride) {
        const int64_t e0 = (int64_t)r * cols;
        const T *x = src + e0;
        T *y = dst + e0;
        if (!BACKWARD) {
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
        } else {
            // dx = scale * (dy - sum(y * dy)) * y; x is the saved forward output here.
            const T *dy = aux + e0;
            if (cols <= 64 * kRegs) {
                float yv[kRegs], gv[kRegs];
                float dot = 0.f;
#pragma unroll
                for (int j = 0; j < kRegs; ++j) {
                    const int col = lane + 64 * j;
                    yv[j] = (col < cols) ? Io<DT>::ld(x + col) : 0.f;
                    gv[j] = (col < cols) ? Io<DT>::ld(dy + col) : 0.f;
                    dot = fmaf(yv[j], gv[j], dot);
                }
                dot = wave_sum(dot);
#pragma unroll
                for (int j = 0; j < kRegs; ++j) {
                    const int col = lane + 64 * j;
                    if (col < cols) Io<DT>::st(y + col, a.scale * (gv[j] - dot) * yv[j]);
                }
            } else {
                float dot = 0.f;
                for (int col = lane; col < cols; col += 64) dot = fmaf(Io<DT>::ld(x + col), Io<DT>::ld(dy + col), dot);
                dot = wave_sum(dot);
                for (int col = lane; col < cols; col += 64)
                    Io<DT>::st(y + col, a.scale * (Io<DT>::ld(dy + col) - dot) * Io<DT>::ld(x + col));
            }
        }
    }
}

template <int DT, bool BACKWARD>
static int launch_softmax_t(const SoftmaxArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    int64_t z = 8;
    if (info) {
        nseg = info->nseg;
        z = std::max<int64_t>(1, std::min<int64_t>(64, (info->max_M + 4 * kSoftmaxWaves - 1) / (4 * kSoftmaxWaves)));
    }
    if (nseg <= 0) return BA_OK;
    hipLaunchKernelGGL((softmax_rows_kernel<DT, BACKWARD>), dim3((unsigned)nseg, (unsigned)args.H, (unsigned)z),
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
        default: return BA_ERR_UNSUPPORTED;
    }
}

}  // namespace ba
