// fp32 varlen GEMM (the reference's generic kernel, csrc/cuda/spBlkGEMM.cu:120-271,
// for T = float): fp32 multiply-add on the vector ALU, accumulation in k order.
// A correctness path for fp32 callers; the fp16/bf16 MFMA kernels are the fast path.
//
// One wavefront computes a 16-row piece of one segment; lane l owns columns
// c0 + l + 64*j, so the stores of one output row are one contiguous run.
#include <algorithm>

#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kF32Threads = 256;
constexpr int kF32Waves = kF32Threads / 64;

// grid (segment, head, z): the wavefronts of the workgroup take the 16-row
// strips of one segment of one head.
__global__ __launch_bounds__(kF32Threads) void gemm_f32_kernel(RunArgs a) {
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const uint32_t magic = hdr->magic;
    const int nseg = hdr->nseg, pkind = hdr->kind, bad = hdr->bad_segments;
    const int64_t d1 = hdr->Dm1, d2 = hdr->Dm2, dO = hdr->Dout;
    if (!((magic == kPlanMagic) & (pkind == 0) & (bad == 0) & (d1 == a.Dm1) & (d2 == a.Dm2) & (dO == a.Dout))) {
        if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    const int g = blockIdx.x;
    if (g >= nseg) return;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int M = rec.M, N = rec.N, K = rec.K;
    if (M < 1 || N < 1) return;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int lane = lane_id();
    const bool t1 = a.flags & kFlagTranspose1, t2 = a.flags & kFlagTranspose2;
    const int64_t h = blockIdx.y;
    const float *as = reinterpret_cast<const float *>(a.A) + h * a.Dm1 + rec.off1;
    const float *bs = reinterpret_cast<const float *>(a.B) + h * a.Dm2 + rec.off2;
    float *os = reinterpret_cast<float *>(a.out) + h * a.Dout + rec.offO;
    const int strips = (M + kStripRows - 1) / kStripRows;
    for (int strip = blockIdx.z * kF32Waves + wave; strip < strips; strip += gridDim.z * kF32Waves) {
        const int r0 = strip * kStripRows;
        const int rows = min(kStripRows, M - r0);
        for (int col = lane; col < N; col += 64) {
            float acc[kStripRows];
#pragma unroll
            for (int r = 0; r < kStripRows; ++r) acc[r] = 0.f;
            for (int t = 0; t < K; ++t) {
                const float bv = t2 ? bs[(int64_t)t * N + col] : bs[(int64_t)col * K + t];
#pragma unroll
                for (int r = 0; r < kStripRows; ++r) {
                    if (r < rows) {
                        const int row = r0 + r;
                        const float av = t1 ? as[(int64_t)t * M + row] : as[(int64_t)row * K + t];
                        acc[r] = fmaf(av, bv, acc[r]);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < kStripRows; ++r)
                if (r < rows) os[(int64_t)(r0 + r) * N + col] = acc[r];
        }
    }
}

int launch_gemm_f32(const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    int64_t z = 4;
    if (info) {
        nseg = info->nseg;
        z = std::max<int64_t>(1, std::min<int64_t>(64, (info->max_M + kStripRows * kF32Waves - 1) / (kStripRows * kF32Waves)));
    }
    if (nseg <= 0) return BA_OK;
    hipLaunchKernelGGL(gemm_f32_kernel, dim3((unsigned)nseg, (unsigned)args.H, (unsigned)z), dim3(kF32Threads), 0,
                       stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
