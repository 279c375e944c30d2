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

__global__ __launch_bounds__(kF32Threads) void gemm_f32_kernel(RunArgs a) {
    PlanHeader *hdr = reinterpret_cast<PlanHeader *>(a.plan);
    if (hdr->magic != kPlanMagic || hdr->kind != 0 || hdr->bad_segments != 0 || hdr->Dm1 != a.Dm1 ||
        hdr->Dm2 != a.Dm2 || hdr->Dout != a.Dout) {
        if (blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&hdr->run_errors, 1);
        return;
    }
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int lane = lane_id();
    const bool t1 = a.flags & kFlagTranspose1, t2 = a.flags & kFlagTranspose2;
    const float *A = reinterpret_cast<const float *>(a.A), *B = reinterpret_cast<const float *>(a.B);
    float *out = reinterpret_cast<float *>(a.out);
    const int64_t gw = (int64_t)blockIdx.x * kF32Waves + wave, nw = (int64_t)gridDim.x * kF32Waves;

    // The plan sorts every segment into exactly one of three lists: GEMM pieces
    // (16 rows x one 256-column chunk), packs of tiny segments (every member is
    // smaller than one piece) and slow strips (16 rows x all columns).  The fp32
    // kernel walks all three with the same inner routine.
    const int kinds[3] = {kPfxPack, kPfxGemm, kPfxSlow};
    for (int phase = 0; phase < 3; ++phase) {
        const int kind = kinds[phase];
        const int64_t per_head = hdr->totals[kind];
        const ConstI32 pfx = pv.pfx[kind];
        for (int64_t it = gw; it < per_head * a.H; it += nw) {
            const int64_t h = it / per_head;
            const int i = (int)(it - h * per_head);
            const int g0 = prefix_search(pfx, nseg, i);
            const int members = kind == kPfxPack ? pv.recs[g0].packLen : 1;
            for (int j = 0; j < members; ++j) {
                const int g = g0 + j;
                const SegRec rec = load_rec(pv.recs, g);
                const int M = rec.M, N = rec.N, K = rec.K;
                int r0 = 0, c0 = 0, c1 = N;
                if (kind == kPfxGemm) {
                    const int local = i - pfx[g];
                    const int chunks = (N + kWaveCols - 1) / kWaveCols;
                    r0 = (local / chunks) * kStripRows; c0 = (local % chunks) * kWaveCols;
                    c1 = min(N, c0 + kWaveCols);
                } else if (kind == kPfxSlow) {
                    r0 = (i - pfx[g]) * kStripRows;
                }
                const float *as = A + h * a.Dm1 + rec.off1;
                const float *bs = B + h * a.Dm2 + rec.off2;
                float *os = out + h * a.Dout + rec.offO;
                const int rows = min(kStripRows, M - r0);
                for (int col = c0 + lane; col < c1; col += 64) {
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
    }
}

int launch_gemm_f32(const RunArgs &args, const ba_plan_info *info, hipStream_t stream) {
    int64_t grid = (int64_t)device_cu_count() * 8;
    if (info) {
        const int64_t items = (info->gemm_items + info->pack_items + info->slow_items) * args.H;
        grid = std::min(grid * 8, (items + kF32Waves - 1) / kF32Waves);
    }
    if (grid <= 0) return BA_OK;
    hipLaunchKernelGGL(gemm_f32_kernel, dim3((unsigned)grid), dim3(kF32Threads), 0, stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
