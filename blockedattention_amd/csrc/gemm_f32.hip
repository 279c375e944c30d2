// fp32 varlen GEMM (the reference's generic kernel, csrc/cuda/spBlkGEMM.cu:120-271,
// for T = float) on the fp32 matrix instruction (v_mfma_f32_16x16x4_f32, fp32
// products and sums), any shape, offset and layout (transpose flags).  It serves
// fp32 callers such as the reference's own test; fp16/bf16 have their own kernels.
//
// Workgroup = 64 rows x 64 columns of one segment and head at a time, k in chunks
// of 64.  A chunk of B_g (64 columns x 64 k) is staged in LDS by the whole
// workgroup with coalesced loads along the operand's contiguous dimension, stored
// [column][k] with an odd pitch; each wavefront stages its own 16 rows of A_g
// [row][k].  A wavefront computes 16 rows x 64 columns as four 16 x 16 tiles: per
// four k it reads one A word and four B words per lane from LDS and issues four
// matrix instructions.
#include <algorithm>

#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kF32Threads = 256;
constexpr int kF32Waves = kF32Threads / 64;
constexpr int kF32Cols = 64;                         // columns per block = lanes
constexpr int kF32K = 64;                            // k per chunk
constexpr int kF32Rows = kStripRows * kF32Waves;     // rows per workgroup round
constexpr int kF32PitchB = kF32K + 1;                // odd: lanes (columns) fall on consecutive banks
constexpr int kF32PitchA = kF32K + 4;                // 16-byte rows, staggered banks

typedef float f32x4v __attribute__((ext_vector_type(4)));

// grid (head, segment, z) with kFlagHeadFast (consecutive workgroups, which go to the dies in turn, are the heads
// of one segment), else (segment, head, z): workgroup z takes the 64-row rounds z, z + gridDim.z, ... of its segment.
__global__ __launch_bounds__(kF32Threads) void gemm_f32_kernel(RunArgs a) {
    __shared__ float sB[kF32Cols * kF32PitchB];
    __shared__ __attribute__((aligned(16))) float sA[kF32Waves][kStripRows * kF32PitchA];
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const uint32_t magic = hdr->magic;
    const int nseg = hdr->nseg, pkind = hdr->kind, bad = hdr->bad_segments;
    const int64_t d1 = hdr->Dm1, d2 = hdr->Dm2, dO = hdr->Dout;
    if (!((magic == kPlanMagic) & (pkind == 0) & (bad == 0) & (d1 == a.Dm1) & (d2 == a.Dm2) & (dO == a.Dout))) {
        if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    const bool head_fast = a.flags & kFlagHeadFast;
    const int g = head_fast ? blockIdx.y : blockIdx.x;
    if (g >= nseg) return;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int M = rec.M, N = rec.N, K = rec.K;
    if (M < 1 || N < 1) return;
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = lane_id();
    const bool t1 = a.flags & kFlagTranspose1, t2 = a.flags & kFlagTranspose2;
    const int64_t h = head_fast ? blockIdx.x : blockIdx.y;
    const float *as = reinterpret_cast<const float *>(a.A) + h * a.Dm1 + rec.off1;
    const float *bs = reinterpret_cast<const float *>(a.B) + h * a.Dm2 + rec.off2;
    float *os = reinterpret_cast<float *>(a.out) + h * a.Dout + rec.offO;
    float *myA = sA[wave];
    const int nkc = (K + kF32K - 1) / kF32K;

    for (int round = blockIdx.z; round * kF32Rows < M; round += gridDim.z) {
        const int r0 = round * kF32Rows + wave * kStripRows;          // this wavefront's 16 rows
        for (int c0 = 0; c0 < N; c0 += kF32Cols) {
            // four 16 x 16 tiles per wavefront: lane (j = lane%16, q = lane/16) holds rows 4q..4q+3 of column j
            f32x4v acc[kF32Cols / 16];
#pragma unroll
            for (int t = 0; t < kF32Cols / 16; ++t) acc[t] = f32x4v{0.f, 0.f, 0.f, 0.f};
            for (int kc = 0; kc < nkc; ++kc) {                         // K = 0: no chunk, the result is zeros
                const int k0 = kc * kF32K;
                __syncthreads();                                       // the previous chunk is consumed
                // Staging: every load is unconditional (index clamped into the segment, value zeroed
                // afterwards where it lies outside), so the sixteen loads of a thread are in flight together.
                // ---- B chunk: sB[col][k] = B_g[c0 + col][k0 + k], zero outside the segment
                {
                    float v[16];
                    if (!t2) {
                        // rows of B_g are contiguous in k: lane = k, each wavefront 16 columns
                        const int kk = tid & 63, k = k0 + kk, cq = (tid >> 6) * 16;
                        const int kc_ = min(k, K - 1);
#pragma unroll
                        for (int i = 0; i < 16; ++i) v[i] = bs[(int64_t)min(c0 + cq + i, N - 1) * K + kc_];
#pragma unroll
                        for (int i = 0; i < 16; ++i)
                            sB[(cq + i) * kF32PitchB + kk] = (c0 + cq + i < N && k < K) ? v[i] : 0.f;
                    } else {
                        // stored K x N: contiguous in the column
                        const int col = tid & 63, kq = (tid >> 6) * 16;
                        const int cc = min(c0 + col, N - 1);
#pragma unroll
                        for (int i = 0; i < 16; ++i) v[i] = bs[(int64_t)min(k0 + kq + i, K - 1) * N + cc];
#pragma unroll
                        for (int i = 0; i < 16; ++i)
                            sB[col * kF32PitchB + kq + i] = (c0 + col < N && k0 + kq + i < K) ? v[i] : 0.f;
                    }
                }
                // ---- this wavefront's rows of A: myA[row][k] = A_g[r0 + row][k0 + k]
                {
                    float v[16];
                    if (!t1) {
                        // lane = k, one row per step
                        const int k = k0 + lane, kc_ = min(k, K - 1);
#pragma unroll
                        for (int r = 0; r < kStripRows; ++r) v[r] = as[(int64_t)min(r0 + r, M - 1) * K + kc_];
#pragma unroll
                        for (int r = 0; r < kStripRows; ++r)
                            myA[r * kF32PitchA + lane] = (r0 + r < M && k < K) ? v[r] : 0.f;
                    } else {
                        // stored K x M: contiguous in the row index; lane = (k quarter, row)
                        const int r = lane & 15, kq = lane >> 4, rc = min(r0 + r, M - 1);
#pragma unroll
                        for (int i = 0; i < 16; ++i) v[i] = as[(int64_t)min(k0 + kq * 16 + i, K - 1) * M + rc];
#pragma unroll
                        for (int i = 0; i < 16; ++i)
                            myA[r * kF32PitchA + kq * 16 + i] = (r0 + r < M && k0 + kq * 16 + i < K) ? v[i] : 0.f;
                    }
                }
                __syncthreads();
                // ---- 64 k on the matrix unit, four k per instruction (v_mfma_f32_16x16x4_f32):
                //      operand lane (i = lane%16, q = lane/16) supplies row / column i at k + q
                const float *arow = myA + (lane & 15) * kF32PitchA + (lane >> 4);
                const float *bcol = sB + (lane & 15) * kF32PitchB + (lane >> 4);
#pragma unroll 4
                for (int k4 = 0; k4 < kF32K; k4 += 4) {
                    const float av = arow[k4];
#pragma unroll
                    for (int t = 0; t < kF32Cols / 16; ++t)
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bcol[t * 16 * kF32PitchB + k4], acc[t], 0, 0, 0);
                }
            }
            const int j = lane & 15, q = lane >> 4;
#pragma unroll
            for (int t = 0; t < kF32Cols / 16; ++t) {
                const int col = c0 + 16 * t + j;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = r0 + 4 * q + e;
                    if (col < N && row < M) os[(int64_t)row * N + col] = acc[t][e];
                }
            }
        }
    }
}

int launch_gemm_f32(const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    int64_t z = 4;
    if (info) {
        nseg = info->nseg;
        const int64_t rounds = (std::max<int64_t>(info->max_M, 1) + kF32Rows - 1) / kF32Rows;
        const int64_t want = ((int64_t)device_cu_count() * 8 + nseg * args.H - 1) / std::max<int64_t>(1, nseg * args.H);
        z = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(rounds, want), 64));
    }
    if (nseg <= 0) return BA_OK;
    RunArgs run = args;
    const bool head_fast = nseg <= 65535;               // segments then ride on gridDim.y
    if (head_fast) run.flags |= kFlagHeadFast;
    hipLaunchKernelGGL(gemm_f32_kernel,
                       head_fast ? dim3((unsigned)args.H, (unsigned)nseg, (unsigned)z) : dim3((unsigned)nseg, (unsigned)args.H, (unsigned)z),
                       dim3(kF32Threads), 0, stream, run);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
