// Varlen GEMM for the element types without a kernel of their own (the reference's generic kernel,
// csrc/cuda/spBlkGEMM.cu:120-271, instantiated by AT_DISPATCH_ALL_TYPES at :1010): fp32 and fp64 on the matrix
// instructions of their type (v_mfma_f32_16x16x4_f32, v_mfma_f64_16x16x4_f64: products and sums in the element
// type), the integer types with plain multiply-adds.  Like the reference, the accumulator has the element type:
// integers wrap modulo 2^bits, which is what unsigned arithmetic at 32 or 64 bits followed by a truncating store
// yields bit for bit.  Any shape, offset and layout (transpose flags); fp16/bf16 have their own kernels.
//
// Workgroup = 64 rows x 64 columns of one segment and head at a time, k in chunks of 64 (32 for the 8-byte
// types).  A chunk of B_g (64 columns x chunk) is staged in LDS by the whole workgroup with coalesced loads along
// the operand's contiguous dimension, stored [column][k] with an odd pitch; each wavefront stages its own 16 rows
// of A_g [row][k].  A wavefront computes 16 rows x 64 columns as four 16 x 16 tiles: per four k it reads one A
// word and four B words per lane from LDS and issues four matrix instructions; the integer types read four A and
// four B words per k and lane and issue sixteen multiply-adds.
#include <algorithm>

#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kGenThreads = 256;
constexpr int kGenWaves = kGenThreads / 64;
constexpr int kGenCols = 64;                         // columns per block = lanes
constexpr int kGenRows = kStripRows * kGenWaves;     // rows per workgroup round

// Element type T -> type S the operands are staged and accumulated in, chunk length, and where a lane's four
// results of a 16 x 16 tile lie: lane (j = lane%16, q = lane/16) holds column j of rows 4q + e (fp32 matrix
// instruction, and the layout the multiply-add path uses) or of rows 4e + q (fp64 matrix instruction).
template <typename T> struct Gen {
    typedef uint32_t S;
    static constexpr int kChunk = 64;
    static constexpr bool kMatrix = false, kRowsStrided = false;
};
template <> struct Gen<int64_t> {
    typedef uint64_t S;
    static constexpr int kChunk = 32;
    static constexpr bool kMatrix = false, kRowsStrided = false;
};
template <> struct Gen<float> {
    typedef float S;
    static constexpr int kChunk = 64;
    static constexpr bool kMatrix = true, kRowsStrided = false;
};
template <> struct Gen<double> {
    typedef double S;
    static constexpr int kChunk = 32;
    static constexpr bool kMatrix = true, kRowsStrided = true;
};

typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef double f64x4v __attribute__((ext_vector_type(4)));

// grid (head, segment, z) with kFlagHeadFast (consecutive workgroups, which go to the dies in turn, are the heads
// of one segment), else (segment, head, z): workgroup z takes the 64-row rounds z, z + gridDim.z, ... of its segment.
template <typename T>
__global__ __launch_bounds__(kGenThreads) void gemm_generic_kernel(RunArgs a) {
    typedef typename Gen<T>::S S;
    constexpr int kChunk = Gen<T>::kChunk;
    constexpr int kPitchB = kChunk + 1;              // odd: lanes (columns) fall on consecutive banks
    constexpr int kPitchA = kChunk + 4;              // staggered banks
    __shared__ S sB[kGenCols * kPitchB];
    __shared__ __attribute__((aligned(16))) S sA[kGenWaves][kStripRows * kPitchA];
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
    const T *as = reinterpret_cast<const T *>(a.A) + h * a.Dm1 + rec.off1;
    const T *bs = reinterpret_cast<const T *>(a.B) + h * a.Dm2 + rec.off2;
    T *os = reinterpret_cast<T *>(a.out) + h * a.Dout + rec.offO;
    S *myA = sA[wave];
    const int nkc = (K + kChunk - 1) / kChunk;
    constexpr int kPer = kChunk / 4;                 // elements of B (of A) a thread (a lane) stages per chunk
    const S zero = S(0);

    for (int round = blockIdx.z; round * kGenRows < M; round += gridDim.z) {
        const int r0 = round * kGenRows + wave * kStripRows;          // this wavefront's 16 rows
        for (int c0 = 0; c0 < N; c0 += kGenCols) {
            // four 16 x 16 tiles per wavefront, four results per lane and tile (layout: see Gen)
            S acc[kGenCols / 16][4];
#pragma unroll
            for (int t = 0; t < kGenCols / 16; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[t][e] = zero;
            for (int kc = 0; kc < nkc; ++kc) {                         // K = 0: no chunk, the result is zeros
                const int k0 = kc * kChunk;
                __syncthreads();                                       // the previous chunk is consumed
                // Staging: every load is unconditional (index clamped into the segment, value zeroed
                // afterwards where it lies outside), so the loads of a thread are in flight together.
                // ---- B chunk: sB[col][k] = B_g[c0 + col][k0 + k], zero outside the segment
                {
                    T v[kPer];
                    if (!t2) {
                        // rows of B_g are contiguous in k: consecutive threads take consecutive k
                        const int kk = tid % kChunk, k = k0 + kk, cq = (tid / kChunk) * kPer;
                        const int kc_ = min(k, K - 1);
#pragma unroll
                        for (int i = 0; i < kPer; ++i) v[i] = bs[(int64_t)min(c0 + cq + i, N - 1) * K + kc_];
#pragma unroll
                        for (int i = 0; i < kPer; ++i)
                            sB[(cq + i) * kPitchB + kk] = (c0 + cq + i < N && k < K) ? (S)v[i] : zero;
                    } else {
                        // stored K x N: contiguous in the column
                        const int col = tid & 63, kq = (tid >> 6) * kPer;
                        const int cc = min(c0 + col, N - 1);
#pragma unroll
                        for (int i = 0; i < kPer; ++i) v[i] = bs[(int64_t)min(k0 + kq + i, K - 1) * N + cc];
#pragma unroll
                        for (int i = 0; i < kPer; ++i)
                            sB[col * kPitchB + kq + i] = (c0 + col < N && k0 + kq + i < K) ? (S)v[i] : zero;
                    }
                }
                // ---- this wavefront's rows of A: myA[row][k] = A_g[r0 + row][k0 + k]
                {
                    T v[kPer];
                    if (!t1) {
                        const int kk = lane % kChunk, k = k0 + kk, rq = (lane / kChunk) * kPer, kc_ = min(k, K - 1);
#pragma unroll
                        for (int r = 0; r < kPer; ++r) v[r] = as[(int64_t)min(r0 + rq + r, M - 1) * K + kc_];
#pragma unroll
                        for (int r = 0; r < kPer; ++r)
                            myA[(rq + r) * kPitchA + kk] = (r0 + rq + r < M && k < K) ? (S)v[r] : zero;
                    } else {
                        // stored K x M: contiguous in the row index; lane = (k quarter, row)
                        const int r = lane & 15, kq = (lane >> 4) * kPer, rc = min(r0 + r, M - 1);
#pragma unroll
                        for (int i = 0; i < kPer; ++i) v[i] = as[(int64_t)min(k0 + kq + i, K - 1) * M + rc];
#pragma unroll
                        for (int i = 0; i < kPer; ++i)
                            myA[r * kPitchA + kq + i] = (r0 + r < M && k0 + kq + i < K) ? (S)v[i] : zero;
                    }
                }
                __syncthreads();
                if constexpr (Gen<T>::kMatrix) {
                    // ---- the chunk on the matrix unit, four k per instruction: operand lane
                    //      (i = lane%16, q = lane/16) supplies row / column i at k + q
                    const S *arow = myA + (lane & 15) * kPitchA + (lane >> 4);
                    const S *bcol = sB + (lane & 15) * kPitchB + (lane >> 4);
#pragma unroll 4
                    for (int k4 = 0; k4 < kChunk; k4 += 4) {
                        const S av = arow[k4];
#pragma unroll
                        for (int t = 0; t < kGenCols / 16; ++t) {
                            const S bv = bcol[t * 16 * kPitchB + k4];
                            if constexpr (sizeof(S) == 4) {
                                f32x4v c = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
                                c = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, c, 0, 0, 0);
                                acc[t][0] = c[0]; acc[t][1] = c[1]; acc[t][2] = c[2]; acc[t][3] = c[3];
                            } else {
                                f64x4v c = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
                                c = __builtin_amdgcn_mfma_f64_16x16x4f64(av, bv, c, 0, 0, 0);
                                acc[t][0] = c[0]; acc[t][1] = c[1]; acc[t][2] = c[2]; acc[t][3] = c[3];
                            }
                        }
                    }
                } else {
                    // ---- multiply-adds: lane (j, q) owns rows 4q..4q+3 of columns j, 16 + j, 32 + j, 48 + j
                    const S *arow = myA + (4 * (lane >> 4)) * kPitchA;
                    const S *bcol = sB + (lane & 15) * kPitchB;
#pragma unroll 4
                    for (int k = 0; k < kChunk; ++k) {
                        S av[4], bv[kGenCols / 16];
#pragma unroll
                        for (int e = 0; e < 4; ++e) av[e] = arow[e * kPitchA + k];
#pragma unroll
                        for (int t = 0; t < kGenCols / 16; ++t) bv[t] = bcol[t * 16 * kPitchB + k];
#pragma unroll
                        for (int t = 0; t < kGenCols / 16; ++t)
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[t][e] += av[e] * bv[t];
                    }
                }
            }
            const int j = lane & 15, q = lane >> 4;
#pragma unroll
            for (int t = 0; t < kGenCols / 16; ++t) {
                const int col = c0 + 16 * t + j;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = r0 + (Gen<T>::kRowsStrided ? 4 * e + q : 4 * q + e);
                    if (col < N && row < M) os[(int64_t)row * N + col] = (T)acc[t][e];
                }
            }
        }
    }
}

template <typename T>
static void launch_generic_t(const RunArgs &run, dim3 grid, hipStream_t stream) {
    hipLaunchKernelGGL(gemm_generic_kernel<T>, grid, dim3(kGenThreads), 0, stream, run);
}

int launch_gemm_generic(int dtype, const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    int64_t z = 4;
    if (info) {
        nseg = info->nseg;
        const int64_t rounds = (std::max<int64_t>(info->max_M, 1) + kGenRows - 1) / kGenRows;
        const int64_t want = ((int64_t)device_cu_count() * 8 + nseg * args.H - 1) / std::max<int64_t>(1, nseg * args.H);
        z = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(rounds, want), 64));
    }
    if (nseg <= 0) return BA_OK;
    RunArgs run = args;
    const bool head_fast = nseg <= 65535;               // segments then ride on gridDim.y
    if (head_fast) run.flags |= kFlagHeadFast;
    const dim3 grid = head_fast ? dim3((unsigned)args.H, (unsigned)nseg, (unsigned)z)
                                : dim3((unsigned)nseg, (unsigned)args.H, (unsigned)z);
    switch (dtype) {
        case BA_F32: launch_generic_t<float>(run, grid, stream); break;
        case BA_F64: launch_generic_t<double>(run, grid, stream); break;
        case BA_U8: launch_generic_t<uint8_t>(run, grid, stream); break;
        case BA_I8: launch_generic_t<int8_t>(run, grid, stream); break;
        case BA_I16: launch_generic_t<int16_t>(run, grid, stream); break;
        case BA_I32: launch_generic_t<int32_t>(run, grid, stream); break;
        case BA_I64: launch_generic_t<int64_t>(run, grid, stream); break;
        default: return BA_ERR_UNSUPPORTED;
    }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
