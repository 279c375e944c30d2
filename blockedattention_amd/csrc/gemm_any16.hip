// fp16 / bf16 varlen GEMM on the matrix instruction for the calls the strip and tile kernels do not take: operands
// stored K x M or K x N (the reference's transpose flags, csrc/cuda/spBlkGEMM.cu:311-329, 382-400), reduction
// lengths that are not multiples of 8, segments that start at odd elements, base pointers without 16-byte
// alignment.  The backward of the product is two such calls (csrc/sparseBlockedAttention.cpp:52-72: dA = dS B
// reduces over N, dB = dS^T A over M, with dS and the saved operands read as they lie).
//
// Workgroup = 64 rows x 64 columns of one segment and head at a time, k in chunks of 64.  Both operand chunks go
// through LDS with a row pitch of 160 bytes.  Staging reads 16 bytes per lane along whatever dimension is contiguous
// in memory, at any 2-byte alignment, through a buffer descriptor that spans exactly the segment (rows past its
// end read as zeros), and writes them to LDS as they come: an operand that is not transposed lies there as
// [row][k] and is read 16 bytes per lane; an operand stored k-major lies there k-major and the matrix operand is
// gathered by the transposing LDS read (ds_read_b64_tr_b16, four k of one row per lane).  Each wavefront
// then computes 16 rows x 64 columns as four 16 x 16 tiles with v_mfma_f32_16x16x32 (fp32 sums).  Column slot n of
// tile t is column 4 n + t, so a lane owns four consecutive columns of each of its rows and the sixteen lanes of a
// row group write 128 contiguous bytes.
#include <algorithm>

#include "ba_gemm_common.hpp"

namespace ba {

constexpr int kAnyThreads = 256;
constexpr int kAnyWaves = kAnyThreads / 64;
constexpr int kAnyTile = 64;                         // rows and columns per workgroup step, k per chunk
constexpr int kAnyPitch = (kAnyTile + 16) * 2;       // bytes per LDS row: 160 = 16 * (2 * odd), the pitch at which the
// 16-byte operand reads (served 32 lanes, 512 bytes at a time) and the transposing 8-byte reads meet no bank conflict

// Sixteen consecutive elements of the segment from byte offset `off` on (kNoLine: zeros).  Two 16-byte loads where
// they lie inside the segment; a piece that reaches past its end is fetched element by element, the hardware
// returning zero for those outside (a wide load that crosses the end of the descriptor's range is dropped whole).
constexpr uint32_t kNoLine = 0x80000000u;
union Line16 {
    u32x4 v[2];
    uint16_t e[16];
};
__device__ __forceinline__ Line16 load_line16(__amdgpu_buffer_rsrc_t res, uint32_t off, uint32_t bytes) {
    Line16 x;
    if (off == kNoLine) {
        x.v[0] = x.v[1] = u32x4{0u, 0u, 0u, 0u};
    } else if (off + 32u <= bytes) {
        x.v[0] = __builtin_amdgcn_raw_buffer_load_b128(res, off, 0, 0);
        x.v[1] = __builtin_amdgcn_raw_buffer_load_b128(res, off + 16u, 0, 0);
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) x.e[i] = __builtin_amdgcn_raw_buffer_load_b16(res, off + 2u * i, 0, 0);
    }
    return x;
}

// One 64 x 64 chunk of an operand on its way into LDS as dst[row][k], in two steps so that the loads of the next
// chunk can be in flight while the matrix instructions work on the current one.  The operand is `rows` x K (or,
// transposed, stored K x rows); the chunk starts at row r0, reduction index k0.  Thread t takes sixteen
// consecutive elements along the contiguous dimension of line t / 4.
__device__ __forceinline__ Line16 fetch_chunk16(__amdgpu_buffer_rsrc_t res, bool transposed, int rows, int K, int r0, int k0,
                                                int tid) {
    const int line = tid >> 2, part = (tid & 3) * 16;
    const uint32_t bytes = (uint32_t)(rows * K) * 2u;
    // not transposed: line = row, the sixteen elements run along k; transposed: line = k, they run along the rows
    const int row = r0 + (transposed ? part : line), k = k0 + (transposed ? line : part);
    const int lead = transposed ? k * rows + row : row * K + k;
    return load_line16(res, row < rows && k < K ? (uint32_t)lead * 2u : kNoLine, bytes);
}
// Into LDS.  An operand that is not transposed lies as dst[row][k].  A transposed one stays k-major, dst[k][..], and
// the matrix operand is gathered by transposing reads (lds_tr8 below): 16-byte writes here instead of sixteen 2-byte
// ones.  X (rows of the output) keeps its rows in order.  Y (columns of the output) permutes each group of sixteen
// columns, 16 a + 4 b + t -> position 16 t + 4 a + b, so that the lane that reads position 16 t + i of a row gets
// column 4 i + t: the columns a lane stores side by side (see the kernel).
template <bool PERMUTE>
__device__ __forceinline__ void put_chunk16(Line16 x, bool transposed, int rows, int K, int r0, int k0, unsigned char *dst,
                                            int tid) {
    const int line = tid >> 2, part = (tid & 3) * 16;
    const int valid = transposed ? rows - (r0 + part) : K - (k0 + part);   // elements of the line from here on
#pragma unroll
    for (int i = 0; i < 16; ++i) x.e[i] = i < valid ? x.e[i] : (uint16_t)0;
    if (!PERMUTE || !transposed) {
        u32x4 *d = reinterpret_cast<u32x4 *>(dst + line * kAnyPitch + part * 2);
        d[0] = x.v[0];
        d[1] = x.v[1];
    } else {
        const uint32_t *w = reinterpret_cast<const uint32_t *>(&x);
#pragma unroll
        for (int t = 0; t < 4; ++t) {                 // elements t, 4 + t, 8 + t, 12 + t of the thread's sixteen
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            const uint32_t lo = __builtin_amdgcn_perm(w[2 + (t >> 1)], w[t >> 1], sel);
            const uint32_t hi = __builtin_amdgcn_perm(w[6 + (t >> 1)], w[4 + (t >> 1)], sel);
            *reinterpret_cast<u32x2 *>(dst + line * kAnyPitch + 32 * t + (part >> 2) * 2) = u32x2{lo, hi};
        }
    }
}
// Eight k of one row (column) of a k-major chunk as matrix operand: two transposing reads of four k each.  In a
// group of sixteen lanes, lane 4 e + a points at positions 4 a .. 4 a + 3 of k row e, and lane i receives position
// i of the four k rows; p is this lane's address for the first four k, the next four lie four rows on.
__device__ __forceinline__ u32x4 lds_tr8(const unsigned char *p) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 *LdsPtr;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(uintptr_t)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(uintptr_t)(p + 4 * kAnyPitch));
    const u32x2 l = __builtin_bit_cast(u32x2, lo), h = __builtin_bit_cast(u32x2, hi);
    return u32x4{l[0], l[1], h[0], h[1]};
}

template <int DT>
__global__ __launch_bounds__(kAnyThreads) void gemm_any16_kernel(RunArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char sX[kAnyTile * kAnyPitch];
    __shared__ __attribute__((aligned(16))) unsigned char sY[kAnyTile * kAnyPitch];
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const int nseg = hdr->nseg;
    const int64_t per_head = hdr->att_blocks64;       // 64-row rounds per head (= the row-block prefix's last entry)
    if (!header_ok(a)) {
        report_mismatch(a);
        return;
    }
    // Two grids.  With the batch's totals on the host (ride_slots = 1): one workgroup per existing
    // (segment, 64-row round, head), head fastest, found by a search in the plan's row-block prefix.  Without:
    // (head, segment, z) or (segment, head, z), workgroup z taking the rounds z, z + gridDim.z, ...
    const bool head_fast = a.flags & kFlagHeadFast;
    // (a step past any segment's round count, small enough that first_round + step cannot overflow)
    constexpr int rounds_never_again = 1 << 26;
    int g, first_round, round_step;
    int64_t h;
    if (a.ride_slots) {
        const int32_t *pfx = plan_rowblocks(a.plan, nseg, 0);
        const int64_t u = blockIdx.x;
        if (u >= per_head * a.H) return;
        h = u % a.H;                                   // consecutive workgroups: the heads of one round, one shape
        const int item = (int)(u / a.H);
        g = prefix_search(pfx, nseg, item);
        first_round = item - ((ConstI32)(uintptr_t)pfx)[g];
        round_step = rounds_never_again;
    } else {
        g = head_fast ? blockIdx.y : blockIdx.x;
        h = head_fast ? blockIdx.x : blockIdx.y;
        first_round = blockIdx.z;
        round_step = gridDim.z;
    }
    if (g >= nseg) return;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int M = rec.M, N = rec.N, K = rec.K;
    if (M < 1 || N < 1) return;
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = lane_id(), n = lane & 15, q = lane >> 4;
    const bool t1 = a.flags & kFlagTranspose1, t2 = a.flags & kFlagTranspose2;
    const __amdgpu_buffer_rsrc_t resX = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(reinterpret_cast<const uint16_t *>(a.A) + h * a.Dm1 + rec.off1), 0, M * K * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t resY = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(reinterpret_cast<const uint16_t *>(a.B) + h * a.Dm2 + rec.off2), 0, N * K * 2, kRsrcFlags);
    uint16_t *os = reinterpret_cast<uint16_t *>(a.out) + h * a.Dout + rec.offO;
    const int nkc = (K + kAnyTile - 1) / kAnyTile;
    // operand addresses of this lane inside a chunk: A operand = row 16 wave + n of X, B operand of tile t =
    // row 4 n + t of Y (column slot n of tile t is column 4 n + t), eight k from 8 q on
    const unsigned char *xa = sX + (16 * wave + n) * kAnyPitch + q * 16;
    const unsigned char *ya = sY + (4 * n) * kAnyPitch + q * 16;
    // the same from k-major chunks (transposed operands): k row 8 q + n / 4 of the step, positions 4 (n % 4) .. of the
    // wavefront's sixteen rows (X) or of tile t's sixteen positions (Y, + 32 t bytes)
    const unsigned char *xt = sX + (8 * q + (n >> 2)) * kAnyPitch + (16 * wave + 4 * (n & 3)) * 2;
    const unsigned char *yt = sY + (8 * q + (n >> 2)) * kAnyPitch + (4 * (n & 3)) * 2;

    // lane (n, q): rows 16 wave + 4 q + i, columns 64 cb + 4 n .. + 3; clears the accumulators for the next block
    auto store_block = [&](int cb, int r0, f32x4 (&acc)[4]) {
        const int col = cb * kAnyTile + 4 * n;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = r0 + 16 * wave + 4 * q + i;
            if (row < M && col < N) {
                uint16_t *p = os + (int64_t)row * N + col;
                if (col + 4 <= N) {
                    *reinterpret_cast<u32x2_unaligned *>(p) =
                        u32x2{Elem<DT>::pack2(acc[0][i], acc[1][i]), Elem<DT>::pack2(acc[2][i], acc[3][i])};
                } else {
#pragma unroll
                    for (int t = 0; t < 3; ++t)
                        if (col + t < N) p[t] = Elem<DT>::from_float(acc[t][i]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    const int rounds = (M + kAnyTile - 1) / kAnyTile;
    const int ncb = (N + kAnyTile - 1) / kAnyTile;
    const int steps = ncb * nkc;                     // (column block, chunk) pairs of one round, chunk fastest
    for (int round = first_round; round < rounds; round += round_step) {
        const int r0 = round * kAnyTile;
        f32x4 acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        Line16 nx, ny;
        if (steps > 0) {
            nx = fetch_chunk16(resX, t1, M, K, r0, 0, tid);
            ny = fetch_chunk16(resY, t2, N, K, 0, 0, tid);
        }
        int cb = 0, kc = 0;
        for (int step = 0; step < steps; ++step) {
            __syncthreads();                                           // the previous chunk is consumed
            put_chunk16<false>(nx, t1, M, K, r0, kc * kAnyTile, sX, tid);
            put_chunk16<true>(ny, t2, N, K, cb * kAnyTile, kc * kAnyTile, sY, tid);
            int cb2 = cb, kc2 = kc + 1;
            if (kc2 == nkc) { kc2 = 0; ++cb2; }
            if (step + 1 < steps) {                                    // in flight under the matrix instructions
                nx = fetch_chunk16(resX, t1, M, K, r0, kc2 * kAnyTile, tid);
                ny = fetch_chunk16(resY, t2, N, K, cb2 * kAnyTile, kc2 * kAnyTile, tid);
            }
            __syncthreads();
#pragma unroll
            for (int ks = 0; ks < kAnyTile / 32; ++ks) {
                const u32x4 av = t1 ? lds_tr8(xt + ks * 32 * kAnyPitch) : *reinterpret_cast<const u32x4 *>(xa + ks * 64);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const u32x4 bv = t2 ? lds_tr8(yt + ks * 32 * kAnyPitch + 32 * t)
                                        : *reinterpret_cast<const u32x4 *>(ya + t * kAnyPitch + ks * 64);
                    acc[t] = Elem<DT>::mfma(av, bv, acc[t]);
                }
            }
            if (kc == nkc - 1) store_block(cb, r0, acc);
            cb = cb2; kc = kc2;
        }
        if (nkc == 0)                                                  // K = 0: the result is zeros
            for (int c = 0; c < ncb; ++c) store_block(c, r0, acc);
    }
}

int launch_gemm_any16(int dtype, const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (info) nseg = info->nseg;
    if (nseg <= 0) return BA_OK;
    RunArgs run = args;
    dim3 grid;
    const int64_t items = info ? (int64_t)info->att_blocks64 * args.H : 0;
    if (info && items < (int64_t(1) << 31)) {
        if (items == 0) return BA_OK;                   // no segment has rows
        run.ride_slots = 1;
        grid = dim3((unsigned)items);
    } else {
        const bool head_fast = nseg <= 65535;           // segments then ride on gridDim.y
        if (head_fast) run.flags |= kFlagHeadFast;
        grid = head_fast ? dim3((unsigned)args.H, (unsigned)nseg, 4u) : dim3((unsigned)nseg, (unsigned)args.H, 4u);
    }
    if (dtype == BA_F16) hipLaunchKernelGGL(gemm_any16_kernel<0>, grid, dim3(kAnyThreads), 0, stream, run);
    else hipLaunchKernelGGL(gemm_any16_kernel<1>, grid, dim3(kAnyThreads), 0, stream, run);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
