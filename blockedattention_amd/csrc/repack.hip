// Repack of one operand of every segment into the layout the MFMA kernels read:
// row-major rows x K with K a multiple of 8 (16-byte rows), zero padded, optionally
// transposed on the way.  It is what turns the GEMMs of the backward pass
// (dA = dS B reduces over N, dB = dS^T A over M: csrc/sparseBlockedAttention.cpp:52-72
// runs them through its generic kernel with the transpose flags), transposed
// forward layouts and reduction lengths that are not multiples of 8 into inputs of
// the fast path; without it those cases take the element-wise kernel.
//
// Per segment g and head: the destination matrix L_g is operand `dst_which` of the
// destination plan (R x C, row-major, at that plan's offset).  Its source is
// operand `src_which` of the source plan, seen as an R_s x C_s matrix with
// (R_s, C_s) = that operand's dimensions, swapped when `swap_dims` is set, and
// stored row-major or, with `column_major`, column-major.  L_g[r][c] = source[r][c]
// inside the source's range, 0 outside.
//
// Row-major source: a straight copy, eight elements per lane (unaligned 16-byte
// loads, aligned 16-byte stores).  Column-major source: 64 x 64 tiles through LDS;
// the lanes read runs of eight along the source's contiguous dimension and write
// runs of eight along the destination's.
#include <algorithm>

#include "ba_device.hpp"
#include "ba_gemm_common.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kRepackThreads = 256;
constexpr int kRepackTile = 64;
constexpr int kRepackPitch = kRepackTile + 8;      // LDS row pitch in elements: rows stay 16-byte aligned

struct RepackArgs {
    const void *src_plan;
    const void *dst_plan;
    const uint16_t *src;
    uint16_t *dst;
    int64_t Dsrc, Ddst;       // elements per head
    int nseg;
    int src_which, dst_which; // 0: A (M x K), 1: B (N x K), 2: out (M x N)
    int swap_dims, column_major;
    int head_fast;            // grid (head, segment, z): consecutive workgroups are the heads of one segment
};

__device__ __forceinline__ void operand_of(const SegRec &r, int which, int &rows, int &cols, int64_t &off) {
    rows = which == 1 ? r.N : r.M;
    cols = which == 2 ? r.N : r.K;
    off = which == 0 ? r.off1 : which == 1 ? r.off2 : r.offO;
}

__global__ __launch_bounds__(kRepackThreads) void repack_kernel(RepackArgs a) {
    __shared__ __attribute__((aligned(16))) uint16_t tile[kRepackTile * kRepackPitch];
    const ConstHdr hs = (ConstHdr)(uintptr_t)a.src_plan, hd = (ConstHdr)(uintptr_t)a.dst_plan;
    const bool ok = (hs->magic == kPlanMagic) & (hd->magic == kPlanMagic) & (hs->nseg == a.nseg) & (hd->nseg == a.nseg) &
                    (hs->bad_segments == 0) & (hd->bad_segments == 0);
    if (!ok) {
        if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(const_cast<void *>(a.dst_plan))->run_errors, 1);
        return;
    }
    const int g = a.head_fast ? blockIdx.y : blockIdx.x;
    if (g >= a.nseg) return;
    const SegRec rs = load_rec(plan_ro(const_cast<void *>(a.src_plan), a.nseg).recs, g);
    const SegRec rd = load_rec(plan_ro(const_cast<void *>(a.dst_plan), a.nseg).recs, g);
    int R, C, Rs, Cs;
    int64_t offd, offs;
    operand_of(rd, a.dst_which, R, C, offd);
    operand_of(rs, a.src_which, Rs, Cs, offs);
    if (a.swap_dims) { const int t = Rs; Rs = Cs; Cs = t; }
    if (R < 1 || C < 1) return;
    const int64_t h = a.head_fast ? blockIdx.x : blockIdx.y;
    const uint16_t *src = a.src + h * a.Dsrc + offs;
    uint16_t *dst = a.dst + h * a.Ddst + offd;
    const int tid = threadIdx.x;
    const bool vec_dst = ((C | (int)(offd & 7) | (int)((h * a.Ddst) & 7)) & 7) == 0 && (((uintptr_t)a.dst) & 15) == 0;

    // one run of eight destination elements (row r, columns c .. c+7)
    auto put = [&](int r, int c, const uint16_t (&v)[8]) {
        uint16_t *p = dst + (int64_t)r * C + c;
        if (vec_dst && c + 8 <= C) {
            *reinterpret_cast<u32x4 *>(p) = u32x4{v[0] | ((uint32_t)v[1] << 16), v[2] | ((uint32_t)v[3] << 16),
                                                  v[4] | ((uint32_t)v[5] << 16), v[6] | ((uint32_t)v[7] << 16)};
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (c + i < C) p[i] = v[i];
        }
    };

    if (!a.column_major) {
        // runs of eight along a row, one run per thread and step
        const int runs = (C + 7) >> 3;
        const int64_t total = (int64_t)R * runs;
        for (int64_t i = (int64_t)blockIdx.z * kRepackThreads + tid; i < total; i += (int64_t)gridDim.z * kRepackThreads) {
            const int r = (int)(i / runs), c = (int)(i % runs) * 8;
            uint16_t v[8];
            const uint16_t *p = src + (int64_t)r * Cs + c;
            if (r < Rs && c + 8 <= Cs) {
                const u32x4 w = *reinterpret_cast<const u32x4_unaligned *>(p);
#pragma unroll
                for (int k = 0; k < 4; ++k) { v[2 * k] = (uint16_t)w[k]; v[2 * k + 1] = (uint16_t)(w[k] >> 16); }
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) v[k] = (r < Rs && c + k < Cs) ? p[k] : (uint16_t)0;
            }
            put(r, c, v);
        }
        return;
    }

    // Column-major source: element (r, c) sits at c * Rs + r.  Tile = 64 destination rows x 64 columns.
    const int tr = (R + kRepackTile - 1) / kRepackTile, tc = (C + kRepackTile - 1) / kRepackTile;
    for (int t = blockIdx.z; t < tr * tc; t += gridDim.z) {
        const int r0 = (t / tc) * kRepackTile, c0 = (t % tc) * kRepackTile;
        if (t != (int)blockIdx.z) __syncthreads();               // the tile buffer is reused
        // read: thread -> (source column c, run of eight rows r): 8 threads per column, 32 columns per pass
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int cl = pass * 32 + (tid >> 3), rl = (tid & 7) * 8;
            const int c = c0 + cl, r = r0 + rl;
            uint16_t v[8];
            const uint16_t *p = src + (int64_t)c * Rs + r;
            if (c < Cs && r + 8 <= Rs) {
                const u32x4 w = *reinterpret_cast<const u32x4_unaligned *>(p);
#pragma unroll
                for (int k = 0; k < 4; ++k) { v[2 * k] = (uint16_t)w[k]; v[2 * k + 1] = (uint16_t)(w[k] >> 16); }
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) v[k] = (c < Cs && r + k < Rs) ? p[k] : (uint16_t)0;
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) tile[(rl + k) * kRepackPitch + cl] = v[k];
        }
        __syncthreads();
        // write: thread -> (destination row r, run of eight columns c)
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int rl = pass * 32 + (tid >> 3), cl = (tid & 7) * 8;
            const int r = r0 + rl, c = c0 + cl;
            if (r < R && c < C) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(&tile[rl * kRepackPitch + cl]);
                uint16_t v[8];
#pragma unroll
                for (int k = 0; k < 4; ++k) { v[2 * k] = (uint16_t)w[k]; v[2 * k + 1] = (uint16_t)(w[k] >> 16); }
                put(r, c, v);
            }
        }
    }
}

int launch_repack(const void *src_plan, int src_which, int swap_dims, int column_major, const void *dst_plan,
                  int dst_which, int64_t nseg, const void *src, void *dst, int64_t H, int64_t Dsrc, int64_t Ddst,
                  const ba_plan_info *dst_info, hipStream_t stream) {
    if (H > 65535) return BA_ERR_UNSUPPORTED;              // heads ride on gridDim.y
    if (nseg <= 0 || H <= 0) return BA_OK;
    // z: tiles (or 2048-element slices) of the largest destination operand, bounded
    int64_t z = 8;
    if (dst_info) {
        const int64_t rows = dst_which == 1 ? dst_info->max_N : dst_info->max_M;
        const int64_t cols = dst_info->max_K;
        const int64_t units = column_major ? ((rows + 63) / 64) * ((cols + 63) / 64) : (rows * ((cols + 7) / 8) + 255) / 256;
        const int64_t want = ((int64_t)device_cu_count() * 8 + nseg * H - 1) / (nseg * H);
        // enough workgroups to fill the machine, and never more than eight tiles of the largest segment in
        // one workgroup (workgroups past a segment's last tile leave at once)
        z = std::max<int64_t>(std::min<int64_t>(units, want), std::min<int64_t>((units + 7) / 8, 64));
        z = std::max<int64_t>(1, std::min<int64_t>(z, 1024));
    }
    RepackArgs a{src_plan, dst_plan, (const uint16_t *)src, (uint16_t *)dst, Dsrc, Ddst, (int)nseg,
                 src_which, dst_which, swap_dims, column_major, nseg <= 65535 ? 1 : 0};
    hipLaunchKernelGGL(repack_kernel,
                       a.head_fast ? dim3((unsigned)H, (unsigned)nseg, (unsigned)z) : dim3((unsigned)nseg, (unsigned)H, (unsigned)z),
                       dim3(kRepackThreads), 0, stream, a);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
