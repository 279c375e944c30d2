// Varlen GEMM (S_g = A_g B_g^T) and the fused GEMM + row softmax for fp16/bf16
// on gfx950: MFMA 16x16x32 with fp32 accumulation, scores kept in registers.
//
// Work decomposition (all counts come scanned from the plan):
//   pack item   one wavefront, several tiny segments sharing one 16x16 MFMA tile
//   strip item  one wavefront, 16 rows x all N <= 256 columns of one segment
//   gemm item   one wavefront, 16 rows x one 256-column chunk (GEMM only, any N)
//   split item  one 16-wave workgroup, 16 rows x all 256 < N <= 4096 columns
//   wide item   one workgroup, 16 rows x N > 4096 columns in two sweeps
//
// The MFMA is issued "transposed": the B_g rows go in as the first operand and
// the A_g rows as the second, so that a lane ends up with four CONSECUTIVE
// columns of ONE score row (row = lane%16, columns 4*(lane/16)+i of each
// 16-wide tile).  Row maxima and sums are then in-lane loops plus two
// cross-lane steps, and stores are 8-byte runs along the row.
//
// Both operands are K-contiguous (A_g is M x K, B_g is N x K), so a lane's
// eight k-values are one 16-byte global load straight into the MFMA operand
// registers; no transposition is ever needed.  Segments that break the
// alignment this needs (K % 8 != 0, odd segment starts, transposed layouts)
// take an element-wise loader into the same MFMA code.
#include <algorithm>

#include "ba_device.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kGroupThreads = 64 * kWavesPerGroup;
constexpr int kMaxTiles = kWaveCols / 16;  // 16 MFMA tiles per wavefront

struct Seg {
    int M, N, K;
    int64_t a, b, o;  // element offsets of the segment inside A, B, out (head included)
};

// Buffer resources of one segment.  Every operand load and result store goes
// through a raw buffer descriptor whose range is exactly the segment: the
// address is one 32-bit lane offset plus a scalar offset, and anything past the
// segment's end (rows >= M of a ragged strip, columns >= N of a ragged tile)
// reads as zero or is dropped by the hardware instead of being clamped in code.
struct SegRes {
    __amdgpu_buffer_rsrc_t a, b, o;
};

constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family)

template <int OUT_BYTES>
__device__ __forceinline__ SegRes make_res(const Seg &s, const void *A, const void *B, void *out) {
    SegRes r;
    r.a = __builtin_amdgcn_make_buffer_rsrc((void *)((const uint16_t *)A + s.a), 0, s.M * s.K * 2, kRsrcFlags);
    r.b = __builtin_amdgcn_make_buffer_rsrc((void *)((const uint16_t *)B + s.b), 0, s.N * s.K * 2, kRsrcFlags);
    r.o = __builtin_amdgcn_make_buffer_rsrc((void *)((char *)out + s.o * OUT_BYTES), 0, s.M * s.N * OUT_BYTES,
                                            kRsrcFlags);
    return r;
}

// ------------------------------------------------------------ operand loads
__device__ __forceinline__ u32x4 load_frag_fast(const uint16_t *__restrict__ row_ptr, int kk, int K) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (kk < K) v = *reinterpret_cast<const u32x4 *>(row_ptr + kk);
    return v;
}

// ------------------------------------------------------------ generic rows
// Fallback for segments the 16-byte operand loads cannot serve (K % 8 != 0,
// odd segment starts, transposed layouts): one wavefront walks rows
// [r_begin, r_end), lanes own columns c_begin + lane + 64*j, fp32 multiply-add
// in k order.  GEMM only writes the products; the fused form sweeps each row
// twice (maximum and sum first, then recompute and store).  Never inlined, so
// its registers do not add to the MFMA paths.
template <int DT> __device__ __forceinline__ float generic_dot(const uint16_t *__restrict__ aseg,
                                                               const uint16_t *__restrict__ bseg, int r, int col,
                                                               int M, int N, int K, bool t1, bool t2) {
    float acc = 0.f;
    for (int t = 0; t < K; ++t) {
        const float av = Elem<DT>::to_float(t1 ? aseg[(int64_t)t * M + r] : aseg[(int64_t)r * K + t]);
        const float bv = Elem<DT>::to_float(t2 ? bseg[(int64_t)t * N + col] : bseg[(int64_t)col * K + t]);
        acc = fmaf(av, bv, acc);
    }
    return acc;
}

template <int DT> __device__ __forceinline__ void store_one(void *out, int64_t e, float v, bool f32out) {
    if (f32out) reinterpret_cast<float *>(out)[e] = v;
    else reinterpret_cast<uint16_t *>(out)[e] = Elem<DT>::from_float(v);
}

template <int DT, bool FUSED>
__device__ __attribute__((noinline)) void generic_rows(const uint16_t *aseg, const uint16_t *bseg, void *out,
                                                       int64_t o, int M, int N, int K, int r_begin, int r_end,
                                                       int c_begin, int c_end, float scale, int flags) {
    const int lane = lane_id();
    const bool t1 = flags & kFlagTranspose1, t2 = flags & kFlagTranspose2, f32out = flags & kFlagOutF32;
    for (int r = r_begin; r < r_end; ++r) {
        const int64_t e0 = o + (int64_t)r * N;
        if (!FUSED) {
            for (int col = c_begin + lane; col < c_end; col += 64)
                store_one<DT>(out, e0 + col, generic_dot<DT>(aseg, bseg, r, col, M, N, K, t1, t2), false);
        } else {
            float c = scale * kLog2e;
            const float sgn = c < 0.f ? -1.f : 1.f;
            c *= sgn;
            float mx = -INFINITY;
            for (int col = lane; col < N; col += 64)
                mx = fmaxf(mx, sgn * generic_dot<DT>(aseg, bseg, r, col, M, N, K, t1, t2));
            mx = wave_max(mx);
            const float bias = -((mx == -INFINITY) ? 0.f : mx) * c;
            float sum = 0.f;
            for (int col = lane; col < N; col += 64)
                sum += __builtin_amdgcn_exp2f(fmaf(sgn * generic_dot<DT>(aseg, bseg, r, col, M, N, K, t1, t2), c, bias));
            sum = wave_sum(sum);
            const float inv = 1.f / sum;
            for (int col = lane; col < N; col += 64)
                store_one<DT>(out, e0 + col,
                              __builtin_amdgcn_exp2f(
                                  fmaf(sgn * generic_dot<DT>(aseg, bseg, r, col, M, N, K, t1, t2), c, bias)) * inv,
                              f32out);
        }
    }
}

// ------------------------------------------------------------------- scores
// acc[t] (t < NT) <- rows r0..r0+15 x columns c0+16t..c0+16t+15 of A_g B_g^T, for
// segments whose operand rows are 16-byte aligned.
// Rows and columns past the segment read as zeros (buffer range check); the
// callers discard those results.
template <int DT, int NT>
__device__ __forceinline__ void stage_scores(f32x4 (&acc)[kMaxTiles], const Seg &s, const SegRes &res, int r0,
                                             int c0) {
    const int lane = lane_id(), l16 = lane & 15, q = lane >> 4;
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int K = s.K;
    // One lane offset serves A and B alike: row l16 of the tile, k-group q.
    const int voff = (l16 * K + q * 8) * 2;
    const int a_soff = r0 * K * 2;
    // Loads are issued in batches of at most kBatch tiles so that the operand
    // registers in flight stay well below the accumulator count.
    constexpr int kBatch = NT < 4 ? NT : 4;
    const int kfull = K & ~31;
    for (int k0 = 0; k0 < kfull; k0 += 32) {
        const u32x4 af = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff, a_soff + k0 * 2, 0);
#pragma unroll
        for (int tb = 0; tb < NT; tb += kBatch) {
            u32x4 bf[kBatch];
#pragma unroll
            for (int t = 0; t < kBatch; ++t)
                bf[t] = __builtin_amdgcn_raw_buffer_load_b128(res.b, voff, ((c0 + (tb + t) * 16) * K + k0) * 2, 0);
#pragma unroll
            for (int t = 0; t < kBatch; ++t) acc[tb + t] = Elem<DT>::mfma(bf[t], af, acc[tb + t]);
        }
    }
    if (kfull < K) {   // K % 32 in {8, 16, 24}: lanes whose k-group lies past K feed zeros
        const bool live = kfull + q * 8 < K;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        u32x4 af = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff, a_soff + kfull * 2, 0);
        af = live ? af : zero;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            u32x4 bf = __builtin_amdgcn_raw_buffer_load_b128(res.b, voff, ((c0 + t * 16) * K + kfull) * 2, 0);
            bf = live ? bf : zero;
            acc[t] = Elem<DT>::mfma(bf, af, acc[t]);
        }
    }
}

// ------------------------------------------------------------ local softmax
// In: raw scores.  Out: acc = exp2((s - m) * c) for this wavefront's columns
// (0 for columns past N), m = the row maximum over these columns (same in the
// four lanes of a row), l = the row sum of acc.  c = scale * log2(e) >= 0.
// m_shift (= m, or 0 when m is -inf) is what was subtracted.
template <int NT>
__device__ __forceinline__ void local_softmax(f32x4 (&acc)[kMaxTiles], int N, int c0, float c, float &m,
                                              float &l) {
    const int q = lane_id() >> 4;
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int col = c0 + t * 16 + q * 4;
        if (c0 + t * 16 + 16 <= N) {
#pragma unroll
            for (int i = 0; i < 4; ++i) mx = fmaxf(mx, acc[t][i]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) mx = (col + i < N) ? fmaxf(mx, acc[t][i]) : mx;
        }
    }
    mx = quad_column_max(mx);
    const float shift = (mx == -INFINITY) ? 0.f : mx;
    const float bias = -shift * c;
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int col = c0 + t * 16 + q * 4;
        if (c0 + t * 16 + 16 <= N) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = __builtin_amdgcn_exp2f(fmaf(acc[t][i], c, bias));
                acc[t][i] = p;
                sum += p;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = (col + i < N) ? __builtin_amdgcn_exp2f(fmaf(acc[t][i], c, bias)) : 0.f;
                acc[t][i] = p;
                sum += p;
            }
        }
    }
    m = mx;
    l = quad_column_sum(sum);
}

// ------------------------------------------------------------------- stores
// Writes acc[t][i] * factor for rows < M and columns < N.  The lane's four
// columns are consecutive in memory: one 8-byte (16-bit output) or 16-byte
// (fp32 output) store when the address allows it, element stores otherwise.
template <int DT, int NT, bool F32OUT>
__device__ __forceinline__ void store_rows(const f32x4 (&acc)[kMaxTiles], const Seg &s, const SegRes &res, int r0,
                                           int c0, float factor, bool out_aligned) {
    const int lane = lane_id(), l16 = lane & 15, q = lane >> 4;
    const int r = r0 + l16;
    if (r >= s.M) return;
    const int e0 = r * s.N;                 // element offset of the row inside the segment
    const int phase = (int)(s.o & 3);       // alignment of the segment start in elements
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int col = c0 + t * 16 + q * 4;
        if (col >= s.N) continue;
        const int e = e0 + col;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = acc[t][i] * factor;
        const bool vec = col + 3 < s.N && ((e + phase) & 3) == 0 && out_aligned;
        if (F32OUT) {
            if (vec) {
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, f32x4{v[0], v[1], v[2], v[3]}),
                                                       res.o, e * 4, 0, 0);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (col + i < s.N)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v[i]), res.o, (e + i) * 4,
                                                              0, 0);
            }
        } else {
            if (vec) {
                __builtin_amdgcn_raw_buffer_store_b64(
                    u32x2{Elem<DT>::pack2(v[0], v[1]), Elem<DT>::pack2(v[2], v[3])}, res.o, e * 2, 0, 0);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (col + i < s.N)
                        __builtin_amdgcn_raw_buffer_store_b16(Elem<DT>::from_float(v[i]), res.o, (e + i) * 2, 0, 0);
            }
        }
    }
}

template <int NT> __device__ __forceinline__ void negate(f32x4 (&acc)[kMaxTiles]) {
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = -acc[t];
}

// One wavefront, one strip, everything in registers.
template <int DT, int NT, bool FUSED, bool F32OUT>
__device__ __forceinline__ void wave_strip(const Seg &s, const RunArgs &a, int r0, int c0, bool out_aligned) {
    f32x4 acc[kMaxTiles];
    const SegRes res = make_res<F32OUT ? 4 : 2>(s, a.A, a.B, a.out);
    stage_scores<DT, NT>(acc, s, res, r0, c0);
    float factor = 1.f;
    if (FUSED) {
        float c = a.scale * kLog2e;
        if (c < 0.f) { negate<NT>(acc); c = -c; }
        float m, l;
        local_softmax<NT>(acc, s.N, c0, c, m, l);
        factor = 1.f / l;
    }
    store_rows<DT, NT, F32OUT>(acc, s, res, r0, c0, factor, out_aligned);
}

template <int DT, bool FUSED, bool F32OUT>
__device__ __forceinline__ void wave_strip_dispatch(int nt, const Seg &s, const RunArgs &a, int r0, int c0,
                                                    bool out_aligned) {
    if (nt <= 1) wave_strip<DT, 1, FUSED, F32OUT>(s, a, r0, c0, out_aligned);
    else if (nt <= 2) wave_strip<DT, 2, FUSED, F32OUT>(s, a, r0, c0, out_aligned);
    else if (nt <= 4) wave_strip<DT, 4, FUSED, F32OUT>(s, a, r0, c0, out_aligned);
    else if (nt <= 8) wave_strip<DT, 8, FUSED, F32OUT>(s, a, r0, c0, out_aligned);
    else wave_strip<DT, 16, FUSED, F32OUT>(s, a, r0, c0, out_aligned);
}

__device__ __forceinline__ Seg load_seg(const PlanRO &pv, int g, int64_t h, const RunArgs &a) {
    const SegRec r = load_rec(pv.recs, g);   // scalar loads
    Seg s;
    s.M = r.M; s.N = r.N; s.K = r.K;
    s.a = h * a.Dm1 + r.off1;
    s.b = h * a.Dm2 + r.off2;
    s.o = h * a.Dout + r.offO;
    return s;
}

template <int DT, bool FUSED>
__device__ __forceinline__ void generic_seg_rows(const Seg &s, const RunArgs &a, int r_begin, int r_end,
                                                 int c_begin, int c_end) {
    generic_rows<DT, FUSED>((const uint16_t *)a.A + s.a, (const uint16_t *)a.B + s.b, a.out, s.o, s.M, s.N, s.K,
                            r_begin, min(r_end, s.M), c_begin, min(c_end, s.N), a.scale, a.flags);
}

// ---------------------------------------------------------------- pack item
// Segments g .. g+len-1 (same K, sum M <= 16, sum N <= 16) share one MFMA tile:
// the tile's rows are the members' A rows back to back, its columns the
// members' B rows back to back; only the block-diagonal products are kept.
template <int DT, bool FUSED, bool F32OUT>
__device__ __forceinline__ void wave_pack(const PlanRO &pv, int g, int len, int64_t h, const RunArgs &a) {
    const int lane = lane_id(), l16 = lane & 15, q = lane >> 4;
    const int K = pv.recs[g].K;
    int rowMem = -1, rowLoc = 0;                   // member and local row of tile row l16 (A side)
    int colMemL = -1, colLocL = 0;                 // member and local row of tile column l16 (B side)
    int cMem[4] = {-1, -1, -1, -1}, cLoc[4] = {0, 0, 0, 0};  // the same for the lane's four output columns
    int mAcc = 0, nAcc = 0;
    for (int j = 0; j < len; ++j) {
        const int mj = pv.recs[g + j].M, nj = pv.recs[g + j].N;
        if (rowMem < 0 && l16 < mAcc + mj) { rowMem = j; rowLoc = l16 - mAcc; }
        if (colMemL < 0 && l16 < nAcc + nj) { colMemL = j; colLocL = l16 - nAcc; }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = q * 4 + i;
            if (cMem[i] < 0 && c < nAcc + nj) { cMem[i] = j; cLoc[i] = c - nAcc; }
        }
        mAcc += mj; nAcc += nj;
    }
    // Rows / columns past the pack reuse the last member's last row (valid memory).
    const int am = rowMem >= 0 ? rowMem : len - 1;
    const int al = rowMem >= 0 ? rowLoc : pv.recs[g + len - 1].M - 1;
    const int bm = colMemL >= 0 ? colMemL : len - 1;
    const int bl = colMemL >= 0 ? colLocL : pv.recs[g + len - 1].N - 1;
    const uint16_t *arow = (const uint16_t *)a.A + h * a.Dm1 + pv.recs[g + am].off1 + (int64_t)al * K;
    const uint16_t *brow = (const uint16_t *)a.B + h * a.Dm2 + pv.recs[g + bm].off2 + (int64_t)bl * K;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        const int kk = k0 + q * 8;
        const u32x4 af = load_frag_fast(arow, kk, K);
        const u32x4 bf = load_frag_fast(brow, kk, K);
        acc = Elem<DT>::mfma(bf, af, acc);
    }
    float v[4];
    bool keep[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { keep[i] = rowMem >= 0 && cMem[i] == rowMem; v[i] = acc[i]; }
    if (FUSED) {
        float c = a.scale * kLog2e;
        if (c < 0.f) {
            c = -c;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = -v[i];
        }
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = keep[i] ? fmaxf(mx, v[i]) : mx;
        mx = quad_column_max(mx);
        const float bias = -((mx == -INFINITY) ? 0.f : mx) * c;
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = keep[i] ? __builtin_amdgcn_exp2f(fmaf(v[i], c, bias)) : 0.f;
            sum += v[i];
        }
        sum = quad_column_sum(sum);
        const float inv = 1.f / sum;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= inv;
    }
    if (rowMem < 0) return;
    const int Nr = pv.recs[g + rowMem].N;
    const int64_t e0 = h * a.Dout + pv.recs[g + rowMem].offO + (int64_t)rowLoc * Nr;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (keep[i]) store_one<DT>(a.out, e0 + cLoc[i], v[i], F32OUT);
}

// Combines the per-wavefront (maximum, sum) pairs of one strip through LDS.
// Returns the factor this wavefront's exp2((s - m_wave) * c) values must be
// multiplied by; gshift receives the subtracted global maximum and ginv 1/sum.
__device__ __forceinline__ float exchange_row_stats(float (*sM)[16], float (*sL)[16], int wave, float m, float l,
                                                    float c, float &gshift, float &ginv) {
    const int lane = lane_id(), l16 = lane & 15;
    if (lane < 16) { sM[wave][l16] = m; sL[wave][l16] = l; }
    __syncthreads();
    float gm = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWavesPerGroup; ++w) gm = fmaxf(gm, sM[w][l16]);
    gshift = (gm == -INFINITY) ? 0.f : gm;
    float gl = 0.f;
#pragma unroll
    for (int w = 0; w < kWavesPerGroup; ++w) {
        const float mw = sM[w][l16];
        const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((mw - gshift) * c);
        gl += sL[w][l16] * f;
    }
    ginv = 1.f / gl;
    const float mine = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m - gshift) * c);
    return mine * ginv;
}

// ------------------------------------------------------------------ kernels
// Three kernels share one plan: wave_items_kernel (packs, strips / GEMM pieces
// and the element-wise fallback; wavefronts never synchronise), split_kernel
// (256 < N <= 4096) and wide_kernel (N > 4096), the latter two with one
// 16-wave workgroup per strip.  Each loops `for (item = first; item < total;
// item += stride)`, with the total read from the plan, so any grid size is
// correct: a grid that covers the items gives one item per wavefront or
// workgroup and leaves balancing to the hardware dispatcher, a smaller grid
// strides.
constexpr int kItemThreads = 256;
constexpr int kItemWaves = kItemThreads / 64;

__device__ __forceinline__ bool plan_matches(PlanHeader *hdr, const RunArgs &a) {
    if (hdr->magic == kPlanMagic && hdr->kind == 0 && hdr->bad_segments == 0 && hdr->Dm1 == a.Dm1 &&
        hdr->Dm2 == a.Dm2 && hdr->Dout == a.Dout)
        return true;
    if (blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&hdr->run_errors, 1);
    return false;
}

// Element-wise path over whole work-item lists: the plan's slow strips always,
// and every other list too when the launch itself rules out the 16-byte loads
// (transposed layouts, unaligned base pointers or head strides).
template <int DT, bool FUSED>
__device__ __attribute__((noinline)) void generic_phase(const RunArgs &a, bool everything, int64_t gw, int64_t nw) {
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const int kinds[5] = {kPfxSlow, kPfxPack, FUSED ? kPfxStrip : kPfxGemm, kPfxSplit, kPfxWide};
    const int nkinds = everything ? (FUSED ? 5 : 3) : 1;
    for (int ki = 0; ki < nkinds; ++ki) {
        const int kind = kinds[ki];
        const int64_t per_head = hdr->totals[kind];
        const ConstI32 pfx = pv.pfx[kind];
        for (int64_t it = gw; it < per_head * a.H; it += nw) {
            const int64_t h = it / per_head;
            const int i = (int)(it - h * per_head);
            const int g = prefix_search(pfx, nseg, i);
            const int local = i - pfx[g];
            if (kind == kPfxPack) {
                const int len = pv.recs[g].packLen;
                for (int j = 0; j < len; ++j) {
                    const Seg s = load_seg(pv, g + j, h, a);
                    generic_seg_rows<DT, FUSED>(s, a, 0, s.M, 0, s.N);
                }
                continue;
            }
            const Seg s = load_seg(pv, g, h, a);
            int r0 = local * kStripRows, c0 = 0, c1 = s.N;
            if (kind == kPfxGemm) {
                const int chunks = (s.N + kWaveCols - 1) / kWaveCols;
                r0 = (local / chunks) * kStripRows; c0 = (local % chunks) * kWaveCols; c1 = c0 + kWaveCols;
            }
            generic_seg_rows<DT, FUSED>(s, a, r0, r0 + kStripRows, c0, c1);
        }
    }
}

template <int DT, bool FUSED, bool F32OUT>
__global__ __launch_bounds__(kItemThreads, 4) void wave_items_kernel(RunArgs a) {
    PlanHeader *hdr = reinterpret_cast<PlanHeader *>(a.plan);
    if (!plan_matches(hdr, a)) return;
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int64_t gw = (int64_t)blockIdx.x * kItemWaves + wave;
    const int64_t nw = (int64_t)gridDim.x * kItemWaves;
    const bool out_aligned = ((uintptr_t)a.out & 15) == 0;
    const bool mfma_ok = (a.flags & kFlagMfmaOk) != 0;
    if (!mfma_ok || hdr->totals[kPfxSlow] != 0) generic_phase<DT, FUSED>(a, !mfma_ok, gw, nw);
    if (!mfma_ok) return;
    {
        const int64_t per_head = hdr->totals[kPfxPack];
        const ConstI32 pfx = pv.pfx[kPfxPack];
        for (int64_t it = gw; it < per_head * a.H; it += nw) {
            const int64_t h = it / per_head;
            const int i = (int)(it - h * per_head);
            const int g = prefix_search(pfx, nseg, i);
            wave_pack<DT, FUSED, F32OUT>(pv, g, pv.recs[g].packLen, h, a);
        }
    }
    {
        const int kind = FUSED ? kPfxStrip : kPfxGemm;
        const int64_t per_head = hdr->totals[kind];
        const ConstI32 pfx = pv.pfx[kind];
        for (int64_t it = gw; it < per_head * a.H; it += nw) {
            const int64_t h = it / per_head;
            const int i = (int)(it - h * per_head);
            const int g = prefix_search(pfx, nseg, i);
            const int local = i - pfx[g];
            const Seg s = load_seg(pv, g, h, a);
            int r0, c0;
            if (FUSED) {
                r0 = local * kStripRows; c0 = 0;
            } else {
                const int chunks = (s.N + kWaveCols - 1) / kWaveCols;
                r0 = (local / chunks) * kStripRows; c0 = (local % chunks) * kWaveCols;
            }
            const int nt = min(kMaxTiles, (s.N - c0 + 15) >> 4);
            wave_strip_dispatch<DT, FUSED, F32OUT>(nt, s, a, r0, c0, out_aligned);
        }
    }
}

// 256 < N <= 4096: each wavefront of the workgroup owns 256 columns of the strip.
template <int DT, bool F32OUT>
__global__ __launch_bounds__(kGroupThreads) void split_kernel(RunArgs a) {
    // Two copies: consecutive strips alternate, so a wavefront that runs ahead
    // never overwrites statistics its neighbours are still reading.
    __shared__ float sM[2][kWavesPerGroup][16];
    __shared__ float sL[2][kWavesPerGroup][16];
    PlanHeader *hdr = reinterpret_cast<PlanHeader *>(a.plan);
    if (!(a.flags & kFlagMfmaOk) || !plan_matches(hdr, a)) return;
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const int wave = uniform((int)(threadIdx.x >> 6));
    const bool out_aligned = ((uintptr_t)a.out & 15) == 0;
    const int64_t per_head = hdr->totals[kPfxSplit];
    const ConstI32 pfx = pv.pfx[kPfxSplit];
    float c = a.scale * kLog2e;
    const bool neg = c < 0.f;
    if (neg) c = -c;
    int xchg = 0;
    for (int64_t it = blockIdx.x; it < per_head * a.H; it += gridDim.x) {
        const int64_t h = it / per_head;
        const int i = (int)(it - h * per_head);
        const int g = prefix_search(pfx, nseg, i);
        const int r0 = (i - pfx[g]) * kStripRows;
        const Seg s = load_seg(pv, g, h, a);
        const SegRes res = make_res<F32OUT ? 4 : 2>(s, a.A, a.B, a.out);
        const int c0 = wave * kWaveCols;
        const int nt = max(0, min(kMaxTiles, (s.N - c0 + 15) >> 4));
        f32x4 acc[kMaxTiles];
        float m = -INFINITY, l = 0.f;
#define BA_SPLIT_STAGE(NT)                              \
    {                                                   \
        stage_scores<DT, NT>(acc, s, res, r0, c0);      \
        if (neg) negate<NT>(acc);                       \
        local_softmax<NT>(acc, s.N, c0, c, m, l);       \
    }
        if (nt > 8) BA_SPLIT_STAGE(16)
        else if (nt > 4) BA_SPLIT_STAGE(8)
        else if (nt > 2) BA_SPLIT_STAGE(4)
        else if (nt > 1) BA_SPLIT_STAGE(2)
        else if (nt > 0) BA_SPLIT_STAGE(1)
#undef BA_SPLIT_STAGE
        const int buf = xchg & 1;
        ++xchg;
        float gshift, ginv;
        const float factor = exchange_row_stats(sM[buf], sL[buf], wave, m, l, c, gshift, ginv);
        if (nt > 8) store_rows<DT, 16, F32OUT>(acc, s, res, r0, c0, factor, out_aligned);
        else if (nt > 4) store_rows<DT, 8, F32OUT>(acc, s, res, r0, c0, factor, out_aligned);
        else if (nt > 2) store_rows<DT, 4, F32OUT>(acc, s, res, r0, c0, factor, out_aligned);
        else if (nt > 1) store_rows<DT, 2, F32OUT>(acc, s, res, r0, c0, factor, out_aligned);
        else if (nt > 0) store_rows<DT, 1, F32OUT>(acc, s, res, r0, c0, factor, out_aligned);
    }
}

// N > 4096: sweep 1 finds the row maximum and sum with an online update per
// 4096-column block, sweep 2 recomputes the scores and stores.
template <int DT, bool F32OUT>
__global__ __launch_bounds__(kGroupThreads) void wide_kernel(RunArgs a) {
    __shared__ float sM[2][kWavesPerGroup][16];
    __shared__ float sL[2][kWavesPerGroup][16];
    PlanHeader *hdr = reinterpret_cast<PlanHeader *>(a.plan);
    if (!(a.flags & kFlagMfmaOk) || !plan_matches(hdr, a)) return;
    const int nseg = hdr->nseg;
    const PlanRO pv = plan_ro(a.plan, nseg);
    const int wave = uniform((int)(threadIdx.x >> 6));
    const bool out_aligned = ((uintptr_t)a.out & 15) == 0;
    const int64_t per_head = hdr->totals[kPfxWide];
    const ConstI32 pfx = pv.pfx[kPfxWide];
    float c = a.scale * kLog2e;
    const bool neg = c < 0.f;
    if (neg) c = -c;
    int xchg = 0;
    for (int64_t it = blockIdx.x; it < per_head * a.H; it += gridDim.x) {
        const int64_t h = it / per_head;
        const int i = (int)(it - h * per_head);
        const int g = prefix_search(pfx, nseg, i);
        const int r0 = (i - pfx[g]) * kStripRows;
        const Seg s = load_seg(pv, g, h, a);
        const SegRes res = make_res<F32OUT ? 4 : 2>(s, a.A, a.B, a.out);
        f32x4 acc[kMaxTiles];
        float run_m = -INFINITY, run_l = 0.f;
        for (int cb = 0; cb < s.N; cb += kSplitCols) {
            const int c0 = cb + wave * kWaveCols;
            if (c0 >= s.N) continue;
            float m, l;
            stage_scores<DT, kMaxTiles>(acc, s, res, r0, c0);
            if (neg) negate<kMaxTiles>(acc);
            local_softmax<kMaxTiles>(acc, s.N, c0, c, m, l);
            const float nm = fmaxf(run_m, m);
            const float nshift = (nm == -INFINITY) ? 0.f : nm;
            const float f_old = (run_m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((run_m - nshift) * c);
            const float f_new = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m - nshift) * c);
            run_l = run_l * f_old + l * f_new;
            run_m = nm;
        }
        const int buf = xchg & 1;
        ++xchg;
        float gshift, ginv;
        exchange_row_stats(sM[buf], sL[buf], wave, run_m, run_l, c, gshift, ginv);
        const float bias = -gshift * c;
        for (int cb = 0; cb < s.N; cb += kSplitCols) {
            const int c0 = cb + wave * kWaveCols;
            if (c0 >= s.N) continue;
            stage_scores<DT, kMaxTiles>(acc, s, res, r0, c0);
            if (neg) negate<kMaxTiles>(acc);
#pragma unroll
            for (int t = 0; t < kMaxTiles; ++t)
#pragma unroll
                for (int k = 0; k < 4; ++k) acc[t][k] = __builtin_amdgcn_exp2f(fmaf(acc[t][k], c, bias));
            store_rows<DT, kMaxTiles, F32OUT>(acc, s, res, r0, c0, ginv, out_aligned);
        }
    }
}

// --------------------------------------------------------------------- host
// Grid sizes.  With a host copy of the plan summary the grids cover the items
// exactly (capped) and kernels with nothing to do are not launched; without
// it every kernel is launched with a resident-size grid and strides.
static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

template <int DT, bool FUSED, bool F32OUT>
static int launch_set(const RunArgs &args, const ba_plan_info *info, hipStream_t stream) {
    const int cus = device_cu_count();
    const int64_t cap = (int64_t)cus * 64;
    int64_t g_items = (int64_t)cus * 8, g_split = cus, g_wide = cus;
    if (info) {
        const bool mfma_ok = args.flags & kFlagMfmaOk;
        int64_t wave_items = (FUSED ? info->strip_items : info->gemm_items) + info->pack_items + info->slow_items;
        if (!mfma_ok && FUSED) wave_items += info->split_items + info->wide_items;
        g_items = std::min(cap, ceil_div(wave_items * args.H, kItemWaves));
        g_split = mfma_ok ? std::min(cap, info->split_items * args.H) : 0;
        g_wide = mfma_ok ? std::min(cap, info->wide_items * args.H) : 0;
    }
    if (g_items > 0)
        hipLaunchKernelGGL((wave_items_kernel<DT, FUSED, F32OUT>), dim3((unsigned)g_items), dim3(kItemThreads), 0,
                           stream, args);
    if (FUSED && g_split > 0)
        hipLaunchKernelGGL((split_kernel<DT, F32OUT>), dim3((unsigned)g_split), dim3(kGroupThreads), 0, stream, args);
    if (FUSED && g_wide > 0)
        hipLaunchKernelGGL((wide_kernel<DT, F32OUT>), dim3((unsigned)g_wide), dim3(kGroupThreads), 0, stream, args);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_strips(int dtype, int fused, const RunArgs &args, const ba_plan_info *info, hipStream_t stream) {
    const bool f32out = args.flags & kFlagOutF32;
    if (dtype == BA_F16) {
        if (!fused) return launch_set<0, false, false>(args, info, stream);
        return f32out ? launch_set<0, true, true>(args, info, stream) : launch_set<0, true, false>(args, info, stream);
    }
    if (dtype == BA_BF16) {
        if (!fused) return launch_set<1, false, false>(args, info, stream);
        return f32out ? launch_set<1, true, true>(args, info, stream) : launch_set<1, true, false>(args, info, stream);
    }
    return BA_ERR_UNSUPPORTED;
}

}  // namespace ba
