// Varlen GEMM (S_g = A_g B_g^T) and the fused GEMM + row softmax for fp16/bf16
// on gfx950: MFMA 16x16x32 with fp32 accumulation, scores kept in registers.
// This file holds the two kernels for segments of up to 256 columns and the
// launcher of a whole call; large segments are tile_kernel.hip.
//
//   strip_kernel    strip-class segments whose B_g fits an LDS window: B_g is
//                   copied to LDS once per workgroup, each wavefront computes
//                   16-row strips with code specialised for the exact tile count
//                   and with lane order following memory order (strips_exact).
//   segment_kernel  everything that needs care instead of speed: packs of tiny
//                   segments sharing one MFMA tile (wave_pack), segments that
//                   break the 16-byte operand alignment (K % 8 != 0, odd segment
//                   starts, transposed layouts: element-wise generic_rows),
//                   strip-class leftovers whose B_g is walked in K slabs
//                   (strips_from_lds).
//
// Both operands are K-contiguous (A_g is M x K, B_g is N x K), so a lane's
// eight k-values are one 16-byte load straight into an MFMA operand register;
// no transposition is ever needed.
#include <algorithm>

#include "ba_gemm_common.hpp"
#include "tile_body.hpp"

namespace ba {

constexpr int kMaxTiles = kWaveCols / 16;  // 16 MFMA tiles per wavefront

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

// ------------------------------------------------------------ local softmax
// Brings raw scores into the form the softmax below takes: the multiplier c =
// scale * log2(e) made non-negative (scores negated for a negative scale, set
// to zero for a zero scale, where every probability is 1/N), and the columns of
// the ragged last tile that lie past N set to -inf, so that no later step needs
// a column mask.  nt = tiles that exist for this wavefront (<= NT).
template <int NT>
__device__ __forceinline__ void prepare_scores(f32x4 (&acc)[kMaxTiles], int nt, int N, int c0, float &c) {
    if (c < 0.f) {
        c = -c;
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = -acc[t];
    } else if (c == 0.f) {
        c = 1.f;
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int last = nt - 1;
    const int rem = N - c0 - last * 16;          // columns of the last tile, 1..16
    if (rem < 16) {
        const int q4 = (lane_id() >> 4) * 4;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t == last) {
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][i] = (q4 + i < rem) ? acc[t][i] : -INFINITY;
            }
        }
    }
}

// In: prepared scores.  Out: acc = exp2((s - m) * c) for this wavefront's
// tiles, m = the row maximum over them (the same in the four lanes of a row),
// l = the row sum of acc.
template <int NT>
__device__ __forceinline__ void local_softmax(f32x4 (&acc)[kMaxTiles], int nt, float c, float &m, float &l) {
    settle_mfma(acc);
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if (t < nt) {
            mx = max3(mx, acc[t][0], acc[t][1]);
            mx = max3(mx, acc[t][2], acc[t][3]);
        }
    }
    mx = quad_column_max(mx);
    const float shift = (mx == -INFINITY) ? 0.f : mx;
    const float bias = -shift * c;
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if (t < nt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = __builtin_amdgcn_exp2f(fmaf(acc[t][i], c, bias));
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
// columns are consecutive in memory and go out as ONE 8-byte (16-bit output)
// or 16-byte (fp32 output) store whatever the address: row starts are only
// element-aligned (odd N), and the memory pipeline takes vector stores at any
// element alignment.  Only the ragged last tile of a row uses element stores.

template <int DT, bool F32OUT>
__device__ __forceinline__ void store_quad(void *__restrict__ out, int64_t e, const f32x4 &v, int valid) {
    if (F32OUT) {
        float *o = reinterpret_cast<float *>(out) + e;
        if (valid >= 4) {
            *reinterpret_cast<f32x4_unaligned *>(o) = v;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i < valid) o[i] = v[i];
        }
    } else {
        uint16_t *o = reinterpret_cast<uint16_t *>(out) + e;
        if (valid >= 4) {
            *reinterpret_cast<u32x2_unaligned *>(o) = u32x2{Elem<DT>::pack2(v[0], v[1]), Elem<DT>::pack2(v[2], v[3])};
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i < valid) o[i] = Elem<DT>::from_float(v[i]);
        }
    }
}

template <int DT, int NT, bool F32OUT>
__device__ __forceinline__ void store_rows(const f32x4 (&acc)[kMaxTiles], int nt, const Seg &s, void *__restrict__ out,
                                           int r0, int c0, float factor) {
    const int lane = lane_id(), l16 = lane & 15, q = lane >> 4;
    const int r = r0 + l16;
    if (r >= s.M) return;
    const int64_t e0 = s.o + (int64_t)r * s.N + c0 + q * 4;
    const int last = nt - 1;
    const int rem = s.N - c0 - last * 16;         // columns of the last tile, 1..16
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        if (t < last || (t == last && rem == 16)) {
            store_quad<DT, F32OUT>(out, e0 + t * 16, acc[t] * factor, 4);
        } else if (t == last) {
            store_quad<DT, F32OUT>(out, e0 + t * 16, acc[t] * factor, rem - q * 4);
        }
    }
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

// ------------------------------------------------------ LDS-staged strips
// All strips of one segment need the same B_g.  The workgroup copies it into
// LDS once, already in MFMA operand order, with direct global->LDS loads (no
// registers in between): block (kstep, tile) is the 1 KiB that the 64 lanes of
// a wavefront feed to one MFMA -- lane i's 16 bytes (row i%16 of the tile, eight
// k-values of group i/16) sit at byte 16*i.  Reading a block back is therefore
// one ds_read_b128 per lane at consecutive addresses: conflict-free by
// construction, no padding or swizzle to compute.  Segments whose B_g exceeds
// the LDS window are walked in K slabs.
constexpr int kLdsBlockBytes = 1024;
constexpr int kRaggedCopyBytes = 16 * 256 + 1024;  // 16 rows of 128 k, and the round-up of the image to whole KiB
constexpr int kSegWaves = 4;
constexpr int kSegThreads = 64 * kSegWaves;
// k-steps (of 32) whose A fragments a wavefront keeps in registers: 4 in the 128-register build, 2 in the
// leaner build (larger K takes more slabs)
template <int MAXNT> struct SlabSteps { static constexpr int value = MAXNT <= 8 ? 2 : 4; };

template <int DT, int NT, bool FUSED, bool F32OUT, int MAXNT>
__device__ __forceinline__ void strips_from_lds(const Seg &s, const RunArgs &a, unsigned char *lds, int lds_blocks,
                                                int r0, bool active, int wave, int nwaves) {
    const int lane = lane_id(), l16 = lane & 15, q = lane >> 4;
    const int K = s.K, N = s.N;
    const int nt = (N + 15) >> 4;                 // tiles that exist (<= NT)
    constexpr int kSlabSteps = SlabSteps<MAXNT>::value;
    const int nks_total = (K + 31) >> 5;
    const int slab_ks = max(1, min(kSlabSteps, lds_blocks / nt));  // k-steps per LDS fill
    const SegRes res = make_res(s, a.A, a.B);
    const int voff = (l16 * K + q * 8) * 2;
    const int a_soff = r0 * K * 2;
    const uint16_t *bseg = (const uint16_t *)a.B + s.b;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    f32x4 acc[kMaxTiles];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int ks0 = 0; ks0 < nks_total; ks0 += slab_ks) {
        const int nks = min(slab_ks, nks_total - ks0);
        if (ks0 > 0) __syncthreads();             // everyone is done reading the previous slab
        // The wavefront's own A fragments of the slab go to registers first, so their
        // latency runs under the LDS fill and nothing is fetched inside the MFMA loop.
        u32x4 af[kSlabSteps];
#pragma unroll
        for (int ksi = 0; ksi < kSlabSteps; ++ksi) {
            af[ksi] = zero;
            if (active && ksi < nks) {
                const int ks = ks0 + ksi;
                af[ksi] = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff, a_soff + ks * 64, 0);
            }
        }
        for (int t = wave; t < nt; t += nwaves) {       // tile t of every k-step of the slab
            const int row = min(t * 16 + l16, N - 1);   // ragged last tile: repeat the last row (masked later)
            const uint16_t *brow = bseg + (int64_t)row * K;
            for (int ksi = 0; ksi < nks; ++ksi) {
                int kk = (ks0 + ksi) * 32 + q * 8;
                kk = kk < K ? kk : 0;                    // ragged last k-step: valid data, multiplied by zeros
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(brow + kk),
                    (__attribute__((address_space(3))) void *)(lds + (ksi * nt + t) * kLdsBlockBytes), 16, 0, 0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0);            // this wavefront's loads and LDS fills have landed
        __syncthreads();
        if (active) {
            // Ragged last k-step: lanes whose k-group lies past K feed a zero A fragment
            // (their B fragment is a repeat of valid row data, see the fill above).
            if ((ks0 + nks) * 32 > K) {
#pragma unroll
                for (int ksi = 0; ksi < kSlabSteps; ++ksi)
                    if (ksi == nks - 1) af[ksi] = ((ks0 + ksi) * 32 + q * 8 < K) ? af[ksi] : zero;
            }
#pragma unroll
            for (int ksi = 0; ksi < kSlabSteps; ++ksi) {
                if (ksi < nks) {
                    const unsigned char *blk = lds + (ksi * nt) * kLdsBlockBytes + lane * 16;
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        if (t < nt) {
                            const u32x4 bf = *reinterpret_cast<const u32x4 *>(blk + t * kLdsBlockBytes);
                            acc[t] = Elem<DT>::mfma(bf, af[ksi], acc[t]);
                        }
                    }
                }
            }
        }
    }
    if (!active) return;
    float factor = 1.f;
    if (FUSED) {
        float c = a.scale * kLog2e;
        prepare_scores<NT>(acc, nt, N, 0, c);
        float m, l;
        local_softmax<NT>(acc, nt, c, m, l);
        factor = 1.f / l;
    }
    store_rows<DT, NT, F32OUT>(acc, nt, s, a.out, r0, 0, factor);
}

template <int DT, bool FUSED, bool F32OUT, int MAXNT>
__device__ __forceinline__ void strips_from_lds_dispatch(int nt, const Seg &s, const RunArgs &a, unsigned char *lds,
                                                         int lds_blocks, int r0, bool active, int wave, int nwaves) {
    if (nt <= 1) strips_from_lds<DT, 1, FUSED, F32OUT, MAXNT>(s, a, lds, lds_blocks, r0, active, wave, nwaves);
    else if (nt <= 2) strips_from_lds<DT, 2, FUSED, F32OUT, MAXNT>(s, a, lds, lds_blocks, r0, active, wave, nwaves);
    else if (nt <= 4) strips_from_lds<DT, 4, FUSED, F32OUT, MAXNT>(s, a, lds, lds_blocks, r0, active, wave, nwaves);
    else if (nt <= 8 || MAXNT <= 8) strips_from_lds<DT, 8, FUSED, F32OUT, MAXNT>(s, a, lds, lds_blocks, r0, active, wave, nwaves);
    else strips_from_lds<DT, 16, FUSED, F32OUT, MAXNT>(s, a, lds, lds_blocks, r0, active, wave, nwaves);
}


// ------------------------------------------------------------ exact strips
// The strip path for segments whose whole B_g fits the LDS window
// (G * ceil(K/32) <= kFastBlocks blocks with G = the even tile count, K <= 128,
// N >= 2): code specialised for the tile count, no per-tile conditions, B_g
// copied to LDS once per workgroup and reused by every strip the workgroup takes.
//
// Layout.  The MFMA takes the strip's A rows as its first operand and B_g rows as
// its second, so a lane holds four ROWS of one column slot.  Both operand orders
// are free, and they are chosen so that memory order follows lane order:
//   * column slot j of tile g is score column G*j + g, so lane j owns the G
//     CONSECUTIVE columns [G*j, G*j + G) of each of its rows (register index = g);
//   * operand row slot m is strip row 4*(m%4) + m/4, so register e of the lanes of
//     row group rg (= lane/16) is strip row 4*e + rg: one store instruction (fixed
//     e) covers the four consecutive strip rows 4e..4e+3, lane after lane, i.e. one
//     contiguous run of 4*N elements of the output.
// Adjacent lanes write adjacent addresses, which is what the memory pipeline
// coalesces; a lane%16 = row layout writes 16 scattered pieces per instruction
// and runs at a fraction of the store rate.
// Ragged N: lanes j < J = N/G own full runs; if v = N - G*J > 0, lane J owns the
// run [N-G, N) instead, overlapping lane J-1 in G-v columns (both lanes compute and
// store identical values there); later lanes repeat column N-1 and store nothing.
// Every store is a full run: there are no partial stores.  The row sum weights each
// value by 1 or 0 (w[g]) so overlapped and repeated columns count once; the row
// maximum needs no mask at all.

//
// B_g in LDS, two layouts.  NAT = 0 (any K <= 128): blocks in MFMA operand order, filled by lanes that
// each fetch the 16 bytes they will read (conflict-free linear reads; the fill gathers 64-byte pieces
// of rows G apart).  NAT = 1 (K = 64) and NAT = 2 (K = 128): B_g as it lies in memory, so the fill is a
// straight coalesced copy; inside every 256-byte window (two rows, or one) the sixteen 16-byte pieces
// are XOR-permuted by the column slot j = row / G their rows belong to, and since the sixteen lanes
// that read one operand together hold the same piece of rows G apart, i.e. of sixteen different slots
// j, they fall into sixteen different bank groups.  The run [N-G, N) of the lane at the ragged end
// (and of the lanes after it) is copied once more, unpermuted, behind the image and read from there.
// SOLO: the calling wavefront has the segment and the LDS it is given to itself (a mini segment, see mini_shape):
// it fills alone, waits for its own loads and passes no barrier, so the wavefronts of a workgroup can work on
// different segments, each in its own code.
template <int DT, int G, bool FUSED, bool F32OUT, int NAT, bool SOLO = false>
__device__ __forceinline__ void strips_exact(const Seg &s, const RunArgs &a, unsigned char *lds, int wave_in,
                                             int first_strip, int strip_step) {
    constexpr int kFillWaves = SOLO ? 1 : kSegWaves;
    const int wave = SOLO ? 0 : wave_in;
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int K = s.K, N = s.N, M = s.M;
    const int nks = (K + 31) >> 5;
    const int strips = (M + kStripRows - 1) / kStripRows;
    const SegRes res = make_res(s, a.A, a.B);
    const u32x4 zero = {0u, 0u, 0u, 0u};

    // ---- this lane's run of columns
    const int J = N / G, v = N - G * J;
    const bool owner = j < J || (j == J && v > 0);
    const int col0 = j < J ? G * j : N - G;                 // first column of the run (owners)

    // ---- this wavefront's first A fragments: operand row slot j is strip row 4*(j%4) + j/4,
    //      k-group rg; rows past M read as zeros (buffer range)
    const int a_lane = ((4 * (j & 3) + (j >> 2)) * K + rg * 8) * 2;
    u32x4 af[kFastSteps];
    auto load_a = [&](int strip) {
        const int voff = a_lane + strip * (kStripRows * 2) * K;
#pragma unroll
        for (int ks = 0; ks < kFastSteps; ++ks)
            if (ks < nks) af[ks] = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff + ks * 64, 0, 0);
    };
    load_a(first_strip);

    // per (column tile g, k-step ks) the operand of this lane is read at vb[variant] + immediate
    const unsigned char *vb[4];
    if constexpr (NAT == 0) {
        // ---- B_g -> LDS, block (ks, g) at (ks * G + g) KiB, in MFMA operand order:
        //      lane (slot j, k-group rg) brings 16 bytes of B_g row col0 + g
        const uint16_t *bseg = (const uint16_t *)a.B + s.b;
        const int brow0 = owner ? col0 : N - 1;
        const int bstep = owner ? 1 : 0;
        const int nblocks = nks * G;
        for (int b = wave; b < nblocks; b += kFillWaves) {
            const int ks = b / G, g = b - ks * G;
            const int row = brow0 + bstep * g;
            int kk = ks * 32 + rg * 8;
            kk = kk < K ? kk : 0;            // ragged last k-step: valid data, multiplied by a zero A fragment
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(bseg + row * K + kk),
                                             (__attribute__((address_space(3))) void *)(lds + b * kLdsBlockBytes),
                                             16, 0, 0);
        }
        vb[0] = vb[1] = vb[2] = vb[3] = lds + lane * 16;
    } else {
        // ---- B_g -> LDS as it lies in memory: position p (16-byte pieces) of the image takes piece
        //      (p & ~15) | ((p & 15) ^ key) of B_g, key = column slot of the window's rows
        constexpr int kPieces = NAT == 1 ? 8 : 16;              // 16-byte pieces per row of B_g
        const uint16_t *bseg = (const uint16_t *)a.B + s.b;
        // Every instruction runs with all 64 lanes (1 KiB of LDS each): lanes past the end of B_g fetch its
        // last piece into positions nobody reads, so the image takes whole KiB and the copy of the ragged
        // run starts on the next KiB.
        const int total = N * kPieces, padded = (total + 63) & ~63;
        for (int p0 = wave * 64; p0 < padded; p0 += kFillWaves * 64) {
            const int p = p0 + lane, w = p >> 4;
            const int key = ((NAT == 1 ? 2 * w : w) / G) & 15;
            const int piece = min((p & ~15) | ((p & 15) ^ key), total - 1);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(bseg + piece * 8),
                                             (__attribute__((address_space(3))) void *)(lds + p0 * 16), 16, 0, 0);
        }
        unsigned char *tail = lds + padded * 16;
        const int tail_pieces = G * kPieces;
        const int tail_key = J & 15;         // no lane with a full run uses this key: the copy's readers collide with none
        for (int p0 = wave * 64; p0 < tail_pieces; p0 += kFillWaves * 64) {
            const int q = p0 + lane;
            const int p = min((q & ~15) | ((q & 15) ^ tail_key), tail_pieces - 1);
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void *)(bseg + ((N - G) * kPieces + p) * 8),
                (__attribute__((address_space(3))) void *)(tail + p0 * 16), 16, 0, 0);
        }
        // rows of this lane: G*j + g in the image (full runs), or g of the copy of the last G rows
        const bool full = j < J;
        const unsigned char *base = full ? lds + (NAT == 1 ? 128 : 256) * (G * j) : tail;
        const int kj = full ? j : tail_key;
#pragma unroll
        for (int c = 0; c < 4; ++c) vb[c] = base + 64 * (c ^ (kj >> 2)) + 16 * (rg ^ (kj & 3));
    }
    // weights of the row sum: 1 for columns this lane alone accounts for
    float w[G];
    if (FUSED) {
#pragma unroll
        for (int g = 0; g < G; ++g) w[g] = (j < J || (j == J && g >= G - v)) ? 1.f : 0.f;
    }
    __builtin_amdgcn_s_waitcnt(0);
    if constexpr (!SOLO) __syncthreads();

    // address of the operand of column tile g, k-step ks (g, ks: unrolled constants)
    auto operand = [&](int g, int ks) -> const unsigned char * {
        if constexpr (NAT == 0) return vb[0] + (ks * G + g) * kLdsBlockBytes;
        else if constexpr (NAT == 1) return vb[(g & 1) * 2 + ks] + 256 * (g >> 1);
        else return vb[ks] + 256 * g;
    };
    const bool ragged_k = (K & 31) != 0;
    const bool k_live = (nks - 1) * 32 + rg * 8 < K;
    // A negative softmax scale is applied as |scale| to negated scores: the sign bits of the A
    // fragments are flipped, so the row maximum below is always the value to subtract.
    const float c_signed = a.scale * kLog2e;
    const bool negate = FUSED && c_signed < 0.f;
    const float c = __builtin_fabsf(c_signed);
    constexpr int kOutBytes = F32OUT ? 4 : 2;
    char *const obase = reinterpret_cast<char *>(a.out) + s.o * kOutBytes;
    const uint32_t run_off = (uint32_t)(rg * N + col0) * kOutBytes;

    for (int strip = first_strip; strip < strips; strip += strip_step) {
        // The operands of B_g are the same for every strip; left alone, the compiler keeps all of them in
        // registers across the loop and spills.  They are cheap to read again: make it.
        asm volatile("" ::: "memory");
        if (ragged_k) {
#pragma unroll
            for (int ks = 0; ks < kFastSteps; ++ks)
                if (ks == nks - 1) af[ks] = k_live ? af[ks] : zero;
        }
        if (negate) {
#pragma unroll
            for (int ks = 0; ks < kFastSteps; ++ks)
                if (ks < nks) af[ks] ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
        }
        f32x4 acc[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const u32x4 bf = *reinterpret_cast<const u32x4 *>(operand(g, 0));
            acc[g] = Elem<DT>::mfma(af[0], bf, f32x4{0.f, 0.f, 0.f, 0.f});
        }
#pragma unroll
        for (int ks = 1; ks < kFastSteps; ++ks) {
            if (ks < nks) {
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const u32x4 bf = *reinterpret_cast<const u32x4 *>(operand(g, ks));
                    acc[g] = Elem<DT>::mfma(af[ks], bf, acc[g]);
                }
            }
        }
        load_a(strip + strip_step);          // next strip's fragments fly under the softmax and the stores

        if (FUSED) softmax_lane_runs<G>(acc, w, c);

        if (owner) {
            const int r0 = strip * kStripRows;
            char *dst = obase + (size_t)r0 * N * kOutBytes + run_off;
            const int row_stride4 = 4 * N * kOutBytes;
            if (r0 + kStripRows <= M) {
#pragma unroll
                for (int e = 0; e < 4; ++e) store_run<DT, G, F32OUT>(dst + e * row_stride4, acc, e);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (r0 + 4 * e + rg < M) store_run<DT, G, F32OUT>(dst + e * row_stride4, acc, e);
            }
        }
    }
}

template <int DT, bool FUSED, bool F32OUT, int MAXNT>
__device__ __forceinline__ void strips_exact_dispatch(int tiles, const Seg &s, const RunArgs &a, unsigned char *lds,
                                                      int wave, int first_strip, int strip_step) {
    // Bytes the in-memory image of B_g takes: whole KiB for the image and for the copy of the last G rows.
    const int pieces = s.N * (s.K >> 3);
    const bool image_fits =
        (((pieces + 63) & ~63) + ((tiles * (s.K >> 3) + 63) & ~63)) * 16 <= a.lds_blocks * kLdsBlockBytes + a.lds_extra;
#define BA_EXACT(G_)                                                                                              \
    case G_:                                                                                                      \
        if (s.K == 64 && image_fits)                                                                              \
            strips_exact<DT, G_, FUSED, F32OUT, 1>(s, a, lds, wave, first_strip, strip_step);                     \
        else if (s.K == 128 && image_fits)                                                                        \
            strips_exact<DT, G_, FUSED, F32OUT, 2>(s, a, lds, wave, first_strip, strip_step);                     \
        else strips_exact<DT, G_, FUSED, F32OUT, 0>(s, a, lds, wave, first_strip, strip_step);                    \
        break;
    switch (tiles) {
        BA_EXACT(2) BA_EXACT(4) BA_EXACT(6) BA_EXACT(8)
        default:
            if (MAXNT > 8) {
                switch (tiles) {
                    BA_EXACT(10) BA_EXACT(12) BA_EXACT(14) BA_EXACT(16)
                    default: break;
                }
            }
            break;
    }
#undef BA_EXACT
}

// One wavefront, one mini segment, `lds` = the wavefront's own kMiniBlocks KiB.
template <int DT, bool FUSED, bool F32OUT>
__device__ __forceinline__ void strips_solo_dispatch(int tiles, const Seg &s, const RunArgs &a, unsigned char *lds) {
    const int pieces = s.N * (s.K >> 3);
    const bool image_fits = (((pieces + 63) & ~63) + ((tiles * (s.K >> 3) + 63) & ~63)) * 16 <= kMiniBlocks * kLdsBlockBytes;
#define BA_SOLO(G_)                                                                                        \
    case G_:                                                                                               \
        if (s.K == 64 && image_fits) strips_exact<DT, G_, FUSED, F32OUT, 1, true>(s, a, lds, 0, 0, 1);     \
        else if (s.K == 128 && image_fits) strips_exact<DT, G_, FUSED, F32OUT, 2, true>(s, a, lds, 0, 0, 1); \
        else strips_exact<DT, G_, FUSED, F32OUT, 0, true>(s, a, lds, 0, 0, 1);                             \
        break;
    switch (tiles) {
        BA_SOLO(2) BA_SOLO(4) BA_SOLO(6) BA_SOLO(8)
        default: break;
    }
#undef BA_SOLO
}

// ------------------------------------------------------------------ kernels
// segment_kernel   grid (segment, head, z): one workgroup per segment and head;
//                  its wavefronts take the segment's 16-row strips (N <= 256),
//                  the pack it leads, or its rows on the element-wise path.
//                  No search: the block index is the segment.
// gemm_large_kernel  GEMM only, N > 256: one wavefront per 16 x 256 piece, found
//                  by a search in the scanned piece counts.
// split_kernel / wide_kernel  fused, N > 256: one 16-wave workgroup per strip.
// The list kernels loop `for (item = first; item < total; item += stride)` with
// the total read from the plan, so any grid size is correct.

// MAXNT = 8 is the build for batches whose widest segment has N <= 128: half the
// accumulator registers, half again as many resident wavefronts.  The host picks it from
// the plan summary; without a summary the 16-tile build runs.
template <int DT, bool FUSED, bool F32OUT, int MAXNT>
__global__ __launch_bounds__(kSegThreads, MAXNT <= 8 ? 6 : 4) void segment_kernel(RunArgs a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const int64_t h = blockIdx.y;
    const bool ok = header_ok(a);
    bool valid;
    const Seg s = load_listed(pv, blockIdx.x, h, a, valid);
    if (!ok) {
        if (!(a.flags & kFlagQuiet)) report_mismatch(a);
        return;
    }
    if (!valid) return;
    const int g = s.index;
    const int kind = s.kind;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int first = blockIdx.z * kSegWaves + wave, stride = gridDim.z * kSegWaves;
    const bool mfma_ok = (a.flags & kFlagMfmaOk) != 0;
    if (kind == kSegEmpty) return;
    if (mfma_ok && a.list < 0 && launch_class(kind, s.M, s.N, s.K) != kListRest) return;   // another kernel's
    if (!mfma_ok || kind == kSegSlow) {
        // Element-wise path.  With MFMA ruled out for the whole launch this also
        // covers the segments the list kernels would have taken.
        for (int r = first; r < s.M; r += stride) generic_seg_rows<DT, FUSED>(s, a, r, r + 1, 0, s.N);
        return;
    }
    if (kind == kSegStrip) {
        // One strip per wavefront; blockIdx.z selects the group of kSegWaves strips.
        const int strips = (s.M + kStripRows - 1) / kStripRows;
        const int nt = (s.N + 15) >> 4;
        for (int base = blockIdx.z * kSegWaves; base < strips; base += gridDim.z * kSegWaves) {
            if (base != (int)blockIdx.z * kSegWaves) __syncthreads();    // LDS is refilled for the next group
            const int strip = base + wave;
            strips_from_lds_dispatch<DT, FUSED, F32OUT, MAXNT>(nt, s, a, lds, a.lds_blocks, strip * kStripRows,
                                                        strip < strips, wave, kSegWaves);
        }
    } else if (kind == kSegPackLead) {
        if (first == 0) wave_pack<DT, FUSED, F32OUT>(pv, g, s.packLen, h, a);
    }
}

// strip_kernel: the strip-class segments whose B_g fits the LDS window, nothing else.
// Grid (segment, head, z); the workgroups with the same (segment, head) share the
// segment's strips round-robin.
// RIDE: the build whose launch also carries the tile kernel's workgroups.  Its grid is flat: the first
// a.tile_groups blocks are tile workgroups (they run longest, so they start first), the rest decode to
// (slot, head, z) with the slot fastest.  Two launches that each fill half the machine become one.
template <int DT, bool FUSED, bool F32OUT, int MAXNT, bool RIDE = false>
__global__ __launch_bounds__(kSegThreads, MAXNT <= 8 ? 4 : 2) void strip_kernel(RunArgs a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    unsigned bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z, gz = gridDim.z;
    if (!RIDE && (a.flags & kFlagHeadFast)) { bx = blockIdx.y; by = blockIdx.x; }
    if constexpr (RIDE) {
        if (bx < (unsigned)a.tile_groups) {
            RunArgs ta = a;
            ta.list = kListTile;
            ta.flags |= kFlagQuiet;
            tile_block<DT, FUSED, F32OUT>(ta, a.tile_zdim, bx, lds);
            return;
        }
        const unsigned lin = bx - (unsigned)a.tile_groups;
        if (a.flags & kFlagHeadFast) {
            by = lin % (unsigned)a.H;
            bx = (lin / (unsigned)a.H) % (unsigned)a.ride_slots;
        } else {
            bx = lin % (unsigned)a.ride_slots;
            by = (lin / (unsigned)a.ride_slots) % (unsigned)a.H;
        }
        bz = lin / ((unsigned)a.ride_slots * (unsigned)a.H);
        gz = (unsigned)a.ride_z;
    }
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const int64_t h = by;
    if (a.mini_first > 0 && bx >= (unsigned)a.mini_first) {
        // The mini entries of the main list (kept at the end of its array, backwards): four to a workgroup, one
        // wavefront and a quarter of the 64 KiB window each, or one workgroup each where the window is smaller.
        const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
        const int count = hdr->mini_count;
        const bool ok = header_ok(a);
        const int wave = uniform((int)(threadIdx.x >> 6));
        const int k = a.mini_solo ? 4 * (int)(bx - (unsigned)a.mini_first) + wave : (int)(bx - (unsigned)a.mini_first);
        // header, count and record are fetched together (the record from a position that exists whatever k is)
        const int64_t cap = plan_cap(a.nseg);
        const SegRec r = load_rec(pv.recs + (int64_t)(kListSmall + 1) * cap, (int)(cap - 1 - min((int64_t)k, cap - 1)));
        if (!ok || k >= count || bz != 0) return;       // (a plan that does not match is reported by the launch's other blocks)
        Seg s;
        s.M = r.M; s.N = r.N; s.K = r.K;
        s.kind = r.kind; s.index = r.index; s.packLen = r.packLen;
        s.a = h * a.Dm1 + r.off1; s.b = h * a.Dm2 + r.off2; s.o = h * a.Dout + r.offO;
        const int tiles = fast_strip_tiles(s.N);
        if (s.kind != kSegStrip || !mini_shape(s.M, s.N, s.K) || tiles > MAXNT) return;
        if (a.mini_solo) strips_solo_dispatch<DT, FUSED, F32OUT>(tiles, s, a, lds + wave * (kMiniBlocks * kLdsBlockBytes));
        else if (strip_blocks(s.N, s.K) <= a.lds_blocks)
            strips_exact_dispatch<DT, FUSED, F32OUT, MAXNT>(tiles, s, a, lds, wave, wave, kSegWaves);
        return;
    }
    if ((a.flags & kFlagSmallToo) && bx >= (unsigned)a.both_split) {
        bx -= (unsigned)a.both_split;
        a.list = kListSmall;
    }
    // header and record are fetched together; nothing waits on the header alone
    const bool ok = header_ok(a);
    bool valid;
    const Seg s = load_listed(pv, bx, h, a, valid);
    if (!ok) {
        if (!(a.flags & kFlagQuiet)) report_mismatch(a);
        return;
    }
    if (!valid) {
        // Blocks behind the kernel's own list: with kFlagPacksToo they take the packs of tiny segments
        // (the rest list then holds nothing but pack leaders), which saves the call a launch.
        if (a.flags & kFlagPacksToo) {
            const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
            const int slot = (int)bx - (int)hdr->totals[a.list], packs = (int)hdr->totals[kListRest];
            if (slot >= 0 && slot < packs && bz == 0 && threadIdx.x < 64) {
                const SegRec r = load_rec(pv.recs + (int64_t)(kListRest + 1) * plan_cap(a.nseg), slot);
                if (r.kind == kSegPackLead) wave_pack<DT, FUSED, F32OUT>(pv, r.index, r.packLen, h, a);
            }
        }
        return;
    }
    const int tiles = fast_strip_tiles(s.N);
    const int need = strip_blocks(s.N, s.K);
    // the lists hold only segments of this kernel; the checks guard against a launch that does not match
    if ((s.kind != kSegStrip) | (need < 1) | (need > a.lds_blocks) | (tiles > MAXNT)) return;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int first = bz * kSegWaves + wave, step = gz * kSegWaves;
    if ((int)bz * kSegWaves * kStripRows >= s.M) return;   // no strip for this workgroup
    strips_exact_dispatch<DT, FUSED, F32OUT, MAXNT>(tiles, s, a, lds, wave, first, step);
}

// --------------------------------------------------------------------- host
// With a host copy of the plan summary the grids cover the work exactly and
// kernels with nothing to do are not launched; without it every kernel is
// launched with a generous grid and reads the counts from the plan.
static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// One call = up to four launches, each walking its own work list of the plan:
//   strip kernel    strip-class segments whose B_g fits its LDS window (main launch: up to 32 KiB;
//                   second launch: up to 64 KiB, fewer resident workgroups)
//   tile kernel     large segments (see tile_segment())
//   segment kernel  packs, the element-wise class, and what the others leave
// With a host copy of the plan summary the grids are exactly the list lengths, empty lists are not
// launched, and launches are merged where that saves one: the packs ride in the first strip launch
// when the rest list holds nothing else, and a modest amount of tile-kernel work rides in the 64 KiB
// strip launch.  Without the summary every kernel is launched over nseg slots and reads its list
// length from the plan.
// The first launch reports a plan that does not match the call; the later ones stay quiet.
template <int DT, bool FUSED, bool F32OUT>
static int launch_set(int dtype, const RunArgs &args_in, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args_in.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    const int cus = device_cu_count();
    const bool mfma_ok = args_in.flags & kFlagMfmaOk;
    const unsigned H = (unsigned)args_in.H;
    if (info) nseg = info->nseg;
    if (nseg <= 0) return BA_OK;
    RunArgs args = args_in;
    const int64_t n_small = !mfma_ok ? 0 : info ? info->list_small : nseg;
    const int64_t n_big = !mfma_ok ? 0 : info ? info->list_big : nseg;
    const int64_t n_tile = !mfma_ok ? 0 : info ? info->list_tile : nseg;
    const int64_t n_rest = !mfma_ok ? nseg : info ? info->list_rest : nseg;
    const int64_t n_mini = !mfma_ok ? 0 : info ? info->list_mini : nseg;    // part of the main strip list, kept apart
    const bool lean = info && info->max_N <= 128;
    // z: enough workgroups to fill the machine, at most one per kSegWaves strips of the tallest segment.  The
    // narrow build (up to eight column tiles, four to five workgroups resident per compute unit) aims at eight
    // workgroups per compute unit; the wide build holds two (64 KiB window) or three (registers), and one round of
    // resident workgroups that loop over their strips beats several rounds of short ones (non-square 512-segment
    // batch: 17.9 us with one workgroup per segment, 19.7 us with four).
    static const int z_env = [] { const char *e = getenv("BLOCKEDATTN_STRIP_Z"); return e ? atoi(e) : 0; }();
    auto strip_z = [&](int64_t slots, int64_t tallest, int per_cu) {
        if (z_env > 0) return (int64_t)z_env;
        if (!info) return (int64_t)2;
        const int64_t groups = ceil_div(ceil_div(std::max<int64_t>(tallest, 1), kStripRows), kSegWaves);
        const int64_t want = ceil_div((int64_t)cus * per_cu, std::max<int64_t>(1, slots * (int64_t)H));
        return std::max<int64_t>(1, std::min<int64_t>(groups, std::min<int64_t>(want, 64)));
    };
    // the rest list is nothing but pack leaders: the first strip launch takes them along
    const bool packs_ride = info && mfma_ok && n_rest > 0 && n_rest == info->pack_items && info->slow_items == 0 &&
                            (n_small > 0 || n_big > 0 || n_mini > 0);
    bool packs_taken = false;
    // a modest amount of tile-kernel work rides in the strip kernel's 64 KiB launch (same LDS, same
    // residency) instead of following it; large tile work keeps its own die-aware launch
    const int64_t tile_z = !info ? 1 : std::max<int64_t>(1, std::min<int64_t>(64, ceil_div(std::max<int64_t>(info->max_M, 1), kTileRows)));
    const int64_t tile_groups = ceil_div(n_tile, kDies) * kDies * (int64_t)H * tile_z;
    const bool tiles_ride = info && n_big > 0 && n_tile > 0 && tile_groups <= 4096 && (dtype == BA_F16 || dtype == BA_BF16);
    bool tiles_taken = false;
    // Both strip lists go in ONE launch with the 64 KiB window, the 64 KiB segments first, where two launches
    // would each be bound by the life of a workgroup rather than by how many are resident: when the main
    // launch's list holds wide segments (more than eight column tiles: three workgroups per compute unit by
    // registers, against two in the 64 KiB launch), or when the batch is small (measured: the non-square
    // 512-segment batch 23.6 -> 19.4 us, the power-law batch 51.2 -> 49.9 us).
    static const int merge_env = [] { const char *e = getenv("BLOCKEDATTN_MERGE_STRIPS"); return e ? atoi(e) : -1; }();
    const bool merge = info && n_small > 0 && n_big > 0 &&
                       (merge_env >= 0 ? merge_env != 0 : info->small_max_N > 128 || (n_small + n_big) * (int64_t)H <= 4096);
    // The mini entries ride in ONE of the strip launches: the merged one, else the main launch if it has entries
    // of its own, else the 64 KiB launch, else a main launch for them alone.
    const int mini_pass = n_mini <= 0 ? -1 : merge ? 1 : n_small > 0 ? 0 : n_big > 0 ? 1 : 0;
    static const int solo_env = [] { const char *e = getenv("BLOCKEDATTN_MINI_SOLO"); return e ? atoi(e) : 1; }();
    for (int pass = 0; pass < 2; ++pass) {
        int64_t slots = pass == 0 ? n_small : n_big;
        if ((slots <= 0 && pass != mini_pass) || (merge && pass == 0)) continue;
        RunArgs fa = args;
        if (merge) {
            fa.flags |= kFlagSmallToo;
            fa.both_split = (int)n_big;
            slots += n_small;
        }
        if (packs_ride && !packs_taken) {
            fa.flags |= kFlagPacksToo;
            slots += n_rest;
            packs_taken = true;
        }
        const bool ride = pass == 1 && tiles_ride;
        if (ride) {
            fa.flags |= kFlagTilesToo;
            fa.tile_zdim = (int)tile_z;
            fa.tile_groups = (int)tile_groups;
            fa.ride_slots = (int)slots;
            fa.ride_z = (int)strip_z(slots, info->max_M, 2);
            tiles_taken = true;
        }
        fa.list = pass == 0 ? kListSmall : kListBig;
        fa.lds_blocks = pass == 0 ? kFastBlocks : kBigBlocks;
        bool lean_pass = lean;
        if (info && pass == 0 && !merge) {
            // the main launch is sized by ITS widest and tallest segment, not the batch's
            const int64_t nt = fast_strip_tiles((int)std::max(info->small_max_N, 1));
            const int64_t nks = ceil_div(std::max<int64_t>(info->max_K, 1), 32);
            fa.lds_blocks = (int)std::min<int64_t>(kFastBlocks, nt * nks);
            lean_pass = info->small_max_N <= 128;
        }
        if (pass == mini_pass) {
            // four mini segments to a workgroup where the window has a quarter for each of them
            fa.mini_first = (int)std::max<int64_t>(slots, 1);
            fa.mini_solo = solo_env && info && fa.lds_blocks >= 4 * kMiniBlocks ? 1 : 0;
            slots = fa.mini_first + (fa.mini_solo ? ceil_div(n_mini, kSegWaves) : n_mini);
            if (ride) fa.ride_slots = (int)slots;
        }
        const int64_t tallest = !info ? 0 : pass == 0 ? info->small_max_M : info->max_M;
        const dim3 grid((unsigned)slots, H, (unsigned)strip_z(slots, tallest, lean_pass ? 8 : pass == 0 ? 3 : 2));
        // room for the copy of the ragged run behind the image of B_g, while the total stays within 64 KiB
        fa.lds_extra = fa.lds_blocks * kLdsBlockBytes + kRaggedCopyBytes <= 65536 ? kRaggedCopyBytes : 0;
        const size_t lds_bytes = (size_t)fa.lds_blocks * kLdsBlockBytes + fa.lds_extra;
        // Head as the fastest index of the grid: consecutive workgroups are the heads of one list entry, so
        // workgroups that start together have one shape and take equally long, and (with the list in work
        // buckets) the longest start first.  Measured against entry-fastest order: 256 x 8 heads fused 15.6 ->
        // 14.9 us, GEMM only 15.5 -> 13.6 us; power-law batch fused 49.3 -> 46.7 us.
        static const int hf = [] { const char *e = getenv("BLOCKEDATTN_HEAD_FAST"); return e ? atoi(e) : 1; }();
        const bool head_fast = hf && (ride || slots <= 65535);      // heads on gridDim.x, entries on gridDim.y
        if (head_fast) fa.flags |= kFlagHeadFast;
        const dim3 grid_hf(H, (unsigned)slots, grid.z);
        if (ride)
            hipLaunchKernelGGL((strip_kernel<DT, FUSED, F32OUT, 16, true>),
                               dim3((unsigned)(tile_groups + slots * (int64_t)H * fa.ride_z)), dim3(kSegThreads), lds_bytes,
                               stream, fa);
        else if (lean_pass)
            hipLaunchKernelGGL((strip_kernel<DT, FUSED, F32OUT, 8>), head_fast ? grid_hf : grid, dim3(kSegThreads), lds_bytes,
                               stream, fa);
        else
            hipLaunchKernelGGL((strip_kernel<DT, FUSED, F32OUT, 16>), head_fast ? grid_hf : grid, dim3(kSegThreads), lds_bytes,
                               stream, fa);
        args.flags |= kFlagQuiet;
    }
    if (n_tile > 0 && !tiles_taken) {
        RunArgs ta = args;
        ta.list = kListTile;
        const int st = launch_tiles(dtype, FUSED ? 1 : 0, ta, n_tile, info, stream);
        if (st != BA_OK) return st;
        args.flags |= kFlagQuiet;
    }
    if (n_rest > 0 && !packs_taken) {
        // z spreads the 16-row strips (or rows) of the largest segment over workgroups
        int64_t z = 4, blocks = 32;
        if (info) {
            const int64_t units = mfma_ok && info->slow_items == 0 ? ceil_div(std::min<int64_t>(info->max_M, 256), kStripRows)
                                                                     : std::min<int64_t>(info->max_M, 4096);
            z = std::max<int64_t>(1, std::min<int64_t>(64, ceil_div(units, kSegWaves)));
            // LDS window for B_g: whole B_g of the largest strip-class segment if it fits 64 KiB
            const int64_t nt = ceil_div(std::min<int64_t>(std::max<int64_t>(info->max_N, 1), kWaveCols), 16);
            const int64_t nks = ceil_div(std::max<int64_t>(info->max_K, 1), 32);
            blocks = std::max<int64_t>(nt, std::min<int64_t>(nt * nks, 64));
        }
        RunArgs seg_args = args;
        seg_args.list = mfma_ok ? kListRest : -1;
        seg_args.lds_blocks = (int)blocks;
        const dim3 grid((unsigned)n_rest, H, (unsigned)z);
        const size_t lds_bytes = (size_t)blocks * kLdsBlockBytes;
        if (lean)
            hipLaunchKernelGGL((segment_kernel<DT, FUSED, F32OUT, 8>), grid, dim3(kSegThreads), lds_bytes, stream,
                               seg_args);
        else
            hipLaunchKernelGGL((segment_kernel<DT, FUSED, F32OUT, 16>), grid, dim3(kSegThreads), lds_bytes, stream,
                               seg_args);
    }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_strips(int dtype, int fused, const RunArgs &args, int64_t nseg, const ba_plan_info *info,
                  hipStream_t stream) {
    const bool f32out = args.flags & kFlagOutF32;
    if (dtype == BA_F16) {
        if (!fused) return launch_set<0, false, false>(dtype, args, nseg, info, stream);
        return f32out ? launch_set<0, true, true>(dtype, args, nseg, info, stream)
                      : launch_set<0, true, false>(dtype, args, nseg, info, stream);
    }
    if (dtype == BA_BF16) {
        if (!fused) return launch_set<1, false, false>(dtype, args, nseg, info, stream);
        return f32out ? launch_set<1, true, true>(dtype, args, nseg, info, stream)
                      : launch_set<1, true, false>(dtype, args, nseg, info, stream);
    }
    return BA_ERR_UNSUPPORTED;
}

}  // namespace ba
