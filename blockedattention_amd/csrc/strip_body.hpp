// Device bodies of the kernels for segments of up to 256 columns: operand loads, the softmax of a 16-row strip
// held in registers, the strip loops over an LDS image of B_g (strips_exact, strips_from_lds), packs of tiny
// segments (wave_pack) and the element-wise path (generic_rows).  Included by the kernels that run them.
#pragma once
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
            store_result<false>(reinterpret_cast<f32x4_unaligned *>(o), v);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (i < valid) o[i] = v[i];
        }
    } else {
        uint16_t *o = reinterpret_cast<uint16_t *>(out) + e;
        if (valid >= 4) {
            store_result<false>(reinterpret_cast<u32x2_unaligned *>(o), u32x2{Elem<DT>::pack2(v[0], v[1]), Elem<DT>::pack2(v[2], v[3])});
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
// STRAIGHT: no branch around a load or a store of the strip loop (loads of k-steps the segment does not have and
// stores of rows and lanes that have nothing to write go outside their descriptor's range instead), so that the
// wait in front of the next strip's first matrix instruction counts this strip's stores as still in flight; with
// the branches the compiler waits for every vector memory operation there.  Measured on one box: 512 segments of
// 16..256 rows and columns 16.5 -> 15.0 us (GEMM only 13.4 -> 12.3), the power-law batch 39.4 -> 37.8 us, but
// 256 segments x 8 heads of 32..128 rows (the narrow build) 14.6 -> 15.6 us: the narrow build keeps the branches.
template <int DT, int G, bool FUSED, bool F32OUT, int NAT, bool SOLO = false, bool STRAIGHT = true>
__device__ __forceinline__ void strips_exact(const Seg &s, const RunArgs &a, unsigned char *lds, int wave_in,
                                             int first_strip, int strip_step) {
    constexpr int kFillWaves = SOLO ? 1 : kSegWaves;
    const int wave = SOLO ? 0 : wave_in;
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int K = s.K, N = s.N, M = s.M;
    const int nks = (NAT && STRAIGHT) ? 2 * NAT : (K + 31) >> 5;    // (the in-memory layouts are those of K = 64 and K = 128)
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
    // (STRAIGHT: a k-step the segment does not have reads outside the descriptor's range, i.e. zeros without touching memory)
    auto load_a = [&](int strip) {
        const int voff = a_lane + strip * (kStripRows * 2) * K;
#pragma unroll
        for (int ks = 0; ks < kFastSteps; ++ks) {
            if constexpr (STRAIGHT) {
                if (!NAT || ks < 2 * NAT)
                    af[ks] = __builtin_amdgcn_raw_buffer_load_b128(res.a, ks < nks ? voff + ks * 64 : (int)0x80000000, 0, 0);
            } else {
                if (ks < nks) af[ks] = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff + ks * 64, 0, 0);
            }
        }
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
    // Results leave through a descriptor that spans exactly the rows of the strip: a row past M, and every row of a
    // lane that owns no run (offset 2^31), is dropped by the range check, not by a branch.
    const uint32_t run_off = (owner || !STRAIGHT) ? (uint32_t)(rg * N + col0) * kOutBytes : 0x80000000u;
    const uint32_t row_stride4 = (uint32_t)(4 * N * kOutBytes);

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

        const int r0 = strip * kStripRows;
        if constexpr (STRAIGHT) {
            const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(obase + (size_t)r0 * N * kOutBytes), 0, min(kStripRows, M - r0) * N * kOutBytes, kRsrcFlags);
#pragma unroll
            for (int e = 0; e < 4; ++e) store_run_buf<DT, G, F32OUT>(ores, run_off + e * row_stride4, acc, e);
        } else if (owner) {
            char *dst = obase + (size_t)r0 * N * kOutBytes + run_off;
            if (r0 + kStripRows <= M) {
#pragma unroll
                for (int e = 0; e < 4; ++e) store_run<DT, G, F32OUT, true>(dst + e * row_stride4, acc, e);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (r0 + 4 * e + rg < M) store_run<DT, G, F32OUT, true>(dst + e * row_stride4, acc, e);
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
            strips_exact<DT, G_, FUSED, F32OUT, 1, false, (MAXNT > 8)>(s, a, lds, wave, first_strip, strip_step); \
        else if (s.K == 128 && image_fits)                                                                        \
            strips_exact<DT, G_, FUSED, F32OUT, 2, false, (MAXNT > 8)>(s, a, lds, wave, first_strip, strip_step); \
        else strips_exact<DT, G_, FUSED, F32OUT, 0, false, (MAXNT > 8)>(s, a, lds, wave, first_strip, strip_step); \
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

}  // namespace ba
