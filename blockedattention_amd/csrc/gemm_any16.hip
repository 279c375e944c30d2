// fp16 / bf16 varlen GEMM on the matrix instruction for the calls the strip and tile kernels do not take: operands
// stored K x M or K x N (the reference's transpose flags, csrc/cuda/spBlkGEMM.cu:311-329, 382-400), reduction
// lengths that are not multiples of 8, segments that start at odd elements, base pointers without 16-byte
// alignment.  The backward of the product is two such calls (csrc/sparseBlockedAttention.cpp:52-72: dA = dS B
// reduces over N, dB = dS^T A over M, with dS and the saved operands read as they lie).
//
// Workgroup = 128 rows x 128 columns of one segment and head at a time (64 x 64 in the build for batches of short
// segments), k in chunks of 64.  Both operand chunks go through LDS with a row pitch of 160 bytes (288 for 128 rows
// stored k-major).  Staging reads 16 bytes per lane along whatever dimension is contiguous
// in memory, at any 2-byte alignment, through a buffer descriptor that spans exactly the segment (rows past its
// end read as zeros), and writes them to LDS as they come: an operand that is not transposed lies there as
// [row][k] and is read 16 bytes per lane; an operand stored k-major lies there k-major and the matrix operand is
// gathered by the transposing LDS read (ds_read_b64_tr_b16, four k of one row per lane).  Each wavefront
// then computes 16 or 32 rows x 64 or 128 columns as 16 x 16 tiles with v_mfma_f32_16x16x32 (fp32 sums).  Column slot n of
// tile t is column 4 n + t (8 n + t in the 128-column step), so a lane owns four (eight) consecutive columns of
// each of its rows and the sixteen lanes of a row group write 128 (256) contiguous bytes.
//
// What bounds it, measured on 16 segments x 16 heads of 1024..4096 rows and columns, K = 128, both operands k-major
// (rocprofv3 counters): the first pipelined build moved 4.7 GB in and 4.6 GB out of memory for 0.34 GB of operands
// and 3.86 GB of results and spent 56 % of its wave cycles in s_waitcnt.  Keeping the X chunks of a round in LDS
// (K <= 128) took the reads to 1.0 GB and the kernel from 1930 to 1660 us; the writes stayed at 1.18 x the result
// (rows start at any 2-byte phase, so every 256-byte piece ends in partial lines).  The ring kernel below writes whole
// lines instead: 1210 us, against 1000 us for the plain-layout kernel on the same batch.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "ba_gemm_common.hpp"

namespace ba {

constexpr int kAnyThreads = 256;
constexpr int kAnyTile = 64;                         // rows and columns per workgroup step, k per chunk
constexpr int kAnyPitch = (kAnyTile + 16) * 2;       // bytes per LDS row: 160 = 16 * (2 * odd), the pitch at which the
// 16-byte operand reads (served 32 lanes, 512 bytes at a time) and the transposing 8-byte reads meet no bank conflict

// Sixteen consecutive elements of the segment from byte offset `off` on (kNoLine: zeros).  Two 16-byte loads where
// they lie inside the segment; a piece that reaches past its end is fetched element by element, the hardware
// returning zero for those outside (a wide load that crosses the end of the descriptor's range is dropped whole).
constexpr int kDies = 8;
constexpr int kAnyDieBlock = 16;
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

// One chunk of an operand (R rows x 64 k, R = 16 * PARTS) on its way into LDS, in two steps so that the loads of
// later chunks can be in flight while the matrix instructions work on the current one.  The operand is `rows` x K
// (or, transposed, stored K x rows); the chunk starts at row r0, reduction index k0.  A chunk is 4 R slots of
// sixteen consecutive elements along the contiguous dimension: not transposed, slot s is k part s % 4 of row s / 4;
// transposed, row part s % PARTS of k line s / PARTS.  A thread takes the slots tid, tid + 256, ...
template <int PARTS>
__device__ __forceinline__ Line16 fetch_chunk16(__amdgpu_buffer_rsrc_t res, bool transposed, int rows, int K, int r0, int k0,
                                                int slot) {
    const int line = transposed ? slot / PARTS : slot >> 2, part = (transposed ? slot % PARTS : slot & 3) * 16;
    const uint32_t bytes = (uint32_t)(rows * K) * 2u;
    const int row = r0 + (transposed ? part : line), k = k0 + (transposed ? line : part);
    const int lead = transposed ? k * rows + row : row * K + k;
    return load_line16(res, row < rows && k < K ? (uint32_t)lead * 2u : kNoLine, bytes);
}
// Into LDS.  An operand that is not transposed lies as dst[row][k] (pitch kAnyPitch).  A transposed one stays
// k-major, dst[k][..] (pitch PITCH_T), and the matrix operand is gathered by transposing reads (lds_tr8 below):
// 16-byte writes here instead of sixteen 2-byte ones.  X (rows of the output) keeps its rows in order.  Y (columns
// of the output) permutes its columns so that the lane that reads position 16 t + i of a k line (slot i of tile t)
// gets the columns a lane stores side by side: column 4 i + t of a 64-column step (16 a + 4 b + t -> position
// 16 t + 4 a + b), column 8 i + t of a 128-column step.
template <bool PERMUTE, int PARTS, int PITCH_T>
__device__ __forceinline__ void put_chunk16(Line16 x, bool transposed, int rows, int K, int r0, int k0, unsigned char *dst,
                                            int slot) {
    const int line = transposed ? slot / PARTS : slot >> 2, part = (transposed ? slot % PARTS : slot & 3) * 16;
    const int valid = transposed ? rows - (r0 + part) : K - (k0 + part);   // elements of the line from here on
    if (valid < 16) {                                 // only the chunk at the end of the rows or of K
#pragma unroll
        for (int i = 0; i < 16; ++i) x.e[i] = i < valid ? x.e[i] : (uint16_t)0;
    }
    if (!transposed) {
        u32x4 *d = reinterpret_cast<u32x4 *>(dst + line * kAnyPitch + part * 2);
        d[0] = x.v[0];
        d[1] = x.v[1];
    } else if (!PERMUTE) {
        u32x4 *d = reinterpret_cast<u32x4 *>(dst + line * PITCH_T + part * 2);
        d[0] = x.v[0];
        d[1] = x.v[1];
    } else if (PARTS == 8) {
        // 128 columns: column 8 i + t -> position 16 t + i (eight tiles; a lane stores eight columns side by side)
        const uint32_t *w = reinterpret_cast<const uint32_t *>(&x);
        unsigned char *d = dst + line * PITCH_T + (part >> 4) * 4;
#pragma unroll
        for (int t = 0; t < 8; ++t) {                 // elements t and 8 + t of the thread's sixteen
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            *reinterpret_cast<uint32_t *>(d + 32 * t) = __builtin_amdgcn_perm(w[4 + (t >> 1)], w[t >> 1], sel);
        }
    } else {
        const uint32_t *w = reinterpret_cast<const uint32_t *>(&x);
        unsigned char *d = dst + line * PITCH_T + ((part >> 4) & 3) * 8;
#pragma unroll
        for (int t = 0; t < 4; ++t) {                 // elements t, 4 + t, 8 + t, 12 + t of the thread's sixteen
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            const uint32_t lo = __builtin_amdgcn_perm(w[2 + (t >> 1)], w[t >> 1], sel);
            const uint32_t hi = __builtin_amdgcn_perm(w[6 + (t >> 1)], w[4 + (t >> 1)], sel);
            *reinterpret_cast<u32x2 *>(d + 32 * t) = u32x2{lo, hi};
        }
    }
}
// Eight k of one row (column) of a k-major chunk as matrix operand: two transposing reads of four k each.  In a
// group of sixteen lanes, lane 4 e + a points at positions 4 a .. 4 a + 3 of k row e, and lane i receives position
// i of the four k rows; p is this lane's address for the first four k, the next four lie four rows on.
// The address is base + off with `off` a constant of the build: the base is turned into an LDS pointer first and the
// constant added to THAT, so that it lands in the instruction's offset field (added to the generic pointer it costs one
// address register per read, sixty-four of them kept across the step loop).
typedef __attribute__((address_space(3))) const unsigned char *LdsBytes;
__device__ __forceinline__ LdsBytes lds_bytes(const unsigned char *p) { return (LdsBytes)(uint32_t)(uintptr_t)p; }
template <int PITCH_T>
__device__ __forceinline__ u32x4 lds_tr8(LdsBytes base, int off) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 *LdsPtr;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(base + off));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(base + off + 4 * PITCH_T));
    const u32x2 l = __builtin_bit_cast(u32x2, lo), h = __builtin_bit_cast(u32x2, hi);
    return u32x4{l[0], l[1], h[0], h[1]};
}

// Workgroup barrier that waits for this wavefront's LDS traffic only: __syncthreads() would also wait for every
// global load in flight, i.e. for the chunks that were just requested for the NEXT steps.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// LDS bytes of one operand buffer holding R = 64 or 128 rows x 64 k in either layout
template <int R> struct AnyBuf {
    static constexpr int pitch_t = (R + 16) * 2;          // k-major: 160 or 288 bytes = 16 * (2 * odd)
    static constexpr int bytes = R * kAnyPitch > kAnyTile * pitch_t ? R * kAnyPitch : kAnyTile * pitch_t;
};

// Results through a ring (128 x 128 build, K <= 128, N >= 128).  A row of the result starts at any 2-byte phase, and
// a 128-byte line written in two partial pieces costs about 2.6 times a line written whole.  The X chunks of a round
// are needed in LDS only until every wavefront holds its A operands in registers; after that each wavefront owns half
// of an X buffer as a ring: one row of 128 columns (plus a copy of the first 16 behind them) per result row.  A
// block's columns go there as they lie in the registers (16-byte writes) and are read back shifted by the row's own
// phase, so that per row and 64 columns exactly ONE line-aligned 128-byte window leaves (eight lanes x 16 bytes,
// eight rows per store instruction); the window of a chunk lags the chunk by the row's phase and takes its first
// columns from the chunk before, which is still in the other half of the ring row.  The pieces at the two ends of
// a row that no window covers whole are written by one unaligned 16-byte store each (columns [0, 8) and [N-8, N);
// where pieces overlap they carry the same values).
constexpr int kAnyRingChunk = 64;                         // columns per window
constexpr int kAnyRingPitch = 288;                        // 128 columns + a copy of the first 16 behind them
constexpr int kAnyRingRows = 32;                          // rows per wavefront
constexpr int kAnyRingBytes = kAnyRingRows * kAnyRingPitch;
constexpr int kAnyRingStores = 4;                         // window stores per wavefront and chunk
constexpr uint32_t kAnyOutOfRange = 0x80000000u;          // byte offset no segment reaches (areas are below 2^31 bytes)
// whole lines leave: with the non-temporal hint they do not wait in L2 behind the launch's own write stream (16 segments
// x 16 heads of 1024..4096 rows, K = 128: 1209 us against 1542 with ordinary stores; the streaming round keeps
// ordinary stores for its partial lines, where the hint measured slower)
constexpr int kAnyRingAux = kResultAux;

// Sixteen bytes of a ring row starting at byte `pos` (any even value below 256): five aligned words, shifted.
__device__ __forceinline__ u32x4 any_ring_read16(const unsigned char *row, int pos) {
    const uint32_t *w = reinterpret_cast<const uint32_t *>(row + (pos & ~3));
    const uint32_t d0 = w[0], d1 = w[1], d2 = w[2], d3 = w[3], d4 = w[4];
    const uint32_t sh = (uint32_t)(pos & 2) * 8;
    return u32x4{__builtin_amdgcn_alignbit(d1, d0, sh), __builtin_amdgcn_alignbit(d2, d1, sh),
                 __builtin_amdgcn_alignbit(d3, d2, sh), __builtin_amdgcn_alignbit(d4, d3, sh)};
}

// One round (128 rows x all columns of a segment and head) of the 128 x 128 build through the ring: K <= 128 (one or
// two chunks; K = 0 runs as one chunk of zeros), N >= 128.
__host__ __device__ constexpr bool any16_ring_segment(int N, int K) { return K <= 2 * kAnyTile && N >= 2 * kAnyRingChunk; }
template <int DT, bool T1, bool T2>
__device__ __forceinline__ void any16_ring_round(__amdgpu_buffer_rsrc_t resX, __amdgpu_buffer_rsrc_t resY, uint16_t *os, int M,
                                                 int N, int K, int r0, unsigned char *any_lds) {
    constexpr int RT = 2, CG = 2;
    constexpr int kRows = kAnyTile * RT, kCols = kAnyTile * CG;
    constexpr int kPitchXT = AnyBuf<kRows>::pitch_t, kPitchYT = AnyBuf<kCols>::pitch_t;
    constexpr int kBufBytes = AnyBuf<kRows>::bytes + AnyBuf<kCols>::bytes;
    static_assert(2 * kAnyRingBytes <= AnyBuf<kRows>::bytes, "two rings per X buffer");
    constexpr bool t1 = T1, t2 = T2;
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = lane_id(), n = lane & 15, q = lane >> 4;
    const int nkc = K > kAnyTile ? 2 : 1;
    const int ncb = (N + kCols - 1) / kCols;
    const int steps = ncb * nkc;
    // operand offsets of this lane inside a buffer (as in the streaming round below)
    const int xa = (16 * RT * wave + n) * kAnyPitch + q * 16;
    const int ya = AnyBuf<kRows>::bytes + (8 * n) * kAnyPitch + q * 16;
    const int xt = (8 * q + (n >> 2)) * kPitchXT + (16 * RT * wave + 4 * (n & 3)) * 2;
    const int yt = AnyBuf<kRows>::bytes + (8 * q + (n >> 2)) * kPitchYT + (4 * (n & 3)) * 2;
    f32x4 acc[RT][4 * CG];
    auto clear = [&]() {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int t = 0; t < 4 * CG; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    clear();
        // ---- A operands to registers through LDS, once per round
        {
            u32x4 xl[2][RT][2];              // plain vectors: the staging union only lives inside the calls
#pragma unroll
            for (int c = 0; c < 2; ++c)
                if (c < nkc) {
#pragma unroll
                    for (int i = 0; i < RT; ++i) {
                        const Line16 l = fetch_chunk16<4 * RT>(resX, t1, M, K, r0, c * kAnyTile, tid + kAnyThreads * i);
                        xl[c][i][0] = l.v[0]; xl[c][i][1] = l.v[1];
                    }
                }
#pragma unroll
            for (int c = 0; c < 2; ++c)
                if (c < nkc) {
#pragma unroll
                    for (int i = 0; i < RT; ++i) {
                        Line16 l;
                        l.v[0] = xl[c][i][0]; l.v[1] = xl[c][i][1];
                        put_chunk16<false, 4 * RT, kPitchXT>(l, t1, M, K, r0, c * kAnyTile, any_lds + c * kBufBytes,
                                                             tid + kAnyThreads * i);
                    }
                }
        }
        struct YStage { u32x4 y[CG][2]; };
        auto fetch_y = [&](YStage &st, int cb, int kc) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < CG; ++i) {
                const Line16 l = fetch_chunk16<4 * CG>(resY, t2, N, K, cb * kCols, kc * kAnyTile, tid + kAnyThreads * i);
                st.y[i][0] = l.v[0]; st.y[i][1] = l.v[1];
            }
        };
        int f_cb = 0, f_kc = 0;
        auto advance = [&]() {
            if (++f_kc == nkc) { f_kc = 0; ++f_cb; }
        };
        YStage sa, sb;
        fetch_y(sa, f_cb, f_kc); advance();            // steps >= 2: N >= 128 is at least one block
        if (steps > 1) { fetch_y(sb, f_cb, f_kc); advance(); }
        lds_barrier();
        u32x4 af[RT][4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const unsigned char *xb = any_lds + (ks >> 1) * kBufBytes;
                if ((ks >> 1) < nkc)
                    af[rt][ks] = t1 ? lds_tr8<kPitchXT>(lds_bytes(xb + xt), 32 * rt + (ks & 1) * 32 * kPitchXT)
                                    : *reinterpret_cast<const u32x4 *>(xb + xa + 16 * rt * kAnyPitch + (ks & 1) * 64);
                else
                    af[rt][ks] = u32x4{0u, 0u, 0u, 0u};
            }
        lds_barrier();                                  // the X buffers are free: they hold the rings from here on

        unsigned char *ring = any_lds + (wave >> 1) * kBufBytes + (wave & 1) * kAnyRingBytes;
        const int wrow0 = r0 + kAnyRingRows * wave;
        const __amdgpu_buffer_rsrc_t out_res = __builtin_amdgcn_make_buffer_rsrc((void *)os, 0, M * N * 2, kRsrcFlags);
        const uint32_t out_phase = (uint32_t)(uintptr_t)os;    // low address bits decide the line phase of a row
        const int nch = (N + kAnyRingChunk - 1) / kAnyRingChunk;
        // store lanes: instruction t writes rows 8 t + lane / 8, piece lane % 8 of the row's aligned window
        const int pq = lane & 7;
        int upos[kAnyRingStores];                   // ring byte of the lane's piece in window 0: 2 (8 pq - d) mod 256
        uint32_t v0[kAnyRingStores];                // byte offset of that piece inside the segment's result
        const unsigned char *rbase0 = ring + (lane >> 3) * kAnyRingPitch;
#pragma unroll
        for (int t = 0; t < kAnyRingStores; ++t) {
            const int rho = wrow0 + 8 * t + (lane >> 3);
            const bool row_ok = rho < M;
            const int rn = row_ok ? rho * N : 0;
            const int d = (int)(((out_phase + 2u * (uint32_t)rn) & 127u) >> 1);   // columns before the row's first line boundary
            upos[t] = (16 * pq - 2 * d) & 255;
            v0[t] = row_ok ? (uint32_t)(2 * (rn + 8 * pq - d)) : kAnyOutOfRange;
        }
        auto copy_heads = [&](int first_row) __attribute__((always_inline)) {
            // the first 32 bytes of sixteen ring rows once more behind the rows: pieces that start in a row's
            // last 16 bytes continue there
            unsigned char *src = ring + (first_row + (lane >> 2)) * kAnyRingPitch + (lane & 3) * 8;
            *reinterpret_cast<u32x2 *>(src + 256) = *reinterpret_cast<const u32x2 *>(src);
            asm volatile("" ::: "memory");
        };
        // the window of chunk c (64 columns, lagging by the row's phase) of every row of the wavefront
        auto emit = [&](int c) __attribute__((always_inline)) {
            asm volatile("" ::: "memory");          // the reads below see the writes above (same wavefront, in order)
            if ((c & 1) == 0) { copy_heads(0); copy_heads(16); }
            const int par = (c & 1) << 7;
            const uint32_t adv = 128u * (uint32_t)c;
            const bool edge = c == 0 || c == nch - 1;
#pragma unroll
            for (int t = 0; t < kAnyRingStores; ++t) {
                const u32x4 v = any_ring_read16(rbase0 + t * 8 * kAnyRingPitch, upos[t] ^ par);
                uint32_t voff = v0[t] == kAnyOutOfRange ? kAnyOutOfRange : v0[t] + adv;
                if (edge) {                         // pieces before column 0 or past column N are dropped
                    const int col = (((upos[t] >> 1) + 64) & 127) - 64 + kAnyRingChunk * c;
                    if (col < 0 || col + 8 > N) voff = kAnyOutOfRange;
                }
                __builtin_amdgcn_raw_buffer_store_b128(v, out_res, voff, 0, kAnyRingAux);
            }
            if (edge) {
                const int et_row = wrow0 + (lane & 31);
                const uint32_t et_off = (lane < 32 && et_row < M) ? (uint32_t)(2 * (et_row * N)) : kAnyOutOfRange;
                const unsigned char *et_base = ring + (lane & 31) * kAnyRingPitch;
                if (c == 0) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(et_base);          // columns [0, 8)
                    __builtin_amdgcn_raw_buffer_store_b128(v, out_res, et_off, 0, kAnyRingAux);
                }
                if (c == nch - 1) {
                    // the window behind the last chunk (what is left of the rows), then columns [N-8, N)
                    const int par2 = (nch & 1) << 7;
#pragma unroll
                    for (int t = 0; t < kAnyRingStores; ++t) {
                        const u32x4 v = any_ring_read16(rbase0 + t * 8 * kAnyRingPitch, upos[t] ^ par2);
                        const int col = (((upos[t] >> 1) + 64) & 127) - 64 + kAnyRingChunk * nch;
                        const uint32_t voff = (col + 8 <= N && v0[t] != kAnyOutOfRange) ? v0[t] + 128u * (uint32_t)nch
                                                                                       : kAnyOutOfRange;
                        __builtin_amdgcn_raw_buffer_store_b128(v, out_res, voff, 0, kAnyRingAux);
                    }
                    const u32x4 v = any_ring_read16(et_base, (2 * (N - 8)) & 255);
                    __builtin_amdgcn_raw_buffer_store_b128(
                        v, out_res, et_off == kAnyOutOfRange ? kAnyOutOfRange : et_off + 2u * (uint32_t)(N - 8), 0, kAnyRingAux);
                }
            }
            asm volatile("" ::: "memory");
        };
        // a finished block: its two chunks into the ring as they lie in the registers (lane n holds columns
        // 8 n .. 8 n + 7 of its rows), the window of each behind it
        auto store_ring = [&](int cbi) __attribute__((always_inline)) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                if (2 * cbi + half >= nch) break;
                if ((n >> 3) == half) {
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            *reinterpret_cast<u32x4 *>(ring + (16 * rt + 4 * q + i) * kAnyRingPitch + 16 * n) =
                                u32x4{Elem<DT>::pack2(acc[rt][0][i], acc[rt][1][i]), Elem<DT>::pack2(acc[rt][2][i], acc[rt][3][i]),
                                      Elem<DT>::pack2(acc[rt][4][i], acc[rt][5][i]), Elem<DT>::pack2(acc[rt][6][i], acc[rt][7][i])};
                }
                emit(2 * cbi + half);
            }
            clear();
        };
        // one chunk of Y against the A operands of k-chunk KC (a constant: af is a register array)
        auto ring_step = [&](int step, int cbi, YStage &st, auto kc_c) __attribute__((always_inline)) {
            constexpr int KC = decltype(kc_c)::value;
            unsigned char *buf = any_lds + (step & 1) * kBufBytes;
#pragma unroll
            for (int i = 0; i < CG; ++i) {
                Line16 l;
                l.v[0] = st.y[i][0]; l.v[1] = st.y[i][1];
                put_chunk16<true, 4 * CG, kPitchYT>(l, t2, N, K, cbi * kCols, KC * kAnyTile, buf + AnyBuf<kRows>::bytes,
                                                    tid + kAnyThreads * i);
            }
            if (step + 2 < steps) { fetch_y(st, f_cb, f_kc); advance(); }
            lds_barrier();
            constexpr int kTiles = 4 * CG, kFrags = (kAnyTile / 32) * kTiles;
            const LdsBytes ybase = lds_bytes(buf + yt);
            auto read_b = [&](int f) __attribute__((always_inline)) {
                const int ks = f / kTiles, t = f % kTiles;
                return t2 ? lds_tr8<kPitchYT>(ybase, ks * 32 * kPitchYT + 32 * t)
                          : *reinterpret_cast<const u32x4 *>(buf + ya + t * kAnyPitch + ks * 64);
            };
            // (the scheduling barriers keep the reads where they are written: left alone, the compiler moves all
            // sixteen ahead of the matrix instructions and spills what the ring needs)
            constexpr int kAhead = 3;
            u32x4 bq[kAhead + 1];
#pragma unroll
            for (int f = 0; f < kAhead; ++f) bq[f] = read_b(f);
#pragma unroll
            for (int f = 0; f < kFrags; ++f) {
                const int ks = f / kTiles, t = f % kTiles;
                if (f + kAhead < kFrags) bq[(f + kAhead) % (kAhead + 1)] = read_b(f + kAhead);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) acc[rt][t] = Elem<DT>::mfma(af[rt][2 * KC + ks], bq[f % (kAhead + 1)], acc[rt][t]);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        using C0 = std::integral_constant<int, 0>;
        using C1 = std::integral_constant<int, 1>;
        if (nkc == 2) {
            for (int cbi = 0; cbi < ncb; ++cbi) {
                ring_step(2 * cbi, cbi, sa, C0{});
                ring_step(2 * cbi + 1, cbi, sb, C1{});
                store_ring(cbi);
            }
        } else {
            for (int cbi = 0; cbi < ncb; cbi += 2) {
                ring_step(cbi, cbi, sa, C0{});
                store_ring(cbi);
                if (cbi + 1 < ncb) {
                    ring_step(cbi + 1, cbi + 1, sb, C0{});
                    store_ring(cbi + 1);
                }
            }
        }
}

// RT = 16-row tiles per wavefront (the workgroup's step covers 64 RT rows), CG = groups of 64 columns per step.
// The loads of a step are issued two steps ahead into registers, the chunks alternate between two LDS buffers:
// one barrier per step, and two steps' worth of loads in flight per workgroup while it computes.  The kernel is
// bound by operand traffic out of L2 (a 64 x 64 step fetches 16 KiB for 32 matrix instructions), which the
// 128 x 128 step halves per result.
template <int DT, int RT, int CG, bool T1, bool T2>
__device__ __forceinline__ void any16_stream_rounds(__amdgpu_buffer_rsrc_t resX, __amdgpu_buffer_rsrc_t resY, uint16_t *os, int M,
                                                    int N, int K, int first_round, int round_step, int rounds,
                                                    unsigned char *any_lds) {
    constexpr int kRows = kAnyTile * RT, kCols = kAnyTile * CG;
    constexpr int kPitchXT = AnyBuf<kRows>::pitch_t, kPitchYT = AnyBuf<kCols>::pitch_t;
    constexpr int kBufBytes = AnyBuf<kRows>::bytes + AnyBuf<kCols>::bytes;
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = lane_id(), n = lane & 15, q = lane >> 4;
    constexpr bool t1 = T1, t2 = T2;                  // the layouts are part of the build: no branch on them in the loop
    const int nkc = (K + kAnyTile - 1) / kAnyTile;
    // operand offsets of this lane inside a buffer: A operand of row tile rt = row 16 (RT wave + rt) + n of X,
    // B operand of tile t = row 4 n + t of Y (64-column step; 8 n + t in the 128-column step: column slot n of tile t
    // is that column), eight k from 8 q on
    const int xa = (16 * RT * wave + n) * kAnyPitch + q * 16;
    const int ya = AnyBuf<kRows>::bytes + ((CG == 2 ? 8 : 4) * n) * kAnyPitch + q * 16;
    // the same from k-major chunks (transposed operands): k row 8 q + n / 4 of the step, positions 4 (n % 4) .. of the
    // row tile's sixteen rows (X) or of tile t's sixteen positions (Y, + 32 t bytes)
    const int xt = (8 * q + (n >> 2)) * kPitchXT + (16 * RT * wave + 4 * (n & 3)) * 2;
    const int yt = AnyBuf<kRows>::bytes + (8 * q + (n >> 2)) * kPitchYT + (4 * (n & 3)) * 2;

    f32x4 acc[RT][4 * CG];
    auto clear = [&]() {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int t = 0; t < 4 * CG; ++t) acc[rt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    // lane (n, q): rows 16 (RT wave + rt) + 4 q + i, columns kCols cb + kLaneCols n .. of the block, side by side: one
    // 8- or 16-byte store per row, the sixteen lanes of a row group writing 128 or 256 contiguous bytes; clears the
    // accumulators
    constexpr int kLaneCols = 4 * CG;
    auto store_block = [&](int cb, int r0) __attribute__((always_inline)) {
        const bool whole = r0 + kRows <= M && (cb + 1) * kCols <= N;       // no row or column of the block is outside
        const int col = cb * kCols + kLaneCols * n;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            uint16_t *p0 = os + (int64_t)(r0 + 16 * (RT * wave + rt) + 4 * q) * N + col;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = r0 + 16 * (RT * wave + rt) + 4 * q + i;
                uint16_t *p = p0 + (int64_t)i * N;
                if (whole || (row < M && col + kLaneCols <= N)) {
                    if constexpr (CG == 2) {
                        store_result<false>(reinterpret_cast<u32x4_unaligned *>(p),
                                     u32x4{Elem<DT>::pack2(acc[rt][0][i], acc[rt][1][i]), Elem<DT>::pack2(acc[rt][2][i], acc[rt][3][i]),
                                           Elem<DT>::pack2(acc[rt][4][i], acc[rt][5][i]), Elem<DT>::pack2(acc[rt][6][i], acc[rt][7][i])});
                    } else {
                        store_result<false>(reinterpret_cast<u32x2_unaligned *>(p),
                                     u32x2{Elem<DT>::pack2(acc[rt][0][i], acc[rt][1][i]), Elem<DT>::pack2(acc[rt][2][i], acc[rt][3][i])});
                    }
                } else if (row < M) {
#pragma unroll
                    for (int t = 0; t < kLaneCols - 1; ++t)
                        if (col + t < N) p[t] = Elem<DT>::from_float(acc[rt][t][i]);
                }
            }
        }
        clear();
    };
    const int ncb = (N + kCols - 1) / kCols;
    const int steps = ncb * nkc;                     // (column block, chunk) pairs of one round, chunk fastest
    // With at most two chunks of k (K <= 128) the X chunks of a round stay in LDS, one per buffer, and are fetched
    // once instead of once per column block; only Y streams.
    const bool x_once = nkc <= 2;
    clear();
    // The workgroup's rounds (first_round, first_round + round_step, ... below `rounds`) are ONE stream of steps: the
    // loads of a round's first chunks are issued during the last steps of the round before, so only the first round
    // of a workgroup waits for memory with nothing to do.
    const int my_rounds = first_round < rounds ? (rounds - 1 - first_round) / round_step + 1 : 0;
    const int total = my_rounds * steps;
    // a stage = the registers of one chunk in flight (plain vectors: the staging union only lives inside the calls)
    struct Stage { u32x4 x[RT][2], y[CG][2]; };
    auto fetch = [&](Stage &st, int round, int cb, int kc) __attribute__((always_inline)) {
        const int r0 = round * kRows;
        if (!x_once || cb == 0) {
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const Line16 l = fetch_chunk16<4 * RT>(resX, t1, M, K, r0, kc * kAnyTile, tid + kAnyThreads * i);
                st.x[i][0] = l.v[0]; st.x[i][1] = l.v[1];
            }
        }
#pragma unroll
        for (int i = 0; i < CG; ++i) {
            const Line16 l = fetch_chunk16<4 * CG>(resY, t2, N, K, cb * kCols, kc * kAnyTile, tid + kAnyThreads * i);
            st.y[i][0] = l.v[0]; st.y[i][1] = l.v[1];
        }
    };
    int f_round = first_round, f_cb = 0, f_kc = 0;        // the chunk the next fetch takes
    auto advance = [&]() {
        if (++f_kc == nkc) {
            f_kc = 0;
            if (++f_cb == ncb) { f_cb = 0; f_round += round_step; }
        }
    };
    Stage sa, sb;
    if (total > 0) { fetch(sa, f_round, f_cb, f_kc); advance(); }
    if (total > 1) { fetch(sb, f_round, f_cb, f_kc); advance(); }
    int c_round = first_round, cb = 0, kc = 0;            // the chunk being computed
    auto do_step = [&](int gs, Stage &st) __attribute__((always_inline)) {
        const int step = cb * nkc + kc;                   // position inside the round: decides the buffers
        const int r0 = c_round * kRows;
        // a new round's X chunks go where the last one's lie: wait until every wavefront has read those
        if (step == 0 && gs > 0) lds_barrier();
        unsigned char *buf = any_lds + (step & 1) * kBufBytes;
        unsigned char *xbuf = any_lds + (x_once ? kc : step & 1) * kBufBytes;
        if (!x_once || cb == 0) {
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                Line16 l;
                l.v[0] = st.x[i][0]; l.v[1] = st.x[i][1];
                put_chunk16<false, 4 * RT, kPitchXT>(l, t1, M, K, r0, kc * kAnyTile, xbuf, tid + kAnyThreads * i);
            }
        }
#pragma unroll
        for (int i = 0; i < CG; ++i) {
            Line16 l;
            l.v[0] = st.y[i][0]; l.v[1] = st.y[i][1];
            put_chunk16<true, 4 * CG, kPitchYT>(l, t2, N, K, cb * kCols, kc * kAnyTile, buf + AnyBuf<kRows>::bytes,
                                                tid + kAnyThreads * i);
        }
        if (gs + 2 < total) { fetch(st, f_round, f_cb, f_kc); advance(); }   // in flight under two steps of matrix instructions
        // every wavefront has written its part of this chunk, and is done reading the chunk before last,
        // whose buffer the NEXT step's writes go to
        lds_barrier();
        // the B operands are read two tiles ahead of the matrix instructions that use them (an LDS round trip
        // is several times a matrix instruction), the A operands of the second k-step while the first computes
        constexpr int kTiles = 4 * CG, kFrags = (kAnyTile / 32) * kTiles;
        const LdsBytes xbase = lds_bytes(xbuf + xt);
        auto read_a = [&](int ks, int rt) __attribute__((always_inline)) {
            return t1 ? lds_tr8<kPitchXT>(xbase, 32 * rt + ks * 32 * kPitchXT)
                      : *reinterpret_cast<const u32x4 *>(xbuf + xa + 16 * rt * kAnyPitch + ks * 64);
        };
        const LdsBytes ybase = lds_bytes(buf + yt);
        auto read_b = [&](int f) __attribute__((always_inline)) {
            const int ks = f / kTiles, t = f % kTiles;
            return t2 ? lds_tr8<kPitchYT>(ybase, ks * 32 * kPitchYT + 32 * t)
                      : *reinterpret_cast<const u32x4 *>(buf + ya + t * kAnyPitch + ks * 64);
        };
        u32x4 av[2][RT], bq[3];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) av[0][rt] = read_a(0, rt);
        bq[0] = read_b(0);
        bq[1] = read_b(1);
#pragma unroll
        for (int f = 0; f < kFrags; ++f) {
            const int ks = f / kTiles, t = f % kTiles;
            if (f + 2 < kFrags) bq[(f + 2) % 3] = read_b(f + 2);
            if (t == 0 && ks + 1 < kAnyTile / 32) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) av[(ks + 1) & 1][rt] = read_a(ks + 1, rt);
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) acc[rt][t] = Elem<DT>::mfma(av[ks & 1][rt], bq[f % 3], acc[rt][t]);
        }
        if (kc == nkc - 1) store_block(cb, r0);
        if (++kc == nkc) {
            kc = 0;
            if (++cb == ncb) { cb = 0; c_round += round_step; }
        }
    };
    for (int gs = 0; gs < total; gs += 2) {
        do_step(gs, sa);
        if (gs + 1 < total) do_step(gs + 1, sb);
    }
    if (nkc == 0)                                                  // K = 0: the result is zeros
        for (int round = first_round; round < rounds; round += round_step)
            for (int c = 0; c < ncb; ++c) store_block(c, round * kRows);
}

// RING: the kernel of the segments that any16_ring_segment accepts (128 x 128 build only); the other build of the pair
// skips those when kFlagRingToo says that the ring kernel runs in the same call.  Two kernels, not one that chooses
// per segment: either round wants all 256 registers, and neither as a function called from the other's kernel nor
// inlined beside it did they keep out of each other's way (spills in the streaming loop, saves around every call).
// block_x: the workgroup's index in the flat grid of a launch with the totals on the host (ride_slots = 1).
template <int DT, int RT, int CG, bool T1, bool T2, bool RING>
__device__ __forceinline__ void any16_workgroup(const RunArgs &a, unsigned block_x, unsigned char *any_lds) {
    static_assert(!RING || (RT == 2 && CG == 2), "the ring belongs to the 128 x 128 build");
    constexpr int kRows = kAnyTile * RT, kCols = kAnyTile * CG;
    const ConstHdr hdr = (ConstHdr)(uintptr_t)a.plan;
    const int nseg = hdr->nseg;
    const int64_t per_head = RT == 2 ? hdr->att_blocks128 : hdr->att_blocks64;   // row rounds per head
    if (!header_ok(a)) {
        if (!(a.flags & kFlagQuiet)) {
            if (!a.ride_slots) report_mismatch(a);
            else if (block_x == 0 && threadIdx.x == 0)       // (the first workgroup of THIS product, wherever it lies in the grid)
                atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        }
        return;
    }
    // Two grids.  With the batch's totals on the host (ride_slots = 1): one workgroup per existing
    // (segment, row round, head), head fastest, found by a search in the plan's row-block prefix.  Without:
    // (head, segment, z) or (segment, head, z), workgroup z taking the rounds z, z + gridDim.z, ...
    const bool head_fast = a.flags & kFlagHeadFast;
    // (a step past any segment's round count, small enough that first_round + step cannot overflow)
    constexpr int rounds_never_again = 1 << 26;
    int g, first_round, round_step;
    int64_t h;
    if (a.ride_slots) {
        const int32_t *pfx = plan_rowblocks(a.plan, nseg, RT == 2 ? 1 : 0);
        // Workgroups go to the eight dies round-robin by their index, and each die has its own L2.  The work items
        // (head slowest, then segment, then row round) are dealt to the dies in blocks of kAnyDieBlock consecutive
        // items: the workgroups a die runs together are then neighbouring row rounds of one segment and head, which
        // read the same Y, so Y comes out of that die's L2 instead of being streamed from memory once per round.
        const int64_t u = block_x;
        const int64_t slot = u / kDies;
        const int64_t v = ((slot / kAnyDieBlock) * kDies + u % kDies) * kAnyDieBlock + slot % kAnyDieBlock;
        if (v >= per_head * a.H) return;
        h = v / per_head;
        const int item = (int)(v % per_head);
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
    if (RING != any16_ring_segment(N, K) && (RING || (a.flags & kFlagRingToo))) return;   // the other kernel's segment
    const __amdgpu_buffer_rsrc_t resX = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(reinterpret_cast<const uint16_t *>(a.A) + h * a.Dm1 + rec.off1), 0, M * K * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t resY = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(reinterpret_cast<const uint16_t *>(a.B) + h * a.Dm2 + rec.off2), 0, N * K * 2, kRsrcFlags);
    uint16_t *os = reinterpret_cast<uint16_t *>(a.out) + h * a.Dout + rec.offO;
    if (RING && threadIdx.x == 0) atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->ring_groups, 1);
    const int rounds = (M + kRows - 1) / kRows;
    if constexpr (RING) {
        for (int round = first_round; round < rounds; round += round_step) {
            any16_ring_round<DT, T1, T2>(resX, resY, os, M, N, K, round * kRows, any_lds);
            if (round + round_step < rounds) lds_barrier();        // the next round's X chunks go where the rings are
        }
    } else {
        any16_stream_rounds<DT, RT, CG, T1, T2>(resX, resY, os, M, N, K, first_round, round_step, rounds, any_lds);
    }
}

template <int DT, int RT, int CG, bool T1, bool T2, bool RING>
__global__ __launch_bounds__(kAnyThreads, RT * CG >= 4 ? 2 : 4) void gemm_any16_kernel(RunArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char any_lds[];
    any16_workgroup<DT, RT, CG, T1, T2, RING>(a, blockIdx.x, any_lds);
}

// Two products in one launch (64 x 64 build, totals on the host): the first `split` workgroups are those of a launch
// over `a`, the rest those of a launch over `b`.  For the two products of the backward pass of a batch of short
// segments, dA = dS B (second operand k-major) and dB = dS^T A (both k-major): each alone is a few rounds of
// workgroups that live for one or two steps, and two launches pay the ramps at both ends twice.
template <int DT>
__global__ __launch_bounds__(kAnyThreads, 4) void gemm_any16_two_kernel(RunArgs a, RunArgs b, unsigned split) {
    extern __shared__ __attribute__((aligned(16))) unsigned char any_lds[];
    if (blockIdx.x < split) any16_workgroup<DT, 1, 1, false, true, false>(a, blockIdx.x, any_lds);
    else any16_workgroup<DT, 1, 1, true, true, false>(b, blockIdx.x - split, any_lds);
}

template <int DT, int RT, int CG, bool T1, bool T2, bool RING>
static void launch_any_build(const RunArgs &run, dim3 grid, hipStream_t stream) {
    constexpr int kLds = 2 * (AnyBuf<kAnyTile * RT>::bytes + AnyBuf<kAnyTile * CG>::bytes);
    if constexpr (kLds > 65536) {
        static const bool attr_set = [] {
            return hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_any16_kernel<DT, RT, CG, T1, T2, RING>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds) == hipSuccess;
        }();
        (void)attr_set;
    }
    hipLaunchKernelGGL((gemm_any16_kernel<DT, RT, CG, T1, T2, RING>), grid, dim3(kAnyThreads), kLds, stream, run);
}
template <int DT, int RT, int CG, bool RING = false>
static void launch_any(const RunArgs &run, dim3 grid, hipStream_t stream) {
    const bool t1 = run.flags & kFlagTranspose1, t2 = run.flags & kFlagTranspose2;
    if (t1 && t2) launch_any_build<DT, RT, CG, true, true, RING>(run, grid, stream);
    else if (t1) launch_any_build<DT, RT, CG, true, false, RING>(run, grid, stream);
    else if (t2) launch_any_build<DT, RT, CG, false, true, RING>(run, grid, stream);
    else launch_any_build<DT, RT, CG, false, false, RING>(run, grid, stream);
}

int launch_gemm_any16(int dtype, const RunArgs &args, int64_t nseg, const ba_plan_info *info, hipStream_t stream) {
    if (args.H > 65535) return BA_ERR_UNSUPPORTED;      // heads ride on gridDim.y
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (info) nseg = info->nseg;
    if (nseg <= 0) return BA_OK;
    RunArgs run = args;
    dim3 grid;
    // 128 x 128 steps where the segments are tall (four 64-row rounds per segment on average): half the operand
    // traffic per result and 16-byte stores; batches of short segments finish in one or two steps per workgroup
    // either way and do better with twice as many, smaller workgroups resident.  Measured, operands stored K x M and
    // K x N, 128 / 64: 16 segments x 16 heads of 1024..4096 rows 1660 / 2120 us; 512 segments of 16..256 rows
    // 24.0 / 20.5 us; 1024 segments, power-law sizes, 85 / 53 us.  BLOCKEDATTN_ANY_TILE=64|128 forces one.
    static const int tile_env = [] { const char *e = getenv("BLOCKEDATTN_ANY_TILE"); return e ? atoi(e) : 0; }();
    const bool big = tile_env ? tile_env == 128 : info && (int64_t)info->att_blocks64 >= 4 * (int64_t)info->nseg;
    const int64_t items = info ? (int64_t)(big ? info->att_blocks128 : info->att_blocks64) * args.H : 0;
    // (one workgroup per existing round, not per (segment, head): a 64 x 64 x 64 step takes a workgroup about a
    // microsecond whatever is in flight, so the rounds of a segment are worth more side by side than one after the
    // other -- 512 segments of 16..256 rows: 20.8 us against 35 / 26 / 22 us with one / two / three workgroups per pair)
    if (info && items < (int64_t(1) << 31) - 1024) {
        if (items == 0) return BA_OK;                   // no segment has rows
        run.ride_slots = 1;
        const int64_t unit = (int64_t)kDies * kAnyDieBlock;           // whole blocks for every die
        grid = dim3((unsigned)((items + unit - 1) / unit * unit));
    } else {
        const bool head_fast = nseg <= 65535;           // segments then ride on gridDim.y
        if (head_fast) run.flags |= kFlagHeadFast;
        grid = head_fast ? dim3((unsigned)args.H, (unsigned)nseg, 4u) : dim3((unsigned)nseg, (unsigned)args.H, 4u);
    }
    // 128 x 128 build: the segments with K <= 128 and at least 128 columns go to the ring kernel (whole-line stores),
    // launched if the batch's extremes allow such a segment; the streaming kernel runs if they allow another kind
    static const bool ring_env = [] { const char *e = getenv("BLOCKEDATTN_ANY_RING"); return !e || atoi(e) != 0; }();
    bool stream_too = true;
    if (big && info && ring_env && info->min_K <= 2 * kAnyTile && info->max_N >= 2 * kAnyRingChunk) {
        if (dtype == BA_F16) launch_any<0, 2, 2, true>(run, grid, stream);
        else launch_any<1, 2, 2, true>(run, grid, stream);
        run.flags |= kFlagRingToo | kFlagQuiet;
        stream_too = info->min_N < 2 * kAnyRingChunk || info->max_K > 2 * kAnyTile;
    }
    if (stream_too) {
        if (dtype == BA_F16) {
            if (big) launch_any<0, 2, 2>(run, grid, stream);
            else launch_any<0, 1, 1>(run, grid, stream);
        } else {
            if (big) launch_any<1, 2, 2>(run, grid, stream);
            else launch_any<1, 1, 1>(run, grid, stream);
        }
    }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

// The two-product launch above, if both calls would take the 64 x 64 build with the plan's totals on the host and
// have the layouts of the backward pass (a: second operand k-major; b: both); BA_ERR_UNSUPPORTED otherwise, and the
// caller makes two calls of launch_gemm_any16.
int launch_gemm_any16_two(int dtype, const RunArgs &a, const ba_plan_info *info_a, const RunArgs &b, const ba_plan_info *info_b,
                          hipStream_t stream) {
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (!info_a || !info_b || a.H != b.H || a.H > 65535) return BA_ERR_UNSUPPORTED;
    static const int tile_env = [] { const char *e = getenv("BLOCKEDATTN_ANY_TILE"); return e ? atoi(e) : 0; }();
    auto big = [&](const ba_plan_info *i) { return tile_env ? tile_env == 128 : (int64_t)i->att_blocks64 >= 4 * (int64_t)i->nseg; };
    if (big(info_a) || big(info_b)) return BA_ERR_UNSUPPORTED;
    const int layout = kFlagTranspose1 | kFlagTranspose2;
    if ((a.flags & layout) != kFlagTranspose2 || (b.flags & layout) != layout) return BA_ERR_UNSUPPORTED;
    const int64_t unit = (int64_t)kDies * kAnyDieBlock;
    const int64_t items_a = (int64_t)info_a->att_blocks64 * a.H, items_b = (int64_t)info_b->att_blocks64 * b.H;
    if (items_a <= 0 || items_b <= 0) return BA_ERR_UNSUPPORTED;
    const int64_t grid_a = (items_a + unit - 1) / unit * unit, grid_b = (items_b + unit - 1) / unit * unit;
    if (grid_a + grid_b >= (int64_t(1) << 31) - 1024) return BA_ERR_UNSUPPORTED;
    RunArgs ra = a, rb = b;
    ra.ride_slots = rb.ride_slots = 1;
    ra.nseg = (int)info_a->nseg;
    rb.nseg = (int)info_b->nseg;
    constexpr int kLds = 2 * (AnyBuf<kAnyTile>::bytes + AnyBuf<kAnyTile>::bytes);
    if (dtype == BA_F16)
        hipLaunchKernelGGL((gemm_any16_two_kernel<0>), dim3((unsigned)(grid_a + grid_b)), dim3(kAnyThreads), kLds, stream, ra, rb,
                           (unsigned)grid_a);
    else
        hipLaunchKernelGGL((gemm_any16_two_kernel<1>), dim3((unsigned)(grid_a + grid_b)), dim3(kAnyThreads), kLds, stream, ra, rb,
                           (unsigned)grid_a);
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
