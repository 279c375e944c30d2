// Varlen attention in one pass: O_g = softmax(scale * Q_g K_g^T) V_g per segment and head, with the
// probabilities never written to memory.  It is what a caller of the reference gets from
// blockGEMM -> blockSoftmax -> blockGEMM (README.md:3; csrc/sparseBlockedAttention.cpp:118-131) when
// the probabilities themselves are not wanted: the M x N array, which bounds every other kernel of
// this library, stays in registers.
//
// Layout: Q_g is the M x K operand of the plan (offset off1), K_g and V_g are N x K (offset off2,
// both with the per-head stride Dm2), O_g is M x K at off1 of a [H, Dm1] buffer.  K <= 128.
//
// Workgroup = 4 wavefronts = 64 queries of one segment and head; the keys go by in blocks of 64.
// Per block the workgroup stages K_g's rows (as they lie, zero padded to a multiple of 32 in k) and
// V_g's rows TRANSPOSED (one LDS row per output column, keys along the row) in LDS.  A wavefront owns
// 16 queries:
//   S^T block  = K_blk Q^T   (matrix instructions, A operand = key rows from LDS, B operand = the
//                wavefront's query rows, held in registers for the whole pass); the lane
//                (j = lane%16, rg = lane/16) then holds query j's scores for keys 16t + 4rg + e;
//   online softmax: reference value m (a lazily raised row maximum) and row sum l per query (per lane;
//                the four lanes of a query exchange the block maximum), accumulators rescaled by
//                2^((m_old - m_new) c) when m is raised;
//   O^T       += V_blk^T P^T (A operand = transposed value rows from LDS, B operand = the lane's own
//                probabilities rounded to the 16-bit type: the k index of the instruction runs over
//                keys in the order the score registers hold them, so P never moves between lanes).
// The query index is lane%16 in scores and outputs alike, so m, l and the rescaling are per lane.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>
#include <utility>

#include "ba_device.hpp"
#include "ba_gemm_common.hpp"
#include "ba_host.hpp"

namespace ba {

constexpr int kAttThreads = 256;
constexpr int kAttWaves = kAttThreads / 64;
constexpr int kAttKeys = 64;                          // keys per block
constexpr int kAttRows = 16 * kAttWaves;              // queries per workgroup round
static_assert(kAttRows == kAttBlockRows, "the plan's row-block prefixes count blocks of kAttRows and 2 kAttRows");
// LDS row pitches.  A 16-byte operand read of a wavefront is served 32 lanes at a time, 512 bytes wide (measured:
// lane * 16 and 288-byte rows run at 4.75 cycles per wavefront read, 272- and 144-byte rows at 8): the lanes
// (j, rg) and (j, rg + 1) of sixteen rows j must land in 32 different 16-byte slots modulo 512 bytes, which a
// pitch of 16 * (2 * odd) bytes does.  Keys: 64 NK + 32 bytes; transposed values (64 keys a row): 160 bytes.  The
// staging writes take what is left (two-way conflicts on a quarter as many instructions).
constexpr int kAttPitchV = kAttKeys * 2 + 32;
// LDS operand reads in flight per wavefront: six, or three in the builds for short segments and head dimensions
// up to 64, which then fit 128 registers and run four wavefronts per SIMD (the launch is bound by the life of a
// workgroup there: 256 segments of 32..128 rows, 31.3 -> 29.0 us)
constexpr int att_ring(int nk, int qt) { return qt == 1 && nk <= 2 ? 3 : 6; }

// LDS operand reads as inline assembly, so that kAttRing of them are in flight under the matrix instructions
// (left to itself the compiler, short of registers, issues each read right before its use and every matrix
// instruction waits a full LDS round trip).  The compiler does not count these reads: lds_wait<n> waits until at
// most n of them are outstanding and hands the register on, so the use cannot move above the wait.  Counting is
// conservative when other LDS or scalar loads are in flight: the counter is then higher, the wait longer.
template <int OFF> __device__ __forceinline__ void lds_read128(u32x4 &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int N> __device__ __forceinline__ void lds_wait(u32x4 &x) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N) : "memory");
}
template <typename F, int... I> __device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}
__device__ __forceinline__ uint32_t lds_offset(const void *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

// Eight consecutive elements k0 .. k0+7 of a row of K elements, zeros at and past K, for rows whose
// length is not a multiple of 8 (pieces straddle nothing, but the row may end inside one): element by
// element, one load in flight, few registers -- the slow path must not set the register count of the
// kernel.  Each step shifts the 128-bit value down by one element and puts the new one on top.
__device__ __forceinline__ u32x4 load8_slow(const uint16_t *row, int k0, int K) {
    uint32_t r0 = 0, r1 = 0, r2 = 0, r3 = 0;
#pragma nounroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t x = row[min(k0 + i, K - 1)];
        r0 = (r0 >> 16) | (r1 << 16);
        r1 = (r1 >> 16) | (r2 << 16);
        r2 = (r2 >> 16) | (r3 << 16);
        r3 = (r3 >> 16) | ((k0 + i < K ? x : 0u) << 16);
    }
    return u32x4{r0, r1, r2, r3};
}

// a * b + c for a, b below 2^24: one instruction
__device__ __forceinline__ uint32_t mad24(uint32_t a, uint32_t b, uint32_t c) { return __umul24(a, b) + c; }

// NK = 32-wide k steps (head dimension padded to 32 * NK).  VEC: the segment's K is a multiple of 8, its
// rows come as 16-byte loads; otherwise element by element.  The two are separate instances of the whole
// body so that the slow loads do not sit inside the fast path's loops.
template <int DT, int NK, int QT, bool VEC>
__device__ __forceinline__ void attention_body(const RunArgs &a, const void *Vbuf, const SegRec &rec, int64_t h, int zblock,
                                               unsigned char *sK, unsigned char *sV) {
    constexpr int KP = 32 * NK;                       // padded head dimension
    constexpr int kPitchK = KP * 2 + 32;              // bytes per LDS row of keys
    constexpr int kPieces = KP / 8;                   // 16-byte pieces per row
    constexpr int kOutTiles = KP / 16;
    constexpr int kAttRing = att_ring(NK, QT);
    const int M = rec.M, N = rec.N, K = rec.K;
    const int tid = threadIdx.x;
    const int wave = uniform(tid >> 6);
    const int lane = lane_id();
    const int j = lane & 15, rg = lane >> 4;
    const uint16_t *qs = reinterpret_cast<const uint16_t *>(a.A) + h * a.Dm1 + rec.off1;
    const uint16_t *ks = reinterpret_cast<const uint16_t *>(a.B) + h * a.Dm2 + rec.off2;
    const uint16_t *vs = reinterpret_cast<const uint16_t *>(Vbuf) + h * a.Dm2 + rec.off2;
    uint16_t *os = reinterpret_cast<uint16_t *>(a.out) + h * a.Dm1 + rec.off1;

    // A negative scale is applied as |scale| to negated scores (sign bits of the query operand flipped),
    // so that the running maximum is always the value to subtract.
    // A scale of zero (uniform probabilities) is applied as scores of zero under a scale of one: the keys past
    // the end of a segment are masked as -inf scores, which a zero factor would turn into NaN.
    const float c_signed = a.scale * kLog2e;
    const float c = c_signed == 0.f ? 1.0f : __builtin_fabsf(c_signed);
    const uint32_t flip = c_signed < 0.f ? 0x80008000u : 0u;
    const uint32_t keep = c_signed == 0.f ? 0u : 0xffffffffu;
    const u32x4 zero4 = u32x4{0u, 0u, 0u, 0u};

    // Staging, per thread: kSteps 16-byte pieces of the key rows (kLpr neighbouring lanes share a row; step s
    // takes rows s * kRowsStep ..) and 4 keys x 8 columns of values (key group tid % 16, piece tid / 16; a load
    // instruction of a wavefront then covers 64 contiguous bytes of sixteen rows, a write 128 of one).  Element
    // offsets inside a segment fit 32 bits (checked by the kernel).
    constexpr int kLpr = NK == 3 ? 16 : kPieces;      // lanes per key row (a power of two; 12 pieces: 4 lanes idle)
    constexpr int kSteps = kLpr / 4, kRowsStep = kAttThreads / kLpr;
    const int k_row = tid / kLpr, k_piece = tid % kLpr;
    const int v_kg = tid & 15, v_piece = tid >> 4;    // sixteen lanes = the sixteen key groups of one piece
    const bool v_thread = v_piece < kPieces;
    // Keys along an LDS row of transposed values stand in the order the probabilities have in a lane's registers:
    // the eight keys 32 cc + 16 h + 4 rg + e (h < 2, e < 4) of lane group rg are 16 contiguous bytes, one operand
    // read.  The thread's four keys 4 v_kg .. + 3 (v_kg = 8 cc + 4 h + rg) go to the 8-byte slot 8 cc + 2 rg + h.
    const int v_slot = (v_kg & 8) + 2 * (v_kg & 3) + ((v_kg >> 2) & 1);
    // VEC: the loads go through buffer descriptors that span exactly the segment's keys and values, so a row
    // past the last key reads as zeros with no code; a piece past the head dimension has an offset that is
    // out of range and stays there (its advance is multiplied by zero).
    const __amdgpu_buffer_rsrc_t resK = __builtin_amdgcn_make_buffer_rsrc((void *)ks, 0, VEC ? N * K * 2 : 0, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t resV = __builtin_amdgcn_make_buffer_rsrc((void *)vs, 0, VEC ? N * K * 2 : 0, kRsrcFlags);
    constexpr uint32_t kNever = 0xfffffff0u;
    const uint32_t row_bytes = 2u * (uint32_t)K;      // all advances below are under 2^24 (K <= 128)
    const uint32_t k_live = 8 * k_piece < K ? 1u : 0u, v_live = 8 * v_piece < K ? 1u : 0u;
    const uint32_t k_byte0 = k_live ? (uint32_t)k_row * row_bytes + 16u * (uint32_t)k_piece : kNever;
    const uint32_t v_byte0 = v_live ? (uint32_t)(4 * v_kg) * row_bytes + 16u * (uint32_t)v_piece : kNever;

    // operand reads: lane (j, rg) reads 16 bytes of key row 16 t + j at k = 32 s + 8 rg, of value row (output
    // column) 16 t + j at the lane group's eight keys of half cc
    const uint32_t k_addr = lds_offset(sK) + (uint32_t)(j * kPitchK + rg * 16);
    const uint32_t v_addr = lds_offset(sV) + (uint32_t)(j * kAttPitchV + rg * 16);

    constexpr int kRoundRows = kAttRows * QT;           // queries per workgroup round
    for (int round = zblock; (int64_t)round * kRoundRows < M; round += a.ride_slots ? (1 << 24) : a.tile_zdim) {
        // strip q of the wavefront: rows round * kRoundRows + 64 q + 16 wave ..; the live ones come first
        const int r0 = round * kRoundRows + wave * 16;
        const int nq = uniform(r0 >= M ? 0 : min(QT, (M - r0 + kAttRows - 1) / kAttRows));   // 0: the wavefront only stages
        // the wavefront's queries as B operand: lane (query j, rg) holds k = 32 s + 8 rg .. + 7
        u32x4 qf[QT][NK];
#pragma unroll
        for (int q = 0; q < QT; ++q) {
            const uint16_t *qrow = qs + (int64_t)min(r0 + kAttRows * q + j, M - 1) * K;
            if constexpr (VEC) {
#pragma unroll
                for (int s = 0; s < NK; ++s)
                    qf[q][s] = *reinterpret_cast<const u32x4_unaligned *>(qrow + min(32 * s + 8 * rg, K - 8));
            } else {
#pragma unroll
                for (int s = 0; s < NK; ++s) qf[q][s] = load8_slow(qrow, 32 * s + 8 * rg, K);
            }
#pragma unroll
            for (int s = 0; s < NK; ++s) {
                qf[q][s] = 32 * s + 8 * rg < K ? qf[q][s] : zero4;
                qf[q][s] = u32x4{(qf[q][s][0] ^ flip) & keep, (qf[q][s][1] ^ flip) & keep, (qf[q][s][2] ^ flip) & keep,
                                 (qf[q][s][3] ^ flip) & keep};
            }
        }
        float m[QT], lsum[QT];
        f32x4 oacc[QT][kOutTiles];
#pragma unroll
        for (int q = 0; q < QT; ++q) {
            m[q] = -INFINITY; lsum[q] = 0.f;
#pragma unroll
            for (int t = 0; t < kOutTiles; ++t) oacc[q][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }

        // The loads run one block ahead of the arithmetic: the loads of block kb + 64 are issued before the
        // matrix work on block kb and land in registers (kw: this thread's pieces of the key rows, vw: its
        // 4 keys x 8 columns of values) while that work runs.  All loads of a block sit in one branch-free
        // sequence (index clamped, value selected afterwards): loads behind a branch wait one by one.
        u32x4 kw[kSteps], vw[4];
        uint32_t k_byte = k_byte0, v_byte = v_byte0;
        auto fetch = [&](int kb) {                     // called for kb = 0, 64, 128, .. in turn
            if constexpr (VEC) {
#pragma unroll
                for (int step = 0; step < kSteps; ++step)
                    kw[step] = __builtin_amdgcn_raw_buffer_load_b128(
                        resK, mad24(k_live, (uint32_t)(step * kRowsStep) * row_bytes, k_byte), 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    vw[i] = __builtin_amdgcn_raw_buffer_load_b128(
                        resV, mad24(v_live, (uint32_t)i * row_bytes, v_byte), 0, 0);
                k_byte = mad24(k_live, (uint32_t)kAttKeys * row_bytes, k_byte);
                v_byte = mad24(v_live, (uint32_t)kAttKeys * row_bytes, v_byte);
            } else {
#pragma unroll
                for (int step = 0; step < kSteps; ++step)
                    kw[step] = load8_slow(ks + (int64_t)min(kb + step * kRowsStep + k_row, N - 1) * K, 8 * k_piece, K);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    vw[i] = load8_slow(vs + (int64_t)min(kb + 4 * v_kg + i, N - 1) * K, 8 * v_piece, K);
                // zeros past the head dimension and past the last key (values: their probabilities are zeros
                // too, but 0 * stale bits could be NaN)
#pragma unroll
                for (int step = 0; step < kSteps; ++step)
                    kw[step] = (kb + step * kRowsStep + k_row < N && 8 * k_piece < K) ? kw[step] : zero4;
#pragma unroll
                for (int i = 0; i < 4; ++i) vw[i] = (kb + 4 * v_kg + i < N && 8 * v_piece < K) ? vw[i] : zero4;
            }
        };
        if (N > 0) fetch(0);

        for (int kb = 0; kb < N; kb += kAttKeys) {
            __syncthreads();                           // the previous block (or round) is consumed
            // ---- keys: sK[key][k], one 16-byte piece per thread and step, pieces of a row on neighbouring lanes
            if (kLpr == kPieces || k_piece < kPieces) {
#pragma unroll
                for (int step = 0; step < kSteps; ++step)
                    *reinterpret_cast<u32x4 *>(sK + (step * kRowsStep + k_row) * kPitchK + k_piece * 16) = kw[step];
            }
            // ---- values, transposed: 8 runs of 4 keys, one per column of the thread's piece
            if (v_thread) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {          // word w of the four rows = columns 2w and 2w + 1
                    const uint32_t lo01 = __builtin_amdgcn_perm(vw[1][w], vw[0][w], 0x05040100u);
                    const uint32_t lo23 = __builtin_amdgcn_perm(vw[3][w], vw[2][w], 0x05040100u);
                    const uint32_t hi01 = __builtin_amdgcn_perm(vw[1][w], vw[0][w], 0x07060302u);
                    const uint32_t hi23 = __builtin_amdgcn_perm(vw[3][w], vw[2][w], 0x07060302u);
                    unsigned char *dst = sV + (8 * v_piece + 2 * w) * kAttPitchV + v_slot * 8;
                    *reinterpret_cast<u32x2 *>(dst) = u32x2{lo01, lo23};
                    *reinterpret_cast<u32x2 *>(dst + kAttPitchV) = u32x2{hi01, hi23};
                }
            }
            __syncthreads();
            if (kb + kAttKeys < N) fetch(kb + kAttKeys);
            if (nq == 0) continue;
            // The arithmetic on one block for NQ live strips, as straight-line code: a branch around every
            // matrix instruction of a strip that may be missing would keep the scheduler from interleaving them.
            auto block_math = [&](auto nq_tag) {
                constexpr int NQ = decltype(nq_tag)::value;
                // ---- scores of 64 keys x 16 queries per strip; a key operand read serves every strip
                f32x4 sacc[NQ][4];
    #pragma unroll
                for (int q = 0; q < NQ; ++q)
    #pragma unroll
                    for (int t = 0; t < 4; ++t) sacc[q][t] = f32x4{0.f, 0.f, 0.f, 0.f};
                u32x4 ring[kAttRing];
                {
                    constexpr int kReads = 4 * NK;         // read i: k step i / 4, key tile i % 4
                    static_for<kAttRing>([&](auto ic) {
                        constexpr int I = decltype(ic)::value;
                        if constexpr (I < kReads) lds_read128<16 * (I % 4) * kPitchK + 64 * (I / 4)>(ring[I], k_addr);
                    });
                    static_for<kReads>([&](auto ic) {
                        constexpr int I = decltype(ic)::value, R = I % kAttRing;
                        constexpr int kBehind = (I + kAttRing < kReads ? I + kAttRing : kReads) - (I + 1);
                        lds_wait<kBehind>(ring[R]);
    #pragma unroll
                        for (int q = 0; q < NQ; ++q) sacc[q][I % 4] = Elem<DT>::mfma(ring[R], qf[q][I / 4], sacc[q][I % 4]);
                        if constexpr (I + kAttRing < kReads)
                            lds_read128<16 * ((I + kAttRing) % 4) * kPitchK + 64 * ((I + kAttRing) / 4)>(ring[R], k_addr);
                    });
                }
                // ---- online softmax; lane holds keys kb + 16 t + 4 rg + e of query j of each strip
                const int left = N - kb;                   // keys of this block that exist
                u32x4 pf[NQ][2];
    #pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    f32x4(&sc)[4] = sacc[q];
                    // keys past the segment's last: -inf, so that they neither raise the maximum nor count
                    // (their exponentials are zeros)
                    if (left < kAttKeys) {
    #pragma unroll
                        for (int t = 0; t < 4; ++t)
    #pragma unroll
                            for (int e = 0; e < 4; ++e) sc[t][e] = 16 * t + 4 * rg + e < left ? sc[t][e] : -INFINITY;
                    }
                    settle_mfma(sc);                       // max3 reads the scores from inline assembly
                    float bm;                              // one statement: no padding between its instructions
                    asm volatile("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\t"
                                 "v_max3_f32 %0, %0, %8, %9\n\tv_max3_f32 %0, %0, %10, %11\n\tv_max3_f32 %0, %0, %12, %13\n\t"
                                 "v_max3_f32 %0, %0, %14, %15\n\tv_max_f32 %0, %0, %16"
                                 : "=&v"(bm)
                                 : "v"(sc[0][0]), "v"(sc[0][1]), "v"(sc[0][2]), "v"(sc[0][3]), "v"(sc[1][0]), "v"(sc[1][1]),
                                   "v"(sc[1][2]), "v"(sc[1][3]), "v"(sc[2][0]), "v"(sc[2][1]), "v"(sc[2][2]), "v"(sc[2][3]),
                                   "v"(sc[3][0]), "v"(sc[3][1]), "v"(sc[3][2]), "v"(sc[3][3]));
                    bm = quad_column_max_swap(bm);
                    // m is the reference the exponentials are taken against, not necessarily the maximum: it is
                    // raised (and the sums so far rescaled) only when a block's maximum passes it by more than
                    // 2^8 in the exponent, so probabilities stay below 256 (fine for both 16-bit types and the
                    // fp32 sums) and most blocks skip the rescale.  The comparison is false, i.e. raises, for the
                    // first block (m = -inf).
                    const bool raise = !((bm - m[q]) * c <= 8.0f);
                    const float m_new = raise ? bm : m[q];
                    const float m_use = m_new == -INFINITY ? 0.f : m_new;
                    const float alpha = !raise ? 1.0f : m[q] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m[q] - m_use) * c);
                    m[q] = m_new;
                    const float bias = -m_use * c;
                    float psum = 0.f;
    #pragma unroll
                    for (int t = 0; t < 4; ++t)
    #pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            float p = __builtin_amdgcn_exp2f(fmaf(sc[t][e], c, bias));
                            sc[t][e] = p;
                            psum += p;
                        }
                    lsum[q] = fmaf(lsum[q], alpha, psum);
                    if (__any(raise)) {
    #pragma unroll
                        for (int t = 0; t < kOutTiles; ++t) oacc[q][t] *= alpha;
                    }
                    // probabilities as B operand, 32 keys per step: k = 8 rg + kk is key 32 cc + 4 rg + kk (kk < 4)
                    // or 32 cc + 16 + 4 rg + kk - 4: what the lane holds in sc[2 cc] and sc[2 cc + 1]
    #pragma unroll
                    for (int cc = 0; cc < 2; ++cc)
                        pf[q][cc] = u32x4{Elem<DT>::pack2(sc[2 * cc][0], sc[2 * cc][1]), Elem<DT>::pack2(sc[2 * cc][2], sc[2 * cc][3]),
                                          Elem<DT>::pack2(sc[2 * cc + 1][0], sc[2 * cc + 1][1]),
                                          Elem<DT>::pack2(sc[2 * cc + 1][2], sc[2 * cc + 1][3])};
                }
                // ---- O^T += V^T P^T; a value operand read serves every strip
                {
                    constexpr int kReads = 2 * kOutTiles;  // read i: key half i / kOutTiles, output tile i % kOutTiles
                    static_for<kAttRing>([&](auto ic) {
                        constexpr int I = decltype(ic)::value;
                        if constexpr (I < kReads) lds_read128<16 * (I % kOutTiles) * kAttPitchV + 64 * (I / kOutTiles)>(ring[I], v_addr);
                    });
                    static_for<kReads>([&](auto ic) {
                        constexpr int I = decltype(ic)::value, R = I % kAttRing;
                        constexpr int kBehind = (I + kAttRing < kReads ? I + kAttRing : kReads) - (I + 1);
                        lds_wait<kBehind>(ring[R]);
    #pragma unroll
                        for (int q = 0; q < NQ; ++q)
                            oacc[q][I % kOutTiles] = Elem<DT>::mfma(ring[R], pf[q][I / kOutTiles], oacc[q][I % kOutTiles]);
                        if constexpr (I + kAttRing < kReads)
                            lds_read128<16 * ((I + kAttRing) % kOutTiles) * kAttPitchV + 64 * ((I + kAttRing) / kOutTiles)>(ring[R], v_addr);
                    });
                }
            };
            if (QT == 1 || nq == 1) block_math(std::integral_constant<int, 1>{});
            else block_math(std::integral_constant<int, QT>{});
        }
        // ---- normalise and store: lane (query j, rg) holds columns 16 t + 4 rg + e.  No key at all: zeros.
#pragma unroll
        for (int q = 0; q < QT; ++q) {
            if (q >= nq) continue;
            const int qr = r0 + kAttRows * q + j;
            const float l = quad_column_sum(lsum[q]);
            const float inv = N > 0 ? 1.0f / l : 0.f;
            if (qr < M) {
                uint16_t *orow = os + (int64_t)qr * K;
#pragma unroll
                for (int t = 0; t < kOutTiles; ++t) {
                    const int c0 = 16 * t + 4 * rg;
                    if (c0 + 4 <= K) {
                        *reinterpret_cast<u32x2_unaligned *>(orow + c0) =
                            u32x2{Elem<DT>::pack2(oacc[q][t][0] * inv, oacc[q][t][1] * inv),
                                  Elem<DT>::pack2(oacc[q][t][2] * inv, oacc[q][t][3] * inv)};
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (c0 + e < K) orow[c0 + e] = Elem<DT>::from_float(oacc[q][t][e] * inv);
                    }
                }
            }
        }
    }
}

template <int DT, int NK, int QT>
__global__ __launch_bounds__(kAttThreads, QT == 2 ? 2 : NK <= 2 ? 4 : 3) void attention_kernel(RunArgs a, const void *Vbuf) {
    constexpr int KP = 32 * NK;
    __shared__ __attribute__((aligned(16))) unsigned char sK[kAttKeys * (KP * 2 + 32)];
    __shared__ __attribute__((aligned(16))) unsigned char sV[KP * kAttPitchV];
    // (the row blocks per head come with the header: one memory round trip less than the prefix's last entry)
    const int64_t per_head = QT == 2 ? ((ConstHdr)(uintptr_t)a.plan)->att_blocks128 : ((ConstHdr)(uintptr_t)a.plan)->att_blocks64;
    if (!header_ok(a)) { report_mismatch(a); return; }
    // Workgroup -> (segment, head, row block).  Consecutive workgroup ids go to the eight dies of the chip in
    // turn, and each die has its own L2: id = die + 8 k.  All row blocks of one (segment, head) pair read the
    // same keys and values, so they should run on ONE die at about the same time.
    // With the row-block prefix (ride_slots = 1, launches that know the batch's totals): the existing
    // (head, segment, row block) items, head-major, are cut into eight contiguous shares, one per die, so the
    // row blocks of a pair sit side by side on one die and no workgroup is launched for a row block that does
    // not exist, except past the end of a share (the grid is sized from an upper bound of the item count).
    // Without it: pair = die + 8 (k mod pairs per die), row block k / pairs per die; a workgroup takes every
    // tile_zdim-th row block of its pair, and the workgroups that find no rows come last.
    const unsigned id = blockIdx.x, die = id & 7u, kk = id >> 3;
    int g, zblock;
    int64_t h;
    if (a.ride_slots) {
        const int32_t *pfx = plan_rowblocks(a.plan, a.nseg, QT - 1);
        const int64_t items = per_head * a.H, share = (items + 7) >> 3;
        const int64_t u = (int64_t)die * share + kk;
        // a grid too small for the plan's items: the host summary the launch was sized from is not this plan's
        if (id == 0 && threadIdx.x == 0 && share * 8 > (int64_t)gridDim.x)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        if (kk >= share || u >= items) return;
        h = u / per_head;
        const int item = (int)(u % per_head);
        g = prefix_search(pfx, a.nseg, item);
        zblock = item - ((ConstI32)(uintptr_t)pfx)[g];
    } else {
        const unsigned pairs8 = (unsigned)a.tile_groups;
        const int64_t pair = (int64_t)die + 8 * (int64_t)(kk % pairs8);
        zblock = (int)(kk / pairs8);
        if (pair >= (int64_t)a.nseg * a.H) return;
        g = (int)(pair / a.H);
        h = pair % a.H;
    }
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const SegRec rec = load_rec(pv.recs, g);
    const int M = rec.M, K = rec.K;
    if (M < 1 || K < 1) return;
    // the launch was sized for a smaller head dimension, or byte offsets inside the segment (of a last block of
    // keys that reaches past the segment's end, too) pass 32 bits
    if (K > KP || ((int64_t)max(M, rec.N) + kAttKeys) * K >= (int64_t(1) << 31)) {
        if (h == 0 && zblock == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    if ((K & 7) == 0) attention_body<DT, NK, QT, true>(a, Vbuf, rec, h, zblock, sK, sV);
    else attention_body<DT, NK, QT, false>(a, Vbuf, rec, h, zblock, sK, sV);
}

template <int DT, int QT>
static void launch_nk(int nk, dim3 grid, hipStream_t stream, const RunArgs &args, const void *V) {
    // args.ride_slots = 1: work items from the plan's row-block prefix; else args.tile_zdim = row blocks per
    // (segment, head) pair, tile_groups = pairs per die
    switch (nk) {
        case 1: hipLaunchKernelGGL((attention_kernel<DT, 1, QT>), grid, dim3(kAttThreads), 0, stream, args, V); break;
        case 2: hipLaunchKernelGGL((attention_kernel<DT, 2, QT>), grid, dim3(kAttThreads), 0, stream, args, V); break;
        case 3: hipLaunchKernelGGL((attention_kernel<DT, 3, QT>), grid, dim3(kAttThreads), 0, stream, args, V); break;
        default: hipLaunchKernelGGL((attention_kernel<DT, 4, QT>), grid, dim3(kAttThreads), 0, stream, args, V); break;
    }
}

// Strips per wavefront: two where segments are tall (each operand read from LDS then feeds two matrix
// instructions and a block of keys is staged half as often), one otherwise (more, lighter workgroups).

int launch_attention(int dtype, const RunArgs &args, const void *V, int64_t nseg, const ba_plan_info *info,
                     hipStream_t stream) {
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    static const int forced = [] { const char *e = getenv("BLOCKEDATTN_ATT_STRIPS"); return e ? atoi(e) : 0; }();
    int nk = 4, qt = 1;
    int64_t max_m = 512;
    if (info) {
        if (info->max_K > 128) return BA_ERR_UNSUPPORTED;
        nseg = info->nseg;
        nk = std::max(1, (info->max_K + 31) / 32);
        max_m = std::max<int64_t>(info->max_M, 1);
        if (info->total_rows >= 256 * std::max<int64_t>(nseg, 1)) qt = 2;   // mean segment height >= 256 (136: one strip is 6 % faster)
    }
    if (forced == 1 || forced == 2) qt = forced;
    // Row blocks per pair: enough for the tallest segment, but no more than four times what the mean segment
    // needs (a workgroup takes every Z-th block of its pair; blocks that do not exist cost a launch each).
    const int64_t round_rows = kAttRows * qt;
    int64_t z = std::min<int64_t>((max_m + round_rows - 1) / round_rows, 64);
    if (info) z = std::min<int64_t>(z, (4 * info->total_rows / std::max<int64_t>(nseg, 1) + round_rows - 1) / round_rows);
    z = std::max<int64_t>(z, 1);
    if (nseg <= 0) return BA_OK;
    RunArgs run = args;
    dim3 grid;
    if (info && info->total_rows >= 0) {
        // the batch's totals are known: one workgroup per existing row block, found through the plan's
        // row-block prefix (segments without keys count: their output rows are zeroed)
        const int64_t items = (int64_t)(qt == 2 ? info->att_blocks128 : info->att_blocks64) * args.H;
        if (items <= 0) return BA_OK;
        const int64_t share = (items + 7) / 8;
        if (share * 8 > 0x7fffffff) return BA_ERR_UNSUPPORTED;
        run.ride_slots = 1;
        grid = dim3((unsigned)(share * 8));
    } else {
        const int64_t pairs8 = (nseg * args.H + 7) / 8;    // pairs per die, rounded up
        if (pairs8 * z * 8 > 0x7fffffff || pairs8 > 0x7fffffff) return BA_ERR_UNSUPPORTED;
        run.tile_zdim = (int)z;
        run.tile_groups = (int)pairs8;
        grid = dim3((unsigned)(pairs8 * z * 8));
    }
    if (dtype == BA_F16) { if (qt == 2) launch_nk<0, 2>(nk, grid, stream, run, V); else launch_nk<0, 1>(nk, grid, stream, run, V); }
    else { if (qt == 2) launch_nk<1, 2>(nk, grid, stream, run, V); else launch_nk<1, 1>(nk, grid, stream, run, V); }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
