// The row-block kernel: S_g = A_g B_g^T and its row softmax for large segments (the tile kernel's class:
// N > 256, or N >= 128 with an operand too large for the strip kernel's LDS window) with K <= 128, written
// so that every line of the result is stored whole.
//
// One workgroup = 8 wavefronts = 256 rows of one segment and head; wavefront w owns rows 32w .. 32w+31 (two
// MFMA row tiles) and ALL columns, 64 at a time.  B_g streams through four 16 KiB LDS stages (64 rows of
// B_g x 128 k, fetched with direct global->LDS loads, 16-byte pieces XOR-permuted inside each 256-byte row
// by row/4 so that the sixteen lanes of an operand read hit sixteen bank groups).  The A fragments of the
// wavefront's rows stay in registers.
//
// Score layout: lane (j = lane%16, rg = lane/16) holds rows 16 rt + 4 rg + i (i = 0..3) and the FOUR
// CONSECUTIVE columns 4j .. 4j+3 of the chunk (column tile ct takes the B rows 4j + ct).
//
// Softmax in two sweeps over the columns.  Sweep 1 sums exp2((s - R) c) per row with R = the row's maximum
// over the FIRST chunk (the sum then holds a term 1, so it cannot vanish; should a later score exceed R by
// more than the exponent range, the sum overflows, which is seen when the sweep ends, and the row block is
// done again with a running maximum).  Sweep 2 recomputes the scores and writes
// exp2(s c - R c - log2(sum)).  The matrix instructions of chunk t+1 and the softmax arithmetic of chunk t
// are threaded through each other by hand, one matrix instruction and one score element at a time (x = s c +
// ref, then exp2 of the previous x, then the use of the exponential before that), with scheduling barriers
// that keep the order: the matrix unit then works in the shadow of the vector and transcendental
// instructions of the same wavefront (measured: a 16x16x32 matrix instruction plus two vector instructions
// plus one exp2 take 23 cycles together, 16 and 24 cycles apart).
//
// Stores.  Rows of the result are N elements long and start at any 2-byte phase; a 128-byte line that is
// written in two partial pieces costs about 2.6 times a line written whole (store microbenchmark: 3.0 to
// 3.4 TB/s against 5.7 TB/s).  So each wavefront passes its 32 x 64 block through a ring in LDS (one row of
// 128 columns per result row, private to the wavefront) and reads it back shifted by the row's own phase:
// per chunk and row exactly ONE line-aligned 128-byte window leaves, eight lanes x 16 bytes, eight rows
// per store instruction.  The pieces at the two ends of a row that the windows cannot cover whole are
// written by one unaligned 16-byte store each (columns [0, 8) and [N-8, N); overlapping pieces carry
// identical values).
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "tile_body.hpp"

namespace ba {

constexpr int kRbWaves = 8;
constexpr int kRbThreads = 64 * kRbWaves;
constexpr int kRbWaveRows = 32;
constexpr int kRbRT = kRbWaveRows / 16;                 // MFMA row tiles per wavefront
constexpr int kRbRows = kRbWaves * kRbWaveRows;          // 256 rows per workgroup
constexpr int kRbCols = 64;                               // columns per chunk
constexpr int kRbRowBytes = 256;                          // one row of B_g in LDS: 128 k
constexpr int kRbStageBytes = kRbCols * kRbRowBytes;      // 16 KiB
constexpr int kRbStages = 4;
constexpr int kRbFillInsts = kRbStageBytes / 1024 / kRbWaves;   // global->LDS instructions per wavefront and chunk (2)
constexpr int kRbStoreInsts = 4;                          // window stores per wavefront and chunk
constexpr int kRingPitch = 288;                           // 128 columns + a copy of the first 16 behind them
constexpr int kRingBytes = kRbWaveRows * kRingPitch;      // per wavefront
constexpr int kRbFlagOffset = kRbStages * kRbStageBytes + kRbWaves * kRingBytes;
constexpr int kRbLdsBytes = kRbFlagOffset + 16;
constexpr uint32_t kOutOfRange = 0x80000000u;             // byte offset no segment reaches (areas are below 2^31 bytes)

__device__ __forceinline__ void wait_vm_upto(int n) {     // n even, wave-uniform; larger values wait for less
    switch (n >> 1) {
        case 0: wait_vm<0>(); break;
        case 1: wait_vm<2>(); break;
        case 2: wait_vm<4>(); break;
        case 3: wait_vm<6>(); break;
        case 4: wait_vm<8>(); break;
        case 5: wait_vm<10>(); break;
        case 6: wait_vm<12>(); break;
        case 7: wait_vm<14>(); break;
        case 8: wait_vm<16>(); break;
        case 9: wait_vm<18>(); break;
        case 10: wait_vm<20>(); break;
        case 11: wait_vm<22>(); break;
        default: wait_vm<24>(); break;
    }
}

// Sixteen bytes of a ring row starting at byte `pos` (any even value below 256): five aligned words, shifted.
__device__ __forceinline__ u32x4 ring_read16(const unsigned char *row, int pos) {
    const uint32_t *w = reinterpret_cast<const uint32_t *>(row + (pos & ~3));
    const uint32_t d0 = w[0], d1 = w[1], d2 = w[2], d3 = w[3], d4 = w[4];
    const uint32_t sh = (uint32_t)(pos & 2) * 8;
    return u32x4{__builtin_amdgcn_alignbit(d1, d0, sh), __builtin_amdgcn_alignbit(d2, d1, sh),
                 __builtin_amdgcn_alignbit(d3, d2, sh), __builtin_amdgcn_alignbit(d4, d3, sh)};
}

// WIDE: the build for 128 < K <= 256.  A chunk of B_g then takes TWO stages (k below 128, k from 128 on), so the four
// stages hold two chunks and a chunk is requested one iteration ahead instead of three; a wavefront keeps sixteen A
// fragments per row tile.
template <int DT, bool FUSED, bool WIDE>
__global__ __launch_bounds__(kRbThreads, 8 / kRbWaves) void rowblock_kernel(RunArgs a, int zdim, int weave) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    constexpr int kSlots = WIDE ? kRbStages / 2 : kRbStages;      // chunks of B_g the stages hold
    constexpr int kSlotStages = WIDE ? 2 : 1;
    const unsigned block = blockIdx.x;
    const int die = block % kDies, slot = block / kDies;
    // `weave` pairs of a die take turns in the die's slots (pair fastest, then the pair's workgroups)
    const int turn = slot % (zdim * weave);
    const int pair = ((slot / (zdim * weave)) * weave + turn % weave) * kDies + die;
    const int z0 = turn / weave;
    const int H = (int)a.H;
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    if (!header_ok(a)) {
        if (!(a.flags & kFlagQuiet) && block == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    // Workgroup -> (list entry, head, row block).  Consecutive workgroup ids go to the eight dies in turn, each with
    // its own L2; all row blocks of one (entry, head) pair read the same B_g, so they run on ONE die, one after
    // the other: id = 8 slot + die works on pair 8 (slot / zdim) + die, row block slot % zdim (weave = 1).  The pairs are
    // numbered entry-major with the entries in order of DECREASING work (M N): the long workgroups start first,
    // the short ones fill the gaps at the end, and every die gets two heads in eight of every entry.
    const int entries = a.list < 0 ? a.nseg : (int)((ConstHdr)(uintptr_t)a.plan)->totals[a.list];
    if (entries <= 0 || pair >= entries * H) return;
    const int h = pair % H;
    int entry = pair / H;
    if (entries <= 64) {
        // rank of every entry by work, one entry per lane; the workgroup takes the entry of rank pair / H
        const int lane0 = lane_id();
        const ConstSeg list = pv.recs + (int64_t)(a.list + 1) * plan_cap(a.nseg);
        int64_t work = -1;
        if (lane0 < entries) {
            const SegRec *r = reinterpret_cast<const SegRec *>((uintptr_t)(list + lane0));
            work = (int64_t)r->M * r->N;
        }
        int rank = 0;
        for (int e = 0; e < entries; ++e) {
            const int64_t other = uniform64(__shfl(work, e));
            rank += (other > work || (other == work && e < lane0)) ? 1 : 0;
        }
        const uint64_t hit = __ballot(lane0 < entries && rank == entry);
        entry = hit ? (int)__builtin_ctzll(hit) : entries;
        if (entry >= entries) return;
    }
    bool valid;
    const Seg s = load_listed(pv, entry, h, a, valid);
    if (!valid || !tile_segment(s.kind, s.N, s.K)) return;
    const int M = s.M, N = s.N, K = s.K;
    if (z0 * kRbRows >= M) return;
    if constexpr (WIDE) {
        if (K <= 128 || K > 256) return;                  // the other kernels of the call take it
        if (threadIdx.x == 0) atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->wide_groups, 1);
    } else if (K > 128) {
        // the wide build or the tile kernel of the same call takes it; without them the launch was sized for another plan
        if (!(a.flags & kFlagWideKToo) && z0 == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const SegRes res = make_res(s, a.A, a.B);
    const char *bseg = reinterpret_cast<const char *>((const uint16_t *)a.B + s.b);
    char *oseg = reinterpret_cast<char *>(a.out) + s.o * 2;
    const __amdgpu_buffer_rsrc_t out_res =
        __builtin_amdgcn_make_buffer_rsrc(oseg, 0, (int)((uint32_t)M * (uint32_t)N * 2u), kRsrcFlags);
    const uint32_t out_phase = (uint32_t)(uintptr_t)oseg;   // low address bits decide the line phase of a row
    unsigned char *ring = lds + kRbStages * kRbStageBytes + wave * kRingBytes;
    volatile int *flags = reinterpret_cast<volatile int *>(lds + kRbFlagOffset);

    const int ncb = (N + kRbCols - 1) / kRbCols;
    const int total = (FUSED ? 2 : 1) * ncb;
    const int ksteps = (K + 31) >> 5;
    const int kpieces = K >> 3;                            // 16-byte pieces per row of B_g
    const float c_signed = a.scale * kLog2e;
    const bool negate = FUSED && c_signed < 0.f;          // |scale| on negated scores
    const float c = __builtin_fabsf(c_signed);
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    // Stale or never written LDS must not reach a matrix instruction as NaN bits: pieces past K and rows past N
    // are never filled, so the stages start as zeros.
    for (int off = (int)threadIdx.x * 16; off < kRbStages * kRbStageBytes; off += kRbThreads * 16)
        *reinterpret_cast<u32x4 *>(lds + off) = zero4;
    __syncthreads();                                      // no fill may land under a late zero

    // Fill of one chunk: instruction i (0..15) covers LDS rows 4i .. 4i+3 of the stage; lane l writes row
    // 4i + l/16, slot l%16, which holds piece (l%16) ^ (i%16) of that row.  Wavefront w issues i = w + kRbWaves n.
    // Address = scalar base of the chunk inside B_g + a lane offset that never changes.
    // Written as assembly on purpose: the compiler orders every LDS access behind ALL outstanding vector memory
    // operations once it has seen a load into LDS (it cannot tell the stages apart), which would make each
    // operand read wait for the fill just requested and for every store in flight.  The waits for the fills
    // are explicit (wait_vm + barrier in the main loop).
    uint32_t fill_off[kRbFillInsts];
#pragma unroll
    for (int n = 0; n < kRbFillInsts; ++n) {
        const int i = wave + kRbWaves * n;
        const int piece = (lane & 15) ^ (i & 15);
        fill_off[n] = (uint32_t)((4 * i + (lane >> 4)) * K + piece * 8) * 2u;
    }
    // `slot`: which of the kSlots chunk places of the stages; span sp of a chunk (k from 128 sp on) goes to stage
    // kSlotStages slot + sp
    auto fill = [&](int cbi, int slot) __attribute__((always_inline)) {
        const int cb = cbi * kRbCols;
#pragma unroll
        for (int sp = 0; sp < kSlotStages; ++sp) {
            // (wave-uniform by construction; pinned so that the assembly below always gets scalar registers)
            const char *base = reinterpret_cast<const char *>(
                (uintptr_t)uniform64((int64_t)(uintptr_t)(bseg + (size_t)cb * K * 2 + 256 * sp)));
            const int span_pieces = kpieces - 16 * sp;          // pieces of a row that this span holds (at most 16 of them)
            const bool whole = span_pieces >= 16 && cb + kRbCols <= N;      // every lane of every instruction has something to fetch
#pragma unroll
            for (int n = 0; n < kRbFillInsts; ++n) {
                const uint32_t dst = (uint32_t)uniform(
                    (int)(uint32_t)(uintptr_t)(lds + (slot * kSlotStages + sp) * kRbStageBytes + (wave + kRbWaves * n) * 1024));
                if (whole) {
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                 :: "v"(fill_off[n]), "s"(base), "s"(dst) : "memory", "m0");
                } else if (cb + 4 * (wave + kRbWaves * n) + (lane >> 4) < N &&
                           ((lane & 15) ^ ((wave + kRbWaves * n) & 15)) < span_pieces) {
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                                 :: "v"(fill_off[n]), "s"(base), "s"(dst) : "memory", "m0");
                }
            }
        }
    };
    // operand read offsets of this lane inside a stage: row 4j + ct, piece 4ks + rg at slot (4ks + rg) ^ j
    int boff[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) boff[ks] = 1024 * j + 16 * ((4 * ks + rg) ^ j);

    // KS = k-steps of 32 the matrix instructions run over: 2 for K <= 64, 4 for K <= 128, 8 in the WIDE build (fragments past K are zeros)
    auto run = [&](auto ks_c) __attribute__((always_inline)) {
    constexpr int KS = decltype(ks_c)::value;
    for (int rb = z0; rb * kRbRows < M; rb += zdim) {
        const int row0 = rb * kRbRows + wave * kRbWaveRows;     // first row of this wavefront
        const bool active = row0 < M;
        // ---- A fragments [rt][ks]: row 16 rt + j, k = 32 ks + 8 rg ..
        u32x4 af[kRbRT][KS];
#pragma unroll
        for (int rt = 0; rt < kRbRT; ++rt) {
            const int voff = ((row0 + 16 * rt + j) * K + rg * 8) * 2;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                u32x4 v = zero4;
                if (ks < ksteps) {
                    v = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff + ks * 64, 0, 0);
                    if (ks * 32 + rg * 8 >= K) v = zero4;            // ragged last k-step
                    if (negate) v ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
                }
                af[rt][ks] = v;
            }
        }
        // ---- store lanes: instruction t writes rows 8t + lane/8, piece lane%8 of the row's aligned window
        const int q = lane & 7;
        int upos[kRbStoreInsts];                   // ring byte of the lane's piece in window 0: 2 (8q - d) mod 256
        uint32_t v0[kRbStoreInsts];                // byte offset of that piece inside the segment's result
        const unsigned char *rbase0 = ring + (lane >> 3) * kRingPitch;
#pragma unroll
        for (int t = 0; t < kRbStoreInsts; ++t) {
            const int rho = row0 + 8 * t + (lane >> 3);
            const bool row_ok = rho < M;
            const int rn = row_ok ? rho * N : 0;
            const int d = (int)(((out_phase + 2u * (uint32_t)rn) & 127u) >> 1);     // columns before the row's first line boundary
            upos[t] = (16 * q - 2 * d) & 255;
            v0[t] = row_ok ? (uint32_t)(2 * (rn + 8 * q - d)) : kOutOfRange;
        }

        bool safe = false;
        for (int attempt = 0; attempt < 2; ++attempt) {
            if (rb != z0 || attempt != 0) {
                wait_vm<0>();
                __syncthreads();                         // everyone is done with the stages and the flags
            }
            if (threadIdx.x == 0) { flags[0] = 0; flags[1] = 0; }
            int f_cbi = 0;                               // chunk (inside its sweep) of the next fill
            for (int k = 0; k < kSlots - 1; ++k)
                if (k < total) {
                    fill(f_cbi, k);
                    if (++f_cbi == ncb) f_cbi = 0;
                }
            // The A fragments are complete before the loop starts: otherwise the compiler, which sees their loads
            // pending on the way into the loop, waits for ALL vector memory operations at their first use in
            // every iteration, stores in flight included.
            wait_vm<0>();
            // per-row state: sweep 1: ref = -R c (bias of the exponent) and the running sum; sweep 2: ref = -R c - log2(sum)
            float ref[kRbRT][4], sum[kRbRT][4], rmax[kRbRT][4];
#pragma unroll
            for (int rt = 0; rt < kRbRT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) { ref[rt][i] = 0.f; sum[rt][i] = 0.f; rmax[rt][i] = -3.0e38f; }
            f32x4 acc[2][kRbRT][4];
            bool restart = false;

            // -------- out of the ring: one line-aligned 128-byte window per row and chunk.  Interior chunks: every
            // piece of the window exists; rows 16h .. 16h+15 of the wavefront leave as soon as they are in the ring
            // (store instructions 2h, 2h+1), in the middle of the matrix instructions.
            auto ring_copy_heads = [&](int first_row) __attribute__((always_inline)) {
                // the first 32 bytes of sixteen ring rows once more behind the rows: pieces that start in a row's
                // last 16 bytes continue there
                const unsigned char *src = ring + (first_row + (lane >> 2)) * kRingPitch + (lane & 3) * 8;
                *reinterpret_cast<u32x2 *>(const_cast<unsigned char *>(src) + 256) = *reinterpret_cast<const u32x2 *>(src);
                asm volatile("" ::: "memory");
            };
            auto ring_store_half = [&](int cbi, auto half_c) __attribute__((always_inline)) {
                constexpr int h = decltype(half_c)::value;
                if (cbi == 0 || cbi == ncb - 1) return;   // first and last chunk: ring_store_edge, behind the matrix instructions
                asm volatile("" ::: "memory");            // the reads below see the writes above (same wavefront, in order)
                if ((cbi & 1) == 0) ring_copy_heads(16 * h);
                const int par = (cbi & 1) << 7;
                const uint32_t adv = 128u * (uint32_t)cbi;      // the range check sees the vector offset only
#pragma unroll
                for (int t = 2 * h; t < 2 * h + 2; ++t) {
                    const u32x4 v = ring_read16(rbase0 + t * 8 * kRingPitch, upos[t] ^ par);
                    __builtin_amdgcn_raw_buffer_store_b128(v, out_res, v0[t] == kOutOfRange ? kOutOfRange : v0[t] + adv, 0, kResultAux);
                }
                asm volatile("" ::: "memory");
            };
            // First or last chunk: pieces before column 0 or past column N are dropped, and the end pieces the
            // windows cannot cover whole are written by one unaligned store each (lane l < 32: row l).
            auto ring_store_edge = [&](int cbi) __attribute__((always_inline)) {
                asm volatile("" ::: "memory");
                if ((cbi & 1) == 0) { ring_copy_heads(0); ring_copy_heads(16); }
                const int par = (cbi & 1) << 7;
                const uint32_t adv = 128u * (uint32_t)cbi;
                const int et_row = row0 + (lane & 31);
                const uint32_t et_off = (lane < 32 && et_row < M) ? (uint32_t)(2 * (et_row * N)) : kOutOfRange;
                const unsigned char *et_base = ring + (lane & 31) * kRingPitch;
#pragma unroll
                for (int t = 0; t < kRbStoreInsts; ++t) {
                    const u32x4 v = ring_read16(rbase0 + t * 8 * kRingPitch, upos[t] ^ par);
                    const int col = (((upos[t] >> 1) + 64) & 127) - 64 + kRbCols * cbi;      // first column of the piece
                    const uint32_t voff = (col < 0 || col + 8 > N || v0[t] == kOutOfRange) ? kOutOfRange : v0[t] + adv;
                    __builtin_amdgcn_raw_buffer_store_b128(v, out_res, voff, 0, kResultAux);
                }
                if (cbi == 0) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(et_base);          // columns [0, 8)
                    __builtin_amdgcn_raw_buffer_store_b128(v, out_res, et_off, 0, kResultAux);
                }
                if (cbi == ncb - 1) {
                    // the window behind the last chunk (what is left of the rows), then columns [N-8, N)
                    const int par2 = (ncb & 1) << 7;
#pragma unroll
                    for (int t = 0; t < kRbStoreInsts; ++t) {
                        const u32x4 v = ring_read16(rbase0 + t * 8 * kRingPitch, upos[t] ^ par2);
                        const int col = (((upos[t] >> 1) + 64) & 127) - 64 + kRbCols * ncb;
                        const uint32_t voff = (col + 8 <= N && v0[t] != kOutOfRange) ? v0[t] + 128u * (uint32_t)ncb : kOutOfRange;
                        __builtin_amdgcn_raw_buffer_store_b128(v, out_res, voff, 0, kResultAux);
                    }
                    const u32x4 v = ring_read16(et_base, (2 * (N - 8)) & 255);
                    __builtin_amdgcn_raw_buffer_store_b128(v, out_res, et_off == kOutOfRange ? kOutOfRange : et_off + 2u * (uint32_t)(N - 8), 0, kResultAux);
                }
                asm volatile("" ::: "memory");
            };

            // -------- the matrix instructions of chunk `it` with the arithmetic of chunk `it - 1` threaded between
            // them by hand: after every matrix instruction comes the share of one (KS = 4) or two (KS = 2) score
            // elements of the previous chunk, and a scheduling barrier keeps that order.  The matrix unit then
            // works under the vector and transcendental instructions of the same wavefront.
            // MODE 0: matrix instructions only; 1: sweep 1 (sum += w * exp2(s c + ref)); 2: values to the ring
            // (sweep 2: exp2(s c + ref); GEMM alone: s itself).  The operand reads of k-step ks + 1 are issued
            // before the matrix instructions of k-step ks.
            auto chunk_body = [&](auto mode_c, auto wt_c, auto buf_c, int stage, int cbi_prev) __attribute__((always_inline)) {
                constexpr int MODE = decltype(mode_c)::value;
                constexpr bool WT = decltype(wt_c)::value;       // sweep 1 only: the chunk has columns that do not exist
                constexpr int b = decltype(buf_c)::value, pb = 1 - b;
                constexpr int EPM = KS == 2 ? 2 : 1;          // score elements per matrix instruction (KS = 8: of the first four k-steps)
                const unsigned char *sb = lds + stage * (kSlotStages * kRbStageBytes);      // (stage: the chunk's slot)
                const int cbp = cbi_prev * kRbCols;
                float w[4];                                   // 0 for columns that do not exist (ragged last chunk)
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) w[ct] = (!WT || cbp + 4 * j + ct < N) ? 1.f : 0.f;
                unsigned char *wrow = ring + (4 * rg) * kRingPitch + (((cbi_prev & 1) << 6) + 4 * j) * 2;
                u32x4 bf[2][4];
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) bf[0][ct] = *reinterpret_cast<const u32x4 *>(sb + boff[0] + 256 * ct);
                // Per score element three steps, one matrix instruction apart, so that no instruction waits for
                // the one just issued: x = s c + ref; p = exp2(x); use of p (sum, or pack into the ring).
                float xprev = 0.f, pprev = 0.f;
                float quad[4];
                constexpr int NE = 32;                        // score elements per lane and chunk
                auto use = [&](auto e_c, float pv) {
                    constexpr int pe = decltype(e_c)::value, prt = pe >> 4, pi = (pe >> 2) & 3, pct = pe & 3;
                    if constexpr (MODE == 1) sum[prt][pi] = WT ? fmaf(pv, w[pct], sum[prt][pi]) : sum[prt][pi] + pv;
                    else if constexpr (MODE == 2) {
                        quad[pct] = pv;
                        if constexpr (pct == 3) {
                            const u32x2 v = {Elem<DT>::pack2(quad[0], quad[1]), Elem<DT>::pack2(quad[2], quad[3])};
                            *reinterpret_cast<u32x2 *>(wrow + (16 * prt + pi) * kRingPitch) = v;
                            if constexpr (pe == 15) ring_store_half(cbi_prev, std::integral_constant<int, 0>{});   // rows 0..15 are in the ring
                        }
                    }
                };
                auto power = [&](float x) {
                    return (MODE == 1 || FUSED) ? __builtin_amdgcn_exp2f(x) : x;
                };
                auto element = [&](auto e_c) {
                    constexpr int e = decltype(e_c)::value, rt2 = e >> 4, i2 = (e >> 2) & 3, ct2 = e & 3;
                    if constexpr (e >= 2) use(std::integral_constant<int, e - 2>{}, pprev);
                    if constexpr (e >= 1) pprev = power(xprev);
                    const float sc = acc[pb][rt2][ct2][i2];
                    xprev = (MODE == 1 || FUSED) ? fmaf(sc, c, ref[rt2][i2]) : sc;
                };
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks + 1 < KS) {
#pragma unroll
                        for (int ct = 0; ct < 4; ++ct)
                            bf[(ks + 1) & 1][ct] = *reinterpret_cast<const u32x4 *>(sb + ((ks + 1) >> 2) * kRbStageBytes + boff[(ks + 1) & 3] + 256 * ct);
                    }
                    auto group = [&](auto qd_c) {
                        constexpr int qd = decltype(qd_c)::value, rt = qd >> 2, ct = qd & 3;
                        acc[b][rt][ct] = Elem<DT>::mfma(af[rt][ks], bf[ks & 1][ct],
                                                        ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[b][rt][ct]);
                        if constexpr (MODE != 0) {
                            if (ks == 0) { if constexpr (EPM == 1) element(std::integral_constant<int, 0 * 8 + qd>{}); else { element(std::integral_constant<int, (0 * 8 + qd) * 2>{}); element(std::integral_constant<int, (0 * 8 + qd) * 2 + 1>{}); } }
                            if (ks == 1) { if constexpr (EPM == 1) element(std::integral_constant<int, 1 * 8 + qd>{}); else { element(std::integral_constant<int, (1 * 8 + qd) * 2>{}); element(std::integral_constant<int, (1 * 8 + qd) * 2 + 1>{}); } }
                            if constexpr (KS >= 4) {
                                if (ks == 2) element(std::integral_constant<int, 2 * 8 + qd>{});
                                if (ks == 3) element(std::integral_constant<int, 3 * 8 + qd>{});
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    };
                    group(std::integral_constant<int, 0>{}); group(std::integral_constant<int, 1>{});
                    group(std::integral_constant<int, 2>{}); group(std::integral_constant<int, 3>{});
                    group(std::integral_constant<int, 4>{}); group(std::integral_constant<int, 5>{});
                    group(std::integral_constant<int, 6>{}); group(std::integral_constant<int, 7>{});
                }
                if constexpr (MODE != 0) {
                    use(std::integral_constant<int, NE - 2>{}, pprev);
                    pprev = power(xprev);
                    use(std::integral_constant<int, NE - 1>{}, pprev);
                    if constexpr (MODE == 2) ring_store_half(cbi_prev, std::integral_constant<int, 1>{});
                }
            };

            // -------- sweep 1: row statistics of one chunk.  stats_reference (first chunk, or every chunk of the
            // repeated sweep) moves the reference to the row maximum so far; stats_sum adds the chunk's terms.
            auto stats_reference = [&](auto buf_c, int cbi) __attribute__((always_inline)) {
                constexpr int b = decltype(buf_c)::value;
                const int cb = cbi * kRbCols;
#pragma unroll
                for (int rt = 0; rt < kRbRT; ++rt) {
                    float mx[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float m = -INFINITY;
#pragma unroll
                        for (int ct = 0; ct < 4; ++ct)
                            m = __builtin_fmaxf(m, cb + 4 * j + ct < N ? acc[b][rt][ct][i] : -INFINITY);
                        mx[i] = m;
                    }
                    row16_max4(mx);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float r_new = __builtin_fmaxf(rmax[rt][i], mx[i]);
                        // the sum so far moves to the new reference (a first chunk has no sum yet)
                        if (cbi != 0) sum[rt][i] *= __builtin_amdgcn_exp2f((rmax[rt][i] - r_new) * c);
                        rmax[rt][i] = r_new;
                        ref[rt][i] = -r_new * c;
                    }
                }
            };
            // after the last chunk of sweep 1: row sums over the sixteen lanes; returns whether any is not finite
            auto finish_stats = [&]() __attribute__((always_inline)) {
                bool bad = false;
#pragma unroll
                for (int rt = 0; rt < kRbRT; ++rt) {
                    float sm[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) sm[i] = sum[rt][i];
                    row16_sum4(sm);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        bad |= !(sm[i] <= 3.0e38f);
                        ref[rt][i] -= __builtin_amdgcn_logf(sm[i]);      // 1/sum goes into the exponent
                    }
                }
                return bad;
            };

            // ... and out of it: one line-aligned window per row, plus the end pieces at the first and last chunk
            // -------- one iteration: matrix instructions of chunk `it` into accumulator set it % 2 from stage
            // it % 2, arithmetic of chunk `it - 1` from the other set.  SYNC: wait for this wavefront's part of
            // chunk `it` (requested one iteration ago, right behind that iteration's barrier, with a scheduling
            // barrier behind it: only that iteration's LATER window stores may still be in flight), barrier (now
            // everyone's part is there and nobody reads the other stage any more), request chunk it + 1.
            using False = std::false_type;
            using True = std::true_type;
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            auto iterate = [&](auto par_c, auto mode_c, auto wt_c, auto later_c, auto sync_c, int it, int cbi_prev) __attribute__((always_inline)) {
                if constexpr (decltype(sync_c)::value) {
                    if constexpr (kSlots == 2) {
                        wait_vm<decltype(later_c)::value>();
                    } else {
                        // fill of chunk `it`: requested kRbStages - 1 iterations ago; the fills requested since and the
                        // window stores of those iterations (each behind its iteration's fill) may stay in flight
                        int later = 0;
#pragma unroll
                        for (int k = 1; k <= kSlots - 2; ++k) {
                            // (the fill of a ragged last chunk is not counted: its instructions for rows past N
                            // are skipped altogether, so fewer than kRbFillInsts may have been issued)
                            const int c = it + k, last = c == ncb - 1 || c == 2 * ncb - 1;
                            if (c < total && !((N & (kRbCols - 1)) != 0 && last)) later += kRbFillInsts;
                        }
                        if (active) {
                            const int first_store = (FUSED ? ncb : 0) + 1;    // first iteration whose body stores (interior chunks: 4 instructions)
#pragma unroll
                            for (int back = 1; back <= kSlots - 1; ++back) {
                                const int cb2 = it - back - first_store;      // chunk that iteration stored
                                if (cb2 >= 1 && cb2 < ncb - 1) later += kRbStoreInsts;
                            }
                        }
                        wait_vm_upto(later);
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    if (it + kSlots - 1 < total) {
                        fill(f_cbi, (it + kSlots - 1) & (kSlots - 1));
                        if (++f_cbi == ncb) f_cbi = 0;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (active) chunk_body(mode_c, wt_c, par_c, it & (kSlots - 1), cbi_prev);   // it % 2 == par
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            };
            const bool ragged = (N & (kRbCols - 1)) != 0;
            // The two accumulator sets alternate; the loops below are unrolled by two so that each body names its
            // registers outright (a run-time choice between the sets makes the compiler merge the two bodies and
            // copy 64 registers per iteration).  for_range(lo, hi, f): f(parity, it) for it = lo .. hi.
            auto for_range = [&](int lo, int hi, auto &&f) __attribute__((always_inline)) {
                int it = lo;
                if (it <= hi && (it & 1)) { f(I1{}, it); ++it; }
                for (; it + 1 <= hi; it += 2) { f(I0{}, it); f(I1{}, it + 1); }
                if (it <= hi) f(I0{}, it);
            };
            iterate(I0{}, I0{}, False{}, I0{}, True{}, 0, 0);
            if (FUSED) {
                // sweep 1: iteration `it` adds the terms of chunk it - 1
                for_range(1, ncb, [&](auto par_c, int it) {
                    constexpr int par = decltype(par_c)::value;
                    if (active && (it == 1 || safe)) stats_reference(std::integral_constant<int, 1 - par>{}, it - 1);
                    if (it == ncb && ragged) iterate(par_c, I1{}, True{}, I0{}, True{}, it, it - 1);
                    else iterate(par_c, I1{}, False{}, I0{}, True{}, it, it - 1);
                });
                // the statistics are complete: an overflowed sum sends the whole workgroup through sweep 1 again
                const bool bad = active && finish_stats();
                if (!safe) {
                    if (__ballot(bad) != 0 && lane == 0) flags[attempt] = 1;
                    wait_vm<0>();
                    __syncthreads();
                    restart = flags[attempt] != 0;
                }
            }
            if (!restart) {
                // sweep 2 (or the GEMM alone): iteration `it` stores chunk it - 1 - first; the iteration behind the
                // last chunk runs the matrix instructions once more, on whatever the stage holds, and drops the
                // result (one code path)
                const int first = FUSED ? ncb : 0;
                for_range(first + 1, total, [&](auto par_c, int it) {
                    const int cbi = it - 1 - first;
                    if (it == total) iterate(par_c, I2{}, False{}, I0{}, False{}, it, cbi);
                    else if (cbi >= 1 && active) iterate(par_c, I2{}, False{}, std::integral_constant<int, kRbStoreInsts>{}, True{}, it, cbi);
                    else iterate(par_c, I2{}, False{}, I0{}, True{}, it, cbi);
                    if (active && (cbi == 0 || cbi == ncb - 1)) ring_store_edge(cbi);
                });
            }
            if (!restart) break;
            safe = true;
        }
    }
    };
    if constexpr (WIDE) run(std::integral_constant<int, 8>{});
    else if (K <= 64) run(std::integral_constant<int, 2>{});
    else run(std::integral_constant<int, 4>{});
}

template <int DT, bool FUSED, bool WIDE = false>
static int launch_rb(const RunArgs &args, unsigned groups, int zdim, int weave, hipStream_t stream) {
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&rowblock_kernel<DT, FUSED, WIDE>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kRbLdsBytes);
    if (attr != hipSuccess) return BA_ERR_LAUNCH;
    hipLaunchKernelGGL((rowblock_kernel<DT, FUSED, WIDE>), dim3(groups), dim3(kRbThreads), kRbLdsBytes, stream, args, zdim, weave);
    return BA_OK;
}

// Launches the row-block kernel over (list entry, head, row block of 256 rows).  Needs the plan summary:
// every segment must have K <= 128 (the A fragments of a wavefront's rows stay in registers); wide: the build for
// 128 < K <= 256, which passes over the segments outside that range.
static int launch_rowblocks_any(bool wide, int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                                hipStream_t stream) {
    if (!info || (args.flags & kFlagOutF32)) return BA_ERR_UNSUPPORTED;
    if (wide ? info->max_K <= 128 : (info->max_K > 128 && !(args.flags & kFlagWideKToo))) return BA_ERR_UNSUPPORTED;
    if (slots <= 0) return BA_OK;
    int64_t pairs = (slots * args.H + kDies - 1) / kDies * kDies;   // (entry, head) pairs, padded to whole dies
    // Workgroups per pair Z (workgroup z of a pair takes its row blocks z, z + Z, ..) and pairs of a die that take
    // turns in the grid.  Sixteen workgroups of one pair that start together fetch the same lines of B_g at the same
    // moment, and a compute unit waits about 10 us between two workgroups (stores of the one draining, dispatch of
    // the next), also for the workgroups that pairs with fewer row blocks than Z leave empty.  Measured on 16 x 16
    // pairs of 4 .. 16 row blocks, fused / product alone: Z = 16 1874 / 1307 us; two pairs taking turns 1795 / 1303;
    // Z = 3 (about three workgroups per compute unit) 1813 / 1201, but then ten pairs are in flight per die, B_g
    // leaves the die's L2 between a workgroup's passes and the launch reads 1.9 GB instead of 0.6.
    // Hence: fused, one workgroup per row block and two pairs taking turns; the product alone, about three workgroups
    // per compute unit (Z = 3 x compute units / pairs).
    // BLOCKEDATTN_ROWBLOCK_Z and BLOCKEDATTN_ROWBLOCK_WEAVE override.
    static const int forced_z = [] { const char *e = getenv("BLOCKEDATTN_ROWBLOCK_Z"); return e ? atoi(e) : 0; }();
    static const int forced_w = [] { const char *e = getenv("BLOCKEDATTN_ROWBLOCK_WEAVE"); return e ? atoi(e) : 0; }();
    const int64_t z_max = std::max<int64_t>(1, std::min<int64_t>(64, (std::max<int64_t>(info->max_M, 1) + kRbRows - 1) / kRbRows));
    int64_t z = fused ? z_max : std::min<int64_t>(z_max, (3 * (int64_t)device_cu_count() + pairs - 1) / pairs);
    if (forced_z > 0) z = std::min<int64_t>(z_max, forced_z);
    const int64_t weave = std::max<int64_t>(1, std::min<int64_t>(forced_w > 0 ? forced_w : (fused ? 2 : 1), pairs / kDies));
    pairs = (pairs / kDies + weave - 1) / weave * weave * kDies;       // whole turns
    const int64_t groups = pairs * z;
    if (pairs > (int64_t(1) << 30) || groups > (int64_t(1) << 31) - 1) return BA_ERR_UNSUPPORTED;
    int st;
    const unsigned g = (unsigned)groups;
    const int zi = (int)z, wi = (int)weave;
    if (dtype == BA_F16) {
        if (wide) st = fused ? launch_rb<0, true, true>(args, g, zi, wi, stream) : launch_rb<0, false, true>(args, g, zi, wi, stream);
        else st = fused ? launch_rb<0, true>(args, g, zi, wi, stream) : launch_rb<0, false>(args, g, zi, wi, stream);
    } else if (dtype == BA_BF16) {
        if (wide) st = fused ? launch_rb<1, true, true>(args, g, zi, wi, stream) : launch_rb<1, false, true>(args, g, zi, wi, stream);
        else st = fused ? launch_rb<1, true>(args, g, zi, wi, stream) : launch_rb<1, false>(args, g, zi, wi, stream);
    } else {
        return BA_ERR_UNSUPPORTED;
    }
    if (st != BA_OK) return st;
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

int launch_rowblocks(int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                     hipStream_t stream) {
    return launch_rowblocks_any(false, dtype, fused, args, slots, info, stream);
}

// The build for 128 < K <= 256 over the same list: the workgroups of every other segment leave at once (the caller
// launches the kernels that take those, with kFlagWideKToo).
int launch_rowblocks_wide_k(int dtype, int fused, const RunArgs &args, int64_t slots, const ba_plan_info *info,
                            hipStream_t stream) {
    return launch_rowblocks_any(true, dtype, fused, args, slots, info, stream);
}

}  // namespace ba
