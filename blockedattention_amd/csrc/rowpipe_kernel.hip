// The pipelined row-block kernel: softmax(scale * A_g B_g^T) for large segments (the tile kernel's class,
// N > 256) with K <= 128 and 16-bit results, written so that the two sweeps of the softmax share one stream
// of B_g through LDS.
//
// One workgroup = 8 wavefronts in two SETS of four.  A set works on one block of 256 rows (wavefront q of the
// set: rows 64 q .. 64 q + 63, four MFMA row tiles, A fragments in registers) and goes through the columns
// twice: sweep 1 sums exp2((s - R) c) per row, sweep 2 recomputes the scores and writes
// exp2(s c - R c - log2(sum)).  The sets are one sweep apart: while set X runs sweep 2 of row block b, set Y
// runs sweep 1 of row block b + 1 ON THE SAME CHUNKS of B_g (64 columns x 128 k, 16 KiB, four LDS stages).
// What that buys, against one sweep after the other in every wavefront:
//   * a wavefront of 64 rows reads each B fragment once for four matrix instructions; with 32 rows the LDS
//     operand reads alone keep the LDS busy for as long as the matrix instructions take;
//   * every chunk is fetched from L2 once for both sweeps;
//   * the wavefronts that store (sweep 2) issue no loads, and the wavefronts that fill the stages (sweep 1, or
//     idle) issue no stores: the in-order memory counter of a filling wavefront holds nothing but fills;
//   * at any time half of the wavefronts of a compute unit store, so the result leaves at an even rate.
//
// A wavefront's 64 x 64 block of a chunk is computed as two halves of 32 columns (column tile ct of the chunk
// takes the B rows 4 j + ct; half h = tiles 2h, 2h + 1), into two accumulator sets that alternate: the 32
// matrix instructions of one half are threaded, one by one, through the softmax arithmetic of the half before
// (per score: x = s c + ref, exp2 of the previous x, use of the exponential before that).  A lane (j = lane %
// 16, rg = lane / 16) holds rows 16 rt + 4 rg + i and, per half, the two consecutive columns 4 j + 2 h + {0, 1}.
//
// Sweep 1 measures every score against R = the row's maximum over the FIRST half chunk (the sum then holds a
// term 1 and cannot vanish).  Should a later score exceed R by more than the exponent range, the sum overflows;
// that is seen when the sweep ends, and the set then repeats the block in two sweeps that cannot overflow (row
// maximum over all columns, then the sum against it) while the other set waits for it where it must.
//
// Stores: as in the row-block kernel, a wavefront's results pass through a ring in LDS (one row of 128 columns
// per result row) and leave as line-aligned 128-byte windows, eight lanes x 16 bytes per row, so that every
// 128-byte line of the result is written whole and once; the row ends that no window covers whole are written
// by one unaligned 16-byte store each.  The ring of wavefront q is used by whichever set is in sweep 2.
#include <stdlib.h>

#include <algorithm>
#include <type_traits>

#include "tile_body.hpp"

namespace ba {

constexpr int kRpWaves = 8;
constexpr int kRpThreads = 64 * kRpWaves;
constexpr int kRpSetWaves = 4;
constexpr int kRpRT = 4;                                  // MFMA row tiles per wavefront
constexpr int kRpWaveRows = 16 * kRpRT;                   // 64
constexpr int kRpBlockRows = kRpSetWaves * kRpWaveRows;   // 256 rows per set and step
constexpr int kRpCols = 64;                               // columns per chunk
constexpr int kRpStageBytes = kRpCols * 256;              // 16 KiB: 64 rows of B_g x 128 k
#ifndef RP_STAGES
#define RP_STAGES 5
#endif
constexpr int kRpStages = RP_STAGES;
constexpr int kRpFillInsts = kRpStageBytes / 1024 / kRpSetWaves;   // global->LDS instructions per filling wavefront and chunk (4)
constexpr int kRpStoreInsts = kRpWaveRows / 8;            // window stores per wavefront and chunk (8)
constexpr int kRpRingPitch = 296;                         // 128 columns + a copy of the first 16 behind them; 74 words: the
                                                          // sixteen rows one 8-byte write instruction touches fall into sixteen bank pairs
constexpr int kRpRingBytes = kRpWaveRows * kRpRingPitch;  // per wavefront of a set
constexpr int kRpFlagOffset = kRpStages * kRpStageBytes + kRpSetWaves * kRpRingBytes;
constexpr int kRpLdsBytes = kRpFlagOffset + 64;
// Cache policy of the result stores: non-temporal.  As ordinary stores they delay the fills of B_g, which every step
// reads again: the filling set waits 2500 cycles per iteration for its chunk with the stores, 540 without them
// (16 x 16 pairs of 1024..4096 rows and columns: 1490 us -> 1365 us with this bit).
constexpr int kRpStoreAux = kResultAux;
constexpr uint32_t kRpOutOfRange = 0x80000000u;           // byte offset no segment reaches (areas are below 2^31 bytes)

enum RpRole : int { kRoleNone = 0, kRoleSum = 1, kRoleMax = 2, kRoleSumSafe = 3, kRoleOut = 4 };

__device__ __forceinline__ void rp_wait_vm_upto(int n) {  // wave-uniform; the largest listed count not above n
    if (n >= 12) wait_vm<12>();
    else if (n >= 8) wait_vm<8>();
    else if (n >= 4) wait_vm<4>();
    else wait_vm<0>();
}

// Sixteen bytes of a ring row starting at byte `pos` (any even value below 256): five aligned words, shifted.
// (One 16-byte LDS read at that address works, but any LDS read wider than its alignment holds the LDS for about
// 57 cycles per wavefront against 8 for an aligned one; five word reads of rows 74 words apart take about 18.)
__device__ __forceinline__ u32x4 rp_ring_read16(const unsigned char *row, int pos) {
    const uint32_t *w = reinterpret_cast<const uint32_t *>(row + (pos & ~3));
    const uint32_t d0 = w[0], d1 = w[1], d2 = w[2], d3 = w[3], d4 = w[4];
    const uint32_t sh = (uint32_t)(pos & 2) * 8;
    return u32x4{__builtin_amdgcn_alignbit(d1, d0, sh), __builtin_amdgcn_alignbit(d2, d1, sh),
                 __builtin_amdgcn_alignbit(d3, d2, sh), __builtin_amdgcn_alignbit(d4, d3, sh)};
}

// A copy of a per-lane constant that the compiler cannot see through: what is derived from it inside a loop is
// computed there (one or two instructions) instead of being kept in registers of its own across the loop.
template <typename T> __device__ __forceinline__ T rp_fresh(T v) {
    asm volatile("" : "+v"(v));
    return v;
}

template <int DT>
__global__ __launch_bounds__(kRpThreads, 1) void rowpipe_kernel(RunArgs a, int zdim, int weave) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
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
    // Workgroup -> (list entry, head, share of the row blocks).  Consecutive workgroup ids go to the eight dies in
    // turn, each with its own L2; all workgroups of one (entry, head) pair read the same B_g, so they run on ONE
    // die.  The pairs are numbered entry-major with the entries in order of DECREASING work (M N).
    const int entries = a.list < 0 ? a.nseg : (int)((ConstHdr)(uintptr_t)a.plan)->totals[a.list];
    if (entries <= 0 || pair >= entries * H) return;
    const int h = pair % H;
    int entry = pair / H;
    if (entries <= 64) {
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
    if (!valid || !pipe_segment(s.kind, s.N, s.K)) return;      // (the tile kernel of the same call takes the others)
    const int M = s.M, N = s.N, K = s.K;
    const int nrb = (M + kRpBlockRows - 1) / kRpBlockRows;
    const int b_begin = (int)((int64_t)z0 * nrb / zdim), b_end = (int)((int64_t)(z0 + 1) * nrb / zdim);
    if (b_begin >= b_end) return;
    const int ncb = (N + kRpCols - 1) / kRpCols;
    static_assert(kRpStages <= 5 && kRpCols == 64, "pipe_segment() admits segments of at least five chunks");
    if (threadIdx.x == 0) atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->pipe_groups, 1);
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int set = wave >> 2, wq = wave & 3;
    const SegRes res = make_res(s, a.A, a.B);
    const char *bseg = reinterpret_cast<const char *>((const uint16_t *)a.B + s.b);
    char *oseg = reinterpret_cast<char *>(a.out) + s.o * 2;
    const __amdgpu_buffer_rsrc_t out_res =
        __builtin_amdgcn_make_buffer_rsrc(oseg, 0, (int)((uint32_t)M * (uint32_t)N * 2u), kRsrcFlags);
    const uint32_t out_phase = (uint32_t)(uintptr_t)oseg;   // low address bits decide the line phase of a row
    unsigned char *ring = lds + kRpStages * kRpStageBytes + wq * kRpRingBytes;
    volatile int *flags = reinterpret_cast<volatile int *>(lds + kRpFlagOffset);   // [parity of the step][set]

    const int ksteps = (K + 31) >> 5;
    const int kpieces = K >> 3;                            // 16-byte pieces per row of B_g
    const float c_signed = a.scale * kLog2e;
    const bool negate = c_signed < 0.f;                    // |scale| on negated scores
    const float c = __builtin_bit_cast(float, uniform(__builtin_bit_cast(int, __builtin_fabsf(c_signed))));   // in a scalar register
    const u32x4 zero4 = {0u, 0u, 0u, 0u};

    // Stale or never written LDS must not reach a matrix instruction as NaN bits: pieces past K are never
    // filled, so the stages start as zeros.
    for (int off = (int)threadIdx.x * 16; off < kRpStages * kRpStageBytes; off += kRpThreads * 16)
        *reinterpret_cast<u32x4 *>(lds + off) = zero4;
    if (threadIdx.x < 4) flags[threadIdx.x] = 0;
    __syncthreads();                                      // no fill may land under a late zero

    // Fill of one chunk by the four wavefronts of a set: instruction i (0..15) covers LDS rows 4i .. 4i+3 of the
    // stage; lane l writes row r = 4i + l/16, slot l%16, which holds piece (l%16) ^ (r%16) of that row (the sixteen
    // lanes of an operand read take sixteen consecutive rows, 256 bytes apart: sixteen slots).  Wavefront q
    // issues i = q + 4 n: row 4q + l/16 + 16 n, piece (l%16) ^ (4q + l/16) whatever n.  Rows past N (ragged last
    // chunk) fetch row N - 1 instead, so that every instruction is issued whatever the shape and the count of
    // outstanding fills is known.  Lanes whose piece lies past K stay idle: the instruction runs under a lane mask
    // set INSIDE the assembly (a branch around it would split the body it is threaded into, and the compiler moves
    // the arithmetic out of a split body).  Written as assembly on purpose: the compiler orders every LDS access
    // behind ALL outstanding vector memory operations once it has seen a load into LDS.
    const int fill_piece = (lane & 15) ^ (4 * wq + (lane >> 4));
    const uint32_t fill_row = (uint32_t)((4 * wq + (lane >> 4)) * K + fill_piece * 8) * 2u;
    uint64_t fill_mask = __ballot(fill_piece < kpieces);      // K = 0: no lane, and then no fill is issued at all
    const bool fills_on = kpieces > 0;
    auto fill_one = [&](auto n_c, int cbi, int stage) __attribute__((always_inline)) {
        constexpr int n = decltype(n_c)::value;
        const int cb = cbi * kRpCols;
        const char *base = reinterpret_cast<const char *>((uintptr_t)uniform64((int64_t)(uintptr_t)(bseg + (size_t)cb * K * 2)));
        const int i = wq + kRpSetWaves * n;
        const uint32_t dst = (uint32_t)uniform((int)(uint32_t)(uintptr_t)(lds + stage * kRpStageBytes + i * 1024));
        // (the row clamp changes nothing in a whole chunk: two instructions, no branch)
        const int r = min(4 * i + (lane >> 4), N - 1 - cb);
        const uint32_t off = rp_fresh(fill_row) + (uint32_t)((r - 4 * wq - (lane >> 4)) * K) * 2u;
        uint64_t saved;
        const uint64_t mask = fill_mask;
        asm volatile("s_mov_b64 %0, exec\n\ts_and_b64 exec, exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                     : "=&s"(saved) : "v"(off), "s"(base), "s"(dst), "s"(mask) : "memory", "m0");
    };
    auto fill = [&](int cbi, int stage) __attribute__((always_inline)) {
        if (!fills_on) return;
        fill_one(std::integral_constant<int, 0>{}, cbi, stage); fill_one(std::integral_constant<int, 1>{}, cbi, stage);
        fill_one(std::integral_constant<int, 2>{}, cbi, stage); fill_one(std::integral_constant<int, 3>{}, cbi, stage);
    };
    // operand read offset of this lane inside a stage: column tile ct, row 16 ct + j, piece 4ks + rg at slot
    // (4ks + rg) ^ j (k-step ks flips bits 2..3 of the slot: offset of k-step 0 exclusive-or 64 ks)
    const int boff0 = 256 * j + 16 * (rg ^ j);

    // ---- per-wavefront state of the block the set works on
    u32x4 af[kRpRT][4];                        // A fragments [rt][ks]: row 16 rt + j, k = 32 ks + 8 rg ..
    float ref[kRpRT];                          // of row 16 rt + j; sweep 1: -R c; sweep 2: -R c - log2(sum)
    float sum[kRpRT];                          // sweep 1: running sum over the lane's columns; maximum sweep: running maximum
    f32x4 acc[2][kRpRT][2];                    // [half][rt][column tile of the half]: columns 4 rg + i of the tile
    u32x4 bf[3][2];                            // B fragments of three k-steps: [buffer][column tile of the half]
    uint32_t v0[kRpStoreInsts];                // sweep 2: byte offset of the lane's piece of window 0 inside the segment's result
    int upos[kRpStoreInsts];                   // ... and ring byte of that piece: 2 (8q - d) mod 256
    int row0 = 0;
    bool active = false;
    const int q8 = lane & 7;
    // (byte offsets inside the workgroup's LDS)
    const int ring_o = kRpStages * kRpStageBytes + wq * kRpRingBytes;
    const int rbase_o = ring_o + (lane >> 3) * kRpRingPitch;                    // store lanes: row lane / 8 of a group of eight
    const int ringw_o = ring_o + j * kRpRingPitch + 8 * rg;                     // ring writes: row j, columns 4 rg ..

    auto load_block = [&](int blk) __attribute__((always_inline)) {
        row0 = blk * kRpBlockRows + wq * kRpWaveRows;
        active = row0 < M;
#pragma unroll
        for (int rt = 0; rt < kRpRT; ++rt) {
            const int voff = ((row0 + 16 * rt + j) * K + rg * 8) * 2;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                u32x4 v = zero4;
                if (ks < ksteps) {
                    v = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff + ks * 64, 0, 0);
                    if (ks * 32 + rg * 8 >= K) v = zero4;            // ragged last k-step
                    if (negate) v ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
                }
                af[rt][ks] = v;
            }
        }
    };
    // store lanes: instruction t writes rows 8t + lane/8, piece lane%8 of the row's aligned window.  A row without
    // a store keeps its offset out of range: the marker plus any advance stays above 2^31.
    auto store_lanes = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < kRpStoreInsts; ++t) {
            const int rho = row0 + 8 * t + (lane >> 3);
            const bool row_ok = rho < M;
            const int rn = row_ok ? rho * N : 0;
            const int d = (int)(((out_phase + 2u * (uint32_t)rn) & 127u) >> 1);     // columns before the row's first line boundary
            upos[t] = (16 * q8 - 2 * d) & 255;
            v0[t] = row_ok ? (uint32_t)(2 * (rn + 8 * q8 - d)) : kRpOutOfRange;
        }
    };

    // -------- out of the ring: one line-aligned 128-byte window per row and chunk.  Interior chunk: the sixteen
    // rows of row tile rt leave once they are in the ring, as two store instructions of eight rows; the LDS read of
    // one is issued a few matrix instructions before its store (load / store+load / store, spread by the caller).
    u32x4 ring_ld = {0u, 0u, 0u, 0u};
    auto ring_load = [&](int cbi, auto t_c) __attribute__((always_inline)) {
        constexpr int t = decltype(t_c)::value;
        asm volatile("" ::: "memory");                    // the read sees the writes above (same wavefront, in order)
        ring_ld = rp_ring_read16(lds + rbase_o + t * 8 * kRpRingPitch, upos[t] ^ ((cbi & 1) << 7));
    };
    auto ring_store = [&](int cbi, auto t_c) __attribute__((always_inline)) {
        constexpr int t = decltype(t_c)::value;
        __builtin_amdgcn_raw_buffer_store_b128(ring_ld, out_res, v0[t] + 128u * (uint32_t)cbi, 0, kRpStoreAux);        // (the range check sees the vector offset only)
        asm volatile("" ::: "memory");
    };
    // First or last chunk: pieces before column 0 or past column N are dropped, and the end pieces the windows
    // cannot cover whole are written by one unaligned store each (lane l: row l).
    auto ring_store_edge = [&](int cbi) __attribute__((always_inline)) {
        asm volatile("" ::: "memory");
        const int par = (cbi & 1) << 7;
        const uint32_t adv = 128u * (uint32_t)cbi;
        const int et_row = row0 + lane;
        const uint32_t et_off = et_row < M ? (uint32_t)(2 * (et_row * N)) : kRpOutOfRange;
        const unsigned char *et_base = ring + lane * kRpRingPitch;
#pragma unroll
        for (int t = 0; t < kRpStoreInsts; ++t) {
            const u32x4 v = rp_ring_read16(lds + rbase_o + t * 8 * kRpRingPitch, upos[t] ^ par);
            const int col = (((upos[t] >> 1) + 64) & 127) - 64 + kRpCols * cbi;      // first column of the piece
            const uint32_t voff = (col < 0 || col + 8 > N) ? kRpOutOfRange : v0[t] + adv;
            __builtin_amdgcn_raw_buffer_store_b128(v, out_res, voff, 0, kRpStoreAux);
        }
        if (cbi == 0) {
            const u32x4 v = rp_ring_read16(et_base, 0);                         // columns [0, 8)
            __builtin_amdgcn_raw_buffer_store_b128(v, out_res, et_off, 0, kRpStoreAux);
        }
        if (cbi == ncb - 1) {
            // the window behind the last chunk (what is left of the rows), then columns [N-8, N)
            const int par2 = (ncb & 1) << 7;
#pragma unroll
            for (int t = 0; t < kRpStoreInsts; ++t) {
                const u32x4 v = rp_ring_read16(lds + rbase_o + t * 8 * kRpRingPitch, upos[t] ^ par2);
                const int col = (((upos[t] >> 1) + 64) & 127) - 64 + kRpCols * ncb;
                const uint32_t voff = col + 8 <= N ? v0[t] + 128u * (uint32_t)ncb : kRpOutOfRange;
                __builtin_amdgcn_raw_buffer_store_b128(v, out_res, voff, 0, kRpStoreAux);
            }
            const u32x4 v = rp_ring_read16(et_base, (2 * (N - 8)) & 255);
            __builtin_amdgcn_raw_buffer_store_b128(v, out_res, et_off + 2u * (uint32_t)(N - 8), 0, kRpStoreAux);
        }
        asm volatile("" ::: "memory");
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using False = std::false_type;
    using True = std::true_type;

    // -------- one half: the 32 matrix instructions of half HB (column tiles 2 HB, 2 HB + 1) of the chunk in `stage`
    // (when MFMA) into accumulator set HB, with the arithmetic of the half before -- half 1 - HB of chunk `cprev`,
    // in the other accumulator set -- threaded between them, one score element per matrix instruction.
    // MODE 0: matrix instructions only; kRoleSum: sum += exp2(s c + ref); kRoleMax: running maximum; kRoleOut:
    // exp2(s c + ref) into the ring, and out of it (INTERIOR: the window of the chunk that HB = 0 completes is not
    // the first or the last of its rows).  FILL: the wavefront requests two of its four pieces of the chunk three
    // ahead (`fcbi` into `fstage`).  RAG: the half before has columns that do not exist (ragged last chunk): they
    // stay out of sum and maximum.  All of these are compile-time flags: a branch inside the body would let the
    // compiler move the arithmetic away from the matrix instructions it is threaded through.
    auto half = [&](auto mode_c, auto h_c, auto mfma_c, auto fill_c, auto rag_c, auto int_c, int stage, int cprev,
                    int fcbi, int fstage) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode_c)::value;
        constexpr int hb = decltype(h_c)::value, pb = 1 - hb;
        constexpr bool MFMA = decltype(mfma_c)::value;
        constexpr bool RAG = decltype(rag_c)::value;
        constexpr bool INTERIOR = MODE == kRoleOut && decltype(int_c)::value;
        const unsigned char *sb = lds + stage * kRpStageBytes + 8192 * hb;
        const int b0 = rp_fresh(boff0);
        const int colp = cprev * kRpCols + 32 * pb + 4 * rg;       // the lane's columns of the half before: colp + 16 ct + i
        // ring position of those columns; the first column tile of a chunk in the first half of the ring also goes
        // behind the row's end (pieces that start in a row's last 16 bytes continue there); in the second half the
        // copy falls on the original
        const int slot = (cprev & 1) << 7;
        unsigned char *wrow = lds + rp_fresh(ringw_o) + slot + 64 * pb;
        unsigned char *wcopy = lds + rp_fresh(ringw_o) + 256 - slot;
        // B fragments: three buffers in rotation over the eight k-steps of a chunk (buffer (4 HB + ks) % 3), read two
        // k-steps -- sixteen matrix instructions -- ahead; half 0 starts with the reads of its first two k-steps (the
        // chunk is only known to be there after the barrier), half 1 finds its first two under way
        auto bread = [&](auto g_c) __attribute__((always_inline)) {
            constexpr int g = decltype(g_c)::value, gh = g >> 2, gk = g & 3;
            const unsigned char *gb = lds + stage * kRpStageBytes + 8192 * gh + (b0 ^ (64 * gk));
            bf[g % 3][0] = *reinterpret_cast<const u32x4 *>(gb);
            bf[g % 3][1] = *reinterpret_cast<const u32x4 *>(gb + 4096);
        };
        if constexpr (MFMA && hb == 0) { bread(std::integral_constant<int, 0>{}); bread(std::integral_constant<int, 1>{}); }
        float xprev = 0.f, pprev = 0.f, q0 = 0.f, q1 = 0.f, q2 = 0.f;
        // element e of a half: row tile e / 8, column tile (e / 4) % 2, column e % 4 of the lane's four
        auto use = [&](auto e_c, float pval) {
            constexpr int pe = decltype(e_c)::value, prt = pe >> 3, pct = (pe >> 2) & 1, pi = pe & 3;
            if constexpr (MODE == kRoleSum) {
                if constexpr (RAG) sum[prt] += colp + 16 * pct + pi < N ? pval : 0.f;
                else sum[prt] += pval;
            } else if constexpr (MODE == kRoleMax) {
                if constexpr (RAG) sum[prt] = __builtin_fmaxf(sum[prt], colp + 16 * pct + pi < N ? pval : -3.0e38f);
                else sum[prt] = __builtin_fmaxf(sum[prt], pval);
            } else if constexpr (MODE == kRoleOut) {
                if constexpr (pi == 0) q0 = pval;
                else if constexpr (pi == 1) q1 = pval;
                else if constexpr (pi == 2) q2 = pval;
                else {
                    const u32x2 v = {Elem<DT>::pack2(q0, q1), Elem<DT>::pack2(q2, pval)};
                    *reinterpret_cast<u32x2 *>(wrow + 16 * prt * kRpRingPitch + 32 * pct) = v;
                    if constexpr (pb == 0 && pct == 0) *reinterpret_cast<u32x2 *>(wcopy + 16 * prt * kRpRingPitch) = v;
                }
                // Out of the ring.  Half 1 of chunk cprev (done during HB = 0) completes the rows, row tile by row
                // tile (row tile rt at element 8 rt + 7), and row tile rt leaves as store instructions 2 rt and
                // 2 rt + 1.  The eight stores of a chunk are spread over both halves, one every eight matrix
                // instructions, each four elements behind its LDS read -- a wavefront that issues its stores in a
                // burst waits for the memory pipeline to take them.  Every read comes after the rows are complete and
                // before HB = 1 writes the next chunk into them (row tile rt from element 8 rt on).
                if constexpr (INTERIOR && hb == 0) {
                    if constexpr (pe == 7) ring_load(cprev, std::integral_constant<int, 0>{});
                    if constexpr (pe == 11) ring_store(cprev, std::integral_constant<int, 0>{});
                    if constexpr (pe == 15) ring_load(cprev, std::integral_constant<int, 1>{});
                    if constexpr (pe == 19) ring_store(cprev, std::integral_constant<int, 1>{});
                    if constexpr (pe == 23) ring_load(cprev, std::integral_constant<int, 2>{});
                    if constexpr (pe == 27) ring_store(cprev, std::integral_constant<int, 2>{});
                    if constexpr (pe == 31) ring_load(cprev, std::integral_constant<int, 3>{});
                }
                if constexpr (INTERIOR && hb == 1) {
                    if constexpr (pe == 3) { ring_store(cprev - 1, std::integral_constant<int, 3>{}); ring_load(cprev - 1, std::integral_constant<int, 4>{}); }
                    if constexpr (pe == 7) ring_store(cprev - 1, std::integral_constant<int, 4>{});
                    if constexpr (pe == 11) ring_load(cprev - 1, std::integral_constant<int, 5>{});
                    if constexpr (pe == 15) { ring_store(cprev - 1, std::integral_constant<int, 5>{}); ring_load(cprev - 1, std::integral_constant<int, 6>{}); }
                    if constexpr (pe == 19) { ring_store(cprev - 1, std::integral_constant<int, 6>{}); ring_load(cprev - 1, std::integral_constant<int, 7>{}); }
                    if constexpr (pe == 23) ring_store(cprev - 1, std::integral_constant<int, 7>{});
                }
            }
        };
        auto power = [&](float x) { return MODE == kRoleMax ? x : __builtin_amdgcn_exp2f(x); };
        auto element = [&](auto e_c) {
            constexpr int e = decltype(e_c)::value, rt2 = e >> 3, ct2 = (e >> 2) & 1, i2 = e & 3;
            if constexpr (e >= 2) use(std::integral_constant<int, e - 2>{}, pprev);
            if constexpr (e >= 1) pprev = power(xprev);
            const float sc = acc[pb][rt2][ct2][i2];
            xprev = MODE == kRoleMax ? sc : fmaf(sc, c, ref[rt2]);
        };
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if constexpr (decltype(fill_c)::value) {
                if (ks == 1) fill_one(std::integral_constant<int, 2 * hb>{}, fcbi, fstage);
                if (ks == 3) fill_one(std::integral_constant<int, 2 * hb + 1>{}, fcbi, fstage);
            }
            if constexpr (MFMA) {
                if (ks == 0 && 4 * hb + 2 < 8) bread(std::integral_constant<int, (4 * hb + 2) & 7>{});
                if (ks == 1 && 4 * hb + 3 < 8) bread(std::integral_constant<int, (4 * hb + 3) & 7>{});
                if (ks == 2 && 4 * hb + 4 < 8) bread(std::integral_constant<int, (4 * hb + 4) & 7>{});
                if (ks == 3 && 4 * hb + 5 < 8) bread(std::integral_constant<int, (4 * hb + 5) & 7>{});
            }
            auto group = [&](auto qd_c) {
                constexpr int qd = decltype(qd_c)::value, rt = qd >> 1, ct = qd & 1;
                // (rows of B_g as the first operand: the lane gets row 16 rt + j, columns 4 rg .. 4 rg + 3 of the tile)
                if constexpr (MFMA)
                    acc[hb][rt][ct] = Elem<DT>::mfma(bf[(4 * hb + ks) % 3][ct], af[rt][ks],
                                                     ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[hb][rt][ct]);
                if constexpr (MODE != 0) {
                    if (ks == 0) element(std::integral_constant<int, 0 * 8 + qd>{});
                    if (ks == 1) element(std::integral_constant<int, 1 * 8 + qd>{});
                    if (ks == 2) element(std::integral_constant<int, 2 * 8 + qd>{});
                    if (ks == 3) element(std::integral_constant<int, 3 * 8 + qd>{});
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            group(I0{}); group(I1{}); group(I2{}); group(I3{});
            group(std::integral_constant<int, 4>{}); group(std::integral_constant<int, 5>{});
            group(std::integral_constant<int, 6>{}); group(std::integral_constant<int, 7>{});
        }
        if constexpr (MODE != 0) {
            use(std::integral_constant<int, 30>{}, pprev);
            pprev = power(xprev);
            use(std::integral_constant<int, 31>{}, pprev);
        }
    };

    // sweep 1, first half chunk: the reference of every row = its maximum over these 32 columns (the lane's
    // eight, then the four lanes that share the row)
    auto stats_reference = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < kRpRT; ++rt) {
            float m = __builtin_fmaxf(__builtin_fmaxf(acc[0][rt][0][0], acc[0][rt][0][1]), __builtin_fmaxf(acc[0][rt][0][2], acc[0][rt][0][3]));
            m = __builtin_fmaxf(m, __builtin_fmaxf(__builtin_fmaxf(acc[0][rt][1][0], acc[0][rt][1][1]), __builtin_fmaxf(acc[0][rt][1][2], acc[0][rt][1][3])));
            ref[rt] = -__builtin_fmaxf(quad_column_max(m), -3.0e38f) * c;
        }
    };
    // after the last chunk of sweep 1: row sums over the four lanes of a row; returns whether any is not finite
    auto finish_stats = [&]() __attribute__((always_inline)) {
        bool bad = false;
#pragma unroll
        for (int rt = 0; rt < kRpRT; ++rt) {
            const float sm = quad_column_sum(sum[rt]);
            bad |= !(sm <= 3.0e38f);
            ref[rt] -= __builtin_amdgcn_logf(sm);                // 1/sum goes into the exponent
        }
        return bad;
    };
    // after the maximum sweep: the reference of every row = its maximum over all columns
    auto finish_max = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < kRpRT; ++rt) ref[rt] = -__builtin_fmaxf(quad_column_max(sum[rt]), -3.0e38f) * c;
    };

    // -------- the steps.  All of this is the same in every wavefront of the workgroup (scalar registers).
    int role[2] = {kRoleNone, kRoleNone};
    int next_block = b_begin;
    int gpos = 0;                                          // chunks gone by since the workgroup started: stage = gpos % 4
    bool first_step = true;
    for (int step = 0;; ++step) {
        // a set without work takes the next row block, unless the other set would then reach sweep 2 together with it
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            if (role[g] == kRoleNone && next_block < b_end && role[1 - g] != kRoleSum && role[1 - g] != kRoleSumSafe) {
                role[g] = kRoleSum;
                if (g == set) load_block(next_block);
                ++next_block;
            }
        }
        if (role[0] == kRoleNone && role[1] == kRoleNone) break;
        const bool final_step = next_block >= b_end && (role[0] == kRoleNone || role[0] == kRoleOut) &&
                                (role[1] == kRoleNone || role[1] == kRoleOut);
        // the set that stores does not fill; of two sets that do not store, the idle one fills
        const int filler_set = role[0] == kRoleOut ? 1 : role[1] == kRoleOut ? 0 : role[1] == kRoleNone ? 1 : 0;
        const bool filler = set == filler_set;
        const int my_role = role[set];
        if (first_step) {
            if (filler) {
                for (int k = 0; k < kRpStages - 1; ++k) fill(k, k);
            }
            wait_vm<0>();                                  // the first chunks, or the A fragments
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            first_step = false;
        }
        // SYNC of iteration i: the filling wavefronts wait for their part of chunk i (requested three iterations
        // ago; the fills of the two iterations since may stay in flight; the first three chunks of a step were
        // complete before the step began), barrier (now everyone's part is there and nobody reads the stage of
        // chunk i - 1 any more), request chunk i + 3 -- which, in any step but the workgroup's last, is a chunk of
        // the next step once the end of B_g is near.  `spread`: the halves of the iteration issue the four
        // instructions of the request one by one instead (a load into LDS holds the wavefront that issues it while
        // the requests before it are taken, about 70 cycles each, so four wavefronts issuing four in a row wait for
        // each other).
        int pf_cbi = 0, pf_stage = 0;
        auto sync = [&](int i, bool spread) __attribute__((always_inline)) {
            if (filler && i >= kRpStages - 1) {
                int later = (kRpStages - 2) * kRpFillInsts;
                if (final_step) {
                    later = 0;
                    for (int d = 1; d <= kRpStages - 2; ++d) later += i + d < ncb ? kRpFillInsts : 0;
                }
                rp_wait_vm_upto(later);
            }
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            int cbi = i + kRpStages - 1;
            if (cbi >= ncb) cbi -= ncb;
            pf_cbi = cbi;
            pf_stage = (gpos + i + kRpStages - 1) % kRpStages;
            if (!spread && filler && (!final_step || i + kRpStages - 1 < ncb)) fill(pf_cbi, pf_stage);
            __builtin_amdgcn_sched_barrier(0);
        };
        // FILL: the wavefront issues its fills from inside the halves (it is this step's filler, the step is not
        // the workgroup's last, so every iteration has a chunk to request, and K > 0).
        auto run = [&](auto mode_c, auto fill_c) __attribute__((always_inline)) {
            constexpr int MODE = decltype(mode_c)::value;
            using Fill = decltype(fill_c);
            using Out = std::integral_constant<bool, MODE == kRoleOut>;
            // (a wavefront without rows only keeps the barriers and its fills: decided once, so that the accumulators
            // are plainly defined before they are used in the branch that computes)
            if (!active) {
                for (int i = 0; i < ncb; ++i) sync(i, false);
                return;
            }
            const bool ragged = (N & (kRpCols - 1)) != 0;
            // chunk 0: nothing to do arithmetic on yet; sweep 1 takes its reference from the first half
            {
                const int stage = gpos % kRpStages;
                sync(0, Fill::value);
                half(I0{}, I0{}, True{}, Fill{}, False{}, False{}, stage, 0, pf_cbi, pf_stage);
                if (MODE == kRoleSum && my_role == kRoleSum) stats_reference();
                half(mode_c, I1{}, True{}, Fill{}, False{}, False{}, stage, 0, pf_cbi, pf_stage);
            }
            // chunk 1: completes chunk 0, whose window is an edge
            {
                sync(1, Fill::value);
                const int stage = (gpos + 1) % kRpStages;
                half(mode_c, I0{}, True{}, Fill{}, False{}, False{}, stage, 0, pf_cbi, pf_stage);
                if (MODE == kRoleOut) ring_store_edge(0);
                half(mode_c, I1{}, True{}, Fill{}, False{}, False{}, stage, 1, pf_cbi, pf_stage);
            }
            for (int i = 2; i < ncb - 1; ++i) {
                sync(i, Fill::value);
                const int stage = (gpos + i) % kRpStages;
                half(mode_c, I0{}, True{}, Fill{}, False{}, Out{}, stage, i - 1, pf_cbi, pf_stage);
                half(mode_c, I1{}, True{}, Fill{}, False{}, Out{}, stage, i, pf_cbi, pf_stage);
            }
            // the last chunk: its columns may end early (sweep 1 and the maximum sweep leave the missing ones out)
            {
                const int i = ncb - 1;
                sync(i, Fill::value);
                const int stage = (gpos + i) % kRpStages;
                half(mode_c, I0{}, True{}, Fill{}, False{}, Out{}, stage, i - 1, pf_cbi, pf_stage);
                if (MODE != kRoleOut && ragged) {
                    half(mode_c, I1{}, True{}, Fill{}, True{}, False{}, stage, i, pf_cbi, pf_stage);
                    half(mode_c, I0{}, False{}, False{}, True{}, False{}, 0, i, 0, 0);
                } else {
                    half(mode_c, I1{}, True{}, Fill{}, False{}, Out{}, stage, i, pf_cbi, pf_stage);
                    half(mode_c, I0{}, False{}, False{}, False{}, False{}, 0, i, 0, 0);
                }
            }
            if (MODE == kRoleOut) ring_store_edge(ncb - 1);
        };
        // Every role keeps its state inside its own branch: what a sweep sets up, it alone uses (the sums of sweep 1,
        // the store lanes of sweep 2), so none of it occupies registers in the other sweeps.
        volatile int *fl = flags + 2 * (step & 1);
        // the set that stores has more to do per chunk than the other: its wavefronts go first where both can issue
        // (measured again with non-temporal stores, when the summing set had become the one the other waits for:
        // equal priorities 1415 us, the summing set first 1455, this 1375)
        if (my_role == kRoleOut) __builtin_amdgcn_s_setprio(3);
        else __builtin_amdgcn_s_setprio(0);
        if (my_role == kRoleOut) {
            store_lanes();
            run(std::integral_constant<int, kRoleOut>{}, False{});
        } else if (my_role == kRoleMax) {
#pragma unroll
            for (int rt = 0; rt < kRpRT; ++rt) sum[rt] = -3.0e38f;
            run(std::integral_constant<int, kRoleMax>{}, False{});
            if (active) finish_max();
        } else if (my_role == kRoleNone) {
            for (int i = 0; i < ncb; ++i) sync(i, false);
        } else {
#pragma unroll
            for (int rt = 0; rt < kRpRT; ++rt) sum[rt] = 0.f;
            if (filler && fills_on) run(std::integral_constant<int, kRoleSum>{}, True{});
            else run(std::integral_constant<int, kRoleSum>{}, False{});
            // the overflow verdict of sweep 1 goes to the whole workgroup through LDS
            const bool bad = active && finish_stats();
            if (my_role == kRoleSum && __ballot(bad) != 0 && lane == 0) fl[set] = 1;
        }
        gpos += ncb;
        if (filler) wait_vm<0>();                         // the next step's first chunks are there before anyone takes over
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        const int over0 = uniform(fl[0]), over1 = uniform(fl[1]);
        if (threadIdx.x == 0) { flags[2 * (1 - (step & 1))] = 0; flags[2 * (1 - (step & 1)) + 1] = 0; }
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int over = g == 0 ? over0 : over1;
            if (role[g] == kRoleSum) role[g] = over ? kRoleMax : kRoleOut;
            else if (role[g] == kRoleMax) role[g] = kRoleSumSafe;
            else if (role[g] == kRoleSumSafe) role[g] = kRoleOut;
            else if (role[g] == kRoleOut) role[g] = kRoleNone;
        }
    }
    wait_vm<0>();
}

template <int DT>
static int launch_rp(const RunArgs &args, unsigned groups, int zdim, int weave, hipStream_t stream) {
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&rowpipe_kernel<DT>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, kRpLdsBytes);
    if (attr != hipSuccess) return BA_ERR_LAUNCH;
    hipLaunchKernelGGL((rowpipe_kernel<DT>), dim3(groups), dim3(kRpThreads), kRpLdsBytes, stream, args, zdim, weave);
    return BA_OK;
}

// Launches the pipelined row-block kernel over (list entry, head, share of the row blocks): the fused pair for
// large segments with K <= 128 and 16-bit results.  `slots` = entries of the tile list (with the plan summary) or
// the segment count (without: the workgroups behind the list's end leave at once); the kernel takes the entries
// that pipe_segment() admits and leaves the others to the tile kernel.
int launch_rowpipe(int dtype, const RunArgs &args, int64_t slots, const ba_plan_info *info, hipStream_t stream) {
    if (args.flags & kFlagOutF32) return BA_ERR_UNSUPPORTED;
    if (slots <= 0) return BA_OK;
    // Without the summary every (segment, head) gets a workgroup that may find nothing, and a workgroup of this kernel
    // holds a whole compute unit while it looks (1024 segments x 4 heads of small segments: + 40 us): only for small
    // batches, where large segments are likely and the empty workgroups are few.
    if (!info && slots * args.H > 1024) return BA_ERR_UNSUPPORTED;
    int64_t pairs = (slots * args.H + kDies - 1) / kDies * kDies;   // (entry, head) pairs, padded to whole dies
    static const int forced_z = [] { const char *e = getenv("BLOCKEDATTN_ROWPIPE_Z"); return e ? atoi(e) : 0; }();
    static const int forced_w = [] { const char *e = getenv("BLOCKEDATTN_ROWPIPE_WEAVE"); return e ? atoi(e) : 0; }();
    // Workgroups per pair Z: workgroup z takes the z-th share of the pair's row blocks, one after the other.  A share
    // of n row blocks takes n + 1 steps, the first and the last with one set idle, so few large shares are better
    // than many small ones -- but a share longer than the chip's mean load per compute unit is the last to finish.
    // Measured on 16 x 16 pairs of 5 .. 16 row blocks: Z = 1 imbalance, Z = 2 1594 us, Z = 3 1649 us; one workgroup
    // per compute unit with an equal share of all the work (contiguous runs of pairs and row blocks): 1744 .. 1906 us,
    // the dies with the narrow pairs finishing last.  BLOCKEDATTN_ROWPIPE_Z and _WEAVE override.
    const int cus = device_cu_count();
    // (without the summary the tallest segment is unknown: up to eight shares, which a short segment leaves empty)
    const int64_t z_max = !info ? 8 : std::max<int64_t>(1, std::min<int64_t>(64, (std::max<int64_t>(info->max_M, 1) + kRpBlockRows - 1) / kRpBlockRows));
    int64_t z = std::min<int64_t>(z_max, std::max<int64_t>(1, (2 * (int64_t)cus + pairs - 1) / pairs));
    if (forced_z > 0) z = std::min<int64_t>(z_max, forced_z);
    const int64_t weave = std::max<int64_t>(1, std::min<int64_t>(forced_w > 0 ? forced_w : 1, pairs / kDies));
    pairs = (pairs / kDies + weave - 1) / weave * weave * kDies;       // whole turns
    const int64_t groups = pairs * z;
    if (pairs > (int64_t(1) << 30) || groups > (int64_t(1) << 31) - 1) return BA_ERR_UNSUPPORTED;
    int st;
    if (dtype == BA_F16) st = launch_rp<0>(args, (unsigned)groups, (int)z, (int)weave, stream);
    else if (dtype == BA_BF16) st = launch_rp<1>(args, (unsigned)groups, (int)z, (int)weave, stream);
    else return BA_ERR_UNSUPPORTED;
    if (st != BA_OK) return st;
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
