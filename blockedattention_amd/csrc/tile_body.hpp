// Body of the tile kernel (included by tile_kernel.hip, and by the strip kernel, whose second launch can
// carry the tile kernel's workgroups along).
//
// Large segments: S_g = A_g B_g^T and its row softmax for segments whose B_g does
// not fit the strip kernel's LDS window (N > 256, or N >= 128 with a long K).
//
// One workgroup = 128 rows of one segment and head; wavefront w owns rows
// 32w .. 32w+31 (two MFMA row tiles) and ALL columns, 128 at a time.  B_g is
// streamed through LDS in chunks of 128 columns x 64 k (16 KiB, two buffers): a
// chunk is a straight copy of 128 consecutive rows of B_g (64 k of each), fetched
// with direct global->LDS loads whose lanes read consecutive 16-byte pieces
// (coalesced), and shared by the eight row tiles of the workgroup.  Inside LDS
// the eight 16-byte pieces of a row are stored XOR-permuted by (row/8)%8, so that
// the MFMA operand reads (lanes = rows eight apart, same k piece) of any eight
// consecutive lanes fall into eight different 16-byte bank groups: no conflicts,
// no padding.
//
// The A fragments of the wavefront's 32 rows for 128 k stay in registers; with
// K <= 128 they are loaded once per workgroup.
//
// Layout of a 32 x 128 score block in a wavefront (MFMA with A rows as the first
// operand): lane (j = lane%16, rg = lane/16), accumulator [rt][ct][e] is row
// 16*rt + 4*rg + e, column 8*j + ct of the block -- column tile ct takes the B
// rows 8*j + ct, so a lane owns EIGHT CONSECUTIVE columns of each of its rows and
// the sixteen lanes of a row group cover the block's 128 columns in order: one
// 16-byte store per lane and row (two for fp32 output), contiguous across adjacent
// lanes, 256 bytes per row and instruction.  The memory pipeline works per lane
// access, so wide per-lane pieces that are contiguous across lanes are what
// reaches the store rate of the machine.
//
// Softmax in two sweeps over the columns.  Sweep 1 keeps, per lane and row, a
// running maximum and a running sum of exp2((s - max) * c) over the lane's own
// columns (rescaled when the maximum moves); after it the sixteen lanes of a row
// group are combined once.  Sweep 2 recomputes the scores and writes
// exp2((s - max) * c - log2(sum)): the division rides in the exponent.  The scores never touch memory; the price is the
// second set of MFMAs, which this memory-bound kernel has room for.
//
// Ragged N: the last column chunk is the 128 columns ENDING at N (it overlaps the
// previous chunk when N % 128 != 0); the overlapped columns get weight 0 in the
// running sum and are stored a second time with identical values.  There are no
// partial stores and no column masks.  Ragged M: rows past M read as zeros
// (buffer range) and are not stored.
#pragma once
#include <type_traits>

#include "ba_gemm_common.hpp"

namespace ba {

constexpr int kTileWaves = 4;
constexpr int kTileThreads = 64 * kTileWaves;
constexpr int kRT = 2;                                   // MFMA row tiles per wavefront
constexpr int kCT = kTileCols / 16;                      // MFMA column tiles per chunk (8)
constexpr int kTileWaveRows = 16 * kRT;                  // 32 rows per wavefront
constexpr int kTileRows = kTileWaves * kTileWaveRows;    // 128 rows per workgroup
constexpr int kSlabK = 64;                               // k per LDS chunk (two MFMA k-steps)
constexpr int kSpanK = 128;                              // k whose A fragments stay in registers
constexpr int kSpanSteps = kSpanK / 32;
constexpr int kTileChunkBytes = kTileCols * kSlabK * 2;  // 16 KiB
constexpr int kStages = 4;                               // LDS chunks in flight or in use
constexpr int kFillInsts = 4;                            // global->LDS instructions per wavefront and chunk
static_assert(kTileCols == 128, "the fill and the operand reads below are written for 128-column chunks");

// Workgroup -> (segment, head, row block).  Workgroups are handed to the eight
// accelerator dies round-robin by their linear index, and each die has its own
// L2: index 8*slot + die is given pair (slot / zdim) * 8 + die and row block
// slot % zdim, so all row blocks of one (segment, head) pair -- which read the
// same B_g -- run on one die, one after the other.
constexpr int kDies = 8;

// s_waitcnt vmcnt(N) only (other counters unbounded).  Vector memory operations of one wavefront
// complete in issue order, so "at most N outstanding" means that all but the last N have completed.
template <int N> __device__ __forceinline__ void wait_vm() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit count");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// The row blocks z0, z0 + zdim, ... (128 rows each) of one segment and head, by one workgroup of kTileThreads
// work-items; lds = its kStages * kTileChunkBytes bytes of LDS (1 KiB aligned).
template <int DT, bool FUSED, bool F32OUT>
__device__ __forceinline__ void tile_rows(const RunArgs &a, const Seg &s, int z0, int zdim, unsigned char *lds) {
    const int M = s.M, N = s.N, K = s.K;
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const SegRes res = make_res(s, a.A, a.B);
    const char *bseg = reinterpret_cast<const char *>((const uint16_t *)a.B + s.b);
    constexpr int kOutBytes = F32OUT ? 4 : 2;
    // Output through a buffer descriptor of exactly the segment: rows past M fall outside and are dropped
    // by the hardware, so every wavefront issues the same number of store instructions.
    const __amdgpu_buffer_rsrc_t out_res = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<char *>(a.out) + s.o * kOutBytes, 0, (int)((uint32_t)M * (uint32_t)N * kOutBytes), kRsrcFlags);
    constexpr int kStoreInsts = (F32OUT ? 2 : 1) * kRT * 4;  // per store iteration and wavefront
    const u32x4 zero = {0u, 0u, 0u, 0u};

    // K = 0: one slab of zeros (no fill is issued for it, the stages are cleared instead), so that the sweeps
    // run and the rows come out as zeros, or as 1/N from the fused call
    const int nslab = K > 0 ? (K + kSlabK - 1) / kSlabK : 1;
    const int nspan = K > 0 ? (K + kSpanK - 1) / kSpanK : 1;
    const int ncb = (N + kTileCols - 1) / kTileCols;
    const int per_sweep = ncb * nslab;
    const int total = (FUSED ? 2 : 1) * per_sweep;
    const int full_cols = (N / kTileCols) * kTileCols;          // columns covered by whole chunks
    const bool overlap = full_cols != N;                         // the last chunk overlaps the one before
    const float c_signed = a.scale * kLog2e;
    const bool negate = FUSED && c_signed < 0.f;                // |scale| on negated scores
    const float c = __builtin_fabsf(c_signed);

    // LDS image of a chunk: two consecutive rows (2 x 128 bytes) form a 256-byte super-row of sixteen
    // 16-byte slots; piece p of row r sits in super-row r/2 at slot ((r%2)*8 + p) ^ ((r/8)%16).  The
    // sixteen lanes of an operand read (rows eight apart, same piece) then hit sixteen different slots.
    // Fill: instruction i of this wavefront covers LDS positions (wave + 4*i)*64 + lane, i.e. super-rows
    // (wave + 4*i)*4 + lane/16, whose XOR key (wave + 4*i)%16 is the same for the whole instruction;
    // its lanes read the two rows of a super-row, 128 contiguous bytes each.
    auto fill = [&](int cbi, int slab, int stage) {
        const int cb = cbi == ncb - 1 ? N - kTileCols : cbi * kTileCols;
        const int k0 = slab * kSlabK;
        const char *src = bseg + ((size_t)cb * K + k0) * 2;
        unsigned char *buf = lds + stage * kTileChunkBytes + wave * 1024;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int v = (lane & 15) ^ ((wave + 4 * i) & 15);
            const int row = 2 * ((wave + 4 * i) * 4 + (lane >> 4)) + (v >> 3);
            const int piece = v & 7;
            const int off = (row * K + piece * 8) * 2;
            if (k0 + piece * 8 < K)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + off),
                                                 (__attribute__((address_space(3))) void *)(buf + 4096 * i), 16, 0,
                                                 0);
        }
    };

    if (K == 0) {
        for (int i = threadIdx.x; i < kStages * kTileChunkBytes / 16; i += kTileThreads)
            reinterpret_cast<u32x4 *>(lds)[i] = zero;
        __syncthreads();
    }
    for (int rb = z0; rb * kTileRows < M; rb += zdim) {
        const int row0 = rb * kTileRows + wave * kTileWaveRows;     // first row of this wavefront
        const bool active = row0 < M;
        // A fragments: [rt][ks], row 16*rt + j of the wavefront's rows, k-group rg, for one span of 128 k
        u32x4 af[kRT][kSpanSteps];
        auto load_a = [&](int k0) {
#pragma unroll
            for (int rt = 0; rt < kRT; ++rt) {
                const int voff = ((row0 + 16 * rt + j) * K + k0 + rg * 8) * 2;
#pragma unroll
                for (int ks = 0; ks < kSpanSteps; ++ks) {
                    if (k0 + ks * 32 < K) {
                        u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff + ks * 64, 0, 0);
                        if (k0 + ks * 32 + rg * 8 >= K) v = zero;        // ragged last k-step
                        if (negate) v ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
                        af[rt][ks] = v;
                    } else if (K == 0 && ks == 0) {
                        af[rt][0] = zero;                                // the one k-step of a K = 0 segment
                    }
                }
            }
        };
        if (rb != z0) __syncthreads();                   // the previous row block is done with every buffer
        // (column chunk, k slab) of the next chunk to fill; wraps around for the second sweep
        int f_cbi = 0, f_slab = 0;
        auto advance = [&]() {
            if (++f_slab == nslab) {
                f_slab = 0;
                if (++f_cbi == ncb) f_cbi = 0;
            }
        };
        // Chunks 0 .. kStages-2 are requested up front; iteration `it` requests chunk it + kStages - 1
        // into the buffer that iteration it - 1 has just finished reading.
#pragma unroll
        for (int k = 0; k < kStages - 1; ++k) {
            if (k < total) {
                fill(f_cbi, f_slab, k);
                advance();
            }
        }
        int cbi = 0, slab = 0;                           // chunk being computed
        if (nspan == 1 && active) load_a(0);

        // sweep 1: running maximum and sum of the lane's own columns; sweep 2: m_run = -max*c - log2(sum) of the row
        float m_run[kRT][4], l_run[kRT][4];
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
            for (int e = 0; e < 4; ++e) { m_run[rt][e] = -3.0e38f; l_run[rt][e] = 0.f; }

        f32x4 acc[kRT][kCT];
        int stage = 0;                                   // buffer of chunk `it`
        // Vector memory instructions this wavefront has issued after the fill of chunk `it`: the fills
        // of the chunks after it, and the stores of the last kStages - 1 iterations (recent_stores keeps
        // 1 for an iteration that stored, newest first).  All of them may stay in flight.
        int recent_stores[kStages - 1];
#pragma unroll
        for (int k = 0; k < kStages - 1; ++k) recent_stores[k] = 0;
        const bool counted = nspan == 1;                 // A reloads in the loop (long K) are not counted
        for (int it = 0; it < total; ++it) {
            {
                // Wait for this wavefront's part of chunk `it`.  What it issued later may stay in flight:
                // the fills of the next kStages-2 chunks and the stores of the last kStages-1 iterations.
                // Near the end (fewer fills ahead) and with A reloads in the loop: wait for everything.
                int stores = 0;
#pragma unroll
                for (int k = 0; k < kStages - 1; ++k) stores += recent_stores[k];
                constexpr int kAhead = kFillInsts * (kStages - 2);
                if (!counted || it + kStages - 2 > total - 1) wait_vm<0>();
                else if (stores == 0) wait_vm<kAhead>();
                else if (stores == 1) wait_vm<kAhead + kStoreInsts>();
                else if (stores == 2) wait_vm<kAhead + 2 * kStoreInsts>();
                else wait_vm<kAhead + 3 * kStoreInsts>();
            }
            // ... everyone's; and the buffer of chunk it-1 is free.  A bare barrier: __syncthreads() would
            // also wait for every outstanding fill and store of this wavefront.
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            const int cb = cbi == ncb - 1 ? N - kTileCols : cbi * kTileCols;
            const int k0 = slab * kSlabK;
            const bool last_slab = slab == nslab - 1;
            const bool last_chunk = cbi == ncb - 1;
            const bool odd_slab = (slab & 1) != 0;       // second half of the A span
            if (it + kStages - 1 < total) {
                fill(f_cbi, f_slab, stage == 0 ? kStages - 1 : stage - 1);
                advance();
            }
            if (++slab == nslab) {                       // what the next iteration computes
                slab = 0;
                if (++cbi == ncb) cbi = 0;
            }
            const unsigned char *buf = lds + stage * kTileChunkBytes;
            stage = stage == kStages - 1 ? 0 : stage + 1;
#pragma unroll
            for (int k = kStages - 2; k > 0; --k) recent_stores[k] = recent_stores[k - 1];
            recent_stores[0] = 0;
            if (!active) continue;
            const bool second = FUSED && it >= per_sweep;
            if (nspan > 1 && !odd_slab) load_a(k0);
            // MFMA operand reads: row 8*j + ct of the chunk = super-row 4*j + ct/2, slot
            // ((ct%2)*8 + piece) ^ j with piece = ksl*4 + rg: two offsets per k-step (ct even / odd), ct/2 as
            // an immediate (256 bytes per super-row); past K any valid piece (the A side is zero)
            auto rd_off = [&](int ksl, int odd) {
                const int piece = (k0 + (ksl * 4 + rg) * 8 < K) ? ksl * 4 + rg : 0;
                return (4 * j * 16 + ((odd * 8 + piece) ^ j)) * 16;
            };
            // one k-step: ksl = k-step inside the LDS chunk, kss = k-step inside the A span
            auto kstep = [&](auto ksl_c, auto kss_c, auto first_c) {
                constexpr int ksl = decltype(ksl_c)::value, kss = decltype(kss_c)::value;
                const unsigned char *src0 = buf + rd_off(ksl, 0), *src1 = buf + rd_off(ksl, 1);
                u32x4 bf[kCT];
#pragma unroll
                for (int ct = 0; ct < kCT; ++ct)
                    bf[ct] = *reinterpret_cast<const u32x4 *>(((ct & 1) ? src1 : src0) + (ct >> 1) * 256);
#pragma unroll
                for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
                    for (int ct = 0; ct < kCT; ++ct)
                        acc[rt][ct] = Elem<DT>::mfma(af[rt][kss], bf[ct],
                                                     decltype(first_c)::value ? f32x4{0.f, 0.f, 0.f, 0.f} : acc[rt][ct]);
            };
            using I0 = std::integral_constant<int, 0>;
            using I1 = std::integral_constant<int, 1>;
            using I2 = std::integral_constant<int, 2>;
            using I3 = std::integral_constant<int, 3>;
            if (!odd_slab) {
                if (k0 == 0) kstep(I0{}, I0{}, std::true_type{});
                else kstep(I0{}, I0{}, std::false_type{});
                if (k0 + 32 < K) kstep(I1{}, I1{}, std::false_type{});
            } else {
                kstep(I0{}, I2{}, std::false_type{});
                if (k0 + 32 < K) kstep(I1{}, I3{}, std::false_type{});
            }
            if (!last_slab) continue;

            if (FUSED && !second) {
#pragma unroll
                for (int rt = 0; rt < kRT; ++rt) settle_mfma(acc[rt]);
                auto update = [&](auto weighted) {
                    float w[kCT];
#pragma unroll
                    for (int ct = 0; ct < kCT; ++ct) w[ct] = 1.f;
                    if (decltype(weighted)::value) {
#pragma unroll
                        for (int ct = 0; ct < kCT; ++ct) w[ct] = cb + 8 * j + ct >= full_cols ? 1.f : 0.f;
                    }
#pragma unroll
                    for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float m_old = m_run[rt][e];
                            float m_new = m_old;
#pragma unroll
                            for (int ct = 0; ct < kCT; ct += 2) m_new = max3(m_new, acc[rt][ct][e], acc[rt][ct + 1][e]);
                            const float bias = -m_new * c;
                            float l = l_run[rt][e] * __builtin_amdgcn_exp2f(fmaf(m_old, c, bias));
#pragma unroll
                            for (int ct = 0; ct < kCT; ++ct) {
                                const float pr = __builtin_amdgcn_exp2f(fmaf(acc[rt][ct][e], c, bias));
                                l = decltype(weighted)::value ? fmaf(pr, w[ct], l) : l + pr;
                            }
                            m_run[rt][e] = m_new;
                            l_run[rt][e] = l;
                        }
                };
                if (overlap && last_chunk) update(std::true_type{});
                else update(std::false_type{});
                if (it == per_sweep - 1) {
                    // combine the sixteen lanes of each row group; leave -max*c - log2(sum) for sweep 2
#pragma unroll
                    for (int rt = 0; rt < kRT; ++rt) {
                        float mx[4], sm[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) mx[e] = m_run[rt][e];
                        row16_max4(mx);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            sm[e] = l_run[rt][e] * __builtin_amdgcn_exp2f((m_run[rt][e] - mx[e]) * c);
                            m_run[rt][e] = -mx[e] * c;
                        }
                        row16_sum4(sm);
#pragma unroll
                        for (int e = 0; e < 4; ++e) m_run[rt][e] -= __builtin_amdgcn_logf(sm[e]);   // 1/sum goes into the exponent
                    }
                }
                continue;
            }

            // store sweep (GEMM only: the raw scores): values first, then one burst of stores
            if (FUSED) {
#pragma unroll
                for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
                    for (int ct = 0; ct < kCT; ++ct)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc[rt][ct][e] = __builtin_amdgcn_exp2f(fmaf(acc[rt][ct][e], c, m_run[rt][e]));
            }
            const uint32_t voff = (uint32_t)((row0 + 4 * rg) * N + cb + 8 * j) * kOutBytes;
#pragma unroll
            for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t off = voff + (uint32_t)((16 * rt + e) * N) * kOutBytes;
                    if (F32OUT) {
                        const f32x4 lo = {acc[rt][0][e], acc[rt][1][e], acc[rt][2][e], acc[rt][3][e]};
                        const f32x4 hi = {acc[rt][4][e], acc[rt][5][e], acc[rt][6][e], acc[rt][7][e]};
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, lo), out_res, off, 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, hi), out_res, off + 16, 0, 0);
                    } else {
                        const u32x4 v = {Elem<DT>::pack2(acc[rt][0][e], acc[rt][1][e]),
                                         Elem<DT>::pack2(acc[rt][2][e], acc[rt][3][e]),
                                         Elem<DT>::pack2(acc[rt][4][e], acc[rt][5][e]),
                                         Elem<DT>::pack2(acc[rt][6][e], acc[rt][7][e])};
                        __builtin_amdgcn_raw_buffer_store_b128(v, out_res, off, 0, 0);
                    }
                }
            recent_stores[0] = 1;
        }
    }
}


// One workgroup of the tile kernel: `block` is its index among the kernel's workgroups (it decides die,
// pair and row block), lds its kStages * kTileChunkBytes bytes of LDS (1 KiB aligned).
template <int DT, bool FUSED, bool F32OUT>
__device__ __forceinline__ void tile_block(const RunArgs &a, int zdim, unsigned block, unsigned char *lds) {
    const int die = block % kDies, slot = block / kDies;
    const int pair = (slot / zdim) * kDies + die;
    const int z0 = slot % zdim;
    const int H = (int)a.H;
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const bool ok = header_ok(a);
    if (!ok) {
        if (!(a.flags & kFlagQuiet) && block == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    // pairs = (entries of the work list, padded to a multiple of the die count) x heads, entry fastest,
    // and the entries rotated by the head: die d works on entries = (d + h) mod 8 of head h, so over the
    // heads every die sees every segment about equally often, however unequal the segments are.
    const int entries = a.list < 0 ? a.nseg : (int)((ConstHdr)(uintptr_t)a.plan)->totals[a.list];
    const int padded = (entries + kDies - 1) / kDies * kDies;
    if (entries <= 0 || pair >= padded * H) return;
    const int h = pair / padded;
    const int entry = (pair % padded + h) % padded;
    if (entry >= entries) return;
    bool valid;
    const Seg s = load_listed(pv, entry, h, a, valid);
    if (!valid) return;
    const int kind = s.kind;
    if (!tile_segment(kind, s.N, s.K)) return;
    if ((a.flags & kFlagPipeToo) && pipe_segment(kind, s.N, s.K)) return;      // the other kernel of this call takes it
    if ((a.flags & kFlagWideKToo) && wide_k_segment(kind, s.N, s.K)) return;   // likewise
    if ((a.flags & kFlagRowsToo) && s.K <= 128) return;
    tile_rows<DT, FUSED, F32OUT>(a, s, z0, zdim, lds);
}

}  // namespace ba
