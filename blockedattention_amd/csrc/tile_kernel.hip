// Large segments: S_g = A_g B_g^T and its row softmax for segments whose B_g does
// not fit the strip kernel's LDS window (N > 256, or N >= 64 with a long K).
//
// One workgroup = 256 rows of one segment and head; wavefront w owns rows
// 64w .. 64w+63 (four MFMA row tiles) and ALL columns, 64 at a time.  B_g is
// streamed through LDS in chunks of 64 columns x 128 k (16 KiB, two buffers): the
// chunk is a straight copy of 64 consecutive rows of B_g, fetched with direct
// global->LDS loads whose lanes read consecutive 16-byte pieces (fully
// coalesced), and reused by all sixteen row tiles of the workgroup.  Inside LDS
// the sixteen 16-byte pieces of a row are stored XOR-permuted by (row/4)%16, so
// that the MFMA operand reads (16 lanes = 16 rows four apart, same k piece) fall
// into 16 different 16-byte bank groups: no conflicts, no padding.
//
// The A fragments of the wavefront's 64 rows stay in registers for the whole
// kernel when K <= 128 (one slab); longer K walks slabs of 128 and reloads them.
//
// Layout of a 64 x 64 score block in a wavefront (MFMA with A rows as the first
// operand): lane (j = lane%16, rg = lane/16), accumulator [rt][ct][e] is row
// 16*rt + 4*rg + e, column 4*j + ct of the block -- column tile ct takes the B
// rows 4*j + ct, so a lane owns FOUR CONSECUTIVE columns of each of its rows and
// the sixteen lanes of a row group cover the block's 64 columns in order: stores
// are 8-byte (16-byte for fp32 output) pieces that are contiguous across adjacent
// lanes, 128 bytes per row and instruction.
//
// Softmax in two sweeps over the columns.  Sweep 1 keeps, per lane and row, a
// running maximum and a running sum of exp2((s - max) * c) over the lane's own
// columns (rescaled when the maximum moves); after it the sixteen lanes of a row
// group are combined once.  Sweep 2 recomputes the scores, and writes
// exp2((s - max) * c) / sum.  The scores never touch memory; the price is the
// second set of MFMAs, which this memory-bound kernel has room for.
//
// Ragged N: the last column chunk is the 64 columns ENDING at N (it overlaps the
// previous chunk when N % 64 != 0); the overlapped columns get weight 0 in the
// running sum and are stored a second time with identical values.  There are no
// partial stores and no column masks.  Ragged M: rows past M read as zeros
// (buffer range) and are not stored.
#include <algorithm>
#include <type_traits>

#include "ba_gemm_common.hpp"

namespace ba {

constexpr int kTileWaves = 4;
constexpr int kTileThreads = 64 * kTileWaves;
constexpr int kTileWaveRows = 64;                        // four MFMA row tiles per wavefront
constexpr int kTileRows = kTileWaves * kTileWaveRows;    // 256 rows per workgroup
constexpr int kTileSlabK = 128;                          // k per LDS chunk
constexpr int kTileSteps = kTileSlabK / 32;
constexpr int kTileChunkBytes = kTileCols * kTileSlabK * 2;   // 16 KiB

// Workgroup -> (segment, head, row block).  Workgroups are handed to the eight
// accelerator dies round-robin by their linear index, and each die has its own
// L2: index 8*slot + die is given pair (slot / zdim) * 8 + die and row block
// slot % zdim, so all row blocks of one (segment, head) pair -- which read the
// same B_g -- run on one die, one after the other.
constexpr int kDies = 8;

template <int DT, bool FUSED, bool F32OUT>
__global__ __launch_bounds__(kTileThreads, 2) void tile_kernel(RunArgs a, int zdim) {
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kTileChunkBytes];
    const int die = blockIdx.x % kDies, slot = blockIdx.x / kDies;
    const int pair = (slot / zdim) * kDies + die;
    const int z0 = slot % zdim;
    const int H = (int)a.H;
    if (pair >= a.nseg * H) return;
    const int g = pair % a.nseg;
    const int64_t h = pair / a.nseg;
    const PlanRO pv = plan_ro(a.plan, a.nseg);
    const bool ok = header_ok(a);
    const Seg s = load_seg(pv, g, h, a);
    const int kind = pv.recs[g].kind;
    if (!ok) {
        if (!(a.flags & kFlagQuiet) && blockIdx.x == 0 && threadIdx.x == 0)
            atomicAdd(&reinterpret_cast<PlanHeader *>(a.plan)->run_errors, 1);
        return;
    }
    if (!tile_segment(kind, s.N, s.K)) return;
    const int M = s.M, N = s.N, K = s.K;
    const int lane = lane_id(), j = lane & 15, rg = lane >> 4;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const SegRes res = make_res(s, a.A, a.B);
    const char *bseg = reinterpret_cast<const char *>((const uint16_t *)a.B + s.b);
    const u32x4 zero = {0u, 0u, 0u, 0u};

    const int nslab = (K + kTileSlabK - 1) / kTileSlabK;
    const int ncb = (N + kTileCols - 1) / kTileCols;
    const int per_sweep = ncb * nslab;
    const int total = (FUSED ? 2 : 1) * per_sweep;
    const int full_cols = (N / kTileCols) * kTileCols;          // columns covered by whole chunks
    const bool overlap = full_cols != N;                         // the last chunk overlaps the one before
    const float c_signed = a.scale * kLog2e;
    const bool negate = FUSED && c_signed < 0.f;                // |scale| on negated scores
    const float c = __builtin_fabsf(c_signed);
    constexpr int kOutBytes = F32OUT ? 4 : 2;

    // Fill: LDS position p (16-byte units) = row * 16 + (piece ^ (row/4)%16).  Instruction i of this
    // wavefront covers positions wave*64 + 256*i + lane: rows wave*4 + 16*i + lane/16, whose
    // row/4 = wave + 4*i is the same for the whole instruction.
    auto fill = [&](int cbi, int slab, int parity) {
        const int cb = cbi == ncb - 1 ? N - kTileCols : cbi * kTileCols;
        const int k0 = slab * kTileSlabK;
        const char *src = bseg + ((size_t)cb * K + k0) * 2;
        unsigned char *buf = lds + parity * kTileChunkBytes + wave * 1024;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = wave * 4 + 16 * i + rg;
            const int piece = j ^ ((wave + 4 * i) & 15);
            const int off = (row * K + piece * 8) * 2;
            if (k0 + piece * 8 < K)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + off),
                                                 (__attribute__((address_space(3))) void *)(buf + 4096 * i), 16, 0,
                                                 0);
        }
    };
    for (int rb = z0; rb * kTileRows < M; rb += zdim) {
        const int row0 = rb * kTileRows + wave * kTileWaveRows;     // first row of this wavefront
        const bool active = row0 < M;
        // A fragments: [rt][ks], row 16*rt + j of the wavefront's rows, k-group rg
        u32x4 af[4][kTileSteps];
        auto load_a = [&](int k0) {
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const int voff = ((row0 + 16 * rt + j) * K + k0 + rg * 8) * 2;
#pragma unroll
                for (int ks = 0; ks < kTileSteps; ++ks) {
                    if (k0 + ks * 32 < K) {
                        u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(res.a, voff + ks * 64, 0, 0);
                        if (k0 + ks * 32 + rg * 8 >= K) v = zero;        // ragged last k-step
                        if (negate) v ^= u32x4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
                        af[rt][ks] = v;
                    }
                }
            }
        };
        if (rb != z0) __syncthreads();                   // the previous row block is done with both buffers
        // (column chunk, k slab) of the chunk being filled; wraps around for the second sweep
        int f_cbi = 0, f_slab = 0;
        auto advance = [&]() {
            if (++f_slab == nslab) {
                f_slab = 0;
                if (++f_cbi == ncb) f_cbi = 0;
            }
        };
        fill(0, 0, 0);
        advance();
        int cbi = 0, slab = 0;                           // chunk being computed
        if (nslab == 1 && active) load_a(0);

        // sweep 1: running maximum and sum of the lane's own columns; sweep 2: -max*c and 1/sum of the row
        float m_run[4][4], l_run[4][4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int e = 0; e < 4; ++e) { m_run[rt][e] = -3.0e38f; l_run[rt][e] = 0.f; }

        f32x4 acc[4][4];
        __builtin_amdgcn_s_waitcnt(0x0F70);              // vmcnt(0): chunk 0 (this wavefront's part) has landed
        for (int it = 0; it < total; ++it) {
            __syncthreads();                             // chunk `it` is complete; the other buffer is free
            const int cb = cbi == ncb - 1 ? N - kTileCols : cbi * kTileCols;
            const int k0 = slab * kTileSlabK;
            const bool last_slab = slab == nslab - 1;
            const bool last_chunk = cbi == ncb - 1;
            if (it + 1 < total) fill(f_cbi, f_slab, (it + 1) & 1);
            cbi = f_cbi; slab = f_slab;                  // what the next iteration computes
            advance();
            if (!active) {
                __builtin_amdgcn_s_waitcnt(0x0F70);
                continue;
            }
            const bool second = FUSED && it >= per_sweep;
            if (nslab > 1) load_a(k0);
            const unsigned char *buf = lds + (it & 1) * kTileChunkBytes;
            // MFMA operand reads: row 4*j + ct of the chunk, piece ks*4 + rg -> one offset per k-step,
            // ct as an immediate (256 bytes per row); past K any valid piece (the A side is zero)
            auto rd_off = [&](int ks) {
                const int piece = (k0 + (ks * 4 + rg) * 8 < K) ? ks * 4 + rg : 0;
                return (4 * j * 16 + (piece ^ j)) * 16;
            };
            {
                u32x4 bf[4];
#pragma unroll
                for (int ct = 0; ct < 4; ++ct) bf[ct] = *reinterpret_cast<const u32x4 *>(buf + rd_off(0) + ct * 256);
                if (k0 == 0) {
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                        for (int ct = 0; ct < 4; ++ct)
                            acc[rt][ct] = Elem<DT>::mfma(af[rt][0], bf[ct], f32x4{0.f, 0.f, 0.f, 0.f});
                } else {
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                        for (int ct = 0; ct < 4; ++ct) acc[rt][ct] = Elem<DT>::mfma(af[rt][0], bf[ct], acc[rt][ct]);
                }
            }
#pragma unroll
            for (int ks = 1; ks < kTileSteps; ++ks) {
                if (k0 + ks * 32 < K) {
                    u32x4 bf[4];
#pragma unroll
                    for (int ct = 0; ct < 4; ++ct)
                        bf[ct] = *reinterpret_cast<const u32x4 *>(buf + rd_off(ks) + ct * 256);
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                        for (int ct = 0; ct < 4; ++ct) acc[rt][ct] = Elem<DT>::mfma(af[rt][ks], bf[ct], acc[rt][ct]);
                }
            }
            if (!last_slab) {
                __builtin_amdgcn_s_waitcnt(0x0F70);
                continue;
            }

            if (FUSED && !second) {
                auto update = [&](auto weighted) {
                    float w[4] = {1.f, 1.f, 1.f, 1.f};
                    if (decltype(weighted)::value) {
#pragma unroll
                        for (int ct = 0; ct < 4; ++ct) w[ct] = cb + 4 * j + ct >= full_cols ? 1.f : 0.f;
                    }
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float m_old = m_run[rt][e];
                            float m_new = max3(m_old, acc[rt][0][e], acc[rt][1][e]);
                            m_new = max3(m_new, acc[rt][2][e], acc[rt][3][e]);
                            const float bias = -m_new * c;
                            float l = l_run[rt][e] * __builtin_amdgcn_exp2f(fmaf(m_old, c, bias));
#pragma unroll
                            for (int ct = 0; ct < 4; ++ct) {
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
                    // combine the sixteen lanes of each row group; leave -max*c and 1/sum for sweep 2
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt) {
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
                        for (int e = 0; e < 4; ++e) l_run[rt][e] = __builtin_amdgcn_rcpf(sm[e]);
                    }
                }
                __builtin_amdgcn_s_waitcnt(0x0F70);
                continue;
            }

            // store sweep (GEMM only: the raw scores): values first, then one burst of stores
            if (FUSED) {
#pragma unroll
                for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                    for (int ct = 0; ct < 4; ++ct)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc[rt][ct][e] =
                                __builtin_amdgcn_exp2f(fmaf(acc[rt][ct][e], c, m_run[rt][e])) * l_run[rt][e];
            }
            char *const obase = reinterpret_cast<char *>(a.out) + (s.o + (int64_t)row0 * N + cb) * kOutBytes;
            const uint32_t voff = (uint32_t)(4 * rg * N + 4 * j) * kOutBytes;
            const int rows_here = M - row0 - 4 * rg;                 // rows of this lane's group that exist
            // The stores of the previous chunk have had this whole iteration to drain, and the fill
            // issued above has had it to land: wait for both here, not at the top of the loop.
            __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (16 * rt + e < rows_here) {
                        char *dst = obase + (size_t)(16 * rt + e) * N * kOutBytes + voff;
                        if (F32OUT)
                            *reinterpret_cast<f32x4_unaligned *>(dst) =
                                f32x4{acc[rt][0][e], acc[rt][1][e], acc[rt][2][e], acc[rt][3][e]};
                        else
                            *reinterpret_cast<u32x2_unaligned *>(dst) =
                                u32x2{Elem<DT>::pack2(acc[rt][0][e], acc[rt][1][e]),
                                      Elem<DT>::pack2(acc[rt][2][e], acc[rt][3][e])};
                    }
                }
        }
    }
}

template <int DT, bool FUSED, bool F32OUT>
static void launch_one(const RunArgs &args, unsigned groups, int zdim, hipStream_t stream) {
    hipLaunchKernelGGL((tile_kernel<DT, FUSED, F32OUT>), dim3(groups), dim3(kTileThreads), 0, stream, args, zdim);
}

// Launches the tile kernel over (segment, head, row block).  With a plan summary the row-block
// dimension covers the tallest segment; without it the workgroups loop over row blocks.
int launch_tiles(int dtype, int fused, const RunArgs &args, int64_t nseg, const ba_plan_info *info,
                 hipStream_t stream) {
    int64_t z = 4;
    if (info) {
        nseg = info->nseg;
        z = std::max<int64_t>(1, std::min<int64_t>(64, (std::max<int64_t>(info->max_M, 1) + kTileRows - 1) / kTileRows));
    }
    if (nseg <= 0) return BA_OK;
    const int64_t pairs = nseg * args.H;
    const int64_t groups = (pairs + kDies - 1) / kDies * kDies * z;
    if (pairs > (int64_t(1) << 30) || groups > (int64_t(1) << 31) - 1) return BA_ERR_UNSUPPORTED;
    const bool f32out = args.flags & kFlagOutF32;
    if (dtype == BA_F16) {
        if (!fused) launch_one<0, false, false>(args, (unsigned)groups, (int)z, stream);
        else if (f32out) launch_one<0, true, true>(args, (unsigned)groups, (int)z, stream);
        else launch_one<0, true, false>(args, (unsigned)groups, (int)z, stream);
    } else if (dtype == BA_BF16) {
        if (!fused) launch_one<1, false, false>(args, (unsigned)groups, (int)z, stream);
        else if (f32out) launch_one<1, true, true>(args, (unsigned)groups, (int)z, stream);
        else launch_one<1, true, false>(args, (unsigned)groups, (int)z, stream);
    } else {
        return BA_ERR_UNSUPPORTED;
    }
    return hipGetLastError() == hipSuccess ? BA_OK : BA_ERR_LAUNCH;
}

}  // namespace ba
