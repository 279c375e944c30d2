// extern "C" entry points of libblockedattn_hip.so: argument checks, flag
// derivation and kernel launches.  No allocation, no host synchronisation
// except ba_plan_read.
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <mutex>

#include "ba_host.hpp"

// Plan buffer of ba_gemm_softmax_static: one array per GPU the library runs on, held until the process ends.
// In host code the name is only a handle for hipGetSymbolAddress; kernels and launch arguments get the
// address that call returns for the current device.
constexpr size_t kStaticPlanBytes = (ba::plan_bytes_for(BA_STATIC_MAX_SEGMENTS) + 255) & ~size_t(255);
static __device__ __align__(256) unsigned char scratch[kStaticPlanBytes];

namespace ba {

// Device address of `scratch` on the current device, looked up once per device.
static void *static_plan_buffer() {
    static std::mutex lock;
    static void *ptr[64] = {nullptr};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> guard(lock);
    if (!ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        ptr[dev] = p;
    }
    return ptr[dev];
}

int device_cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// The MFMA paths load operand rows 16 bytes at a time: that needs untransposed
// layouts, 16-byte aligned base pointers and, with more than one head, per-head
// strides that keep every head's rows aligned.  (Per-segment alignment is
// settled by the scheduler.)
static int mfma_flag(const RunArgs &r) {
    if (r.flags & (kFlagTranspose1 | kFlagTranspose2)) return 0;
    if ((((uintptr_t)r.A | (uintptr_t)r.B) & 15) != 0) return 0;
    if (r.H > 1 && ((r.Dm1 | r.Dm2) & 7) != 0) return 0;
    return kFlagMfmaOk;
}

static bool bad_sizes(int64_t H, int64_t d1, int64_t d2, int64_t d3) { return H < 0 || d1 < 0 || d2 < 0 || d3 < 0; }

}  // namespace ba

using namespace ba;

extern "C" {

__attribute__((visibility("default"))) const char *ba_status_string(int status) {
    switch (status) {
        case BA_OK: return "ok";
        case BA_ERR_INVALID_ARG: return "invalid argument";
        case BA_ERR_WORKSPACE: return "plan buffer too small or misaligned";
        case BA_ERR_UNSUPPORTED: return "unsupported dtype or flag combination";
        case BA_ERR_LAUNCH: return "HIP launch or copy failed";
        case BA_ERR_BAD_METADATA: return "segment metadata rejected on the device";
        default: return "unknown status";
    }
}

__attribute__((visibility("default"))) int ba_abi_version(void) { return BA_ABI_VERSION; }

__attribute__((visibility("default"))) size_t ba_plan_bytes(int64_t nseg) {
    if (nseg < 0) return 0;
    return (plan_bytes_for(nseg) + 255) & ~size_t(255);
}

__attribute__((visibility("default"))) int ba_plan_gemm(void *plan, size_t plan_bytes, int64_t nseg, int mode,
                                                        int64_t *MList, int64_t *NList, int64_t *KList,
                                                        int64_t *accum1, int64_t *accum2, int64_t *accumOut,
                                                        ba_stream_t stream) {
    return launch_schedule(plan, plan_bytes, nseg, mode, 0, MList, NList, KList, accum1, accum2, accumOut,
                           (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_plan_softmax(void *plan, size_t plan_bytes, int64_t nseg,
                                                           const int64_t *rowList, const int64_t *colList,
                                                           int64_t *accum, int accum_given, ba_stream_t stream) {
    return launch_schedule(plan, plan_bytes, nseg, accum_given ? BA_META_GIVEN : BA_META_FROM_LISTS, 1,
                           const_cast<int64_t *>(rowList), const_cast<int64_t *>(colList), nullptr, nullptr,
                           nullptr, accum, (hipStream_t)stream);
}

// host copy of a plan header -> the public summary
static int info_from_header(const PlanHeader &h, ba_plan_info *info) {
    if (h.magic != kPlanMagic) return BA_ERR_INVALID_ARG;
    memset(info, 0, sizeof(*info));
    info->nseg = h.nseg;
    info->Dm1 = h.Dm1; info->Dm2 = h.Dm2; info->Dout = h.Dout;
    info->total_rows = h.total_rows;
    info->gemm_items = h.totals[kPfxGemm];
    info->strip_items = h.totals[kPfxStrip];
    info->split_items = h.totals[kPfxSplit];
    info->wide_items = h.totals[kPfxWide];
    info->pack_items = h.totals[kPfxPack];
    info->slow_items = h.totals[kPfxSlow];
    info->max_M = h.max_M; info->max_N = h.max_N; info->max_K = h.max_K;
    info->bad_segments = h.bad_segments;
    info->run_errors = h.run_errors;
    info->list_small = (int32_t)h.totals[kListSmall];
    info->list_big = (int32_t)h.totals[kListBig];
    info->list_tile = (int32_t)h.totals[kListTile];
    info->list_rest = (int32_t)h.totals[kListRest];
    info->list_rows = (int32_t)h.totals[kListRows];
    info->small_max_N = h.small_max_N;
    info->small_max_M = h.small_max_M;
    info->att_blocks64 = h.att_blocks64;
    info->att_blocks128 = h.att_blocks128;
    info->list_mini = h.mini_count;
    info->list_pipe = h.pipe_count;
    info->pipe_groups = h.pipe_groups;
    info->min_N = h.min_N; info->min_K = h.min_K;
    info->ring_groups = h.ring_groups;
    info->wide_groups = h.wide_groups;
    return (h.bad_segments || h.run_errors) ? BA_ERR_BAD_METADATA : BA_OK;
}

static int read_header_through(const void *plan, ba_plan_info *info, PlanHeader *staging, hipStream_t stream) {
    if (hipMemcpyAsync(staging, plan, sizeof(PlanHeader), hipMemcpyDeviceToHost, stream) != hipSuccess) return BA_ERR_LAUNCH;
    if (hipStreamSynchronize(stream) != hipSuccess) return BA_ERR_LAUNCH;
    const PlanHeader h = *staging;
    return info_from_header(h, info);
}

__attribute__((visibility("default"))) int ba_plan_read(const void *plan, ba_plan_info *info, ba_stream_t stream) {
    if (!plan || !info) return BA_ERR_INVALID_ARG;
    // The header lands in pinned host memory (one 256-byte buffer per calling thread, allocated at the thread's
    // first call and kept for the life of the process): the copy then needs no staging by the runtime.
    static thread_local PlanHeader *pinned = [] {
        void *p = nullptr;
        return hipHostMalloc(&p, sizeof(PlanHeader), hipHostMallocDefault) == hipSuccess ? (PlanHeader *)p : nullptr;
    }();
    PlanHeader on_stack;
    return read_header_through(plan, info, pinned ? pinned : &on_stack, (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_plan_read_into(const void *plan, ba_plan_info *info, void *staging,
                                                             ba_stream_t stream) {
    if (!plan || !info || !staging || ((uintptr_t)staging & 15)) return BA_ERR_INVALID_ARG;
    return read_header_through(plan, info, reinterpret_cast<PlanHeader *>(staging), (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_plan_gemm_notify(void *plan, size_t plan_bytes, int64_t nseg, int mode,
                                                               int64_t *MList, int64_t *NList, int64_t *KList,
                                                               int64_t *accum1, int64_t *accum2, int64_t *accumOut,
                                                               void *mailbox, uint32_t ticket, ba_stream_t stream) {
    if (!mailbox) return BA_ERR_INVALID_ARG;
    return launch_schedule(plan, plan_bytes, nseg, mode, 0, MList, NList, KList, accum1, accum2, accumOut,
                           (hipStream_t)stream, mailbox, ticket);
}

__attribute__((visibility("default"))) int ba_plan_softmax_notify(void *plan, size_t plan_bytes, int64_t nseg,
                                                                  const int64_t *rowList, const int64_t *colList,
                                                                  int64_t *accum, int accum_given, void *mailbox,
                                                                  uint32_t ticket, ba_stream_t stream) {
    if (!mailbox) return BA_ERR_INVALID_ARG;
    return launch_schedule(plan, plan_bytes, nseg, accum_given ? BA_META_GIVEN : BA_META_FROM_LISTS, 1,
                           const_cast<int64_t *>(rowList), const_cast<int64_t *>(colList), nullptr, nullptr,
                           nullptr, accum, (hipStream_t)stream, mailbox, ticket);
}

__attribute__((visibility("default"))) int ba_plan_wait(const void *mailbox, uint32_t ticket, ba_plan_info *info,
                                                        int64_t timeout_us) {
    if (!mailbox || !info) return BA_ERR_INVALID_ARG;
    const uint32_t *word = reinterpret_cast<const uint32_t *>(reinterpret_cast<const char *>(mailbox) + kMailboxTicket);
    const auto t0 = std::chrono::steady_clock::now();
    for (uint64_t spins = 0;; ++spins) {
        if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == ticket) break;
        __builtin_ia32_pause();                            // a polite spin: the sibling hardware thread gets the core
        if ((spins & 1023) == 1023 && timeout_us >= 0 &&
            std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count() > timeout_us)
            return BA_ERR_LAUNCH;
    }
    PlanHeader h;
    memcpy(&h, mailbox, sizeof(PlanHeader));
    return info_from_header(h, info);
}

__attribute__((visibility("default"))) int ba_varlen_gemm(void *plan, const ba_plan_info *info, int64_t nseg,
                                                          int dtype,
                                                          const void *A, const void *B, void *out, int64_t H,
                                                          int64_t Dm1, int64_t Dm2, int64_t Dout, int transpose1,
                                                          int transpose2, ba_stream_t stream) {
    if (!plan || nseg < 0 || nseg > (int64_t(1) << 30) || bad_sizes(H, Dm1, Dm2, Dout)) return BA_ERR_INVALID_ARG;
    if (H == 0 || Dout == 0 || nseg == 0) return BA_OK;
    if (!out || (Dm1 > 0 && !A) || (Dm2 > 0 && !B)) return BA_ERR_INVALID_ARG;
    RunArgs args{plan, A, B, out, H, Dm1, Dm2, Dout, 1.0f, 0, 0, 0, (int)nseg};
    if (transpose1) args.flags |= kFlagTranspose1;
    if (transpose2) args.flags |= kFlagTranspose2;
    args.flags |= mfma_flag(args);
    if (dtype != BA_F16 && dtype != BA_BF16) return launch_gemm_generic(dtype, args, nseg, info, (hipStream_t)stream);
    // Transposed layouts and unaligned operands, or a batch most of whose segments break the 16-byte operand
    // alignment (reduction lengths that are not multiples of 8, as in the backward products): the kernel that
    // stages both operands through LDS.  Everything else: the strip, tile and segment kernels.
    if (!(args.flags & kFlagMfmaOk) || (info && info->slow_items > 0 && 32 * info->slow_items > info->total_rows))
        return launch_gemm_any16(dtype, args, nseg, info, (hipStream_t)stream);
    return launch_strips(dtype, 0, args, nseg, info, (hipStream_t)stream);
}

// ba_varlen_gemm twice -- (plan_a: out_a = A_a B_a^T with B_a stored K x N) and (plan_b: out_b = A_b B_b^T with both
// operands stored k-major) -- as one launch, where that is possible; BA_ERR_UNSUPPORTED, with nothing launched, where
// it is not (the caller then makes the two calls).
__attribute__((visibility("default"))) int ba_varlen_gemm_two(int dtype, int64_t H, void *plan_a, const ba_plan_info *info_a,
                                                              const void *A_a, const void *B_a, void *out_a, int64_t Dm1_a,
                                                              int64_t Dm2_a, int64_t Dout_a, void *plan_b,
                                                              const ba_plan_info *info_b, const void *A_b, const void *B_b,
                                                              void *out_b, int64_t Dm1_b, int64_t Dm2_b, int64_t Dout_b,
                                                              ba_stream_t stream) {
    if (!plan_a || !plan_b || !info_a || !info_b) return BA_ERR_UNSUPPORTED;
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (bad_sizes(H, Dm1_a, Dm2_a, Dout_a) || bad_sizes(H, Dm1_b, Dm2_b, Dout_b)) return BA_ERR_INVALID_ARG;
    if (H == 0 || Dout_a == 0 || Dout_b == 0 || info_a->nseg <= 0 || info_b->nseg <= 0) return BA_ERR_UNSUPPORTED;
    if (!out_a || !out_b || !A_a || !B_a || !A_b || !B_b) return BA_ERR_UNSUPPORTED;
    RunArgs a{plan_a, A_a, B_a, out_a, H, Dm1_a, Dm2_a, Dout_a, 1.0f, kFlagTranspose2, 0, 0, (int)info_a->nseg};
    RunArgs b{plan_b, A_b, B_b, out_b, H, Dm1_b, Dm2_b, Dout_b, 1.0f, kFlagTranspose1 | kFlagTranspose2, 0, 0, (int)info_b->nseg};
    return launch_gemm_any16_two(dtype, a, info_a, b, info_b, (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_blocked_softmax(void *plan, const ba_plan_info *info, int64_t nseg,
                                                              int dtype,
                                                              const void *src, void *dst, int64_t H, int64_t Dsrc,
                                                              float scale, ba_stream_t stream) {
    if (!plan || nseg < 0 || H < 0 || Dsrc < 0) return BA_ERR_INVALID_ARG;
    if (H == 0 || Dsrc == 0 || nseg == 0) return BA_OK;
    if (!src || !dst) return BA_ERR_INVALID_ARG;
    return launch_softmax(dtype, plan, nseg, src, dst, H, Dsrc, scale, info, (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_blocked_softmax_backward(void *plan, const ba_plan_info *info,
                                                                       int64_t nseg, int dtype, const void *y,
                                                                       const void *dy,
                                                                       void *dx, int64_t H, int64_t Dsrc,
                                                                       float scale, ba_stream_t stream) {
    if (!plan || nseg < 0 || H < 0 || Dsrc < 0) return BA_ERR_INVALID_ARG;
    if (H == 0 || Dsrc == 0 || nseg == 0) return BA_OK;
    if (!y || !dy || !dx) return BA_ERR_INVALID_ARG;
    return launch_softmax_backward(dtype, plan, nseg, y, dy, dx, H, Dsrc, scale, info, (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_gemm_softmax(void *plan, const ba_plan_info *info, int64_t nseg,
                                                           int dtype,
                                                           const void *A, const void *B, void *out, int out_dtype,
                                                           int64_t H, int64_t Dm1, int64_t Dm2, int64_t Dout,
                                                           float scale, ba_stream_t stream) {
    if (!plan || nseg < 0 || nseg > (int64_t(1) << 30) || bad_sizes(H, Dm1, Dm2, Dout)) return BA_ERR_INVALID_ARG;
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (out_dtype != dtype && out_dtype != BA_F32) return BA_ERR_UNSUPPORTED;
    if (H == 0 || Dout == 0 || nseg == 0) return BA_OK;
    if (!out || (Dm1 > 0 && !A) || (Dm2 > 0 && !B)) return BA_ERR_INVALID_ARG;
    RunArgs args{plan, A, B, out, H, Dm1, Dm2, Dout, scale, 0, 0, 0, (int)nseg};
    args.flags |= mfma_flag(args);
    if (out_dtype == BA_F32) args.flags |= kFlagOutF32;
    return launch_strips(dtype, 1, args, nseg, info, (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_gemm_softmax_static(int64_t nseg, int mode, int64_t *MList,
                                                                  int64_t *NList, int64_t *KList, int64_t *accum1,
                                                                  int64_t *accum2, int64_t *accumOut, int dtype,
                                                                  const void *A, const void *B, void *out,
                                                                  int out_dtype, int64_t H, int64_t Dm1, int64_t Dm2,
                                                                  int64_t Dout, float scale, ba_stream_t stream) {
    if (nseg < 0 || bad_sizes(H, Dm1, Dm2, Dout)) return BA_ERR_INVALID_ARG;
    if (nseg > BA_STATIC_MAX_SEGMENTS) return BA_ERR_WORKSPACE;
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (out_dtype != dtype && out_dtype != BA_F32) return BA_ERR_UNSUPPORTED;
    // Small batches: one launch that reads the metadata itself; neither the scheduler nor the plan buffer is used.
    static const bool onecall = [] { const char *e = getenv("BLOCKEDATTN_ONECALL"); return !e || atoi(e) != 0; }();
    if (onecall && nseg >= 1 && nseg <= kOneCallMaxSegments && nseg * H <= kOneCallMaxPairs && mode != BA_META_FROM_ACCUM &&
        H > 0 && Dout > 0 && H * Dout <= kOneCallMaxElements && H * (Dm1 + Dm2) <= kOneCallMaxElements) {
        if (mode < 0 || mode > 2 || !MList || !NList || !KList) return BA_ERR_INVALID_ARG;
        if (mode == BA_META_GIVEN && (!accum1 || !accum2 || !accumOut)) return BA_ERR_INVALID_ARG;
        if (!out || (Dm1 > 0 && !A) || (Dm2 > 0 && !B)) return BA_ERR_INVALID_ARG;
        // (the buffer's first 256 bytes take the verdict of the call: see ba_static_read)
        RunArgs args{static_plan_buffer(), A, B, out, H, Dm1, Dm2, Dout, scale, 0, 0, 0, (int)nseg};
        if (!args.plan) return BA_ERR_LAUNCH;
        args.flags |= mfma_flag(args);
        if (out_dtype == BA_F32) args.flags |= kFlagOutF32;
        return launch_onecall(dtype, args, mode, MList, NList, KList, accum1, accum2, accumOut, (hipStream_t)stream);
    }
    void *plan = static_plan_buffer();
    if (!plan) return BA_ERR_LAUNCH;
    // The scheduler rewrites the whole header (run-error counter included), every record and every list entry
    // a kernel can reach, so nothing of the previous call's plan is read.
    const int st = launch_schedule(plan, kStaticPlanBytes, nseg, mode, 0, MList, NList, KList, accum1, accum2, accumOut,
                                   (hipStream_t)stream);
    if (st != BA_OK) return st;
    if (H == 0 || Dout == 0 || nseg == 0) return BA_OK;
    if (!out || (Dm1 > 0 && !A) || (Dm2 > 0 && !B)) return BA_ERR_INVALID_ARG;
    RunArgs args{plan, A, B, out, H, Dm1, Dm2, Dout, scale, 0, 0, 0, (int)nseg};
    args.flags |= mfma_flag(args);
    if (out_dtype == BA_F32) args.flags |= kFlagOutF32;
    return launch_strips(dtype, 1, args, nseg, nullptr, (hipStream_t)stream);
}

__attribute__((visibility("default"))) int ba_static_read(ba_plan_info *info, ba_stream_t stream) {
    if (!info) return BA_ERR_INVALID_ARG;
    void *plan = static_plan_buffer();
    if (!plan) return BA_ERR_LAUNCH;
    return ba_plan_read(plan, info, stream);
}

__attribute__((visibility("default"))) int ba_varlen_attention(void *plan, const ba_plan_info *info, int64_t nseg,
                                                               int dtype, const void *Q, const void *K,
                                                               const void *V, void *out, int64_t H, int64_t Dm1,
                                                               int64_t Dm2, int64_t Dout, float scale,
                                                               ba_stream_t stream) {
    if (!plan || nseg < 0 || nseg > (int64_t(1) << 30) || bad_sizes(H, Dm1, Dm2, Dout)) return BA_ERR_INVALID_ARG;
    if (dtype != BA_F16 && dtype != BA_BF16) return BA_ERR_UNSUPPORTED;
    if (H == 0 || Dm1 == 0 || nseg == 0) return BA_OK;
    if (!out || !Q || (Dm2 > 0 && (!K || !V))) return BA_ERR_INVALID_ARG;
    RunArgs args{plan, Q, K, out, H, Dm1, Dm2, Dout, scale, 0, 0, 0, (int)nseg};
    return launch_attention(dtype, args, V, nseg, info, (hipStream_t)stream);
}

}  // extern "C"
