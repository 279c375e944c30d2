/*
 * blocked_attention.h -- C ABI of the MI355X (gfx950) varlen GEMM + blocked
 * softmax library (libblockedattn_hip.so).
 *
 * Everything is plain pointers and sizes: no torch types, no C++ types, no
 * exceptions.  All data and metadata pointers are DEVICE pointers unless a
 * parameter says "host".  All entry points are stream-ordered on `stream` (a
 * hipStream_t passed as void*; NULL is the null stream), return a ba_status
 * and, except ba_plan_read, never synchronise with the host and never
 * allocate: the only scratch is the caller-provided plan buffer.
 *
 * The reference (Sophie10001b/blockedAttention) has no C ABI; its boundary is
 * a pybind11 torch extension.  Each entry point below names the reference
 * interface it stands in for (paths relative to the reference checkout).
 *
 * Layout contract (csrc/cuda/spBlkGEMM.cu:133-150, 985-1008;
 * csrc/cuda/spBlkSoftmax.cu:95-107, 375-398): operands are [H, D] row-major,
 * segment g occupies [accum[g], accum[g+1]) of the last dimension, row-major
 * inside the segment; head h of a buffer starts at h * D elements.
 */
#ifndef BLOCKED_ATTENTION_H
#define BLOCKED_ATTENTION_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BA_ABI_VERSION 5

typedef void *ba_stream_t; /* hipStream_t */

typedef enum ba_status {
    BA_OK = 0,
    BA_ERR_INVALID_ARG = 1,  /* null pointer, negative size, unknown enum */
    BA_ERR_WORKSPACE = 2,    /* plan buffer too small or misaligned */
    BA_ERR_UNSUPPORTED = 3,  /* dtype / flag combination not built */
    BA_ERR_LAUNCH = 4,       /* HIP reported an error at launch or copy */
    BA_ERR_BAD_METADATA = 5  /* ba_plan_read: the device-side checks rejected segments */
} ba_status;

/* Element types: the set of the reference's AT_DISPATCH_ALL_TYPES_AND2(Half, BFloat16)
 * (csrc/cuda/spBlkGEMM.cu:1010).  The softmax takes the four floating types
 * (csrc/cuda/spBlkSoftmax.cu:400), the fused pair and the attention BA_F16 / BA_BF16. */
typedef enum ba_dtype {
    BA_F16 = 0, BA_BF16 = 1, BA_F32 = 2, BA_F64 = 3,
    BA_U8 = 4, BA_I8 = 5, BA_I16 = 6, BA_I32 = 7, BA_I64 = 8
} ba_dtype;

/* Which half of the metadata the caller supplies
 * (the three cases of csrc/sparseBlockedAttention.cpp:22-44). */
typedef enum ba_meta_mode {
    BA_META_FROM_LISTS = 0, /* lists are inputs, prefix sums are written   (cpp:22-29) */
    BA_META_FROM_ACCUM = 1, /* prefix sums are inputs, lists are written   (cpp:30-40) */
    BA_META_GIVEN = 2       /* both are inputs                             (cpp:41-44) */
} ba_meta_mode;

/* Host-visible summary of a plan (filled by ba_plan_read). */
typedef struct ba_plan_info {
    int64_t nseg;
    int64_t Dm1, Dm2, Dout; /* last prefix-sum entries = elements per head */
    int64_t total_rows;     /* rows of the softmax: sum of M over the segments with N >= 1 */
    /* work-item totals (16-row strips) by segment shape */
    int64_t gemm_items;     /* 16 x <=256 output pieces of segments with N > 256 */
    int64_t strip_items;    /* 16-row strips of aligned segments with N <= 256 */
    int64_t split_items;    /* 16-row strips with 256 < N <= 4096 */
    int64_t wide_items;     /* 16-row strips with N > 4096 */
    int64_t pack_items;     /* packs of tiny segments sharing one wavefront */
    int64_t slow_items;     /* 16-row strips of segments that need the element-wise path */
    int32_t max_M, max_N, max_K;
    int32_t bad_segments;   /* segments rejected by the device-side checks */
    int32_t run_errors;     /* kernels that refused to run against this plan */
    /* segments per launch class (lengths of the plan's work lists) */
    int32_t list_small;     /* strip kernel, main launch */
    int32_t list_big;       /* strip kernel, second launch with the 64 KiB window */
    int32_t list_tile;      /* tile kernel (large segments) */
    int32_t list_rest;      /* segment kernel: packs, element-wise class, leftovers */
    int32_t small_max_N;    /* widest segment of the strip kernel's main launch */
    int32_t small_max_M;    /* tallest segment of the strip kernel's main launch */
    int32_t list_rows;      /* softmax row kernel: segments with N > 256 (GEMM and softmax plans) */
    /* GEMM plans: row blocks of 64 and of 128 rows per head, summed over the segments with M >= 1 whatever
     * their N and K (one-pass attention: a segment without keys still has its output rows zeroed) */
    int32_t att_blocks64, att_blocks128;
    /* segments of the strip kernel's main launch that one wavefront can take alone (at most 64 rows, B_g of
     * at most 16 KiB); list_small counts the others */
    int32_t list_mini;
    /* segments of list_tile that the pipelined row-block kernel takes in a fused call with 16-bit results
     * (K <= 128), and how many workgroups of that kernel have found work in this plan since it was built */
    int32_t list_pipe;
    int32_t pipe_groups;
    /* smallest N and K over the segments that have rows and columns (0: none has), and how many workgroups of
     * the GEMM for transposed layouts have written their rows as whole lines (128 x 128 build, K <= 128,
     * N >= 128) since the plan was built */
    int32_t min_N, min_K;
    int32_t ring_groups;
    /* workgroups of the row-block kernel's build for 128 < K <= 256 (large segments, 16-bit results, whole-line
     * stores) that have found work in this plan since it was built */
    int32_t wide_groups;
} ba_plan_info;

const char *ba_status_string(int status);
int ba_abi_version(void);

/* Bytes of device memory a plan for nseg segments needs (256-byte aligned
 * buffer).  Depends on nseg only, so it can be sized without knowing any
 * segment shape. */
size_t ba_plan_bytes(int64_t nseg);

/*
 * Device-side segment scheduler for the GEMM (and the fused pair).
 * Stands in for the metadata derivation of sparseBlockedGEMM::forward
 * (csrc/sparseBlockedAttention.cpp:17-44) and for the host-side tile list of
 * __getTiling (csrc/cuda/spBlkGEMM.cu:943-983): one kernel, no host round
 * trip.  Depending on `mode` it reads or writes MList/NList/KList (int64[nseg])
 * and accum1/accum2/accumOut (int64[nseg+1]); the plan receives offsets, sizes
 * and one compacted work list per compute-kernel launch.
 * In BA_META_FROM_ACCUM the lists are derived in exact integer arithmetic.
 * Output pointers may be NULL when the caller does not need that half.
 */
int ba_plan_gemm(void *plan, size_t plan_bytes, int64_t nseg, int mode,
                 int64_t *MList, int64_t *NList, int64_t *KList,
                 int64_t *accum1, int64_t *accum2, int64_t *accumOut,
                 ba_stream_t stream);

/*
 * Scheduler for the standalone softmax.  Stands in for
 * sparseBlockedSoftmax::forward's prefix sum (csrc/sparseBlockedAttention.cpp:85-91)
 * and the per-row list of __getTiling (csrc/cuda/spBlkSoftmax.cu:358-373).
 * accum_given != 0: accum (int64[nseg+1]) is an input; else, if non-NULL, it is written.
 */
int ba_plan_softmax(void *plan, size_t plan_bytes, int64_t nseg,
                    const int64_t *rowList, const int64_t *colList,
                    int64_t *accum, int accum_given, ba_stream_t stream);

/* Copies the plan summary to the host and waits for it (the one blocking
 * call, and the one that allocates: 256 bytes of pinned host memory at a
 * thread's first call, kept for the life of the process, through which the
 * summary travels).  Returns BA_ERR_BAD_METADATA if the scheduler rejected any
 * segment or a kernel refused to run against the plan.
 *
 * The compute entry points below take `nseg` (the segment count the plan was
 * built for; it sizes the launch grids) and the summary as `info` (a HOST
 * pointer, may be NULL).  With it they launch exactly the kernels the plan has
 * work for, with grids that cover the work; without it they launch every
 * kernel with a resident-size grid and let the kernels read the counts from
 * the plan, which costs a few extra (empty) launches but no synchronisation.
 * The results are identical either way. */
int ba_plan_read(const void *plan, ba_plan_info *host_info, ba_stream_t stream);

/* ba_plan_read without the library's own pinned buffer: the summary travels through `staging`, at least 256 bytes
 * of host memory of the caller (pinned: no staging copy by the runtime), 16-byte aligned.  No counterpart in the
 * reference (which reads its totals with .item(), csrc/cuda/spBlkGEMM.cu:996-998); for callers that want no
 * allocation of any kind inside the library. */
int ba_plan_read_into(const void *plan, ba_plan_info *host_info, void *staging, ba_stream_t stream);

/* The schedulers once more, for calls whose metadata is new every time: in addition to the plan they write the
 * summary into `mailbox` -- BA_MAILBOX_BYTES of host memory that the GPU can write and the CPU reads coherently
 * (hipHostMalloc with hipHostMallocCoherent | hipHostMallocMapped), 16-byte aligned, caller-owned -- and behind it
 * the 32-bit `ticket`.  ba_plan_wait spins on the host until the mailbox shows that ticket (timeout_us < 0: without
 * limit; on a timeout BA_ERR_LAUNCH) and then returns what ba_plan_read would: no copy, no stream synchronisation.
 * Use a ticket that differs from the one the mailbox showed last.  They replace the same reference code as
 * ba_plan_gemm / ba_plan_softmax; the hand-over itself has no counterpart there. */
#define BA_MAILBOX_BYTES 320
int ba_plan_gemm_notify(void *plan, size_t plan_bytes, int64_t nseg, int mode,
                        int64_t *MList, int64_t *NList, int64_t *KList,
                        int64_t *accum1, int64_t *accum2, int64_t *accumOut,
                        void *mailbox, uint32_t ticket, ba_stream_t stream);
int ba_plan_softmax_notify(void *plan, size_t plan_bytes, int64_t nseg,
                           const int64_t *rowList, const int64_t *colList,
                           int64_t *accum, int accum_given, void *mailbox, uint32_t ticket, ba_stream_t stream);
int ba_plan_wait(const void *mailbox, uint32_t ticket, ba_plan_info *host_info, int64_t timeout_us);

/*
 * out[h, accumOut[g] + r*N_g + c] = sum_t A(h,g,r,t) * B(h,g,c,t), one rounding
 * to the operand dtype at the store.  Stands in for sparseBlockedGEMMLaunch
 * (csrc/sparseBlockedAttention.h:18, csrc/cuda/spBlkGEMM.cu:985-1033).
 * Dm1/Dm2/Dout are the per-head strides of A/B/out in elements and must equal
 * the plan's totals, otherwise the kernel writes nothing and records a run
 * error in the plan.  transpose1/transpose2 select the K x M / K x N segment
 * layouts (spBlkGEMM.cu:292-329, 363-400).  dtype: BA_F16, BA_BF16 (MFMA,
 * fp32 accumulate), or any other ba_dtype with the reference's generic kernel's
 * arithmetic (spBlkGEMM.cu:159: the accumulator has the element type; integer
 * results are exact modulo 2^bits).
 */
int ba_varlen_gemm(void *plan, const ba_plan_info *info, int64_t nseg, int dtype, const void *A, const void *B, void *out,
                   int64_t H, int64_t Dm1, int64_t Dm2, int64_t Dout,
                   int transpose1, int transpose2, ba_stream_t stream);

/*
 * dst row = softmax(scale * src row) for every row of every segment, computed
 * in fp32 (BA_F64: in double), one rounding at the store.  dtype: BA_F16,
 * BA_BF16, BA_F32 or BA_F64 (likewise in the backward below).  Stands in for sparseBlockedSoftmaxLaunch
 * (csrc/sparseBlockedAttention.h:20, csrc/cuda/spBlkSoftmax.cu:375-416);
 * scale = 1.0f reproduces it.  No column limit.  src == dst is allowed.
 */
int ba_blocked_softmax(void *plan, const ba_plan_info *info, int64_t nseg, int dtype, const void *src, void *dst,
                       int64_t H, int64_t Dsrc, float scale, ba_stream_t stream);

/*
 * dx row = scale * (dy row - sum(y row * dy row)) * y row, y being the saved
 * output of ba_blocked_softmax with the same scale.  Stands in for
 * sparseBlockedSoftmaxBackwardLaunch (csrc/sparseBlockedAttention.h:21,
 * csrc/cuda/spBlkSoftmax.cu:418-459).  dx may alias dy.
 */
int ba_blocked_softmax_backward(void *plan, const ba_plan_info *info, int64_t nseg, int dtype, const void *y, const void *dy,
                                void *dx, int64_t H, int64_t Dsrc, float scale, ba_stream_t stream);

/*
 * Fused pair: out = softmax(scale * A_g B_g^T) per segment with the scores kept
 * in fp32 registers between the two steps.  Equivalent to ba_varlen_gemm
 * followed by ba_blocked_softmax on (M, N, accumOut) without the intermediate
 * 16-bit rounding; it has no single counterpart in the reference (which offers
 * only the two separate launchers above) and takes a plan from ba_plan_gemm.
 * out_dtype: the operand dtype, or BA_F32 for fp32 probabilities.
 */
int ba_gemm_softmax(void *plan, const ba_plan_info *info, int64_t nseg, int dtype, const void *A, const void *B, void *out,
                    int out_dtype, int64_t H, int64_t Dm1, int64_t Dm2, int64_t Dout, float scale,
                    ba_stream_t stream);

/*
 * Varlen attention in one pass: out_g = softmax(scale * Q_g K_g^T) V_g per
 * segment and head, the M x N probabilities never written to memory.  It
 * stands in for the chain a caller of the reference runs for attention
 * (README.md:3): sparseBlockedGEMMLaunch, sparseBlockedSoftmaxLaunch and
 * sparseBlockedGEMMLaunch again with transpose2 on the values
 * (csrc/sparseBlockedAttention.h:18-20); the reference has no fused form.
 * Takes a plan from ba_plan_gemm over (M, N, K): Q_g is the M x K operand
 * (accum1 offsets, Dm1 per head), K_g and V_g are both N x K (accum2 offsets,
 * Dm2 per head), out_g is M x K at accum1 offsets of an [H, Dm1] buffer.  Dout
 * is the plan's third total (checked, nothing of that size is touched).
 * Every K_g <= 128 (larger: BA_ERR_UNSUPPORTED with info, a run error in the
 * plan without); any alignment.  N_g = 0 gives zeros.  The probabilities are
 * rounded to dtype before the second product; sums are fp32.
 * dtype: BA_F16 or BA_BF16.
 */
int ba_varlen_attention(void *plan, const ba_plan_info *info, int64_t nseg, int dtype, const void *Q, const void *K,
                        const void *V, void *out, int64_t H, int64_t Dm1, int64_t Dm2, int64_t Dout, float scale,
                        ba_stream_t stream);

/*
 * ba_gemm_softmax for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  Scheduler and fused pair in one
 * call: the plan lives in a buffer that is part of the library's device image
 * (one copy per GPU, held until the process ends), so the caller passes only
 * the metadata (mode and pointers as for ba_plan_gemm), operands and output.
 * Nothing is allocated and nothing is read back: the kernels take their work
 * lists from the plan on the device, exactly as ba_gemm_softmax does with
 * info == NULL, and give the same results.  Metadata the scheduler rejects
 * leaves `out` unwritten; ba_static_read (below) tells, at the price of a
 * synchronisation.
 * The FIRST call on a device looks up the buffer's address and sets kernel
 * attributes (host-side calls that do not belong in a stream capture): make
 * one call per device outside any capture, with any small batch, before the
 * calls that are captured.
 * Small batches (at most 512 segments, 1024 (segment, head) pairs and 2^24
 * values in each of A + B and out; modes BA_META_FROM_LISTS and BA_META_GIVEN)
 * run as ONE kernel launch that derives every segment's offsets and class from
 * the metadata itself: no scheduler launch, and the buffer is not touched (what
 * the reference does in host round trips at spBlkGEMM.cu:943-983 and 985-1033
 * happens inside the compute kernel).  The results are those of the plan-driven
 * kernels, except that tiny segments are not packed into shared tiles.
 * At most BA_STATIC_MAX_SEGMENTS segments: more returns BA_ERR_WORKSPACE.
 * All calls on one GPU share that GPU's buffer: calls that overlap on one GPU
 * (different streams or threads) race; calls on one stream do not.
 */
#define BA_STATIC_MAX_SEGMENTS 4096
int ba_gemm_softmax_static(int64_t nseg, int mode, int64_t *MList, int64_t *NList, int64_t *KList,
                           int64_t *accum1, int64_t *accum2, int64_t *accumOut, int dtype, const void *A,
                           const void *B, void *out, int out_dtype, int64_t H, int64_t Dm1, int64_t Dm2, int64_t Dout,
                           float scale, ba_stream_t stream);

/* Two calls of ba_varlen_gemm as ONE launch: (plan_a, transpose1 = 0, transpose2 = 1) and (plan_b, transpose1 = 1,
 * transpose2 = 1), the layouts of the two products of the backward pass (dA = dS B over plan_a = the forward's
 * metadata with N and K exchanged, dB = dS^T A over plan_b; reference: csrc/sparseBlockedAttention.cpp:52-72 makes the
 * two calls one after the other).  Only where both would run as the 64 x 64 build of the kernel for transposed
 * layouts with the summaries given (16-bit types, batches of short segments: there each product alone is a few rounds
 * of short-lived workgroups); otherwise BA_ERR_UNSUPPORTED and nothing is launched: make the two calls instead. */
int ba_varlen_gemm_two(int dtype, int64_t H, void *plan_a, const ba_plan_info *info_a, const void *A_a, const void *B_a,
                       void *out_a, int64_t Dm1_a, int64_t Dm2_a, int64_t Dout_a, void *plan_b, const ba_plan_info *info_b,
                       const void *A_b, const void *B_b, void *out_b, int64_t Dm1_b, int64_t Dm2_b, int64_t Dout_b,
                       ba_stream_t stream);

/* ba_plan_read on the buffer of ba_gemm_softmax_static (current device): the verdict of the LAST call of that entry
 * point on `stream` -- BA_ERR_BAD_METADATA with bad_segments / run_errors set when that call's metadata was
 * rejected or its totals did not match the sizes passed, in which case it wrote nothing.  Blocks like ba_plan_read
 * (so not for use under stream capture); after a single-launch call only nseg, Dm1, Dm2, Dout, bad_segments and
 * run_errors of the summary are meaningful.  No counterpart in the reference. */
int ba_static_read(ba_plan_info *host_info, ba_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* BLOCKED_ATTENTION_H */
