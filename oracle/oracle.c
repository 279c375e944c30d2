/*
 * CPU restatement of blockedAttention's varlen ("blocked") GEMM and blocked row
 * softmax, in plain C.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP library is
 * compared against; nothing in the shipped package links, imports or calls it.
 * Only the tests, the smoke check and the benchmark's CPU-baseline leg may.
 *
 * Every function names the reference lines whose semantics it restates
 * (paths relative to the reference checkout).  No reference code is copied:
 * the reference computes these results with CUDA tiles; this file states the
 * same results as direct loops.
 *
 * Pinning (see tests/test_oracle_*.py): prefix sums against the seed-0 known
 * totals and numpy.cumsum; list derivation by round trip and brute force over
 * [1,40]^3; GEMM by the integer closed form of the (11,13,5) arange case, by
 * identity operands and by dense batched matmul for equal-sized segments;
 * softmax by scipy.special.softmax, rows summing to one, constant rows and
 * shift invariance; work-lists by exact-cover brute force.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------- metadata */

/*
 * Lists -> exclusive prefix sums.
 * csrc/sparseBlockedAttention.cpp:22-29: accum1 = cumsum([0, M*K]),
 * accum2 = cumsum([0, N*K]), accumOut = cumsum([0, M*N]); int64, length B+1.
 */
ORACLE_API void oracle_lists_to_accum(const int64_t *M, const int64_t *N, const int64_t *K, int64_t B,
                                      int64_t *accum1, int64_t *accum2, int64_t *accumOut) {
    accum1[0] = accum2[0] = accumOut[0] = 0;
    for (int64_t g = 0; g < B; ++g) {
        accum1[g + 1] = accum1[g] + M[g] * K[g];
        accum2[g + 1] = accum2[g] + N[g] * K[g];
        accumOut[g + 1] = accumOut[g] + M[g] * N[g];
    }
}

/*
 * Softmax prefix sum from rows/cols.
 * csrc/sparseBlockedAttention.cpp:85-91: accum = cumsum([0, rows*cols]).
 */
ORACLE_API void oracle_softmax_accum(const int64_t *rows, const int64_t *cols, int64_t B, int64_t *accum) {
    accum[0] = 0;
    for (int64_t g = 0; g < B; ++g) accum[g + 1] = accum[g] + rows[g] * cols[g];
}

static int64_t isqrt_i64(int64_t v) {
    if (v <= 0) return 0;
    int64_t r = (int64_t)sqrt((double)v);
    while (r * r > v) --r;
    while ((r + 1) * (r + 1) <= v) ++r;
    return r;
}

/*
 * Prefix sums -> lists.
 * csrc/sparseBlockedAttention.cpp:30-40: mk, nk, mn are adjacent differences;
 * M = sqrt(mk*mn/nk), N = mn/M, K = mk/M.  The reference evaluates this in
 * float32 and truncates; here it is exact integer arithmetic (the float route
 * can be off by one for large sizes, and the result must equal the lists that
 * generated the sums).  A segment whose three areas are all zero yields
 * (0,0,0); one with a single non-zero area has one empty dimension (the
 * reference divides 0 by 0 there).  Returns the number of segments whose areas are not consistent with
 * any integer (M,N,K) (their lists are set to -1).
 */
ORACLE_API int64_t oracle_accum_to_lists(const int64_t *accum1, const int64_t *accum2, const int64_t *accumOut,
                                         int64_t B, int64_t *M, int64_t *N, int64_t *K) {
    int64_t bad = 0;
    for (int64_t g = 0; g < B; ++g) {
        int64_t mk = accum1[g + 1] - accum1[g];
        int64_t nk = accum2[g + 1] - accum2[g];
        int64_t mn = accumOut[g + 1] - accumOut[g];
        if (mk == 0 && nk == 0 && mn == 0) { M[g] = N[g] = K[g] = 0; continue; }
        /* One empty dimension leaves exactly one area: the sums fix only the product of the other two
         * dimensions, and no result depends on how it splits (nothing is computed, or zeros fill M*N
         * elements).  Convention: the whole product goes to the first of the two, the other is 1. */
        if (mk == 0 && mn == 0 && nk > 0) { M[g] = 0; N[g] = nk; K[g] = 1; continue; }
        if (nk == 0 && mn == 0 && mk > 0) { M[g] = mk; N[g] = 0; K[g] = 1; continue; }
        if (mk == 0 && nk == 0 && mn > 0) { M[g] = mn; N[g] = 1; K[g] = 0; continue; }
        int ok = mk > 0 && nk > 0 && mn > 0;
        int64_t m = 0, n = 0, k = 0;
        if (ok) {
            /* M^2 = mk*mn/nk.  128-bit product: areas can exceed 2^32. */
            __int128 num = (__int128)mk * (__int128)mn;
            ok = (num % nk) == 0 && (num / nk) <= (__int128)INT64_MAX;
            if (ok) {
                int64_t m2 = (int64_t)(num / nk);
                m = isqrt_i64(m2);
                ok = m > 0 && m * m == m2 && mn % m == 0 && mk % m == 0;
                if (ok) { n = mn / m; k = mk / m; ok = n * k == nk; }
            }
        }
        if (!ok) { M[g] = N[g] = K[g] = -1; ++bad; } else { M[g] = m; N[g] = n; K[g] = k; }
    }
    return bad;
}

/* --------------------------------------------------------------- work-lists */

static int lower_bound3(const int *v, int x) { int i = 0; while (i < 3 && v[i] < x) ++i; return i; }
static int upper_bound3(const int *v, int x) { int i = 0; while (i < 3 && v[i] <= x) ++i; return i; }

/*
 * The reference's global tile choice.
 * csrc/cuda/spBlkGEMM.cu:947-967 with the tile menus of spBlkGEMM.cuh:10-12:
 * one (BM,BN,BK) for the whole batch from trunc(mean) and max of M and N.
 * half_like selects the "+1 BK" adjustment for fp16/bf16 (:963-967).
 * The float32 mean mirrors MList.mean(torch::kFloat).
 */
ORACLE_API void oracle_ref_tile_choice(const int64_t *M, const int64_t *N, int64_t B, int half_like,
                                       int *bm, int *bn, int *bk) {
    static const int BML[3] = {32, 64, 128}, BNL[3] = {32, 64, 128}, BKL[3] = {8, 16, 32};
    double sm = 0, sn = 0;
    int64_t maxM = 0, maxN = 0;
    for (int64_t g = 0; g < B; ++g) {
        sm += (double)M[g]; sn += (double)N[g];
        if (M[g] > maxM) maxM = M[g];
        if (N[g] > maxN) maxN = N[g];
    }
    int avgM = (int)(float)(sm / (double)B), avgN = (int)(float)(sn / (double)B);
    int mi = avgM == (int)maxM ? lower_bound3(BML, avgM) : upper_bound3(BML, avgM);
    if (mi == 3) mi = 2;
    if (mi > 0 && BML[mi] > maxM && avgM != (int)maxM) mi -= 1;
    int ni = avgN == (int)maxN ? lower_bound3(BNL, avgN) : upper_bound3(BNL, avgN);
    if (ni == 3) ni = 2;
    if (ni > 0 && BNL[ni] > maxN && avgN != (int)maxN) ni -= 1;
    int ki = 3 - (mi < ni ? mi : ni) - 1;
    if (half_like && ki < 2) ki += 1;
    *bm = BML[mi]; *bn = BNL[ni]; *bk = BKL[ki];
}

/*
 * GEMM tile work-list: (segment, tile) pairs, segment-major, tile t of a
 * segment covering rows (t / NTile)*BM.. and columns (t % NTile)*BN..
 * csrc/cuda/spBlkGEMM.cu:972-982 (list), :146-150 (tile -> origin).
 * If list is NULL only the count is returned.
 */
ORACLE_API int64_t oracle_gemm_worklist(const int64_t *M, const int64_t *N, int64_t B, int bm, int bn,
                                        int64_t *list) {
    int64_t n = 0;
    for (int64_t g = 0; g < B; ++g) {
        int64_t tiles = ((M[g] + bm - 1) / bm) * ((N[g] + bn - 1) / bn);
        for (int64_t t = 0; t < tiles; ++t) {
            if (list) { list[2 * n] = g; list[2 * n + 1] = t; }
            ++n;
        }
    }
    return n;
}

/*
 * Softmax row work-list: one (segment, row) pair per row, segment-major.
 * csrc/cuda/spBlkSoftmax.cu:358-373.
 */
ORACLE_API int64_t oracle_softmax_worklist(const int64_t *rows, int64_t B, int64_t *list) {
    int64_t n = 0;
    for (int64_t g = 0; g < B; ++g)
        for (int64_t r = 0; r < rows[g]; ++r) {
            if (list) { list[2 * n] = g; list[2 * n + 1] = r; }
            ++n;
        }
    return n;
}

/* --------------------------------------------------------------------- GEMM */

/*
 * out[h, accumOut[g] + r*N + c] = sum_t A(h,g,r,t) * B(h,g,c,t), float accumulate,
 * csrc/cuda/spBlkGEMM.cu:133-150 (segment origins: h*D + accum[g]) and
 * :985-1008 (H = numel/Dm1, out is [H, Dout]).
 * Operand addressing, csrc/cuda/spBlkGEMM.cu:292-329 and :363-400:
 *   transpose1 == 0: A element (r,t) at accum1[g] + r*K + t   (segment stored M x K)
 *   transpose1 != 0: at accum1[g] + t*M + r                    (segment stored K x M)
 *   transpose2 == 0: B element (c,t) at accum2[g] + c*K + t   (segment stored N x K)
 *   transpose2 != 0: at accum2[g] + t*N + c                    (segment stored K x N)
 * Accumulation runs t = 0..K-1 in order in float, the accumulator type of the
 * reference's fp32 kernel (:159); K == 0 yields zeros (:200-207).
 */
ORACLE_API void oracle_varlen_gemm_f32(const float *A, const float *Bm, float *out, int64_t H,
                                       int64_t Dm1, int64_t Dm2, int64_t Dout, int64_t nseg,
                                       const int64_t *accum1, const int64_t *accum2, const int64_t *accumOut,
                                       const int64_t *M, const int64_t *N, const int64_t *K,
                                       int transpose1, int transpose2) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const float *a = A + h * Dm1 + accum1[g];
            const float *b = Bm + h * Dm2 + accum2[g];
            float *o = out + h * Dout + accumOut[g];
            const int64_t m = M[g], n = N[g], k = K[g];
            for (int64_t r = 0; r < m; ++r)
                for (int64_t c = 0; c < n; ++c) {
                    float acc = 0.0f;
                    for (int64_t t = 0; t < k; ++t) {
                        float av = transpose1 ? a[t * m + r] : a[r * k + t];
                        float bv = transpose2 ? b[t * n + c] : b[c * k + t];
                        acc += av * bv;
                    }
                    o[r * n + c] = acc;
                }
        }
}

/* Same result with a double accumulator: the reference value the tolerance
 * statements are made against when float summation order matters. */
ORACLE_API void oracle_varlen_gemm_f64acc(const float *A, const float *Bm, float *out, int64_t H,
                                          int64_t Dm1, int64_t Dm2, int64_t Dout, int64_t nseg,
                                          const int64_t *accum1, const int64_t *accum2, const int64_t *accumOut,
                                          const int64_t *M, const int64_t *N, const int64_t *K,
                                          int transpose1, int transpose2) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const float *a = A + h * Dm1 + accum1[g];
            const float *b = Bm + h * Dm2 + accum2[g];
            float *o = out + h * Dout + accumOut[g];
            const int64_t m = M[g], n = N[g], k = K[g];
            for (int64_t r = 0; r < m; ++r)
                for (int64_t c = 0; c < n; ++c) {
                    double acc = 0.0;
                    for (int64_t t = 0; t < k; ++t) {
                        double av = transpose1 ? a[t * m + r] : a[r * k + t];
                        double bv = transpose2 ? b[t * n + c] : b[c * k + t];
                        acc += av * bv;
                    }
                    o[r * n + c] = (float)acc;
                }
        }
}

/*
 * The same kernel for T = double (csrc/cuda/spBlkGEMM.cu:1010 instantiates it for every element type;
 * :159 accumulates in T).
 */
ORACLE_API void oracle_varlen_gemm_f64(const double *A, const double *Bm, double *out, int64_t H,
                                       int64_t Dm1, int64_t Dm2, int64_t Dout, int64_t nseg,
                                       const int64_t *accum1, const int64_t *accum2, const int64_t *accumOut,
                                       const int64_t *M, const int64_t *N, const int64_t *K,
                                       int transpose1, int transpose2) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const double *a = A + h * Dm1 + accum1[g];
            const double *b = Bm + h * Dm2 + accum2[g];
            double *o = out + h * Dout + accumOut[g];
            const int64_t m = M[g], n = N[g], k = K[g];
            for (int64_t r = 0; r < m; ++r)
                for (int64_t c = 0; c < n; ++c) {
                    double acc = 0.0;
                    for (int64_t t = 0; t < k; ++t) {
                        double av = transpose1 ? a[t * m + r] : a[r * k + t];
                        double bv = transpose2 ? b[t * n + c] : b[c * k + t];
                        acc += av * bv;
                    }
                    o[r * n + c] = acc;
                }
        }
}

/*
 * ... and for the integer element types (uint8, int8, int16, int32, int64).  The accumulator has the
 * element type (:159), so every partial sum is reduced modulo 2^bits; since that reduction commutes with
 * sums and products, the result is the exact sum of products reduced once at the end.  Operands and
 * results travel as int64 holding values of the element type; bits in {8, 16, 32, 64}, is_signed says
 * how the low bits of the result are read.
 */
ORACLE_API void oracle_varlen_gemm_i64(const int64_t *A, const int64_t *Bm, int64_t *out, int64_t H,
                                       int64_t Dm1, int64_t Dm2, int64_t Dout, int64_t nseg,
                                       const int64_t *accum1, const int64_t *accum2, const int64_t *accumOut,
                                       const int64_t *M, const int64_t *N, const int64_t *K,
                                       int transpose1, int transpose2, int bits, int is_signed) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const int64_t *a = A + h * Dm1 + accum1[g];
            const int64_t *b = Bm + h * Dm2 + accum2[g];
            int64_t *o = out + h * Dout + accumOut[g];
            const int64_t m = M[g], n = N[g], k = K[g];
            for (int64_t r = 0; r < m; ++r)
                for (int64_t c = 0; c < n; ++c) {
                    uint64_t acc = 0;                     /* wraps modulo 2^64, a multiple of 2^bits */
                    for (int64_t t = 0; t < k; ++t) {
                        uint64_t av = (uint64_t)(transpose1 ? a[t * m + r] : a[r * k + t]);
                        uint64_t bv = (uint64_t)(transpose2 ? b[t * n + c] : b[c * k + t]);
                        acc += av * bv;
                    }
                    if (bits < 64) {
                        acc &= (((uint64_t)1) << bits) - 1;
                        if (is_signed && (acc >> (bits - 1))) acc |= ~((((uint64_t)1) << bits) - 1);
                    }
                    o[r * n + c] = (int64_t)acc;
                }
        }
}

/* ------------------------------------------------------------------ softmax */

/*
 * Row (h,g,r) starts at h*Dsrc + accum[g] + r*cols[g] and has cols[g] entries
 * (csrc/cuda/spBlkSoftmax.cu:95-107); y = exp(x - max x) / sum exp(x - max x)
 * (:109-136).  The reference has no scale; scale multiplies x first and 1.0
 * reproduces the reference.  A row of all -inf gives NaN like torch.softmax.
 * Evaluated in double and rounded to float once.
 */
ORACLE_API void oracle_blocked_softmax_f32(const float *src, float *out, int64_t H, int64_t Dsrc, int64_t nseg,
                                           const int64_t *accum, const int64_t *rows, const int64_t *cols,
                                           float scale) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const int64_t nc = cols[g];
            for (int64_t r = 0; r < rows[g]; ++r) {
                const float *x = src + h * Dsrc + accum[g] + r * nc;
                float *y = out + h * Dsrc + accum[g] + r * nc;
                double mx = -INFINITY;
                for (int64_t c = 0; c < nc; ++c) {
                    double v = (double)x[c] * (double)scale;
                    if (v > mx) mx = v;
                }
                double sum = 0.0;
                for (int64_t c = 0; c < nc; ++c) sum += exp((double)x[c] * (double)scale - mx);
                for (int64_t c = 0; c < nc; ++c)
                    y[c] = (float)(exp((double)x[c] * (double)scale - mx) / sum);
            }
        }
}

/*
 * The same for T = double (csrc/cuda/spBlkSoftmax.cu:400 instantiates the kernels for double as well),
 * evaluated in long double and rounded to double once; and its backward.
 */
ORACLE_API void oracle_blocked_softmax_f64(const double *src, double *out, int64_t H, int64_t Dsrc, int64_t nseg,
                                           const int64_t *accum, const int64_t *rows, const int64_t *cols,
                                           double scale) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const int64_t nc = cols[g];
            for (int64_t r = 0; r < rows[g]; ++r) {
                const double *x = src + h * Dsrc + accum[g] + r * nc;
                double *y = out + h * Dsrc + accum[g] + r * nc;
                long double mx = -INFINITY;
                for (int64_t c = 0; c < nc; ++c) {
                    long double v = (long double)x[c] * (long double)scale;
                    if (v > mx) mx = v;
                }
                long double sum = 0.0L;
                for (int64_t c = 0; c < nc; ++c) sum += expl((long double)x[c] * (long double)scale - mx);
                for (int64_t c = 0; c < nc; ++c)
                    y[c] = (double)(expl((long double)x[c] * (long double)scale - mx) / sum);
            }
        }
}

ORACLE_API void oracle_blocked_softmax_backward_f64(const double *y, const double *dy, double *dx, int64_t H,
                                                    int64_t Dsrc, int64_t nseg, const int64_t *accum,
                                                    const int64_t *rows, const int64_t *cols, double scale) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const int64_t nc = cols[g];
            for (int64_t r = 0; r < rows[g]; ++r) {
                const int64_t base = h * Dsrc + accum[g] + r * nc;
                long double dot = 0.0L;
                for (int64_t c = 0; c < nc; ++c) dot += (long double)y[base + c] * (long double)dy[base + c];
                for (int64_t c = 0; c < nc; ++c)
                    dx[base + c] = (double)((long double)scale * ((long double)dy[base + c] - dot) * (long double)y[base + c]);
            }
        }
}

/*
 * Softmax backward: dx = scale * (dy - sum_c(y*dy)) * y per row, y the forward
 * output (csrc/cuda/spBlkSoftmax.cu:140-180; the reference has scale = 1).
 * Evaluated in double and rounded to float once.
 */
ORACLE_API void oracle_blocked_softmax_backward_f32(const float *y, const float *dy, float *dx, int64_t H,
                                                    int64_t Dsrc, int64_t nseg, const int64_t *accum,
                                                    const int64_t *rows, const int64_t *cols, float scale) {
    for (int64_t h = 0; h < H; ++h)
        for (int64_t g = 0; g < nseg; ++g) {
            const int64_t nc = cols[g];
            for (int64_t r = 0; r < rows[g]; ++r) {
                const int64_t e0 = h * Dsrc + accum[g] + r * nc;
                double dot = 0.0;
                for (int64_t c = 0; c < nc; ++c) dot += (double)y[e0 + c] * (double)dy[e0 + c];
                for (int64_t c = 0; c < nc; ++c)
                    dx[e0 + c] = (float)((double)scale * ((double)dy[e0 + c] - dot) * (double)y[e0 + c]);
            }
        }
}

/*
 * The pair the benchmark names: softmax(scale * A_g B_g^T) per segment, the
 * scores kept in float between the two steps (no 16-bit rounding), i.e.
 * oracle_varlen_gemm_f32 followed by oracle_blocked_softmax_f32 with
 * rows = M, cols = N, accum = accumOut.  scores may be NULL; if given it
 * receives the unscaled scores.
 */
ORACLE_API int oracle_gemm_softmax_f32(const float *A, const float *Bm, float *probs, float *scores, int64_t H,
                                       int64_t Dm1, int64_t Dm2, int64_t Dout, int64_t nseg,
                                       const int64_t *accum1, const int64_t *accum2, const int64_t *accumOut,
                                       const int64_t *M, const int64_t *N, const int64_t *K, float scale) {
    float *s = scores ? scores : (float *)malloc((size_t)(H * Dout) * sizeof(float));
    if (!s) return 1;
    oracle_varlen_gemm_f32(A, Bm, s, H, Dm1, Dm2, Dout, nseg, accum1, accum2, accumOut, M, N, K, 0, 0);
    oracle_blocked_softmax_f32(s, probs, H, Dout, nseg, accumOut, M, N, scale);
    if (!scores) free(s);
    return 0;
}
