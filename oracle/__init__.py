"""CPU checker for the varlen GEMM + blocked softmax path.

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke`` and
by the benchmark's CPU-baseline leg.  The shipped package never imports it.

Two independent statements of the same results live here:

* ``liboracle.so`` (oracle.c) -- plain C loops, reached through ctypes;
* ``per_segment_torch`` -- one ``torch.matmul`` + ``torch.softmax`` per head and
  segment in fp32, the CPU path the benchmark times beside the GPU.

``attention`` / ``per_segment_torch_attention`` state the one-pass attention
(probabilities times values) the same two ways; tests/test_oracle_values.py pins
them with closed forms (uniform scores give column means, one-hot values return
the probabilities, a dominant key returns its value row) and a brute-force loop.

``varlen_gemm_typed`` / ``blocked_softmax_f64`` restate the same operators for the
other element types of the reference's dispatch (fp64; uint8, int8, int16, int32,
int64 with the accumulator in the element type); tests/test_oracle_values.py pins
them with the arange closed form reduced modulo 2^bits, numpy's wrapping integer
matmul, numpy / scipy in float64 and torch.autograd in float64.

Both follow the semantics of the reference at
csrc/sparseBlockedAttention.cpp:11-50, 81-101, csrc/cuda/spBlkGEMM.cu:133-150,
292-329, 363-400, 985-1008 and csrc/cuda/spBlkSoftmax.cu:95-136, 375-398.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_I64P = ctypes.POINTER(ctypes.c_int64)
_F32P = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile oracle.c into liboracle.so with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_accum_to_lists.restype = ctypes.c_int64
        _lib.oracle_gemm_worklist.restype = ctypes.c_int64
        _lib.oracle_softmax_worklist.restype = ctypes.c_int64
        _lib.oracle_gemm_softmax_f32.restype = ctypes.c_int
    return _lib


def _i64(a):
    a = np.ascontiguousarray(np.asarray(a, dtype=np.int64))
    return a, a.ctypes.data_as(_I64P)


def _f32(a):
    a = np.ascontiguousarray(np.asarray(a, dtype=np.float32))
    return a, a.ctypes.data_as(_F32P)


# ------------------------------------------------------------------ metadata
def lists_to_accum(M, N, K):
    M, pM = _i64(M); N, pN = _i64(N); K, pK = _i64(K)
    B = M.shape[0]
    a1 = np.empty(B + 1, np.int64); a2 = np.empty(B + 1, np.int64); ao = np.empty(B + 1, np.int64)
    lib().oracle_lists_to_accum(pM, pN, pK, ctypes.c_int64(B), a1.ctypes.data_as(_I64P),
                                a2.ctypes.data_as(_I64P), ao.ctypes.data_as(_I64P))
    return a1, a2, ao


def softmax_accum(rows, cols):
    rows, pr = _i64(rows); cols, pc = _i64(cols)
    B = rows.shape[0]
    acc = np.empty(B + 1, np.int64)
    lib().oracle_softmax_accum(pr, pc, ctypes.c_int64(B), acc.ctypes.data_as(_I64P))
    return acc


def accum_to_lists(a1, a2, ao):
    a1, p1 = _i64(a1); a2, p2 = _i64(a2); ao, po = _i64(ao)
    B = a1.shape[0] - 1
    M = np.empty(B, np.int64); N = np.empty(B, np.int64); K = np.empty(B, np.int64)
    bad = lib().oracle_accum_to_lists(p1, p2, po, ctypes.c_int64(B), M.ctypes.data_as(_I64P),
                                      N.ctypes.data_as(_I64P), K.ctypes.data_as(_I64P))
    return M, N, K, int(bad)


def ref_tile_choice(M, N, half_like):
    M, pM = _i64(M); N, pN = _i64(N)
    bm = ctypes.c_int(); bn = ctypes.c_int(); bk = ctypes.c_int()
    lib().oracle_ref_tile_choice(pM, pN, ctypes.c_int64(M.shape[0]), ctypes.c_int(int(half_like)),
                                 ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(bk))
    return bm.value, bn.value, bk.value


def gemm_worklist(M, N, bm, bn):
    M, pM = _i64(M); N, pN = _i64(N)
    B = ctypes.c_int64(M.shape[0])
    n = lib().oracle_gemm_worklist(pM, pN, B, bm, bn, None)
    out = np.empty(2 * n, np.int64)
    lib().oracle_gemm_worklist(pM, pN, B, bm, bn, out.ctypes.data_as(_I64P))
    return out.reshape(n, 2)


def softmax_worklist(rows):
    rows, pr = _i64(rows)
    B = ctypes.c_int64(rows.shape[0])
    n = lib().oracle_softmax_worklist(pr, B, None)
    out = np.empty(2 * n, np.int64)
    lib().oracle_softmax_worklist(pr, B, out.ctypes.data_as(_I64P))
    return out.reshape(n, 2)


# -------------------------------------------------------------------- values
def varlen_gemm(A, Bm, M, N, K, transpose1=False, transpose2=False, f64acc=False):
    """A: [H, Dm1], Bm: [H, Dm2] float arrays -> float32 [H, Dout]."""
    A, pA = _f32(A); Bm, pB = _f32(Bm)
    M, pM = _i64(M); N, pN = _i64(N); K, pK = _i64(K)
    a1, a2, ao = lists_to_accum(M, N, K)
    H = A.shape[0]
    assert A.shape[1] == a1[-1] and Bm.shape[1] == a2[-1] and Bm.shape[0] == H
    out = np.empty((H, int(ao[-1])), np.float32)
    fn = lib().oracle_varlen_gemm_f64acc if f64acc else lib().oracle_varlen_gemm_f32
    c = ctypes.c_int64
    fn(pA, pB, out.ctypes.data_as(_F32P), c(H), c(int(a1[-1])), c(int(a2[-1])), c(int(ao[-1])),
       c(M.shape[0]), a1.ctypes.data_as(_I64P), a2.ctypes.data_as(_I64P), ao.ctypes.data_as(_I64P),
       pM, pN, pK, ctypes.c_int(int(transpose1)), ctypes.c_int(int(transpose2)))
    return out


_INT_BITS = {"uint8": (8, 0), "int8": (8, 1), "int16": (16, 1), "int32": (32, 1), "int64": (64, 1)}


def varlen_gemm_typed(A, Bm, M, N, K, transpose1=False, transpose2=False):
    """The generic kernel for the element type of A: float64 (accumulated in double) or one of the integer
    types (exact modulo 2^bits).  A: [H, Dm1], Bm: [H, Dm2] numpy arrays of one dtype -> [H, Dout], same dtype."""
    A = np.ascontiguousarray(A); Bm = np.ascontiguousarray(Bm)
    assert A.dtype == Bm.dtype
    M, pM = _i64(M); N, pN = _i64(N); K, pK = _i64(K)
    a1, a2, ao = lists_to_accum(M, N, K)
    H = A.shape[0]
    assert A.shape[1] == a1[-1] and Bm.shape[1] == a2[-1] and Bm.shape[0] == H
    c = ctypes.c_int64
    meta = (c(H), c(int(a1[-1])), c(int(a2[-1])), c(int(ao[-1])), c(M.shape[0]), a1.ctypes.data_as(_I64P),
            a2.ctypes.data_as(_I64P), ao.ctypes.data_as(_I64P), pM, pN, pK, ctypes.c_int(int(transpose1)),
            ctypes.c_int(int(transpose2)))
    if A.dtype == np.float64:
        out = np.empty((H, int(ao[-1])), np.float64)
        P = ctypes.POINTER(ctypes.c_double)
        lib().oracle_varlen_gemm_f64(A.ctypes.data_as(P), Bm.ctypes.data_as(P), out.ctypes.data_as(P), *meta)
        return out
    bits, signed = _INT_BITS[A.dtype.name]
    a64 = np.ascontiguousarray(A.astype(np.int64)); b64 = np.ascontiguousarray(Bm.astype(np.int64))
    out = np.empty((H, int(ao[-1])), np.int64)
    lib().oracle_varlen_gemm_i64(a64.ctypes.data_as(_I64P), b64.ctypes.data_as(_I64P), out.ctypes.data_as(_I64P), *meta,
                                 ctypes.c_int(bits), ctypes.c_int(signed))
    return out.astype(A.dtype)          # values already lie in the type's range


def blocked_softmax_f64(src, rows, cols, scale=1.0, dy=None):
    """Row softmax of float64 [H, D] (dy given: its backward, src then being the forward output)."""
    src = np.ascontiguousarray(src, np.float64)
    rows, pR = _i64(rows); cols, pC = _i64(cols)
    accum = softmax_accum(rows, cols)
    H = src.shape[0]
    assert src.shape[1] == accum[-1]
    out = np.empty_like(src)
    P = ctypes.POINTER(ctypes.c_double)
    c = ctypes.c_int64
    if dy is None:
        lib().oracle_blocked_softmax_f64(src.ctypes.data_as(P), out.ctypes.data_as(P), c(H), c(int(accum[-1])),
                                         c(rows.shape[0]), accum.ctypes.data_as(_I64P), pR, pC, ctypes.c_double(scale))
    else:
        dy = np.ascontiguousarray(dy, np.float64)
        lib().oracle_blocked_softmax_backward_f64(src.ctypes.data_as(P), dy.ctypes.data_as(P), out.ctypes.data_as(P), c(H),
                                                  c(int(accum[-1])), c(rows.shape[0]), accum.ctypes.data_as(_I64P), pR, pC,
                                                  ctypes.c_double(scale))
    return out


def blocked_softmax(src, rows, cols, scale=1.0, accum=None):
    src, ps = _f32(src)
    rows, pr = _i64(rows); cols, pc = _i64(cols)
    acc = softmax_accum(rows, cols) if accum is None else np.ascontiguousarray(accum, dtype=np.int64)
    H, D = src.shape
    out = np.empty_like(src) if accum is None else np.zeros_like(src)
    c = ctypes.c_int64
    lib().oracle_blocked_softmax_f32(ps, out.ctypes.data_as(_F32P), c(H), c(D), c(rows.shape[0]),
                                     acc.ctypes.data_as(_I64P), pr, pc, ctypes.c_float(scale))
    return out


def blocked_softmax_backward(y, dy, rows, cols, scale=1.0):
    y, py = _f32(y); dy, pdy = _f32(dy)
    rows, pr = _i64(rows); cols, pc = _i64(cols)
    acc = softmax_accum(rows, cols)
    H, D = y.shape
    dx = np.empty_like(y)
    c = ctypes.c_int64
    lib().oracle_blocked_softmax_backward_f32(py, pdy, dx.ctypes.data_as(_F32P), c(H), c(D), c(rows.shape[0]),
                                              acc.ctypes.data_as(_I64P), pr, pc, ctypes.c_float(scale))
    return dx


def gemm_softmax(A, Bm, M, N, K, scale=1.0, return_scores=False):
    A, pA = _f32(A); Bm, pB = _f32(Bm)
    M, pM = _i64(M); N, pN = _i64(N); K, pK = _i64(K)
    a1, a2, ao = lists_to_accum(M, N, K)
    H = A.shape[0]
    probs = np.empty((H, int(ao[-1])), np.float32)
    scores = np.empty_like(probs) if return_scores else None
    c = ctypes.c_int64
    rc = lib().oracle_gemm_softmax_f32(pA, pB, probs.ctypes.data_as(_F32P),
                                       scores.ctypes.data_as(_F32P) if return_scores else None,
                                       c(H), c(int(a1[-1])), c(int(a2[-1])), c(int(ao[-1])), c(M.shape[0]),
                                       a1.ctypes.data_as(_I64P), a2.ctypes.data_as(_I64P),
                                       ao.ctypes.data_as(_I64P), pM, pN, pK, ctypes.c_float(scale))
    assert rc == 0
    return (probs, scores) if return_scores else probs


def attention(Q, Km, V, M, N, K, scale=1.0):
    """O_g = softmax(scale * Q_g K_g^T) V_g in the C loops: the fused pair above, then the varlen GEMM
    again with the probabilities as the M x N operand (reduction over N) and V_g (N x K, i.e. stored
    "reduction x columns") as the transposed second operand -- the chain a caller of the reference runs
    (README.md:3; csrc/cuda/spBlkGEMM.cu:363-400 for transpose2).  fp32 [H, sum(M*K)]."""
    probs = gemm_softmax(Q, Km, M, N, K, scale)
    return varlen_gemm(probs, V, M, K, N, transpose2=True)


# ---------------------------------------------- per-segment torch (CPU baseline)
def per_segment_torch(A, Bm, M, N, K, scale=1.0, want="probs"):
    """One fp32 torch.matmul (+ torch.softmax) per head and segment on host tensors.

    A: [H, Dm1], Bm: [H, Dm2] torch CPU tensors of any float dtype (upcast to
    fp32).  want: "scores", "probs" or "both".  Returns fp32 [H, Dout] tensors.
    """
    import torch
    A = A.float(); Bm = Bm.float()
    H = A.shape[0]
    M = [int(v) for v in M]; N = [int(v) for v in N]; K = [int(v) for v in K]
    Dout = sum(m * n for m, n in zip(M, N))
    scores = torch.empty((H, Dout), dtype=torch.float32) if want in ("scores", "both") else None
    probs = torch.empty((H, Dout), dtype=torch.float32) if want in ("probs", "both") else None
    o1 = o2 = oo = 0
    for m, n, k in zip(M, N, K):
        a = A[:, o1:o1 + m * k].reshape(H, m, k)
        b = Bm[:, o2:o2 + n * k].reshape(H, n, k)
        s = torch.matmul(a, b.transpose(1, 2))
        if scores is not None:
            scores[:, oo:oo + m * n] = s.reshape(H, m * n)
        if probs is not None:
            probs[:, oo:oo + m * n] = torch.softmax(s * scale, dim=-1).reshape(H, m * n)
        o1 += m * k; o2 += n * k; oo += m * n
    if want == "both":
        return scores, probs
    return scores if want == "scores" else probs


def per_segment_torch_softmax(src, rows, cols, scale=1.0):
    import torch
    src = src.float()
    H = src.shape[0]
    out = torch.empty_like(src)
    o = 0
    for r, c in zip([int(v) for v in rows], [int(v) for v in cols]):
        out[:, o:o + r * c] = torch.softmax(src[:, o:o + r * c].reshape(H, r, c) * scale, -1).reshape(H, r * c)
        o += r * c
    return out


def per_segment_torch_attention(Q, Km, V, M, N, K, scale=1.0):
    """softmax(scale * Q_g K_g^T) V_g with one fp32 torch.matmul / softmax / matmul per segment."""
    import torch
    Q = Q.float(); Km = Km.float(); V = V.float()
    H = Q.shape[0]
    out = torch.zeros_like(Q)
    o1 = o2 = 0
    for m, n, k in zip([int(v) for v in M], [int(v) for v in N], [int(v) for v in K]):
        q = Q[:, o1:o1 + m * k].reshape(H, m, k)
        kk = Km[:, o2:o2 + n * k].reshape(H, n, k)
        vv = V[:, o2:o2 + n * k].reshape(H, n, k)
        if n > 0:
            p = torch.softmax(torch.matmul(q, kk.transpose(1, 2)) * scale, dim=-1)
            out[:, o1:o1 + m * k] = torch.matmul(p, vv).reshape(H, m * k)
        o1 += m * k; o2 += n * k
    return out
