"""Pins the oracle's floating-point side on the CPU against closed forms and libraries.

GEMM: the integer closed form of the reference's arange case (11,13,5)
(a transposed operand, a wrong stride or a dropped k term changes it), identity
operands, dense batched matmul for equal-sized segments, numpy per segment for
both transposed layouts.  Softmax: scipy.special.softmax, rows summing to one,
constant rows, shift invariance, all -inf rows.  Backward: torch.autograd.
The two independent statements (C loops, per-segment torch) must agree.
"""
import numpy as np
import pytest
import scipy.special
import torch

import oracle
from blockedattention_amd import workloads


def test_gemm_integer_closed_form_11_13_5():
    # csrc/sparseBlockedAttention.cpp:216-241: H=1, (M,N,K)=(11,13,5), inputs arange.
    A = np.arange(55, dtype=np.float32)[None]
    B = np.arange(65, dtype=np.float32)[None]
    out = oracle.varlen_gemm(A, B, [11], [13], [5])
    expect = np.array([[sum((5 * r + t) * (5 * c + t) for t in range(5)) for c in range(13)] for r in range(11)])
    assert np.array_equal(out.reshape(11, 13), expect.astype(np.float32))


def test_gemm_identity_operand_reproduces_a():
    rng = np.random.default_rng(0)
    M, K = np.array([7, 3]), np.array([5, 9])
    A = rng.standard_normal((2, int((M * K).sum()))).astype(np.float32)
    eye = np.concatenate([np.eye(5).ravel(), np.eye(9).ravel()]).astype(np.float32)
    out = oracle.varlen_gemm(A, np.stack([eye, eye]), M, K, K)     # N = K, B = I
    assert np.array_equal(out, A)


def test_gemm_equal_segments_match_dense_bmm():
    rng = np.random.default_rng(1)
    H, B, n, K = 3, 6, 10, 16
    A = rng.standard_normal((H, B * n * K)).astype(np.float32)
    Bm = rng.standard_normal((H, B * n * K)).astype(np.float32)
    out = oracle.varlen_gemm(A, Bm, [n] * B, [n] * B, [K] * B, f64acc=True)
    dense = np.einsum("hbik,hbjk->hbij", A.reshape(H, B, n, K).astype(np.float64),
                      Bm.reshape(H, B, n, K).astype(np.float64))
    np.testing.assert_allclose(out, dense.reshape(H, -1).astype(np.float32), rtol=1e-6, atol=1e-6)
    out32 = oracle.varlen_gemm(A, Bm, [n] * B, [n] * B, [K] * B)
    np.testing.assert_allclose(out32, out, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("t1,t2", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm_transposed_layouts_match_numpy(t1, t2):
    rng = np.random.default_rng(2)
    M, N, K = np.array([5, 8, 1]), np.array([4, 3, 6]), np.array([7, 2, 9])
    H = 2
    A = rng.standard_normal((H, int((M * K).sum()))).astype(np.float32)
    Bm = rng.standard_normal((H, int((N * K).sum()))).astype(np.float32)
    out = oracle.varlen_gemm(A, Bm, M, N, K, transpose1=t1, transpose2=t2, f64acc=True)
    o1 = o2 = oo = 0
    for m, n, k in zip(M, N, K):
        a = A[:, o1:o1 + m * k].reshape(H, k, m).transpose(0, 2, 1) if t1 else A[:, o1:o1 + m * k].reshape(H, m, k)
        b = Bm[:, o2:o2 + n * k].reshape(H, k, n).transpose(0, 2, 1) if t2 else Bm[:, o2:o2 + n * k].reshape(H, n, k)
        ref = np.einsum("hik,hjk->hij", a.astype(np.float64), b.astype(np.float64)).reshape(H, -1)
        np.testing.assert_allclose(out[:, oo:oo + m * n], ref, rtol=1e-6, atol=1e-6)
        o1 += m * k; o2 += n * k; oo += m * n


def test_gemm_zero_k_and_empty_segments():
    # segment 0 has K = 0 (2x3 zeros), segment 1 has no rows, segment 2 has no columns
    out = oracle.varlen_gemm(np.ones((1, 21), np.float32), np.ones((1, 20), np.float32), [2, 0, 3], [3, 4, 0], [0, 5, 7])
    assert out.shape == (1, 6) and np.array_equal(out, np.zeros((1, 6), np.float32))


def test_softmax_matches_scipy_and_invariants():
    rng = np.random.default_rng(4)
    rows, cols = np.array([33, 99, 64, 2]), np.array([64, 64, 64, 2047])   # reference check shapes + a long row
    H = 3
    src = (rng.standard_normal((H, int((rows * cols).sum()))) * 3).astype(np.float32)
    for scale in (1.0, 0.125, -0.5):
        out = oracle.blocked_softmax(src, rows, cols, scale)
        o = 0
        for r, c in zip(rows, cols):
            blk = src[:, o:o + r * c].reshape(H, r, c).astype(np.float64) * scale
            np.testing.assert_allclose(out[:, o:o + r * c].reshape(H, r, c), scipy.special.softmax(blk, axis=-1),
                                       rtol=2e-6, atol=1e-9)
            np.testing.assert_allclose(out[:, o:o + r * c].reshape(H, r, c).sum(-1), 1.0, rtol=1e-5)
            o += r * c
    shifted = oracle.blocked_softmax(src + 11.0, rows, cols)
    np.testing.assert_allclose(shifted, oracle.blocked_softmax(src, rows, cols), rtol=1e-4, atol=1e-7)


def test_softmax_constant_and_all_neg_inf_rows():
    out = oracle.blocked_softmax(np.full((1, 12), 3.5, np.float32), [2], [6])
    np.testing.assert_allclose(out, 1.0 / 6.0, rtol=1e-7)
    x = np.array([[-np.inf, -np.inf, 0.0, -np.inf]], np.float32)
    out = oracle.blocked_softmax(x, [2], [2])
    assert np.isnan(out[0, :2]).all() and out[0, 2] == 1.0 and out[0, 3] == 0.0
    ref = torch.softmax(torch.tensor(x).reshape(2, 2), -1).reshape(1, 4).numpy()
    assert np.array_equal(np.isnan(out), np.isnan(ref))


def test_softmax_with_gapped_prefix_sum():
    src = np.arange(12, dtype=np.float32)[None]
    out = oracle.blocked_softmax(src, [1, 1], [3, 4], accum=[0, 5, 12])     # gap of 2 after the first segment
    np.testing.assert_allclose(out[0, 0:3], scipy.special.softmax(src[0, 0:3]), rtol=1e-6)
    np.testing.assert_allclose(out[0, 5:9], scipy.special.softmax(src[0, 5:9]), rtol=1e-6)


def test_softmax_backward_matches_autograd():
    rng = np.random.default_rng(5)
    rows, cols = [4, 7], [9, 3]
    x = torch.tensor(rng.standard_normal((2, 57)), dtype=torch.float64, requires_grad=True)
    dy = rng.standard_normal((2, 57)).astype(np.float32)
    for scale in (1.0, 0.3):
        y = torch.cat([torch.softmax(x[:, :36].reshape(2, 4, 9) * scale, -1).reshape(2, -1),
                       torch.softmax(x[:, 36:].reshape(2, 7, 3) * scale, -1).reshape(2, -1)], -1)
        (gx,) = torch.autograd.grad(y, x, torch.tensor(dy, dtype=torch.float64))
        got = oracle.blocked_softmax_backward(y.detach().numpy().astype(np.float32), dy, rows, cols, scale)
        np.testing.assert_allclose(got, gx.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("cfg", [1, 4])
def test_c_oracle_and_per_segment_torch_agree(cfg):
    w = workloads.make(cfg)
    if cfg == 4:     # first 40 segments keep the C loops short
        w.M, w.N, w.K = w.M[:40], w.N[:40], w.K[:40]
    A, B = w.operands()
    sc_t, pr_t = oracle.per_segment_torch(A, B, w.M, w.N, w.K, w.scale, want="both")
    pr_c, sc_c = oracle.gemm_softmax(A.float().numpy(), B.float().numpy(), w.M, w.N, w.K, w.scale, return_scores=True)
    np.testing.assert_allclose(sc_c, sc_t.numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(pr_c, pr_t.numpy(), rtol=1e-4, atol=1e-6)
    ref = oracle.per_segment_torch_softmax(sc_t, w.M, w.N, w.scale)
    np.testing.assert_allclose(ref.numpy(), pr_t.numpy(), rtol=1e-6, atol=1e-8)


# ------------------------------------------------------------------ attention (probabilities times values)
def _attention_inputs(seed, M, N, K, H=2):
    rng = np.random.default_rng(seed)
    M, N, K = np.asarray(M), np.asarray(N), np.asarray(K)
    Q = rng.standard_normal((H, int((M * K).sum()))).astype(np.float32)
    Km = rng.standard_normal((H, int((N * K).sum()))).astype(np.float32)
    V = rng.standard_normal((H, int((N * K).sum()))).astype(np.float32)
    return Q, Km, V, M, N, K


def test_attention_brute_force_loops():
    # plain Python in float64, index by index: a transposed operand or a wrong offset changes it
    Q, Km, V, M, N, K = _attention_inputs(3, [3, 1, 4], [5, 2, 3], [2, 4, 3])
    scale = 0.7
    got = oracle.attention(Q, Km, V, M, N, K, scale)
    expect = np.zeros_like(got, dtype=np.float64)
    for h in range(Q.shape[0]):
        o1 = o2 = 0
        for m, n, k in zip(M, N, K):
            for r in range(m):
                s = [scale * sum(float(Q[h, o1 + r * k + t]) * float(Km[h, o2 + c * k + t]) for t in range(k)) for c in range(n)]
                e = [np.exp(x - max(s)) for x in s]
                for d in range(k):
                    expect[h, o1 + r * k + d] = sum(e[c] * float(V[h, o2 + c * k + d]) for c in range(n)) / sum(e)
            o1 += m * k; o2 += n * k
    assert np.allclose(got, expect, rtol=1e-5, atol=1e-6)


def test_attention_uniform_scores_give_column_means():
    Q, Km, V, M, N, K = _attention_inputs(4, [4, 2], [6, 9], [8, 3])
    got = oracle.attention(np.zeros_like(Q), Km, V, M, N, K, 1.0)
    o1 = o2 = 0
    for m, n, k in zip(M, N, K):
        mean = V[:, o2:o2 + n * k].reshape(-1, n, k).mean(axis=1)
        assert np.allclose(got[:, o1:o1 + m * k].reshape(-1, m, k), mean[:, None, :], atol=1e-6)
        o1 += m * k; o2 += n * k


def test_attention_one_hot_values_return_the_probabilities():
    # V_g[n][d] = (n == d): O_g = the first K columns of P_g (N <= K pads with zeros)
    Q, Km, V, M, N, K = _attention_inputs(5, [5, 3], [4, 7], [6, 7])
    V = np.zeros_like(V)
    o2 = 0
    for n, k in zip(N, K):
        V[:, o2:o2 + n * k] = np.eye(n, k, dtype=np.float32).ravel()
        o2 += n * k
    got = oracle.attention(Q, Km, V, M, N, K, 0.5)
    probs = oracle.gemm_softmax(Q, Km, M, N, K, 0.5)
    o1 = oo = 0
    for m, n, k in zip(M, N, K):
        P = probs[:, oo:oo + m * n].reshape(-1, m, n)
        want = np.zeros((Q.shape[0], m, k), np.float32)
        want[:, :, :min(n, k)] = P[:, :, :min(n, k)]
        assert np.allclose(got[:, o1:o1 + m * k].reshape(-1, m, k), want, atol=1e-6)
        o1 += m * k; oo += m * n


def test_attention_dominant_key_returns_its_value_row():
    Q, Km, V, M, N, K = _attention_inputs(6, [3], [5], [4], H=1)
    Km[:] = 0.0
    Km[0, 2 * 4:3 * 4] = 100.0 * np.sign(Q[0, :4])          # key 2 dominates query 0
    got = oracle.attention(Q, Km, V, M, N, K, 1.0)
    assert np.allclose(got[0, :4], V[0, 2 * 4:3 * 4], atol=1e-4)


def test_attention_two_statements_agree():
    Q, Km, V, M, N, K = _attention_inputs(7, [9, 0, 17, 5], [12, 4, 0, 33], [8, 16, 5, 24], H=3)
    a = oracle.attention(Q, Km, V, M, N, K, 0.3)
    b = oracle.per_segment_torch_attention(torch.from_numpy(Q), torch.from_numpy(Km), torch.from_numpy(V), M, N, K, 0.3)
    assert np.allclose(a, b.numpy(), rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- the other element types
@pytest.mark.parametrize("dtype", ["int64", "int32", "int16", "int8", "uint8"])
def test_integer_gemm_closed_form_11_13_5(dtype):
    # the reference's arange case again, in the integer types; for the narrow ones the closed form is reduced
    # modulo 2^bits (the accumulator has the element type, csrc/cuda/spBlkGEMM.cu:159)
    A = np.arange(55).astype(dtype)[None]
    B = np.arange(65).astype(dtype)[None]
    out = oracle.varlen_gemm_typed(A, B, [11], [13], [5])
    exact = np.array([[sum((5 * r + t) * (5 * c + t) for t in range(5)) for c in range(13)] for r in range(11)])
    assert out.dtype == np.dtype(dtype)
    assert np.array_equal(out.reshape(11, 13), exact.astype(np.int64).astype(dtype))      # astype wraps
    if dtype in ("int64", "int32"):
        assert np.array_equal(out.reshape(11, 13).astype(np.int64), exact)                # no wrap at these sizes


@pytest.mark.parametrize("dtype", ["int64", "int32", "int16", "int8", "uint8"])
@pytest.mark.parametrize("t1,t2", [(False, False), (True, True)])
def test_integer_gemm_wraps_like_numpy(dtype, t1, t2):
    # numpy's integer matmul keeps the element type and wraps: an independent statement of the same arithmetic
    rng = np.random.default_rng(5)
    info = np.iinfo(dtype)
    M, N, K = np.array([5, 8, 1]), np.array([4, 3, 6]), np.array([70, 2, 90])
    H = 2
    A = rng.integers(info.min, info.max, (H, int((M * K).sum())), dtype=dtype, endpoint=True)
    Bm = rng.integers(info.min, info.max, (H, int((N * K).sum())), dtype=dtype, endpoint=True)
    out = oracle.varlen_gemm_typed(A, Bm, M, N, K, transpose1=t1, transpose2=t2)
    o1 = o2 = oo = 0
    for m, n, k in zip(M, N, K):
        a = A[:, o1:o1 + m * k].reshape(H, k, m).transpose(0, 2, 1) if t1 else A[:, o1:o1 + m * k].reshape(H, m, k)
        b = Bm[:, o2:o2 + n * k].reshape(H, k, n).transpose(0, 2, 1) if t2 else Bm[:, o2:o2 + n * k].reshape(H, n, k)
        with np.errstate(over="ignore"):
            ref = np.matmul(a, b.transpose(0, 2, 1))
        assert ref.dtype == np.dtype(dtype)
        assert np.array_equal(out[:, oo:oo + m * n].reshape(H, m, n), ref)
        o1 += m * k; o2 += n * k; oo += m * n


def test_f64_gemm_matches_numpy_and_the_closed_form():
    A = np.arange(55, dtype=np.float64)[None]; B = np.arange(65, dtype=np.float64)[None]
    exact = np.array([[sum((5 * r + t) * (5 * c + t) for t in range(5)) for c in range(13)] for r in range(11)])
    assert np.array_equal(oracle.varlen_gemm_typed(A, B, [11], [13], [5]).reshape(11, 13), exact.astype(np.float64))
    rng = np.random.default_rng(6)
    M, N, K = np.array([5, 8, 1]), np.array([4, 3, 6]), np.array([70, 2, 90])
    A = rng.standard_normal((2, int((M * K).sum()))); Bm = rng.standard_normal((2, int((N * K).sum())))
    out = oracle.varlen_gemm_typed(A, Bm, M, N, K, transpose2=True)
    o1 = o2 = oo = 0
    for m, n, k in zip(M, N, K):
        a = A[:, o1:o1 + m * k].reshape(2, m, k); b = Bm[:, o2:o2 + n * k].reshape(2, k, n)
        np.testing.assert_allclose(out[:, oo:oo + m * n].reshape(2, m, n), np.matmul(a, b), rtol=1e-13, atol=1e-13)
        o1 += m * k; o2 += n * k; oo += m * n


def test_f64_softmax_matches_scipy_and_autograd():
    rng = np.random.default_rng(7)
    rows, cols = np.array([3, 5, 1]), np.array([7, 300, 2])
    x = rng.standard_normal((2, int((rows * cols).sum()))) * 4
    y = oracle.blocked_softmax_f64(x, rows, cols, scale=0.7)
    dy = rng.standard_normal(x.shape)
    dx = oracle.blocked_softmax_f64(y, rows, cols, scale=0.7, dy=dy)
    o = 0
    for r, c in zip(rows, cols):
        seg = x[:, o:o + r * c].reshape(2, r, c)
        np.testing.assert_allclose(y[:, o:o + r * c].reshape(2, r, c), scipy.special.softmax(0.7 * seg, axis=-1),
                                   rtol=1e-14, atol=1e-16)
        t = torch.tensor(seg, dtype=torch.float64, requires_grad=True)
        torch.softmax(0.7 * t, dim=-1).backward(torch.tensor(dy[:, o:o + r * c].reshape(2, r, c)))
        np.testing.assert_allclose(dx[:, o:o + r * c].reshape(2, r, c), t.grad.numpy(), rtol=1e-12, atol=1e-14)
        o += r * c
