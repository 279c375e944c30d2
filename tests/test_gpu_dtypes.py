"""The element types without a matrix-instruction kernel of their own in 16 bits: fp64 and the integer types through
the varlen GEMM (the reference instantiates its generic kernel for them, csrc/cuda/spBlkGEMM.cu:1010), fp64 through
the blocked softmax (csrc/cuda/spBlkSoftmax.cu:400).  Integers are bit-exact against the oracle's integer loops;
fp64 within 1e-12 relative of them (the order of summation differs)."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi
from _util import dev_i64, make_plan

pytestmark = pytest.mark.gpu

INT_TYPES = [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64]
SHAPES = dict(M=[11, 70, 1, 16, 130, 5], N=[13, 3, 40, 64, 65, 200], K=[5, 100, 33, 64, 1, 129])


def _operands(dtype, M, N, K, H, seed):
    rng = np.random.default_rng(seed)
    d1 = int((np.asarray(M) * np.asarray(K)).sum()); d2 = int((np.asarray(N) * np.asarray(K)).sum())
    npdt = np.dtype(str(dtype).replace("torch.", ""))
    if npdt.kind == "f":
        return rng.standard_normal((H, d1)).astype(npdt), rng.standard_normal((H, d2)).astype(npdt)
    info = np.iinfo(npdt)
    return (rng.integers(info.min, info.max, (H, d1), dtype=npdt, endpoint=True),
            rng.integers(info.min, info.max, (H, d2), dtype=npdt, endpoint=True))


def _run_gemm(dev, A, B, M, N, K, t1=False, t2=False):
    plan = make_plan(dev, M, N, K)
    i = plan.info
    At, Bt = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
    out = torch.empty((A.shape[0], i.Dout), dtype=At.dtype, device=dev)
    capi.varlen_gemm(plan, At, Bt, out, A.shape[0], i.Dm1, i.Dm2, i.Dout, t1, t2)
    torch.cuda.synchronize()
    assert plan.read().run_errors == 0
    return out.cpu().numpy()


@pytest.mark.parametrize("dtype", INT_TYPES)
@pytest.mark.parametrize("t1,t2", [(False, False), (True, False), (False, True), (True, True)])
def test_integer_gemm_is_bit_exact(dev, dtype, t1, t2):
    A, B = _operands(dtype, **SHAPES, H=3, seed=1)
    got = _run_gemm(dev, A, B, SHAPES["M"], SHAPES["N"], SHAPES["K"], t1, t2)
    ref = oracle.varlen_gemm_typed(A, B, SHAPES["M"], SHAPES["N"], SHAPES["K"], t1, t2)
    assert got.dtype == ref.dtype and np.array_equal(got, ref)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32, torch.float64])
def test_arange_closed_form(dev, dtype):
    # the reference's own example (csrc/sparseBlockedAttention.cpp:216-241): (M, N, K) = (11, 13, 5), inputs arange
    npdt = np.dtype(str(dtype).replace("torch.", ""))
    A = np.arange(55).astype(npdt)[None]; B = np.arange(65).astype(npdt)[None]
    got = _run_gemm(dev, A, B, [11], [13], [5]).reshape(11, 13)
    exact = np.array([[sum((5 * r + t) * (5 * c + t) for t in range(5)) for c in range(13)] for r in range(11)])
    assert np.array_equal(got, exact.astype(npdt))


@pytest.mark.parametrize("t1,t2", [(False, False), (True, False), (False, True), (True, True)])
def test_f64_gemm(dev, t1, t2):
    A, B = _operands(torch.float64, **SHAPES, H=2, seed=2)
    got = _run_gemm(dev, A, B, SHAPES["M"], SHAPES["N"], SHAPES["K"], t1, t2)
    ref = oracle.varlen_gemm_typed(A, B, SHAPES["M"], SHAPES["N"], SHAPES["K"], t1, t2)
    scale = np.abs(ref).max()
    assert np.abs(got - ref).max() <= 1e-12 * scale       # far below anything fp32 arithmetic could reach


def test_f64_gemm_benchmark_shapes(dev):
    # the smallest benchmark configuration at full size in double
    from blockedattention_amd import workloads
    w = workloads.make(1)
    A, B = _operands(torch.float64, w.M, w.N, w.K, 1, seed=3)
    got = _run_gemm(dev, A, B, w.M, w.N, w.K)
    ref = oracle.varlen_gemm_typed(A, B, w.M, w.N, w.K)
    assert np.abs(got - ref).max() <= 1e-12 * np.abs(ref).max()


def test_f64_softmax_forward_and_backward(dev):
    rng = np.random.default_rng(4)
    rows = np.array([3, 17, 1, 40, 5]); cols = np.array([7, 300, 2, 64, 5000])
    H = 2
    x = rng.standard_normal((H, int((rows * cols).sum()))) * 4
    x[0, :7] = -np.inf                                       # a row without finite entries: NaN, like torch.softmax
    dy = rng.standard_normal(x.shape)
    rd, cd = dev_i64(rows, dev), dev_i64(cols, dev)
    acc = torch.empty(len(rows) + 1, dtype=torch.int64, device=dev)
    plan = capi.plan_softmax(len(rows), dev, rd, cd, acc)
    plan.read()
    xt = torch.from_numpy(x).to(dev); y = torch.empty_like(xt)
    capi.blocked_softmax(plan, xt, y, H, x.shape[1], 0.75)        # the C ABI takes the scale as a float: one that float holds exactly
    ref = oracle.blocked_softmax_f64(x, rows, cols, scale=0.75)
    got = y.cpu().numpy()
    assert np.isnan(got[0, :7]).all() and np.isnan(ref[0, :7]).all()
    np.testing.assert_allclose(got[:, 7:], ref[:, 7:], rtol=1e-12, atol=1e-15)
    yt = torch.from_numpy(np.nan_to_num(ref)).to(dev); dyt = torch.from_numpy(dy).to(dev); dx = torch.empty_like(yt)
    capi.blocked_softmax_backward(plan, yt, dyt, dx, H, x.shape[1], 0.75)        # the C ABI takes the scale as a float: one that float holds exactly
    refb = oracle.blocked_softmax_f64(np.nan_to_num(ref), rows, cols, scale=0.75, dy=dy)
    np.testing.assert_allclose(dx.cpu().numpy(), refb, rtol=1e-11, atol=1e-14)
    assert plan.read().run_errors == 0


def test_torch_ops_take_the_other_dtypes(dev):
    import blockAttention
    Ml, Nl, Kl = [11, 20], [13, 7], [5, 40]
    M = torch.tensor(Ml, device=dev); N = torch.tensor(Nl, device=dev); K = torch.tensor(Kl, device=dev)
    d1 = int((M * K).sum()); d2 = int((N * K).sum())
    a = torch.arange(d1, device=dev, dtype=torch.int32).reshape(1, d1) % 97
    b = torch.arange(d2, device=dev, dtype=torch.int32).reshape(1, d2) % 89
    out = blockAttention.sparseBlockedGEMM(a, b, None, None, None, M, N, K, False, False)
    ref = oracle.varlen_gemm_typed(a.cpu().numpy(), b.cpu().numpy(), Ml, Nl, Kl)
    assert out.dtype == torch.int32 and np.array_equal(out.cpu().numpy(), ref)
    # fp64 with autograd: GEMM then softmax, gradients against per-segment torch in double
    g = torch.Generator(device="cpu").manual_seed(5)
    A = torch.randn(2, d1, generator=g, dtype=torch.float64); B = torch.randn(2, d2, generator=g, dtype=torch.float64)
    dY = torch.randn(2, int((M * N).sum()), generator=g, dtype=torch.float64)
    Ad = A.to(dev).requires_grad_(True); Bd = B.to(dev).requires_grad_(True)
    S = blockAttention.sparseBlockedGEMM(Ad, Bd, None, None, None, M, N, K, False, False)
    P = blockAttention.sparseBlockedSoftmax(S, M, N, None)
    P.backward(dY.to(dev))
    Ar = A.clone().requires_grad_(True); Br = B.clone().requires_grad_(True)
    outs = []; o1 = o2 = 0
    for m, n, k in zip(Ml, Nl, Kl):
        a_ = Ar[:, o1:o1 + m * k].reshape(2, m, k); b_ = Br[:, o2:o2 + n * k].reshape(2, n, k)
        outs.append(torch.softmax(a_ @ b_.transpose(1, 2), dim=-1).reshape(2, m * n))
        o1 += m * k; o2 += n * k
    Pr = torch.cat(outs, dim=1)
    Pr.backward(dY)
    assert P.dtype == torch.float64
    torch.testing.assert_close(P.detach().cpu(), Pr.detach(), rtol=1e-11, atol=1e-13)
    torch.testing.assert_close(Ad.grad.cpu(), Ar.grad, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(Bd.grad.cpu(), Br.grad, rtol=1e-10, atol=1e-12)
