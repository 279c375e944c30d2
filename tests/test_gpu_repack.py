"""ba_repack_operand: operands copied / transposed into zero-padded 16-byte rows, and the GEMMs of the
backward pass run through the fast path on the repacked operands."""
import numpy as np
import pytest
import torch

from blockedattention_amd import capi
from _util import assert_scores_close, make_plan

pytestmark = pytest.mark.gpu


def ceil8(x):
    return (np.asarray(x, np.int64) + 7) // 8 * 8


def segments(t, sizes):
    """Split [H, sum(r*c)] into per-segment [H, r, c] views."""
    out, o = [], 0
    for r, c in sizes:
        out.append(t[:, o:o + r * c].reshape(t.shape[0], r, c)); o += r * c
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_repack_pads_and_transposes(dev, dtype):
    M = np.array([5, 64, 130, 1, 33, 70]); N = np.array([7, 64, 65, 9, 200, 3]); K = np.array([16, 24, 8, 40, 64, 8])
    H = 3
    g = torch.Generator().manual_seed(1)
    S = torch.randn((H, int((M * N).sum())), generator=g).to(dtype)          # an M x N operand (scores / gradient)
    B = torch.randn((H, int((N * K).sum())), generator=g).to(dtype)
    fwd = make_plan(dev, M, N, K)
    N8 = ceil8(N)
    bwd = make_plan(dev, M, K, N8)                                           # dA = dS B: rows M, columns K, reduce over N
    X = torch.full((H, int((M * N8).sum())), float("nan"), dtype=dtype, device=dev)
    Y = torch.full((H, int((K * N8).sum())), float("nan"), dtype=dtype, device=dev)
    capi.repack_operand(fwd, 2, bwd, 0, S.to(dev), X, H, S.shape[1], X.shape[1])
    capi.repack_operand(fwd, 1, bwd, 1, B.to(dev), Y, H, B.shape[1], Y.shape[1], swap_dims=True, column_major=True)
    for got, ref, n, n8 in zip(segments(X.cpu(), zip(M, N8)), segments(S, zip(M, N)), N, N8):
        assert torch.equal(got[:, :, :n], ref) and (got[:, :, n:] == 0).all()
    for got, ref, n, n8 in zip(segments(Y.cpu(), zip(K, N8)), segments(B, zip(N, K)), N, N8):
        assert torch.equal(got[:, :, :n], ref.transpose(1, 2)) and (got[:, :, n:] == 0).all()
    # the product of the repacked operands is dS B, segment by segment, on the MFMA path
    assert bwd.info.slow_items == 0
    dA = torch.full((H, int((M * K).sum())), float("nan"), dtype=dtype, device=dev)
    capi.varlen_gemm(bwd, X, Y, dA, H, X.shape[1], Y.shape[1], dA.shape[1])
    ref = torch.cat([(s.float() @ b.float()).reshape(H, -1) for s, b in zip(segments(S, zip(M, N)), segments(B, zip(N, K)))], 1)
    assert_scores_close(dA, ref, "dA")
    assert fwd.read().run_errors == 0 and bwd.read().run_errors == 0


def test_repack_column_major_source_without_swap(dev):
    # a forward operand stored K x M (the reference's transpose1): the M x K operand, column-major
    M = np.array([9, 100, 64]); N = np.array([4, 4, 4]); K = np.array([12, 70, 64])
    H, dtype = 2, torch.float16
    g = torch.Generator().manual_seed(2)
    At = torch.randn((H, int((M * K).sum())), generator=g).to(dtype)         # segments stored K x M
    fwd = make_plan(dev, M, N, K)
    K8 = ceil8(K)
    dst = make_plan(dev, M, N, K8)
    X = torch.full((H, int((M * K8).sum())), float("nan"), dtype=dtype, device=dev)
    capi.repack_operand(fwd, 0, dst, 0, At.to(dev), X, H, At.shape[1], X.shape[1], column_major=True)
    for got, ref, k in zip(segments(X.cpu(), zip(M, K8)), segments(At, zip(K, M)), K):
        assert torch.equal(got[:, :, :k], ref.transpose(1, 2)) and (got[:, :, k:] == 0).all()
