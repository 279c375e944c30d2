"""The drop-in Python API (blockedAttention.blockGEMM / blockSoftmax) and the
extension ops on the GPU: forward parity, the three metadata forms, autograd."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import workloads
from _util import assert_probs_close, assert_scores_close, random_operands

pytestmark = pytest.mark.gpu


def dl(x, dev):
    return torch.as_tensor(np.asarray(x, np.int64)).to(dev)


def test_reference_script_flow(dev):
    # test/pytest.py:36-46 and :54-59 with the reference's own shapes.
    import blockedAttention
    h, m, n, k = 128, 33, 99, 64
    g = torch.Generator().manual_seed(0)
    A = torch.randn((h, m * k + n * k + k * k), generator=g); B = torch.randn(A.shape, generator=g)
    ML = dl([m, n, k], dev); KL = dl([k, k, k], dev)
    res = blockedAttention.blockGEMM(A.to(dev), B.to(dev), None, None, None, ML, ML, KL)
    assert res.shape == (h, m * m + n * n + k * k) and res.dtype == torch.float32
    sc = oracle.per_segment_torch(A, B, [m, n, k], [m, n, k], [k] * 3, want="scores")
    torch.testing.assert_close(res.cpu(), sc, rtol=1e-4, atol=1e-4)
    sm = blockedAttention.blockSoftmax(res, ML, ML)
    torch.testing.assert_close(sm.cpu(), oracle.per_segment_torch_softmax(res.cpu(), [m, n, k], [m, n, k]),
                               rtol=1e-5, atol=1e-7)
    raw = blockedAttention.blockSoftmax(A.to(dev), ML, KL)
    chk = torch.cat([A[:, :m * k].reshape(h, m, k).softmax(-1).reshape(h, -1),
                     A[:, m * k:(m * k + n * k)].reshape(h, n, k).softmax(-1).reshape(h, -1),
                     A[:, (m * k + n * k):].reshape(h, k, k).softmax(-1).reshape(h, -1)], -1)
    assert (raw.cpu() - chk).abs().mean().item() < 1e-8


@pytest.mark.parametrize("cfg", [1, 2])
def test_three_metadata_forms_agree(dev, cfg):
    import blockedAttention
    w = workloads.make(cfg)
    A, B = w.operands()
    Ad, Bd = A.to(dev), B.to(dev)
    ML, NL, KL = dl(w.M, dev), dl(w.N, dev), dl(w.K, dev)
    a1, a2, ao = [dl(a, dev) for a in oracle.lists_to_accum(w.M, w.N, w.K)]
    r_lists = blockedAttention.blockGEMM(Ad, Bd, MList=ML, NList=NL, KList=KL)
    r_accum = blockedAttention.blockGEMM(Ad, Bd, a1, a2, ao)
    r_both = blockedAttention.blockGEMM(Ad, Bd, a1, a2, ao, ML, NL, KL)
    assert torch.equal(r_lists, r_accum) and torch.equal(r_lists, r_both)
    assert_scores_close(r_lists, oracle.per_segment_torch(A, B, w.M, w.N, w.K, want="scores"))
    p1 = blockedAttention.blockSoftmax(r_lists, ML, NL, scale=w.scale)
    p2 = blockedAttention.blockSoftmax(r_lists, ML, NL, ao, scale=w.scale)
    assert torch.equal(p1, p2)
    fused = blockedAttention.blockGEMMSoftmax(Ad, Bd, MList=ML, NList=NL, KList=KL, scale=w.scale)
    assert_probs_close(fused, oracle.per_segment_torch(A, B, w.M, w.N, w.K, w.scale))
    f32 = blockedAttention.blockGEMMSoftmax(Ad, Bd, a1, a2, ao, scale=w.scale, out_fp32=True)
    assert f32.dtype == torch.float32
    assert (f32.cpu() - oracle.per_segment_torch(A, B, w.M, w.N, w.K, w.scale)).abs().max().item() < 2e-5


def test_leading_dims_are_flattened_and_result_is_2d(dev):
    import blockedAttention
    M, N, K = [5, 20], [7, 3], [8, 16]
    A, B = random_operands(M, N, K, 6, torch.float16)
    ML, NL, KL = dl(M, dev), dl(N, dev), dl(K, dev)
    out = blockedAttention.blockGEMM(A.reshape(2, 3, -1).to(dev), B.reshape(2, 3, -1).to(dev), MList=ML, NList=NL, KList=KL)
    assert out.shape == (6, 95)
    assert_scores_close(out, oracle.per_segment_torch(A, B, M, N, K, want="scores"))


def test_errors_are_runtime_errors(dev):
    import blockedAttention
    M, N, K = dl([4], dev), dl([4], dev), dl([8], dev)
    A = torch.zeros((1, 32), dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError, match="same dtype"):
        blockedAttention.blockGEMM(A, A.float(), MList=M, NList=N, KList=K)
    with pytest.raises(RuntimeError, match="int64"):
        blockedAttention.blockGEMM(A, A, MList=M.int(), NList=N, KList=K)
    with pytest.raises(RuntimeError, match="contiguous"):
        blockedAttention.blockGEMM(torch.zeros((32, 2), dtype=torch.float16, device=dev).t()[:1], A, MList=M, NList=N, KList=K)
    with pytest.raises(RuntimeError, match="segments need"):
        blockedAttention.blockGEMM(A[:, :24], A, MList=M, NList=N, KList=K)
    with pytest.raises(RuntimeError, match="either"):
        blockedAttention.blockGEMM(A, A)
    with pytest.raises(RuntimeError, match="rejected"):
        blockedAttention.blockGEMM(A, A, MList=dl([-4], dev), NList=N, KList=K)
    with pytest.raises(RuntimeError, match="not supported"):
        blockedAttention.blockGEMM(A.to(torch.complex64), A.to(torch.complex64), MList=M, NList=N, KList=K)
    empty = blockedAttention.blockGEMM(A[:, :0], A[:, :0], MList=dl([], dev), NList=dl([], dev), KList=dl([], dev))
    assert empty.shape == (1, 0)


def test_autograd_matches_per_segment_torch(dev):
    import blockedAttention
    M, N, K = [5, 33, 16], [7, 20, 64], [8, 16, 24]
    g = torch.Generator().manual_seed(3)
    A0 = torch.randn((2, 5 * 8 + 33 * 16 + 16 * 24), generator=g); B0 = torch.randn((2, 7 * 8 + 20 * 16 + 64 * 24), generator=g)
    ML, NL, KL = dl(M, dev), dl(N, dev), dl(K, dev)
    A = A0.to(dev).requires_grad_(); B = B0.to(dev).requires_grad_()
    probs = blockedAttention.blockSoftmax(blockedAttention.blockGEMM(A, B, MList=ML, NList=NL, KList=KL), ML, NL, scale=0.25)
    wgt = torch.randn(probs.shape, generator=g)
    (probs * wgt.to(dev)).sum().backward()
    Ar = A0.clone().requires_grad_(); Br = B0.clone().requires_grad_()
    parts = []
    o1 = o2 = 0
    for m, n, k in zip(M, N, K):
        a = Ar[:, o1:o1 + m * k].reshape(2, m, k); b = Br[:, o2:o2 + n * k].reshape(2, n, k)
        parts.append(torch.softmax(a @ b.transpose(1, 2) * 0.25, -1).reshape(2, -1))
        o1 += m * k; o2 += n * k
    ref = torch.cat(parts, -1)
    (ref * wgt).sum().backward()
    torch.testing.assert_close(probs.detach().cpu(), ref.detach(), rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(A.grad.cpu(), Ar.grad, rtol=1e-3, atol=1e-5)
    torch.testing.assert_close(B.grad.cpu(), Br.grad, rtol=1e-3, atol=1e-5)


def test_repeated_metadata_reuses_the_schedule(dev):
    import blockedAttention
    blockedAttention.set_schedule_cache(8)
    M = [33, 7, 120, 64]; K = [64] * 4
    A, B = random_operands(M, M, K, 2, torch.float16, seed=2)
    Ad, Bd = A.to(dev), B.to(dev)
    ML, KL = dl(M, dev), dl(K, dev)
    ref = oracle.per_segment_torch(A, B, M, M, K, 0.125, want="probs")
    before = blockedAttention.schedule_cache_stats()
    for _ in range(3):                                   # e.g. one call per layer with the batch's metadata
        assert_probs_close(blockedAttention.blockGEMMSoftmax(Ad, Bd, MList=ML, NList=ML, KList=KL, scale=0.125), ref, "cached")
    after = blockedAttention.schedule_cache_stats()
    assert after["misses"] - before["misses"] == 1 and after["hits"] - before["hits"] == 2
    # an in-place change of a metadata tensor is seen through its version counter: new schedule, new result
    M2 = [33, 7, 120, 32]
    ML[3] = 32
    A2, B2 = random_operands(M2, M2, K, 2, torch.float16, seed=3)
    out = blockedAttention.blockGEMMSoftmax(A2.to(dev), B2.to(dev), MList=ML, NList=ML, KList=KL, scale=0.125)
    assert_probs_close(out, oracle.per_segment_torch(A2, B2, M2, M2, K, 0.125, want="probs"), "after the change")
    assert blockedAttention.schedule_cache_stats()["misses"] - after["misses"] == 1
    # GEMM, softmax and the backward share the cache through their own keys
    sc = blockedAttention.blockGEMM(A2.to(dev), B2.to(dev), None, None, None, ML, ML, KL)
    pr = blockedAttention.blockSoftmax(sc, ML, ML)
    pr2 = blockedAttention.blockSoftmax(sc, ML, ML)
    assert torch.equal(pr, pr2)
    blockedAttention.set_schedule_cache(0)
    off = blockedAttention.schedule_cache_stats()
    blockedAttention.blockSoftmax(sc, ML, ML)
    now = blockedAttention.schedule_cache_stats()
    assert (now["hits"], now["misses"], now["entries"]) == (off["hits"], off["misses"], 0)
    blockedAttention.set_schedule_cache(8)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_autograd_16bit_through_the_any_layout_gemms(dev, dtype):
    # dA = dS B (reduction over N) and dB = dS^T A (over M) with N, M that are not multiples of 8
    autograd_16bit(dev, dtype, [5, 33, 16, 130], [7, 20, 64, 257], [8, 16, 24, 64])


def test_autograd_16bit_large_segments_of_every_reduction_length(dev):
    # forward: the row-block kernel (K <= 128), its wide build (K <= 256) and the tile kernel (beyond) in one call;
    # backward: products with 300..400 columns and reductions over them
    autograd_16bit(dev, torch.bfloat16, [300, 130, 40, 280], [400, 300, 257, 310], [256, 136, 64, 264])


def autograd_16bit(dev, dtype, M, N, K):
    import blockedAttention
    g = torch.Generator().manual_seed(4)
    A0 = torch.randn((2, int(np.dot(M, K))), generator=g).to(dtype); B0 = torch.randn((2, int(np.dot(N, K))), generator=g).to(dtype)
    ML, NL, KL = dl(M, dev), dl(N, dev), dl(K, dev)
    A = A0.to(dev).requires_grad_(); B = B0.to(dev).requires_grad_()
    out = blockedAttention.blockGEMM(A, B, MList=ML, NList=NL, KList=KL)
    wgt = torch.randn(out.shape, generator=g).to(dtype)
    for _ in range(2):                                           # the second pass reuses the derived schedules
        A.grad = None; B.grad = None
        out.backward(wgt.to(dev), retain_graph=True)
    o1 = o2 = oo = 0
    for m, n, k in zip(M, N, K):
        a = A0[:, o1:o1 + m * k].reshape(2, m, k).float(); b = B0[:, o2:o2 + n * k].reshape(2, n, k).float()
        ds = wgt[:, oo:oo + m * n].reshape(2, m, n).float()
        assert_scores_close(A.grad[:, o1:o1 + m * k].reshape(2, m, k), ds @ b, f"dA {m}x{n}x{k}")
        assert_scores_close(B.grad[:, o2:o2 + n * k].reshape(2, n, k), ds.transpose(1, 2) @ a, f"dB {m}x{n}x{k}")
        o1 += m * k; o2 += n * k; oo += m * n
    assert A.grad.dtype == dtype and A.grad.shape == A.shape and B.grad.shape == B.shape


def test_transposed_and_unaligned_forward_16bit(dev):
    import blockedAttention
    M, N, K = [9, 100, 64, 3], [17, 40, 64, 300], [12, 70, 64, 20]           # K not multiples of 8
    g = torch.Generator().manual_seed(6)
    a = [torch.randn((2, m, k), generator=g).half() for m, k in zip(M, K)]
    b = [torch.randn((2, n, k), generator=g).half() for n, k in zip(N, K)]
    ref = torch.cat([(x.float() @ y.float().transpose(1, 2)).reshape(2, -1) for x, y in zip(a, b)], 1)
    ML, NL, KL = dl(M, dev), dl(N, dev), dl(K, dev)
    for t1 in (False, True):
        for t2 in (False, True):
            A = torch.cat([(x.transpose(1, 2) if t1 else x).reshape(2, -1) for x in a], 1).contiguous().to(dev)
            B = torch.cat([(y.transpose(1, 2) if t2 else y).reshape(2, -1) for y in b], 1).contiguous().to(dev)
            out = blockedAttention.blockGEMM(A, B, None, None, None, ML, NL, KL, t1, t2)
            assert_scores_close(out, ref, f"transpose1={t1} transpose2={t2}")
