"""Scheduler, GEMM, softmax, fused pair and one-pass attention recorded into a HIP graph: the device-side scheduler lets a replay pick up a
new segmentation (same totals) without the host reading anything back."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi
from _util import assert_probs_close, assert_scores_close, dev_i64, random_operands

pytestmark = pytest.mark.gpu


def test_graph_replays_follow_the_lists_on_the_device(dev):
    rng = np.random.default_rng(3)
    n = rng.integers(8, 200, 40).astype(np.int64)
    n[:4] = [300, 5, 7, 260]                                  # tile-class, pack, and wide-row segments too
    K = np.full(40, 64, np.int64)
    H, dtype, scale = 3, torch.float16, 0.125
    d1, do = int((n * K).sum()), int((n * n).sum())
    Md, Nd, Kd = dev_i64(n, dev), dev_i64(n, dev), dev_i64(K, dev)
    a1 = torch.empty(41, dtype=torch.int64, device=dev); a2 = torch.empty_like(a1); ao = torch.empty_like(a1)
    A = torch.empty((H, d1), dtype=dtype, device=dev); B = torch.empty_like(A)
    scores = torch.empty((H, do), dtype=dtype, device=dev); probs = torch.empty_like(scores)
    fused = torch.empty_like(scores)
    V = torch.empty_like(B); att = torch.empty_like(A)
    plan = capi.Plan(40, dev)

    def record():
        capi.plan_gemm(40, dev, Md, Nd, Kd, a1, a2, ao, mode=capi.META_FROM_LISTS, plan=plan)
        capi.varlen_gemm(plan, A, B, scores, H, d1, d1, do)
        capi.blocked_softmax(plan, scores, probs, H, do, scale)
        capi.gemm_softmax(plan, A, B, fused, H, d1, d1, do, scale)
        capi.varlen_attention(plan, A, B, V, att, H, d1, d1, do, scale)

    record()                                                   # eager once (lazy initialisation outside capture)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        record()
    for replay in range(3):
        order = rng.permutation(40)                            # same totals, new offsets and list membership
        m = n[order]
        Ah, Bh = random_operands(m, m, K, H, dtype, seed=10 + replay)
        Md.copy_(dev_i64(m, dev)); Nd.copy_(Md)
        A.copy_(Ah); B.copy_(Bh)
        Vh = random_operands(m, m, K, H, dtype, seed=30 + replay)[1]
        V.copy_(Vh); att.fill_(float("nan"))
        scores.fill_(float("nan")); probs.fill_(float("nan")); fused.fill_(float("nan"))
        junk = torch.randn(1 << 20, device=dev).sum()          # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        sc, pr = oracle.per_segment_torch(Ah, Bh, m, m, K, scale, want="both")
        assert_scores_close(scores, sc, f"replay {replay} scores")
        assert_probs_close(fused, pr, f"replay {replay} fused")
        assert_probs_close(probs, oracle.per_segment_torch_softmax(scores.cpu(), m, m, scale), f"replay {replay} softmax")
        assert_scores_close(att, oracle.per_segment_torch_attention(Ah, Bh, Vh, m, m, K, scale), f"replay {replay} attention")
        assert torch.equal(ao.cpu(), torch.as_tensor(oracle.lists_to_accum(m, m, K)[2]))
        assert float(junk) == float(junk)
    assert plan.read().run_errors == 0
