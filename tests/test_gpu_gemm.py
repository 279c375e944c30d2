"""Varlen GEMM through the C ABI against the oracle (scores within rel 1e-2)."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi, workloads
from _util import assert_scores_close, dev_i64, make_plan, random_operands, run_all

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg", [1, 2, 3, 4])
def test_benchmark_configs(dev, cfg):
    w = workloads.make(cfg)
    run_all(dev, w.M, w.N, w.K, w.heads, w.dtype, w.scale, dist=w.dist, sigma=w.sigma)


def test_integer_closed_form_11_13_5(dev):
    # csrc/sparseBlockedAttention.cpp:216-241; values are exact in fp16 products and fp32 sums,
    # results up to 19630 are not all fp16-representable, so compare after the one rounding.
    A = torch.arange(55, dtype=torch.float32).reshape(1, 55)
    B = torch.arange(65, dtype=torch.float32).reshape(1, 65)
    expect = torch.tensor([[sum((5 * r + t) * (5 * c + t) for t in range(5)) for c in range(13)] for r in range(11)],
                          dtype=torch.float32).reshape(1, -1)
    plan = make_plan(dev, [11], [13], [5])
    assert plan.info.slow_items == 1                 # K = 5: element-wise path
    for dtype in (torch.float16, torch.float32):
        out = torch.empty((1, 143), dtype=dtype, device=dev)
        capi.varlen_gemm(plan, A.to(dtype).to(dev), B.to(dtype).to(dev), out, 1, 55, 65, 143)
        assert torch.equal(out.cpu(), expect.to(dtype))


def test_reference_profile_shapes_fp32(dev):
    # test/pytest.py:7-19: H=128, (33,33,64), (99,99,64), (64,64,64), fp32, lists only.
    M = [33, 99, 64]; K = [64] * 3
    A, B = random_operands(M, M, K, 128, torch.float32, seed=1)
    plan = make_plan(dev, M, M, K)
    out = torch.empty((128, plan.info.Dout), dtype=torch.float32, device=dev)
    capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, 128, plan.info.Dm1, plan.info.Dm2, plan.info.Dout)
    ref = oracle.per_segment_torch(A, B, M, M, K, want="scores")
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-4)


def test_odd_k_61_half_from_prefix_sums(dev):
    # csrc/sparseBlockedAttention.cpp:170-192: H=128, (33,33,61) + (127,127,61), half, prefix sums only.
    M = np.array([33, 127]); K = np.array([61, 61]); H = 128
    a1, a2, ao = [torch.as_tensor(a).to(dev) for a in oracle.lists_to_accum(M, M, K)]
    plan = capi.plan_gemm(2, dev, None, None, None, a1, a2, ao, mode=capi.META_FROM_ACCUM)
    info = plan.read()
    assert info.slow_items == 3 + 8 and info.gemm_items == 0
    A, B = random_operands(M, M, K, H, torch.float16, seed=2)
    out = torch.empty((H, info.Dout), dtype=torch.float16, device=dev)
    capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, H, info.Dm1, info.Dm2, info.Dout)
    assert_scores_close(out, oracle.per_segment_torch(A, B, M, M, K, want="scores"), "K=61")
    fused = torch.empty_like(out)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), fused, H, info.Dm1, info.Dm2, info.Dout, 0.125)
    torch.testing.assert_close(fused.float().cpu(), oracle.per_segment_torch(A, B, M, M, K, 0.125), rtol=0, atol=1e-3)


def test_legacy_square_graphs(dev):
    # csrc/sparseBlockedAttention.cpp:147-151: n = {10,5,20,5,60}, d = 32, H = 8.
    n = [10, 5, 20, 5, 60]
    run_all(dev, n, n, [32] * 5, 8, torch.float16, 32 ** -0.5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("t1,t2", [(True, False), (False, True), (True, True)])
def test_transposed_layouts(dev, dtype, t1, t2):
    rng = np.random.default_rng(11)
    M = rng.integers(1, 70, 9); N = rng.integers(1, 300, 9); K = rng.choice([8, 24, 64, 5], 9); H = 3
    A, B = random_operands(M, N, K, H, dtype, seed=3)
    plan = make_plan(dev, M, N, K)
    out = torch.full((H, plan.info.Dout), float("nan"), dtype=dtype, device=dev)
    capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, H, plan.info.Dm1, plan.info.Dm2, plan.info.Dout, t1, t2)
    ref = oracle.varlen_gemm(A.float().numpy(), B.float().numpy(), M, N, K, t1, t2, f64acc=True)
    assert_scores_close(out, torch.from_numpy(ref), f"transpose {t1} {t2}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("t1,t2", [(True, False), (False, True), (True, True)])
def test_transposed_layouts_of_tall_segments(dev, dtype, t1, t2):
    # averages of four and more 64-row blocks per segment: the 128 x 128 build, whose segments with K <= 128 and
    # N >= 128 write whole lines through a ring (odd N: every row at another phase; N at and around the 64-column
    # chunk and 128-column block boundaries; rows that end inside a block); K = 136 and N = 100 take the other path
    M = [300, 257, 512, 129, 640, 384, 1, 260, 200]; N = [128, 129, 191, 193, 255, 257, 300, 1000, 100]
    K = [128, 64, 72, 8, 100, 40, 128, 136, 64]; H = 2
    A, B = random_operands(M, N, K, H, dtype, seed=13)
    plan = make_plan(dev, M, N, K)
    assert plan.info.att_blocks64 >= 4 * len(M)
    ref = torch.from_numpy(oracle.varlen_gemm(A.float().numpy(), B.float().numpy(), M, N, K, t1, t2, f64acc=True))
    i = plan.info
    for shift in (0, 1, 3):                                    # the result's base pointer at several 2-byte phases
        flat = torch.full((H * i.Dout + 8,), float("nan"), dtype=dtype, device=dev)
        out = flat[shift:shift + H * i.Dout].view(H, i.Dout)
        capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, H, i.Dm1, i.Dm2, i.Dout, t1, t2)
        assert_scores_close(out, ref, f"transpose {t1} {t2} shift {shift}")
        assert torch.isnan(flat[:shift]).all() and torch.isnan(flat[shift + H * i.Dout:]).all(), "wrote outside the result"
    # the plan counts the workgroups that went through the ring: 128-row rounds of the seven segments with
    # K <= 128 and N >= 128, per head and call
    ring_rounds = sum(-(-m // 128) for m, n, k in zip(M, N, K) if k <= 128 and n >= 128)
    assert (plan.info.min_N, plan.info.min_K) == (100, 8)
    assert plan.read().ring_groups == 3 * H * ring_rounds
    # without the host summary: the 64 x 64 build, four workgroups per (segment, head), each taking every fourth
    # round as one stream of steps (the loads of a round's first chunks issued during the round before)
    plan.info = None
    out = torch.full((H, i.Dout), float("nan"), dtype=dtype, device=dev)
    capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, H, i.Dm1, i.Dm2, i.Dout, t1, t2)
    assert_scores_close(out, ref, f"transpose {t1} {t2} without the summary")


def test_ragged_edges_and_degenerate_segments(dev):
    # rows/cols not multiples of 16, N across the 256-column chunk boundary, K % 32 in {8,16,24},
    # K = 0 (zeros), M = 0 and N = 0 (no work), odd N (unaligned row starts in the output).
    M = [1, 17, 16, 31, 5, 0, 7, 40, 3]; N = [1, 255, 257, 513, 33, 9, 0, 300, 1031]; K = [8, 16, 24, 40, 0, 8, 8, 72, 96]
    run_all(dev, M, N, K, 2, torch.float16, 0.2, check_softmax=False)
    run_all(dev, M, N, K, 3, torch.bfloat16, 0.2, check_softmax=False)


def test_unaligned_base_pointers_and_odd_head_stride(dev):
    M = np.array([20, 9]); N = np.array([18, 40]); K = np.array([8, 16]); H = 2
    A, B = random_operands(M, N, K, H, torch.float16, seed=5)
    plan = make_plan(dev, M, N, K)
    i = plan.info
    ref = oracle.per_segment_torch(A, B, M, N, K, want="scores")
    big = torch.zeros(H * i.Dm1 + 1, dtype=torch.float16, device=dev)
    big[1:] = A.reshape(-1).to(dev)                            # base pointer 2 bytes off
    out = torch.empty((H, i.Dout), dtype=torch.float16, device=dev)
    capi.varlen_gemm(plan, big[1:], B.to(dev), out, H, i.Dm1, i.Dm2, i.Dout)
    assert_scores_close(out, ref, "unaligned A")
    # an aligned segment followed by K = 4 with odd M: the per-head stride (60) is not a multiple
    # of 8 elements, so heads 1 and 2 start unaligned and no segment may use 16-byte loads
    M2, N2, K2 = [6, 3], [10, 5], [8, 4]
    A2, B2 = random_operands(M2, N2, K2, 3, torch.bfloat16, seed=6)
    plan2 = make_plan(dev, M2, N2, K2)
    assert (plan2.info.Dm1, plan2.info.Dm2, plan2.info.Dout, plan2.info.strip_items) == (60, 100, 75, 1)
    out2 = torch.empty((3, 75), dtype=torch.bfloat16, device=dev)
    capi.varlen_gemm(plan2, A2.to(dev), B2.to(dev), out2, 3, 60, 100, 75)
    assert_scores_close(out2, oracle.per_segment_torch(A2, B2, M2, N2, K2, want="scores"), "odd head stride")


def test_gapped_prefix_sums_given_with_lists(dev):
    M, N, K = [4, 20], [6, 33], [8, 16]
    a1 = [0, 40, 40 + 320]; a2 = [0, 56, 56 + 528]; ao = [0, 30, 30 + 660]      # gaps of 8, 8 and 6 elements
    d = lambda x: torch.as_tensor(np.asarray(x, np.int64)).to(dev)
    plan = capi.plan_gemm(2, dev, d(M), d(N), d(K), d(a1), d(a2), d(ao), mode=capi.META_GIVEN)
    info = plan.read()
    assert (info.Dm1, info.Dm2, info.Dout) == (360, 584, 690)
    g = torch.Generator().manual_seed(0)
    A = torch.randn((2, 360), generator=g).half(); B = torch.randn((2, 584), generator=g).half()
    out = torch.full((2, 690), 9.0, dtype=torch.float16, device=dev)
    capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, 2, 360, 584, 690)
    o = out.float().cpu()
    for m, n, k, o1, o2, oo in zip(M, N, K, a1, a2, ao):
        ref = A[:, o1:o1 + m * k].float().reshape(2, m, k) @ B[:, o2:o2 + n * k].float().reshape(2, n, k).transpose(1, 2)
        assert_scores_close(o[:, oo:oo + m * n], ref.reshape(2, -1), "gapped")
    assert (o[:, 24:30] == 9.0).all()                          # the gap is never written


def test_gapped_prefix_sums_with_a_transposed_operand(dev):
    # the any-layout 16-bit kernel behind caller-given prefix sums with holes in all three tensors: B_g stored K x N
    # (and then both operands k-major); the holes of the output keep what they held
    rng = np.random.default_rng(17)
    n = 9
    M = rng.integers(1, 150, n).astype(np.int64); N = rng.integers(1, 200, n).astype(np.int64)
    K = rng.choice([8, 24, 40, 64, 100, 136], n).astype(np.int64)
    gap = rng.integers(1, 4, n).astype(np.int64) * 3            # odd holes: later segments start at odd elements
    start = lambda area: np.concatenate([[0], np.cumsum(area + gap)]).astype(np.int64)
    a1, a2, ao = start(M * K), start(N * K), start(M * N)
    H = 2
    g = torch.Generator().manual_seed(4)
    A = torch.randn((H, int(a1[-1])), generator=g).half(); B = torch.randn((H, int(a2[-1])), generator=g).half()
    plan = capi.plan_gemm(n, dev, dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), dev_i64(a1, dev), dev_i64(a2, dev),
                          dev_i64(ao, dev), mode=capi.META_GIVEN)
    plan.read()
    for t1, t2 in ((False, True), (True, True)):
        out = torch.full((H, int(ao[-1])), 9.0, dtype=torch.float16, device=dev)
        capi.varlen_gemm(plan, A.to(dev), B.to(dev), out, H, int(a1[-1]), int(a2[-1]), int(ao[-1]), t1, t2)
        o = out.float().cpu()
        for i in range(n):
            m, nn, k = int(M[i]), int(N[i]), int(K[i])
            a = A[:, a1[i]:a1[i] + m * k].float(); b = B[:, a2[i]:a2[i] + nn * k].float()
            a = a.reshape(H, k, m).transpose(1, 2) if t1 else a.reshape(H, m, k)
            b = b.reshape(H, k, nn) if t2 else b.reshape(H, nn, k).transpose(1, 2)
            assert_scores_close(o[:, ao[i]:ao[i] + m * nn], (a @ b).reshape(H, -1), f"segment {i}, transposes {t1} {t2}")
            assert (o[:, ao[i] + m * nn:ao[i + 1]] == 9.0).all(), f"the hole behind segment {i} was written"


def test_many_tiny_segments_are_packed(dev):
    rng = np.random.default_rng(13)
    n = rng.integers(1, 9, 400)
    plan = run_all(dev, n, n, [64] * 400, 4, torch.float16, 0.125)
    assert plan.info.pack_items > 100
    m = rng.integers(1, 6, 300); nn = rng.integers(1, 6, 300)      # non-square tiny segments, bf16, K = 128
    plan = run_all(dev, m, nn, [128] * 300, 2, torch.bfloat16, 128 ** -0.5)
    assert plan.info.pack_items > 50


def test_unsupported_dtype_and_empty_calls(dev):
    plan = make_plan(dev, [4], [4], [8])
    x = torch.zeros((1, 32), dtype=torch.complex64, device=dev)     # not one of the reference's dispatch types
    with pytest.raises(capi.BlockedAttentionError, match="unsupported dtype"):
        capi.varlen_gemm(plan, x, x, x, 1, 32, 32, 16)
    e = torch.empty((0, 32), dtype=torch.float16, device=dev)
    capi.varlen_gemm(plan, e, e, torch.empty((0, 16), dtype=torch.float16, device=dev), 0, 32, 32, 16)


def test_two_products_in_one_launch(dev):
    # the backward pass's two products of a batch of short segments as ONE launch: the same bits as the two calls, and
    # BA_ERR_UNSUPPORTED (nothing written) where the library wants two calls (tall segments: the 128 x 128 build)
    rng = np.random.default_rng(61)
    for nseg, top, dtype in ((90, 130, torch.float16), (33, 70, torch.bfloat16), (6, 900, torch.float16)):
        M = rng.integers(1, top, nseg); N = rng.integers(1, top, nseg); K = rng.choice([8, 32, 64, 72, 128], nseg)
        H = 3
        A, B = random_operands(M, N, K, H, dtype, seed=nseg)
        dS = torch.randn((H, int((M * N).sum()))).to(dtype)
        Ad, Bd, dSd = A.to(dev), B.to(dev), dS.to(dev)
        # dA = dS B: rows M, columns K, reduction N, B stored N x K = k-major; dB = dS^T A: rows N, columns K, reduction M
        d_out, d_a, d_b = int((M * N).sum()), int((M * K).sum()), int((N * K).sum())
        acc = lambda x: dev_i64(np.concatenate([[0], np.cumsum(x)]), dev)
        plan_a = capi.plan_gemm(nseg, dev, dev_i64(M, dev), dev_i64(K, dev), dev_i64(N, dev), acc(M * N), acc(N * K), acc(M * K),
                                mode=capi.META_GIVEN)
        plan_b = capi.plan_gemm(nseg, dev, dev_i64(N, dev), dev_i64(K, dev), dev_i64(M, dev), acc(M * N), acc(M * K), acc(N * K),
                                mode=capi.META_GIVEN)
        plan_a.read(); plan_b.read()
        one = [torch.full((H, d), float("nan"), dtype=dtype, device=dev) for d in (d_a, d_b)]
        capi.varlen_gemm(plan_a, dSd, Bd, one[0], H, d_out, d_b, d_a, False, True)
        capi.varlen_gemm(plan_b, dSd, Ad, one[1], H, d_out, d_a, d_b, True, True)
        two = [torch.full((H, d), float("nan"), dtype=dtype, device=dev) for d in (d_a, d_b)]
        ran = capi.varlen_gemm_two(plan_a, dSd, Bd, two[0], (d_out, d_b, d_a), plan_b, dSd, Ad, two[1], (d_out, d_a, d_b), H)
        assert ran == (top < 200)
        if ran:
            assert torch.equal(one[0], two[0]) and torch.equal(one[1], two[1])
            ref = oracle.varlen_gemm(dS.float().numpy(), B.float().numpy(), M, K, N, False, True, f64acc=True)
            assert_scores_close(two[0], torch.from_numpy(ref), "dA")
        else:
            assert torch.isnan(two[0]).all() and torch.isnan(two[1]).all()
    # sizes that do not match the second plan: that product writes nothing and its plan counts a run error, the
    # first product is done all the same
    M, N, K = (rng.integers(1, 60, 12) for _ in range(3))
    K = 8 * (K // 8 + 1)
    A, B = random_operands(M, N, K, H, torch.float16, seed=5)
    dS = torch.randn((H, int((M * N).sum()))).half()
    d_out, d_a, d_b = int((M * N).sum()), int((M * K).sum()), int((N * K).sum())
    acc = lambda x: dev_i64(np.concatenate([[0], np.cumsum(x)]), dev)
    plan_a = capi.plan_gemm(12, dev, dev_i64(M, dev), dev_i64(K, dev), dev_i64(N, dev), acc(M * N), acc(N * K), acc(M * K), mode=capi.META_GIVEN)
    plan_b = capi.plan_gemm(12, dev, dev_i64(N, dev), dev_i64(K, dev), dev_i64(M, dev), acc(M * N), acc(M * K), acc(N * K), mode=capi.META_GIVEN)
    plan_a.read(); plan_b.read()
    out_a = torch.full((H, d_a), float("nan"), dtype=torch.float16, device=dev)
    out_b = torch.full((H, d_b + 8), float("nan"), dtype=torch.float16, device=dev)
    assert capi.varlen_gemm_two(plan_a, dS.to(dev), B.to(dev), out_a, (d_out, d_b, d_a), plan_b, dS.to(dev), A.to(dev), out_b,
                                (d_out, d_a, d_b + 8), H)
    torch.cuda.synchronize()
    assert torch.isnan(out_b).all() and not torch.isnan(out_a).any()
    assert plan_b.read(raise_on_bad=False).run_errors == 1 and plan_a.read().run_errors == 0

