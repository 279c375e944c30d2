"""One-pass varlen attention (ba_varlen_attention) through the C ABI against the oracle.

Bound, from what the kernel rounds: sums are fp32; every probability is rounded once to the 16-bit type
before the second product (relative error u = 2^-11 for fp16, 2^-9 for bf16), which moves output element
(r, d) by at most u * sum_n P[r, n] |V[n, d]|, and the result is rounded once at the store (u * |o|).  With
a factor two of room: |o - ref| <= 2u * ((P |V|)[r, d] + |ref|) + 1e-3 * rms(ref)."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi, workloads
from _util import assert_scores_close, make_plan


def assert_outputs_close(got, ref, p_abs_v, what=""):
    u = 2.0 ** -11 if got.dtype == torch.float16 else 2.0 ** -9
    got = got.float().cpu()
    assert not torch.isnan(got).any(), f"{what}: NaN"
    rms = float(ref.pow(2).mean().sqrt()) if ref.numel() else 0.0
    excess = (got - ref).abs() - (2 * u * (p_abs_v + ref.abs()) + 1e-3 * rms)
    assert excess.numel() == 0 or excess.max().item() <= 0, f"{what}: off by {float((got - ref).abs().max())}"

pytestmark = pytest.mark.gpu


def operands(M, N, K, H, dtype, seed=0, sigma=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    d1 = int((np.asarray(M) * np.asarray(K)).sum()); d2 = int((np.asarray(N) * np.asarray(K)).sum())
    Q = (torch.randn((H, d1), generator=g) * sigma).to(dtype)
    Km = (torch.randn((H, d2), generator=g) * sigma).to(dtype)
    V = torch.randn((H, d2), generator=g).to(dtype)
    return Q, Km, V


def run(dev, M, N, K, H, dtype, scale, seed=0, sigma=1.0, summary=True):
    M = np.asarray(M, np.int64); N = np.asarray(N, np.int64); K = np.asarray(K, np.int64)
    Q, Km, V = operands(M, N, K, H, dtype, seed, sigma)
    plan = make_plan(dev, M, N, K, read=summary)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    out = torch.full((H, d1), float("nan"), dtype=dtype, device=dev)
    print(f"attention case M={M[:6]} N={N[:6]} K={K[:6]} H={H} {dtype} scale={scale}", flush=True)
    capi.varlen_attention(plan, Q.to(dev), Km.to(dev), V.to(dev), out, H, d1, d2, do, scale)
    ref = oracle.per_segment_torch_attention(Q, Km, V, M, N, K, scale)
    assert_outputs_close(out, ref, oracle.per_segment_torch_attention(Q, Km, V.abs(), M, N, K, scale), "attention")
    info = plan.read()
    assert info.run_errors == 0
    return out, ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_small_and_ragged_segments(dev, dtype):
    M = [1, 16, 17, 63, 64, 65, 130, 5, 200]; N = [1, 7, 64, 65, 63, 128, 129, 300, 31]
    K = [64, 64, 64, 64, 64, 64, 64, 64, 64]
    run(dev, M, N, K, 3, dtype, 0.125)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_head_dimensions(dev, dtype):
    # every multiple of 8 up to 128 (zero padded to 32 inside), mixed in one call
    K = list(range(8, 129, 8))
    M = [20 + 3 * i for i in range(len(K))]; N = [90 - 5 * i for i in range(len(K))]
    run(dev, M, N, K, 2, dtype, 0.2, seed=1)
    for k in (8, 32, 40, 96, 128):                      # one head dimension per call: each build of the kernel
        run(dev, [33, 70], [50, 129], [k, k], 2, dtype, k ** -0.5, seed=k)


def test_head_dimensions_not_multiples_of_eight_and_odd_offsets(dev):
    M = [3, 11, 40, 7, 65]; N = [5, 66, 13, 130, 64]; K = [5, 33, 100, 1, 127]
    run(dev, M, N, K, 3, torch.float16, 0.3)
    run(dev, M, N, K, 1, torch.bfloat16, 0.1, seed=2)


def test_vector_loads_at_odd_element_offsets(dev):
    # segments whose head dimension is a multiple of 8 (16-byte loads through the segment's buffer descriptor)
    # but that start at an odd element: the segments before them have odd sizes
    M = [3, 40, 5, 70, 1, 130]; N = [5, 100, 7, 65, 3, 200]; K = [5, 64, 7, 128, 1, 96]
    run(dev, M, N, K, 2, torch.float16, 0.2, seed=5)
    run(dev, M, N, K, 3, torch.bfloat16, 0.1, seed=6)


def test_empty_segments_and_no_keys(dev):
    # M = 0: nothing; N = 0: zeros (a sum over no keys)
    M = [4, 0, 9, 30]; N = [6, 5, 0, 70]; K = [16, 8, 24, 64]
    out, ref = run(dev, M, N, K, 2, torch.float16, 0.5)
    assert torch.equal(out[:, 64:64 + 9 * 24].cpu(), torch.zeros(2, 9 * 24, dtype=torch.float16))


def test_tall_segment_without_keys_among_others(dev):
    # A tall N = 0 segment has row blocks of its own (zeros to write): the launch is sized from the plan's
    # row-block totals, which count it, so neither its rows nor its neighbours' are left unwritten.
    M = [64, 1000, 64]; N = [64, 0, 64]; K = [64, 64, 64]
    for dtype in (torch.float16, torch.bfloat16):
        out, ref = run(dev, M, N, K, 8, dtype, 0.125)
        assert torch.equal(out[:, 64 * 64:64 * 64 + 1000 * 64].cpu(), torch.zeros(8, 1000 * 64, dtype=dtype))
    plan = make_plan(dev, M, N, K)
    assert plan.info.att_blocks64 == 1 + 16 + 1 and plan.info.att_blocks128 == 1 + 8 + 1
    assert plan.info.total_rows == 128


def test_negative_and_zero_scale(dev):
    M = [9, 70]; N = [100, 17]; K = [16, 64]
    for scale in (-0.3, 0.0):
        run(dev, M, N, K, 2, torch.float16, scale)
    # tall segments (two strips per wavefront), last key block ragged: a zero scale must still give the mean of
    # the values over the keys that exist
    for scale in (-0.2, 0.0):
        run(dev, [300, 520], [130, 77], [128, 64], 2, torch.bfloat16, scale, seed=7)


def test_long_segments_many_key_blocks(dev):
    # the running maximum changes over many blocks; large scores exercise the rescaling
    run(dev, [100, 257], [3000, 1025], [128, 64], 2, torch.bfloat16, 128 ** -0.5, sigma=1.0)
    run(dev, [70], [2000], [64], 1, torch.float16, 1.0, sigma=2.0, seed=3)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_batches(dev, seed):
    # random batches: segment counts, heights, widths and head dimensions drawn anew (multiples of 8 or anything),
    # with empty segments among them; both strip counts and every head-dimension build come up over the seeds
    rng = np.random.default_rng(seed)
    nseg = int(rng.integers(1, 40))
    tall = seed % 2 == 0
    M = rng.integers(0, 700 if tall else 150, nseg); N = rng.integers(0, 400, nseg)
    kmax = int(rng.choice([16, 32, 64, 96, 128]))
    K = rng.integers(1, kmax // 8 + 1, nseg) * 8 if seed % 3 else rng.integers(1, kmax + 1, nseg)
    dtype = torch.float16 if seed % 2 else torch.bfloat16
    run(dev, M, N, K, int(rng.integers(1, 4)), dtype, float(rng.uniform(0.05, 0.3)), seed=seed)


def test_launch_without_the_host_summary(dev):
    M = [33, 5, 300, 64]; N = [40, 200, 70, 64]; K = [64, 128, 32, 72]
    run(dev, M, N, K, 2, torch.float16, 0.125, summary=False)


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_benchmark_configurations(dev, cfg):
    # configuration 5 (segments of 1024 .. 4096 rows) at full segment sizes on one head
    w = workloads.make(cfg)
    run(dev, w.M, w.N, w.K, min(w.heads, 2) if cfg < 5 else 1, w.dtype, w.scale, sigma=w.sigma)


def test_tall_segments_row_blocks_side_by_side(dev):
    # mean height >= 512: two strips per wavefront and the row blocks of a (segment, head) pair on one die
    run(dev, [600, 1000, 513], [300, 700, 64], [64, 64, 64], 3, torch.float16, 0.125)
    run(dev, [700, 520], [130, 900], [128, 40], 2, torch.bfloat16, 0.1, seed=4)


def test_matches_the_three_call_chain(dev):
    # the chain the one-pass kernel replaces: fused scores+softmax, then probabilities times values
    import blockedAttention
    M = [50, 120, 8]; N = [64, 33, 200]; K = [64, 64, 64]
    Q, Km, V = operands(M, N, K, 2, torch.float16, seed=5)
    Md, Nd, Kd = (torch.tensor(x, dtype=torch.int64, device=dev) for x in (M, N, K))
    P = blockedAttention.blockGEMMSoftmax(Q.to(dev), Km.to(dev), MList=Md, NList=Nd, KList=Kd, scale=0.125)
    chain = blockedAttention.blockGEMM(P, V.to(dev), None, None, None, Md, Kd, Nd, False, True)
    one = blockedAttention.blockFusedAttention(Q.to(dev), Km.to(dev), V.to(dev), Md, Nd, Kd, scale=0.125)
    assert one.shape == chain.shape and one.dtype == chain.dtype
    assert_scores_close(one, chain.float().cpu(), "one pass against the chain")


def test_head_dimension_above_128_is_refused(dev):
    plan = make_plan(dev, [4], [4], [136])
    t = torch.zeros((1, 4 * 136), dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError, match="unsupported"):
        capi.varlen_attention(plan, t, t, t, torch.empty_like(t), 1, 4 * 136, 4 * 136, 16, 1.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_backward_matches_per_segment_autograd(dev, dtype):
    # dq, dk, dv of the one-pass operator against torch.autograd on the per-segment fp32 oracle (same 16-bit
    # inputs).  The backward rounds the recomputed scores and probabilities, dP, dS and the results to the
    # 16-bit type (u = 2^-11 / 2^-9 each), and dS = P (dP - sum P dP) cancels: the bound is that of the scores,
    # |g - ref| <= tol (|ref| + rms(ref)), with tol = 20 u (1e-2 for fp16, 4e-2 for bf16).
    import blockedAttention
    M = [50, 120, 8, 33]; N = [64, 33, 200, 7]; K = [64, 64, 64, 64]
    Q, Km, V = operands(M, N, K, 2, dtype, seed=9, sigma=0.5)
    Md, Nd, Kd = (torch.tensor(x, dtype=torch.int64, device=dev) for x in (M, N, K))
    q, k, v = (t.to(dev).requires_grad_() for t in (Q, Km, V))
    out = blockedAttention.blockFusedAttention(q, k, v, Md, Nd, Kd, scale=0.125)
    g = torch.Generator(device="cpu").manual_seed(10)
    wgt = torch.randn(out.shape, generator=g).to(dtype)
    out.backward(wgt.to(dev))
    qr, kr, vr = (t.float().requires_grad_() for t in (Q, Km, V))
    ref = oracle.per_segment_torch_attention(qr, kr, vr, M, N, K, 0.125)
    ref.backward(wgt.float())
    tol = 1e-2 if dtype == torch.float16 else 4e-2
    for name, got, want in (("dq", q.grad, qr.grad), ("dk", k.grad, kr.grad), ("dv", v.grad, vr.grad)):
        assert got.dtype == dtype and got.shape == want.shape
        got = got.float().cpu()
        assert not torch.isnan(got).any(), name
        rms = float(want.pow(2).mean().sqrt())
        excess = (got - want).abs() - (tol * want.abs() + tol * rms)
        assert excess.max().item() <= 0, f"{name}: off by {float((got - want).abs().max())} (rms {rms})"


def test_backward_needs_the_size_lists(dev):
    import blockedAttention
    M = np.array([4, 9]); N = np.array([5, 3]); K = np.array([8, 8])
    a1, a2, ao = (torch.from_numpy(x).to(dev) for x in oracle.lists_to_accum(M, N, K))
    q = torch.randn((1, int((M * K).sum())), device=dev, dtype=torch.float16, requires_grad=True)
    kv = torch.randn((1, int((N * K).sum())), device=dev, dtype=torch.float16)
    out = blockedAttention.blockFusedAttention(q, kv, kv, mat1Accum=a1, mat2Accum=a2, outAccum=ao)
    with pytest.raises(RuntimeError, match="MList"):
        out.sum().backward()
