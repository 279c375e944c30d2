"""Fused GEMM + softmax through the C ABI: every width class, fp32 output, the
large configuration at full size through size-independent properties."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi, workloads
from _util import assert_probs_close, make_plan, random_operands, run_all

pytestmark = pytest.mark.gpu


def test_split_and_wide_rows(dev):
    # 256 < N <= 4096: one workgroup per strip; N > 4096: two sweeps.
    M = [20, 3, 33, 16, 5]; N = [257, 4096, 1000, 4097, 9001]; K = [64, 128, 32, 72, 8]
    plan = run_all(dev, M, N, K, 2, torch.float16, 0.2, check_gemm=False)
    assert plan.info.split_items == 2 + 1 + 3 and plan.info.wide_items == 1 + 1
    run_all(dev, M, N, K, 2, torch.bfloat16, 0.1, seed=1, check_gemm=False)


def test_negative_and_zero_scale(dev):
    M = [9, 30, 4]; N = [300, 17, 5000]; K = [16, 64, 8]
    for scale in (-0.3, 0.0):
        run_all(dev, M, N, K, 2, torch.float16, scale, check_gemm=False)


def test_fp32_probabilities(dev):
    w = workloads.make(3)
    M, N, K = w.M[:200], w.N[:200], w.K[:200]
    A, B = random_operands(M, N, K, 2, torch.bfloat16)
    plan = make_plan(dev, M, N, K)
    i = plan.info
    out = torch.full((2, i.Dout), float("nan"), dtype=torch.float32, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, 2, i.Dm1, i.Dm2, i.Dout, w.scale)
    ref = oracle.per_segment_torch(A, B, M, N, K, w.scale)
    assert (out.cpu() - ref).abs().max().item() <= 2e-5        # fp32 output: the 1e-3 bound holds with room


def test_large_segments_one_head_against_oracle(dev):
    # Configuration 5 shape (n in [1024, 4096], K = 128, bf16) on its three smallest segments.
    w = workloads.make(5)
    idx = np.argsort(w.M)[:3]
    M = w.M[idx]
    A, B = random_operands(M, M, [128] * 3, 1, torch.bfloat16, sigma=w.sigma)
    plan = make_plan(dev, M, M, [128] * 3)
    i = plan.info
    out = torch.empty((1, i.Dout), dtype=torch.bfloat16, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, 1, i.Dm1, i.Dm2, i.Dout, w.scale)
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, M, [128] * 3, w.scale), "cfg5 subset")


def test_config5_full_size_properties(dev):
    # 16 segments x 16 heads, 1.93e9 probabilities: rows sum to one, and sampled rows match the oracle.
    w = workloads.make(5)
    A, B = w.operands()
    plan = make_plan(dev, w.M, w.N, w.K)
    Ad, Bd = A.to(dev), B.to(dev)
    out = torch.empty((w.heads, w.Dout), dtype=torch.bfloat16, device=dev)
    capi.gemm_softmax(plan, Ad, Bd, out, w.heads, w.Dm1, w.Dm2, w.Dout, w.scale)
    a1, a2, ao = oracle.lists_to_accum(w.M, w.N, w.K)
    rng = np.random.default_rng(0)
    for g in range(w.nseg):
        n = int(w.M[g])
        blk = out[:, ao[g]:ao[g + 1]].reshape(w.heads, n, n)
        sums = blk.float().sum(-1)
        assert (sums - 1).abs().max().item() < 2e-2, g          # bf16 rounding of n values of ~1/n
        h = int(rng.integers(0, w.heads)); r = int(rng.integers(0, n))
        a = A[h, a1[g] + r * 128:a1[g] + (r + 1) * 128].float()
        b = B[h, a2[g]:a2[g + 1]].float().reshape(n, 128)
        ref = torch.softmax((b @ a) * w.scale, -1)
        got = blk[h, r].float().cpu()
        assert ((got - ref).abs() <= 1e-3 + ref * 2.0 ** -8).all(), (g, h, r)
        assert ((got - ref.bfloat16().float()).abs() <= ref * 2.0 ** -7 + 1e-9).all(), (g, h, r)
    assert plan.read().run_errors == 0


def test_long_k_and_every_launch_class(dev):
    # K > 128 (A fragments reloaded per 128-k span in the tile kernel, K slabs in the segment kernel),
    # ragged K, and one call that exercises all four work lists at once.
    M = [40, 130, 20, 64, 7, 5, 300, 33]; N = [48, 300, 200, 256, 6, 9, 129, 64]; K = [160, 256, 200, 128, 16, 16, 136, 264]
    for dtype, scale in ((torch.float16, 0.05), (torch.bfloat16, -0.05)):
        plan = run_all(dev, M, N, K, 2, dtype, scale, seed=3)
        i = plan.info
        # (64,256,128): 16 tiles x 4 k-steps = 64 blocks -> big; (7,6,16)+(5,9,16) pack; N >= 128 with long K -> tile
        assert i.list_big == 1 and i.list_tile == 3 and i.list_small == 0
        assert i.list_small + i.list_big + i.list_tile + i.list_rest + 1 == len(M)      # one pack follower


def test_work_lists_match_the_shape_rules(dev):
    # The lengths of the work lists against the classification restated on the host.
    for cfg in (1, 2, 3, 4, 5):
        w = workloads.make(cfg)
        plan = make_plan(dev, w.M, w.N, w.K)
        i = plan.info
        tiles = 2 * ((w.N + 31) // 32); nks = (w.K + 31) // 32
        blocks = np.where((w.N >= 2) & (w.N <= 256) & (nks >= 1) & (nks <= 4), tiles * nks, 0)
        aligned = (w.K % 8 == 0)                       # offsets of these configurations are multiples of 8 with K
        packed = i.list_small + i.list_mini + i.list_big + i.list_tile + i.list_rest
        small = int(((blocks >= 1) & (blocks <= 32) & aligned).sum())
        big = int(((blocks > 32) & (blocks <= 64) & aligned).sum())
        assert i.list_big == big, cfg
        main = i.list_small + i.list_mini                # the main strip list: its mini entries are counted apart
        assert main <= small and small - main <= 2 * i.pack_items * 8, cfg   # packs take tiny ones
        assert i.list_mini <= int(((w.M <= 64) & (blocks >= 1) & (blocks <= 16) & (tiles <= 8) & aligned).sum()), cfg
        assert i.list_tile == int(((w.N > 256) | ((w.N >= 128) & (blocks == 0))).sum()), cfg
        assert packed <= w.nseg
        assert i.list_rows == int(((w.N > 256) & (w.M >= 1)).sum()), cfg     # the softmax row kernel's list


def test_launches_without_the_host_summary(dev):
    # Nothing is read back between the scheduler and the kernels: every kernel is launched over nseg slots
    # with default z and finds its list (or nothing) in the plan.  All five lists, tall and wide segments.
    M = [40, 130, 20, 64, 7, 5, 300, 33, 700, 12, 1]; N = [48, 300, 200, 256, 6, 9, 129, 64, 40, 5000, 1]
    K = [160, 256, 200, 128, 16, 16, 136, 264, 64, 8, 8]
    for dtype, scale in ((torch.float16, 0.05), (torch.bfloat16, -0.05)):
        plan = run_all(dev, M, N, K, 2, dtype, scale, seed=5, summary=False)
        i = plan.info
        assert i.list_big == 1 and i.list_tile == 4 and i.list_rows == 2 and i.pack_items == 1


def test_both_strip_lists_merged_and_separate(dev):
    # Segments for both LDS windows of the strip kernel (B_g up to 32 KiB / up to 64 KiB), packs and tile-kernel
    # segments in one batch.  Few (list entry, head) pairs, or wide segments in the 32 KiB list: one launch takes
    # both lists.  Many pairs and a narrow 32 KiB list: one launch per list.
    rng = np.random.default_rng(21)
    def batch(nseg, wide_small):
        M = rng.integers(1, 40, nseg); K = np.full(nseg, 128)
        N = np.where(rng.random(nseg) < 0.8, rng.integers(2, 129, nseg), rng.integers(129, 257, nseg))
        if wide_small:
            K[:8] = 32; N[:8] = 250                      # 16 tiles x 1 k-step: the 32 KiB list, wider than 128
        N[-1] = 300; M[-1] = 130                         # one tile-kernel segment rides along
        return M, N, K
    for nseg, heads, wide_small in ((40, 2, False), (40, 2, True), (1200, 7, False), (1200, 7, True)):
        M, N, K = batch(nseg, wide_small)
        plan = run_all(dev, M, N, K, heads, torch.bfloat16, 0.09, seed=nseg + heads, check_softmax=False)
        i = plan.info
        assert i.list_small > 0 and i.list_big > 0 and i.list_tile == 1
        assert (i.small_max_N > 128) == wide_small
        assert i.list_mini > 0                           # narrow segments of few rows: one wavefront each
        assert ((i.list_small + i.list_big) * heads > 4096) == (nseg == 1200)


def test_more_list_entries_than_the_second_grid_dimension_holds(dev):
    # 66 000 strip-class segments: the list entries cannot ride on gridDim.y (65 535 at most), so the launches
    # fall back to the entry as the fastest grid index; the scheduler takes 65 passes.
    rng = np.random.default_rng(8)
    nseg = 66000
    M = rng.integers(17, 25, nseg); N = rng.integers(17, 25, nseg); K = np.full(nseg, 8)
    plan = run_all(dev, M, N, K, 2, torch.float16, 0.3, seed=2)
    assert plan.info.list_small + plan.info.list_mini == nseg and plan.info.list_mini > 0


def test_mini_segments_alone_and_among_others(dev):
    # Segments of at most 64 rows whose B_g takes at most 16 KiB: one wavefront each, four to a workgroup where the
    # launch has the 64 KiB window (a wide segment in the batch), one workgroup each otherwise.  Every boundary of the
    # class: 64 / 65 rows, 16 / 17 operand blocks, every tile count up to eight, every B_g layout (K = 64, 128, other),
    # ragged columns, one row, groups of four that are not full.
    rng = np.random.default_rng(31)
    M = np.array([64, 65, 1, 16, 17, 33, 48, 64, 5, 64, 20, 64, 31])
    N = np.array([64, 64, 2, 33, 127, 128, 96, 129, 250, 17, 64, 61, 256])
    K = np.array([128, 128, 128, 64, 64, 64, 72, 48, 32, 128, 104, 120, 32])
    wide = (np.array([200]), np.array([256]), np.array([128]))        # B_g of 64 KiB: the launch gets the wide window
    for extra, heads, dtype, scale in ((None, 3, torch.float16, 0.2), (wide, 2, torch.bfloat16, -0.1),
                                       (wide, 5, torch.float16, 0.0)):
        m, n, k = (M, N, K) if extra is None else tuple(np.concatenate([a, b]) for a, b in zip((M, N, K), extra))
        plan = run_all(dev, m, n, k, heads, dtype, scale, seed=3)
        i = plan.info
        assert i.list_mini == 8 and i.list_big == (0 if extra is None else 1)
        run_all(dev, m, n, k, heads, dtype, scale, seed=4, summary=False)
    # many of them, a count that is not a multiple of four, among two wide segments
    nseg = 203
    m = rng.integers(1, 65, nseg); n = rng.integers(2, 65, nseg); k = np.full(nseg, 128)
    m[[7, 150]] = 180; n[[7, 150]] = 250
    plan = run_all(dev, m, n, k, 3, torch.bfloat16, 128 ** -0.5, seed=5)
    assert plan.info.list_mini >= 150 and plan.info.list_big == 2
