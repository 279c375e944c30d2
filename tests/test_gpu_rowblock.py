"""Large segments with K <= 256 (the row-block kernels: 256 rows per workgroup or per wavefront set, 64 columns at
a time, results through an LDS ring into line-aligned stores; the fused pair with K <= 128 runs the two sweeps of
adjacent row blocks side by side on one stream of B_g; 128 < K <= 256 takes a build with two LDS stages per chunk)
against the oracle: every line phase, ragged rows and columns, every reduction length, the overflow path of the
first sweep, GEMM alone and fused."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi
from _util import assert_probs_close, assert_scores_close, make_plan, random_operands, run_all

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_shapes_and_phases(dev, dtype):
    # odd and even widths (rows then start at every 2-byte phase of a 128-byte line), widths around the chunk
    # and ring sizes, heights around the workgroup's 256 rows and a wavefront's 32, one row, K from 8 to 128
    # (and K = 0: no operand bytes at all, zeros for the product and 1/N for the fused pair)
    M = [300, 256, 257, 1, 40, 33, 513, 31, 40]; N = [257, 300, 1000, 5000, 320, 321, 263, 384, 300]
    K = [64, 128, 8, 40, 96, 104, 120, 32, 0]
    plan = run_all(dev, M, N, K, 3, dtype, 0.11, seed=7)
    assert plan.info.list_tile == len(M)


def test_every_width_modulo_the_chunk(dev):
    # N mod 64 = 0..63 at two sizes: the ragged last chunk, the window behind it and the unaligned end pieces
    N = np.concatenate([np.arange(257, 321), [448, 449, 511, 512, 513]]); M = np.full(N.size, 37); K = np.full(N.size, 16)
    run_all(dev, M, N, K, 1, torch.float16, 0.3, seed=3, check_softmax=False)
    run_all(dev, M[::7], N[::7], K[::7], 2, torch.bfloat16, -0.2, seed=4, check_softmax=False)


def test_negative_and_zero_scale_large(dev):
    for scale in (-0.3, 0.0):
        run_all(dev, [70, 290], [700, 333], [64, 128], 2, torch.float16, scale, check_gemm=False)


def test_scores_far_above_the_first_chunk(dev):
    # The first sweep measures every score against the row maximum of the FIRST 64 columns.  Here the later
    # columns exceed it by far more than the exponent range: the sums overflow, and the workgroup repeats the
    # sweep with a running maximum.  Rows of a second segment in the same call take the fast path.
    M = np.array([100, 64]); N = np.array([700, 300]); K = np.array([128, 64])
    A, B = random_operands(M, N, K, 2, torch.float16, seed=11)
    A = A.abs() + 1; B = B.abs()
    Bs = B[:, :700 * 128].reshape(2, 700, 128)
    Bs[:, :64] *= 0.01                                        # tiny scores in the first chunk
    Bs[:, 300:310] *= 4                                       # the rows' maxima, hundreds above
    plan = make_plan(dev, M, N, K)
    i = plan.info
    out = torch.full((2, i.Dout), float("nan"), dtype=torch.float16, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, 2, i.Dm1, i.Dm2, i.Dout, 1.0)
    ref = oracle.per_segment_torch(A, B, M, N, K, 1.0)
    assert_probs_close(out, ref, "overflow path")
    assert float(out[:, :100 * 700].float().max()) > 0.05     # sharply peaked rows, as constructed
    assert plan.read().run_errors == 0


def test_overflow_in_the_middle_of_a_run_of_row_blocks(dev):
    # Seven row blocks of one segment go through a workgroup's two wavefront sets, one sweep apart.  Only rows of the
    # fourth block overflow the first sweep: that set repeats its block in two safe sweeps while the other set waits
    # where it must, and the blocks before and after take the ordinary path.  A second head keeps both orders of
    # the sets in play (its shares of row blocks start at another parity).
    M = np.array([1700]); N = np.array([900]); K = np.array([64])
    A, B = random_operands(M, N, K, 2, torch.float16, seed=13)
    A = A.abs() * 0.5 + 0.5; B = B.abs()
    Bs = B.reshape(2, 900, 64)
    Bs[:, :64] *= 0.01                                        # tiny scores in the first chunk
    As = A.reshape(2, 1700, 64)
    As[:, :768] *= 0.02; As[:, 1024:] *= 0.02                 # only rows 768 .. 1023 reach far above it
    Bs[:, 500:520] *= 6
    plan = make_plan(dev, M, N, K)
    i = plan.info
    out = torch.full((2, i.Dout), float("nan"), dtype=torch.float16, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, 2, i.Dm1, i.Dm2, i.Dout, 1.0)
    ref = oracle.per_segment_torch(A, B, M, N, K, 1.0)
    assert_probs_close(out, ref, "overflow in one row block of seven")
    peaked = out[:, 768 * 900:1024 * 900].float().max()
    assert float(peaked) > 0.04                               # sharply peaked rows, as constructed
    assert plan.read().run_errors == 0


def test_unaligned_output_base_and_many_heads(dev):
    # the result tensor starts 2 bytes past a 256-byte boundary and Dout is odd: every head has its own phases
    M = np.array([131, 50]); N = np.array([259, 641]); K = np.array([64, 64])
    H = 5
    A, B = random_operands(M, N, K, H, torch.bfloat16, seed=5)
    plan = make_plan(dev, M, N, K)
    i = plan.info
    assert i.Dout % 2 == 1
    buf = torch.full((H * i.Dout + 1,), float("nan"), dtype=torch.bfloat16, device=dev)
    out = buf[1:].view(H, i.Dout)
    assert out.data_ptr() % 4 == 2
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, H, i.Dm1, i.Dm2, i.Dout, 0.125)
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, 0.125), "unaligned base")
    assert torch.isnan(buf[0])                                 # nothing written in front of the result
    sc = torch.full((H * i.Dout + 1,), float("nan"), dtype=torch.bfloat16, device=dev)
    capi.varlen_gemm(plan, A.to(dev), B.to(dev), sc[1:].view(H, i.Dout), H, i.Dm1, i.Dm2, i.Dout)
    assert_scores_close(sc[1:].view(H, i.Dout), oracle.per_segment_torch(A, B, M, N, K, 0.125, want="both")[0], "scores")
    assert torch.isnan(sc[0])


def test_gaps_between_segments_stay_untouched(dev):
    # prefix sums given with gaps: the elements between two segments' results keep what they held
    M = np.array([40, 70]); N = np.array([300, 260]); K = np.array([32, 32])
    A, B = random_operands(M, N, K, 1, torch.float16, seed=6)
    a1 = np.array([0, 40 * 32, 40 * 32 + 70 * 32]); a2 = np.array([0, 300 * 32, 300 * 32 + 260 * 32])
    ao = np.array([0, 40 * 300 + 37, 40 * 300 + 37 + 70 * 260 + 5])
    from _util import dev_i64
    plan = capi.plan_gemm(2, dev, dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), dev_i64(a1, dev), dev_i64(a2, dev),
                          dev_i64(ao, dev), mode=capi.META_GIVEN)
    plan.read()
    out = torch.full((1, int(ao[-1])), 7.0, dtype=torch.float16, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, 1, int(a1[-1]), int(a2[-1]), int(ao[-1]), 0.2)
    ref = oracle.per_segment_torch(A, B, M, N, K, 0.2)
    got = out.cpu()
    assert_probs_close(got[:, :40 * 300], ref[:, :40 * 300], "first")
    assert_probs_close(got[:, ao[1]:ao[1] + 70 * 260], ref[:, 40 * 300:], "second")
    assert (got[:, 40 * 300:ao[1]] == 7).all() and (got[:, ao[1] + 70 * 260:] == 7).all()


def test_nearly_empty_last_row_block_under_load(dev):
    # The last row block of each segment holds a handful of rows, so most wavefronts of its workgroup only move
    # key chunks; N is ragged, so part of the last chunk's loads are never issued.  Many heads keep the chip busy
    # while these workgroups run, which is when a load that is waited for too late shows.
    M = np.array([267, 523, 11, 290]); N = np.array([1483, 2571, 900, 2594]); K = np.array([128, 128, 64, 128])
    for rep in range(2):
        run_all(dev, M, N, K, 16, torch.float16, 0.05, seed=21 + rep)


def test_k_zero_in_the_tile_kernel(dev):
    # without the host summary the large segments run in the tile kernel, and so do large segments of 256 columns
    # or fewer in a fused call: K = 0 has no operand bytes there either, and the rows are zeros (product) or 1/N
    # (fused pair); the K = 136 neighbour takes the row-block kernel's wide build
    run_all(dev, [40, 200, 70], [300, 130, 260], [0, 0, 64], 2, torch.float16, 0.2, summary=False)
    run_all(dev, [40, 200, 70], [300, 130, 260], [0, 0, 136], 2, torch.bfloat16, 0.2)


def fused_only(dev, M, N, K, H, dtype, scale, summary, seed=0, out_dtype=None):
    M = np.asarray(M, np.int64); N = np.asarray(N, np.int64); K = np.asarray(K, np.int64)
    A, B = random_operands(M, N, K, H, dtype, seed)
    plan = make_plan(dev, M, N, K, read=summary)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    out = torch.full((H, do), float("nan"), dtype=out_dtype or dtype, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, H, d1, d2, do, scale)
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, scale), "fused")
    info = plan.read()
    assert info.run_errors == 0
    return info


def test_the_pipelined_kernel_is_chosen_segment_by_segment(dev):
    # K = 136, 160 and 256 send a segment to the row-block kernel's wide build; its neighbours with K <= 128 still take
    # the pipelined row-block kernel, in the same call (the plan counts them, the kernels count the workgroups that worked)
    M = [300, 520, 100, 260, 700, 64]; N = [400, 300, 1000, 263, 513, 200]; K = [128, 136, 64, 160, 8, 256]
    for dtype in (torch.float16, torch.bfloat16):
        info = fused_only(dev, M, N, K, 2, dtype, 0.13, summary=True, seed=3)
        assert info.list_tile == 6 and info.list_pipe == 3
        assert info.pipe_groups >= 3 * 2                      # at least one workgroup per eligible segment and head
        assert info.wide_groups >= 3 * 2


def test_the_pipelined_kernel_runs_without_the_host_summary(dev):
    # no summary was read between scheduler and kernels (graph replays, the one-call entry point): the large
    # segments with K <= 128 still go through the pipelined kernel, the others through the tile kernel
    M = [300, 520, 1030, 260]; N = [400, 300, 1000, 263]; K = [128, 136, 64, 96]
    info = fused_only(dev, M, N, K, 3, torch.bfloat16, 0.2, summary=False, seed=5)
    assert info.list_pipe == 3 and info.pipe_groups >= 3 * 3
    # all of them eligible: the tile kernel is still launched (nothing told the host) and finds nothing
    info = fused_only(dev, M[:1] + M[2:], N[:1] + N[2:], K[:1] + K[2:], 2, torch.float16, 0.2, summary=False, seed=6)
    assert info.list_pipe == 3 and info.pipe_groups >= 3 * 2


def test_fp32_probabilities_of_large_segments_stay_in_the_tile_kernel(dev):
    info = fused_only(dev, [300, 260], [400, 263], [128, 96], 2, torch.bfloat16, 0.2, summary=True, seed=7,
                      out_dtype=torch.float32)
    assert info.list_pipe == 2 and info.pipe_groups == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reduction_lengths_between_128_and_256(dev, dtype):
    # every multiple of 8 that needs the second span, widths at every phase, heights around 256 and 32 rows;
    # neighbours with K <= 128 and K > 256 go to the other kernels of the same call
    M = [300, 256, 257, 1, 40, 33, 513, 31, 100, 90]; N = [257, 300, 1000, 3000, 320, 321, 263, 384, 300, 290]
    K = [136, 256, 160, 200, 248, 144, 192, 232, 128, 264]
    plan = run_all(dev, M, N, K, 3, dtype, 0.11, seed=7, sigma=0.5)
    info = plan.read()
    assert info.list_tile == len(M)
    # GEMM and fused call: at least one workgroup per eligible segment and head in each
    assert info.wide_groups >= 2 * 8 * 3


def test_widths_modulo_the_chunk_and_negative_scale(dev):
    N = np.concatenate([np.arange(257, 321, 3), [448, 449, 511, 512, 513]]); M = np.full(N.size, 37); K = np.full(N.size, 136)
    K[::2] = 256
    run_all(dev, M, N, K, 1, torch.float16, 0.3, seed=3, check_softmax=False, sigma=0.5)
    run_all(dev, M[::3], N[::3], K[::3], 2, torch.bfloat16, -0.2, seed=4, check_softmax=False, sigma=0.5)


def test_overflow_of_the_first_sweep(dev):
    M = np.array([100, 64]); N = np.array([700, 300]); K = np.array([256, 160])
    A, B = random_operands(M, N, K, 2, torch.float16, seed=11)
    A = A.abs() * 0.7 + 0.7; B = B.abs()
    Bs = B[:, :700 * 256].reshape(2, 700, 256)
    Bs[:, :64] *= 0.01
    Bs[:, 300:310] *= 4
    plan = make_plan(dev, M, N, K)
    i = plan.info
    out = torch.full((2, i.Dout), float("nan"), dtype=torch.float16, device=dev)
    capi.gemm_softmax(plan, A.to(dev), B.to(dev), out, 2, i.Dm1, i.Dm2, i.Dout, 1.0)
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, 1.0), "overflow path")
    info = plan.read()
    assert info.run_errors == 0 and info.wide_groups >= 4


def test_many_heads_and_tall_segments(dev):
    M = np.array([1267, 523, 11, 290]); N = np.array([1483, 2571, 900, 2594]); K = np.array([256, 136, 64, 200])
    for rep in range(2):
        plan = run_all(dev, M, N, K, 8, torch.bfloat16, 0.05, seed=21 + rep, sigma=0.5, check_softmax=False)
    assert plan.read().wide_groups > 0


def test_the_product_alone_is_routed_segment_by_segment(dev):
    # K <= 128 to the row-block kernel, 128 < K <= 256 to its wide build, K > 256 to the tile kernel, in one call
    M = [300, 520, 100, 260, 700, 64]; N = [400, 300, 1000, 263, 513, 200]; K = [128, 136, 64, 160, 8, 264]
    plan = run_all(dev, M, N, K, 2, torch.bfloat16, 0.13, seed=3, sigma=0.5, check_softmax=False)
    assert plan.read().wide_groups >= 2 * 2 * 2
    # nothing beyond K = 256: the tile kernel is not launched for the product
    plan = run_all(dev, M[:5], N[:5], K[:5], 2, torch.float16, 0.13, seed=4, sigma=0.5, check_softmax=False)
    assert plan.read().wide_groups >= 2 * 2 * 2
    # only wide segments
    plan = run_all(dev, [300, 64], [400, 300], [256, 136], 2, torch.float16, 0.2, seed=5, sigma=0.5)
    assert plan.read().wide_groups >= 2 * 2 * 2


def test_without_the_summary_the_tile_kernel_takes_them(dev):
    plan = run_all(dev, [300, 100], [400, 300], [256, 136], 2, torch.float16, 0.2, summary=False, sigma=0.5)
    assert plan.read().wide_groups == 0
