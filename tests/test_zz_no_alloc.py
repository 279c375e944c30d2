"""The entry point that allocates nothing: ba_gemm_softmax_static keeps its plan in a buffer of the library's
device image.  Checked bit for bit against ba_gemm_softmax (caller-provided plan) on two calls in a row, the
second with a smaller batch, and against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi
from _util import assert_probs_close, dev_i64, make_plan, random_operands

pytestmark = pytest.mark.gpu


def both_ways(dev, M, N, K, H, dtype, scale, seed):
    M = np.asarray(M, np.int64); N = np.asarray(N, np.int64); K = np.asarray(K, np.int64)
    A, B = random_operands(M, N, K, H, dtype, seed)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    Ad, Bd = A.to(dev), B.to(dev)
    Md, Nd, Kd = dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev)
    plan = make_plan(dev, M, N, K, read=False)          # no host summary: the launches the static call makes
    want = torch.full((H, do), float("nan"), dtype=dtype, device=dev)
    capi.gemm_softmax(plan, Ad, Bd, want, H, d1, d2, do, scale)
    got = torch.full((H, do), float("nan"), dtype=dtype, device=dev)
    # one call first: the code object is loaded and the buffer's address looked up (once per device); then two calls
    # between which the DEVICE's free memory (hipMemGetInfo: whatever allocates, torch's allocator or the library
    # itself) must not move
    capi.gemm_softmax_static(Md, Nd, Kd, Ad, Bd, got, H, d1, d2, do, scale)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    before = torch.cuda.memory_allocated(dev)
    got.fill_(float("nan"))
    capi.gemm_softmax_static(Md, Nd, Kd, Ad, Bd, got, H, d1, d2, do, scale)
    capi.gemm_softmax_static(Md, Nd, Kd, Ad, Bd, got, H, d1, d2, do, scale)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before, "the device's free memory moved across the calls"
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "static plan and caller's plan disagree"
    assert_probs_close(got, oracle.per_segment_torch(A, B, M, N, K, scale), "static")
    return got


def test_two_calls_in_a_row_the_second_smaller(dev):
    rng = np.random.default_rng(5)
    n = 640                                                 # beyond the one-launch path: scheduler, plan buffer, kernels
    M = rng.integers(1, 90, n); N = rng.integers(1, 200, n); K = rng.choice(np.arange(8, 129, 8), n)
    N[7] = 700; M[7] = 150; K[7] = 136                   # one segment of the tile kernel (in every batch below)
    N[520] = 600; M[520] = 300; K[520] = 128             # and one of the pipelined row-block kernel (in the two large ones)
    both_ways(dev, M, N, K, 3, torch.bfloat16, 0.11, seed=1)
    both_ways(dev, M[:530], N[:530], K[:530], 2, torch.float16, 0.2, seed=2)   # smaller batch into the same buffer
    both_ways(dev, M[:40], N[:40], K[:40], 2, torch.float16, 0.2, seed=2)      # small enough for the single launch
    both_ways(dev, [5], [9], [16], 1, torch.float16, 1.0, seed=3)


def test_prefix_sums_are_written_and_the_limit_is_enforced(dev):
    M = np.array([33, 99, 64]); N = np.array([33, 99, 64]); K = np.array([64, 64, 64])
    A, B = random_operands(M, N, K, 2, torch.float16, 4)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    acc = [torch.zeros(4, dtype=torch.int64, device=dev) for _ in range(3)]
    out = torch.empty((2, do), dtype=torch.float16, device=dev)
    capi.gemm_softmax_static(dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev), A.to(dev), B.to(dev), out, 2, d1, d2,
                             do, 0.125, *acc)
    for got, ref in zip(acc, oracle.lists_to_accum(M, N, K)):
        assert np.array_equal(got.cpu().numpy(), ref)
    assert_probs_close(out, oracle.per_segment_torch(A, B, M, N, K, 0.125), "static, accum written")
    lib = capi.load()
    p = ctypes.c_void_p(out.data_ptr())
    too_many = capi.STATIC_MAX_SEGMENTS + 1
    assert lib.ba_gemm_softmax_static(too_many, 0, p, p, p, None, None, None, 0, p, p, p, 0, 1, 8, 8, 8, 1.0, None) == 2
    assert lib.ba_gemm_softmax_static(1, 0, p, p, p, None, None, None, 2, p, p, p, 2, 1, 8, 8, 8, 1.0, None) == 3
