"""Standalone blocked softmax (and its backward) through the C ABI against the oracle."""
import numpy as np
import pytest
import torch

import oracle
from blockedattention_amd import capi
from _util import assert_probs_close, dev_i64

pytestmark = pytest.mark.gpu


def run_softmax(dev, rows, cols, H, dtype, scale=1.0, seed=0, spread=3.0, accum=None):
    D = int((np.asarray(rows) * np.asarray(cols)).sum()) if accum is None else int(accum[-1])
    g = torch.Generator().manual_seed(seed)
    src = (torch.randn((H, D), generator=g) * spread).to(dtype)
    acc = None if accum is None else dev_i64(accum, dev)
    plan = capi.plan_softmax(len(rows), dev, dev_i64(rows, dev), dev_i64(cols, dev), acc, accum_given=accum is not None)
    info = plan.read()
    assert info.Dout == D
    out = torch.full((H, D), float("nan"), dtype=dtype, device=dev)
    capi.blocked_softmax(plan, src.to(dev), out, H, D, scale)
    return src, out, plan


def test_reference_live_check_shape(dev):
    # test/pytest.py:54-59: rows x cols = 33x64, 99x64, 64x64, H = 128, fp32, per-segment softmax(-1).
    rows, cols = [33, 99, 64], [64, 64, 64]
    src, out, _ = run_softmax(dev, rows, cols, 128, torch.float32, spread=1.0)
    ref = torch.cat([src[:, :2112].reshape(128, 33, 64).softmax(-1).reshape(128, -1),
                     src[:, 2112:8448].reshape(128, 99, 64).softmax(-1).reshape(128, -1),
                     src[:, 8448:].reshape(128, 64, 64).softmax(-1).reshape(128, -1)], -1)
    assert (out.cpu() - ref).abs().mean().item() < 1e-8
    torch.testing.assert_close(out.cpu(), ref, rtol=1e-5, atol=1e-7)


def test_long_rows_127x2047_half(dev):
    # csrc/sparseBlockedAttention.cpp:265-284: 3 segments of 127 x 2047, H = 7, half.
    rows, cols = [127] * 3, [2047] * 3
    src, out, _ = run_softmax(dev, rows, cols, 7, torch.float16, spread=2.0)
    assert_probs_close(out, oracle.per_segment_torch_softmax(src, rows, cols), "127x2047")
    sums = out.float().cpu().reshape(7, 3 * 127, 2047).sum(-1)
    torch.testing.assert_close(sums, torch.ones_like(sums), rtol=0, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_mixed_widths_scale_and_no_column_limit(dev, dtype):
    rows = [3, 5, 0, 2, 4, 1]; cols = [1, 63, 12, 1025, 9000, 64]       # 9000 > the reference's 8191 limit
    for scale in (1.0, 0.125, -0.7, 0.0):
        src, out, _ = run_softmax(dev, rows, cols, 2, dtype, scale=scale, seed=4)
        assert_probs_close(out, oracle.per_segment_torch_softmax(src, rows, cols, scale), f"scale {scale}")


def test_in_place_and_gapped_prefix_sum(dev):
    rows, cols, accum = [2, 3], [5, 1100], [0, 16, 16 + 3300]
    src, out, plan = run_softmax(dev, rows, cols, 2, torch.float16, accum=accum)
    buf = src.to(dev).clone()
    capi.blocked_softmax(plan, buf, buf, 2, accum[-1], 1.0)
    assert torch.equal(buf[:, :10], out[:, :10]) and torch.equal(buf[:, 16:], out[:, 16:])
    assert torch.equal(buf[:, 10:16].cpu(), src[:, 10:16])              # the gap is untouched
    ref = oracle.blocked_softmax(src.float().numpy(), rows, cols, 1.0, accum=accum)
    assert np.abs(out.float().cpu().numpy()[:, :10] - ref[:, :10]).max() < 1e-3
    assert np.abs(out.float().cpu().numpy()[:, 16:] - ref[:, 16:]).max() < 1e-3


def test_in_place_rows_wider_than_the_register_path(dev):
    # 4613 = 9 * 512 + 5: the last step's run reaches back into columns the step before has already written.
    rows, cols = [3, 2, 5], [4613, 513, 8200]
    for dtype in (torch.float16, torch.float32):
        src, out, plan = run_softmax(dev, rows, cols, 2, dtype, scale=0.3, seed=5)
        buf = src.to(dev).clone()
        capi.blocked_softmax(plan, buf, buf, 2, src.shape[1], 0.3)
        assert torch.equal(buf, out)
        assert_probs_close(out, oracle.per_segment_torch_softmax(src, rows, cols, 0.3), "wide in place")


def test_all_neg_inf_row_is_nan_like_torch(dev):
    x = torch.tensor([[float("-inf")] * 4 + [0.0, float("-inf"), 1.0, 2.0]], dtype=torch.float32)
    plan = capi.plan_softmax(1, dev, dev_i64([2], dev), dev_i64([4], dev))
    plan.read()
    out = torch.empty((1, 8), dtype=torch.float32, device=dev)
    capi.blocked_softmax(plan, x.to(dev), out, 1, 8, 1.0)
    ref = torch.softmax(x.reshape(2, 4), -1).reshape(1, 8)
    assert torch.isnan(out[0, :4]).all() and torch.isnan(ref[0, :4]).all()
    torch.testing.assert_close(out[0, 4:].cpu(), ref[0, 4:])


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_backward_matches_oracle(dev, dtype):
    rows, cols = [33, 4, 2], [64, 7, 1500]
    src, y, plan = run_softmax(dev, rows, cols, 3, dtype, scale=0.5, seed=8)
    g = torch.Generator().manual_seed(9)
    dy = torch.randn(y.shape, generator=g).to(dtype)
    dx = torch.empty_like(y)
    capi.blocked_softmax_backward(plan, y, dy.to(dev), dx, 3, y.shape[1], 0.5)
    ref = oracle.blocked_softmax_backward(y.float().cpu().numpy(), dy.float().numpy(), rows, cols, 0.5)
    tol = 2e-3 if dtype == torch.float16 else 1e-6
    assert np.abs(dx.float().cpu().numpy() - ref).max() <= tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_backward_wide_ragged_rows_and_in_place(dev, dtype):
    # row lengths around the 512-column steps (remainders 1, 5, 511, 0) and past the 4096-column register path
    rows, cols = [2, 3, 1, 2, 2], [513, 4613, 1023, 1024, 300]
    src, y, plan = run_softmax(dev, rows, cols, 2, dtype, scale=1.0, seed=11)
    g = torch.Generator().manual_seed(12)
    dy = torch.randn(y.shape, generator=g).to(dtype)
    dx = torch.empty_like(y)
    capi.blocked_softmax_backward(plan, y, dy.to(dev), dx, 2, y.shape[1], 1.0)
    ref = oracle.blocked_softmax_backward(y.float().cpu().numpy(), dy.float().numpy(), rows, cols, 1.0)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-6
    assert np.abs(dx.float().cpu().numpy() - ref).max() <= tol
    buf = dy.to(dev).clone()                                   # dx written over dy
    capi.blocked_softmax_backward(plan, y, buf, buf, 2, y.shape[1], 1.0)
    assert torch.equal(buf, dx)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_backward_rows_held_in_registers(dev, dtype):
    # one row length per count of 512-column steps (1..8: both inputs of a row are read once and kept in registers;
    # fp32 up to 2048 columns, the wider rows streamed twice), odd lengths, and without the host summary, so that a
    # wavefront takes several rows one after the other (the next row's loads under the current row's arithmetic)
    rows = [37] * 8 + [5]
    cols = [301, 777, 1283, 2048, 2049, 2901, 3583, 4096, 4100]
    H = 2
    src, y, plan = run_softmax(dev, rows, cols, H, dtype, scale=0.7, seed=21)
    g = torch.Generator().manual_seed(22)
    dy = torch.randn(y.shape, generator=g).to(dtype)
    ref = oracle.blocked_softmax_backward(y.float().cpu().numpy(), dy.float().numpy(), rows, cols, 0.7)
    tol = {torch.float16: 2e-3, torch.bfloat16: 2e-2, torch.float32: 1e-6}[dtype]
    for with_summary in (True, False):
        if not with_summary:
            plan.info = None
        dx = torch.full_like(y, float("nan"))
        capi.blocked_softmax_backward(plan, y, dy.to(dev), dx, H, y.shape[1], 0.7)
        assert np.abs(dx.float().cpu().numpy() - ref).max() <= tol, f"summary {with_summary}"
        buf = y.clone()                                        # dx written over y
        capi.blocked_softmax_backward(plan, buf, dy.to(dev), buf, H, y.shape[1], 0.7)
        assert torch.equal(buf, dx)

