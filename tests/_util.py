"""Helpers shared by the GPU parity tests: run the C ABI on seeded inputs and
compare with the oracle.  Tolerances follow the build's contract:

* scores: |x - ref| <= 1e-2 * |ref| + 4 u rms(ref), u = 2^-11 (fp16) or 2^-9 (bf16): the relative bound the
  contract states plus a few output ulps of the segment's score scale for values near zero
  (fp32 accumulate, one 16-bit rounding)
* probabilities, fp16 / fp32 output: |p - ref| <= 1e-3
* probabilities, bf16 output: one bf16 rounding of a value in [0.5, 1) is already
  2^-9 = 1.95e-3, so the bound is |p - ref| <= 1e-3 + 2^-8 * ref (half an ulp
  relative plus margin); the tests also report the error against the
  bf16-rounded oracle.
"""
import numpy as np
import torch

import oracle
from blockedattention_amd import capi


def dev_i64(a, dev):
    return torch.as_tensor(np.asarray(a, dtype=np.int64)).to(dev)


def make_plan(dev, M, N, K, read=True):
    B = len(M)
    Md, Nd, Kd = dev_i64(M, dev), dev_i64(N, dev), dev_i64(K, dev)
    a1 = torch.empty(B + 1, dtype=torch.int64, device=dev); a2 = torch.empty_like(a1); ao = torch.empty_like(a1)
    plan = capi.plan_gemm(B, dev, Md, Nd, Kd, a1, a2, ao, mode=capi.META_FROM_LISTS)
    if read:
        plan.read()
    plan.keep = (Md, Nd, Kd, a1, a2, ao)
    return plan


def random_operands(M, N, K, H, dtype, seed=0, dist="normal", sigma=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    d1 = int((np.asarray(M) * np.asarray(K)).sum()); d2 = int((np.asarray(N) * np.asarray(K)).sum())
    if dist == "normal":
        A = torch.randn((H, d1), generator=g) * sigma; B = torch.randn((H, d2), generator=g) * sigma
    else:
        A = torch.rand((H, d1), generator=g) * 2 - 1; B = torch.rand((H, d2), generator=g) * 2 - 1
    return A.to(dtype), B.to(dtype)


def score_atol(dtype, ref):
    """A few output ulps of the score scale: 4 u rms(ref)."""
    u = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -9}.get(dtype, 2.0 ** -20)
    rms = float(ref.float().pow(2).mean().sqrt()) if ref.numel() else 0.0
    return 4 * u * rms


def assert_scores_close(got, ref, what=""):
    atol = score_atol(got.dtype, ref)
    got = got.float().cpu(); ref = ref.float()
    assert not torch.isnan(got).any(), f"{what}: NaN in scores"
    err = (got - ref).abs() - (1e-2 * ref.abs() + atol)
    assert err.numel() == 0 or err.max().item() <= 0, f"{what}: scores off by {float((got - ref).abs().max())}"


def assert_probs_close(got, ref, what=""):
    dtype = got.dtype
    got = got.float().cpu(); ref = ref.float()
    assert not torch.isnan(got).any(), f"{what}: NaN in probabilities"
    if got.numel() == 0:
        return
    diff = (got - ref).abs()
    if dtype == torch.bfloat16:
        bound = 1e-3 + ref * 2.0 ** -8
        assert (diff <= bound).all(), f"{what}: bf16 probabilities off by {float(diff.max())}"
        vs_rounded = (got - ref.to(torch.bfloat16).float()).abs()
        ulp = torch.maximum(ref, torch.tensor(1e-30)) * 2.0 ** -7
        assert (vs_rounded <= ulp + 1e-6).all(), f"{what}: more than one bf16 ulp from the rounded oracle"
    else:
        assert diff.max().item() <= 1e-3, f"{what}: probabilities off by {float(diff.max())}"


def run_all(dev, M, N, K, H, dtype, scale, seed=0, dist="normal", sigma=1.0, check_gemm=True, check_softmax=True,
            summary=True):
    """GEMM, fused pair and standalone softmax through the C ABI against the oracle.

    summary=False: the launches get no host copy of the plan summary (nothing was read back between the
    scheduler and the kernels): grids are sized by the segment count alone and the kernels take the list
    lengths from the plan on the device."""
    M = np.asarray(M, np.int64); N = np.asarray(N, np.int64); K = np.asarray(K, np.int64)
    A, B = random_operands(M, N, K, H, dtype, seed, dist, sigma)
    plan = make_plan(dev, M, N, K, read=summary)
    d1, d2, do = int((M * K).sum()), int((N * K).sum()), int((M * N).sum())
    if summary:
        assert (plan.info.Dm1, plan.info.Dm2, plan.info.Dout) == (d1, d2, do)
    sc, pr = oracle.per_segment_torch(A, B, M, N, K, scale, want="both")
    Ad, Bd = A.to(dev), B.to(dev)
    out = torch.full((H, do), float("nan"), dtype=dtype, device=dev)
    if check_gemm:
        capi.varlen_gemm(plan, Ad, Bd, out, H, d1, d2, do)
        assert_scores_close(out, sc, "gemm")
    fused = torch.full((H, do), float("nan"), dtype=dtype, device=dev)
    capi.gemm_softmax(plan, Ad, Bd, fused, H, d1, d2, do, scale)
    assert_probs_close(fused, pr, "fused")
    if check_gemm and check_softmax:
        sm = torch.full((H, do), float("nan"), dtype=dtype, device=dev)
        capi.blocked_softmax(plan, out, sm, H, do, scale)
        assert_probs_close(sm, oracle.per_segment_torch_softmax(out.cpu(), M, N, scale), "softmax")
    assert plan.info is not None or not summary
    info = plan.read()
    assert info.run_errors == 0 and (info.Dm1, info.Dm2, info.Dout) == (d1, d2, do)
    return plan
