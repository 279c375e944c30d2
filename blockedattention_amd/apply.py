"""Python surface of the operators: the reference's ``blockGEMM`` and
``blockSoftmax`` (blockedAttention/apply.py:6-41) with identical names,
argument order and defaults, plus the fused pair.

All three forward to the compiled extension ``blockAttention`` (built in-tree
by ``python -m blockedattention_amd.build``); there is no Python or CPU
fallback.  The reference wrapper passes ``srcAccum`` to the extension in the
wrong position (apply.py:41 against csrc/sparseBlockedAttention.cpp:127-128);
here the call follows the extension's order, so ``blockSoftmax(x, rows, cols)``
works as documented.
"""
from typing import Optional

import torch

from . import blockAttention


def blockGEMM(
    mat1: torch.Tensor, mat2: torch.Tensor,
    mat1Accum: Optional[torch.Tensor] = None, mat2Accum: Optional[torch.Tensor] = None,
    outAccum: Optional[torch.Tensor] = None,
    MList: Optional[torch.Tensor] = None, NList: Optional[torch.Tensor] = None, KList: Optional[torch.Tensor] = None,
    transpose1: Optional[bool] = False, transpose2: Optional[bool] = False,
) -> torch.Tensor:
    """Varlen GEMM ``out_g = A_g @ B_g^T`` over segments stored back to back.

    ``mat1`` is ``[H, sum(M_g*K_g)]``, ``mat2`` is ``[H, sum(N_g*K_g)]`` and the
    result ``[H, sum(M_g*N_g)]``; segment ``g`` is row-major ``M_g x K_g``
    (``K_g x M_g`` with ``transpose1``), ``N_g x K_g`` (``K_g x N_g`` with
    ``transpose2``) and ``M_g x N_g``.  Give either the three exclusive prefix
    sums (int64, one more entry than segments) or the three size lists (int64),
    or both.
    """
    return blockAttention.sparseBlockedGEMM(mat1, mat2, mat1Accum, mat2Accum, outAccum, MList, NList, KList,
                                            bool(transpose1), bool(transpose2))


def blockSoftmax(
    src: torch.Tensor,
    rowList: torch.Tensor, colList: torch.Tensor, srcAccum: Optional[torch.Tensor] = None,
    scale: float = 1.0,
) -> torch.Tensor:
    """Row softmax inside every ``rowList[g] x colList[g]`` block of ``src`` (``[H, sum(rows*cols)]``).

    ``srcAccum`` (the exclusive prefix sum of ``rows*cols``) is optional.
    ``scale`` multiplies the input first; the default 1.0 is the reference's
    behaviour.
    """
    if scale == 1.0:
        return blockAttention.sparseBlockedSoftmax(src, rowList, colList, srcAccum)
    return blockAttention.sparseBlockedSoftmaxScaled(src, rowList, colList, srcAccum, float(scale))


def blockGEMMSoftmax(
    mat1: torch.Tensor, mat2: torch.Tensor,
    mat1Accum: Optional[torch.Tensor] = None, mat2Accum: Optional[torch.Tensor] = None,
    outAccum: Optional[torch.Tensor] = None,
    MList: Optional[torch.Tensor] = None, NList: Optional[torch.Tensor] = None, KList: Optional[torch.Tensor] = None,
    scale: float = 1.0, out_fp32: bool = False,
) -> torch.Tensor:
    """Fused ``softmax(scale * A_g @ B_g^T)`` per segment (forward only).

    Same operands and metadata as ``blockGEMM`` (untransposed layouts); the
    scores stay in fp32 registers between the product and the softmax, so the
    result is what ``blockSoftmax(blockGEMM(...), MList, NList, scale=scale)``
    computes without the intermediate 16-bit rounding.
    """
    return blockAttention.sparseBlockedGEMMSoftmax(mat1, mat2, mat1Accum, mat2Accum, outAccum, MList, NList, KList,
                                                   float(scale), bool(out_fp32))


class _FusedAttention(torch.autograd.Function):
    """Forward: the one-pass kernel.  Backward: the probabilities are recomputed and the gradient taken through
    the operators the kernel replaces (dV = P^T dO and dP = dO V^T as two blockGEMM calls, dq and dk by the
    backward passes of blockSoftmax and blockGEMM), so only q, k and v are kept between the passes -- never an
    ``M x N`` array."""

    @staticmethod
    def forward(ctx, q, k, v, MList, NList, KList, mat1Accum, mat2Accum, outAccum, scale):
        out = blockAttention.sparseBlockedAttention(q, k, v, mat1Accum, mat2Accum, outAccum, MList, NList, KList,
                                                    scale)
        ctx.save_for_backward(q, k, v)
        ctx.meta = (MList, NList, KList, mat1Accum, mat2Accum, outAccum)
        ctx.scale = scale
        return out

    @staticmethod
    def backward(ctx, grad_out):
        q, k, v = ctx.saved_tensors
        MList, NList, KList, mat1Accum, mat2Accum, outAccum = ctx.meta
        if MList is None or NList is None or KList is None:
            raise RuntimeError("blockFusedAttention: the backward pass needs MList, NList and KList "
                               "(prefix sums alone do not describe the second product)")
        grad_out = grad_out.reshape(q.shape[:-1].numel(), -1).contiguous()
        with torch.enable_grad():
            qg, kg = (t.detach().requires_grad_(True) for t in (q, k))
            probs = blockSoftmax(blockGEMM(qg, kg, mat1Accum, mat2Accum, outAccum, MList, NList, KList),
                                 MList, NList, outAccum, scale=ctx.scale)
        with torch.no_grad():
            # dV_g = P_g^T dO_g: N x K, reduction over M, both operands stored reduction-major
            dv = blockGEMM(probs.detach(), grad_out, None, None, None, NList, KList, MList, True, True)
            # dP_g = dO_g V_g^T: M x N, reduction over K, both operands row-major
            dprobs = blockGEMM(grad_out, v.detach(), mat1Accum, mat2Accum, outAccum, MList, NList, KList)
        dq, dk = torch.autograd.grad(probs, (qg, kg), dprobs)
        return dq.view_as(q), dk.view_as(k), dv.view_as(v), None, None, None, None, None, None, None


def blockFusedAttention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
    MList: Optional[torch.Tensor] = None, NList: Optional[torch.Tensor] = None, KList: Optional[torch.Tensor] = None,
    mat1Accum: Optional[torch.Tensor] = None, mat2Accum: Optional[torch.Tensor] = None,
    outAccum: Optional[torch.Tensor] = None,
    scale: float = 1.0,
) -> torch.Tensor:
    """``softmax(scale * Q_g @ K_g^T) @ V_g`` per segment in one pass.

    ``q`` is ``[H, sum(M*K)]`` (the first operand of ``blockGEMM``), ``k`` and ``v`` are both
    ``[H, sum(N*K)]`` (its second operand's layout); the metadata is ``blockGEMM``'s.  The result,
    ``[H, sum(M*K)]``, is what ``blockGEMM(blockSoftmax(blockGEMM(q, k, ...), M, N, scale=scale), v, ...,
    transpose2=True)`` computes, without the ``M x N`` arrays ever reaching memory.  Head dimensions up
    to 128.  Differentiable in q, k and v when the size lists are given: the backward pass recomputes the
    probabilities and runs the backward of that chain.
    """
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return _FusedAttention.apply(q, k, v, MList, NList, KList, mat1Accum, mat2Accum, outAccum, float(scale))
    return blockAttention.sparseBlockedAttention(q, k, v, mat1Accum, mat2Accum, outAccum, MList, NList, KList,
                                                 float(scale))


def set_schedule_cache(capacity: int) -> None:
    """How many schedules the operators keep for metadata tensors they have seen (default 8; 0 = off).

    A call whose metadata tensors are the same objects, unmodified (PyTorch's version counters), as in an
    earlier call reuses that call's device-side plan and skips the scheduler and its host synchronisation.
    Turn it off only if metadata tensors are rewritten through raw pointers, which PyTorch cannot see."""
    blockAttention.set_schedule_cache(int(capacity))


def schedule_cache_stats() -> dict:
    hits, misses, entries, capacity = blockAttention.schedule_cache_stats()
    return {"hits": hits, "misses": misses, "entries": entries, "capacity": capacity}
