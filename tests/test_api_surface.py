"""The Python surface keeps the reference's names, argument order and defaults
(blockedAttention/apply.py:6-11, 27-30; csrc/sparseBlockedAttention.cpp:118-136)."""
import inspect

import pytest
import torch


def test_drop_in_names_import():
    import blockAttention
    import blockedAttention
    assert blockedAttention.__all__[:2] == ["blockGEMM", "blockSoftmax"]
    for op in ("sparseBlockedGEMM", "sparseBlockedSoftmax"):
        assert callable(getattr(blockAttention, op))


def test_block_gemm_signature():
    import blockedAttention
    sig = inspect.signature(blockedAttention.blockGEMM)
    assert list(sig.parameters) == ["mat1", "mat2", "mat1Accum", "mat2Accum", "outAccum", "MList", "NList", "KList",
                                    "transpose1", "transpose2"]
    defaults = [p.default for p in sig.parameters.values()]
    assert defaults == [inspect.Parameter.empty] * 2 + [None] * 6 + [False, False]


def test_block_softmax_signature():
    import blockedAttention
    sig = inspect.signature(blockedAttention.blockSoftmax)
    assert list(sig.parameters)[:4] == ["src", "rowList", "colList", "srcAccum"]
    assert sig.parameters["srcAccum"].default is None
    extra = list(sig.parameters.values())[4:]
    assert all(p.default is not inspect.Parameter.empty for p in extra)     # additions are optional
    assert sig.parameters["scale"].default == 1.0


def test_extension_ops_take_none_for_optional_tensors_and_reject_cpu_tensors():
    import blockAttention
    lists = [torch.tensor([1]), torch.tensor([1]), torch.tensor([4])]
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        blockAttention.sparseBlockedGEMM(torch.zeros(1, 4), torch.zeros(1, 4), None, None, None, *lists, False, False)
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        blockAttention.sparseBlockedSoftmax(torch.zeros(1, 4), lists[0], lists[2], None)
    with pytest.raises(RuntimeError, match="rowList and colList"):
        blockAttention.sparseBlockedSoftmax(torch.zeros(1, 4), None, None, None)
