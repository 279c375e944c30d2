"""MI355X-native varlen ("blocked") GEMM and blocked row softmax.

``blockGEMM`` / ``blockSoftmax`` keep the reference package's signatures;
``blockGEMMSoftmax`` is the fused pair, ``blockFusedAttention`` the one-pass
``softmax(scale q k^T) v``.  ``capi`` exposes the C ABI directly.
Importing the operators needs the in-tree build (``python -m
blockedattention_amd.build``); nothing falls back to PyTorch or the CPU.
"""

__all__ = ["blockGEMM", "blockSoftmax", "blockGEMMSoftmax", "blockFusedAttention", "set_schedule_cache", "schedule_cache_stats"]


def __getattr__(name):
    # The operators pull in the compiled extension; keep `import
    # blockedattention_amd.workloads` (numpy/torch only) usable without it.
    if name in __all__:
        from . import apply
        return getattr(apply, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
