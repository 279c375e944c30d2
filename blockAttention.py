"""Drop-in name of the reference's compiled module (setup.py:16 there): re-exports the in-tree extension."""
from blockedattention_amd.blockAttention import (  # noqa: F401
    schedule_cache_stats, set_schedule_cache, sparseBlockedAttention, sparseBlockedGEMM, sparseBlockedGEMMSoftmax,
    sparseBlockedSoftmax, sparseBlockedSoftmaxScaled)
