"""Drop-in name of the reference's compiled module (setup.py:16 there): re-exports the in-tree extension."""
from blockedattention_amd.blockAttention import (  # noqa: F401
    sparseBlockedGEMM, sparseBlockedGEMMSoftmax, sparseBlockedSoftmax, sparseBlockedSoftmaxScaled)
