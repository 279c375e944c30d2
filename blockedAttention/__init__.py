"""Drop-in name of the reference package: ``import blockedAttention`` keeps working."""
from blockedattention_amd.apply import blockGEMM, blockGEMMSoftmax, blockSoftmax

__all__ = ["blockGEMM", "blockSoftmax", "blockGEMMSoftmax"]
