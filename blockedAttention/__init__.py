"""Drop-in name of the reference package: ``import blockedAttention`` keeps working."""
from blockedattention_amd.apply import (blockFusedAttention, blockGEMM, blockGEMMSoftmax, blockSoftmax,
                                        schedule_cache_stats, set_schedule_cache)

__all__ = ["blockGEMM", "blockSoftmax", "blockGEMMSoftmax", "blockFusedAttention", "set_schedule_cache", "schedule_cache_stats"]
