"""disagmoe/utils/constants.py:20-22 of the reference: the expert batch below which ``MoEExperts`` uses its static buffers."""
from disagmoe_amd.models.experts import MAX_BATCH_SIZE

__all__ = ["MAX_BATCH_SIZE"]
