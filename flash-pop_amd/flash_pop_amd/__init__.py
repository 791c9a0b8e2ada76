"""MI355X-native drop-in for flash-pop's retention operators (HIP kernels behind a C ABI)."""
from .fused_retention import fused_chunk_retention, FusedChunkRetention  # noqa: F401
from .pop_retention import (  # noqa: F401
    flash_pop_retention, FlashPOPRetention, flash_pop_retention_with_suffixes, FlashPOPRetentionWithSuffixes)
from .recurrent import retention_recurrent  # noqa: F401
from .xpos_emb import XPos  # noqa: F401
from .gated_norm import gated_group_norm  # noqa: F401

__all__ = ["XPos", "gated_group_norm", "retention_recurrent", "fused_chunk_retention", "flash_pop_retention", "flash_pop_retention_with_suffixes",
           "FusedChunkRetention", "FlashPOPRetention", "FlashPOPRetentionWithSuffixes"]
