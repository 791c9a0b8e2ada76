"""MI355X-native drop-in for flash-pop's retention operators (HIP kernels behind a C ABI)."""
from .fused_retention import fused_chunk_retention, FusedChunkRetention  # noqa: F401
from .pop_retention import flash_pop_retention, FlashPOPRetention  # noqa: F401

__all__ = ["fused_chunk_retention", "flash_pop_retention", "FusedChunkRetention", "FlashPOPRetention"]
