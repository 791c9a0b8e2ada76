"""CPU oracle for the retention hot path.  Test infrastructure: imported only by tests/,
__graft_entry__.smoke() and the cpu_baseline leg of bench.py, never by the shipped package."""
from .retention_oracle import (  # noqa: F401
    head_decays,
    decay_mask,
    retention_chunk,
    chunkwise_retention,
    pop_retention,
    retention_chunk_grads,
    recurrent_step,
    pop_suffix_retention,
    pop_fused_retention,
    rms_error_ratio,
)
from .layer_oracle import position_thetas, rotary, gated_group_norm  # noqa: F401
