"""retention_recurrent(query, key, value, head_decays, prev_state) -> (retention, state)

One decode step for all heads in one kernel launch, in place of the einsums of the reference's
retention_recurrent (flash_pop/retnet.py:79-101): state = prev_state * gamma + (key / sqrt(dk))^T
value, retention = query . state.  query, key [B,H,dk], value [B,H,dv], prev_state [B,H,dk,dv] or
None; bf16 CUDA tensors.  head_decays is the tuple of H floats the other ops take (the reference
passes the same numbers as a [1,H,1,1] tensor).  Inference only: no autograd graph is recorded.
With in_place=True the new state overwrites prev_state (no second state buffer, half the
allocations of a decode loop)."""
import torch

from .. import _ops


@torch.no_grad()
def retention_recurrent(query, key, value, head_decays, prev_state, in_place=False):
    if isinstance(head_decays, torch.Tensor):
        head_decays = tuple(head_decays.flatten().tolist())
    return _ops.decode_step(query, key, value, prev_state, head_decays, in_place)
