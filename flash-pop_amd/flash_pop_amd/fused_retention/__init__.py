"""fused_chunk_retention(q, k, v, s, head_decays) -> (o, s_out)

Same call signature and returns as the reference's FusedChunkRetention
(flash_pop/fused_retention/__init__.py:10-67): q, k [B,T,H,dk], v [B,T,H,dv], s [B,H,dk,dv],
all bfloat16 on the GPU; head_decays a tuple of H Python floats.  K is divided by sqrt(dk)
inside.  Gradients flow to q, k, v and s.  `s` may also be None (zeros), a superset of the
reference, whose callers substitute zeros themselves (flash_pop/retnet.py:279-282).
"""
import torch

from .. import _ops


class FusedChunkRetention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, s, head_decays):
        q, k, v, s, shape = _ops.prepare(q, k, v, s, head_decays)
        # what the reference saves for its backward (fused_retention/__init__.py:30) plus, where it
        # pays, the states the forward passes through every few chunks
        o, s_out, ckpt, every = _ops.retention_fwd(q, k, v, s, head_decays, shape, for_backward=any(ctx.needs_input_grad[:4]))
        ctx.save_for_backward(q, k, v, s, ckpt)
        ctx.set_materialize_grads(False)   # an output nobody differentiates arrives as None, not as a tensor of zeros
        ctx.every = every
        ctx.workspace_spent = False
        ctx.head_decays = tuple(head_decays)
        ctx.shape = shape
        return o, s_out

    @staticmethod
    def backward(ctx, d_o, d_s_out):
        q, k, v, s, ckpt = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros((*q.shape[:3], v.shape[3]), dtype=q.dtype, device=q.device)
        want_ds0 = s is not None and ctx.needs_input_grad[3]
        # a forward that cut its sequences leaves its workspace (ctx.every == 0): the first backward
        # starts from the states in it and overwrites them, a second one (retain_graph) recomputes them
        kept = ckpt is not None and ctx.every == 0
        dq, dk, dv, d_s0 = _ops.retention_bwd(q, k, v, s, ctx.head_decays, ctx.shape, d_o, d_s_out, None, None, want_ds0,
                                              ckpt, ctx.every, states_kept=kept and not ctx.workspace_spent)
        ctx.workspace_spent = ctx.workspace_spent or kept
        return dq, dk, dv, d_s0, None


fused_chunk_retention = FusedChunkRetention.apply
