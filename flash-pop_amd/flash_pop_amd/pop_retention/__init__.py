"""flash_pop_retention(q, k, v, s, head_decays, block_size) -> (o, block_states)

Same call signature and returns as the reference's FlashPOPRetention
(flash_pop/pop_retention/__init__.py:11-52): block_states is [B, T // block_size, H, dk, dv],
the recurrent state after every full block; there is no final-state output.  The block size
is kept on the autograd context, so T need not be a multiple of it in the backward pass
(the reference re-derives it as T // num_blocks, pop_retention/__init__.py:39-40).

flash_pop_retention_with_suffixes(q, k, v, s, head_decays, block_size, q_sfx, k_sfx, v_sfx)
    -> (o, o_sfx, last_state)

One POP layer step in a single walk: what POPDecoderLayer.pop_forward obtains from
flash_pop_retention followed by fused_chunk_retention on the suffix batch seeded with
[s, block_states] (flash_pop/pop_retnet.py:107-171), without writing the block states, reading
them back or concatenating them.  q_sfx, k_sfx, v_sfx are [B * (N + 1), Ls, H, d] with the block
index fastest (N = T // block_size, any Ls >= 1); last_state is the state after the last full
block, the reference's `states[:, -1]`.  Tokens after the last block boundary (T % block_size of
them) are context like any others; no suffix follows them.
"""
import torch

from .. import _ops


class FlashPOPRetention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, s, head_decays, block_size):
        block_size = int(block_size)
        assert block_size >= 1, f"block_size must be positive, got {block_size}"
        q, k, v, s, shape = _ops.prepare(q, k, v, s, head_decays)
        o, states = _ops.pop_retention_fwd(q, k, v, s, head_decays, block_size, shape)
        ctx.save_for_backward(q, k, v, s)
        ctx.set_materialize_grads(False)   # an output nobody differentiates arrives as None, not as a tensor of zeros
        ctx.head_decays = tuple(head_decays)
        ctx.shape = shape
        ctx.block_size = block_size
        return o, states

    @staticmethod
    def backward(ctx, d_o, d_block_states):
        q, k, v, s = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros((*q.shape[:3], v.shape[3]), dtype=q.dtype, device=q.device)
        want_ds0 = s is not None and ctx.needs_input_grad[3]
        dq, dk, dv, d_s0 = _ops.retention_bwd(q, k, v, s, ctx.head_decays, ctx.shape, d_o, None, d_block_states,
                                              ctx.block_size, want_ds0)
        return dq, dk, dv, d_s0, None, None


flash_pop_retention = FlashPOPRetention.apply


class FlashPOPRetentionWithSuffixes(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, s, head_decays, block_size, q_sfx, k_sfx, v_sfx):
        block_size = int(block_size)
        assert block_size >= 1, f"block_size must be positive, got {block_size}"
        q, k, v, s, shape = _ops.prepare(q, k, v, s, head_decays)
        sfx = _ops.prepare_suffixes(q_sfx, k_sfx, v_sfx, shape, block_size)
        o, o_sfx, last_state = _ops.pop_fused_fwd(q, k, v, s, sfx, head_decays, block_size, shape)
        ctx.save_for_backward(q, k, v, s, *sfx)
        ctx.set_materialize_grads(False)   # an output nobody differentiates arrives as None, not as a tensor of zeros
        ctx.head_decays = tuple(head_decays)
        ctx.shape = shape
        ctx.block_size = block_size
        return o, o_sfx, last_state

    @staticmethod
    def backward(ctx, d_o, d_o_sfx, d_last_state):
        q, k, v, s, *sfx = ctx.saved_tensors
        if d_o is None:
            d_o = torch.zeros((*q.shape[:3], v.shape[3]), dtype=q.dtype, device=q.device)
        if d_o_sfx is None:
            d_o_sfx = torch.zeros((*sfx[0].shape[:3], v.shape[3]), dtype=q.dtype, device=q.device)
        want_ds0 = s is not None and ctx.needs_input_grad[3]
        (dq, dk, dv, dq_s, dk_s, dv_s), d_s0 = _ops.pop_fused_bwd(q, k, v, s, sfx, ctx.head_decays, ctx.block_size,
                                                                   ctx.shape, d_o, d_o_sfx, d_last_state, want_ds0)
        return dq, dk, dv, d_s0, None, None, dq_s, dk_s, dv_s


flash_pop_retention_with_suffixes = FlashPOPRetentionWithSuffixes.apply
