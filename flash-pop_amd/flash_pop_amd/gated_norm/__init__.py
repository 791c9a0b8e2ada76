"""gated_group_norm(retention, gate, eps=1e-6) -> bf16(GroupNorm_per_head(retention)) * bf16(swish(gate))

The step between the retention op and the output projection in the reference's layer
(flash_pop/retnet.py:294-309): GroupNorm with one group per head, computed in fp32, no affine
parameters (retnet.py:194-201), rounded to bf16, times swish(g_proj(x)) -- in one HIP launch
with the reference's rounding points.  retention [..., H, dv] (the op's output), gate [..., H*dv]
(the output of g_proj before the activation); returns [..., H*dv].  bfloat16 on the GPU;
dv = 8 * 2^k <= 512.  Gradients flow to both inputs (one launch).
"""
import torch

from .. import _ops


class GatedGroupNorm(torch.autograd.Function):

    @staticmethod
    def forward(ctx, retention, gate, eps):
        retention, gate = retention.contiguous(), gate.contiguous()
        ctx.save_for_backward(retention, gate)
        ctx.eps = eps
        return _ops.gated_norm_fwd(retention, gate, eps)

    @staticmethod
    def backward(ctx, d_out):
        retention, gate = ctx.saved_tensors
        d_r, d_g = _ops.gated_norm_bwd(retention, gate, d_out, ctx.eps)
        return d_r, d_g, None


def gated_group_norm(retention, gate, eps: float = 1e-6):
    return GatedGroupNorm.apply(retention, gate, eps)
