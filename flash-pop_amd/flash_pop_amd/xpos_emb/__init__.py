"""XPos(head_dim_qk)(q, k, start_idx) -> (q, k)

The rotary position embedding the reference's layer applies to q and k right before the
retention op (flash_pop/xpos_emb.py:78-126, called at flash_pop/retnet.py:273-278), as one HIP
launch for both tensors instead of a chain of elementwise kernels: pairs (x[2i], x[2i+1]) of
every head are rotated by float(position) * theta_i, theta_i = 1 / 10000^(i / (d/2 - 1))
(xpos_emb.py:26-28).  q, k [B,T,H,d] bfloat16 on the GPU; start_idx is an int (position of the
first token of every sequence) or a LongTensor with one start position per sequence, as in the
reference (xpos_emb.py:50-66).  Sines and cosines are computed in the kernel, so there is no
cache to grow or invalidate.  Gradients flow to q and k (the rotation by the negative angle).
"""
import torch

from .. import _ops


def position_thetas(head_dim: int, scale: float = 10000.0) -> torch.Tensor:
    """d/2 fp32 frequencies, one per rotation pair (flash_pop/xpos_emb.py:26-28 before the repeat)."""
    return 1 / (scale ** torch.linspace(0, 1, steps=head_dim // 2))


class RotaryQK(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, theta, start_idx):
        ctx.theta, ctx.start = theta, start_idx
        return _ops.rotary_qk(q, k, theta, start_idx)

    @staticmethod
    def backward(ctx, d_q, d_k):
        d_q, d_k = _ops.rotary_qk(d_q, d_k, ctx.theta, ctx.start, inverse=True)
        return d_q, d_k, None, None


class XPos:

    def __init__(self, head_dim_qk: int, seq_len_estimate: int = 2 ** 12, start_idx=0, device=None, dtype=None) -> None:
        # seq_len_estimate, start_idx and dtype size the reference's sin/cos cache; nothing is cached here
        assert head_dim_qk % 8 == 0, f"head_dim_qk must be a multiple of 8, got {head_dim_qk}"
        self.head_dim = head_dim_qk
        self.thetas = position_thetas(head_dim_qk)
        self._on_device = {}

    def _theta(self, device):
        if device not in self._on_device:
            self._on_device[device] = self.thetas.to(device)
        return self._on_device[device]

    def __call__(self, q, k, start_idx, *args, **kwargs):
        assert q.shape[-1] == self.head_dim, f"built for head dimension {self.head_dim}, got {q.shape[-1]}"
        return RotaryQK.apply(q, k, self._theta(q.device), start_idx)
