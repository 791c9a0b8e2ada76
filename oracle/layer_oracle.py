"""CPU restatement of the two elementwise stages around the retention op.  TEST INFRASTRUCTURE ONLY
(same rules as retention_oracle.py: imported by tests/, the smoke entry and the benchmark's checker
legs, never by the shipped package).

  * flash_pop/xpos_emb.py:11-29    per-pair frequencies                          -> position_thetas
  * flash_pop/xpos_emb.py:32-40,42-75,120-126  x cos + (i x) sin at position * theta -> rotary
  * flash_pop/retnet.py:194-201,294-309  GroupNorm per head (fp32, no affine) -> dtype, times
    swish(g_proj(x))                                                              -> gated_group_norm

Conventions carried over: features come in adjacent pairs (x[2i], x[2i+1]) that share theta_i
(the reference repeats each theta twice, xpos_emb.py:29); angles are float32 products of the
integer position and theta (xpos_emb.py:69), sines and cosines float32; the normalised values
are rounded to the working dtype before the gate multiplies them, and the gate activation is
evaluated in the working dtype (retnet.py:297,308-309).

Pinning status (tests/test_oracle.py): rotary against complex multiplication by exp(i pos theta)
in float64, the identity at position 0, a quarter turn, norm preservation, additivity of
positions and the relative-position property of the q.k scores; gated_group_norm against
torch.nn.functional.group_norm and silu (the library routines the reference itself calls) and
against zero-mean / unit-variance and shift / scale invariance of the normalised part.
"""
from __future__ import annotations

import torch
from torch import Tensor


def position_thetas(head_dim: int, scale: float = 10000.0) -> Tensor:
    """theta_i = scale^(-i / (d/2 - 1)), i = 0 .. d/2 - 1, float32 (xpos_emb.py:26-28, one per pair)."""
    x = torch.linspace(0, 1, steps=head_dim // 2)
    return 1 / (scale ** x)


def rotary(x: Tensor, positions: Tensor, thetas: Tensor, inverse: bool = False) -> Tensor:
    """x [B, T, H, d]; positions integer, broadcastable to [B, T]; thetas [d/2].
    out = x cos + (i x) sin with (i x)[2j] = -x[2j+1], (i x)[2j+1] = x[2j] (xpos_emb.py:33-40)."""
    B, T = x.shape[:2]
    pos = torch.broadcast_to(positions, (B, T)).reshape(B, T, 1, 1)
    th = thetas.float().repeat_interleave(2).reshape(1, 1, 1, -1)
    angles = pos * th                                       # integer * float32 -> float32 (xpos_emb.py:69)
    sin, cos = torch.sin(angles), torch.cos(angles)
    if inverse:
        sin = -sin
    xf = x.float()
    ix = torch.stack((-xf[..., 1::2], xf[..., 0::2]), dim=-1).flatten(start_dim=-2)
    return (xf * cos + ix * sin).to(x.dtype)


def gated_group_norm(r: Tensor, g: Tensor, eps: float = 1e-6) -> Tensor:
    """r [..., H, dv] retention output, g [..., H*dv] gate pre-activation, both in the working dtype.
    n = ((r - mean) / sqrt(var + eps)) per (row, head) in float32, biased variance, -> dtype;
    out = n * swish(g) evaluated in the working dtype (retnet.py:297,308-309)."""
    rf = r.float()
    mean = rf.mean(dim=-1, keepdim=True)
    var = ((rf - mean) ** 2).mean(dim=-1, keepdim=True)
    n = ((rf - mean) / torch.sqrt(var + eps)).to(r.dtype).flatten(start_dim=-2)
    gate = (g.float() * torch.sigmoid(g.float())).to(g.dtype)
    return n * gate
