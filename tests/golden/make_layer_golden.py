"""Writes tests/golden/layer_golden.npz: seeded bf16-representable inputs of the two elementwise
stages around the retention op, with outputs and gradients evaluated in float64 from formulations
that share no code with the oracle: the rotation as a complex multiplication by exp(i pos theta),
its gradient as the multiplication by the conjugate; the normalisation through
torch.nn.functional.group_norm and silu in float64 with autograd.  No reference import.

    python tests/golden/make_layer_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
B, T, H, D, DV = 3, 40, 2, 32, 64
START = (0, 1000, 77)      # first position of each sequence


def bf16_values(*shape, gen, scale=1.0, shift=0.0):
    return (torch.randn(*shape, generator=gen) * scale + shift).to(torch.bfloat16).double()


def main():
    g = torch.Generator().manual_seed(20240)
    q, k, cq, ck = (bf16_values(B, T, H, D, gen=g) for _ in range(4))
    theta32 = 1 / (10000.0 ** torch.linspace(0, 1, steps=D // 2))                  # the published frequencies, float32
    pos = torch.tensor(START)[:, None] + torch.arange(T)[None]                      # [B, T]
    angle = (pos.float()[:, :, None] * theta32[None, None, :]).double()             # formed in float32, as specified
    w = torch.polar(torch.ones_like(angle), angle)[:, :, None, :]                   # exp(i angle), [B, T, 1, D/2]
    as_complex = lambda x: torch.complex(x[..., 0::2], x[..., 1::2])
    as_pairs = lambda z: torch.stack((z.real, z.imag), dim=-1).flatten(-2)
    out = {"q": q, "k": k, "d_q_rot": cq, "d_k_rot": ck, "theta": theta32, "start": torch.tensor(START),
           "q_rot": as_pairs(as_complex(q) * w), "k_rot": as_pairs(as_complex(k) * w),
           "dq": as_pairs(as_complex(cq) * w.conj()), "dk": as_pairs(as_complex(ck) * w.conj())}

    rows = 50
    r = bf16_values(rows, H, DV, gen=g, scale=2.5, shift=0.75).requires_grad_()
    gate = bf16_values(rows, H * DV, gen=g).requires_grad_()
    d_out = bf16_values(rows, H * DV, gen=g)
    # no intermediate rounding here: the vectors give the exact function; the op's bf16 rounding
    # points are covered by its tolerance
    y = F.group_norm(r.reshape(rows, H * DV), H, eps=1e-6) * F.silu(gate)
    d_r, d_gate = torch.autograd.grad(y, (r, gate), d_out)
    out.update({"r": r.detach(), "gate": gate.detach(), "d_out": d_out, "y": y.detach(), "d_r": d_r, "d_gate": d_gate,
                "eps": torch.tensor(1e-6)})
    np.savez_compressed(os.path.join(HERE, "layer_golden.npz"),
                        **{n: (t.numpy() if t.dtype in (torch.int64, torch.float32) else t.float().numpy()) for n, t in out.items()})


if __name__ == "__main__":
    main()
