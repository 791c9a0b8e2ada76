"""Writes tests/golden/retention_golden.npz: seeded bf16-representable inputs and the outputs,
final state, block states and gradients of retention evaluated in float64 by an O(T^2) closed
form built from index arithmetic only (no chunking, no oracle code).  The reference ships no
golden vectors for this path and is not imported here.

    python tests/golden/make_golden.py
"""
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
B, T, H, DK, DV, BLOCK = 1, 150, 2, 64, 64, 64
DECAYS = tuple(1.0 - 2.0 ** (-5 - h) for h in range(H))


def closed_form(q, k, v, s0):
    g = torch.tensor(DECAYS, dtype=torch.float64)
    t = torch.arange(q.shape[1], dtype=torch.float64)
    dist = t[:, None] - t[None, :]
    D = torch.where(dist >= 0, g[:, None, None] ** dist.clamp(min=0), torch.zeros((), dtype=torch.float64))
    scores = torch.einsum("bihd,bjhd->bhij", q, k) / math.sqrt(DK) * D[None]
    o = torch.einsum("bhij,bjhe->bihe", scores, v) + torch.einsum("bihd,bhde,hi->bihe", q, s0, g[:, None] ** (t + 1)[None])

    def state_after(n):
        tt = torch.arange(n, dtype=torch.float64)
        w = g[:, None] ** (n - 1 - tt)[None]
        return torch.einsum("bjhd,hj,bjhe->bhde", k[:, :n] / math.sqrt(DK), w, v[:, :n]) + s0 * (g ** n)[None, :, None, None]

    blocks = torch.stack([state_after((m + 1) * BLOCK) for m in range(T // BLOCK)], dim=1)
    return o, state_after(T), blocks


def main():
    gen = torch.Generator().manual_seed(20240607)
    rnd = lambda *shape, scale=1.0: (torch.randn(*shape, generator=gen) * scale).to(torch.bfloat16).double()
    q, k, v = rnd(B, T, H, DK), rnd(B, T, H, DK), rnd(B, T, H, DV)
    s0 = rnd(B, H, DK, DV, scale=0.3)
    d_o, d_s = rnd(B, T, H, DV), rnd(B, H, DK, DV)
    d_blocks = rnd(B, T // BLOCK, H, DK, DV)
    leaves = [x.clone().requires_grad_() for x in (q, k, v, s0)]
    o, S, blocks = closed_form(*leaves)
    plain = torch.autograd.grad((o * d_o).sum() + (S * d_s).sum(), leaves, retain_graph=True)
    pop = torch.autograd.grad((o * d_o).sum() + (blocks * d_blocks).sum(), leaves)
    f32 = lambda x: x.detach().to(torch.float32).numpy()
    np.savez_compressed(
        os.path.join(HERE, "retention_golden.npz"),
        decays=np.array(DECAYS), block=np.array(BLOCK),
        q=f32(q), k=f32(k), v=f32(v), s0=f32(s0), d_o=f32(d_o), d_s=f32(d_s), d_blocks=f32(d_blocks),
        o=f32(o), s_out=f32(S), blocks=f32(blocks),
        dq=f32(plain[0]), dk=f32(plain[1]), dv=f32(plain[2]), ds0=f32(plain[3]),
        pop_dq=f32(pop[0]), pop_dk=f32(pop[1]), pop_dv=f32(pop[2]), pop_ds0=f32(pop[3]))


if __name__ == "__main__":
    main()
