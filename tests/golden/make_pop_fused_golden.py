"""Writes tests/golden/pop_fused_golden.npz: seeded bf16-representable inputs of one fused POP
step (context of N blocks plus N + 1 suffixes) with outputs and gradients evaluated in float64 by
an O(T^2) closed form built from index arithmetic only: suffix n is the tail of plain retention
over concat(context[:n * block], suffix n).  No chunking, no oracle code, no reference import.

    python tests/golden/make_pop_fused_golden.py
"""
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
B, N, BLOCK, LS, H, DK, DV = 1, 2, 64, 16, 2, 64, 64
T = N * BLOCK
DECAYS = tuple(1.0 - 2.0 ** (-5 - h) for h in range(H))


def closed_form(q, k, v, s0):
    """Outputs and final state of retention over the whole of q, k, v [1, n, H, d]."""
    n = q.shape[1]
    g = torch.tensor(DECAYS, dtype=torch.float64)
    t = torch.arange(n, dtype=torch.float64)
    dist = t[:, None] - t[None, :]
    D = torch.where(dist >= 0, g[:, None, None] ** dist.clamp(min=0), torch.zeros((), dtype=torch.float64))
    scores = torch.einsum("bihd,bjhd->bhij", q, k) / math.sqrt(DK) * D[None]
    o = torch.einsum("bhij,bjhe->bihe", scores, v) + torch.einsum("bihd,bhde,hi->bihe", q, s0, g[:, None] ** (t + 1)[None])
    w = g[:, None] ** (n - 1 - t)[None]
    S = torch.einsum("bjhd,hj,bjhe->bhde", k / math.sqrt(DK), w, v) + s0 * (g ** n)[None, :, None, None]
    return o, S


def fused(q, k, v, s0, qs, ks, vs):
    o, last = closed_form(q, k, v, s0)
    tails = []
    for n in range(N + 1):
        cat = lambda ctx, sfx: torch.cat((ctx[:, :n * BLOCK], sfx[n:n + 1]), dim=1)
        o_n, _ = closed_form(cat(q, qs), cat(k, ks), cat(v, vs), s0)
        tails.append(o_n[:, n * BLOCK:])
    return o, torch.cat(tails, dim=0), last


def main():
    gen = torch.Generator().manual_seed(20240608)
    rnd = lambda *shape, scale=1.0: (torch.randn(*shape, generator=gen) * scale).to(torch.bfloat16).double()
    q, k, v = rnd(B, T, H, DK), rnd(B, T, H, DK), rnd(B, T, H, DV)
    s0 = rnd(B, H, DK, DV, scale=0.3)
    qs, ks, vs = rnd(N + 1, LS, H, DK), rnd(N + 1, LS, H, DK), rnd(N + 1, LS, H, DV)
    d_o, d_os, d_last = rnd(B, T, H, DV), rnd(N + 1, LS, H, DV), rnd(B, H, DK, DV)
    leaves = [x.clone().requires_grad_() for x in (q, k, v, s0, qs, ks, vs)]
    o, o_sfx, last = fused(*leaves)
    grads = torch.autograd.grad((o * d_o).sum() + (o_sfx * d_os).sum() + (last * d_last).sum(), leaves)
    f32 = lambda x: x.detach().to(torch.float32).numpy()
    names = ("dq", "dk", "dv", "ds0", "dq_sfx", "dk_sfx", "dv_sfx")
    np.savez_compressed(
        os.path.join(HERE, "pop_fused_golden.npz"),
        decays=np.array(DECAYS), block=np.array(BLOCK),
        q=f32(q), k=f32(k), v=f32(v), s0=f32(s0), q_sfx=f32(qs), k_sfx=f32(ks), v_sfx=f32(vs),
        d_o=f32(d_o), d_o_sfx=f32(d_os), d_last=f32(d_last),
        o=f32(o), o_sfx=f32(o_sfx), last=f32(last), **{n: f32(g) for n, g in zip(names, grads)})


if __name__ == "__main__":
    main()
