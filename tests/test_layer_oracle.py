"""Pins the oracle's rotary embedding and gated per-head normalisation against formulations that
do not share their code: complex multiplication in float64, geometric properties of rotations,
and the library routines (group_norm, silu) that the reference itself calls."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle


def test_thetas_closed_form():
    th = oracle.position_thetas(64)
    assert th.shape == (32,) and th.dtype == torch.float32
    want = [10000.0 ** (-i / 31.0) for i in range(32)]
    np.testing.assert_allclose(th.numpy(), want, rtol=2e-6)
    assert th[0] == 1.0 and abs(float(th[-1]) - 1e-4) < 1e-9


def test_rotary_is_complex_multiplication():
    g = torch.Generator().manual_seed(0)
    B, T, H, d = 2, 9, 3, 16
    x = torch.randn(B, T, H, d, generator=g)
    start = torch.tensor([5, 1000])
    pos = start[:, None] + torch.arange(T)[None]
    th = oracle.position_thetas(d)
    got = oracle.rotary(x, pos, th).double().numpy()
    z = x.double().numpy()[..., 0::2] + 1j * x.double().numpy()[..., 1::2]
    # the angle is formed in float32 by the reference; reproduce that single rounding, then go exact
    ang = (pos.float()[:, :, None, None] * th.float()[None, None, None, :]).double().numpy()
    w = z * np.exp(1j * ang)
    np.testing.assert_allclose(got[..., 0::2], w.real, atol=2e-6)
    np.testing.assert_allclose(got[..., 1::2], w.imag, atol=2e-6)


def test_rotary_special_positions():
    x = torch.arange(8.0).reshape(1, 1, 1, 8) + 1
    th = torch.tensor([math.pi / 2, math.pi, 0.0, 2 * math.pi])
    same = oracle.rotary(x, torch.zeros(1, 1, dtype=torch.long), th)
    assert torch.equal(same, x)                                           # position 0 is the identity
    out = oracle.rotary(x, torch.ones(1, 1, dtype=torch.long), th)[0, 0, 0]
    want = torch.tensor([-2.0, 1.0, -3.0, -4.0, 5.0, 6.0, 7.0, 8.0])     # quarter turn, half turn, none, full
    torch.testing.assert_close(out, want, atol=2e-6, rtol=0)


def test_rotary_properties():
    g = torch.Generator().manual_seed(1)
    B, T, H, d = 1, 12, 2, 32
    q = torch.randn(B, T, H, d, generator=g, dtype=torch.float64)
    k = torch.randn(B, T, H, d, generator=g, dtype=torch.float64)
    th = oracle.position_thetas(d)
    pos = torch.arange(T)[None]
    rq, rk = oracle.rotary(q, pos, th), oracle.rotary(k, pos, th)
    # norms of pairs are preserved
    torch.testing.assert_close(rq.pow(2).sum(-1), q.pow(2).sum(-1), atol=1e-5, rtol=1e-6)
    # inverse undoes it
    torch.testing.assert_close(oracle.rotary(rq, pos, th, inverse=True), q, atol=1e-5, rtol=0)
    # rotating by a then b is rotating by a + b
    twice = oracle.rotary(oracle.rotary(q, pos, th), 3 * pos, th)
    torch.testing.assert_close(twice, oracle.rotary(q, 4 * pos, th), atol=1e-5, rtol=0)
    # scores depend on the distance between positions only
    s0 = torch.einsum("bihd,bjhd->bhij", rq, rk)
    rq7, rk7 = oracle.rotary(q, pos + 7, th), oracle.rotary(k, pos + 7, th)
    torch.testing.assert_close(torch.einsum("bihd,bjhd->bhij", rq7, rk7), s0, atol=1e-4, rtol=0)
    # and the direction matters: q rotates forward with its own position, k with its own (not the transpose)
    i, j = 5, 2
    dist = oracle.rotary(k[:, j:j + 1], torch.full((1, 1), j - i), th)
    torch.testing.assert_close((q[:, i] * dist[:, 0]).sum(-1), s0[:, :, i, j], atol=1e-4, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_group_norm_is_the_library_composition(dtype):
    g = torch.Generator().manual_seed(2)
    rows, H, dv = 37, 4, 32
    r = (torch.randn(rows, H, dv, generator=g) * 3 + 1.5).to(dtype)
    gate = torch.randn(rows, H * dv, generator=g).to(dtype)
    got = oracle.gated_group_norm(r, gate, eps=1e-6)
    # the reference's calls (flash_pop/retnet.py:297,308-309)
    n = F.group_norm(r.reshape(rows, H * dv).float(), H, eps=1e-6).to(dtype)
    want = n * F.silu(gate)
    assert got.dtype == dtype
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=2e-6, rtol=2e-6)
    else:
        # identical up to a last-bit difference where fp32 results sit on a bf16 rounding boundary
        diff = (got.float() - want.float()).abs()
        assert float((diff > 0).float().mean()) < 0.01
        assert float((diff / want.float().abs().clamp_min(1e-3)).max()) < 2 ** -6


def test_gated_group_norm_invariants():
    g = torch.Generator().manual_seed(3)
    rows, H, dv = 5, 3, 64
    r = torch.randn(rows, H, dv, generator=g, dtype=torch.float32)
    ones = torch.full((rows, H * dv), 30.0)                      # swish(30) = 30 to fp32 precision
    n = (oracle.gated_group_norm(r, ones, eps=0.0) / 30.0).reshape(rows, H, dv)
    torch.testing.assert_close(n.mean(-1), torch.zeros(rows, H), atol=1e-6, rtol=0)
    torch.testing.assert_close(n.pow(2).mean(-1), torch.ones(rows, H), atol=1e-5, rtol=0)
    shifted = (oracle.gated_group_norm(r * 7.0 + 3.0, ones, eps=0.0) / 30.0).reshape(rows, H, dv)
    torch.testing.assert_close(shifted, n, atol=2e-5, rtol=0)
    # each head is normalised on its own: changing head 0 leaves the others untouched
    r2 = r.clone()
    r2[:, 0] *= 5
    n2 = (oracle.gated_group_norm(r2, ones, eps=0.0) / 30.0).reshape(rows, H, dv)
    assert torch.equal(n2[:, 1:], n[:, 1:])
    # eps enters under the square root, next to the biased variance
    const = torch.zeros(1, 1, 8)
    const[0, 0, 0] = 1.0                                          # mean 1/8, var 7/64
    out = oracle.gated_group_norm(const, torch.full((1, 8), 30.0), eps=0.25) / 30.0
    assert abs(float(out[0, 0]) - (1 - 1 / 8) / math.sqrt(7 / 64 + 0.25)) < 1e-6
