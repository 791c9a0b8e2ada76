"""GPU parity tests for the two elementwise stages around the retention op: the rotary embedding of
q and k and the per-head normalisation with the swish gate, through the C ABI and through the
Python wrappers with autograd.  The oracle runs on the CPU on the same seeded bf16 inputs.

Bar: floating point, bf16 storage.  Both kernels round where the oracle rounds, so results are equal
except where an fp32 intermediate sits within an ulp of a bf16 rounding boundary (sin, cos, exp and
the reduction order differ in their last bits): at most 1 % of the elements may differ, none by more
than one bf16 step per rounding point on its way (2^-7 relative each: one for the rotation, three for
the gated normalisation; absolute floor 1e-5 for results of cancellations); gradients, which the kernel evaluates in fp32 without the
intermediate bf16 tensors of a torch graph, meet the retention tests' bar (rtol 2e-2, atol 2e-2 RMS,
RMS error ratio < 0.005)."""
import pytest
import torch
import torch.nn.functional as F

import helpers as hp
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _say(msg):
    print(msg, flush=True)


def assert_same_up_to_rounding(got, ref, name, max_fraction=0.01, floor=1e-5, steps=1):
    """`steps`: bf16 steps a differing element may be off by (one per rounding point on its way).
    `floor`: results that come out of a cancellation (x cos - y sin near zero, r - mean near zero)
    carry the fp32 rounding of their terms, about 1e-7 times the inputs, as an absolute error."""
    g, r = got.detach().cpu().float(), ref.detach().cpu().float()
    assert g.shape == r.shape, f"{name}: shape {tuple(g.shape)} != {tuple(r.shape)}"
    assert torch.isfinite(g).all(), f"{name}: non-finite values"
    diff = (g - r).abs()
    frac = float((diff > 0).float().mean())
    assert frac <= max_fraction, f"{name}: {frac:.4f} of the elements differ"
    step = (r.abs() * 2.0 ** -7 * steps).clamp_min(floor)
    assert bool((diff <= step).all()), f"{name}: differences beyond {steps} bf16 step(s), max ratio {float((diff / step).max()):.2f}"


@pytest.mark.parametrize("B,T,H,d,start", [
    (8, 2048, 12, 64, 0),                       # the model configuration's q, k
    (2, 300, 16, 128, 4096),
    (65, 16, 12, 64, "per-sequence"),           # suffixes: one start position per sequence
    (1, 7, 1, 256, 1_000_000),
])
def test_rotary_matches_oracle(hip_lib, B, T, H, d, start):
    _say(f"[rotary] B{B} T{T} H{H} d{d} start={start}")
    g = torch.Generator().manual_seed(B + T)
    q, k = (torch.randn(B, T, H, d, generator=g).to(hp.BF16) for _ in range(2))
    theta = oracle.position_thetas(d)
    start_cpu = torch.arange(B) * 64 + 5 if start == "per-sequence" else start
    pos = (start_cpu[:, None] if start == "per-sequence" else start_cpu) + torch.arange(T)[None]
    start_dev = start_cpu.to(DEV) if start == "per-sequence" else start_cpu
    rq, rk = hp.raw_rotary(hip_lib, q.to(DEV), k.to(DEV), theta.to(DEV), start_dev)
    # large positions: float32 angles carry errors of 2^-24 * angle, which sinf implementations
    # resolve differently; the bar is the same, only more elements sit near a rounding boundary
    frac = 0.01 if T + (0 if start == "per-sequence" else start) < 100_000 else 0.1
    assert_same_up_to_rounding(rq, oracle.rotary(q, pos, theta), "q", frac)
    assert_same_up_to_rounding(rk, oracle.rotary(k, pos, theta), "k", frac)
    # q alone; in place; back
    only_q, none = hp.raw_rotary(hip_lib, q.to(DEV), None, theta.to(DEV), start_dev)
    assert none is None and torch.equal(only_q, rq)
    q2, k2 = q.to(DEV), k.to(DEV)
    hp.raw_rotary(hip_lib, q2, k2, theta.to(DEV), start_dev, in_place=True)
    assert torch.equal(q2, rq) and torch.equal(k2, rk)
    back, _ = hp.raw_rotary(hip_lib, rq, rk, theta.to(DEV), start_dev, inverse=True)
    hp.assert_close(back, q.float(), "inverse(forward(q))")


def test_xpos_wrapper_and_its_gradient(hip_lib):
    from flash_pop_amd import XPos
    B, T, H, d = 3, 130, 4, 64
    _say(f"[xpos autograd] B{B} T{T} H{H} d{d}")
    g = torch.Generator().manual_seed(11)
    q, k, cq, ck = (torch.randn(B, T, H, d, generator=g).to(hp.BF16) for _ in range(4))
    xpos = XPos(d)
    assert torch.equal(xpos.thetas, oracle.position_thetas(d))
    for start in (17, torch.tensor([0, 64, 8000])):
        qd, kd = q.to(DEV).requires_grad_(), k.to(DEV).requires_grad_()
        s_dev = start.to(DEV) if isinstance(start, torch.Tensor) else start
        rq, rk = xpos(qd, kd, s_dev)
        torch.autograd.backward([rq, rk], [cq.to(DEV), ck.to(DEV)])
        pos = (start[:, None] if isinstance(start, torch.Tensor) else start) + torch.arange(T)[None]
        qf, kf = q.float().requires_grad_(), k.float().requires_grad_()
        oq, ok = oracle.rotary(qf, pos, xpos.thetas), oracle.rotary(kf, pos, xpos.thetas)
        torch.autograd.backward([oq, ok], [cq.float(), ck.float()])
        assert_same_up_to_rounding(rq, oq.detach().to(hp.BF16), "q")
        assert_same_up_to_rounding(rk, ok.detach().to(hp.BF16), "k")
        assert_same_up_to_rounding(qd.grad, qf.grad.to(hp.BF16), "dq")
        assert_same_up_to_rounding(kd.grad, kf.grad.to(hp.BF16), "dk")


def test_rotary_keeps_scores_relative_at_full_size(hip_lib):
    """Size-independent property at the benchmark's shape: pair norms are preserved and q.k scores
    depend on the distance only (rotating both by 5000 more positions changes nothing)."""
    B, T, H, d = 8, 4096, 16, 128
    _say(f"[rotary properties] B{B} T{T} H{H} d{d}")
    g = torch.Generator(device=DEV).manual_seed(5)
    q, k = (torch.randn(B, T, H, d, generator=g, device=DEV).to(hp.BF16) for _ in range(2))
    theta = oracle.position_thetas(d).to(DEV)
    q0, k0 = hp.raw_rotary(hip_lib, q, k, theta, 0)
    q1, k1 = hp.raw_rotary(hip_lib, q, k, theta, 5000)
    pair = lambda t: t.float().unflatten(-1, (d // 2, 2)).square().sum(-1)
    err = (pair(q0) - pair(q)).abs() / pair(q).clamp_min(1e-3)
    assert float(err.max()) < 0.03 and float(err.mean()) < 3e-3
    i = torch.arange(100, 164, device=DEV)
    s0 = torch.einsum("bihd,bjhd->bhij", q0[:, i].float(), k0[:, i - 40].float())
    s1 = torch.einsum("bihd,bjhd->bhij", q1[:, i].float(), k1[:, i - 40].float())
    assert float((s0 - s1).abs().max()) < 0.02 * float(s0.square().mean().sqrt()) + 0.5
    assert float((s0 - s1).square().mean().sqrt() / s0.square().mean().sqrt()) < 0.01


@pytest.mark.parametrize("rows,H,dv", [(8 * 2048, 12, 128), (8 * 65 * 16, 12, 128), (1001, 3, 64), (77, 2, 256), (5, 1, 8)])
def test_gated_group_norm_matches_oracle(hip_lib, rows, H, dv):
    _say(f"[gated norm] rows{rows} H{H} dv{dv}")
    g = torch.Generator().manual_seed(rows + dv)
    r = (torch.randn(rows, H, dv, generator=g) * 3 + 0.7).to(hp.BF16)
    gate = torch.randn(rows, H * dv, generator=g).to(hp.BF16)
    d_out = torch.randn(rows, H * dv, generator=g).to(hp.BF16)
    out = hp.raw_gated_norm_fwd(hip_lib, r.to(DEV), gate.to(DEV))
    # three rounding points (normalised value, gate, product): a flipped first rounding moves the product by a
    # step, and its own rounding can add to that
    assert_same_up_to_rounding(out, oracle.gated_group_norm(r, gate), "out", steps=3)
    d_r, d_g = hp.raw_gated_norm_bwd(hip_lib, r.to(DEV), gate.to(DEV), d_out.to(DEV))
    d_r_ref, d_g_ref = hp.oracle_gated_norm_grads(r, gate, d_out)
    hp.assert_close(d_r, d_r_ref, "d_r")
    hp.assert_close(d_g, d_g_ref, "d_g")


def test_gated_group_norm_wrapper_against_the_torch_composition(hip_lib):
    """The reference's own call sequence (group_norm in fp32 -> bf16, times silu of the gate) run by
    torch on the GPU, forward and autograd, against the one-launch op."""
    from flash_pop_amd import gated_group_norm
    B, T, H, dv = 2, 257, 6, 128
    _say(f"[gated norm wrapper] B{B} T{T} H{H} dv{dv}")
    g = torch.Generator().manual_seed(21)
    r = (torch.randn(B, T, H, dv, generator=g) * 2).to(hp.BF16).to(DEV)
    gate = torch.randn(B, T, H * dv, generator=g).to(hp.BF16).to(DEV)
    d_out = torch.randn(B, T, H * dv, generator=g).to(hp.BF16).to(DEV)
    r1, g1 = r.clone().requires_grad_(), gate.clone().requires_grad_()
    out = gated_group_norm(r1, g1, 1e-6)
    out.backward(d_out)
    r2, g2 = r.clone().requires_grad_(), gate.clone().requires_grad_()
    n = F.group_norm(r2.reshape(B * T, H * dv).float(), H, eps=1e-6).to(hp.BF16).reshape(B, T, H * dv)
    ref = n * F.silu(g2)
    ref.backward(d_out)
    assert out.shape == ref.shape
    assert_same_up_to_rounding(out, ref, "out", steps=3)
    hp.assert_close(r1.grad, r2.grad.float(), "d_r")
    hp.assert_close(g1.grad, g2.grad.float(), "d_g")


def test_gated_group_norm_statistics_at_full_size(hip_lib):
    """Size-independent property: with a gate of swish^-1(1) the output is the normalised tensor,
    whose heads have zero mean and unit variance whatever the scale and offset of the input."""
    rows, H, dv = 32768, 16, 128
    _say(f"[gated norm properties] rows{rows} H{H} dv{dv}")
    g = torch.Generator(device=DEV).manual_seed(9)
    scale = torch.rand(rows, H, 1, generator=g, device=DEV) * 50 + 0.1
    r = (torch.randn(rows, H, dv, generator=g, device=DEV) * scale + scale).to(hp.BF16)
    one = torch.full((rows, H * dv), 1.2784645, device=DEV).to(hp.BF16)      # swish(1.2785) = 1.0 in bf16
    assert float(F.silu(one[0, 0])) == 1.0
    n = hp.raw_gated_norm_fwd(hip_lib, r, one).float().reshape(rows, H, dv)
    assert float(n.mean(-1).abs().max()) < 0.01
    assert float((n.square().mean(-1) - 1).abs().max()) < 0.01
