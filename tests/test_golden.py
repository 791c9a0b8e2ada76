"""The committed golden vectors (tests/golden/*.npz, float64 closed forms on seeded
bf16-representable inputs) against the oracle on the CPU and against the HIP ops on the GPU."""
import os

import numpy as np
import pytest
import torch

import helpers as hp
import oracle

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "retention_golden.npz")


@pytest.fixture(scope="module")
def gold():
    z = np.load(PATH, allow_pickle=False)
    g = {k: torch.from_numpy(z[k]) for k in z.files}
    g["decays"] = tuple(float(x) for x in z["decays"])
    g["block"] = int(z["block"])
    return g


def test_oracle_matches_golden(gold):
    ins = [gold[n].double().requires_grad_() for n in ("q", "k", "v", "s0")]
    o, S = oracle.chunkwise_retention(*ins, gold["decays"], chunk_size=64)
    assert torch.allclose(o.float(), gold["o"], rtol=1e-5, atol=1e-5) and torch.allclose(S.float(), gold["s_out"], rtol=1e-5, atol=1e-5)
    grads = torch.autograd.grad((o * gold["d_o"].double()).sum() + (S * gold["d_s"].double()).sum(), ins)
    for name, got in zip(("dq", "dk", "dv", "ds0"), grads):
        assert torch.allclose(got.float(), gold[name], rtol=1e-5, atol=1e-4), name
    ins = [gold[n].double().requires_grad_() for n in ("q", "k", "v", "s0")]
    o, blocks = oracle.pop_retention(*ins, gold["decays"], gold["block"])
    assert torch.allclose(blocks.float(), gold["blocks"], rtol=1e-5, atol=1e-5)
    grads = torch.autograd.grad((o * gold["d_o"].double()).sum() + (blocks * gold["d_blocks"].double()).sum(), ins)
    for name, got in zip(("pop_dq", "pop_dk", "pop_dv", "pop_ds0"), grads):
        assert torch.allclose(got.float(), gold[name], rtol=1e-5, atol=1e-4), name


@pytest.mark.gpu
def test_hip_ops_match_golden(gold):
    from flash_pop_amd import fused_chunk_retention, flash_pop_retention
    dev = "cuda:0"
    bf = lambda n: gold[n].to(torch.bfloat16).to(dev)
    leaves = [bf(n).requires_grad_() for n in ("q", "k", "v", "s0")]
    o, S = fused_chunk_retention(*leaves, gold["decays"])
    torch.autograd.backward([o, S], [bf("d_o"), bf("d_s")])
    hp.assert_close(o, gold["o"], "o", head_dim=2)
    hp.assert_close(S, gold["s_out"], "s_out", head_dim=1)
    for name, leaf in zip(("dq", "dk", "dv", "ds0"), leaves):
        hp.assert_close(leaf.grad, gold[name], name, head_dim=1 if name == "ds0" else 2)
    leaves = [bf(n).requires_grad_() for n in ("q", "k", "v", "s0")]
    o, blocks = flash_pop_retention(*leaves, gold["decays"], gold["block"])
    torch.autograd.backward([o, blocks], [bf("d_o"), bf("d_blocks")])
    hp.assert_close(blocks, gold["blocks"], "blocks", head_dim=2)
    for name, leaf in zip(("pop_dq", "pop_dk", "pop_dv", "pop_ds0"), leaves):
        hp.assert_close(leaf.grad, gold[name], name, head_dim=1 if name == "pop_ds0" else 2)


FUSED_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pop_fused_golden.npz")
FUSED_INPUTS = ("q", "k", "v", "s0", "q_sfx", "k_sfx", "v_sfx")
FUSED_GRADS = ("dq", "dk", "dv", "ds0", "dq_sfx", "dk_sfx", "dv_sfx")


@pytest.fixture(scope="module")
def gold_fused():
    z = np.load(FUSED_PATH, allow_pickle=False)
    g = {k: torch.from_numpy(z[k]) for k in z.files}
    g["decays"] = tuple(float(x) for x in z["decays"])
    g["block"] = int(z["block"])
    return g


def test_oracle_matches_fused_pop_golden(gold_fused):
    g = gold_fused
    q, k, v, s0, qs, ks, vs = ins = [g[n].double().requires_grad_() for n in FUSED_INPUTS]
    o, o_sfx, last = oracle.pop_fused_retention(q, k, v, s0, qs, ks, vs, g["decays"], g["block"])
    for name, got in (("o", o), ("o_sfx", o_sfx), ("last", last)):
        assert torch.allclose(got.float(), g[name], rtol=1e-5, atol=1e-5), name
    loss = (o * g["d_o"].double()).sum() + (o_sfx * g["d_o_sfx"].double()).sum() + (last * g["d_last"].double()).sum()
    for name, got in zip(FUSED_GRADS, torch.autograd.grad(loss, ins)):
        assert torch.allclose(got.float(), g[name], rtol=1e-5, atol=1e-4), name


@pytest.mark.gpu
def test_fused_pop_op_matches_golden(gold_fused):
    from flash_pop_amd import flash_pop_retention_with_suffixes
    g = gold_fused
    bf = lambda n: g[n].to(torch.bfloat16).to("cuda:0")
    q, k, v, s0, qs, ks, vs = leaves = [bf(n).requires_grad_() for n in FUSED_INPUTS]
    o, o_sfx, last = flash_pop_retention_with_suffixes(q, k, v, s0, g["decays"], g["block"], qs, ks, vs)
    torch.autograd.backward([o, o_sfx, last], [bf("d_o"), bf("d_o_sfx"), bf("d_last")])
    hp.assert_close(o, g["o"], "o", head_dim=2)
    hp.assert_close(o_sfx, g["o_sfx"], "o_sfx", head_dim=2)
    hp.assert_close(last, g["last"], "last", head_dim=1)
    for name, leaf in zip(FUSED_GRADS, leaves):
        hp.assert_close(leaf.grad, g[name], name, head_dim=1 if name == "ds0" else 2)


LAYER_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layer_golden.npz")


@pytest.fixture(scope="module")
def gold_layer():
    z = np.load(LAYER_PATH, allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files}


def test_layer_oracle_matches_golden(gold_layer):
    g = gold_layer
    T = g["q"].shape[1]
    pos = g["start"][:, None] + torch.arange(T)[None]
    for x, want, d_x, d_want in (("q", "q_rot", "d_q_rot", "dq"), ("k", "k_rot", "d_k_rot", "dk")):
        assert torch.allclose(oracle.rotary(g[x], pos, g["theta"]), g[want], rtol=0, atol=2e-6), x
        assert torch.allclose(oracle.rotary(g[d_x], pos, g["theta"], inverse=True), g[d_want], rtol=0, atol=2e-6), d_x
    y = oracle.gated_group_norm(g["r"], g["gate"], float(g["eps"]))
    assert torch.allclose(y, g["y"], rtol=1e-5, atol=1e-5)
    d_r, d_gate = hp.oracle_gated_norm_grads(g["r"].to(hp.BF16), g["gate"].to(hp.BF16), g["d_out"].to(hp.BF16), float(g["eps"]))
    hp.assert_close(d_r, g["d_r"], "d_r")
    hp.assert_close(d_gate, g["d_gate"], "d_gate")


@pytest.mark.gpu
def test_layer_ops_match_golden(gold_layer):
    from flash_pop_amd import XPos, gated_group_norm
    g, dev = gold_layer, "cuda:0"
    bf = lambda n: g[n].to(torch.bfloat16).to(dev)
    q, k = bf("q").requires_grad_(), bf("k").requires_grad_()
    xpos = XPos(q.shape[-1])
    assert torch.equal(xpos.thetas, g["theta"])
    rq, rk = xpos(q, k, g["start"].to(dev))
    torch.autograd.backward([rq, rk], [bf("d_q_rot"), bf("d_k_rot")])
    for got, want in ((rq, "q_rot"), (rk, "k_rot"), (q.grad, "dq"), (k.grad, "dk")):
        hp.assert_close(got, g[want], want)
    r, gate = bf("r").requires_grad_(), bf("gate").requires_grad_()
    y = gated_group_norm(r, gate, float(g["eps"]))
    y.backward(bf("d_out"))
    hp.assert_close(y, g["y"], "y")
    hp.assert_close(r.grad, g["d_r"], "d_r")
    hp.assert_close(gate.grad, g["d_gate"], "d_gate")
