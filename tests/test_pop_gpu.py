"""GPU parity tests for flash_pop_retention and the POP suffix path, through the C ABI.
Same bar as test_retention_gpu.py."""
import pytest
import torch

import helpers as hp
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _say(msg):
    print(msg, flush=True)


def run_pop(B, T, H, dk, dv, block, state_std, seed, decay_range=(5, 12), oracle_batches=None):
    from flash_pop_amd import flash_pop_retention
    _say(f"[pop] B{B} T{T} H{H} dk{dk} dv{dv} block={block} s0={state_std} seed={seed}")
    decays = oracle.head_decays(H, decay_range)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=seed, state_std=state_std)
    d_o, d_b = hp.make_cotangents([(B, T, H, dv), (B, T // block, H, dk, dv)], seed=seed + 1)
    leaves = [None if t is None else t.to(DEV).requires_grad_() for t in (q, k, v, s)]
    o, states = flash_pop_retention(*leaves, decays, block)
    assert states.shape == (B, T // block, H, dk, dv) and states.dtype == torch.bfloat16
    torch.autograd.backward([o, states], [d_o.to(DEV), d_b.to(DEV)])
    torch.cuda.synchronize()
    for b in (range(B) if oracle_batches is None else oracle_batches):
        sl = slice(b, b + 1)
        o_ref, st_ref, grads = hp.oracle_pop(q[sl], k[sl], v[sl], None if s is None else s[sl], decays, block,
                                             d_o[sl], d_b[sl])
        hp.assert_close(o[sl], o_ref, f"o[b={b}]", head_dim=2)
        hp.assert_close(states[sl], st_ref, f"states[b={b}]", head_dim=2)
        for name, leaf, ref in zip(("dq", "dk", "dv", "ds0"), leaves, grads):
            if ref is not None:
                hp.assert_close(leaf.grad[sl], ref, f"{name}[b={b}]", head_dim=1 if name == "ds0" else 2)
    return o, states


@pytest.mark.parametrize("B,T,H,dk,dv,block", [
    (4, 287, 4, 64, 128, 144),     # generation scenario (tests/test_pop_retention.py:161-181)
    (4, 28, 4, 64, 128, 15),       # block shorter than a chunk (:183-196)
    (2, 640, 4, 64, 128, 32),      # training scenario (:216-230)
    (2, 300, 4, 64, 128, 15),      # (:232-246)
    (2, 512, 4, 64, 64, 500),      # reference bwd test shape (:249-262): T % block != 0
    (2, 1440, 4, 64, 128, 144),    # 10 blocks of 144
    (2, 256, 2, 128, 128, 64),     # block == chunk, headline head dims
    (1, 40, 2, 64, 64, 100),       # no full block: empty block_states
    (1, 192, 2, 128, 256, 64),
    (2, 300, 2, 192, 64, 48),      # 192-wide keys: three visits per chunk, block states written and their gradients read
    (8, 1024, 12, 64, 128, 64),    # 96 streams, whole chunks per block: the backward that carries dS once adds the block-state gradients on its way
    (6, 832, 16, 128, 128, 128),   # ... two chunks per block, tokens after the last boundary
    (11, 768, 8, 128, 64, 256),    # ... the sequence ends on a block boundary
])
def test_pop_parity_sweep(B, T, H, dk, dv, block):
    run_pop(B, T, H, dk, dv, block, 0.3, seed=T + block)


@pytest.mark.parametrize("choice", [1, 2])
def test_pop_backward_forced_choice(hip_lib, choice):
    """Both backward paths of a shape with whole chunks per block (8 streams: the passes by shape), against the oracle."""
    assert hip_lib.fp_set_backward_choice(choice, -1) == 0
    try:
        run_pop(2, 640, 4, 64, 128, 128, 0.3, seed=choice)
    finally:
        assert hip_lib.fp_set_backward_choice(0, -1) == 0


def test_pop_without_state_argument():
    run_pop(2, 130, 2, 64, 64, 64, None, seed=4)


def test_pop_outputs_equal_plain_outputs():
    """The context outputs of the POP op are those of the plain entry point (same chunk partition
    when block is a chunk multiple -> bit-identical), and its last block state is the plain final
    state.  The plain side is called through the C ABI: the Python op may cut such a shape into
    segments, which rounds differently."""
    from flash_pop_amd import flash_pop_retention, _lib
    B, T, H, d, block = 2, 1024, 4, 128, 128
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, T, H, d, d, seed=21, state_std=0.1, device=DEV)
    o_pop, states = flash_pop_retention(q, k, v, s, decays, block)
    o, S = hp.raw_fwd(_lib.load(), q, k, v, s, decays)
    torch.cuda.synchronize()
    assert torch.equal(o_pop, o) and torch.equal(states[:, -1], S)


def _suffix_case(B, N, block, Ls, H, dk, dv, seed, oracle_batches, oracle_device="cpu", literal=None):
    """Context through flash_pop_retention, N + 1 suffixes per sequence through
    fused_chunk_retention started from [S0, block states] (flash_pop/pop_retnet.py:152-171),
    gradients chained through both ops by autograd."""
    from flash_pop_amd import flash_pop_retention, fused_chunk_retention
    T = N * block
    _say(f"[pop+suffix] B{B} N{N} block{block} Ls{Ls} H{H} dk{dk} dv{dv}")
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=seed, state_std=0.05)
    qs, ks, vs, _ = hp.make_inputs(B * (N + 1), Ls, H, dk, dv, seed=seed + 1)
    d_o, d_os = hp.make_cotangents([(B, T, H, dv), (B * (N + 1), Ls, H, dv)], seed=seed + 2)
    ctx_leaves = [t.to(DEV).requires_grad_() for t in (q, k, v, s)]
    sfx_leaves = [t.to(DEV).requires_grad_() for t in (qs, ks, vs)]
    o, states = flash_pop_retention(*ctx_leaves, decays, block)
    starts = torch.cat((ctx_leaves[3][:, None], states), dim=1).flatten(0, 1)
    o_sfx, _ = fused_chunk_retention(*sfx_leaves, starts, decays)
    torch.autograd.backward([o, o_sfx], [d_o.to(DEV), d_os.to(DEV)])
    torch.cuda.synchronize()

    for b in oracle_batches:
        sl, ssl = slice(b, b + 1), slice(b * (N + 1), (b + 1) * (N + 1))
        ins = [t[sl].to(oracle_device).float().requires_grad_() for t in (q, k, v, s)]
        sins = [t[ssl].to(oracle_device).float().requires_grad_() for t in (qs, ks, vs)]
        o_ref, st_ref = oracle.pop_retention(*ins, decays, block)
        os_ref = oracle.pop_suffix_retention(*sins, ins[3], st_ref, decays)
        loss = (o_ref * d_o[sl].to(oracle_device).float()).sum() + (os_ref * d_os[ssl].to(oracle_device).float()).sum()
        grads = torch.autograd.grad(loss, ins + sins)
        pairs = [(f"ctx o[b={b}]", o[sl], o_ref.detach(), 2), (f"suffix o[b={b}]", o_sfx[ssl], os_ref.detach(), 2)]
        for name, leaf, ref in zip(("dq", "dk", "dv", "ds0"), ctx_leaves, grads[:4]):
            pairs.append((f"ctx {name}[b={b}]", leaf.grad[sl], ref, 1 if name == "ds0" else 2))
        for name, leaf, ref in zip(("dq", "dk", "dv"), sfx_leaves, grads[4:]):
            pairs.append((f"suffix {name}[b={b}]", leaf.grad[ssl], ref, 2))
        for name, got, ref, head_dim in pairs:
            hp.assert_close(got, ref, name, head_dim=head_dim)
            if literal is not None:
                hp.check_literal(got, ref, name, literal)


def test_pop_suffix_path_small():
    _suffix_case(B=2, N=3, block=32, Ls=8, H=2, dk=64, dv=64, seed=30, oracle_batches=[0, 1])


def test_config4_pop_with_suffixes():
    """Benchmark configuration 4: B8 H16 d128, T4096 in 64-token blocks, 16-token suffixes at every boundary
    (N + 1 = 65 per sequence, the first from S0).  Every sequence against the oracle, which runs on the GPU."""
    _suffix_case(B=8, N=64, block=64, Ls=16, H=16, dk=128, dv=128, seed=40, oracle_batches=range(8), oracle_device=DEV,
                 literal={})
