"""GPU parity tests for flash_pop_retention_with_suffixes (context + suffixes in one walk),
through the autograd Function and the C ABI.  The oracle composes the two steps the way the
reference's layer does.  Same bar as test_retention_gpu.py."""
import pytest
import torch

import helpers as hp
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GRADS = ("dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0")


def _say(msg):
    print(msg, flush=True)


def run_fused(B, N, block, Ls, H, dk, dv, state_std, seed, decay_range=None, oracle_batches=None, d_last=True,
              oracle_device="cpu", literal=None, tail=0):
    """N full blocks followed by `tail` < block tokens; N + 1 suffixes of Ls tokens per sequence."""
    from flash_pop_amd.pop_retention import flash_pop_retention_with_suffixes
    assert 0 <= tail < block
    T = N * block + tail
    _say(f"[fused pop] B{B} N{N} block{block} tail{tail} Ls{Ls} H{H} dk{dk} dv{dv} s0={state_std} seed={seed}")
    decays = oracle.head_decays(H, decay_range)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=seed, state_std=state_std)
    sfx = hp.make_suffix_inputs(B, N, Ls, H, dk, dv, seed=seed + 1)
    cot = hp.make_cotangents([(B, T, H, dv), tuple(sfx[2].shape), (B, H, dk, dv)], seed=seed + 2)
    if not d_last:
        cot[2] = None
    ctx = [None if t is None else t.to(DEV).requires_grad_() for t in (q, k, v, s)]
    sx = [t.to(DEV).requires_grad_() for t in sfx]
    o, o_sfx, last = flash_pop_retention_with_suffixes(*ctx, decays, block, *sx)
    outs, cots = [o, o_sfx], [cot[0].to(DEV), cot[1].to(DEV)]
    if d_last:
        outs.append(last)
        cots.append(cot[2].to(DEV))
    torch.autograd.backward(outs, cots)
    torch.cuda.synchronize()
    for b in (range(B) if oracle_batches is None else oracle_batches):
        sl, ssl = slice(b, b + 1), slice(b * (N + 1), (b + 1) * (N + 1))
        cut = lambda t, w: None if t is None else t[w]
        o_ref, os_ref, last_ref, g_ref = hp.oracle_fused(
            q[sl], k[sl], v[sl], cut(s, sl), [t[ssl] for t in sfx], decays, block,
            (cot[0][sl], cot[1][ssl], cut(cot[2], sl)), device=oracle_device)
        pairs = [(f"o[b={b}]", o[sl], o_ref, 2), (f"o_sfx[b={b}]", o_sfx[ssl], os_ref, 2), (f"last S[b={b}]", last[sl], last_ref, 1)]
        leaves = ctx[:3] + sx + [ctx[3]]
        for name, leaf, ref in zip(GRADS, leaves, g_ref):
            if ref is None:
                continue
            w = sl if "sfx" not in name else ssl
            pairs.append((f"{name}[b={b}]", leaf.grad[w], ref, 1 if name == "ds0" else 2))
        for name, got, ref, head_dim in pairs:
            hp.assert_close(got, ref, name, head_dim=head_dim)
            if literal is not None:
                hp.check_literal(got, ref, name, literal)
    return o, o_sfx, last


@pytest.mark.parametrize("B,N,block,Ls,H,dk,dv", [
    (2, 4, 64, 16, 4, 128, 128),     # block == chunk, headline head dims
    (2, 3, 144, 16, 4, 64, 128),     # reference generation block size: two full chunks and a short one
    (3, 5, 15, 7, 2, 64, 64),        # block and suffix shorter than a chunk
    (1, 2, 256, 64, 2, 128, 64),     # suffix as long as a chunk
    (2, 8, 32, 1, 2, 64, 128),       # one-token suffixes
    (1, 3, 64, 16, 2, 256, 128),     # 256-wide keys: two visits per chunk in the forward and dv passes
    (1, 2, 96, 24, 2, 128, 256),     # 256-wide values: two visits per chunk in the dq and dk passes
    (2, 3, 64, 16, 2, 192, 192),     # 192-wide keys and values: three visits per chunk in every pass
    (3, 8, 64, 16, 16, 128, 128),    # 48 streams: the fewest that take the backward with the suffixes folded into the chunks
    (8, 8, 64, 16, 12, 64, 128),     # ... the same backward for 64-wide keys (96 streams)
    (4, 4, 128, 40, 12, 128, 64),    # ... 64-wide values, suffixes as extra stops of the walks
    (8, 8, 64, 9, 8, 64, 64),        # ... 64 x 64 states, folded suffixes of 9 tokens
    (3, 4, 128, 33, 16, 128, 128),   # ... with suffixes too long to fold: stops of its walks
])
def test_fused_parity_sweep(B, N, block, Ls, H, dk, dv):
    run_fused(B, N, block, Ls, H, dk, dv, 0.3, seed=N * block + Ls, decay_range=(5, 12))


@pytest.mark.parametrize("B,N,block,Ls,H,dk,dv,tail", [
    (2, 3, 64, 16, 4, 128, 128, 40),     # tokens after the last block boundary, fewer than a chunk
    (2, 2, 144, 16, 2, 64, 128, 100),    # ... more than a chunk (the reference's generation block size)
    (2, 0, 500, 9, 2, 64, 64, 300),      # no full block: one suffix per sequence, reading the initial state
    (1, 2, 64, 16, 2, 256, 128, 17),     # with two visits per chunk
    (2, 3, 64, 100, 4, 128, 128, 0),     # suffixes longer than a chunk: two parts
    (1, 2, 96, 200, 2, 64, 128, 50),     # four parts and a tail
    (1, 2, 64, 128, 2, 128, 64, 0),      # two full parts, dk != dv
])
def test_fused_trailing_tokens_and_long_suffixes(B, N, block, Ls, H, dk, dv, tail):
    """What the reference's layer accepts beyond whole blocks and short suffixes: T % block_size != 0
    (the context goes on after the last boundary, last_state stays the last full block's,
    flash_pop/pop_retnet.py:169) and suffixes of any length."""
    run_fused(B, N, block, Ls, H, dk, dv, 0.3, seed=N * block + Ls + tail, decay_range=(5, 12), tail=tail)
    # (without a full block and without an initial state the reference's layer has no state batch to
    # build its suffix call from, pop_retnet.py:161-164, and the oracle follows it: zeros instead)
    run_fused(B, N, block, Ls, H, dk, dv, None if N else 0.0, seed=N * block + Ls + tail + 1, decay_range=(5, 12), tail=tail,
              d_last=False)


def test_folded_suffix_backward_is_deterministic():
    """Two runs of the fused POP backward (dk = dv = 128, 16-token suffixes: two launches, no atomics) give the same bits."""
    from flash_pop_amd import _lib
    lib = _lib.load()
    B, N, block, Ls, H = 4, 16, 64, 16, 16
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, N * block, H, 128, 128, seed=71, state_std=0.2, device=DEV)
    sfx = hp.make_suffix_inputs(B, N, Ls, H, 128, 128, seed=72, device=DEV)
    cot = hp.make_cotangents([(B, N * block, H, 128), tuple(sfx[2].shape), (B, H, 128, 128)], seed=73, device=DEV)
    first = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot)
    second = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot)
    torch.cuda.synchronize()
    for name, x, y in zip(("dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0"), first, second):
        assert torch.equal(x, y), name


def test_fused_without_state_and_without_last_state_gradient():
    run_fused(2, 3, 64, 8, 2, 64, 64, None, seed=5)
    run_fused(1, 2, 96, 8, 2, 128, 128, 0.2, seed=6, d_last=False)


def test_fused_matches_the_two_op_path():
    """Context outputs are bit-identical to flash_pop_retention's when block is a chunk multiple
    (same partition, same arithmetic); suffix outputs agree with the two-op path to the parity bar
    (there the block states pass through bf16 on the way)."""
    from flash_pop_amd import flash_pop_retention, fused_chunk_retention
    from flash_pop_amd.pop_retention import flash_pop_retention_with_suffixes
    B, N, block, Ls, H, d = 2, 6, 128, 16, 4, 128
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, N * block, H, d, d, seed=61, state_std=0.1, device=DEV)
    sfx = hp.make_suffix_inputs(B, N, Ls, H, d, d, seed=62, device=DEV)
    o, o_sfx, last = flash_pop_retention_with_suffixes(q, k, v, s, decays, block, *sfx)
    o2, states = flash_pop_retention(q, k, v, s, decays, block)
    starts = torch.cat((s[:, None], states), dim=1).flatten(0, 1)
    o_sfx2, _ = fused_chunk_retention(*sfx, starts, decays)
    assert torch.equal(o, o2) and torch.equal(last, states[:, -1])
    hp.assert_close(o_sfx, o_sfx2.float(), "o_sfx vs two-op path", head_dim=2)


def test_fused_raw_abi_optional_outputs():
    """s_out and d_s0 may be NULL; the other outputs do not change."""
    from flash_pop_amd import _lib
    lib = _lib.load()
    B, N, block, Ls, H, d = 1, 2, 64, 16, 2, 64
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, N * block, H, d, d, seed=71, state_std=0.3, device=DEV)
    sfx = hp.make_suffix_inputs(B, N, Ls, H, d, d, seed=72, device=DEV)
    cot = hp.make_cotangents([(B, N * block, H, d), tuple(sfx[2].shape), (B, H, d, d)], seed=73, device=DEV)
    a = hp.raw_fused_fwd(lib, q, k, v, s, sfx, decays, block)
    b = hp.raw_fused_fwd(lib, q, k, v, s, sfx, decays, block, want_state=False)
    ga = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot)
    gb = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot, want_ds0=False)
    torch.cuda.synchronize()
    assert b[2] is None and torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert gb[6] is None and all(torch.equal(x, y) for x, y in zip(ga[:6], gb[:6]))


def test_fused_argument_errors():
    from flash_pop_amd.pop_retention import flash_pop_retention_with_suffixes
    decays = oracle.head_decays(2)
    q, k, v, s = hp.make_inputs(1, 128, 2, 64, 64, seed=1, state_std=0.1, device=DEV)
    sfx = hp.make_suffix_inputs(1, 2, 8, 2, 64, 64, seed=2, device=DEV)
    with pytest.raises(ValueError, match="one additional suffix block"):
        flash_pop_retention_with_suffixes(q, k, v, s, decays, 32, *sfx)


def test_config4_fused():
    """Benchmark configuration 4 in one walk: B8 H16 d128, T4096 in 64-token blocks, 65 suffixes of 16 tokens
    per sequence.  Every sequence against the oracle, which runs on the GPU."""
    run_fused(8, 64, 64, 16, 16, 128, 128, 0.05, seed=40, oracle_device=DEV, literal={})


def test_config5_layer_shapes_fused_pop_and_decode():
    """The retention shapes of benchmark configuration 5 (B8, 12 heads, dk 64, dv 128, T2048 in
    64-token blocks with 16-token suffixes): the fused POP op with all gradients against the oracle
    on every sequence, then 256 recurrent decode steps from its last state against the oracle's
    recurrent step (state rounded to bf16 after every step, as the kernel stores it)."""
    from flash_pop_amd import retention_recurrent
    B, H, dk, dv = 8, 12, 64, 128
    o, o_sfx, last = run_fused(B, 32, 64, 16, H, dk, dv, 0.05, seed=50, oracle_device=DEV, literal={})
    decays = oracle.head_decays(H)
    q, k, v, _ = hp.make_inputs(B, 256, H, dk, dv, seed=51)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    state = last.detach().clone()
    ref_state = last.detach().float()
    outs, refs = [], []
    for t in range(256):
        o_t, state = retention_recurrent(qd[:, t], kd[:, t], vd[:, t], decays, state, in_place=True)
        outs.append(o_t)
        r_t, ref_state = oracle.recurrent_step(qd[:, t].float(), kd[:, t].float(), vd[:, t].float(), ref_state, decays)
        ref_state = ref_state.to(hp.BF16).float()
        refs.append(r_t)
    torch.cuda.synchronize()
    hp.assert_close(torch.stack(outs, 1), torch.stack(refs, 1), "decode o", head_dim=2)
    hp.assert_close(state, ref_state, "decode state", head_dim=1)
