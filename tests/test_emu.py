"""Runs the real kernel body and the real C-ABI layer on the CPU (one OS thread per GPU lane,
tests/emu/) and compares with the oracle.  This checks indexing, chunk scheduling, the pass
mapping and ragged/unaligned handling without a GPU; it assumes the documented MFMA lane
layout, which only the GPU parity tests can confirm."""
import os
import subprocess

import pytest
import torch

import helpers as hp
import oracle

EMU_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu")


@pytest.fixture(scope="module")
def emu_lib():
    subprocess.run([os.path.join(EMU_DIR, "build_emu.sh")], check=True)
    from flash_pop_amd import _lib
    return _lib.bind(os.path.join(EMU_DIR, "libflashpop_emu.so"))


@pytest.fixture
def choose_backward(emu_lib):
    """choose_backward(1 | 2): force the pass-per-gradient backward / the fused kernel for this test."""
    def choose(choice, every=-1):
        assert emu_lib.fp_set_backward_choice(choice, every) == 0
    yield choose
    assert emu_lib.fp_set_backward_choice(0, 512) == 0


PASSES, FUSED, PACED = 1, 2, 3


def _check_all(pairs):
    for name, got, ref in pairs:
        if ref is not None:
            hp.assert_close(got, ref, name)


@pytest.mark.parametrize("B,T,H,dk,dv,state_std", [
    (1, 150, 2, 128, 128, 0.5),     # ragged tail, initial state
    (1, 100, 2, 64, 128, None),     # dk != dv, no initial state
    (2, 64, 1, 128, 64, 0.0),       # exactly one chunk, zero state
    (1, 70, 1, 256, 64, 0.3),       # widest contraction (two visits per chunk), state stored as it is
    (1, 100, 1, 64, 256, 0.3),      # widest contraction in the dq and dk passes, state read transposed
    (1, 5, 3, 64, 64, 0.5),         # shorter than a chunk
    (5, 16, 1, 128, 128, 0.5),      # several short sequences per workgroup (suffix-like), odd count
    (5, 100, 1, 64, 128, None),     # several multi-chunk sequences per workgroup (the harness has 8 units), no initial state
    (1, 150, 1, 192, 64, 0.3),      # 192-wide keys: three visits per chunk in the forward and dv passes
    (1, 100, 2, 64, 192, 0.3),      # 192-wide values: three visits per chunk in the dq and dk passes
    (1, 130, 1, 192, 192, None),    # both, no initial state
])
def test_plain_fwd_bwd(emu_lib, B, T, H, dk, dv, state_std):
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T, state_std=state_std)
    d_o, d_s = hp.make_cotangents([(B, T, H, dv), (B, H, dk, dv)], seed=T + 1)
    o, S = hp.raw_fwd(emu_lib, q, k, v, s, decays)
    dq, dk_, dv_, ds0 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, d_s)
    o_ref, S_ref, (gq, gk, gv, gs) = hp.oracle_plain(q, k, v, s, decays, d_o, d_s)
    _check_all([("o", o, o_ref), ("S", S, S_ref), ("dq", dq, gq), ("dk", dk_, gk), ("dv", dv_, gv), ("ds0", ds0, gs)])


@pytest.mark.parametrize("B,T,H,dk,dv,block", [
    (1, 150, 2, 128, 128, 64),      # block == chunk
    (1, 287, 1, 64, 128, 144),      # block > chunk, ragged last block (reference generation shape)
    (2, 28, 1, 64, 64, 15),         # block < chunk
    (1, 130, 1, 64, 64, 32),        # block divides chunk
    (1, 40, 1, 64, 64, 100),        # no full block at all
    (1, 130, 1, 256, 64, 32),       # widest contraction with block states written and their gradients read
    (1, 130, 1, 192, 128, 48),      # three visits per chunk with block states
])
def test_pop_fwd_bwd(emu_lib, B, T, H, dk, dv, block):
    decays = oracle.head_decays(H, (5, 12))
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T + block, state_std=0.5)
    d_o, d_b = hp.make_cotangents([(B, T, H, dv), (B, T // block, H, dk, dv)], seed=T)
    o, states = hp.raw_pop_fwd(emu_lib, q, k, v, s, decays, block)
    dq, dk_, dv_, ds0 = hp.raw_pop_bwd(emu_lib, q, k, v, s, decays, block, d_o, d_b)
    o_ref, st_ref, (gq, gk, gv, gs) = hp.oracle_pop(q, k, v, s, decays, block, d_o, d_b)
    _check_all([("o", o, o_ref), ("states", states, st_ref), ("dq", dq, gq), ("dk", dk_, gk), ("dv", dv_, gv),
                ("ds0", ds0, gs)])


@pytest.mark.parametrize("B,T,H,dk,dv,block,state_std", [
    (1, 256, 1, 128, 128, 64, 0.5),     # a block state behind every chunk, the last one at the end of the sequence
    (1, 330, 2, 64, 128, 128, 0.5),     # two chunks per block, tokens after the last block boundary
    (1, 256, 1, 128, 64, 128, None),    # the sequence ends on a block boundary, no initial state
    (1, 300, 1, 64, 64, 192, 0.3),      # 64 x 64 states
    (1, 200, 1, 128, 128, 576, 0.5),    # no full block: nothing to add
])
def test_pop_backward_in_the_kernel_that_carries_ds_once(emu_lib, choose_backward, B, T, H, dk, dv, block, state_std):
    """flash_pop_retention's backward with whole chunks per block: the gradients of the block states join dS in the
    fused backward where its reverse walk crosses their boundaries.  Against the oracle and the pass-per-gradient path."""
    decays = oracle.head_decays(H, (5, 12))
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T + block, state_std=state_std)
    d_o, d_b = hp.make_cotangents([(B, T, H, dv), (B, T // block, H, dk, dv)], seed=T)
    choose_backward(FUSED)
    grads = hp.raw_pop_bwd(emu_lib, q, k, v, s, decays, block, d_o, d_b)
    _, _, ref = hp.oracle_pop(q, k, v, s, decays, block, d_o, d_b)
    _check_all([(n, g, r) for n, g, r in zip(("dq", "dk", "dv", "ds0"), grads, ref)])
    choose_backward(PASSES)
    other = hp.raw_pop_bwd(emu_lib, q, k, v, s, decays, block, d_o, d_b)
    assert not all(torch.equal(x, y) for x, y in zip(grads, other) if x is not None), "both calls took the same kernels"
    for n, x, y in zip(("dq", "dk", "dv", "ds0"), grads, other):
        if x is not None:
            assert hp.error_report(x, y.float())["rms_ratio"] < 0.004, n


FUSED_NAMES = ("dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0")


@pytest.mark.parametrize("B,nblk,block,Ls,H,dk,dv,state_std,tail", [
    (1, 2, 64, 16, 2, 128, 128, 0.5, 0),    # block == chunk
    (2, 2, 80, 5, 1, 64, 128, None, 0),     # block of a full and a short chunk, no initial state
    (1, 3, 24, 64, 1, 128, 64, 0.5, 0),     # block shorter than a chunk, suffix as long as one
    (1, 1, 130, 1, 1, 64, 64, 0.0, 0),      # one block of three chunks, one-token suffixes
    (1, 2, 40, 9, 1, 256, 64, 0.5, 0),      # two visits per chunk in the forward and dv passes
    (1, 2, 64, 16, 1, 64, 256, 0.5, 0),     # ... in the dq and dk passes
    (2, 2, 64, 16, 1, 128, 128, 0.5, 37),   # tokens after the last block boundary (less than a chunk)
    (1, 1, 150, 7, 2, 64, 128, None, 100),  # ... more than a chunk of them, no initial state
    (1, 0, 90, 12, 1, 64, 64, 0.5, 70),     # no full block at all: one suffix, read from the initial state
    (1, 2, 40, 9, 1, 256, 64, 0.5, 11),     # ... with two visits per chunk
    (1, 2, 64, 100, 1, 128, 128, 0.5, 0),   # suffixes longer than a chunk: two parts
    (1, 1, 80, 130, 2, 64, 128, None, 30),  # ... three parts, tokens after the last boundary, no initial state
    (1, 1, 64, 128, 1, 64, 128, 0.3, 0),    # ... two full parts, dk != dv
    (1, 2, 40, 9, 1, 192, 64, 0.5, 0),      # three visits per chunk in the forward and dv passes
    (1, 2, 40, 9, 1, 128, 192, 0.5, 13),    # ... in the dq and dk passes, with trailing tokens
])
def test_fused_pop_fwd_bwd(emu_lib, B, nblk, block, Ls, H, dk, dv, state_std, tail):
    decays = oracle.head_decays(H, (4, 9))
    T = nblk * block + tail
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T + Ls, state_std=state_std)
    sfx = hp.make_suffix_inputs(B, nblk, Ls, H, dk, dv, seed=T + Ls + 1)
    cot = hp.make_cotangents([(B, T, H, dv), tuple(sfx[2].shape), (B, H, dk, dv)], seed=T + 2)
    o, o_sfx, S = hp.raw_fused_fwd(emu_lib, q, k, v, s, sfx, decays, block)
    grads = hp.raw_fused_bwd(emu_lib, q, k, v, s, sfx, decays, block, cot)
    o_ref, os_ref, S_ref, g_ref = hp.oracle_fused(q, k, v, s, sfx, decays, block, cot)
    _check_all([("o", o, o_ref), ("o_sfx", o_sfx, os_ref), ("s_out", S, S_ref)])
    _check_all([(n, g, r) for n, g, r in zip(FUSED_NAMES, grads, g_ref)])


@pytest.mark.parametrize("B,T,H,dk,dv,state_std,segments", [
    (1, 512, 1, 64, 64, 0.5, 2),       # the harness pretends to have 8 compute units: 1 stream -> 2 segments of 4 chunks
    (1, 1024, 1, 64, 128, None, 4),    # dk != dv, no initial state, 4 segments
    (1, 256, 1, 64, 64, 0.5, 1),       # too short to cut: same path as the plain entry point
    (1, 512, 1, 256, 64, 0.5, 2),      # 256-wide keys: the state-only walk visits every chunk twice
    (1, 512, 1, 192, 64, 0.5, 2),      # 192-wide keys: three visits
    (1, 640, 1, 128, 128, 0.5, 2),     # 128-wide keys: the state-only kernel with the whole state tile per workgroup, 5 chunks
    (1, 512, 1, 128, 256, None, 2),    # ... two workgroups per sequence (256-wide values), 4 chunks per segment
])
def test_split_sequences_fwd_bwd(emu_lib, B, T, H, dk, dv, state_std, segments):
    decays = (0.97,) * H
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T, state_std=state_std)
    d_o, d_s = hp.make_cotangents([(B, T, H, dv), (B, H, dk, dv)], seed=T + 1)
    o, S, nbytes = hp.raw_split_fwd(emu_lib, q, k, v, s, decays)
    assert nbytes == (2 * 2 * B * segments * H * dk * dv if segments > 1 else 0)
    dq, dk_, dv_, ds0 = hp.raw_split_bwd(emu_lib, q, k, v, s, decays, d_o, d_s)
    o_ref, S_ref, (gq, gk, gv, gs) = hp.oracle_plain(q, k, v, s, decays, d_o, d_s)
    _check_all([("o", o, o_ref), ("S", S, S_ref), ("dq", dq, gq), ("dk", dk_, gk), ("dv", dv_, gv), ("ds0", ds0, gs)])
    # the backward that starts from the segment states the forward left in its workspace: same bits
    o2, S2, _, ws = hp.raw_split_fwd(emu_lib, q, k, v, s, decays, keep_workspace=True)
    again = hp.raw_split_bwd(emu_lib, q, k, v, s, decays, d_o, d_s, forward_workspace=ws)
    assert torch.equal(o2, o) and all(torch.equal(a, b) for a, b in zip(again, (dq, dk_, dv_, ds0)))


@pytest.mark.parametrize("B,nblk,block,Ls,H,state_std,dk,dv", [
    (1, 2, 128, 16, 1, 0.5, 128, 128),     # two chunks per block
    (1, 4, 64, 64, 1, None, 128, 128),     # block == chunk, suffixes as long as a chunk, no initial state
    (1, 1, 192, 1, 2, 0.3, 128, 128),      # three chunks per block, one-token suffixes, two heads
    (1, 8, 64, 9, 1, 0.3, 128, 128),       # short suffixes folded into every chunk; 9 suffixes over 3 workgroups of the second kernel
    (1, 4, 64, 16, 2, 0.3, 64, 128),       # 64-wide keys: folded suffixes
    (1, 2, 128, 40, 1, None, 128, 64),     # 64-wide values: suffixes as stops, no initial state
    (1, 4, 64, 9, 1, 0.5, 64, 64),         # 64 x 64 states: four state tiles for eight waves
])
def test_fused_pop_backward_that_carries_ds_once(emu_lib, choose_backward, B, nblk, block, Ls, H, state_std, dk, dv):
    """dk, dv of 64 or 128, whole chunks per block (forced here at lengths below the eight chunks from which the
    library chooses it by itself): the fused POP backward runs in
    the kernel that walks backward once for dk and dv beside a forward walk for dq, with the
    suffixes as extra stops at the block boundaries or folded into the chunks there.  Same results as the
    pass-per-gradient path."""
    decays = oracle.head_decays(H, (4, 9))
    T = nblk * block
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T + Ls, state_std=state_std)
    sfx = hp.make_suffix_inputs(B, nblk, Ls, H, dk, dv, seed=T + Ls + 1)
    cot = hp.make_cotangents([(B, T, H, dv), tuple(sfx[2].shape), (B, H, dk, dv)], seed=T + 2)
    choose_backward(FUSED)
    grads = hp.raw_fused_bwd(emu_lib, q, k, v, s, sfx, decays, block, cot)
    _, _, _, g_ref = hp.oracle_fused(q, k, v, s, sfx, decays, block, cot)
    _check_all([(n, g, r) for n, g, r in zip(FUSED_NAMES, grads, g_ref)])
    choose_backward(PASSES)
    other = hp.raw_fused_bwd(emu_lib, q, k, v, s, sfx, decays, block, cot)
    differs = False
    for name, x, y in zip(FUSED_NAMES, grads, other):
        if x is not None:
            assert hp.error_report(x, y.float())["rms_ratio"] < 0.004, name
            differs = differs or not torch.equal(x, y)
    assert differs, "the forced choice made no difference: both calls took the same kernels"


@pytest.mark.parametrize("B,T,H,state_std,every,dk,dv", [
    (1, 330, 1, 0.5, 128, 128, 128),      # ragged tail beyond the last checkpoint, initial state
    (1, 256, 1, None, 128, 128, 128),     # the sequence ends on a checkpoint, no initial state
    (2, 200, 1, 0.3, 64, 128, 128),       # a checkpoint after every chunk, two sequences
    (1, 200, 1, 0.2, 1024, 128, 128),     # interval longer than the sequence: no checkpoint at all
    (1, 260, 1, 0.4, 0, 128, 128),        # no checkpoint buffer: the fused backward walks forward from s0
    (1, 330, 2, 0.5, 128, 64, 128),       # 64-wide keys
    (1, 210, 1, None, 0, 128, 64),        # 64-wide values, no checkpoints, no initial state
    (1, 300, 1, 0.3, 128, 64, 64),        # 64 x 64 states
    (1, 330, 2, 0.5, -128, 128, 128),     # the two workgroups of a stream paced (the harness runs them in turn: no waiting)
])
def test_fused_backward_with_checkpoints(emu_lib, choose_backward, B, T, H, state_std, every, dk, dv):
    """dk, dv of 64 or 128 (forced here at lengths below the eight chunks from which the library chooses it by
    itself): the backward that carries dS once, beside the
    workgroup that re-runs the state from the checkpoints the forward left (segments taken from
    the last to the first)."""
    choose_backward(PACED if every < 0 else FUSED)
    every = abs(every)
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T, state_std=state_std)
    d_o, d_s = hp.make_cotangents([(B, T, H, dv), (B, H, dk, dv)], seed=T + 1)
    if every:
        o, S, dq, dk_, dv_, ds0 = hp.raw_ckpt_fwd_bwd(emu_lib, q, k, v, s, decays, d_o, d_s, every)
    else:
        o, S = hp.raw_fwd(emu_lib, q, k, v, s, decays)
        dq, dk_, dv_, ds0 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, d_s)
    o_ref, S_ref, (gq, gk, gv, gs) = hp.oracle_plain(q, k, v, s, decays, d_o, d_s)
    _check_all([("o", o, o_ref), ("S", S, S_ref), ("dq", dq, gq), ("dk", dk_, gk), ("dv", dv_, gv), ("ds0", ds0, gs)])
    # the checkpoints only serve dq: everything else is bit for bit what the entry points without them give
    o2, S2 = hp.raw_fwd(emu_lib, q, k, v, s, decays)
    g2 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, d_s)
    assert torch.equal(o, o2) and torch.equal(S, S2)
    assert torch.equal(dk_, g2[1]) and torch.equal(dv_, g2[2])
    assert (ds0 is None and g2[3] is None) or torch.equal(ds0, g2[3])
    # and the pass-per-gradient backward gives other bits: the forced choice is what ran
    choose_backward(PASSES)
    g3 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, d_s)
    assert not torch.equal(g3[1], dk_)


@pytest.mark.parametrize("B,T,H,dk,dv,state_std,want_ds0", [
    (5, 16, 2, 128, 128, 0.5, True),     # more (sequence, head) pairs than the harness runs workgroups
    (7, 31, 1, 64, 128, 0.5, True),      # two k-steps along the tokens, 64-wide keys
    (3, 9, 2, 128, 64, None, True),      # no state: no read-out, no d_s0
    (4, 32, 1, 64, 64, 0.3, True),       # the longest sequence the kernel takes
    (2, 1, 3, 128, 128, 0.5, True),      # one token
    (3, 17, 2, 64, 128, 0.5, False),     # d_s0 not wanted
])
def test_many_short_sequences(emu_lib, choose_backward, B, T, H, dk, dv, state_std, want_ds0):
    """At most 32 tokens per sequence, a state per sequence (the suffix call of the reference's POP layer): forward
    and, with no gradient of the final state, backward take one (sequence, head) pair per step in kernels of their
    own."""
    decays = oracle.head_decays(H, (4, 9))
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=T + dk, state_std=state_std)
    d_o, = hp.make_cotangents([(B, T, H, dv)], seed=T + 1)
    o, S = hp.raw_fwd(emu_lib, q, k, v, s, decays)
    o_only, none = hp.raw_fwd(emu_lib, q, k, v, s, decays, want_state=False)
    grads = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, None, want_ds0=want_ds0)
    o_ref, S_ref, ref = hp.oracle_plain(q, k, v, s, decays, d_o, None)
    _check_all([("o", o, o_ref), ("S", S, S_ref)])
    assert none is None and torch.equal(o_only, o)
    _check_all([(n, g, r) for n, g, r in zip(("dq", "dk", "dv", "ds0"), grads, ref) if g is not None])
    choose_backward(PASSES)
    o_p, S_p = hp.raw_fwd(emu_lib, q, k, v, s, decays)
    assert not torch.equal(S_p, S), "the forced choice made no difference: both forwards took the same kernel"
    assert hp.error_report(o, o_p.float())["rms_ratio"] < 0.004 and hp.error_report(S, S_p.float())["rms_ratio"] < 0.006
    other = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, None, want_ds0=want_ds0)
    for n, x, y in zip(("dq", "dk", "dv", "ds0"), grads, other):
        if x is not None:
            assert hp.error_report(x, y.float())["rms_ratio"] < 0.004, n
    # with a gradient of the final state the chunk kernels run, and give the same dq (the short kernel's only
    # state term) up to the rounding of its partial sums
    d_s, = hp.make_cotangents([(B, H, dk, dv)], seed=T + 2)
    choose_backward(0)
    with_ds = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, d_s, want_ds0=want_ds0)
    _, _, ref_ds = hp.oracle_plain(q, k, v, s, decays, d_o, d_s)
    _check_all([(n, g, r) for n, g, r in zip(("dq", "dk", "dv", "ds0"), with_ds, ref_ds) if g is not None])


def test_c_entry_points_refuse_a_capturing_stream(emu_lib):
    """The entry points that launch the pass kernels return FP_ERR_LAUNCH, before launching anything, when
    their stream is recording a HIP graph (the harness's stand-in for hipStreamIsCapturing is a flag);
    the decode step stays capturable."""
    import ctypes
    decays = oracle.head_decays(1)
    q, k, v, s = hp.make_inputs(1, 70, 1, 64, 64, seed=1, state_std=0.5)
    d_o, = hp.make_cotangents([(1, 70, 1, 64)], seed=2)
    sfx = hp.make_suffix_inputs(1, 1, 8, 1, 64, 64, seed=3)
    cot = hp.make_cotangents([(1, 70, 1, 64), tuple(sfx[2].shape), (1, 1, 64, 64)], seed=4)
    calls = [
        lambda: hp.raw_fwd(emu_lib, q, k, v, s, decays),
        lambda: hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, None),
        lambda: hp.raw_pop_fwd(emu_lib, q, k, v, s, decays, 32),
        lambda: hp.raw_pop_bwd(emu_lib, q, k, v, s, decays, 32, d_o, None),
        lambda: hp.raw_fused_fwd(emu_lib, q, k, v, s, sfx, decays, 64),
        lambda: hp.raw_fused_bwd(emu_lib, q, k, v, s, sfx, decays, 64, cot),
        lambda: hp.raw_split_fwd(emu_lib, q, k, v, s, decays),
        lambda: hp.raw_split_bwd(emu_lib, q, k, v, s, decays, d_o, None),
        lambda: hp.raw_ckpt_fwd_bwd(emu_lib, q, k, v, s, decays, d_o, None, 64),
    ]
    emu_lib.emu_set_capturing(1)
    try:
        for call in calls:
            with pytest.raises(AssertionError, match="rc=-5: .*capturing a HIP graph"):
                call()
        o = torch.zeros(1, 70, 1, 64, dtype=hp.BF16)
        rc = emu_lib.fp_retention_fwd_split_static(hp._p(q), hp._p(k), hp._p(v), hp._p(s), hp._dec(decays), hp._p(o), None,
                                                  1, 70, 1, 64, 64, None)
        assert rc == -5 and b"capturing" in emu_lib.fp_last_error()
        hp.raw_decode_step(emu_lib, q[:, 0], k[:, 0], v[:, 0], s, decays)
    finally:
        emu_lib.emu_set_capturing(0)
    hp.raw_fwd(emu_lib, q, k, v, s, decays)


def test_checkpoint_size_query(emu_lib, choose_backward):
    """fp_retention_checkpoint_bytes: 0 where the fused backward would not run or the sequence is
    no longer than one interval, else B * (T / every) state matrices."""
    import ctypes
    every = ctypes.c_int(-1)
    choose_backward(FUSED)
    assert emu_lib.fp_retention_checkpoint_bytes(2, 4096, 4, 128, 128, ctypes.byref(every)) == 2 * 2 * (4096 // 512) * 4 * 128 * 128
    assert every.value == 512
    assert emu_lib.fp_retention_checkpoint_bytes(2, 512, 4, 128, 128, ctypes.byref(every)) == 0 and every.value == 0
    assert emu_lib.fp_retention_checkpoint_bytes(2, 4096, 4, 64, 128, ctypes.byref(every)) == 2 * 2 * (4096 // 512) * 4 * 64 * 128
    assert emu_lib.fp_retention_checkpoint_bytes(2, 4096, 4, 64, 256, ctypes.byref(every)) == 0
    assert emu_lib.fp_retention_checkpoint_bytes(2, 4096, 4, 128, 128, None) > 0
    choose_backward(PASSES)
    assert emu_lib.fp_retention_checkpoint_bytes(2, 4096, 4, 128, 128, ctypes.byref(every)) == 0


@pytest.mark.parametrize("B,H,dk,dv", [(2, 3, 64, 128), (1, 2, 128, 64), (1, 1, 256, 256), (1, 2, 192, 192), (2, 1, 64, 192),
                                       (1, 130, 64, 64)])   # more than 128 heads
def test_decode_step(emu_lib, B, H, dk, dv):
    """Three chained steps (no state, fresh buffer, in place) against the oracle's recurrent step."""
    decays = oracle.head_decays(H)
    g = torch.Generator().manual_seed(dk + dv)
    state, ref_state = None, None
    for step in range(3):
        q, k = (torch.randn(B, H, dk, generator=g).to(hp.BF16) for _ in range(2))
        v = torch.randn(B, H, dv, generator=g).to(hp.BF16)
        o, state = hp.raw_decode_step(emu_lib, q, k, v, state, decays, in_place=step == 2)
        o_ref, ref_state = oracle.recurrent_step(q.float(), k.float(), v.float(), ref_state, decays)
        hp.assert_close(o, o_ref, f"o step {step}")
        hp.assert_close(state, ref_state, f"state step {step}")
        ref_state = state.float()    # follow the kernel's bf16 state, as a decode loop does


def test_optional_outputs_and_determinism(emu_lib):
    decays = oracle.head_decays(2)
    q, k, v, s = hp.make_inputs(1, 90, 2, 64, 64, seed=3, state_std=0.5)
    o1, S1 = hp.raw_fwd(emu_lib, q, k, v, s, decays)
    o2, none = hp.raw_fwd(emu_lib, q, k, v, s, decays, want_state=False)
    assert none is None and torch.equal(o1, o2)
    d_o, = hp.make_cotangents([(1, 90, 2, 64)], seed=4)
    g1 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, None)
    g2 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, None, want_ds0=False)
    assert g2[3] is None and all(torch.equal(a, b) for a, b in zip(g1[:3], g2[:3]))
    z = torch.zeros(1, 2, 64, 64, dtype=hp.BF16)
    g3 = hp.raw_bwd(emu_lib, q, k, v, s, decays, d_o, z)
    assert all(torch.equal(a, b) for a, b in zip(g1, g3))


def test_gamma_one_and_tiny(emu_lib):
    """gamma = 1 (no decay) and a gamma small enough that gamma^63 underflows."""
    decays = (1.0, 1e-3)
    q, k, v, s = hp.make_inputs(1, 130, 2, 64, 64, seed=9, state_std=0.5)
    o, S = hp.raw_fwd(emu_lib, q, k, v, s, decays)
    o_ref, S_ref = hp.oracle_plain(q, k, v, s, decays)
    hp.assert_close(o, o_ref, "o")
    hp.assert_close(S, S_ref, "S")


@pytest.mark.parametrize("B,T,H,d,vec", [(2, 37, 3, 64, False), (3, 5, 2, 128, True), (1, 300, 1, 8, False),
                                         (1, 4096, 5, 64, False)])   # enough tokens for one thread to take all heads
def test_rotary(emu_lib, B, T, H, d, vec):
    """Rotation of q and k (also q alone, in place, and back) against the oracle."""
    g = torch.Generator().manual_seed(d + T)
    q, k = (torch.randn(B, T, H, d, generator=g).to(hp.BF16) for _ in range(2))
    theta = oracle.position_thetas(d)
    start = torch.tensor([7, 4000, 123456][:B]) if vec else 1000
    pos = (start[:, None] if vec else start) + torch.arange(T)[None]
    rq, rk = hp.raw_rotary(emu_lib, q, k, theta, start)

    def same(got, ref):
        """Equal, or (libm's and torch's sine may differ in the last place of an fp32 angle of a few
        thousand radians) a handful of elements apart by one bf16 step."""
        diff = (got.float() - ref.float()).abs()
        return bool((diff > 0).float().mean() < 1e-4) and bool((diff <= ref.float().abs() * 2.0 ** -7 + 1e-5).all())

    assert same(rq, oracle.rotary(q, pos, theta)) and same(rk, oracle.rotary(k, pos, theta))
    only_q, none = hp.raw_rotary(emu_lib, q, None, theta, start)
    assert none is None and torch.equal(only_q, rq)
    back_q, back_k = hp.raw_rotary(emu_lib, rq, rk, theta, start, inverse=True)
    assert same(back_q, oracle.rotary(rq, pos, theta, inverse=True))
    hp.assert_close(back_k, k.float(), "round trip")
    q2, k2 = q.clone(), k.clone()
    hp.raw_rotary(emu_lib, q2, k2, theta, start, in_place=True)
    assert torch.equal(q2, rq) and torch.equal(k2, rk)


@pytest.mark.parametrize("rows,H,dv", [(19, 3, 64), (5, 2, 128), (3, 1, 256), (70, 5, 8)])
def test_gated_group_norm(emu_lib, rows, H, dv):
    g = torch.Generator().manual_seed(rows + dv)
    r = (torch.randn(rows, H, dv, generator=g) * 2 + 0.5).to(hp.BF16)
    gate = torch.randn(rows, H * dv, generator=g).to(hp.BF16)
    d_out = torch.randn(rows, H * dv, generator=g).to(hp.BF16)
    out = hp.raw_gated_norm_fwd(emu_lib, r, gate)
    ref = oracle.gated_group_norm(r, gate)
    # same rounding points as the oracle: equal except where an fp32 value sits on a bf16 rounding boundary
    differ = (out.float() - ref.float()).abs()
    assert float((differ > 0).float().mean()) < 0.01, float((differ > 0).float().mean())
    hp.assert_close(out, ref.float(), "out")
    d_r, d_g = hp.raw_gated_norm_bwd(emu_lib, r, gate, d_out)
    d_r_ref, d_g_ref = hp.oracle_gated_norm_grads(r, gate, d_out)
    hp.assert_close(d_r, d_r_ref, "d_r")
    hp.assert_close(d_g, d_g_ref, "d_g")
