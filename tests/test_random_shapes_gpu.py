"""Seeded random sweep of shapes on the GPU against the oracle: sequence lengths around chunk and
block boundaries, block sizes below, at and above the chunk, suffix lengths 1..64, all head-dimension
pairs, random decays including 1.0, with and without an initial state.  Same bar as the other GPU
tests; every case prints its parameters before it runs."""
import random

import pytest
import torch

import helpers as hp
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DIMS = (64, 128, 192, 256)


def _decays(rng, H):
    return tuple(1.0 if rng.random() < 0.15 else 1.0 - 2.0 ** -rng.uniform(2.0, 12.0) for _ in range(H))


def _check(names, got, ref, heads_at):
    for n, g, r in zip(names, got, ref):
        if r is not None:
            hp.assert_close(g, r, n, head_dim=heads_at(n))


def test_random_plain_and_pop_cases():
    rng = random.Random(20240611)
    from flash_pop_amd import _lib
    lib = _lib.load()
    for case in range(24):
        B, H = rng.randint(1, 3), rng.randint(1, 5)
        dk, dv = rng.choice(DIMS), rng.choice(DIMS)
        T = rng.choice([1, 2, 31, 63, 64, 65, 127, 128, 129, 200, 257, 320])
        block = rng.choice([0, 0, 1, 7, 16, 63, 64, 65, 100, 128, 192])
        state_std = rng.choice([None, 0.0, 0.3])
        decays = _decays(rng, H)
        print(f"[random {case}] B{B} T{T} H{H} dk{dk} dv{dv} block{block} s0={state_std}", flush=True)
        q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=1000 + case, state_std=state_std, device=DEV)
        if block == 0:
            d_o, d_s = hp.make_cotangents([(B, T, H, dv), (B, H, dk, dv)], seed=2000 + case, device=DEV)
            o, S = hp.raw_fwd(lib, q, k, v, s, decays)
            grads = hp.raw_bwd(lib, q, k, v, s, decays, d_o, d_s)
            torch.cuda.synchronize()
            o_ref, S_ref, g_ref = hp.oracle_plain(q, k, v, s, decays, d_o, d_s)
            _check(("o", "S", "dq", "dk", "dv", "ds0"), (o, S, *grads), (o_ref, S_ref, *g_ref),
                   lambda n: 1 if n in ("S", "ds0") else 2)
        else:
            d_o, d_b = hp.make_cotangents([(B, T, H, dv), (B, T // block, H, dk, dv)], seed=2000 + case, device=DEV)
            o, states = hp.raw_pop_fwd(lib, q, k, v, s, decays, block)
            grads = hp.raw_pop_bwd(lib, q, k, v, s, decays, block, d_o, d_b)
            torch.cuda.synchronize()
            o_ref, st_ref, g_ref = hp.oracle_pop(q, k, v, s, decays, block, d_o, d_b)
            _check(("o", "states", "dq", "dk", "dv", "ds0"), (o, states, *grads), (o_ref, st_ref, *g_ref),
                   lambda n: 1 if n == "ds0" else 2)


def test_random_fused_pop_cases():
    rng = random.Random(20240612)
    from flash_pop_amd import _lib
    lib = _lib.load()
    names = ("o", "o_sfx", "s_out", "dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0")
    for case in range(16):
        B, H = rng.randint(1, 3), rng.randint(1, 4)
        dk, dv = rng.choice(DIMS), rng.choice(DIMS)
        block = rng.choice([1, 5, 16, 63, 64, 65, 100, 128, 144])
        nblk = rng.randint(1, 4)
        Ls = rng.choice([1, 2, 15, 16, 17, 32, 33, 64])
        state_std = rng.choice([None, 0.3])
        decays = _decays(rng, H)
        T = nblk * block
        print(f"[random fused {case}] B{B} N{nblk} block{block} Ls{Ls} H{H} dk{dk} dv{dv} s0={state_std}", flush=True)
        q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=3000 + case, state_std=state_std, device=DEV)
        sfx = hp.make_suffix_inputs(B, nblk, Ls, H, dk, dv, seed=4000 + case, device=DEV)
        cot = hp.make_cotangents([(B, T, H, dv), tuple(sfx[2].shape), (B, H, dk, dv)], seed=5000 + case, device=DEV)
        o, o_sfx, S = hp.raw_fused_fwd(lib, q, k, v, s, sfx, decays, block)
        grads = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot)
        torch.cuda.synchronize()
        o_ref, os_ref, S_ref, g_ref = hp.oracle_fused(q, k, v, s, sfx, decays, block, cot)
        _check(names, (o, o_sfx, S, *grads), (o_ref, os_ref, S_ref, *g_ref), lambda n: 1 if n in ("s_out", "ds0") else 2)


def test_random_fused_pop_cases_any_length():
    """Tokens after the last block boundary (also no full block at all) and suffixes of up to 200 tokens."""
    rng = random.Random(20240613)
    from flash_pop_amd import _lib
    lib = _lib.load()
    names = ("o", "o_sfx", "s_out", "dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0")
    for case in range(16):
        B, H = rng.randint(1, 2), rng.randint(1, 3)
        Ls = rng.choice([1, 16, 63, 64, 65, 100, 128, 129, 200])
        dims = DIMS if Ls <= 64 else (64, 128)        # suffixes in several parts: one visit per chunk only
        dk, dv = rng.choice(dims), rng.choice(dims)
        block = rng.choice([5, 16, 63, 64, 65, 100, 128, 144])
        nblk = rng.randint(0, 3)
        tail = rng.choice([0, 1, block // 2, block - 1])
        if nblk == 0 and tail == 0:
            tail = block - 1
        state_std = 0.3 if nblk == 0 else rng.choice([None, 0.3])   # (the oracle needs a state to read when there is no block)
        decays = _decays(rng, H)
        T = nblk * block + tail
        print(f"[random fused any {case}] B{B} N{nblk} block{block} tail{tail} Ls{Ls} H{H} dk{dk} dv{dv} s0={state_std}", flush=True)
        q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=6000 + case, state_std=state_std, device=DEV)
        sfx = hp.make_suffix_inputs(B, nblk, Ls, H, dk, dv, seed=7000 + case, device=DEV)
        cot = hp.make_cotangents([(B, T, H, dv), tuple(sfx[2].shape), (B, H, dk, dv)], seed=8000 + case, device=DEV)
        o, o_sfx, S = hp.raw_fused_fwd(lib, q, k, v, s, sfx, decays, block)
        grads = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot)
        torch.cuda.synchronize()
        o_ref, os_ref, S_ref, g_ref = hp.oracle_fused(q, k, v, s, sfx, decays, block, cot)
        _check(names, (o, o_sfx, S, *grads), (o_ref, os_ref, S_ref, *g_ref), lambda n: 1 if n in ("s_out", "ds0") else 2)


def test_random_cases_for_the_backward_that_carries_ds_once():
    """dk = dv = 128 with enough streams and at least eight chunks: plain (with random checkpoint
    intervals) and with POP suffixes at block boundaries that are multiples of 64."""
    rng = random.Random(20240614)
    from flash_pop_amd import _lib
    lib = _lib.load()
    for case in range(10):
        H = rng.choice([8, 16, 32])
        B = 96 // H * rng.randint(1, 2)
        decays = _decays(rng, H)
        state_std = rng.choice([None, 0.2])
        if case % 2 == 0:
            T = rng.choice([512, 513, 640, 1000, 1537])
            every = rng.choice([64, 128, 320, 512, 1024])
            print(f"[random carried {case}] plain B{B} T{T} H{H} every{every} s0={state_std}", flush=True)
            q, k, v, s = hp.make_inputs(B, T, H, 128, 128, seed=9000 + case, state_std=state_std, device=DEV)
            d_o, d_s = hp.make_cotangents([(B, T, H, 128), (B, H, 128, 128)], seed=9500 + case, device=DEV)
            got = hp.raw_ckpt_fwd_bwd(lib, q, k, v, s, decays, d_o, d_s, every)
            torch.cuda.synchronize()
            o_ref, S_ref, g_ref = hp.oracle_plain(q, k, v, s, decays, d_o, d_s, device=DEV)
            _check(("o", "S", "dq", "dk", "dv", "ds0"), got, (o_ref, S_ref, *g_ref), lambda n: 1 if n in ("S", "ds0") else 2)
        else:
            block = rng.choice([64, 128, 192, 256])
            nblk = max(512 // block, rng.randint(2, 6))
            Ls = rng.choice([1, 9, 16, 17, 40, 64])
            T = nblk * block
            print(f"[random carried {case}] pop B{B} N{nblk} block{block} Ls{Ls} H{H} s0={state_std}", flush=True)
            q, k, v, s = hp.make_inputs(B, T, H, 128, 128, seed=9000 + case, state_std=state_std, device=DEV)
            sfx = hp.make_suffix_inputs(B, nblk, Ls, H, 128, 128, seed=9200 + case, device=DEV)
            cot = hp.make_cotangents([(B, T, H, 128), tuple(sfx[2].shape), (B, H, 128, 128)], seed=9500 + case, device=DEV)
            grads = hp.raw_fused_bwd(lib, q, k, v, s, sfx, decays, block, cot)
            torch.cuda.synchronize()
            _, _, _, g_ref = hp.oracle_fused(q, k, v, s, sfx, decays, block, cot, device=DEV)
            _check(("dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0"), grads, g_ref, lambda n: 1 if n == "ds0" else 2)
