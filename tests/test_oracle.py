"""Pins the CPU oracle against formulations that do not share its code:
an O(T^2) closed form in float64, pure-Python brute force, the token recurrence,
autograd / gradcheck, invariances the mathematics fixes and the gamma=1 / gamma->0
special cases.  A dropped term, wrong exponent, transposed operand or missing
1/sqrt(dk) in the oracle fails at least one of these."""
import math

import pytest
import torch

import oracle
from oracle import retention_oracle as ro

torch.manual_seed(1234)
F64 = torch.float64


def rand_inputs(B, T, H, dk, dv, with_state=True, dtype=F64, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, dk, generator=g, dtype=dtype)
    k = torch.randn(B, T, H, dk, generator=g, dtype=dtype)
    v = torch.randn(B, T, H, dv, generator=g, dtype=dtype)
    s = torch.randn(B, H, dk, dv, generator=g, dtype=dtype) * 0.3 if with_state else None
    return q, k, v, s


def closed_form(q, k, v, s0, decays):
    """o_t = sum_{j<=t} g^(t-j) (q_t . k_j/sqrt(dk)) v_j + g^(t+1) q_t S0 ;
    S_T = g^T S0 + sum_j g^(T-1-j) (k_j/sqrt(dk))^T v_j.   Built from index arithmetic only."""
    B, T, H, dk = q.shape
    g = torch.tensor(decays, dtype=F64)
    t = torch.arange(T, dtype=F64)
    dist = t[:, None] - t[None, :]
    D = torch.where(dist >= 0, g[:, None, None] ** dist.clamp(min=0), torch.zeros((), dtype=F64))   # [H,T,T]
    scores = torch.einsum("bihd,bjhd->bhij", q, k) / math.sqrt(dk) * D[None]
    o = torch.einsum("bhij,bjhe->bihe", scores, v)
    w_end = g[:, None] ** (T - 1 - t)[None]                                                      # [H,T]
    S = torch.einsum("bjhd,hj,bjhe->bhde", k / math.sqrt(dk), w_end, v)
    if s0 is not None:
        o = o + torch.einsum("bihd,bhde,hi->bihe", q, s0, g[:, None] ** (t + 1)[None])
        S = S + s0 * (g ** T)[None, :, None, None]
    return o, S


def brute_force(q, k, v, s0, decays):
    """Pure-Python token recurrence on nested lists (tiny shapes only)."""
    B, T, H, dk = q.shape
    dv = v.shape[3]
    o = torch.zeros(B, T, H, dv, dtype=F64)
    S_out = torch.zeros(B, H, dk, dv, dtype=F64)
    for b in range(B):
        for h in range(H):
            S = [[(float(s0[b, h, a, c]) if s0 is not None else 0.0) for c in range(dv)] for a in range(dk)]
            for t in range(T):
                for a in range(dk):
                    ka = float(k[b, t, h, a]) / math.sqrt(dk)
                    for c in range(dv):
                        S[a][c] = decays[h] * S[a][c] + ka * float(v[b, t, h, c])
                for c in range(dv):
                    o[b, t, h, c] = sum(float(q[b, t, h, a]) * S[a][c] for a in range(dk))
            S_out[b, h] = torch.tensor(S, dtype=F64)
    return o, S_out


def test_head_decays_closed_form():
    d = oracle.head_decays(16)
    assert len(d) == 16 and all(isinstance(x, float) for x in d)
    for h, g in enumerate(d):
        assert g == 1.0 - 2.0 ** (-5 - h)
    d2 = oracle.head_decays(4, (5, 12))
    assert d2[0] == 1 - 2.0 ** -5 and abs(d2[-1] - (1 - 2.0 ** -12)) < 1e-15


def test_decay_mask_entries():
    like = torch.zeros(1, dtype=F64)
    decays = (0.9, 0.5, 1.0)
    m = oracle.decay_mask(decays, 7, like)
    assert m.shape == (3, 7, 7)
    for h, g in enumerate(decays):
        for i in range(7):
            for j in range(7):
                want = g ** (i - j) if i >= j else 0.0
                assert abs(m[h, i, j].item() - want) < 1e-14
    # a tiny gamma must not produce inf/nan on the masked side
    assert torch.isfinite(oracle.decay_mask((1e-30,), 64, like)).all()


def test_brute_force_tiny():
    decays = (0.8, 0.95)
    q, k, v, s = rand_inputs(2, 5, 2, 3, 2, seed=1)
    o_bf, S_bf = brute_force(q, k, v, s, decays)
    for cs in (1, 2, 5, 512):
        o, S = oracle.chunkwise_retention(q, k, v, s, decays, chunk_size=cs)
        assert torch.allclose(o, o_bf, atol=1e-12) and torch.allclose(S, S_bf, atol=1e-12)
    o_cf, S_cf = closed_form(q, k, v, s, decays)
    assert torch.allclose(o_cf, o_bf, atol=1e-12) and torch.allclose(S_cf, S_bf, atol=1e-12)
    # no initial state == zero initial state
    o0, S0 = oracle.chunkwise_retention(q, k, v, None, decays, chunk_size=2)
    o0_bf, S0_bf = brute_force(q, k, v, None, decays)
    assert torch.allclose(o0, o0_bf, atol=1e-12) and torch.allclose(S0, S0_bf, atol=1e-12)


@pytest.mark.parametrize("T,chunk", [(64, 64), (200, 64), (257, 32), (130, 512), (96, 1)])
@pytest.mark.parametrize("with_state", [False, True])
def test_chunkwise_vs_closed_form(T, chunk, with_state):
    decays = oracle.head_decays(3)
    q, k, v, s = rand_inputs(2, T, 3, 16, 24, with_state, seed=T)
    o, S = oracle.chunkwise_retention(q, k, v, s, decays, chunk_size=chunk)
    o_cf, S_cf = closed_form(q, k, v, s, decays)
    assert torch.allclose(o, o_cf, atol=1e-10), (o - o_cf).abs().max()
    assert torch.allclose(S, S_cf, atol=1e-10)


def test_recurrent_step_equals_chunkwise():
    decays = (0.9, 0.97, 0.5)
    q, k, v, s = rand_inputs(2, 37, 3, 8, 5, seed=3)
    state, outs = s, []
    for t in range(q.shape[1]):
        o_t, state = oracle.recurrent_step(q[:, t], k[:, t], v[:, t], state, decays)
        outs.append(o_t)
    o, S = oracle.chunkwise_retention(q, k, v, s, decays, chunk_size=16)
    assert torch.allclose(torch.stack(outs, 1), o, atol=1e-11) and torch.allclose(state, S, atol=1e-11)
    # first step without a state
    o1, S1 = oracle.recurrent_step(q[:, 0], k[:, 0], v[:, 0], None, decays)
    o1c, S1c = closed_form(q[:, :1], k[:, :1], v[:, :1], None, decays)
    assert torch.allclose(o1, o1c[:, 0], atol=1e-12) and torch.allclose(S1, S1c, atol=1e-12)


def test_split_sequence_invariance_and_linearity():
    decays = oracle.head_decays(2)
    q, k, v, s = rand_inputs(1, 150, 2, 8, 8, seed=5)
    o, S = oracle.chunkwise_retention(q, k, v, s, decays, 64)
    o1, S1 = oracle.chunkwise_retention(q[:, :70], k[:, :70], v[:, :70], s, decays, 64)
    o2, S2 = oracle.chunkwise_retention(q[:, 70:], k[:, 70:], v[:, 70:], S1, decays, 64)
    assert torch.allclose(torch.cat((o1, o2), 1), o, atol=1e-11) and torch.allclose(S2, S, atol=1e-11)
    # linear in (v, s0) jointly
    oa, Sa = oracle.chunkwise_retention(q, k, 2 * v, 2 * s, decays, 64)
    assert torch.allclose(oa, 2 * o, atol=1e-11) and torch.allclose(Sa, 2 * S, atol=1e-11)


def test_special_gammas():
    q, k, v, _ = rand_inputs(1, 40, 1, 4, 6, False, seed=7)
    s = 1 / math.sqrt(4)
    # gamma = 1: causal linear attention, state = cumulative sum of k^T v
    o, S = oracle.chunkwise_retention(q, k, v, None, (1.0,), 16)
    kv = torch.einsum("btd,bte->btde", k[:, :, 0] * s, v[:, :, 0]).cumsum(1)
    assert torch.allclose(o[:, :, 0], torch.einsum("btd,btde->bte", q[:, :, 0], kv), atol=1e-11)
    assert torch.allclose(S[:, 0], kv[:, -1], atol=1e-11)
    # gamma -> 0: only the diagonal survives, the state is the last outer product
    o, S = oracle.chunkwise_retention(q, k, v, None, (0.0,), 16)
    diag = (q[:, :, 0] * k[:, :, 0] * s).sum(-1, keepdim=True) * v[:, :, 0]
    assert torch.allclose(o[:, :, 0], diag, atol=1e-12)
    assert torch.allclose(S[0, 0], torch.outer(k[0, -1, 0] * s, v[0, -1, 0]), atol=1e-12)


def _autograd_grads(fn, inputs, cotangents):
    leaves = [x.clone().requires_grad_() for x in inputs]
    outs = fn(*leaves)
    loss = sum((o * c).sum() for o, c in zip(outs, cotangents))
    return torch.autograd.grad(loss, leaves)


def test_chunk_grads_vs_autograd_of_closed_form():
    decays = (0.9, 0.99)
    q, k, v, s = rand_inputs(2, 33, 2, 6, 5, seed=11)
    g = torch.Generator().manual_seed(2)
    do = torch.randn(q.shape[0], 33, 2, 5, generator=g, dtype=F64)
    dS = torch.randn(s.shape, generator=g, dtype=F64)
    want = _autograd_grads(lambda *a: closed_form(*a, decays), (q, k, v, s), (do, dS))
    got = oracle.retention_chunk_grads(q, k, v, s, decays, do, dS)
    for name, a, b in zip("dq dk dv ds".split(), got, want):
        assert torch.allclose(a, b, atol=1e-10), name


def test_chunkwise_autograd_vs_closed_form_autograd_and_gradcheck():
    decays = oracle.head_decays(2)
    q, k, v, s = rand_inputs(1, 70, 2, 4, 3, seed=13)
    g = torch.Generator().manual_seed(3)
    do = torch.randn(1, 70, 2, 3, generator=g, dtype=F64)
    dS = torch.randn(s.shape, generator=g, dtype=F64)
    want = _autograd_grads(lambda *a: closed_form(*a, decays), (q, k, v, s), (do, dS))
    got = _autograd_grads(lambda *a: oracle.chunkwise_retention(*a, decays, 32), (q, k, v, s), (do, dS))
    for a, b in zip(got, want):
        assert torch.allclose(a, b, atol=1e-10)
    small = [x[:, :9].clone().requires_grad_() for x in (q, k, v)] + [s.clone().requires_grad_()]
    assert torch.autograd.gradcheck(lambda *a: oracle.chunkwise_retention(*a, decays, 4), small, atol=1e-7)


@pytest.mark.parametrize("T,bs", [(287, 144), (28, 15), (128, 64), (300, 15), (64, 100)])
def test_pop_block_states_are_prefix_states(T, bs):
    decays = oracle.head_decays(2, (5, 12))
    q, k, v, s = rand_inputs(2, T, 2, 8, 6, seed=T + bs)
    o, states = oracle.pop_retention(q, k, v, s, decays, bs)
    assert states.shape == (2, T // bs, 2, 8, 6)
    o_cf, _ = closed_form(q, k, v, s, decays)
    assert torch.allclose(o, o_cf, atol=1e-10)
    for m in range(T // bs):
        end = (m + 1) * bs
        _, S_prefix = closed_form(q[:, :end], k[:, :end], v[:, :end], s, decays)
        assert torch.allclose(states[:, m], S_prefix, atol=1e-10)


def test_pop_suffix_equals_concatenated_context():
    """Suffix n must equal the tail of a plain run over context[: n*bs] ++ suffix_n,
    which also pins that suffix tokens never touch the main state."""
    decays = (0.9, 0.97)
    B, N, bs, Ls, H, dk, dv = 2, 3, 5, 4, 2, 4, 3
    q, k, v, s = rand_inputs(B, N * bs, H, dk, dv, seed=21)
    qs, ks, vs, _ = rand_inputs(B * (N + 1), Ls, H, dk, dv, False, seed=22)
    _, states = oracle.pop_retention(q, k, v, s, decays, bs)
    got = oracle.pop_suffix_retention(qs, ks, vs, s, states, decays).view(B, N + 1, Ls, H, dv)
    for b in range(B):
        for n in range(N + 1):
            i = b * (N + 1) + n
            cat = lambda ctx, sfx: torch.cat((ctx[b:b + 1, :n * bs], sfx[i:i + 1]), dim=1)
            o_cf, _ = closed_form(cat(q, qs), cat(k, ks), cat(v, vs), s[b:b + 1], decays)
            assert torch.allclose(got[b, n], o_cf[0, n * bs:], atol=1e-10)
    # state0=None means zeros
    got0 = oracle.pop_suffix_retention(qs, ks, vs, None, states, decays)
    gotz = oracle.pop_suffix_retention(qs, ks, vs, torch.zeros_like(s), states, decays)
    assert torch.equal(got0, gotz)


def test_pop_fused_is_the_composition_and_pins_last_state():
    decays = (0.9, 0.97)
    B, N, bs, Ls, H, dk, dv = 2, 3, 5, 4, 2, 4, 3
    for T in (N * bs, N * bs + 2):          # with and without a ragged tail after the last block
        q, k, v, s = rand_inputs(B, T, H, dk, dv, seed=31)
        qs, ks, vs, _ = rand_inputs(B * (N + 1), Ls, H, dk, dv, False, seed=32)
        o, o_sfx, last = oracle.pop_fused_retention(q, k, v, s, qs, ks, vs, decays, bs)
        o_cf, _ = closed_form(q, k, v, s, decays)
        _, S_blocks = closed_form(q[:, :N * bs], k[:, :N * bs], v[:, :N * bs], s, decays)
        assert torch.allclose(o, o_cf, atol=1e-10) and torch.allclose(last, S_blocks, atol=1e-10)
        for b in range(B):
            for n in range(N + 1):
                i = b * (N + 1) + n
                cat = lambda ctx, sfx: torch.cat((ctx[b:b + 1, :n * bs], sfx[i:i + 1]), dim=1)
                ref, _ = closed_form(cat(q, qs), cat(k, ks), cat(v, vs), s[b:b + 1], decays)
                assert torch.allclose(o_sfx[i], ref[0, n * bs:], atol=1e-10)
    # no full block: the last state is the initial one
    q, k, v, s = rand_inputs(1, 3, 2, 4, 3, seed=33)
    qs, ks, vs, _ = rand_inputs(1, 2, 2, 4, 3, False, seed=34)
    _, _, last = oracle.pop_fused_retention(q, k, v, s, qs, ks, vs, decays, 5)
    assert torch.equal(last, s)


def test_fp32_matches_fp64_at_config1():
    """Benchmark configuration 1 (fp32, B1 H4 T512 d64, chunk 64, no initial state): the fp32 oracle
    is within 1e-4 of the float64 closed form."""
    decays = oracle.head_decays(4)
    q, k, v, _ = rand_inputs(1, 512, 4, 64, 64, False, dtype=torch.float32, seed=0)
    o, S = oracle.chunkwise_retention(q, k, v, None, decays, chunk_size=64)
    o_cf, S_cf = closed_form(q.double(), k.double(), v.double(), None, decays)
    assert S.shape == (1, 4, 64, 64)
    assert torch.allclose(o.double(), o_cf, rtol=1e-4, atol=1e-4)
    assert torch.allclose(S.double(), S_cf, rtol=1e-4, atol=1e-4)
    assert ro.rms_error_ratio(o, o_cf) < 1e-5
