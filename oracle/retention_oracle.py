"""CPU restatement of flash-pop's PyTorch retention path.  TEST INFRASTRUCTURE ONLY.

This module is the parity checker for the HIP kernels.  Nothing in the shipped
package imports it; only the tests, the smoke entry and the CPU-baseline leg of
the benchmark do.  It restates, in plain torch, what the reference computes in

  * flash_pop/fused_retention/reference.py:10-50   one-chunk retention           -> retention_chunk
  * flash_pop/fused_retention/reference.py:53-69   chunk loop carrying the state -> chunkwise_retention
  * flash_pop/fused_retention/reference.py:72-111  closed-form one-chunk grads   -> retention_chunk_grads
  * flash_pop/fused_retention/__init__.py:73-102   per-head decay mask           -> decay_mask
  * tests/test_pop_retention.py:13-32              POP oracle (block states)     -> pop_retention
  * flash_pop/retnet.py:70-76                      per-head decay values         -> head_decays
  * flash_pop/retnet.py:79-101                     one-token recurrent step      -> recurrent_step
  * flash_pop/pop_retnet.py:152-171                POP suffix state selection    -> pop_suffix_retention
  * flash_pop/pop_retnet.py:107,152-171            context + suffixes of one layer -> pop_fused_retention

Conventions carried over from the reference: tensors are [B, T, H, d]; the
state is [B, H, dk, dv]; the public entry points divide K by sqrt(dk)
(reference.py:57) and never scale Q; within a chunk of length L the read-out
of the carried state is weighted gamma^(i+1), keys entering the state are
weighted gamma^(L-1-j) and the carried state is decayed by gamma^L
(reference.py:31-35,41,45); POP keeps a block state only for blocks that end
at or before T (tests/test_pop_retention.py:29).

Pinning status.  Every function here is pinned by tests/test_oracle.py against
independent formulations (an O(T^2) closed form in float64, the token-by-token
recurrence, pure-Python brute force on tiny shapes, autograd and gradcheck,
chunk-size and split-sequence invariance, and the gamma=1 / gamma->0 special
cases).  The reference ships no golden vectors for this path, so the committed
fixtures under tests/golden/ are produced from this module after those checks.
The only thing left unpinned is the bit-level rounding order of the
reference's bf16 casts, which the stated tolerances deliberately do not fix.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch
from torch import Tensor


def head_decays(num_heads: int, decay_range: Optional[tuple] = None) -> tuple:
    """gamma_h = 1 - 2^(-5-h), or exponents spread linearly over `decay_range`
    (flash_pop/retnet.py:70-76).  Returned as Python floats, as the ops expect."""
    if decay_range is None:
        exps = -5.0 - np.arange(num_heads, dtype=np.float64)
    else:
        exps = -np.linspace(decay_range[0], decay_range[1], num_heads, dtype=np.float64)
    return tuple(float(g) for g in (1.0 - np.exp2(exps)))


def _gammas(decays: Sequence[float], like: Tensor) -> Tensor:
    # The reference builds gamma (and the mask) in float32 whatever the input dtype
    # (fused_retention/__init__.py:73,87); keep float64 when the caller works in float64
    # so that the closed-form checks are not limited by that.
    dt = torch.float64 if like.dtype == torch.float64 else torch.float32
    return torch.tensor(list(decays), dtype=dt, device=like.device)


def decay_mask(decays: Sequence[float], n: int, like: Tensor) -> Tensor:
    """[H, n, n] lower-triangular gamma_h^(i-j) (fused_retention/__init__.py:87-96)."""
    g = _gammas(decays, like)
    pos = torch.arange(n, device=like.device, dtype=g.dtype)
    dist = pos[:, None] - pos[None, :]
    keep = dist >= 0
    # exponent clamped on the masked side so that tiny gammas cannot overflow there
    powers = g[:, None, None] ** dist.clamp(min=0)[None]
    return powers * keep[None]


def retention_chunk(q: Tensor, k_scaled: Tensor, v: Tensor, state: Optional[Tensor], decays: Sequence[float]):
    """One chunk; `k_scaled` is already divided by sqrt(dk) (reference.py:10-50).

    Returns (o [B,L,H,dv], new_state [B,H,dk,dv])."""
    dt = q.dtype
    L = q.shape[1]
    g = _gammas(decays, q)
    qh, kh, vh = (x.permute(0, 2, 1, 3) for x in (q, k_scaled, v))          # [B,H,L,d]
    scores = (qh @ kh.transpose(-1, -2)).tril()
    scores = (scores * decay_mask(decays, L, q).to(dt)[None]).tril()
    out = scores.to(dt) @ vh                                                  # [B,H,L,dv]

    steps = torch.arange(1, L + 1, device=q.device, dtype=dt)                # inner position + 1
    key_w = (g[:, None] ** (L - steps)[None]).to(dt)                         # [H,L]  gamma^(L-1-j)
    new_state = (kh * key_w[None, :, :, None]).transpose(-1, -2) @ vh         # [B,H,dk,dv]
    if state is not None:
        new_state = new_state + state * (g ** L)[None, :, None, None]
        read_w = (g[:, None] ** steps[None]).to(dt)                           # [H,L]  gamma^(i+1)
        out = out + (qh.to(dt) @ state.to(dt)) * read_w[None, :, :, None]
    return out.permute(0, 2, 1, 3).to(dt), new_state.to(dt)


def chunkwise_retention(q: Tensor, k: Tensor, v: Tensor, state: Optional[Tensor], decays: Sequence[float],
                        chunk_size: int = 512):
    """Chunk loop carrying the state; scales K by dk^-1/2 (reference.py:53-69)."""
    T = q.shape[1]
    k = k / (k.shape[3] ** 0.5)
    outs = []
    for t0 in range(0, T, chunk_size):
        sl = slice(t0, t0 + chunk_size)
        o, state = retention_chunk(q[:, sl], k[:, sl], v[:, sl], state, decays)
        outs.append(o)
    return torch.cat(outs, dim=1), state


def pop_retention(q: Tensor, k: Tensor, v: Tensor, state: Optional[Tensor], decays: Sequence[float],
                  block_size: int):
    """Retention chunked at `block_size`, also returning the state after every FULL block,
    stacked as [B, T // block_size, H, dk, dv] (tests/test_pop_retention.py:13-32)."""
    T = q.shape[1]
    k = k / (k.shape[3] ** 0.5)
    outs, states = [], []
    for m in range(math.ceil(T / block_size)):
        sl = slice(m * block_size, (m + 1) * block_size)
        o, state = retention_chunk(q[:, sl], k[:, sl], v[:, sl], state, decays)
        outs.append(o)
        if (m + 1) * block_size <= T:
            states.append(state)
    if states:
        block_states = torch.stack(states, dim=1)
    else:
        B, _, H, dk = q.shape
        block_states = q.new_zeros(B, 0, H, dk, v.shape[3])
    return torch.cat(outs, dim=1), block_states


def retention_chunk_grads(q: Tensor, k: Tensor, v: Tensor, state: Tensor, decays: Sequence[float],
                          d_out: Tensor, d_new_state: Tensor):
    """Closed-form gradients of ONE chunk covering the whole sequence, w.r.t. the UNscaled k
    (reference.py:72-111).  Returns (dq, dk, dv, dstate)."""
    dt = q.dtype
    L, dk = q.shape[1], q.shape[3]
    s = dk ** -0.5
    g = _gammas(decays, q)
    D = decay_mask(decays, L, q).to(dt)[None]                                # [1,H,L,L]
    steps = torch.arange(1, L + 1, device=q.device, dtype=dt)
    read_w = (g[:, None] ** steps[None]).to(dt)[None, :, :, None]            # gamma^(i+1)
    key_w = (g[:, None] ** (L - steps)[None]).to(dt)[None, :, :, None]       # gamma^(L-1-j)
    qh, kh, vh, doh = (x.permute(0, 2, 1, 3) for x in (q, k, v, d_out))

    P = (doh @ vh.transpose(-1, -2)) * D * s                                  # [B,H,L,L]
    do_w = doh * read_w
    dq = P @ kh + do_w @ state.transpose(-1, -2)
    dk_ = P.transpose(-1, -2) @ qh + (vh @ d_new_state.transpose(-1, -2)) * key_w * s
    A = (qh @ kh.transpose(-1, -2)) * D * s
    dv = A.transpose(-1, -2) @ doh + ((kh * s * key_w) @ d_new_state)
    dstate = qh.transpose(-1, -2) @ do_w + d_new_state * (g ** L)[None, :, None, None].to(dt)
    back = lambda x: x.permute(0, 2, 1, 3)
    return back(dq), back(dk_), back(dv), dstate


def recurrent_step(q: Tensor, k: Tensor, v: Tensor, state: Optional[Tensor], decays: Sequence[float]):
    """One token: S <- gamma S + (k / sqrt(dk))^T v ; o = q S   (flash_pop/retnet.py:79-101).
    q, k: [B,H,dk], v: [B,H,dv]."""
    g = _gammas(decays, q).to(q.dtype)
    new_state = (k / (k.shape[-1] ** 0.5))[..., :, None] * v[..., None, :]
    if state is not None:
        new_state = new_state + state * g[None, :, None, None]
    out = (q[..., None, :] @ new_state).squeeze(-2)
    return out, new_state


def pop_suffix_retention(q_sfx: Tensor, k_sfx: Tensor, v_sfx: Tensor, state0: Optional[Tensor],
                         block_states: Tensor, decays: Sequence[float], chunk_size: int = 512):
    """POP suffixes (flash_pop/pop_retnet.py:152-171): suffix n of batch item b starts from the
    state BEFORE block n, i.e. state0 (zeros if None) for n = 0 and block_states[b, n-1] after;
    suffix tokens never update the main state.  q_sfx etc. are [B*(N+1), Ls, H, d] with the
    block index fastest, block_states is [B, N, H, dk, dv].  Returns the suffix outputs."""
    B, N = block_states.shape[:2]
    first = torch.zeros_like(block_states[:, :1]) if state0 is None else state0[:, None].to(block_states.dtype)
    starts = torch.cat((first, block_states), dim=1).flatten(0, 1)
    assert q_sfx.shape[0] == B * (N + 1)
    out, _ = chunkwise_retention(q_sfx, k_sfx, v_sfx, starts, decays, chunk_size)
    return out


def pop_fused_retention(q: Tensor, k: Tensor, v: Tensor, state0: Optional[Tensor], q_sfx: Tensor, k_sfx: Tensor,
                        v_sfx: Tensor, decays: Sequence[float], block_size: int):
    """One POP layer step as the reference composes it (flash_pop/pop_retnet.py:107 then :152-171):
    the context through the block-state retention, then the N + 1 suffixes per sequence from
    [state0, block states].  Returns (o, o_sfx, state after the last FULL block), the last being
    what the reference keeps as the new recurrent state (`last_state = states[:, -1]`, :169); with
    no full block it is state0 (zeros if None)."""
    o, block_states = pop_retention(q, k, v, state0, decays, block_size)
    o_sfx = pop_suffix_retention(q_sfx, k_sfx, v_sfx, state0, block_states, decays)
    if block_states.shape[1] > 0:
        last = block_states[:, -1]
    elif state0 is not None:
        last = state0
    else:
        last = q.new_zeros(q.shape[0], q.shape[2], q.shape[3], v.shape[3])
    return o, o_sfx, last


def rms_error_ratio(approx: Tensor, ref: Tensor) -> float:
    """RMS(approx - ref) / RMS(ref): the metric the reference's tests hold outputs and states to,
    with the bar 0.005 (tests/test_fused_retention.py:36-39,119,131)."""
    a, r = approx.double().flatten(), ref.double().flatten()
    return ((a - r).square().mean().sqrt() / r.square().mean().sqrt().clamp_min(1e-300)).item()
