"""Tensor-level plumbing shared by the two autograd Functions: checks, allocation, raw calls."""
from __future__ import annotations

import ctypes

import torch

from . import _lib


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def refuse_capture(what):
    """The pass kernels must not be recorded into a HIP graph: instantiating a graph that holds
    them has crashed the host process (a segmentation fault inside the runtime, after every
    launch had been recorded without error).  Until that is understood the ops raise instead."""
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError(
            f"{what} cannot be captured into a HIP graph with this ROCm / PyTorch build "
            "(graph instantiation crashes the process); call it eagerly, outside torch.cuda.graph")


def prepare(q, k, v, s, head_decays):
    """Validate like the reference's asserts (fused_retention/__init__.py:20,
    pop_retention/__init__.py:17-18) and return contiguous tensors plus the shape."""
    if q.dim() != 4 or k.shape != q.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise ValueError(f"expected q, k [B,T,H,dk] and v [B,T,H,dv]; got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    B, T, H, dk = q.shape
    dv = v.shape[3]
    assert len(head_decays) == H, f"got {len(head_decays)} head decays for {H} heads"
    for name, t in (("q", q), ("k", k), ("v", v), ("s", s)):
        if t is None:
            continue
        assert t.dtype == torch.bfloat16, f"{name}: only bfloat16 is supported, got {t.dtype}"
        if not t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}: flash_pop_amd runs on the GPU only")
    if s is not None and tuple(s.shape) != (B, H, dk, dv):
        raise ValueError(f"expected state [B,H,dk,dv] = {(B, H, dk, dv)}, got {tuple(s.shape)}")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    s = None if s is None else s.contiguous()
    return q, k, v, s, (B, T, H, dk, dv)


def _workspace(lib, shape, device):
    """Scratch for the split-sequence entry points: long sequences with few (batch, head) streams
    are cut into segments so that the whole device works on them.  None when the library would not
    cut this shape.  The tensor comes from torch's stream-ordered allocator, so handing it back
    right after the call is safe."""
    nbytes = lib.fp_retention_workspace_bytes(*shape)
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


def retention_fwd(q, k, v, s, decays, shape, for_backward=False):
    """-> (o, s_out, states or None, checkpoint interval).  With `for_backward` the forward also
    leaves the states that make the backward cheaper, where the library says they pay: checkpoints
    every `interval` tokens, or (interval 0) the workspace of a forward that cut its sequences into
    segments, which holds the state at the start of every segment."""
    refuse_capture("retention_fwd")
    lib = _lib.load()
    B, T, H, dk, dv = shape
    o = torch.empty((B, T, H, dv), dtype=q.dtype, device=q.device)
    s_out = torch.empty((B, H, dk, dv), dtype=q.dtype, device=q.device)
    ckpt, every = None, 0
    with torch.cuda.device(q.device):
        ws = _workspace(lib, shape, q.device)
        if ws is None and for_backward:
            n = ctypes.c_int(0)
            nbytes = lib.fp_retention_checkpoint_bytes(B, T, H, dk, dv, ctypes.byref(n))
            if nbytes:
                every = n.value
                ckpt = torch.empty((B, T // every, H, dk, dv), dtype=q.dtype, device=q.device)
        if ckpt is not None:
            rc = lib.fp_retention_fwd_ckpt(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(o),
                                           _ptr(s_out), _ptr(ckpt), every, B, T, H, dk, dv, _stream())
        elif ws is None:
            rc = lib.fp_retention_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(o),
                                      _ptr(s_out), B, T, H, dk, dv, _stream())
        else:
            rc = lib.fp_retention_fwd_split(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(o),
                                            _ptr(s_out), B, T, H, dk, dv, _ptr(ws), ws.numel(), _stream())
    _lib.check(lib, rc)
    return o, s_out, ckpt if ckpt is not None else (ws if for_backward else None), every


def pop_retention_fwd(q, k, v, s, decays, block_size, shape):
    refuse_capture("pop_retention_fwd")
    lib = _lib.load()
    B, T, H, dk, dv = shape
    o = torch.empty((B, T, H, dv), dtype=q.dtype, device=q.device)
    states = torch.empty((B, T // block_size, H, dk, dv), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.fp_pop_retention_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(o),
                                      _ptr(states) if states.numel() else None, B, T, H, dk, dv, block_size, _stream())
    _lib.check(lib, rc)
    return o, states


def retention_bwd(q, k, v, s, decays, shape, d_o, d_s_out, d_blocks, block_size, want_ds0, ckpt=None, every=0,
                  states_kept=True):
    """Gradients for both ops; block_size is None for the plain op.  ckpt, every: what retention_fwd
    left for this call (every = 0 with a tensor: the forward's workspace, which still holds the
    forward's segment states if `states_kept`)."""
    refuse_capture("retention_bwd")
    lib = _lib.load()
    B, T, H, dk, dv = shape
    d_o = d_o.contiguous()
    d_s_out = None if d_s_out is None else d_s_out.contiguous()
    d_blocks = None if d_blocks is None or d_blocks.numel() == 0 else d_blocks.contiguous()
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    d_s0 = torch.empty((B, H, dk, dv), dtype=q.dtype, device=q.device) if want_ds0 else None
    with torch.cuda.device(q.device):
        kept = ckpt is not None and every == 0      # the workspace of a forward that cut its sequences
        ws = ckpt if kept else _workspace(lib, shape, q.device) if block_size is None else None
        if ckpt is not None and not kept and block_size is None:
            rc = lib.fp_retention_bwd_ckpt(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(d_o),
                                           _ptr(d_s_out), _ptr(ckpt), every, _ptr(dq), _ptr(dk_), _ptr(dv_), _ptr(d_s0),
                                           B, T, H, dk, dv, _stream())
        elif ws is not None:
            rc = lib.fp_retention_bwd_split(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(d_o),
                                            _ptr(d_s_out), _ptr(dq), _ptr(dk_), _ptr(dv_), _ptr(d_s0), B, T, H, dk, dv,
                                            _ptr(ws), ws.numel(), int(kept and states_kept), _stream())
        elif block_size is None:
            rc = lib.fp_retention_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(d_o),
                                      _ptr(d_s_out), _ptr(dq), _ptr(dk_), _ptr(dv_), _ptr(d_s0), B, T, H, dk, dv,
                                      _stream())
        else:
            rc = lib.fp_pop_retention_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(d_o),
                                          _ptr(d_blocks), _ptr(dq), _ptr(dk_), _ptr(dv_), _ptr(d_s0), B, T, H, dk, dv,
                                          block_size, _stream())
    _lib.check(lib, rc)
    return dq, dk_, dv_, d_s0


def prepare_suffixes(q_sfx, k_sfx, v_sfx, shape, block_size):
    """Checks of the suffix batch as POPDecoderLayer._suffixes_forward makes them
    (flash_pop/pop_retnet.py:154-159): one suffix per block boundary, N + 1 per sequence."""
    B, T, H, dk, dv = shape
    n = B * (T // block_size + 1)
    if q_sfx.dim() != 4 or k_sfx.shape != q_sfx.shape or v_sfx.dim() != 4 or v_sfx.shape[:3] != q_sfx.shape[:3]:
        raise ValueError("expected q_sfx, k_sfx [B*(N+1),Ls,H,dk] and v_sfx [B*(N+1),Ls,H,dv]")
    if q_sfx.shape[0] != n or q_sfx.shape[2] != H or q_sfx.shape[3] != dk or v_sfx.shape[3] != dv:
        raise ValueError(f"got suffix tensors {tuple(q_sfx.shape)}, {tuple(v_sfx.shape)} for {n} suffixes of "
                         f"{H} heads with dk={dk}, dv={dv}: make sure there is one additional suffix block")
    for name, t in (("q_sfx", q_sfx), ("k_sfx", k_sfx), ("v_sfx", v_sfx)):
        assert t.dtype == torch.bfloat16, f"{name}: only bfloat16 is supported, got {t.dtype}"
        if not t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}: flash_pop_amd runs on the GPU only")
    return q_sfx.contiguous(), k_sfx.contiguous(), v_sfx.contiguous()


def pop_fused_fwd(q, k, v, s, sfx, decays, block_size, shape):
    refuse_capture("pop_fused_fwd")
    lib = _lib.load()
    B, T, H, dk, dv = shape
    o = torch.empty((B, T, H, dv), dtype=q.dtype, device=q.device)
    o_sfx = torch.empty_like(sfx[2])
    s_out = torch.empty((B, H, dk, dv), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.fp_pop_fused_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _ptr(sfx[0]), _ptr(sfx[1]), _ptr(sfx[2]),
                                  _lib.decays_array(decays), _ptr(o), _ptr(o_sfx), _ptr(s_out), B, T, H, dk, dv,
                                  block_size, sfx[0].shape[1], _stream())
    _lib.check(lib, rc)
    return o, o_sfx, s_out


def pop_fused_bwd(q, k, v, s, sfx, decays, block_size, shape, d_o, d_o_sfx, d_s_out, want_ds0):
    refuse_capture("pop_fused_bwd")
    lib = _lib.load()
    B, T, H, dk, dv = shape
    d_o, d_o_sfx = d_o.contiguous(), d_o_sfx.contiguous()
    d_s_out = None if d_s_out is None else d_s_out.contiguous()
    outs = [torch.empty_like(t) for t in (q, k, v, *sfx)]
    d_s0 = torch.empty((B, H, dk, dv), dtype=q.dtype, device=q.device) if want_ds0 else None
    with torch.cuda.device(q.device):
        rc = lib.fp_pop_fused_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _ptr(sfx[0]), _ptr(sfx[1]), _ptr(sfx[2]),
                                  _lib.decays_array(decays), _ptr(d_o), _ptr(d_o_sfx), _ptr(d_s_out),
                                  *[_ptr(t) for t in outs], _ptr(d_s0), B, T, H, dk, dv, block_size,
                                  sfx[0].shape[1], _stream())
    _lib.check(lib, rc)
    return outs, d_s0


def decode_step(q, k, v, s, decays, in_place=False):
    """q, k [B,H,dk], v [B,H,dv], s [B,H,dk,dv] or None -> (o [B,H,dv], new state)."""
    lib = _lib.load()
    if q.dim() != 3 or k.shape != q.shape or v.dim() != 3 or v.shape[:2] != q.shape[:2]:
        raise ValueError(f"expected q, k [B,H,dk] and v [B,H,dv]; got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    B, H, dk = q.shape
    dv = v.shape[2]
    assert len(decays) == H, f"got {len(decays)} head decays for {H} heads"
    for name, t in (("q", q), ("k", k), ("v", v), ("s", s)):
        if t is None:
            continue
        assert t.dtype == torch.bfloat16, f"{name}: only bfloat16 is supported, got {t.dtype}"
        if not t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}: flash_pop_amd runs on the GPU only")
    if s is not None and tuple(s.shape) != (B, H, dk, dv):
        raise ValueError(f"expected state [B,H,dk,dv] = {(B, H, dk, dv)}, got {tuple(s.shape)}")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    if in_place:
        if s is None or not s.is_contiguous():
            raise ValueError("an in-place step needs a contiguous state tensor")
        s_out = s
    else:
        s = None if s is None else s.contiguous()
        s_out = torch.empty((B, H, dk, dv), dtype=q.dtype, device=q.device)
    o = torch.empty((B, H, dv), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = lib.fp_retention_decode_step(_ptr(q), _ptr(k), _ptr(v), _ptr(s), _lib.decays_array(decays), _ptr(o),
                                          _ptr(s_out), B, H, dk, dv, _stream())
    _lib.check(lib, rc)
    return o, s_out


def _check_bf16_cuda(**tensors):
    for name, t in tensors.items():
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}: flash_pop_amd runs on the GPU only")
        assert t.dtype == torch.bfloat16, f"{name}: only bfloat16 is supported, got {t.dtype}"


def rotary_qk(q, k, theta, start, inverse=False):
    """q, k [B,T,H,d] (k may be None) rotated by position * theta; start an int or an int64 tensor [B]."""
    lib = _lib.load()
    _check_bf16_cuda(q=q, k=k)
    if q.dim() != 4 or (k is not None and k.shape != q.shape):
        raise ValueError(f"expected q, k [B,T,H,d]; got {tuple(q.shape)}, {None if k is None else tuple(k.shape)}")
    B, T, H, d = q.shape
    if tuple(theta.shape) != (d // 2,) or theta.dtype != torch.float32 or theta.device != q.device:
        raise ValueError(f"theta must be {d // 2} floats on {q.device}")
    start0 = 0
    if isinstance(start, torch.Tensor):
        if start.dim() != 1 or start.shape[0] != B:
            raise ValueError(f"start positions: expected one per sequence ({B}), got shape {tuple(start.shape)}")
        start = start.to(device=q.device, dtype=torch.long).contiguous()
    else:
        start0, start = int(start), None
    q = q.contiguous()
    k = None if k is None else k.contiguous()
    q_out = torch.empty_like(q)
    k_out = None if k is None else torch.empty_like(k)
    if q.numel() == 0:
        return q_out, k_out
    with torch.cuda.device(q.device):
        rc = lib.fp_rotary_qk(_ptr(q), _ptr(k), _ptr(q_out), _ptr(k_out), _ptr(theta.contiguous()), _ptr(start), start0,
                              B, T, H, d, int(bool(inverse)), _stream())
    _lib.check(lib, rc)
    return q_out, k_out


def _norm_shapes(r, g):
    if r.dim() < 2 or g.numel() != r.numel() or g.shape[-1] != r.shape[-2] * r.shape[-1]:
        raise ValueError(f"expected r [..., H, dv] and g [..., H * dv]; got {tuple(r.shape)}, {tuple(g.shape)}")
    H, dv = r.shape[-2:]
    return r.numel() // (H * dv), H, dv


def gated_norm_fwd(r, g, eps):
    """bf16(GroupNorm per head of r) * bf16(swish(g)): r [..., H, dv], g [..., H*dv] -> [..., H*dv]."""
    lib = _lib.load()
    _check_bf16_cuda(r=r, g=g)
    rows, H, dv = _norm_shapes(r, g)
    r, g = r.contiguous(), g.contiguous()
    out = torch.empty_like(g)
    if rows == 0:
        return out
    with torch.cuda.device(r.device):
        rc = lib.fp_gated_group_norm_fwd(_ptr(r), _ptr(g), _ptr(out), rows, H, dv, float(eps), _stream())
    _lib.check(lib, rc)
    return out


def gated_norm_bwd(r, g, d_out, eps):
    lib = _lib.load()
    _check_bf16_cuda(r=r, g=g, d_out=d_out)
    rows, H, dv = _norm_shapes(r, g)
    d_out = d_out.contiguous()
    d_r, d_g = torch.empty_like(r), torch.empty_like(g)
    if rows == 0:
        return d_r, d_g
    with torch.cuda.device(r.device):
        rc = lib.fp_gated_group_norm_bwd(_ptr(r), _ptr(g), _ptr(d_out), _ptr(d_r), _ptr(d_g), rows, H, dv, float(eps),
                                         _stream())
    _lib.check(lib, rc)
    return d_r, d_g
