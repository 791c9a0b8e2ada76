"""A minimal POP-RetNet decoder around the retention ops, for model-level parity tests and the
model leg of the benchmark.  Test infrastructure: plain torch modules, written for this harness.

It follows the structure of the reference's model (flash_pop/retnet.py:105-366 multi-scale
retention, :370-512 decoder layer, flash_pop/pop_retnet.py:82-171 POP layer step,
flash_pop/xpos_emb.py rotary embedding): pre-LayerNorm in fp32, q/k rotated by position * theta,
retention, GroupNorm over each head's outputs (fp32, no affine, eps 1e-6), swish gate, output
projection, swish FFN.  Unlike the reference, d_model need not equal H * dv: v and the gate are
projected d_model -> H * dv and the output H * dv -> d_model, which reduces to the reference's
layer when the two are equal.

The retention, the rotary embedding of q and k and the normalisation + gate come from a backend
object, so that the same seeded model can run on the HIP ops and on plain fp32 torch formulas
(the oracle's for the retention; evaluated on whatever device the tensors are on).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F


@dataclass
class HarnessConfig:
    vocab: int = 32000
    d_model: int = 768
    layers: int = 12
    heads: int = 12
    dk: int = 64
    dv: int = 128
    ffn: int = 3072
    block: int = 64          # context tokens per observation block
    sfx_len: int = 16        # prediction tokens per POP suffix
    dtype: torch.dtype = torch.bfloat16


def head_decays(heads: int) -> tuple:
    return tuple(1.0 - 2.0 ** (-5.0 - h) for h in range(heads))       # flash_pop/retnet.py:70-76


class HipBackend:
    """The ops of flash_pop_amd."""
    name = "hip"

    def __init__(self, layer_ops: bool = True):
        """layer_ops=False keeps the rotary embedding and the normalisation + gate as eager torch
        formulas around the HIP retention ops (what a caller that only switches the ops gets)."""
        self._xpos = {}
        self.layer_ops = layer_ops

    def plain(self, q, k, v, s, decays):
        from flash_pop_amd import fused_chunk_retention
        return fused_chunk_retention(q, k, v, s, decays)

    def pop(self, q, k, v, s, decays, block, q_s, k_s, v_s):
        from flash_pop_amd import flash_pop_retention_with_suffixes
        return flash_pop_retention_with_suffixes(q, k, v, s, decays, block, q_s, k_s, v_s)

    def step(self, q, k, v, s, decays, in_place=False):
        from flash_pop_amd import retention_recurrent
        return retention_recurrent(q, k, v, decays, s, in_place=in_place)

    def rotate(self, q, k, start):
        if not self.layer_ops:
            return OracleBackend.rotate(self, q, k, start)
        from flash_pop_amd import XPos
        d = q.shape[-1]
        if d not in self._xpos:
            self._xpos[d] = XPos(d)
        return self._xpos[d](q, k, start)

    def norm_gate(self, retention, gate):
        if not self.layer_ops:
            return OracleBackend.norm_gate(self, retention, gate)
        from flash_pop_amd import gated_group_norm
        return gated_group_norm(retention, gate, 1e-6)


class OracleBackend:
    """The oracle's formulas in fp32 on the bf16 inputs, results rounded to bf16 like the ops' outputs."""
    name = "oracle"

    def plain(self, q, k, v, s, decays):
        import oracle
        o, S = oracle.chunkwise_retention(q.float(), k.float(), v.float(), None if s is None else s.float(), decays, 64)
        return o.to(q.dtype), S.to(q.dtype)

    def pop(self, q, k, v, s, decays, block, q_s, k_s, v_s):
        import oracle
        f = lambda t: None if t is None else t.float()
        o, o_s, last = oracle.pop_fused_retention(f(q), f(k), f(v), f(s), f(q_s), f(k_s), f(v_s), decays, block)
        return o.to(q.dtype), o_s.to(q.dtype), last.to(q.dtype)

    def rotate(self, q, k, start):
        return rotate(q, start), rotate(k, start)

    def norm_gate(self, retention, gate):
        r = retention.float()
        r = (r - r.mean(-1, keepdim=True)) * torch.rsqrt(r.var(-1, unbiased=False, keepdim=True) + 1e-6)
        return r.flatten(-2).to(gate.dtype) * F.silu(gate)

    def step(self, q, k, v, s, decays, in_place=False):
        import oracle
        o, S = oracle.recurrent_step(q.float(), k.float(), v.float(), None if s is None else s.float(), decays)
        return o.to(q.dtype), S.to(q.dtype)


def rotate(x: torch.Tensor, start) -> torch.Tensor:
    """Pairs (x[2i], x[2i+1]) rotated by position * theta_i, theta_i = 10000^(-i / (d/2 - 1))
    (flash_pop/xpos_emb.py:24-40).  x [B, T, H, d]; the position of token t of sequence b is
    start + t (start an int) or start[b] + t (start an integer tensor of B elements)."""
    d, T = x.shape[-1], x.shape[1]
    theta = 1.0 / (10000.0 ** torch.linspace(0, 1, d // 2)).to(x.device)
    first = start.reshape(-1, 1) if isinstance(start, torch.Tensor) else start
    positions = first + torch.arange(T, device=x.device)[None]              # [B or 1, T]
    ang = positions[..., None, None].float() * theta                       # [B or 1, T, 1, d/2]
    sin, cos = torch.sin(ang), torch.cos(ang)
    xf = x.float()
    even, odd = xf[..., 0::2], xf[..., 1::2]
    out = torch.stack((even * cos - odd * sin, odd * cos + even * sin), dim=-1).flatten(-2)
    return out.to(x.dtype)


class Retention(nn.Module):
    def __init__(self, cfg: HarnessConfig):
        super().__init__()
        self.cfg = cfg
        D, H, dk, dv = cfg.d_model, cfg.heads, cfg.dk, cfg.dv
        self.q_proj = nn.Linear(D, H * dk)
        self.k_proj = nn.Linear(D, H * dk)
        self.v_proj = nn.Linear(D, H * dv)
        self.g_proj = nn.Linear(D, H * dv)
        self.out_proj = nn.Linear(H * dv, D)
        for lin in (self.q_proj, self.k_proj, self.v_proj, self.g_proj, self.out_proj):
            nn.init.xavier_normal_(lin.weight)
            nn.init.zeros_(lin.bias)
        self.decays = head_decays(H)

    def qkv(self, backend, x, start):
        """x [B, T, D]; start: position of the first token, an int or one integer per sequence."""
        H, dk, dv = self.cfg.heads, self.cfg.dk, self.cfg.dv
        q, k = backend.rotate(self.q_proj(x).unflatten(-1, (H, dk)), self.k_proj(x).unflatten(-1, (H, dk)), start)
        v = self.v_proj(x).unflatten(-1, (H, dv))
        return q, k, v

    def finish(self, backend, x, retention):
        """GroupNorm per head in fp32, swish gate, output projection.  retention [..., H, dv]."""
        return self.out_proj(backend.norm_gate(retention, self.g_proj(x)))


class Layer(nn.Module):
    def __init__(self, cfg: HarnessConfig):
        super().__init__()
        self.cfg = cfg
        self.norm1 = nn.LayerNorm(cfg.d_model, eps=1e-6)
        self.norm2 = nn.LayerNorm(cfg.d_model, eps=1e-6)
        self.retention = Retention(cfg)
        self.linear1 = nn.Linear(cfg.d_model, cfg.ffn)
        self.linear2 = nn.Linear(cfg.ffn, cfg.d_model)
        for lin in (self.linear1, self.linear2):
            nn.init.xavier_normal_(lin.weight)
            nn.init.zeros_(lin.bias)

    def _norm(self, norm, x):
        return F.layer_norm(x.float(), (self.cfg.d_model,), norm.weight.float(), norm.bias.float(), norm.eps).to(x.dtype)

    def _ffn(self, x):
        return x + self.linear2(F.silu(self.linear1(self._norm(self.norm2, x))))

    def pop_forward(self, backend, x, sfx, start, state):
        """x [B,T,D], sfx [B*(N+1), Ls, D]: the layer step of flash_pop/pop_retnet.py:82-150, with
        both retentions handed to the backend in one call.  Returns (x, sfx, last state)."""
        r, cfg = self.retention, self.cfg
        B, T = x.shape[:2]
        n1 = sfx.shape[0] // B
        xn, sn = self._norm(self.norm1, x), self._norm(self.norm1, sfx)
        sfx_start = (start + torch.arange(n1, device=x.device) * cfg.block).repeat(B)       # pop_retnet.py:175-179
        q, k, v = r.qkv(backend, xn, start)
        qs, ks, vs = r.qkv(backend, sn, sfx_start)
        o, o_s, last = backend.pop(q, k, v, state, r.decays, cfg.block, qs, ks, vs)
        x = self._ffn(x + r.finish(backend, xn, o))
        sfx = self._ffn(sfx + r.finish(backend, sn, o_s))
        return x, sfx, last

    def chunkwise(self, backend, x, start, state):
        r = self.retention
        xn = self._norm(self.norm1, x)
        q, k, v = r.qkv(backend, xn, start)
        o, state = backend.plain(q, k, v, state, r.decays)
        return self._ffn(x + r.finish(backend, xn, o)), state

    def recurrent(self, backend, x, index, state, in_place=False):
        """x [B, D], one token at position `index` (an int, or a one-element tensor on the device)
        (flash_pop/retnet.py:325-366, 493-512)."""
        r = self.retention
        xn = self._norm(self.norm1, x)
        start = index.expand(x.shape[0]) if isinstance(index, torch.Tensor) else index
        q, k, v = r.qkv(backend, xn[:, None], start)
        o, state = backend.step(q[:, 0], k[:, 0], v[:, 0], state, r.decays, in_place=in_place)
        return self._ffn(x + r.finish(backend, xn, o)), state


class PopRetNetLM(nn.Module):
    def __init__(self, cfg: HarnessConfig):
        super().__init__()
        self.cfg = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.d_model)
        self.layers = nn.ModuleList(Layer(cfg) for _ in range(cfg.layers))
        self.norm = nn.LayerNorm(cfg.d_model, eps=1e-6)
        self.head = nn.Linear(cfg.d_model, cfg.vocab, bias=False)
        nn.init.normal_(self.embed.weight, std=cfg.d_model ** -0.5)
        nn.init.normal_(self.head.weight, std=cfg.d_model ** -0.5)

    def _logits(self, x):
        x = F.layer_norm(x.float(), (self.cfg.d_model,), self.norm.weight.float(), self.norm.bias.float(), self.norm.eps)
        return self.head(x.to(self.cfg.dtype))

    def pop_forward(self, backend, tokens, sfx_tokens, states: Optional[List] = None, start: int = 0):
        """tokens [B,T] (T a multiple of the block), sfx_tokens [B*(T/block + 1), Ls].
        Returns (context logits, suffix logits, per-layer last states)."""
        x, sfx = self.embed(tokens), self.embed(sfx_tokens)
        states = states if states is not None else [None] * len(self.layers)
        new_states = []
        for layer, st in zip(self.layers, states):
            x, sfx, last = layer.pop_forward(backend, x, sfx, start, st)
            new_states.append(last)
        return self._logits(x), self._logits(sfx), new_states

    def chunkwise(self, backend, tokens, states: Optional[List] = None, start: int = 0):
        x = self.embed(tokens)
        states = states if states is not None else [None] * len(self.layers)
        new_states = []
        for layer, st in zip(self.layers, states):
            x, st = layer.chunkwise(backend, x, start, st)
            new_states.append(st)
        return self._logits(x), new_states

    @torch.no_grad()
    def recurrent(self, backend, token, states: List, index, in_place=False):
        """One decode step: token [B] -> (logits [B, vocab], new states)."""
        x = self.embed(token)
        new_states = []
        for layer, st in zip(self.layers, states):
            x, st = layer.recurrent(backend, x, index, st, in_place)
            new_states.append(st)
        return self._logits(x), new_states


class GraphedGreedyDecoder:
    """Greedy decoding with one decode step captured in a HIP graph: the step is a chain of small
    launches (12 layers of projections, norms and the decode-step kernel), so replaying it as a
    graph removes the per-launch host cost.  Everything the step reads or writes lives in fixed
    buffers: the token, the position, the per-layer states (updated in place) and the logits."""

    def __init__(self, model: PopRetNetLM, backend, states: List, token: torch.Tensor, index: int):
        self.model, self.backend = model, backend
        self.states = [s.clone().contiguous() for s in states]
        self.token = token.clone()
        self.pos = torch.full((1,), index, device=token.device, dtype=torch.long)
        self.logits = None
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):            # warm-up outside the capture: lazy initialisation, autotuning
            keep = [s.clone() for s in self.states], self.token.clone(), self.pos.clone()
            for _ in range(2):
                self._step()
            for dst, src in zip(self.states, keep[0]):
                dst.copy_(src)
            self.token.copy_(keep[1])
            self.pos.copy_(keep[2])
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._step()

    def _step(self):
        logits, _ = self.model.recurrent(self.backend, self.token, self.states, self.pos, in_place=True)
        self.logits = logits
        self.token.copy_(logits.argmax(-1))
        self.pos.add_(1)

    def step(self):
        """Advance by one token; returns the logits buffer (overwritten by the next step)."""
        self.graph.replay()
        return self.logits


def build(cfg: HarnessConfig, seed: int, device) -> PopRetNetLM:
    torch.manual_seed(seed)
    model = PopRetNetLM(cfg)          # initialised on the CPU: the same weights whatever the device
    return model.to(device=device, dtype=cfg.dtype)


def synthetic_batch(cfg: HarnessConfig, B: int, T: int, seed: int, device):
    """Uniform random token ids for the context, the suffixes and their next-token targets."""
    g = torch.Generator().manual_seed(seed)
    n1 = T // cfg.block + 1
    draw = lambda *shape: torch.randint(0, cfg.vocab, shape, generator=g).to(device)
    return draw(B, T), draw(B * n1, cfg.sfx_len), draw(B, T), draw(B * n1, cfg.sfx_len)


def pop_loss(model: PopRetNetLM, backend, batch):
    tokens, sfx_tokens, targets, sfx_targets = batch
    logits, sfx_logits, states = model.pop_forward(backend, tokens, sfx_tokens)
    loss = F.cross_entropy(logits.float().flatten(0, 1), targets.flatten()) + \
        F.cross_entropy(sfx_logits.float().flatten(0, 1), sfx_targets.flatten())
    return loss, logits, sfx_logits, states
