"""Model-level parity: a small POP-RetNet decoder (tests/model_harness.py) run once on the HIP ops
and once on the oracle's formulas, from the same seeded weights and tokens.  Everything around the
retention is the same torch code in both runs, so what is compared is how the ops' bf16 rounding
propagates through layers, loss and gradients."""
import pytest
import torch

import model_harness as mh
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SMALL = dict(vocab=512, d_model=256, layers=2, heads=4, dk=64, dv=128, ffn=512, block=64, sfx_len=16)


def _say(msg):
    print(msg, flush=True)


def _ratio(a, b):
    return oracle.rms_error_ratio(a.detach().float().cpu(), b.detach().float().cpu())


def test_pop_training_step_hip_vs_oracle_backend():
    cfg = mh.HarnessConfig(**SMALL)
    B, T = 2, 256
    _say(f"[model] POP step, {cfg.layers} layers d_model {cfg.d_model} H{cfg.heads} dk{cfg.dk} dv{cfg.dv} B{B} T{T}")
    batch = mh.synthetic_batch(cfg, B, T, seed=3, device=DEV)
    results = {}
    for backend in (mh.HipBackend(), mh.OracleBackend()):
        model = mh.build(cfg, seed=11, device=DEV)
        loss, logits, sfx_logits, states = mh.pop_loss(model, backend, batch)
        loss.backward()
        torch.cuda.synchronize()
        results[backend.name] = (loss.item(), logits, sfx_logits, states,
                                 {n: p.grad for n, p in model.named_parameters()})
    hip, ref = results["hip"], results["oracle"]
    assert abs(hip[0] - ref[0]) < 2e-3 * abs(ref[0]), (hip[0], ref[0])
    assert _ratio(hip[1], ref[1]) < 2e-2 and _ratio(hip[2], ref[2]) < 2e-2
    for a, b in zip(hip[3], ref[3]):
        assert _ratio(a, b) < 1e-2
    worst = max((_ratio(hip[4][n], g), n) for n, g in ref[4].items() if g is not None)
    _say(f"[model] loss {hip[0]:.5f} vs {ref[0]:.5f}; logits {_ratio(hip[1], ref[1]):.4f}; worst grad {worst}")
    assert all(g is not None and torch.isfinite(g).all() for g in hip[4].values())
    assert worst[0] < 5e-2, worst


def test_recurrent_decode_continues_the_pop_states():
    """Context through pop_forward, then 32 tokens one at a time with the decode-step kernel from
    the states it returned, against the chunkwise forward over all the tokens at once."""
    cfg = mh.HarnessConfig(**SMALL)
    B, T, extra = 2, 128, 32
    backend = mh.HipBackend()
    model = mh.build(cfg, seed=12, device=DEV).eval()
    g = torch.Generator().manual_seed(5)
    tokens = torch.randint(0, cfg.vocab, (B, T + extra), generator=g).to(DEV)
    sfx = torch.randint(0, cfg.vocab, (B * (T // cfg.block + 1), cfg.sfx_len), generator=g).to(DEV)
    with torch.no_grad():
        full_logits, _ = model.chunkwise(backend, tokens)
        ctx_logits, _, states = model.pop_forward(backend, tokens[:, :T], sfx)
        assert _ratio(ctx_logits, full_logits[:, :T]) < 1e-2
        outs = []
        for t in range(extra):
            logits, states = model.recurrent(backend, tokens[:, T + t], states, T + t)
            outs.append(logits)
    torch.cuda.synchronize()
    r = _ratio(torch.stack(outs, dim=1), full_logits[:, T:])
    _say(f"[model] decode vs chunkwise logits, RMS ratio {r:.4f}")
    assert r < 3e-2


def test_graph_captured_decode_step_equals_eager():
    """One decode step captured in a HIP graph and replayed 12 times, with eager work and
    synchronisations between the replays; every replay is compared with the eager decode loop."""
    cfg = mh.HarnessConfig(**SMALL)
    B, T, steps = 2, 64, 12
    backend = mh.HipBackend()
    model = mh.build(cfg, seed=13, device=DEV).eval()
    g = torch.Generator().manual_seed(6)
    tokens = torch.randint(0, cfg.vocab, (B, T), generator=g).to(DEV)
    with torch.no_grad():
        _, states = model.chunkwise(backend, tokens)
        first = tokens[:, -1].clone()
        eager_logits, eager_tokens, st, tok = [], [], [s.clone() for s in states], first
        for i in range(steps):
            logits, st = model.recurrent(backend, tok, st, T + i)
            tok = logits.argmax(-1)
            eager_logits.append(logits.clone())
            eager_tokens.append(tok.clone())
        dec = mh.GraphedGreedyDecoder(model, backend, states, first, T)
        for i in range(steps):
            logits = dec.step().clone()
            torch.cuda.synchronize()
            scratch = torch.randn(256, 256, device=DEV) @ torch.randn(256, 256, device=DEV)   # unrelated eager work
            torch.cuda.synchronize()
            assert torch.equal(logits, eager_logits[i]), f"replay {i}: logits differ from the eager step"
            assert torch.equal(dec.token, eager_tokens[i]), f"replay {i}"
            del scratch
        assert int(dec.pos.item()) == T + steps
