"""The benchmark's literal tolerance, rtol = atol = 2e-2, as a measurement.

The inputs are unnormalised N(0,1) tensors, so retention sums reach an RMS of 4 to more than 100 per head
and any evaluation with bf16 operands leaves the literal bar |x - ref| <= 2e-2 + 2e-2 |ref| for a share of
the small elements.  That holds for the reference's own bf16 PyTorch path too, which is how
MultiScaleRetention calls chunkwise_retention (flash_pop/retnet.py:243-245, 287-289: bf16 tensors, chunk
size 512, retnet.py:138) and what the reference's tests put beside the kernel (tests/test_fused_retention.py:
76-96, bf16 and fp32 reference side by side).  Here both are held against the same fp32 oracle on the same
inputs at the full size of benchmark configurations 2, 3 and 4: the share of elements outside the literal bar
for the HIP ops must not exceed what the reference's bf16 path leaves outside (times 1.25, with a floor for
tensors where both are nearly clean)."""
import pytest
import torch

import helpers as hp
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MARGIN = 1.25
FLOOR = 2e-3          # shares below this are within noise of each other (a few hundred elements per million)
REF_CHUNK = 512       # MultiScaleRetention.Config.chunk_size, the chunk of the reference's PyTorch path


def _shares(got, ref):
    return hp.error_report(got, ref)["frac_outside"]


def _report(title, names, hip, bf16):
    print(f"[literal 2e-2] {title}: share of elements outside |x - ref| <= 2e-2 + 2e-2 |ref| (worst batch entry)", flush=True)
    print(f"[literal 2e-2]   {'tensor':8s} {'HIP ops':>10s} {'reference bf16 path':>20s}", flush=True)
    for n in names:
        print(f"[literal 2e-2]   {n:8s} {hip[n]:10.3e} {bf16[n]:20.3e}", flush=True)
    for n in names:
        assert hip[n] <= max(MARGIN * bf16[n], FLOOR), (
            f"{title}, {n}: {hip[n]:.3e} of the HIP result is outside the literal bar, the reference's bf16 path leaves {bf16[n]:.3e}")


def _plain(B, T, H, dk, dv, state_std, seed, with_ds):
    from flash_pop_amd import fused_chunk_retention
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=seed, state_std=state_std)
    d_o, d_s = hp.make_cotangents([(B, T, H, dv), (B, H, dk, dv)], seed=seed + 1)
    leaves = [t.to(DEV).requires_grad_() for t in (q, k, v, s)]
    o, S = fused_chunk_retention(*leaves, decays)
    torch.autograd.backward([o, S], [d_o.to(DEV), d_s.to(DEV) if with_ds else torch.zeros_like(S)])
    names = ["o", "S", "dq", "dk", "dv", "ds0"]
    hip, bf16 = dict.fromkeys(names, 0.0), dict.fromkeys(names, 0.0)
    for b in range(B):
        sl = slice(b, b + 1)
        args = (q[sl], k[sl], v[sl], s[sl], decays, d_o[sl], d_s[sl] if with_ds else None)
        o32, S32, g32 = hp.oracle_plain(*args, device=DEV)
        o16, S16, g16 = hp.oracle_plain(*args, chunk=REF_CHUNK, dtype=torch.bfloat16, device=DEV)
        got = [o[sl], S[sl]] + [l.grad[sl] for l in leaves]
        for n, x, x16, ref in zip(names, got, [o16, S16, *g16], [o32, S32, *g32]):
            hip[n] = max(hip[n], _shares(x, ref))
            bf16[n] = max(bf16[n], _shares(x16, ref))
    return names, hip, bf16


def test_config2_against_the_reference_bf16_path():
    _report("config 2 (B8 H16 T4096 dk = dv = 128)", *_plain(8, 4096, 16, 128, 128, 0.0, seed=0, with_ds=False))


def test_config3_against_the_reference_bf16_path():
    _report("config 3 (B2 H8 T16384 dk128 dv256, carried state)", *_plain(2, 16384, 8, 128, 256, 0.02, seed=3, with_ds=True))


def test_config4_against_the_reference_bf16_path():
    """The fused POP op against the reference's composition of its two bf16 calls (the context in blocks of 64
    tokens as tests/test_pop_retention.py:13-32 runs it, the suffixes through chunkwise_retention)."""
    from flash_pop_amd.pop_retention import flash_pop_retention_with_suffixes
    B, N, block, Ls, H, dk, dv = 8, 64, 64, 16, 16, 128, 128
    T = N * block
    decays = oracle.head_decays(H)
    q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=40, state_std=0.05)
    sfx = hp.make_suffix_inputs(B, N, Ls, H, dk, dv, seed=41)
    cot = hp.make_cotangents([(B, T, H, dv), tuple(sfx[2].shape), (B, H, dk, dv)], seed=42)
    ctx = [t.to(DEV).requires_grad_() for t in (q, k, v, s)]
    sx = [t.to(DEV).requires_grad_() for t in sfx]
    o, o_sfx, last = flash_pop_retention_with_suffixes(*ctx, decays, block, *sx)
    torch.autograd.backward([o, o_sfx, last], [c.to(DEV) for c in cot])
    names = ["o", "o_sfx", "last", "dq", "dk", "dv", "dq_sfx", "dk_sfx", "dv_sfx", "ds0"]
    hip, bf16 = dict.fromkeys(names, 0.0), dict.fromkeys(names, 0.0)
    for b in range(B):
        sl, ssl = slice(b, b + 1), slice(b * (N + 1), (b + 1) * (N + 1))
        args = (q[sl], k[sl], v[sl], s[sl], [t[ssl] for t in sfx], decays, block, (cot[0][sl], cot[1][ssl], cot[2][sl]))
        o32, os32, l32, g32 = hp.oracle_fused(*args, device=DEV)
        o16, os16, l16, g16 = hp.oracle_fused(*args, dtype=torch.bfloat16, device=DEV)
        leaves = ctx[:3] + sx + [ctx[3]]
        got = [o[sl], o_sfx[ssl], last[sl]] + [l.grad[ssl if i in (3, 4, 5) else sl] for i, l in enumerate(leaves)]
        for n, x, x16, ref in zip(names, got, [o16, os16, l16, *g16], [o32, os32, l32, *g32]):
            hip[n] = max(hip[n], _shares(x, ref))
            bf16[n] = max(bf16[n], _shares(x16, ref))
    _report("config 4 (config 2 in 64-token blocks + 65 suffixes x 16 tokens per sequence)", names, hip, bf16)
