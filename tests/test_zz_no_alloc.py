"""The entry point that allocates nothing: fp_retention_fwd_split_static keeps its segment states
in the library's own device array.  Called through the C ABI and compared bit for bit with
fp_retention_fwd_split (caller's workspace) on calls in a row, each with a smaller input than
the one before; sizes beyond the array are rejected."""
import pytest
import torch

import helpers as hp
import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _static_fwd(lib, q, k, v, s, decays, stream=None):
    B, T, H, dk = q.shape
    dv = v.shape[3]
    o = torch.full((B, T, H, dv), float("nan"), dtype=hp.BF16, device=q.device)
    S = torch.full((B, H, dk, dv), float("nan"), dtype=hp.BF16, device=q.device)
    rc = lib.fp_retention_fwd_split_static(hp._p(q), hp._p(k), hp._p(v), hp._p(s), hp._dec(decays), hp._p(o), hp._p(S),
                                           B, T, H, dk, dv, stream)
    return rc, o, S


def test_static_scratch_forward_matches_workspace_forward(hip_lib):
    lib = hip_lib
    stream = torch.cuda.current_stream().cuda_stream
    # the long-context benchmark shape (B2 H8 T16384 dk128 dv256: 16 MiB of segment states, the whole array),
    # then two smaller calls on the same array, the last one the smallest
    for B, T, H, dk, dv, seed in ((2, 16384, 8, 128, 256, 4), (1, 4096, 2, 128, 128, 5), (1, 2048, 2, 128, 128, 6)):
        print(f"[no-alloc] B{B} T{T} H{H} dk{dk} dv{dv}", flush=True)
        decays = oracle.head_decays(H)
        q, k, v, s = hp.make_inputs(B, T, H, dk, dv, seed=seed, state_std=0.1, device=DEV)
        assert 0 < lib.fp_retention_workspace_bytes(B, T, H, dk, dv) <= (16 << 20), "the shape is meant to be cut into segments"
        o_ref, S_ref, _ = hp.raw_split_fwd(lib, q, k, v, s, decays, stream)
        rc, o, S = _static_fwd(lib, q, k, v, s, decays, stream)
        torch.cuda.synchronize()
        assert rc == 0, lib.fp_last_error().decode()
        assert torch.equal(o, o_ref) and torch.equal(S, S_ref)
        o_or, S_or = hp.oracle_plain(q, k, v, s, decays, device=DEV)
        hp.assert_close(o, o_or, "o", head_dim=2)
        hp.assert_close(S, S_or, "S", head_dim=1)


def test_static_scratch_rejects_what_does_not_fit(hip_lib):
    """Segment states take 64 KiB x max(dk, dv) x compute units / 256: more than the 16 MiB array only on a
    device with more than 256 compute units.  Where such a shape exists the call must refuse it."""
    lib = hip_lib
    B, T, H, d = 1, 32768, 1, 256
    if lib.fp_retention_workspace_bytes(B, T, H, d, d) <= (16 << 20):
        pytest.skip("no supported shape needs more than the 16 MiB array on this device")
    q = torch.zeros(B, T, H, d, dtype=hp.BF16, device=DEV)
    rc, _, _ = _static_fwd(lib, q, q, q, None, oracle.head_decays(H))
    assert rc == -2 and b"scratch" in lib.fp_last_error()
