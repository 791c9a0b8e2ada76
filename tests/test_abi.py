"""The C-ABI library loads, exports every symbol include/flashpop_hip.h declares, and rejects
bad arguments before touching a GPU (so these run on a CPU-only machine)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flashpop_hip.h")


@pytest.fixture(scope="module")
def lib():
    from flash_pop_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return _lib.load()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(lib):
    from flash_pop_amd import _lib
    names = declared_functions()
    assert names == sorted(_lib.SIGNATURES), (names, sorted(_lib.SIGNATURES))
    for n in names:
        assert hasattr(lib, n), f"{n} not exported"
    assert lib.fp_version() == 1008


def test_argument_checks_return_codes(lib):
    dec = (ctypes.c_double * 2)(0.9, 0.95)
    p = ctypes.c_void_p(0x1000)   # never dereferenced: every call below fails its checks first
    null = None
    ok_dims = (1, 8, 2, 64, 64)
    assert lib.fp_retention_fwd(null, p, p, null, dec, p, null, *ok_dims, None) == -1
    assert b"NULL" in lib.fp_last_error()
    assert lib.fp_retention_fwd(p, p, p, null, None, p, null, *ok_dims, None) == -1
    assert lib.fp_retention_fwd(p, p, p, null, dec, p, null, 1, 0, 2, 64, 64, None) == -2
    assert lib.fp_retention_fwd(p, p, p, null, dec, p, null, 1, 8, 2, 96, 64, None) == -3
    assert b"dk and dv" in lib.fp_last_error()
    assert lib.fp_retention_fwd(p, p, p, null, dec, p, null, 1, 8, 2, 64, 32, None) == -3
    bad = (ctypes.c_double * 2)(0.9, 1.5)
    assert lib.fp_retention_fwd(p, p, p, null, bad, p, null, *ok_dims, None) == -4
    bad0 = (ctypes.c_double * 2)(0.0, 0.5)
    assert lib.fp_retention_fwd(p, p, p, null, bad0, p, null, *ok_dims, None) == -4
    assert lib.fp_retention_bwd(p, p, p, null, dec, null, null, p, p, p, null, *ok_dims, None) == -1
    # fused POP op: positive block size and suffix length, head dims of 64, 128 or 256, no NULL tensors
    fused = lambda T, dk, blk, ls, o_sfx=p: lib.fp_pop_fused_fwd(p, p, p, null, p, p, p, dec, p, o_sfx, null,
                                                                 1, T, 2, dk, 64, blk, ls, None)
    assert fused(100, 64, 0, 16) == -2 and b"block_size" in lib.fp_last_error()
    assert fused(128, 64, 64, 0) == -2 and b"suffix length" in lib.fp_last_error()
    assert fused(128, 256, 64, 65) == -3 and b"suffixes longer than" in lib.fp_last_error()
    assert fused(128, 96, 64, 16) == -3
    assert fused(128, 64, 64, 16, null) == -1
    assert lib.fp_pop_fused_bwd(p, p, p, null, p, p, p, dec, p, null, null, p, p, p, p, p, p, null,
                                1, 128, 2, 64, 64, 64, 16, None) == -1
    assert lib.fp_pop_retention_fwd(p, p, p, null, dec, p, p, *ok_dims, 0, None) == -2
    assert lib.fp_pop_retention_fwd(p, p, p, null, dec, p, null, *ok_dims, 4, None) == -1
    assert lib.fp_pop_retention_bwd(p, p, p, null, dec, p, p, p, p, null, null, *ok_dims, 4, None) == -1
    big = (ctypes.c_double * 513)(*([0.9] * 513))
    assert lib.fp_retention_fwd(p, p, p, null, big, p, null, 1, 8, 513, 64, 64, None) == -2   # more than 512 heads


def test_backward_choice_switch_checks_its_arguments(lib):
    assert lib.fp_set_backward_choice(4, -1) == -6 and b"backward choice" in lib.fp_last_error()
    assert lib.fp_set_backward_choice(0, 100) == -6 and b"multiple of 64" in lib.fp_last_error()
    assert lib.fp_set_backward_choice(1, 256) == 0
    n = ctypes.c_int(-1)
    # the passes are forced: no checkpoints are asked for, whatever the shape
    assert lib.fp_retention_checkpoint_bytes(8, 4096, 16, 128, 128, ctypes.byref(n)) == 0 and n.value == 0
    assert lib.fp_set_backward_choice(2, 256) == 0
    assert lib.fp_retention_checkpoint_bytes(1, 4096, 1, 128, 128, ctypes.byref(n)) == 2 * 16 * 128 * 128 and n.value == 256
    assert lib.fp_set_backward_choice(0, 512) == 0


def test_environment_switches_are_validated_once():
    """FLASHPOP_BWD / FLASHPOP_CKPT are read once per process; a value that is neither of the
    documented ones makes every entry point fail (checked in child processes: nothing is launched)."""
    import subprocess
    import sys
    from flash_pop_amd import _lib
    code = ("import ctypes, sys; sys.path.insert(0, %r); from flash_pop_amd import _lib; lib = _lib.load();"
            "d = (ctypes.c_double * 1)(0.9); p = ctypes.c_void_p(0x1000);"
            "rc = lib.fp_retention_fwd(None, p, p, None, d, p, None, 1, 8, 1, 64, 64, None);"
            "print(rc, lib.fp_last_error().decode())") % os.path.dirname(os.path.dirname(_lib.LIB_PATH))
    run = lambda env: subprocess.run([sys.executable, "-c", code], env={**os.environ, **env}, capture_output=True, text=True).stdout
    assert run({"FLASHPOP_BWD": "fuse"}).startswith("-6 FLASHPOP_BWD=fuse")
    assert run({"FLASHPOP_CKPT": "100"}).startswith("-6 FLASHPOP_CKPT=100")
    assert run({"FLASHPOP_BWD": "passes", "FLASHPOP_CKPT": "256"}).startswith("-1 ")
    assert run({"FLASHPOP_BWD": "paced"}).startswith("-1 ")


def test_python_wrappers_refuse_cpu_tensors():
    import torch
    from flash_pop_amd import fused_chunk_retention, flash_pop_retention
    q = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        fused_chunk_retention(q, q, q, None, (0.9, 0.9))
    with pytest.raises(RuntimeError, match="GPU only"):
        flash_pop_retention(q, q, q, None, (0.9, 0.9), 4)
    with pytest.raises(AssertionError, match="bfloat16"):
        fused_chunk_retention(q.float(), q.float(), q.float(), None, (0.9, 0.9))
    with pytest.raises(AssertionError, match="head decays"):
        fused_chunk_retention(q, q, q, None, (0.9,))


def test_new_entry_points_check_their_arguments(lib):
    dec = (ctypes.c_double * 2)(0.9, 0.95)
    p, null = ctypes.c_void_p(0x1000), None
    # decode step: shape, NULL and dimension checks come before any launch
    assert lib.fp_retention_decode_step(p, p, p, null, dec, p, null, 1, 2, 64, 64, None) == -1
    assert lib.fp_retention_decode_step(p, p, p, null, dec, p, p, 1, 2, 64, 96, None) == -3
    assert lib.fp_retention_decode_step(p, p, p, null, dec, p, p, 0, 2, 64, 64, None) == -2
    # split entry points: same checks as the plain ones, and an invalid shape needs no workspace
    assert lib.fp_retention_workspace_bytes(0, 64, 2, 64, 64) == 0
    assert lib.fp_retention_workspace_bytes(1, 64, 2, 96, 64) == 0
    assert lib.fp_retention_fwd_split(null, p, p, null, dec, p, null, 1, 8, 2, 64, 64, null, 0, None) == -1
    assert lib.fp_retention_bwd_split(p, p, p, null, dec, null, null, p, p, p, null, 1, 8, 2, 64, 64, null, 0, 0, None) == -1


def test_new_python_wrappers_refuse_cpu_tensors():
    import torch
    from flash_pop_amd import flash_pop_retention_with_suffixes, retention_recurrent
    q = torch.zeros(1, 8, 2, 64, dtype=torch.bfloat16)
    sfx = torch.zeros(3, 2, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        flash_pop_retention_with_suffixes(q, q, q, None, (0.9, 0.9), 4, sfx, sfx, sfx)
    x = torch.zeros(1, 2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        retention_recurrent(x, x, x, (0.9, 0.9), None)
    with pytest.raises(ValueError, match=r"\[B,H,dk\]"):
        retention_recurrent(x[0], x[0], x[0], (0.9, 0.9), None)


def test_layer_entry_points_check_their_arguments(lib):
    p, odd, null = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1008), None
    # rotary: NULLs, k given on one side only, shape, head dimension, alignment
    assert lib.fp_rotary_qk(null, p, p, p, p, null, 0, 1, 4, 2, 64, 0, None) == -1
    assert lib.fp_rotary_qk(p, p, p, p, null, null, 0, 1, 4, 2, 64, 0, None) == -1
    assert lib.fp_rotary_qk(p, p, p, null, p, null, 0, 1, 4, 2, 64, 0, None) == -1
    assert lib.fp_rotary_qk(p, p, p, p, p, null, 0, 1, 0, 2, 64, 0, None) == -2
    assert lib.fp_rotary_qk(p, p, p, p, p, null, 0, 1, 4, 2, 60, 0, None) == -3
    assert lib.fp_rotary_qk(odd, p, p, p, p, null, 0, 1, 4, 2, 64, 0, None) == -2
    assert b"aligned" in lib.fp_last_error()
    # gated norm: NULLs, rows, group width (8 * 2^k <= 512), eps, alignment
    assert lib.fp_gated_group_norm_fwd(p, null, p, 4, 2, 64, 1e-6, None) == -1
    assert lib.fp_gated_group_norm_bwd(p, p, p, p, null, 4, 2, 64, 1e-6, None) == -1
    assert lib.fp_gated_group_norm_fwd(p, p, p, 0, 2, 64, 1e-6, None) == -2
    assert lib.fp_gated_group_norm_fwd(p, p, p, 4, 2, 96, 1e-6, None) == -3
    assert lib.fp_gated_group_norm_fwd(p, p, p, 4, 2, 1024, 1e-6, None) == -3
    assert lib.fp_gated_group_norm_fwd(p, p, p, 4, 2, 64, -1.0, None) == -2
    assert lib.fp_gated_group_norm_bwd(p, p, odd, p, p, 4, 2, 64, 1e-6, None) == -2


def test_layer_wrappers_refuse_cpu_tensors_and_bad_shapes():
    import torch
    from flash_pop_amd import XPos, gated_group_norm
    q = torch.zeros(2, 8, 2, 64, dtype=torch.bfloat16)
    xpos = XPos(64)
    assert xpos.thetas.shape == (32,) and float(xpos.thetas[0]) == 1.0
    with pytest.raises(RuntimeError, match="GPU only"):
        xpos(q, q, 0)
    with pytest.raises(AssertionError, match="head dimension"):
        XPos(128)(q, q, 0)
    with pytest.raises(RuntimeError, match="GPU only"):
        gated_group_norm(q, q.flatten(-2))


def test_pass_ops_refuse_graph_capture(monkeypatch):
    """Capturing the pass kernels into a HIP graph has crashed the host process, so the Python
    ops raise while the current stream is capturing.  The flag is mocked: no GPU is touched."""
    import torch
    from flash_pop_amd import _ops
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    q = torch.zeros(1, 4, 1, 64, dtype=torch.bfloat16)
    sfx = (q, q, q)
    calls = [
        lambda: _ops.retention_fwd(q, q, q, None, (0.9,), (1, 4, 1, 64, 64)),
        lambda: _ops.pop_retention_fwd(q, q, q, None, (0.9,), 2, (1, 4, 1, 64, 64)),
        lambda: _ops.retention_bwd(q, q, q, None, (0.9,), (1, 4, 1, 64, 64), q, None, None, None, False),
        lambda: _ops.pop_fused_fwd(q, q, q, None, sfx, (0.9,), 2, (1, 4, 1, 64, 64)),
        lambda: _ops.pop_fused_bwd(q, q, q, None, sfx, (0.9,), 2, (1, 4, 1, 64, 64), q, q, None, False),
    ]
    for call in calls:
        with pytest.raises(RuntimeError, match="cannot be captured into a HIP graph"):
            call()
    # the small kernels (decode step, rotary, gated norm) stay capturable: no guard in their wrappers
    import inspect
    for name in ("decode_step", "rotary_qk", "gated_norm_fwd", "gated_norm_bwd"):
        assert "refuse_capture" not in inspect.getsource(getattr(_ops, name))
