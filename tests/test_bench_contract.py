"""bench.py's host-side pieces that need no GPU: the byte and FLOP counts it prices the step with,
the traffic figure it reads back from profiles/, and its refusal to run on more than one GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_algorithmic_counts_of_config2():
    """Per token and head: forward 2 (2 dk + 2 dv) bytes and 2 [C (dk + dv) + 2 dk dv] FLOP, backward
    2 (4 dk + 3 dv) bytes and 2 [C (3 dk + 2 dv) + 4 dk dv] FLOP, chunk C = 64."""
    B, T, H, d = 8, 4096, 16, 128
    b_fwd, b_bwd = bench.algorithmic_bytes(B, T, H, d, d)
    f_fwd, f_bwd = bench.algorithmic_flops(B, T, H, d, d)
    n = B * T * H
    assert (b_fwd, b_bwd) == (4 * n * d * 2, 7 * n * d * 2) == (536870912, 939524096)
    assert f_fwd == n * 2 * (64 * 256 + 2 * 128 * 128) and f_bwd == n * 2 * (64 * 640 + 4 * 128 * 128)
    assert abs((f_fwd + f_bwd) / 1e9 - 163.2) < 0.1 and abs((b_fwd + b_bwd) / 1e9 - 1.476) < 1e-3


def test_traffic_is_read_from_the_profile_summaries():
    nbytes, commit = bench.profiled_traffic("retention_bwd_fused_kernel")
    assert nbytes is not None and commit, "profiles/ holds no HBM_TRAFFIC line for the backward kernel"
    # more than the algorithm's 939.5 MB (the dq walk reads k, v, dO again), less than twice that
    assert 939524096 < nbytes < 2 * 939524096
    assert bench.profiled_traffic("no_such_kernel") == (None, None)


def test_more_than_one_gpu_is_refused():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "one GPU only" in res.stderr
