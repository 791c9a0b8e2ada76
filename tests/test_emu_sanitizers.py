"""Builds the CPU thread harness and the C-ABI layer with AddressSanitizer and UBSan and runs
every entry point on exact-size heap buffers (tests/emu/asan_driver.cpp).  An out-of-bounds access
of a kernel body, in global memory or in its LDS block, or undefined integer behaviour fails here,
on the host, instead of faulting a GPU."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
EMU = os.path.join(HERE, "emu")


def test_all_entry_points_under_asan_and_ubsan(tmp_path):
    exe = str(tmp_path / "asan_driver")
    build_env = dict(os.environ, EMU_OUT=exe, EMU_MAIN=os.path.join(EMU, "asan_driver.cpp"), EMU_OPT="-O1",
                     EMU_FLAGS="-fsanitize=address,undefined -fno-sanitize-recover=all -fno-omit-frame-pointer")
    subprocess.run([os.path.join(EMU, "build_emu.sh")], check=True, env=build_env)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    res = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=1500)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-6000:]
    assert res.stdout.count("ok ") == 40 and "FAILED" not in res.stdout, res.stdout
