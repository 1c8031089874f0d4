"""The C-language parity program (tests/c_abi_parity.c): host code in C over the ABI of
include/iris_dev.h, as the reference's callers are, checked against the oracle from C."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "c_abi_parity.bin")


def _run():
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-s", "-C", ROOT, "ctest"])
    return subprocess.run([BIN], capture_output=True, text=True, timeout=110)


def test_c_program_reports_missing_gpu():
    """Without a gfx950 device iris_dev_init() fails and the program says so: no CPU fallback."""
    import ctypes
    try:
        n = ctypes.c_int(0)
        has_gpu = ctypes.CDLL("libamdhip64.so").hipGetDeviceCount(ctypes.byref(n)) == 0 and n.value > 0
    except OSError:
        has_gpu = False
    if has_gpu:
        pytest.skip("a GPU is present; the GPU test covers the program")
    r = _run()
    assert r.returncode == 3 and "no usable gfx950 device" in r.stderr


@pytest.mark.gpu
def test_c_program_parity_on_gpu():
    r = _run()
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout and "kernel: fa_hd512" in r.stdout


@pytest.mark.gpu
def test_path_only_archive_runs_behind_a_host_backend():
    """tests/path_only_link.c: a host program with its own init / memory entries / stream, linked against
    libiris_dev_path.a, normalises Q and K and runs attention over a constant V: every output must be that constant."""
    exe = os.path.join(ROOT, "tests", "path_only_link.bin")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-s", "-C", ROOT, "path", "pathcheck"])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and r.stdout.startswith("ok (fa_hd128)"), r.stdout + r.stderr
