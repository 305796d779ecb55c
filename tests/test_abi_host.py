"""The C ABI without torch: tests/abi_host_check.cpp (plain HIP host code, hipMalloc'd buffers, its
own stream) is built by tests/Makefile (ahead of time, or here when it is missing) and run as a child process."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "_build", "abi_host_check")


def _need_binary():
    """The program is built ahead of time (by __graft_entry__.build()); when nothing is built yet -- a fresh checkout --
    build it, and the two libraries it links, here."""
    if os.path.exists(BIN):
        return
    from af3_kernels_amd import build as hip_build
    from oracle import af3_oracle
    hip_build.build()
    af3_oracle.build()
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "tests")], capture_output=True, text=True)
    if r.returncode != 0 or not os.path.exists(BIN):
        pytest.fail(f"could not build {BIN}:\n{r.stdout}{r.stderr}")


def test_host_program_links_the_library_and_lists_its_cases():
    _need_binary()
    r = subprocess.run([BIN, "--list"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == "abi version 4" and len(lines) >= 5


@pytest.mark.gpu
def test_c_callers_get_the_formula_through_the_abi_alone():
    _need_binary()
    print("running", BIN, flush=True)
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count(" ok") >= 9 and "FAIL" not in r.stdout
