"""Runs the native parity program: the C++ launcher mirror (include/rivoli_launchers.hpp) driven
with plain HIP allocations, no Python in the loop, checked against the CPU oracle by the program
itself. It is built ahead of time by tests/native/Makefile (part of the build entry point)."""
import os
import subprocess

import pytest

from tests.gpu_util import torch_cuda

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "native", "launchers_parity")


@pytest.mark.gpu
def test_native_launchers_parity():
    torch_cuda()                                            # skips where there is no GPU
    if not os.path.exists(BIN):
        pytest.skip("native parity program not built (the build entry point runs make -C tests/native)")
    res = subprocess.run([BIN], capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stdout + res.stderr
    lines = res.stdout.strip().splitlines()
    assert lines[-1] == "native parity ok" and not [ln for ln in lines if ln.startswith("FAIL")], res.stdout
    assert sum(ln.startswith("ok") for ln in lines) >= 12


def test_native_program_is_built_by_the_build_entry_point():
    """The round's GPU box does not compile: the binary must come from the build step."""
    with open(os.path.join(os.path.dirname(HERE), "__graft_entry__.py")) as f:
        assert '"tests", "native"' in f.read()
