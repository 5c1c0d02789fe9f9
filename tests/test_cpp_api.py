"""Runs the C++ header-layer test binary (tests/cpp/test_core_api.cpp): the dlprim::core
names over the C ABI, used the way the reference's own callers use them."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "bin", "test_core_api")


def run(arg):
    if not os.path.exists(BIN):
        pytest.fail("tests/bin/test_core_api is not built: run `make -C tests/cpp` (or __graft_entry__.build())")
    r = subprocess.run([BIN, arg], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok" in r.stdout


def test_cpp_host_side():
    run("host")


@pytest.mark.gpu
def test_cpp_core_api_on_device():
    run("0")
