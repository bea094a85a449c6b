"""Runs tests/cpp/test_quant_kernel.bin: the reference crate's own unit tests replayed
through the C++ mirror of its interface (include/oxq/quant_kernel.hpp -> C ABI)."""
import os
import subprocess

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "test_quant_kernel.bin")


def _run(mode):
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built: run `python -m oxillama_amd.build`")
    p = subprocess.run([BIN, mode], capture_output=True, text=True, timeout=120)
    print(p.stdout)
    print(p.stderr)
    assert p.returncode == 0, p.stdout[-4000:]
    assert " 0 failed" in p.stdout


def test_cpp_mirror_host_cases():
    _run("--host")


@pytest.mark.gpu
def test_cpp_mirror_gpu_cases():
    _run("--gpu")
