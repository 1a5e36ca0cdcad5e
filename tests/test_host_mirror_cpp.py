"""The C++ host-side mirror (izwi_amd/host/izwi_qmm.hpp) through its own test program.

The program is built by __graft_entry__.build() (tests/cpp/Makefile); on a machine
without the binary the CPU test builds it with g++ first.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "host_mirror_test")


def _binary(may_build: bool) -> str:
    if not os.path.exists(BINARY):
        if not may_build:
            pytest.fail("tests/cpp/host_mirror_test is not built (run __graft_entry__.build())")
        subprocess.check_call(["make", "-C", os.path.join(HERE, "cpp")])
    return BINARY


def _run(mode: str, may_build: bool):
    fixture = os.path.join(HERE, "golden", "tiny.gguf")
    proc = subprocess.run([_binary(may_build), mode, fixture], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "all checks passed" in proc.stdout


def test_cpp_mirror_host_logic():
    _run("cpu", may_build=True)


def test_cpp_mirror_fails_loudly_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    _run("nodevice", may_build=True)


@pytest.mark.gpu
def test_cpp_mirror_reference_packed_case_and_q4k_projection():
    _run("gpu", may_build=False)
