"""Runs the C++ mirror of the Kernel / Layer interface (include/rmi_hip_kernel.hpp)
on the GPU; the binary is built by __graft_entry__.build()."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_kernel_hpp")


def test_cpp_header_compiles():
    """CPU check: the header and its test are valid C++17 against the C ABI (syntax only)."""
    subprocess.check_call(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "cpp", "test_kernel_hpp.cpp")])


@pytest.mark.gpu
def test_cpp_kernel_interface_on_gpu():
    assert os.path.exists(BIN), "tests/cpp/test_kernel_hpp is missing: run __graft_entry__.build()"
    out = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and "all C++ interface checks passed" in out.stdout
