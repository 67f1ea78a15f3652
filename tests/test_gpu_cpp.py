"""Runs the prebuilt C++ test of the C ABI (tests/cpp/ring_gpu_test.cc) on the
GPU: the data path driven without Python or torch, bit-exact against the C
oracle for float32, int32 and int64 at 1-8 ranks, ragged counts included."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cpp", "build", "ring_gpu_test")


@pytest.mark.gpu
def test_c_abi_from_cpp_without_python():
    assert os.path.exists(EXE), "build it first: python tensorflow-allreduce_amd/build.py"
    out = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr
