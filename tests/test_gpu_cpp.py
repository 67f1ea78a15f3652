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


@pytest.mark.gpu
def test_reference_side_binding_keeps_the_synchronous_seam():
    """tensorflow-allreduce_amd/integration/ring_hip_binding.cc, the file that
    replaces the reference's ring.cu.cc: CopyTensorData<GPUDevice> and
    AccumulateTensorData<GPUDevice, T> called as ring.h calls them, complete on
    return, and the reference's loop over them, bit-exact against the oracle."""
    exe = os.path.join(ROOT, "tests", "cpp", "build", "binding_gpu_test")
    assert os.path.exists(exe), "build it first: python tensorflow-allreduce_amd/build.py"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr
