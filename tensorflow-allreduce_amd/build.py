"""Builds the native libraries of this package in-tree for gfx950.

    python tensorflow-allreduce_amd/build.py

  lib/libring_hip.so      HIP kernels + the C ABI of include/ring_abi.h
                          (csrc/ring_kernels.hip), linked against the HIP
                          runtime only.
  lib/libmpi_collectives.so
                          the plugin library (csrc/host/*.cc): op registry, the
                          six MPI ops and their kernels, readiness table,
                          background thread and host-side ring driver. Plain
                          C++ (g++), no GPU code; calls libring_hip.so through
                          the C ABI.

  tests/cpp/build/ring_gpu_test
                          a C++ test of the C ABI (test code, linked with the
                          oracle), run on the GPU by tests/test_gpu_cpp.py.
  tests/cpp/build/binding_gpu_test
                          integration/ring_hip_binding.cc (the file that takes
                          the place of the reference's ring.cu.cc) with its
                          test, run on the GPU by tests/test_gpu_cpp.py.

hipcc cross-compiles for gfx950 without a GPU. Packed FP32 instructions are
disabled for all device code.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_DIR = os.path.join(HERE, "lib")
RING_HIP_SO = os.path.join(LIB_DIR, "libring_hip.so")
PLUGIN_SO = os.path.join(LIB_DIR, "libmpi_collectives.so")
HOST_SOURCES = ["framework.cc", "wire.cc", "ring_driver.cc", "transport.cc", "collective_ops.cc"]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-pthread", "-Wall", "-Wextra"]

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-fno-fast-math", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-command-line-argument",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (expected on PATH or at /opt/rocm/bin/hipcc)")
    return exe


def build_ring_hip(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc()] + HIP_FLAGS + [
        "-I", os.path.join(ROOT, "include"),
        "-o", RING_HIP_SO,
        os.path.join(HERE, "csrc", "ring_kernels.hip"),
    ]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return RING_HIP_SO


def build_plugin(verbose=True):
    """libmpi_collectives.so; needs libring_hip.so to link against."""
    cxx = shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("g++ not found")
    cmd = [cxx] + CXX_FLAGS + [
        "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc", "host"),
        "-o", PLUGIN_SO,
    ] + [os.path.join(HERE, "csrc", "host", f) for f in HOST_SOURCES] + [
        "-L", LIB_DIR, "-lring_hip", "-Wl,-rpath,$ORIGIN",
    ]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed:\n" + res.stdout)
    if verbose and res.stdout.strip():
        print(res.stdout)
    return PLUGIN_SO


def build_cpp_gpu_test(verbose=True):
    """tests/cpp/build/ring_gpu_test: the C ABI exercised from C++ without Python
    or torch, checked against the C oracle. Built here (on the CPU) so the GPU
    run only has to execute it."""
    cxx = shutil.which("g++") or shutil.which("c++")
    out_dir = os.path.join(ROOT, "tests", "cpp", "build")
    os.makedirs(out_dir, exist_ok=True)
    exe = os.path.join(out_dir, "ring_gpu_test")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    obj = os.path.join(out_dir, "ring_oracle.o")
    cmds = [
        ["gcc", "-O2", "-std=gnu11", "-fno-fast-math", "-c", os.path.join(ROOT, "oracle", "ring_oracle.c"), "-o", obj],
        [cxx, "-O2", "-std=c++17", "-Wall", "-Wextra", "-pthread", "-D__HIP_PLATFORM_AMD__",
         "-I", os.path.join(rocm, "include"), "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "oracle"),
         "-o", exe, os.path.join(ROOT, "tests", "cpp", "ring_gpu_test.cc"), obj,
         "-L", LIB_DIR, "-lmpi_collectives", "-lring_hip", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
         "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath," + os.path.join(rocm, "lib")],
    ]
    # the reference-side binding (integration/ring_hip_binding.cc, the file that takes the place of
    # the reference's ring.cu.cc) and its test: the seam called as ring.h calls it
    binding_exe = os.path.join(out_dir, "binding_gpu_test")
    cmds.append([cxx, "-O2", "-std=c++17", "-Wall", "-Wextra", "-pthread", "-D__HIP_PLATFORM_AMD__",
                 "-I", os.path.join(rocm, "include"), "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "oracle"),
                 "-o", binding_exe, os.path.join(ROOT, "tests", "cpp", "binding_gpu_test.cc"),
                 os.path.join(HERE, "integration", "ring_hip_binding.cc"), obj,
                 "-L", LIB_DIR, "-lring_hip", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
                 "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath," + os.path.join(rocm, "lib")])
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if res.returncode != 0:
            raise RuntimeError("building the C++ GPU tests failed:\n" + res.stdout)
    return exe


def build_launch_bound_steps(verbose=True):
    """examples/build/launch_bound_steps: a small tensor's allreduce step driven
    from C++ through the C ABI, eager and as recorded HIP graphs (host clock)."""
    cxx = shutil.which("g++") or shutil.which("c++")
    out_dir = os.path.join(HERE, "examples", "build")
    os.makedirs(out_dir, exist_ok=True)
    exe = os.path.join(out_dir, "launch_bound_steps")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [cxx, "-O2", "-std=c++17", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(rocm, "include"), "-I", os.path.join(ROOT, "include"),
           "-o", exe, os.path.join(HERE, "examples", "launch_bound_steps.cc"),
           "-L", LIB_DIR, "-lmpi_collectives", "-lring_hip", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed:\n" + res.stdout)
    return exe


def build_all(verbose=True):
    return [build_ring_hip(verbose), build_plugin(verbose), build_cpp_gpu_test(verbose),
            build_launch_bound_steps(verbose)]


if __name__ == "__main__":
    for path in build_all():
        print("built", path)
    sys.exit(0)
