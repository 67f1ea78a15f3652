"""Builds and runs the C++ unit tests of the plugin's host code (no GPU)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "tensorflow-allreduce_amd", "csrc", "host")


def test_wire_format_and_framework_types(tmp_path):
    exe = str(tmp_path / "wire_test")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-fsanitize=address,undefined",
                    "-fno-sanitize-recover=all", "-I", HOST, "-o", exe,
                    os.path.join(ROOT, "tests", "cpp", "wire_test.cc"),
                    os.path.join(HOST, "wire.cc"), os.path.join(HOST, "framework.cc")], check=True)
    # the harness preloads a library of its own; the sanitizer runtime must come first
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=0")
    out = subprocess.run([exe], check=True, capture_output=True, text=True, env=env)
    assert out.stdout.strip() == "ok"


def test_coordinator_under_thread_sanitizer(tmp_path):
    """The readiness table, the background thread and the op contexts with one
    thread per rank, built from source with -fsanitize=thread. No GPU: the
    submitted collectives fail the cross-rank checks before any device work."""
    exe = str(tmp_path / "coordinator_test")
    lib_dir = os.path.join(ROOT, "tensorflow-allreduce_amd", "lib")
    sources = [os.path.join(HOST, f) for f in ("framework.cc", "wire.cc", "ring_driver.cc", "transport.cc", "collective_ops.cc")]
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Wextra", "-fsanitize=thread", "-pthread",
                    "-I", HOST, "-I", os.path.join(ROOT, "include"), "-o", exe,
                    os.path.join(ROOT, "tests", "cpp", "coordinator_test.cc")] + sources +
                   ["-L", lib_dir, "-lring_hip", "-Wl,-rpath," + lib_dir], check=True)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:report_signal_unsafe=0")
    out = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr
