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
