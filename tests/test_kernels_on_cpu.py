"""Checks of the device code that need no GPU.

1. The kernel library compiled as plain C++ against a CPU stand-in of the HIP
   runtime (tests/cpp/hip_cpu_shim) and run under AddressSanitizer and UBSan
   (tests/cpp/kernel_emulation_test.cc): indexing and alignment of every kernel
   on exact-size buffers, results against plain loops.
2. A scan of the gfx950 assembly hipcc emits for the kernels: a scalar select
   (s_cselect) must take its condition code from a compare, not from whatever
   arithmetic instruction ran last. hipcc 7.2 has produced that for a uniform
   64-bit `min` ahead of a branch (v_cmp into vcc, branch on vcc, s_cselect on
   a stale SCC): every lane of a partial tile then ran, out of bounds on the
   GPU while the same source was correct on the CPU.
3. The plugin's host code linked over the same CPU build of the kernels
   (tests/cpp/plugin_emulation_test.cc): the coordinator's paths that end in a
   launch, under the sanitizers, against the C oracle.
4. ring_set_option against concurrent launches under ThreadSanitizer.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tensorflow-allreduce_amd", "csrc", "ring_kernels.hip")
BUILD = os.path.join(ROOT, "tests", "cpp", "build")
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fno-fast-math", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _clang():
    for exe in ("/opt/rocm/lib/llvm/bin/clang++", shutil.which("amdclang++"), shutil.which("clang++")):
        if exe and os.path.exists(exe):
            return exe
    return None


SANITIZERS = {
    "asan": ["-fsanitize=address,undefined", "-fno-sanitize-recover=all"],
    "tsan": ["-fsanitize=thread"],
}
SHIM = os.path.join(ROOT, "tests", "cpp", "hip_cpu_shim")


def _flags(sanitizer):
    return ["-std=c++17", "-O0", "-g"] + SANITIZERS[sanitizer] + ["-fno-omit-frame-pointer", "-pthread"]


def _run(cmd, **kw):
    __tracebackhide__ = True  # a failure shows the command and its output, not this frame's arguments (the environment)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    assert res.returncode == 0, " ".join(cmd) + "\n" + res.stdout[-4000:]
    return res.stdout


def _kernel_library_for_the_cpu(clang, sanitizer="asan"):
    """The kernel library as a sanitized CPU object, compiled once for the tests that link it."""
    os.makedirs(BUILD, exist_ok=True)
    obj = os.path.join(BUILD, "ring_kernels_cpu_%s.o" % sanitizer)
    sources = [SRC, os.path.join(ROOT, "include", "ring_abi.h"), os.path.join(SHIM, "hip", "hip_runtime.h"),
               os.path.join(SHIM, "hip", "hip_ext.h"), os.path.abspath(__file__)]
    if not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(f) for f in sources):
        _run([clang, "-x", "c++"] + _flags(sanitizer) + ["-I", SHIM, "-I", os.path.join(ROOT, "include"), "-c", "-o", obj, SRC])
    return obj


def test_kernels_under_sanitizers_on_the_cpu():
    clang = _clang()
    if clang is None:
        pytest.skip("no clang++ (the kernels use clang vector extensions)")
    obj = _kernel_library_for_the_cpu(clang)
    exe = os.path.join(BUILD, "kernel_emulation_test")
    _run([clang] + _flags("asan") + ["-I", SHIM, "-I", os.path.join(ROOT, "include"), "-o", exe,
                                     os.path.join(ROOT, "tests", "cpp", "kernel_emulation_test.cc"), obj])
    # The same cases once more under ThreadSanitizer, for one element type: the lanes of a workgroup are
    # threads and __syncthreads a real barrier, so a table in LDS that is read without a barrier behind its
    # writes is a data race it reports.
    tsan_exe = os.path.join(BUILD, "kernel_emulation_test_tsan")
    _run([clang] + _flags("tsan") + ["-I", SHIM, "-I", os.path.join(ROOT, "include"), "-o", tsan_exe,
                                     os.path.join(ROOT, "tests", "cpp", "kernel_emulation_test.cc"),
                                     _kernel_library_for_the_cpu(clang, "tsan")])
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:report_signal_unsafe=0")
    # one process per element type, side by side: the stand-in runs a workgroup's lanes as OS threads
    # and spends its time handing them work
    procs = [(t, subprocess.Popen([exe, t], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
             for t in ("float32", "int32", "int64")]
    procs.append(("float32 under ThreadSanitizer",
                  subprocess.Popen([tsan_exe, "float32"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)))
    for t, proc in procs:
        try:
            out, _ = proc.communicate(timeout=900)
        except subprocess.TimeoutExpired:
            for _, other in procs:
                other.kill()
            raise
        assert proc.returncode == 0 and "kernel emulation: ok" in out, t + "\n" + out[-4000:]


def test_random_shapes_through_the_emulated_kernels():
    """A short, fixed sweep of tests/cpp/kernel_emulation_fuzz.cc (random shapes,
    element types and launch options through the emulation test's cases); the
    program takes a seed and a case count for longer ones. Two seeds side by
    side."""
    clang = _clang()
    if clang is None:
        pytest.skip("no clang++ (the kernels use clang vector extensions)")
    obj = _kernel_library_for_the_cpu(clang)
    exe = os.path.join(BUILD, "kernel_emulation_fuzz")
    _run([clang] + _flags("asan") + ["-I", SHIM, "-I", os.path.join(ROOT, "include"), "-o", exe,
                                     os.path.join(ROOT, "tests", "cpp", "kernel_emulation_fuzz.cc"), obj])
    procs = [subprocess.Popen([exe, seed, "15"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
             for seed in ("1", "2")]
    for proc in procs:
        try:
            out, _ = proc.communicate(timeout=900)
        except subprocess.TimeoutExpired:
            for other in procs:
                other.kill()
            raise
        assert proc.returncode == 0 and "15 cases ok" in out, out[-3000:]


@pytest.mark.parametrize("sanitizer", ["asan", "tsan"])
def test_plugin_over_the_emulated_kernels_under_sanitizers(sanitizer):
    """The plugin's host code over the same CPU build of the kernel library:
    the coordinator's paths that end in a launch (separate rings of a tick,
    fused groups, prepared batches, allgather, a bad node among good ones,
    ranks submitting from threads of their own), bit for bit against the C
    oracle, once under AddressSanitizer and UBSan and once under
    ThreadSanitizer."""
    clang = _clang()
    if clang is None:
        pytest.skip("no clang++ (the kernels use clang vector extensions)")
    obj = _kernel_library_for_the_cpu(clang, sanitizer)
    host = os.path.join(ROOT, "tensorflow-allreduce_amd", "csrc", "host")
    oracle_obj = os.path.join(BUILD, "ring_oracle_cpu.o")
    _run(["gcc", "-O1", "-g", "-std=gnu11", "-fno-fast-math", "-c", os.path.join(ROOT, "oracle", "ring_oracle.c"),
          "-o", oracle_obj])
    exe = os.path.join(BUILD, "plugin_emulation_test_" + sanitizer)
    _run([clang] + _flags(sanitizer) + ["-I", host, "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "oracle"),
                                        "-o", exe, os.path.join(ROOT, "tests", "cpp", "plugin_emulation_test.cc")] +
         [os.path.join(host, f) for f in ("framework.cc", "wire.cc", "ring_driver.cc", "transport.cc", "collective_ops.cc")] +
         [obj, oracle_obj])
    # (AddressSanitizer's leak check is on: what a world, a batch or a plan allocates goes when it is destroyed)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1", TSAN_OPTIONS="halt_on_error=1:report_signal_unsafe=0")
    out = _run([exe], timeout=900, env=env)
    assert "plugin emulation: ok" in out, out[-4000:]


SCC_WRITER = re.compile(r"^\s*(s_cmp|s_bitcmp|s_and_b|s_or_b|s_xor_b|s_andn2|s_orn2|s_add|s_sub|s_lshl|s_lshr|s_ashr|"
                        r"s_bfe|s_not|s_min|s_max|s_abs|s_mul_hi|s_nand|s_nor|s_xnor|s_absdiff|s_wqm|s_quadmask|"
                        r"s_bcnt|s_and_saveexec|s_or_saveexec)")


def stale_selects(asm_text):
    """s_cselect instructions whose SCC was last written by an add / subtract /
    shift although a vector compare stands between the two: the select was
    meant to follow that compare."""
    lines = asm_text.split("\n")
    found = []
    for i, line in enumerate(lines):
        if not re.match(r"^\s*s_cselect", line):
            continue
        j, vcmp = i - 1, False
        while j >= 0 and not re.match(r"^\.LBB|^_Z", lines[j]) and not SCC_WRITER.match(lines[j]):
            vcmp = vcmp or bool(re.match(r"^\s*v_cmp", lines[j]))
            j -= 1
        if j >= 0 and vcmp and re.match(r"^\s*(s_add|s_sub|s_lshl|s_lshr|s_mul)", lines[j]):
            found.append((i + 1, line.strip(), lines[j].strip()))
    return found


def test_scan_recognises_the_pattern():
    bad = """
\ts_add_u32 s26, s40, s26
\ts_addc_u32 s27, s41, s27
\tv_cmp_lt_u64_e32 vcc, s[6:7], v[52:53]
\ts_cbranch_vccz .LBB26_31
\ts_cselect_b32 s34, s6, 0x400
"""
    good = """
\tv_cmp_lt_u64_e32 vcc, s[16:17], v[2:3]
\ts_and_b64 s[4:5], vcc, exec
\ts_cselect_b32 s24, s16, s14
"""
    assert len(stale_selects(bad)) == 1
    assert stale_selects(good) == []


def test_no_scalar_select_on_a_stale_condition_code():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    os.makedirs(BUILD, exist_ok=True)
    asm = os.path.join(BUILD, "ring_kernels_gfx950.s")
    # the assembly of this source and these flags is kept between runs (minutes of compiling otherwise)
    sources = [SRC, os.path.join(ROOT, "include", "ring_abi.h"), os.path.abspath(__file__)]
    if not os.path.exists(asm) or os.path.getmtime(asm) < max(os.path.getmtime(f) for f in sources):
        _run([hipcc] + HIP_FLAGS + ["-I", os.path.join(ROOT, "include"), "-S", "--cuda-device-only", "-o", asm, SRC])
    text = open(asm).read()
    found = stale_selects(text)
    assert not found, "scalar selects on a stale condition code: %r" % (found[:5],)
    # The kernels that hold a launch's payload in registers must really hold it there: a body too large to
    # unroll, or one lane too many registers, and the compiler moves the array to scratch memory (a kernel
    # several times slower with the same results, which no parity test would notice).
    in_registers = kernels_in_scratch(text, ("rows_phased_kernel", "unpack_phased_kernel"))
    assert in_registers["seen"] >= 20, in_registers
    assert not in_registers["scratch"], "payload in scratch memory: %r" % (in_registers["scratch"][:5],)


def kernels_in_scratch(asm_text, names):
    """Of the kernels whose mangled name contains one of `names`: how many the
    code object's metadata lists, and which of them have a private segment or
    spilled vector registers."""
    seen, scratch = 0, []
    for block in asm_text.split("- .agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", block)
        if not name or not any(n in name.group(1) for n in names):
            continue
        seen += 1
        private = int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", block).group(1))
        spilled = int(re.search(r"\.vgpr_spill_count:\s+(\d+)", block).group(1))
        if private or spilled:
            scratch.append((name.group(1), private, spilled))
    return {"seen": seen, "scratch": scratch}


def test_options_set_while_another_thread_launches_under_thread_sanitizer():
    """ring_set_option from one thread while another launches copies, accumulates and
    unpacks through the CPU stand-in: no data race, and every output right."""
    clang = _clang()
    if clang is None:
        pytest.skip("no clang++ (the kernels use clang vector extensions)")
    obj = _kernel_library_for_the_cpu(clang, "tsan")
    exe = os.path.join(BUILD, "options_race_test")
    _run([clang] + _flags("tsan") + ["-I", SHIM, "-I", os.path.join(ROOT, "include"), "-o", exe,
                                     os.path.join(ROOT, "tests", "cpp", "options_race_test.cc"), obj])
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1:report_signal_unsafe=0")
    out = _run([exe], timeout=600, env=env)
    assert "options race test: ok" in out, out[-4000:]
