"""TEST INFRASTRUCTURE ONLY: ctypes front-end of the CPU oracle.

Loads ``oracle/build/liboracle.so`` (built from ``ring_oracle.c`` by
``oracle/Makefile``), the CPU restatement of the reference ring
(tensorflow/contrib/mpi_collectives/ring.h:136-301, ring.cc:36-51). Only the
tests, the smoke check and the benchmark's cpu_baseline leg import this
module; the product package never does.
"""
import ctypes
import json
import os
import shutil
import signal
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "build", "liboracle.so")
_MPI_BIN = os.path.join(_HERE, "build", "ring_mpi")

F32, I32, I64 = 0, 1, 2
_NP = {F32: np.float32, I32: np.int32, I64: np.int64}
_CODE = {np.dtype(np.float32): F32, np.dtype(np.int32): I32, np.dtype(np.int64): I64}
DTYPE_NAME = {F32: "f32", I32: "i32", I64: "i64"}


class Tap(ctypes.Structure):
    _fields_ = [("rs_recv", ctypes.c_void_p), ("ag_recv", ctypes.c_void_p),
                ("slot_elems", ctypes.c_size_t)]


def build():
    """Compile the oracle with its Makefile (gcc only)."""
    subprocess.run(["make", "-s", "-C", _HERE], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        sz, vp, ci = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int
        psz = ctypes.POINTER(ctypes.c_size_t)
        L.oracle_dtype_size.restype = sz
        L.oracle_dtype_size.argtypes = [ci]
        L.oracle_segment_table.restype = None
        L.oracle_segment_table.argtypes = [sz, ci, psz, psz]
        L.oracle_temp_elements.restype = sz
        L.oracle_temp_elements.argtypes = [sz, ci]
        L.oracle_allgather_table.restype = None
        L.oracle_allgather_table.argtypes = [psz, ci, sz, psz]
        L.oracle_accumulate.restype = None
        L.oracle_accumulate.argtypes = [ci, vp, vp, sz]
        L.oracle_copy.restype = None
        L.oracle_copy.argtypes = [vp, vp, sz]
        pvp = ctypes.POINTER(vp)
        L.oracle_ring_allreduce_threads.restype = ci
        L.oracle_ring_allreduce_threads.argtypes = [ci, ci, sz, pvp, pvp, ctypes.POINTER(Tap)]
        L.oracle_ring_allreduce_rank_prestaged.restype = ci
        L.oracle_ring_allreduce_rank_prestaged.argtypes = [ci, ci, ci, vp, vp, sz, pvp, pvp]
        L.oracle_ring_allreduce_lockstep.restype = ci
        L.oracle_ring_allreduce_lockstep.argtypes = [ci, ci, sz, pvp, pvp]
        L.oracle_ring_allgather_threads.restype = ci
        L.oracle_ring_allgather_threads.argtypes = [ci, ci, pvp, psz, sz, pvp]
        L.oracle_time_allreduce_threads.restype = ci
        L.oracle_time_allreduce_threads.argtypes = [ci, ci, sz, pvp, pvp, ci, ci,
                                                    ctypes.POINTER(ctypes.c_double)]
        _lib = L
    return _lib


def dtype_code(dt):
    return _CODE[np.dtype(dt)]


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _ptr_array(arrays):
    return (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])


def segment_table(count, n):
    """(sizes, starts) of the n ring segments of a count-element tensor."""
    sizes = (ctypes.c_size_t * n)()
    starts = (ctypes.c_size_t * n)()
    lib().oracle_segment_table(count, n, sizes, starts)
    return list(sizes), list(starts)


def temp_elements(count, n):
    return int(lib().oracle_temp_elements(count, n))


def allgather_table(rows, elems_per_row):
    n = len(rows)
    r = (ctypes.c_size_t * n)(*rows)
    starts = (ctypes.c_size_t * n)()
    lib().oracle_allgather_table(r, n, elems_per_row, starts)
    return list(starts)


def accumulate(dst, src):
    """dst += src in place (numpy arrays of one of the three dtypes)."""
    assert dst.dtype == src.dtype and dst.size == src.size
    assert dst.flags.c_contiguous and src.flags.c_contiguous
    lib().oracle_accumulate(dtype_code(dst.dtype), _ptr(dst), _ptr(src), dst.size)
    return dst


def _check_inputs(inputs):
    inputs = [np.ascontiguousarray(x).reshape(-1) for x in inputs]
    dt = inputs[0].dtype
    cnt = inputs[0].size
    for x in inputs:
        assert x.dtype == dt and x.size == cnt
    return inputs, dtype_code(dt), cnt


def ring_allreduce(inputs, tap=False):
    """Run every rank of the reference ring allreduce (one thread per rank).

    Returns outputs (list of arrays), or (outputs, rs_recv, ag_recv) with
    tap=True: rs_recv[r][i] / ag_recv[r][i] are what rank r received at
    reduce-scatter / allgather step i, each padded to ceil(count/n) elements.
    """
    inputs, code, cnt = _check_inputs(inputs)
    n = len(inputs)
    outs = [np.empty_like(x) for x in inputs]
    taps = None
    rs = ag = None
    if tap:
        slot = temp_elements(cnt, n)
        rs = [np.zeros((max(n - 1, 0), slot), dtype=inputs[0].dtype) for _ in range(n)]
        ag = [np.zeros((max(n - 1, 0), slot), dtype=inputs[0].dtype) for _ in range(n)]
        taps = (Tap * n)()
        for r in range(n):
            taps[r].rs_recv = rs[r].ctypes.data
            taps[r].ag_recv = ag[r].ctypes.data
            taps[r].slot_elems = slot
    rc = lib().oracle_ring_allreduce_threads(n, code, cnt, _ptr_array(inputs),
                                             _ptr_array(outs), taps)
    if rc:
        raise RuntimeError("oracle allreduce failed: %d" % rc)
    return (outs, rs, ag) if tap else outs


def ring_allreduce_rank_prestaged(n, r, inp, rs_segments, ag_segments):
    """One rank of the reference ring on given incoming segments (the per-rank
    data path): rs_segments[i] / ag_segments[i] are what rank r receives at
    step i of the reduce-scatter / allgather. Returns that rank's output."""
    inp = np.ascontiguousarray(inp).reshape(-1)
    rs = [np.ascontiguousarray(x, dtype=inp.dtype).reshape(-1) for x in rs_segments]
    ag = [np.ascontiguousarray(x, dtype=inp.dtype).reshape(-1) for x in ag_segments]
    assert len(rs) == n - 1 and len(ag) == n - 1
    sizes, _ = segment_table(inp.size, n)
    for i in range(n - 1):
        assert rs[i].size >= sizes[(r - i - 1) % n] and ag[i].size >= sizes[(r - i) % n]
    out = np.empty_like(inp)
    rc = lib().oracle_ring_allreduce_rank_prestaged(n, r, dtype_code(inp.dtype), _ptr(inp), _ptr(out), inp.size,
                                                    _ptr_array(rs), _ptr_array(ag))
    if rc != 0:
        raise RuntimeError("oracle_ring_allreduce_rank_prestaged failed: %d" % rc)
    return out


def ring_allreduce_lockstep(inputs):
    inputs, code, cnt = _check_inputs(inputs)
    n = len(inputs)
    outs = [np.empty_like(x) for x in inputs]
    rc = lib().oracle_ring_allreduce_lockstep(n, code, cnt, _ptr_array(inputs),
                                              _ptr_array(outs))
    if rc:
        raise RuntimeError("oracle lockstep allreduce failed: %d" % rc)
    return outs


def ring_allgather(inputs):
    """inputs[k]: rank k's array [rows_k, ...]; returns each rank's output."""
    inputs = [np.ascontiguousarray(x) for x in inputs]
    n = len(inputs)
    dt = inputs[0].dtype
    tail = inputs[0].shape[1:]
    for x in inputs:
        assert x.dtype == dt and x.shape[1:] == tail and x.ndim >= 1
    rows = [x.shape[0] for x in inputs]
    epr = int(np.prod(tail, dtype=np.int64)) if tail else 1
    outs = [np.empty((sum(rows),) + tail, dtype=dt) for _ in range(n)]
    rows_c = (ctypes.c_size_t * n)(*rows)
    rc = lib().oracle_ring_allgather_threads(n, dtype_code(dt), _ptr_array(inputs),
                                             rows_c, epr, _ptr_array(outs))
    if rc:
        raise RuntimeError("oracle allgather failed: %d" % rc)
    return outs


def time_allreduce_threads(inputs, warmup, reps):
    """Seconds per allreduce (slowest rank) for `reps` timed repetitions."""
    inputs, code, cnt = _check_inputs(inputs)
    n = len(inputs)
    outs = [np.empty_like(x) for x in inputs]
    secs = (ctypes.c_double * reps)()
    rc = lib().oracle_time_allreduce_threads(n, code, cnt, _ptr_array(inputs),
                                             _ptr_array(outs), warmup, reps, secs)
    if rc:
        raise RuntimeError("oracle timing failed: %d" % rc)
    return list(secs), outs


def mpirun_path():
    """An mpirun that matches the MPI ring_mpi was linked against, or None."""
    if not os.path.exists(_MPI_BIN):
        return None
    for cand in ("/opt/conda/bin/mpirun", shutil.which("mpirun")):
        if cand and os.path.exists(cand):
            return cand
    return None


def _run_mpi(argv, timeout):
    """mpirun with its proxies and ranks in a process group of their own, which is
    ended once mpirun has returned (or timed out): nothing it started outlives the call."""
    proc = subprocess.Popen(argv, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                            start_new_session=True)
    try:
        out, err = proc.communicate(timeout=timeout)
    except subprocess.TimeoutExpired:
        proc.kill()
        proc.communicate()
        raise
    finally:
        try:
            os.killpg(proc.pid, signal.SIGKILL)   # the group this call created, whatever is left of it
        except (ProcessLookupError, PermissionError):
            pass
    if proc.returncode != 0:
        raise subprocess.CalledProcessError(proc.returncode, argv, out, err)
    return out, err


def mpi_check(inputs, workdir, timeout=120):
    """Run the per-rank restatement over real MPI; returns the outputs."""
    inputs, code, cnt = _check_inputs(inputs)
    n = len(inputs)
    for r, x in enumerate(inputs):
        x.tofile(os.path.join(workdir, "in_%d.bin" % r))
    _run_mpi([mpirun_path(), "-np", str(n), _MPI_BIN, "check", DTYPE_NAME[code], str(cnt), workdir], timeout)
    return [np.fromfile(os.path.join(workdir, "out_%d.bin" % r), dtype=inputs[0].dtype)
            for r in range(n)]


def mpi_time(n, code, count, warmup, reps, timeout=300):
    """Time RingAllreduce over real MPI; returns the parsed JSON line."""
    stdout, stderr = _run_mpi([mpirun_path(), "-np", str(n), _MPI_BIN, "time",
                               DTYPE_NAME[code], str(count), str(warmup), str(reps)], timeout)
    for line in stdout.splitlines():
        line = line.strip()
        if line.startswith("{"):
            return json.loads(line)
    raise RuntimeError("ring_mpi printed no result: " + stdout + stderr)
