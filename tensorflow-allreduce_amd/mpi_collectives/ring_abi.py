"""ctypes binding of the C ABI in include/ring_abi.h (lib/libring_hip.so).

The library holds the hand-written gfx950 kernels of the ring's per-rank data
path. There is no CPU fallback: if the library is missing, or an entry point
fails, a RingError is raised.
"""
import ctypes
import os

F32, I32, I64 = 0, 1, 2
DTYPE_SIZE = {F32: 4, I32: 4, I64: 8}
PHASE_REDUCE_SCATTER, PHASE_ALLGATHER, PHASE_GATHER = 0, 1, 2
# enum ring_form / ring_role: which form a launch takes (describe_rows_launch, describe_unpack_launch)
FORM_TILES, FORM_PACED, FORM_REGISTERS_2, FORM_REGISTERS_1 = 0, 1, 2, 3
FORM_NAMES = {FORM_TILES: "tiles", FORM_PACED: "paced tiles", FORM_REGISTERS_2: "in registers, two workgroups per CU",
              FORM_REGISTERS_1: "in registers, one workgroup per CU"}
ROLE_COPY, ROLE_ACCUMULATE, ROLE_ALLGATHER = 0, 1, 2

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "lib", "libring_hip.so")

# Every symbol include/ring_abi.h declares.
EXPORTS = (
    "ring_abi_version", "ring_status_string", "ring_last_hip_error", "ring_dtype_size",
    "ring_set_option", "ring_event_create", "ring_event_destroy", "ring_event_elapsed_us",
    "ring_time_next_launch", "ring_event_record", "ring_event_synchronize", "ring_stream_wait_event", "ring_graph_begin_capture", "ring_graph_end_capture", "ring_graph_launch", "ring_graph_destroy", "ring_segment_table", "ring_temp_elements", "ring_allgather_table",
    "ring_schedule", "ring_stream_create", "ring_stream_destroy", "ring_stream_synchronize",
    "ring_copy_bytes", "ring_accumulate_f32", "ring_accumulate_i32", "ring_accumulate_i64",
    "ring_accumulate", "ring_reduce_scatter_steps", "ring_reduce_scatter_steps_from",
    "ring_allgather_steps", "ring_apply_rows", "ring_apply_rows_avg", "ring_fold_rows", "ring_fold_and_copy_rows", "ring_fold_to_all_rows", "ring_fusion_allreduce_all",
    "ring_fusion_plan_create", "ring_fusion_plan_destroy", "ring_fusion_plan_elements", "ring_fusion_plan_dtype",
    "ring_fusion_pack", "ring_fusion_unpack", "ring_fusion_unpack_scaled", "ring_fusion_gather",
    "ring_fusion_scatter", "ring_fusion_fold_scatter", "ring_scale", "ring_fusion_run_static",
    "ring_describe_rows_launch", "ring_describe_unpack_launch", "ring_probe_stream",
    "ring_get_device", "ring_set_device", "ring_describe_scatter_launch",
)


class RingError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = "%s: %s (status %d" % (where, status_string(status), status)
        if status == 3:
            msg += ", hipError %d" % lib().ring_last_hip_error()
        super().__init__(msg + ")")


class Step(ctypes.Structure):
    """ring_step: one received segment of a step table."""
    _fields_ = [("dst_offset", ctypes.c_uint64), ("src", ctypes.c_void_p),
                ("count", ctypes.c_uint64)]


class Row(ctypes.Structure):
    """ring_row: dst = a, or dst = b + a when b is not null."""
    _fields_ = [("dst", ctypes.c_void_p), ("a", ctypes.c_void_p), ("b", ctypes.c_void_p),
                ("count", ctypes.c_uint64)]


_lib = None


class FoldRow(ctypes.Structure):
    """ring_fold_row: dst = srcs[m-1] + (... + (srcs[1] + srcs[0]))."""
    _fields_ = [("dst", ctypes.c_void_p), ("srcs", ctypes.POINTER(ctypes.c_void_p)), ("count", ctypes.c_uint64)]


class FoldToAllRow(ctypes.Structure):
    """ring_fold_to_all_row: the fold of srcs stored to every pointer of dsts."""
    _fields_ = [("dsts", ctypes.POINTER(ctypes.c_void_p)), ("srcs", ctypes.POINTER(ctypes.c_void_p)),
                ("count", ctypes.c_uint64)]


class FusionSpan(ctypes.Structure):
    """ring_fusion_span: `count` elements of a plan's fused space from `begin`."""
    _fields_ = [("begin", ctypes.c_uint64), ("count", ctypes.c_uint64), ("incoming", ctypes.c_void_p),
                ("out", ctypes.c_void_p)]


def make_spans(spans):
    """spans: iterable of (begin, count, incoming_or_None, out_or_None) -> ctypes array, length."""
    spans = list(spans)
    arr = (FusionSpan * max(len(spans), 1))()
    for i, (b, c, inc, out) in enumerate(spans):
        arr[i].begin, arr[i].count, arr[i].incoming, arr[i].out = b, c, inc, out
    return arr, len(spans)


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python tensorflow-allreduce_amd/build.py` "
                "(the ring data path has no CPU fallback)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        ci, sz, vp = ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p
        psz = ctypes.POINTER(ctypes.c_size_t)
        pint = ctypes.POINTER(ctypes.c_int)
        sig = {
            "ring_abi_version": (ci, []),
            "ring_status_string": (ctypes.c_char_p, [ci]),
            "ring_last_hip_error": (ci, []),
            "ring_dtype_size": (sz, [ci]),
            "ring_set_option": (ci, [ctypes.c_char_p, ci]),
            "ring_event_create": (ci, [ctypes.POINTER(vp)]),
            "ring_event_destroy": (ci, [vp]),
            "ring_event_elapsed_us": (ci, [vp, vp, ctypes.POINTER(ctypes.c_double)]),
            "ring_time_next_launch": (ci, [vp, vp]),
            "ring_event_record": (ci, [vp, vp]),
            "ring_event_synchronize": (ci, [vp]),
            "ring_stream_wait_event": (ci, [vp, vp]),
            "ring_graph_begin_capture": (ci, [vp]),
            "ring_graph_end_capture": (ci, [vp, ctypes.POINTER(vp)]),
            "ring_graph_launch": (ci, [vp, vp]),
            "ring_graph_destroy": (ci, [vp]),
            "ring_segment_table": (ci, [sz, ci, psz, psz]),
            "ring_temp_elements": (sz, [sz, ci]),
            "ring_allgather_table": (ci, [psz, ci, sz, psz]),
            "ring_schedule": (ci, [ci, ci, ci, ci, pint, pint]),
            "ring_stream_create": (ci, [ctypes.POINTER(vp)]),
            "ring_stream_destroy": (ci, [vp]),
            "ring_stream_synchronize": (ci, [vp]),
            "ring_copy_bytes": (ci, [vp, vp, sz, vp]),
            "ring_accumulate_f32": (ci, [vp, vp, sz, vp]),
            "ring_accumulate_i32": (ci, [vp, vp, sz, vp]),
            "ring_accumulate_i64": (ci, [vp, vp, sz, vp]),
            "ring_accumulate": (ci, [ci, vp, vp, sz, vp]),
            "ring_reduce_scatter_steps": (ci, [vp, ctypes.POINTER(Step), ci, ci, vp]),
            "ring_reduce_scatter_steps_from": (ci, [vp, vp, ctypes.POINTER(Step), ci, ci, vp]),
            "ring_allgather_steps": (ci, [vp, ctypes.POINTER(Step), ci, ci, vp]),
            "ring_apply_rows": (ci, [ctypes.POINTER(Row), ci, ci, vp]),
            "ring_apply_rows_avg": (ci, [ctypes.POINTER(Row), ci, ctypes.POINTER(ctypes.c_ubyte), ci, ci, vp]),
            "ring_fold_rows": (ci, [ctypes.POINTER(FoldRow), ci, ci, ci, ci, vp]),
            "ring_fold_and_copy_rows": (ci, [ctypes.POINTER(FoldRow), ci, ci, ci, ctypes.POINTER(Row), ci, ci, vp]),
            "ring_fold_to_all_rows": (ci, [ctypes.POINTER(FoldToAllRow), ci, ci, ci, ci, ci, vp]),
            "ring_fusion_allreduce_all": (ci, [ctypes.POINTER(vp), ctypes.POINTER(vp), ci, ci, vp]),
            "ring_fusion_plan_create": (ci, [ctypes.POINTER(vp), psz, ci, ci, ctypes.POINTER(vp)]),
            "ring_fusion_plan_destroy": (ci, [vp]),
            "ring_fusion_plan_elements": (sz, [vp]),
            "ring_fusion_plan_dtype": (ci, [vp]),
            "ring_fusion_pack": (ci, [vp, vp, vp]),
            "ring_fusion_unpack": (ci, [vp, vp, vp]),
            "ring_fusion_unpack_scaled": (ci, [vp, vp, ci, vp]),
            "ring_fusion_gather": (ci, [vp, ctypes.POINTER(FusionSpan), ci, vp]),
            "ring_fusion_scatter": (ci, [vp, ctypes.POINTER(FusionSpan), ci, ci, vp]),
            "ring_fusion_fold_scatter": (ci, [vp, ctypes.c_uint64, ctypes.c_uint64, ctypes.POINTER(vp), ci, vp,
                                              ctypes.POINTER(FusionSpan), ci, ci, vp]),
            "ring_scale": (ci, [ci, vp, sz, ci, vp]),
            "ring_fusion_run_static": (ci, [ci, ctypes.POINTER(vp), psz, ci, ci, vp, ci, vp]),
            "ring_describe_rows_launch": (ci, [ctypes.POINTER(Row), ci, ci, ci, ci, pint]),
            "ring_describe_unpack_launch": (ci, [ctypes.c_uint64, ci, ci, ci, ci, pint]),
            "ring_probe_stream": (ci, [ctypes.POINTER(Row), ci, ci, ci, vp]),
            "ring_describe_scatter_launch": (ci, [vp, ctypes.POINTER(FusionSpan), ci, ci, ci, pint]),
            "ring_get_device": (ci, [pint]),
            "ring_set_device": (ci, [ci]),
        }
        for name in EXPORTS:
            fn = getattr(L, name)          # AttributeError if the symbol is missing
            fn.restype, fn.argtypes = sig[name]
        if L.ring_abi_version() != 1:
            raise RuntimeError("libring_hip.so has ABI version %d, expected 1" % L.ring_abi_version())
        _lib = L
    return _lib


def status_string(status):
    return lib().ring_status_string(status).decode()


def check(status, where):
    if status != 0:
        raise RingError(status, where)


def set_option(name, value):
    check(lib().ring_set_option(name.encode(), int(value)), "ring_set_option(%s)" % name)


def make_rows(rows):
    """rows: iterable of (dst_ptr, a_ptr, b_ptr_or_None, count) -> ctypes array, length."""
    rows = list(rows)
    arr = (Row * max(len(rows), 1))()
    for i, (dst, a, b, cnt) in enumerate(rows):
        arr[i].dst, arr[i].a, arr[i].b, arr[i].count = dst, a, b, cnt
    return arr, len(rows)


def describe_rows_launch(rows, dtype, role, cus=256):
    """The form (FORM_*) a launch of `rows` (dst, a, b, count) takes on a GPU of
    `cus` compute units; needs no GPU, pointers only matter for their alignment."""
    arr, n = make_rows(rows)
    form = ctypes.c_int(-1)
    check(lib().ring_describe_rows_launch(arr, n, dtype, role, cus, ctypes.byref(form)), "ring_describe_rows_launch")
    return form.value


def describe_unpack_launch(total_elements, n_tensors, dtype, divisor=0, cus=256):
    """The form (FORM_*) the unpack of such a fused buffer takes; needs no GPU."""
    form = ctypes.c_int(-1)
    check(lib().ring_describe_unpack_launch(total_elements, n_tensors, dtype, divisor, cus, ctypes.byref(form)),
          "ring_describe_unpack_launch")
    return form.value


def probe_stream(rows, dtype, mode, stream):
    """Measurement only: one direction of a copy launch. rows: (dst, a, None, count);
    mode 0 reads every `a`, mode 1 writes every `dst` (2 / 3: ordinary cache policy)."""
    arr, n = make_rows(rows)
    check(lib().ring_probe_stream(arr, n, dtype, mode, stream), "ring_probe_stream")


# ---- timing of single launches -----------------------------------------------------

def event_create():
    e = ctypes.c_void_p()
    check(lib().ring_event_create(ctypes.byref(e)), "ring_event_create")
    return e.value


def event_destroy(event):
    check(lib().ring_event_destroy(event), "ring_event_destroy")


def event_elapsed_us(start, stop):
    us = ctypes.c_double()
    check(lib().ring_event_elapsed_us(start, stop, ctypes.byref(us)), "ring_event_elapsed_us")
    return us.value


def time_next_launch(start, stop):
    check(lib().ring_time_next_launch(start, stop), "ring_time_next_launch")


# ---- host tables ----------------------------------------------------------------

def segment_table(count, n):
    sizes = (ctypes.c_size_t * max(n, 1))()
    starts = (ctypes.c_size_t * max(n, 1))()
    check(lib().ring_segment_table(count, n, sizes, starts), "ring_segment_table")
    return list(sizes), list(starts)


def temp_elements(count, n):
    return int(lib().ring_temp_elements(count, n))


def allgather_table(rows, elems_per_row):
    n = len(rows)
    r = (ctypes.c_size_t * max(n, 1))(*rows)
    starts = (ctypes.c_size_t * max(n, 1))()
    check(lib().ring_allgather_table(r, n, elems_per_row, starts), "ring_allgather_table")
    return list(starts)[:n]


def schedule(phase, n, r, step):
    send, recv = ctypes.c_int(), ctypes.c_int()
    check(lib().ring_schedule(phase, n, r, step, ctypes.byref(send), ctypes.byref(recv)),
          "ring_schedule")
    return send.value, recv.value


# ---- stream ---------------------------------------------------------------------

def stream_create():
    s = ctypes.c_void_p()
    check(lib().ring_stream_create(ctypes.byref(s)), "ring_stream_create")
    return s.value


def stream_destroy(stream):
    check(lib().ring_stream_destroy(stream), "ring_stream_destroy")


def stream_wait_event(stream, event):
    """Work enqueued on `stream` from now on waits for what `event` (a hipEvent_t
    handle, e.g. torch.cuda.Event.cuda_event) marked on its own stream."""
    check(lib().ring_stream_wait_event(stream, event), "ring_stream_wait_event")


def stream_synchronize(stream):
    check(lib().ring_stream_synchronize(stream), "ring_stream_synchronize")


# ---- device primitives (raw pointers) ---------------------------------------------

def copy_bytes(dst, src, nbytes, stream):
    check(lib().ring_copy_bytes(dst, src, nbytes, stream), "ring_copy_bytes")


def accumulate(dtype, dst, src, count, stream):
    check(lib().ring_accumulate(dtype, dst, src, count, stream), "ring_accumulate")


def make_steps(rows):
    """rows: iterable of (dst_offset_elems, src_ptr, count) -> ctypes array."""
    rows = list(rows)
    arr = (Step * max(len(rows), 1))()
    for i, (off, src, cnt) in enumerate(rows):
        arr[i].dst_offset, arr[i].src, arr[i].count = off, src, cnt
    return arr, len(rows)


def reduce_scatter_steps(buffer, steps, n_steps, dtype, stream):
    check(lib().ring_reduce_scatter_steps(buffer, steps, n_steps, dtype, stream),
          "ring_reduce_scatter_steps")


def reduce_scatter_steps_from(inp, buffer, steps, n_steps, dtype, stream):
    check(lib().ring_reduce_scatter_steps_from(inp, buffer, steps, n_steps, dtype, stream),
          "ring_reduce_scatter_steps_from")


def allgather_steps(buffer, steps, n_steps, dtype, stream):
    check(lib().ring_allgather_steps(buffer, steps, n_steps, dtype, stream),
          "ring_allgather_steps")


def apply_rows(rows, dtype, stream):
    """rows: iterable of (dst, a, b_or_None, count) raw device pointers."""
    rows = list(rows)
    arr = (Row * max(len(rows), 1))()
    for i, (d, a, b, cnt) in enumerate(rows):
        arr[i].dst, arr[i].a, arr[i].b, arr[i].count = d, a, b, cnt
    check(lib().ring_apply_rows(arr, len(rows), dtype, stream), "ring_apply_rows")


def apply_rows_avg(rows, divide, divisor, dtype, stream):
    """As apply_rows; rows with divide[k] true (all rows when divide is None)
    also divide by `divisor` (tf.div semantics)."""
    rows = list(rows)
    arr = (Row * max(len(rows), 1))()
    for i, (d, a, b, cnt) in enumerate(rows):
        arr[i].dst, arr[i].a, arr[i].b, arr[i].count = d, a, b, cnt
    flags = None if divide is None else (ctypes.c_ubyte * max(len(rows), 1))(*[1 if f else 0 for f in divide])
    check(lib().ring_apply_rows_avg(arr, len(rows), flags, divisor, dtype, stream), "ring_apply_rows_avg")


def _fold_array(rows, m):
    rows = list(rows)
    arr = (FoldRow * max(len(rows), 1))()
    keep = []
    for i, (d, srcs, cnt) in enumerate(rows):
        ptrs = (ctypes.c_void_p * m)(*srcs)
        keep.append(ptrs)
        arr[i].dst, arr[i].srcs, arr[i].count = d, ctypes.cast(ptrs, ctypes.POINTER(ctypes.c_void_p)), cnt
    return arr, len(rows), keep


def fold_rows(rows, m, divisor, dtype, stream):
    """rows: iterable of (dst, [m source pointers in fold order], count)."""
    arr, n, _keep = _fold_array(rows, m)
    check(lib().ring_fold_rows(arr, n, m, divisor, dtype, stream), "ring_fold_rows")


def fold_and_copy_rows(fold, m, divisor, copies, dtype, stream):
    """fold: as fold_rows; copies: iterable of (dst, src, count); one launch."""
    arr, n, _keep = _fold_array(fold, m)
    copies = list(copies)
    carr = (Row * max(len(copies), 1))()
    for i, (d, a, cnt) in enumerate(copies):
        carr[i].dst, carr[i].a, carr[i].b, carr[i].count = d, a, None, cnt
    check(lib().ring_fold_and_copy_rows(arr, n, m, divisor, carr, len(copies), dtype, stream),
          "ring_fold_and_copy_rows")


def fold_to_all_rows(rows, m, n_dst, divisor, dtype, stream):
    """rows: iterable of ([n_dst destination pointers], [m source pointers in fold order], count)."""
    rows = list(rows)
    arr = (FoldToAllRow * max(len(rows), 1))()
    keep = []
    for i, (dsts, srcs, cnt) in enumerate(rows):
        d = (ctypes.c_void_p * n_dst)(*dsts)
        p = (ctypes.c_void_p * m)(*srcs)
        keep += [d, p]
        arr[i].dsts = ctypes.cast(d, ctypes.POINTER(ctypes.c_void_p))
        arr[i].srcs = ctypes.cast(p, ctypes.POINTER(ctypes.c_void_p))
        arr[i].count = cnt
    check(lib().ring_fold_to_all_rows(arr, len(rows), m, n_dst, divisor, dtype, stream), "ring_fold_to_all_rows")


def scale(dtype, data, count, divisor, stream):
    check(lib().ring_scale(dtype, data, count, divisor, stream), "ring_scale")


def fusion_run_static(unpack, ptrs, counts, dtype, fused, divisor, stream):
    """Pack (unpack false) or unpack (optionally divided) without a plan and
    without any allocation: the offset table is built in the library's static
    device array. Limits: 1024 non-empty tensors, 65536 tiles of 16 KiB."""
    k = len(ptrs)
    p = (ctypes.c_void_p * max(k, 1))(*ptrs)
    c = (ctypes.c_size_t * max(k, 1))(*counts)
    check(lib().ring_fusion_run_static(1 if unpack else 0, p, c, k, dtype, fused, divisor, stream),
          "ring_fusion_run_static")


def fusion_allreduce_all(in_plans, out_plans, divisor, stream):
    """The fused allreduce of ranks that share the GPU, without a fused buffer:
    in_plans[k] / out_plans[k] are FusionPlans over rank k's input and output tensors."""
    n = len(in_plans)
    a = (ctypes.c_void_p * n)(*[p._h for p in in_plans])
    b = (ctypes.c_void_p * n)(*[p._h for p in out_plans])
    check(lib().ring_fusion_allreduce_all(a, b, n, divisor, stream), "ring_fusion_allreduce_all")


class FusionPlan:
    """Offset table of k tensors packed back to back (ring_fusion_plan)."""

    def __init__(self, ptrs, counts, dtype):
        k = len(ptrs)
        p = (ctypes.c_void_p * max(k, 1))(*ptrs)
        c = (ctypes.c_size_t * max(k, 1))(*counts)
        h = ctypes.c_void_p()
        check(lib().ring_fusion_plan_create(p, c, k, dtype, ctypes.byref(h)),
              "ring_fusion_plan_create")
        self._h = h.value
        self.dtype = dtype
        self.elements = int(lib().ring_fusion_plan_elements(self._h))

    def pack(self, fused, stream):
        check(lib().ring_fusion_pack(self._h, fused, stream), "ring_fusion_pack")

    def unpack(self, fused, stream):
        check(lib().ring_fusion_unpack(self._h, fused, stream), "ring_fusion_unpack")

    def unpack_scaled(self, fused, divisor, stream):
        check(lib().ring_fusion_unpack_scaled(self._h, fused, divisor, stream), "ring_fusion_unpack_scaled")

    def gather(self, spans, stream):
        """spans: (ctypes array, n) from make_spans: out = tensors (+ incoming) per span."""
        check(lib().ring_fusion_gather(self._h, spans[0], spans[1], stream), "ring_fusion_gather")

    def scatter(self, spans, divisor, stream):
        """tensors = incoming (/ divisor) per span."""
        check(lib().ring_fusion_scatter(self._h, spans[0], spans[1], divisor, stream), "ring_fusion_scatter")

    def fold_scatter(self, fold_begin, fold_count, staged, wire, finished, divisor, stream):
        """The direct form in one launch: the owned span folded from `staged`
        (pointers, in fold order) and the tensors, the sum to `wire`, the
        tensors = sum (/ divisor); `finished` spans (make_spans) scattered."""
        m = len(staged)
        sp = (ctypes.c_void_p * max(m, 1))(*staged)
        check(lib().ring_fusion_fold_scatter(self._h, fold_begin, fold_count, sp, m, wire, finished[0], finished[1],
                                             divisor, stream), "ring_fusion_fold_scatter")

    def close(self):
        if self._h:
            check(lib().ring_fusion_plan_destroy(self._h), "ring_fusion_plan_destroy")
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
