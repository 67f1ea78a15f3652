"""CPU-side tests: the two libraries load and export what include/*.h declares,
the op registry matches the reference's registrations, the host tables agree
with the oracle, and the error behaviour of the ops follows the reference's
tests (tensorflow/contrib/mpi_collectives/mpi_ops_test.py:158-202, 265-297)
and messages (mpi_ops.cc:277-432, 827-847). No kernel is launched here."""
import ctypes
import os
import re

import numpy
import pytest
import torch

import gpu_util

import mpi_collectives as mpi
from mpi_collectives import _plugin, mpi_ops, ring_abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:ring|mpic)_[a-z0-9_]+)\s*\(", text)) - {"mpic_alloc_fn"})


def test_ring_abi_exports_every_declared_symbol():
    names = declared_functions("ring_abi.h")
    assert len(names) >= 25
    L = ctypes.CDLL(ring_abi.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n
    assert sorted(ring_abi.EXPORTS) == names
    assert ring_abi.lib().ring_abi_version() == 1


def test_plugin_exports_every_declared_symbol():
    names = declared_functions("mpi_collectives.h")
    L = ctypes.CDLL(_plugin.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n
    assert sorted(_plugin.EXPORTS) == names


def test_op_registry_matches_reference_registrations():
    _plugin.load_library()
    assert _plugin.op_names() == ['MPIInit', 'MPISize', 'MPIRank', 'MPILocalRank', 'MPIAllreduce', 'MPIAllgather']
    # mpi_ops.cc:1119-1126, 1233-1245
    assert _plugin.op_signature('MPIAllreduce') == "MPIAllreduce(tensor: T) -> (sum: T); T: {int32, int64, float32}"
    assert _plugin.op_signature('MPIAllgather') == \
        "MPIAllgather(tensor: T, sizes: S) -> (gathered: T); T: {int32, int64, float32}; S: {int64}"
    assert _plugin.op_signature('MPISize') == "MPISize() -> (size: int32)"
    assert _plugin.op_signature('NoSuchOp') is None
    assert "Perform an MPI Allreduce on a tensor" in _plugin.op_doc('MPIAllreduce')
    L = _plugin.lib()
    for op in ('MPIInit', 'MPISize', 'MPIRank', 'MPILocalRank'):
        assert L.mpic_op_has_kernel(op.encode(), b"CPU") and L.mpic_op_has_kernel(op.encode(), b"GPU")
    for op in ('MPIAllreduce', 'MPIAllgather'):       # collectives: GPU kernels only, no host path
        assert L.mpic_op_has_kernel(op.encode(), b"GPU") and not L.mpic_op_has_kernel(op.encode(), b"CPU")
    # shape functions: identity; first dimension unknown
    assert _plugin.infer_shape('MPIAllreduce', [17, 3]) == [17, 3]
    assert _plugin.infer_shape('MPIAllgather', [17, 3]) == [None, 3]
    assert _plugin.infer_shape('MPISize', []) == []


def test_load_library_checks_the_op_list():
    assert mpi_ops._load_library('libmpi_collectives.so', ['MPISize', 'MPIAllreduce']) is not None
    with pytest.raises(NameError, match="Could not find operator MPIBroadcast in dynamic library"):
        mpi_ops._load_library('libmpi_collectives.so', ['MPISize', 'MPIBroadcast'])


def test_host_tables_agree_with_oracle(oracle):
    for n in (1, 2, 3, 6, 8, 64):
        for count in (0, 1, n - 1, n + 1, 4913, 10_000_019):
            assert ring_abi.segment_table(count, n) == oracle.segment_table(count, n)
            assert ring_abi.temp_elements(count, n) == oracle.temp_elements(count, n)
    rows = [17, 32, 81, 12, 15, 23, 22]
    assert ring_abi.allgather_table(rows, 289) == oracle.allgather_table(rows, 289)
    L = ring_abi.lib()
    sizes = (ctypes.c_size_t * 1)()
    assert L.ring_segment_table(5, 0, sizes, sizes) == 2           # n < 1
    assert ring_abi.temp_elements(5, 0) == 0


def test_sizes_that_do_not_fit_are_refused_not_wrapped():
    """Element counts whose sum or product wraps 64 bits come back as an error
    from the host-side tables and from the two fusion entry points that add
    counts up, before anything is allocated or launched (no GPU needed)."""
    L = ring_abi.lib()
    top = 2 ** 64 - 1
    with pytest.raises(ring_abi.RingError):
        ring_abi.allgather_table([top // 2, top // 2], 8)            # rows x elements per row wraps
    with pytest.raises(ring_abi.RingError):
        ring_abi.allgather_table([top // 2, top // 2 + 2], 1)        # the sum of the rows wraps
    assert ring_abi.allgather_table([top // 4, 1], 2) == [0, 2 * (top // 4)]
    # a fusion plan over tensors whose counts add up past 64 bits (the pointers are never dereferenced:
    # the call is refused while it looks at the sizes)
    ptrs = (ctypes.c_void_p * 2)(4096, 8192)
    plan = ctypes.c_void_p()
    for counts in ((top, 2), (top // 4, top // 4 + 1), (top // 8 + 1, top // 8 + 1)):
        c = (ctypes.c_size_t * 2)(*counts)
        assert L.ring_fusion_plan_create(ptrs, c, 2, ring_abi.F32, ctypes.byref(plan)) == 2, counts
        assert not plan.value
    # the allocation-free entry point: beyond its stated size it says so, also when the sum wraps
    for counts in ((2, top), (top, top), (2 ** 40, 1)):
        c = (ctypes.c_size_t * 2)(*counts)
        assert L.ring_fusion_run_static(0, ptrs, c, 2, ring_abi.F32, ctypes.c_void_p(4096), 0, None) == 5, counts
    # the segment table and the temp size of a count at the top of the range
    sizes, starts = ring_abi.segment_table(top, 4)
    assert sum(sizes) == top and starts[3] + sizes[3] == top
    assert ring_abi.temp_elements(top, 3) == top // 3


def test_schedule_is_the_reference_index_algebra():
    # ring.h:184-185, 212-213, 280-281
    for n in (2, 3, 8):
        for r in range(n):
            for i in range(n - 1):
                assert ring_abi.schedule(ring_abi.PHASE_REDUCE_SCATTER, n, r, i) == ((r - i) % n, (r - i - 1) % n)
                assert ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i) == ((r - i + 1) % n, (r - i) % n)
                assert ring_abi.schedule(ring_abi.PHASE_GATHER, n, r, i) == ((r - i) % n, (r - i - 1) % n)
            # a rank's reduce-scatter touches every segment but its own, once; its
            # allgather every segment but (r+1)
            rs = [ring_abi.schedule(0, n, r, i)[1] for i in range(n - 1)]
            ag = [ring_abi.schedule(1, n, r, i)[1] for i in range(n - 1)]
            assert sorted(rs) == sorted(set(range(n)) - {r})
            assert sorted(ag) == sorted(set(range(n)) - {(r + 1) % n})
    with pytest.raises(ring_abi.RingError):
        ring_abi.schedule(0, 4, 0, 3)                               # step out of range
    assert ring_abi.lib().ring_dtype_size(0) == 4 and ring_abi.lib().ring_dtype_size(2) == 8
    assert ring_abi.lib().ring_dtype_size(5) == 0


def test_ops_before_init_fail_like_the_reference():
    L = _plugin.load_library()
    w = ctypes.c_void_p()
    assert L.mpic_world_create(2, ctypes.byref(w)) == 0
    try:
        op = _plugin.PendingOp(w.value, 0, 'MPISize', 'MPISize', [], 'CPU')
        with pytest.raises(mpi.FailedPreconditionError,
                           match="MPI has not been initialized; use tf.contrib.mpi.Session."):
            op.wait()
    finally:
        L.mpic_world_destroy(w.value)
    with pytest.raises(mpi.FailedPreconditionError):
        mpi.size()                                                    # no session at all


def test_size_rank_local_rank():
    with mpi.Session(size=5, device="CPU") as session:
        assert mpi.size() == 5 and mpi.rank() == 0
        for r in range(5):
            with session.as_rank(r):
                assert (mpi.size(), mpi.rank(), mpi.local_rank()) == (5, r, r)
        with pytest.raises(mpi.InvalidArgumentError):
            with session.as_rank(5):
                pass
    # outside a launcher the default world has one rank (mpi_ops_test.py:61-62)
    with mpi.Session(device="CPU") as session:
        assert mpi.size() == 1 and mpi.rank() == 0


def test_size_from_launcher_environment(monkeypatch):
    monkeypatch.setenv("PMI_SIZE", "3")
    with mpi.Session(device="CPU"):
        assert mpi.size() == 3


def test_collectives_have_no_cpu_kernel():
    with mpi.Session(size=2, device="CPU"):
        with pytest.raises(mpi.NotFoundError, match="No OpKernel was registered to support Op 'MPIAllreduce'"):
            mpi.allreduce(torch.ones(4))
        with pytest.raises(mpi.NotFoundError):
            mpi.allgather(torch.ones(4, 2))


def _submit_all(session, op, tensors, name, extra=None):
    """Submit `op` as every rank through the GPU kernel registration. The
    tensors are host tensors: the cross-rank checks run before any device work,
    and a collective that passes them is then refused for being in host memory."""
    ops = []
    for r, t in enumerate(tensors):
        inputs = [t] + ([extra] if extra is not None else [])
        ops.append(session._submit(r, op, name, inputs, "GPU"))
    return ops


def _errors(ops):
    out = []
    for p in ops:
        with pytest.raises(mpi.OpError) as e:
            p.wait()
        out.append(e.value)
    return out


def test_allreduce_error_matrix():
    """mpi_ops_test.py:158-202: every rank gets FailedPrecondition."""
    with mpi.Session(size=3, device="CPU") as s:
        # same rank, different dimension
        errs = _errors(_submit_all(s, 'MPIAllreduce', [torch.zeros([17 + r] * 3) for r in range(3)], "a"))
        assert all(isinstance(e, mpi.FailedPreconditionError) for e in errs)
        assert errs[0].message == ("Mismatched allreduce tensor shapes: One rank reduced a tensor of shape "
                                   "[17,17,17], but another rank sent a tensor of shape [18,18,18].")
        assert len({e.message for e in errs}) == 1
        s._pending.clear()
        # same number of elements, different rank
        shapes = [[17, 23 * 57], [17, 23, 57], [17, 23, 57]]
        errs = _errors(_submit_all(s, 'MPIAllreduce', [torch.zeros(sh) for sh in shapes], "b"))
        assert all(isinstance(e, mpi.FailedPreconditionError) for e in errs)
        assert "of shape [17,1311], but another rank sent a tensor of shape [17,23,57]" in errs[0].message
        s._pending.clear()
        # different types
        ts = [torch.ones([17] * 3, dtype=torch.int32 if r % 2 == 0 else torch.float32) for r in range(3)]
        errs = _errors(_submit_all(s, 'MPIAllreduce', ts, "c"))
        assert errs[0].message == ("Mismatched data types: One rank had type TF_MPI_INT32, "
                                   "but another rank had type TF_MPI_FLOAT32.")
        s._pending.clear()
        # a consistent request on host tensors is refused, not computed on the CPU
        errs = _errors(_submit_all(s, 'MPIAllreduce', [torch.zeros(4)] * 3, "d"))
        assert "GPU kernels only" in errs[0].message
        s._pending.clear()


def test_allgather_error_matrix():
    """mpi_ops_test.py:265-297 and the remaining branches of mpi_ops.cc:352-411."""
    sizes = torch.tensor([17, 17, 17], dtype=torch.int64)
    with mpi.Session(size=3, device="CPU") as s:
        ts = [torch.ones([17, 10 * (r + 1), 17]) for r in range(3)]
        errs = _errors(_submit_all(s, 'MPIAllgather', ts, "g1", sizes))
        assert all(isinstance(e, mpi.FailedPreconditionError) for e in errs)
        assert errs[0].message == ("Mismatched allgather tensor shapes: One rank gathered a tensor with dimension 1 "
                                   "equal to 10, but another rank sent a tensor with dimension 1 equal to 20.")
        s._pending.clear()
        ts = [torch.ones([17] * 3, dtype=torch.int32 if r % 2 == 0 else torch.float32) for r in range(3)]
        errs = _errors(_submit_all(s, 'MPIAllgather', ts, "g2", sizes))
        assert errs[0].message.startswith("Mismatched data types: One rank had type TF_MPI_INT32")
        s._pending.clear()
        ts = [torch.ones([17, 17]), torch.ones([17, 17, 1]), torch.ones([17, 17])]
        errs = _errors(_submit_all(s, 'MPIAllgather', ts, "g3", sizes))
        assert errs[0].message == ("Mismatched allgather tensor shapes: One rank gathered a tensor of rank 2, "
                                   "but another rank sent a tensor of rank 3.")
        s._pending.clear()
        errs = _errors(_submit_all(s, 'MPIAllgather', [torch.ones([])] * 3, "g4", torch.zeros((), dtype=torch.int64)))
        assert errs[0].message == "Rank zero tried to gather a rank-zero tensor."
        s._pending.clear()
        # one rank reduces while the others gather
        ops = [s._submit(0, 'MPIAllreduce', "mix", [torch.ones(17, 2)], "GPU")]
        ops += [s._submit(r, 'MPIAllgather', "mix", [torch.ones(17, 2), sizes], "GPU") for r in (1, 2)]
        errs = _errors(ops)
        assert errs[0].message == "Mismatched MPI operations: One rank did an 0, but another rank did an 1."
        s._pending.clear()


def test_unsupported_dtype_is_rejected_before_anything_runs():
    with mpi.Session(size=2, device="CPU") as s:
        p = s._submit(0, 'MPIAllreduce', "x", [torch.ones(4, dtype=torch.float64)], "GPU")
        with pytest.raises(mpi.FailedPreconditionError, match="Invalid tensor type passed."):
            p.wait()                                                 # mpi_ops.cc:844
        s._pending.clear()
        p = s._submit(0, 'MPIAllreduce', "y", [torch.ones(4, dtype=torch.float16)], "GPU")
        with pytest.raises(mpi.FailedPreconditionError, match="Invalid tensor type passed."):
            p.wait()
        s._pending.clear()


def test_run_refuses_to_wait_for_ranks_that_never_submitted():
    with mpi.Session(size=3, device="CPU") as s:
        s._submit(0, 'MPIAllreduce', "lonely", [torch.zeros(4)], "GPU")
        with pytest.raises(mpi.FailedPreconditionError, match="submitted by ranks \\[0\\] of 3"):
            s.run()
        pending = s._pending[0]
    # closing the session shuts the background thread down and fails the op
    with pytest.raises(mpi.UnknownError, match="shut down"):
        pending.wait()


def test_fused_divisor_arguments_and_failure_drain():
    """A negative divisor is refused before the op starts; when several ops of
    one run fail, every one of them is completed and the first error raised."""
    with mpi.Session(size=2, device="CPU") as s:
        with pytest.raises(mpi.InvalidArgumentError, match="bad divisor"):
            _plugin.PendingOp(s._world, 0, 'MPIAllreduce', 'neg', [torch.zeros(4)], 'GPU', divisor=-1)
        for r in range(2):
            for name in ("a", "b"):
                # host tensors: both collectives are refused ("GPU kernels only")
                s._submit(r, 'MPIAllreduce', name, [torch.zeros(4)], "GPU", 2)
        with pytest.raises(mpi.FailedPreconditionError, match="GPU kernels only"):
            s.run()
        assert not s._pending and not s._submitted


def test_loopback_transport_matches_messages_and_times_out():
    """Host-side behaviour of the in-process transport: argument checks, a wait
    or a send without a peer gives up after the timeout, zero-byte messages
    match in order without touching a device."""
    import time
    L = _plugin.load_library()
    h = ctypes.c_void_p()
    assert L.mpic_loopback_create(0, 1.0, ctypes.byref(h)) == 3
    assert L.mpic_loopback_create(2, 0.0, ctypes.byref(h)) == 3
    assert L.mpic_loopback_create(2, 0.2, ctypes.byref(h)) == 0
    try:
        t0, t1 = _plugin.Transport(), _plugin.Transport()
        assert L.mpic_loopback_endpoint(h.value, 2, ctypes.byref(t0)) == 3
        assert L.mpic_loopback_endpoint(h.value, 0, ctypes.byref(t0)) == 0
        assert L.mpic_loopback_endpoint(h.value, 1, ctypes.byref(t1)) == 0
        req = ctypes.c_void_p()
        assert t0.irecv(t0.user, None, 8, 1, 12, ctypes.byref(req)) != 0          # bytes without a buffer
        assert t0.irecv(t0.user, None, 0, 5, 12, ctypes.byref(req)) != 0          # no such rank
        began = time.perf_counter()
        assert t0.send(t0.user, None, 0, 1, 12) != 0                              # nobody receives
        assert 0.15 < time.perf_counter() - began < 5.0
        assert t1.irecv(t1.user, None, 0, 0, 12, ctypes.byref(req)) == 0
        first = req.value
        assert t1.irecv(t1.user, None, 0, 0, 12, ctypes.byref(req)) == 0
        assert t1.wait(t1.user, req.value) != 0                                   # second message never sent
        assert t0.send(t0.user, None, 0, 1, 12) == 0
        assert t1.wait(t1.user, first) == 0
        assert t0.send(t0.user, None, 0, 1, 7) != 0                               # other tag: no match
        # a cancelled receive is gone: the next send finds nothing to match
        assert t1.irecv(t1.user, None, 0, 0, 12, ctypes.byref(req)) == 0
        assert t1.cancel(t1.user, req.value) == 0
        assert t0.send(t0.user, None, 0, 1, 12) != 0
        # so is one whose wait timed out
        assert t1.irecv(t1.user, None, 0, 0, 12, ctypes.byref(req)) == 0
        assert t1.wait(t1.user, req.value) != 0
        assert t0.send(t0.user, None, 0, 1, 12) != 0
    finally:
        L.mpic_loopback_destroy(h.value)
    # the ring over a transport checks its arguments before it touches the device
    bad = _plugin.Transport()
    x = ctypes.create_string_buffer(64)
    addr = ctypes.addressof(x)
    assert L.mpic_ring_allreduce_transport(2, 0, _plugin.DT_FLOAT, addr, addr, addr, 8, 16, None, None, 0) == 3
    assert L.mpic_ring_allreduce_transport(2, 0, _plugin.DT_FLOAT, addr, addr, addr, 8, 16, ctypes.byref(bad), None, 0) == 3
    assert L.mpic_ring_allreduce_transport(2, 2, _plugin.DT_FLOAT, addr, addr, addr, 8, 16, ctypes.byref(bad), None, 0) == 3
    assert L.mpic_ring_allreduce_transport(2, 0, _plugin.DT_DOUBLE, addr, addr, addr, 8, 16, ctypes.byref(bad), None, 0) == 9
    assert b"Invalid tensor type" in L.mpic_last_error()


def test_node_names_are_uniquified_like_graph_nodes():
    with mpi.Session(size=2, device="CPU") as s:
        assert [s._node_name(0, 'MPIAllreduce', None) for _ in range(3)] == \
            ['MPIAllreduce', 'MPIAllreduce_1', 'MPIAllreduce_2']
        assert s._node_name(1, 'MPIAllreduce', None) == 'MPIAllreduce'
        assert s._node_name(0, 'MPIAllgather', 'allgather') == 'allgather'
        assert s._node_name(0, 'MPIAllgather', 'allgather') == 'allgather_1'


def test_prestaged_world_checks_its_arguments():
    L = _plugin.load_library()
    w = ctypes.c_void_p()
    assert L.mpic_world_create_prestaged(4, 4, ctypes.byref(w)) == 3      # rank out of range
    assert L.mpic_world_create_prestaged(4, -1, ctypes.byref(w)) == 3
    assert L.mpic_world_create(0, ctypes.byref(w)) == 3
    with mpi.Session(size=4, rank=2, device="CPU") as s:
        assert mpi.rank() == 2 and mpi.size() == 4
        with pytest.raises(mpi.InvalidArgumentError):
            with s.as_rank(1):
                pass
        with pytest.raises(mpi.InvalidArgumentError):
            s.stage_peers("x", [torch.zeros(1)], [torch.zeros(1)])        # needs n-1 = 3 segments
        # nothing staged for this name
        p = s._submit(2, 'MPIAllreduce', "nostage", [torch.zeros(8)], "GPU")
        with pytest.raises(mpi.FailedPreconditionError, match="GPU kernels only|No pre-staged"):
            p.wait()
        s._pending.clear()


def test_resnet50_shape_set():
    shapes = gpu_util.resnet50_shapes()
    sizes = [int(numpy.prod(s)) for s in shapes]
    assert len(shapes) == 161 and sum(sizes) == 25_557_032
    assert min(sizes) == 64 and max(sizes) == 2_359_296
    assert sum(1 for s in sizes if s <= 2048) == 107


def test_fusion_buffer_arguments_and_flush():
    L = _plugin.load_library()
    w = ctypes.c_void_p()
    assert L.mpic_world_create(2, ctypes.byref(w)) == 0
    try:
        assert L.mpic_world_set_fusion_buffer(w.value, None, 1024) == 3        # a size without a buffer
        assert L.mpic_world_set_fusion_buffer(w.value, 4096 + 8, 1024) == 3    # not 16-byte aligned
        assert L.mpic_world_set_fusion_buffer(w.value, 4096, 1000) == 3        # not a multiple of 16
        assert L.mpic_world_set_fusion_buffer(w.value, None, 0) == 0           # off
        assert L.mpic_world_flush(w.value) == 0                                # harmless without pending work
        assert L.mpic_world_flush(None) == 3
    finally:
        L.mpic_world_destroy(w.value)


def test_zero_sized_dimensions_survive_the_coordinator():
    """A zero-sized dimension encodes as a zero byte; the reference's messages
    are cut at the first one (mpi_ops.cc:703, 773). Here shapes with zeros are
    compared, and reported, in full."""
    with mpi.Session(size=2, device="CPU") as s:
        errs = _errors(_submit_all(s, 'MPIAllreduce', [torch.zeros([0, 5]), torch.zeros([0, 6])], "z"))
        assert errs[0].message == ("Mismatched allreduce tensor shapes: One rank reduced a tensor of shape [0,5], "
                                   "but another rank sent a tensor of shape [0,6].")
        s._pending.clear()
        # equal empty shapes pass the checks (and are then refused for living in host memory)
        errs = _errors(_submit_all(s, 'MPIAllreduce', [torch.zeros([0, 5]), torch.zeros([0, 5])], "z2"))
        assert "GPU kernels only" in errs[0].message
        s._pending.clear()


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the behaviour on a machine without a GPU")
def test_without_a_gpu_every_device_call_fails_and_nothing_is_computed_on_the_host():
    L = ring_abi.lib()
    a = numpy.ones(1024, dtype=numpy.float32)
    b = numpy.full(1024, 2.0, dtype=numpy.float32)
    assert L.ring_accumulate(ring_abi.F32, a.ctypes.data, b.ctypes.data, 1024, None) == 3      # RING_ERR_HIP
    assert L.ring_last_hip_error() != 0
    assert L.ring_copy_bytes(a.ctypes.data, b.ctypes.data, 4096, None) == 3
    assert L.ring_scale(ring_abi.F32, a.ctypes.data, 1024, 2, None) == 3
    stream = ctypes.c_void_p()
    assert L.ring_stream_create(ctypes.byref(stream)) == 3
    ptrs = (ctypes.c_void_p * 1)(a.ctypes.data)
    counts = (ctypes.c_size_t * 1)(1024)
    plan = ctypes.c_void_p()
    assert L.ring_fusion_plan_create(ptrs, counts, 1, ring_abi.F32, ctypes.byref(plan)) == 3 and not plan.value
    srcs = (ctypes.c_void_p * 2)(a.ctypes.data, b.ctypes.data)
    fold = (ring_abi.FoldRow * 1)()
    fold[0].dst, fold[0].srcs, fold[0].count = a.ctypes.data, ctypes.cast(srcs, ctypes.POINTER(ctypes.c_void_p)), 1024
    assert L.ring_fold_rows(fold, 1, 2, 0, ring_abi.F32, None) == 3
    assert L.ring_fold_rows(fold, 1, 2, 0, 7, None) == 1                                        # RING_ERR_DTYPE
    assert L.ring_fold_rows(fold, 1, 0, 0, ring_abi.F32, None) == 2                             # no sources
    assert L.ring_fold_rows(fold, 1, 257, 0, ring_abi.F32, None) == 2                           # too many sources
    assert L.ring_fold_rows(fold, 0, 2, 0, ring_abi.F32, None) == 0                             # nothing to do
    assert L.ring_event_record(None, None) == 2 and L.ring_event_synchronize(None) == 2
    assert (a == 1.0).all()                                # the host never stood in for the device
    with pytest.raises(ring_abi.RingError, match="HIP runtime call failed"):
        ring_abi.accumulate(ring_abi.F32, a.ctypes.data, b.ctypes.data, 1024, None)
    # a GPU session cannot even initialise: its dedicated stream cannot be created
    with pytest.raises(mpi.UnknownError, match="Could not create the MPI stream"):
        mpi.Session(size=2, device="GPU")


def test_bench_refuses_more_than_one_gpu_and_needs_a_gpu():
    """bench.py's contract on this tier: one GPU only, said in a message; and no
    number without the device (the benchmark never falls back to the host)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    two = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert two.returncode != 0 and "ONE GPU" in two.stderr and not two.stdout.strip()
    if not torch.cuda.is_available():
        one = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--no-cpu-baseline"], capture_output=True,
                             text=True)
        assert one.returncode != 0 and "no GPU is visible" in one.stderr and not one.stdout.strip()


def test_ops_submitted_from_many_threads_keep_their_own_outputs():
    """One thread per virtual rank, all submitting at once (the mode
    Session.as_rank supports for ranks driven like separate processes): every op
    instance must receive exactly the outputs its own allocator callback made.
    The scalar ops run on the CPU device, so this needs no GPU."""
    import threading
    n, rounds = 16, 200
    with mpi.Session(size=n, device="CPU") as session:
        errors, start = [], threading.Barrier(n)

        def drive(r):
            try:
                start.wait()
                for _ in range(rounds):
                    with session.as_rank(r):
                        p = session._submit(r, 'MPIRank', session._node_name(r, 'MPIRank', None), [], "CPU")
                        outs = p.wait()
                        assert len(outs) == 1, "rank %d: %d outputs" % (r, len(outs))
                        assert int(outs[0].item()) == r, "rank %d got the output of rank %d" % (r, int(outs[0].item()))
            except Exception as e:                      # reported from the main thread
                errors.append(e)

        threads = [threading.Thread(target=drive, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors[:3]
    assert not _plugin._live_ops


def test_direct_form_refuses_more_ranks_than_a_fold_addresses():
    """The direct pre-staged forms fold at most 256 copies of a segment: a larger
    ring is refused with a message that says so, before anything is launched."""
    L = _plugin.load_library()
    n = 257
    ptrs = (ctypes.c_void_p * n)(*([0x1000] * n))
    rc = L.mpic_ring_allreduce_direct_prestaged(n, 0, _plugin.DT_FLOAT, 0x1000, 0x2000, 1000, ptrs, ptrs, None, 1)
    assert rc == _plugin.INVALID_ARGUMENT
    assert b"at most 256 copies" in L.mpic_last_error()


# ---- which form a launch takes (host-only query; every form gives the same bytes, so only this pins the choice)

def _allgather_rows(count, n, rank, esz, misalign=0):
    """The copy rows of rank `rank`'s allgather phase on a `count`-element tensor at n ranks, as
    ring_allgather_steps hands them to the launcher (addresses made up: only their alignment matters)."""
    sizes, starts = ring_abi.segment_table(count, n)
    segs = [ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, rank, i)[1] for i in range(n - 1)]
    out, staged = 1 << 32, 1 << 40
    return [(out + misalign + starts[g] * esz, staged + (i << 30), None, sizes[g]) for i, g in enumerate(segs)]


def _equal_rows(n_rows, elems, esz=4):
    return [((1 << 32) + k * elems * esz, (1 << 40) + (k << 30), None, elems) for k in range(n_rows)]


def test_launch_forms_of_the_benchmark_shapes_on_256_compute_units():
    A = ring_abi
    form = lambda rows, dt: A.describe_rows_launch(rows, dt, A.ROLE_ALLGATHER, 256)
    # float32 64 MiB, N=8: 7 x 8 MiB fill the chip with exactly 7 paced tiles of 32 KiB per CU
    for rank in range(8):
        assert form(_allgather_rows(16 * 1024 * 1024, 8, rank, 4), A.F32) == A.FORM_PACED
    # int32 / int64 ragged 10,000,019 at N=6: 5 rows of 6.4 / 12.7 MiB
    for rank in range(6):
        assert form(_allgather_rows(10_000_019, 6, rank, 4), A.I32) == A.FORM_REGISTERS_2
        assert form(_allgather_rows(10_000_019, 6, rank, 8), A.I64) == A.FORM_REGISTERS_1
    # the fused ResNet-50 buffer at N=8: 7 rows of 12.2 MiB; and its unpack with the divide by 8 (97.5 MiB)
    assert form(_allgather_rows(25_557_032, 8, 0, 4), A.F32) == A.FORM_REGISTERS_1
    assert A.describe_unpack_launch(25_557_032, 161, A.F32, 8, 256) == A.FORM_REGISTERS_1
    assert A.describe_unpack_launch(25_557_032, 161, A.F32, 0, 256) == A.FORM_REGISTERS_1
    # float32 1 GiB at N=64: 63 rows of 16 MiB, far beyond what is resident at once
    assert form(_allgather_rows(268_435_456, 64, 0, 4), A.F32) == A.FORM_TILES
    # the variable allgather at N=16 (16 unequal rows, about 130 MiB)
    rows = [(1 << 32, 1 << 40, None, r * 1024) for r in (3000, 17, 4096, 2222, 1, 999, 4000, 3100, 2900, 12, 3500, 2048, 77,
                                                       4095, 1800, 2600)]
    assert form(rows, A.F32) == A.FORM_TILES
    # the in->out copy and the accumulates have one form
    assert A.describe_rows_launch(_equal_rows(1, 16 * 1024 * 1024), A.F32, A.ROLE_COPY, 256) == A.FORM_TILES
    acc = [(d, a, d, c) for d, a, _, c in _equal_rows(7, 2 * 1024 * 1024)]
    assert A.describe_rows_launch(acc, A.F32, A.ROLE_ACCUMULATE, 256) == A.FORM_TILES


def test_launch_forms_change_where_they_were_measured_to():
    A = ring_abi
    MiB = 1 << 18   # float32 elements
    form = lambda rows, cus=256, dt=A.F32: A.describe_rows_launch(rows, dt, A.ROLE_ALLGATHER, cus)
    assert form(_equal_rows(7, 2 * MiB)) == A.FORM_TILES                 # 14 MiB, under 2 paced tiles per CU: bound by the dispatch
    assert form(_equal_rows(8, 2 * MiB)) == A.FORM_PACED                 # 16 MiB: 2 tiles of 32 KiB per CU
    assert form(_equal_rows(7, 4 * MiB)) == A.FORM_PACED                 # 28 MiB: under 124 KiB per CU the paced tiles win
    assert form(_equal_rows(7, 7 * MiB + MiB // 2)) == A.FORM_REGISTERS_2  # 52.5 MiB: the paced tiles leave CUs over
    assert form(_equal_rows(7, 8 * MiB)) == A.FORM_PACED                 # 56 MiB: exactly 7 tiles per CU
    assert form(_equal_rows(7, 8 * MiB + 8192)) == A.FORM_REGISTERS_1    # one tile per row more: above 224 KiB per CU
    assert form(_equal_rows(7, 16 * MiB)) == A.FORM_REGISTERS_1          # 112 MiB: all the registers hold
    assert form(_equal_rows(7, 16 * MiB + 65536 * 4)) == A.FORM_TILES    # a 17th round per row does not fit
    assert form(_equal_rows(8, 14 * MiB)) == A.FORM_REGISTERS_1          # 8 rows of 14 rounds
    assert form(_equal_rows(9, 8 * MiB)) == A.FORM_TILES                 # more than 8 rows: not in registers, too many tiles to pace
    assert form(_equal_rows(9, 6 * MiB)) == A.FORM_PACED                 # 9 rows, 54 MiB: all tiles resident
    assert form(_equal_rows(1, 60 * MiB)) == A.FORM_REGISTERS_1          # one row (ring_allgather_steps of one step)
    assert form(_equal_rows(7, 8 * MiB), cus=64) == A.FORM_TILES         # a chip none of this was measured on
    assert form(_equal_rows(7, 2 * MiB), cus=64) == A.FORM_PACED
    # a row with a second operand, or an empty row kept by the caller, leaves the registers form
    mixed = _equal_rows(7, 12 * MiB)
    mixed[3] = (mixed[3][0], mixed[3][1], mixed[3][0], mixed[3][3])
    assert form(mixed) == A.FORM_TILES
    # the unpack: by itself from 1 MiB, two workgroups per CU up to 75 MiB, one up to 112 MiB
    unpack = lambda elems, k=100, dt=A.F32, div=0, cus=256: A.describe_unpack_launch(elems, k, dt, div, cus)
    assert unpack(MiB // 2) == A.FORM_TILES
    assert unpack(MiB) == A.FORM_REGISTERS_2
    assert unpack(75 * MiB) == A.FORM_REGISTERS_2
    assert unpack(75 * MiB + 1024) == A.FORM_REGISTERS_1
    assert unpack(112 * MiB) == A.FORM_REGISTERS_1
    assert unpack(112 * MiB + 4) == A.FORM_TILES
    assert unpack(64 * MiB, k=1024) == A.FORM_REGISTERS_2 and unpack(64 * MiB, k=1025) == A.FORM_TILES
    assert unpack(64 * MiB, cus=64) == A.FORM_TILES
    # divisors: a power of two everywhere; any other one for float32 up to 64 MiB; the integers' floor division as tiles
    assert unpack(97 * MiB, div=8) == A.FORM_REGISTERS_1 and unpack(97 * MiB, dt=A.I32, div=8) == A.FORM_REGISTERS_1
    assert unpack(64 * MiB, div=6) == A.FORM_REGISTERS_2 and unpack(64 * MiB + 1024, div=6) == A.FORM_TILES
    assert unpack(32 * MiB, dt=A.I32, div=6) == A.FORM_TILES and unpack(16 * MiB, dt=A.I64, div=3) == A.FORM_TILES


def test_launch_form_query_follows_the_options_and_checks_its_arguments():
    A = ring_abi
    rows = _allgather_rows(10_000_019, 6, 0, 4)
    try:
        A.set_option("phased_copy", 0)
        assert A.describe_rows_launch(rows, A.I32, A.ROLE_ALLGATHER, 256) == A.FORM_PACED
        assert A.describe_unpack_launch(25_557_032, 161, A.F32, 8, 256) == A.FORM_TILES
        A.set_option("paced_copy", 0)
        assert A.describe_rows_launch(rows, A.I32, A.ROLE_ALLGATHER, 256) == A.FORM_TILES
        A.set_option("paced_copy", 1)
        assert A.describe_rows_launch(_equal_rows(3, 1000), A.F32, A.ROLE_ALLGATHER, 256) == A.FORM_PACED
        A.set_option("phased_copy", 1)
        assert A.describe_rows_launch(_equal_rows(3, 1000), A.F32, A.ROLE_ALLGATHER, 256) == A.FORM_REGISTERS_2
    finally:
        A.set_option("phased_copy", -1)
        A.set_option("paced_copy", -1)
    assert A.describe_rows_launch(rows, A.I32, A.ROLE_ALLGATHER, 256) == A.FORM_REGISTERS_2
    with pytest.raises(A.RingError):
        A.describe_rows_launch(rows, 7, A.ROLE_ALLGATHER, 256)
    with pytest.raises(A.RingError):
        A.describe_rows_launch(rows, A.I32, 5, 256)
    with pytest.raises(A.RingError):
        A.describe_rows_launch(rows, A.I32, A.ROLE_ALLGATHER, 0)
    with pytest.raises(A.RingError):
        A.describe_unpack_launch(1 << 20, 10, A.F32, -1, 256)


def test_a_batch_outlives_its_world_but_cannot_be_submitted():
    """mpic_batch_submit after mpic_world_destroy answers FAILED_PRECONDITION instead of
    walking into the freed world; the batch can still be waited for and destroyed."""
    L = _plugin.lib()
    world = ctypes.c_void_p()
    assert L.mpic_world_create(2, ctypes.byref(world)) == _plugin.OK
    names = (ctypes.c_char_p * 1)(b"grad")
    dtypes = (ctypes.c_int * 1)(_plugin.DT_FLOAT)
    ndims = (ctypes.c_int * 1)(1)
    dims = (ctypes.c_int64 * 1)(16)
    ins = (ctypes.c_void_p * 1)(0x1000)          # never dereferenced: nothing is submitted
    outs = (ctypes.c_void_p * 1)(0x2000)
    batches = []
    for _ in range(2):
        b = ctypes.c_void_p()
        assert L.mpic_batch_create(world, 0, 1, names, dtypes, ndims, dims, ins, outs, 0, ctypes.byref(b)) == _plugin.OK
        batches.append(b)
    assert L.mpic_batch_busy(batches[0]) == 0
    assert L.mpic_batch_destroy(batches[0]) == _plugin.OK      # before its world: unregisters itself
    assert L.mpic_world_destroy(world) == _plugin.OK
    rc = L.mpic_batch_submit(batches[1])
    assert _plugin.error_for(rc, "").__class__ is mpi.FailedPreconditionError
    assert b"destroyed" in L.mpic_last_error()
    assert L.mpic_batch_wait(batches[1], None) == _plugin.OK
    assert L.mpic_batch_destroy(batches[1]) == _plugin.OK      # after its world


def test_dimensions_that_are_negative_or_do_not_fit_are_refused():
    """mpic_context_add_input, mpic_allreduce_batch and mpic_batch_create take dimensions from the
    embedder: a negative one, or a shape whose byte size wraps, is INVALID_ARGUMENT before anything is
    filed (no GPU needed: nothing is computed)."""
    L = _plugin.load_library()
    w = ctypes.c_void_p()
    assert L.mpic_world_create(2, ctypes.byref(w)) == 0
    try:
        c = ctypes.c_void_p()
        assert L.mpic_context_create(w, 0, b"MPIAllreduce", b"x", b"GPU", _plugin.ALLOC_FN(0), None, ctypes.byref(c)) == 0
        for dims in ((-1,), (4, -2), (2 ** 40, 2 ** 40), (2 ** 62, 2), (2 ** 60,)):
            d = (ctypes.c_int64 * len(dims))(*dims)
            assert L.mpic_context_add_input(c, _plugin.DT_FLOAT, len(dims), d, ctypes.c_void_p(4096), 0) == _plugin.INVALID_ARGUMENT, dims
        d = (ctypes.c_int64 * 2)(2 ** 30, 2 ** 29)                  # 2^59 elements: the largest that still fits
        assert L.mpic_context_add_input(c, _plugin.DT_FLOAT, 2, d, ctypes.c_void_p(4096), 0) == 0
        assert L.mpic_context_destroy(c) == 0
        names = (ctypes.c_char_p * 2)(b"a", b"b")
        dtypes = (ctypes.c_int * 2)(_plugin.DT_FLOAT, _plugin.DT_FLOAT)
        ndims = (ctypes.c_int * 2)(1, 2)
        ptrs = (ctypes.c_void_p * 2)(4096, 8192)
        for dims in ((4, 3, -1), (4, 2 ** 40, 2 ** 40)):
            d = (ctypes.c_int64 * 3)(*dims)
            contexts = (ctypes.c_void_p * 2)()
            assert L.mpic_allreduce_batch(w, 0, 2, names, dtypes, ndims, d, ptrs, ptrs, 0, contexts) == _plugin.INVALID_ARGUMENT
            assert not contexts[0] and not contexts[1]
            batch = ctypes.c_void_p()
            assert L.mpic_batch_create(w, 0, 2, names, dtypes, ndims, d, ptrs, ptrs, 0, ctypes.byref(batch)) == _plugin.INVALID_ARGUMENT
            assert not batch.value
    finally:
        assert L.mpic_world_destroy(w) == 0


def test_allgather_sizes_that_are_negative_or_do_not_fit_are_refused():
    """MPIAllgather's `sizes` input comes from the embedder (the reference takes it from the sizing
    pre-pass, mpi_ops.py:152-160): a negative entry, or entries whose gathered tensor would not fit,
    end the op with InvalidArgument before anything is filed."""
    L = _plugin.load_library()
    w = ctypes.c_void_p()
    assert L.mpic_world_create(2, ctypes.byref(w)) == 0
    try:
        init = ctypes.c_void_p()
        assert L.mpic_context_create(w, 0, b"MPIInit", b"MPIInit", b"CPU", _plugin.ALLOC_FN(0), None, ctypes.byref(init)) == 0
        assert L.mpic_context_compute(init) == 0 and L.mpic_context_wait(init) == 0 and L.mpic_context_destroy(init) == 0
        for sizes, message in (((3, -1), b"non-negative"), ((2 ** 62, 2 ** 62), b"non-negative"),
                               ((2 ** 40, 2 ** 40), b"too large")):
            c = ctypes.c_void_p()
            assert L.mpic_context_create(w, 0, b"MPIAllgather", b"g", b"GPU", _plugin.ALLOC_FN(0), None, ctypes.byref(c)) == 0
            dims = (ctypes.c_int64 * 2)(3, 2 ** 20)
            assert L.mpic_context_add_input(c, _plugin.DT_FLOAT, 2, dims, ctypes.c_void_p(4096), 0) == 0
            host_sizes = (ctypes.c_int64 * 2)(*sizes)
            one = (ctypes.c_int64 * 1)(2)
            assert L.mpic_context_add_input(c, _plugin.DT_INT64, 1, one, host_sizes, 1) == 0
            assert L.mpic_context_compute(c) == 0
            assert L.mpic_context_wait(c) == _plugin.INVALID_ARGUMENT, sizes
            assert message in L.mpic_context_message(c), (sizes, L.mpic_context_message(c))
            assert L.mpic_context_destroy(c) == 0
    finally:
        assert L.mpic_world_destroy(w) == 0


def test_a_batch_that_fails_gives_its_node_names_back():
    """An entry the plugin cannot describe (more than 8 dimensions) fails the whole allreduce_batch
    call and files nothing; the auto-generated node names it took are given back, so the rank's
    next unnamed op still matches the other ranks'."""
    with mpi.Session(size=2) as session:
        with session.as_rank(0):
            good = torch.zeros(4)
            with pytest.raises(mpi.OpError):
                mpi.allreduce_batch([good, torch.zeros((1,) * 9), good])
            assert session._node_name(0, 'MPIAllreduce', None) == 'MPIAllreduce'
            assert session._node_name(0, 'MPIAllreduce', None) == 'MPIAllreduce_1'
