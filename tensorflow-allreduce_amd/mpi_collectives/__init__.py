"""MI355X-native ring collectives with the API of tensorflow.contrib.mpi_collectives.

This package mirrors ``tensorflow/contrib/mpi_collectives/__init__.py``:
``allreduce``, ``allgather``, ``DistributedOptimizer`` and ``Session`` (plus
``size``, ``rank``, ``local_rank``, ``init``), over torch tensors that live in
the HBM of one MI355X. The per-rank data path of the ring (segment split,
reduce-scatter accumulate, allgather copies, fusion pack/unpack) runs in
hand-written gfx950 kernels behind a C ABI; there is no CPU implementation.

Ranks are *virtual*. Where the reference runs one MPI process per rank, a
``Session`` here owns all ranks in one process, on one GPU:

    import mpi_collectives as mpi

    with mpi.Session(size=8) as session:            # runs init(), like mpi.Session
        sums = []
        for r in range(8):                          # what each process would do
            with session.as_rank(r):
                sums.append(mpi.allreduce(x[r], average=False))
        sums = session.run(sums)                    # list of torch tensors

As in graph-mode TensorFlow the collective calls return handles; a reduction
"will not start until all processes are ready", so values exist once every
rank has submitted the op and ``session.run`` has been called. A session can
instead hold ONE real rank whose peers' incoming segments were staged in HBM
beforehand (``Session(size=8, rank=3)`` + ``session.stage_peers``); its
collectives complete at once.

@@Session
@@DistributedOptimizer
@@allreduce
@@allreduce_batch
@@allgather
"""
import contextlib
import os
import threading

import torch

from . import _plugin, mpi_ops, ring_abi
from ._plugin import (FailedPreconditionError, InternalError, InvalidArgumentError,  # noqa: F401
                      NotFoundError, OpError, UnknownError)
from .mpi_ops import _allreduce, allgather, init, local_rank, rank, size  # noqa: F401

_TORCH2RING = {torch.float32: ring_abi.F32, torch.int32: ring_abi.I32, torch.int64: ring_abi.I64}


class PendingTensor:
    """Handle of a collective's result (the graph tensor of the reference).

    ``session.run(handle)`` or ``handle.result()`` returns the torch tensor once
    every rank has submitted the op."""

    def __init__(self, session):
        self._session = session
        self._value = None
        self._error = None
        self._ready = False
        self._post = []       # fn(tensor) -> tensor applied to the value when it arrives
        self._first_op = None  # the op (chain) whose completion produces the value

    def _set(self, value=None, error=None):
        if error is None:
            for fn in self._post:
                value = fn(value)
        self._value, self._error, self._ready = value, error, True

    def result(self):
        """The tensor. If it is not there yet, runs the session: every rank must
        already have submitted the op (a single thread driving all ranks)."""
        if not self._ready:
            self._session.run()
        if self._error is not None:
            raise self._error
        return self._value

    def wait(self):
        """The tensor, blocking until the collective has run. For ranks driven
        from separate threads, as separate MPI processes would be: the call
        returns once the other ranks' threads have submitted the op."""
        op = self._first_op
        while op is not None and not self._ready:
            self._session._flush()
            self._session._complete(op)
            op = op.next_op
        if self._session.stream:
            ring_abi.stream_synchronize(self._session.stream)     # post-processing (the average) is asynchronous
        if self._error is not None:
            raise self._error
        return self._value


class IndexedSlices:
    """A sparse representation of a set of tensor slices at given indices
    (the tf.IndexedSlices the reference's allreduce accepts)."""

    def __init__(self, values, indices, dense_shape=None):
        self.values, self.indices, self.dense_shape = values, indices, dense_shape


def _env_size():
    """Ranks from the launcher's environment, the variables the reference's
    tests read (mpi_ops_test.py:30-62); 1 when not started under mpirun."""
    for var in ("PMI_SIZE", "OMPI_COMM_WORLD_SIZE"):
        if os.environ.get(var):
            return int(os.environ[var])
    return 1


class Session:
    """Runs MPI ops for a set of virtual ranks; the counterpart of
    tf.contrib.mpi.Session (``__init__.py:237-273``): it initializes MPI
    immediately upon starting.

    Args:
      target, graph, config: accepted for signature compatibility; unused.
      size: number of ranks in the ring (default: the launcher's environment,
        else 1).
      rank: None if all `size` ranks live in this session; otherwise the one
        real rank, whose peers are pre-staged with `stage_peers`.
      device: "GPU" (default when a GPU is present) or "CPU": where init() runs.
        Collectives have GPU kernels only.
      fusion_threshold: bytes per rank of a fusion buffer (0 = off, the
        reference's behaviour). When set, the allreduces submitted between two
        `run` calls are packed, per element type and up to this many bytes, into
        one buffer per rank and reduced by a single ring; each result is then
        the ring applied to the packed buffer, which for float32 rounds
        differently from one ring per tensor.
    """

    def __init__(self, target='', graph=None, config=None, size=None, rank=None, device=None,
                 fusion_threshold=0):
        del target, graph, config
        L = _plugin.load_library('libmpi_collectives.so', mpi_ops._REQUIRED_OPS)
        self.size = int(size) if size is not None else _env_size()
        self.real_rank = rank
        self.device = device or ("GPU" if torch.cuda.is_available() else "CPU")
        import ctypes
        h = ctypes.c_void_p()
        if rank is None:
            rc = L.mpic_world_create(self.size, ctypes.byref(h))
        else:
            rc = L.mpic_world_create_prestaged(self.size, int(rank), ctypes.byref(h))
        if rc != 0:
            raise _plugin.error_for(rc, "could not create an MPI world of size %r, rank %r" % (size, rank))
        self._world = h.value
        self._lock = threading.RLock()   # ranks may be driven from separate threads
        self._pending = []          # ops submitted and not yet waited for
        self._submitted = {}        # node name -> set of ranks, for the run() guard
        self._batches = []          # AllreduceBatch objects built on this session
        self._counters = {}         # (rank, op) -> next auto-name index
        self._keep = []             # staged buffers kept alive until consumed
        self._prev = None
        self._fusion_buffer = None
        self._enter_scope()
        try:
            # Initialize MPI on the relevant device (__init__.py:271-273).
            self.run(init())
            if fusion_threshold and rank is None and self.size > 1:
                per_rank = (int(fusion_threshold) + 15) // 16 * 16
                self._fusion_buffer = torch.empty(per_rank * self.size, dtype=torch.uint8, device="cuda")
                rc = L.mpic_world_set_fusion_buffer(self._world, self._fusion_buffer.data_ptr(), per_rank)
                if rc != 0:
                    raise InvalidArgumentError("could not install a fusion buffer of %d bytes per rank" % per_rank)
        except Exception:
            self.close()
            raise

    # -- scoping ---------------------------------------------------------------
    def _enter_scope(self):
        self._prev = (mpi_ops._scope.session, mpi_ops._scope.rank)
        mpi_ops._scope.session = self
        mpi_ops._scope.rank = self.real_rank if self.real_rank is not None else 0

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False

    @contextlib.contextmanager
    def as_rank(self, r):
        """Run the enclosed MPI ops as virtual rank `r`."""
        if not 0 <= r < self.size or (self.real_rank is not None and r != self.real_rank):
            raise InvalidArgumentError("rank %r is not a rank of this session" % (r,))
        prev = (mpi_ops._scope.session, mpi_ops._scope.rank)
        mpi_ops._scope.session, mpi_ops._scope.rank = self, r
        try:
            yield self
        finally:
            mpi_ops._scope.session, mpi_ops._scope.rank = prev

    def close(self):
        if self._world is not None:
            _plugin.lib().mpic_world_destroy(self._world)      # fails whatever is still running
            self._world = None
            for b in list(self._batches):
                b.close()
            if mpi_ops._scope.session is self and self._prev is not None:
                mpi_ops._scope.session, mpi_ops._scope.rank = self._prev
            self._pending, self._keep = [], []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- world ---------------------------------------------------------------------
    @property
    def stream(self):
        """The world's dedicated HIP stream (CudaStreamForMPI), as an integer handle."""
        return _plugin.lib().mpic_world_stream(self._world)

    def set_option(self, name, value):
        """"batched", "fuse_copy", "direct" or "sync": see mpic_world_set_option."""
        rc = _plugin.lib().mpic_world_set_option(self._world, name.encode(), int(value))
        if rc != 0:
            raise InvalidArgumentError("unknown session option %r" % name)

    def stage_peers(self, name, rs_segments, ag_segments):
        """Pre-stage what the left neighbour sends for the collective with node
        name `name`: lists of n-1 CUDA tensors (reduce-scatter steps, allgather
        steps). For an allgather pass rs_segments=None."""
        import ctypes
        n1 = self.size - 1
        rs = list(rs_segments) if rs_segments is not None else None
        ag = list(ag_segments)
        if len(ag) != n1 or (rs is not None and len(rs) != n1):
            raise InvalidArgumentError("a ring of %d ranks needs %d staged segments per phase" % (self.size, n1))
        arr_ag = (ctypes.c_void_p * max(n1, 1))(*[t.data_ptr() if t.numel() else None for t in ag])
        arr_rs = None
        if rs is not None:
            arr_rs = (ctypes.c_void_p * max(n1, 1))(*[t.data_ptr() if t.numel() else None for t in rs])
        rc = _plugin.lib().mpic_stage_peers(self._world, name.encode(), arr_rs, arr_ag)
        if rc != 0:
            raise InvalidArgumentError("stage_peers needs a session created with rank=...")
        self._keep.append((rs, ag))

    # -- op submission (used by mpi_ops) ------------------------------------------------
    def _node_name(self, r, op, name):
        """TensorFlow uniquifies node names per graph: op, op_1, op_2, ... Every
        rank builds the same graph, so the k-th unnamed op matches across ranks."""
        base = name if name is not None else op
        with self._lock:
            k = self._counters.get((r, base), 0)
            self._counters[(r, base)] = k + 1
        return base if k == 0 else "%s_%d" % (base, k)

    def _order_after_producers(self, inputs):
        """The inputs' producers must have finished before the ring reads them. The
        reference defers the enqueue with a host callback on the producer's stream
        (mpi_ops.cc:1099-1105); here the world's stream waits, on the device, for an
        event recorded on the stream the inputs were produced on: torch's current
        stream (inputs produced on another stream must be ordered with it first).
        Nothing on the host blocks."""
        if not any(t.is_cuda for t in inputs):
            return
        producers = torch.cuda.current_stream(inputs[0].device)
        if not self.stream:
            producers.synchronize()      # before MPIInit there is no stream to order
        elif not producers.query():
            ready = torch.cuda.Event()
            ready.record(producers)
            ring_abi.stream_wait_event(self.stream, ready.cuda_event)

    def _submit_batch(self, r, names, tensors, divisor=0):
        """One MPIAllreduce node per tensor, all filed with one call into the plugin.
        Returns one handle per tensor."""
        inputs = [t.contiguous() for t in tensors]
        self._order_after_producers(inputs)
        with self._lock:
            counters_before = dict(self._counters)
        node_names = [self._node_name(r, 'MPIAllreduce', name) for name in names]
        # the outputs: one allocation per element type, cut into the tensors' shapes
        outputs = [None] * len(inputs)
        by_dtype = {}
        for j, t in enumerate(inputs):
            by_dtype.setdefault((t.dtype, t.device), []).append(j)
        for (dtype, device), idx in by_dtype.items():
            flat = torch.empty(sum(inputs[j].numel() for j in idx), dtype=dtype, device=device)
            for j, piece in zip(idx, flat.split([inputs[j].numel() for j in idx])):
                outputs[j] = piece.view(inputs[j].shape)
        try:
            batch = _plugin.PendingBatch(self._world, r, node_names, inputs, outputs, divisor)
        except OpError:
            # nothing was filed: give the names back, or this rank's next unnamed op would carry another
            # name than the same op on the ranks whose call succeeded
            with self._lock:
                for key in [k for k in self._counters if k[0] == r]:
                    if key in counters_before:
                        self._counters[key] = counters_before[key]
                    else:
                        del self._counters[key]
            raise
        batch.rank = r
        batch.next_op = batch.on_done = batch.handle = batch.fail_handle = None
        batch.lock = threading.Lock()
        batch.completed = False
        batch.error = None
        batch.handles = []
        for _ in inputs:
            h = PendingTensor(self)
            h._first_op = batch
            batch.handles.append(h)
        with self._lock:
            for name in node_names:
                self._submitted.setdefault(name, set()).add(r)
            self._pending.append(batch)
        return batch.handles

    def _submit(self, r, op, node_name, inputs, device, divisor=0):
        self._order_after_producers(inputs)
        pending = _plugin.PendingOp(self._world, r, op, node_name, inputs, device, divisor)
        pending.rank = r
        pending.node_names = [node_name]
        pending.handle = pending.fail_handle = pending.on_done = pending.next_op = None
        pending.lock = threading.Lock()
        pending.completed = False
        pending.error = None
        if op in ("MPIAllreduce", "MPIAllgather"):
            with self._lock:
                self._submitted.setdefault(node_name, set()).add(r)
                self._pending.append(pending)
        return pending

    @property
    def _immediate(self):
        return self.real_rank is not None or self.size == 1

    def _result(self, pending):
        handle = PendingTensor(self)
        handle._first_op = pending
        pending.handle = handle
        if self._immediate:
            self._drain()
        return handle

    def _chain_allgather(self, r, sizing, tensor, name, dev, divisor=0):
        handle = PendingTensor(self)
        handle._first_op = sizing

        def after_sizing(outputs):
            sizes = outputs[0].cpu() if outputs[0].is_cuda else outputs[0]   # host-memory `sizes` input
            node = self._node_name(r, 'MPIAllgather', name)
            with self.as_rank(r):
                second = self._submit(r, 'MPIAllgather', node, [tensor, sizes], dev, divisor)
            second.handle = handle
            sizing.next_op = second

        sizing.on_done = after_sizing
        sizing.fail_handle = handle
        if self._immediate:
            self._drain()
        return handle

    def _after(self, handle, fn):
        """Run fn(tensor) -> tensor on the result of `handle` once it exists."""
        if not handle._ready:
            handle._post.append(fn)
        elif handle._error is None:
            handle._value = fn(handle._value)
            if self.stream:
                ring_abi.stream_synchronize(self.stream)

    def _flush(self):
        """Start a coordinator tick: negotiate and run what was submitted."""
        _plugin.lib().mpic_world_flush(self._world)

    def _complete(self, p):
        """Wait for op p (blocks until every rank has submitted it), then run
        its continuation and publish its result; once per op, from any thread."""
        with p.lock:
            if p.completed:
                return p.error
            if isinstance(p, AllreduceBatch):
                errors = p._c.wait()
                p.errors = errors
                p.error = next((e for e in errors if e is not None), None) if errors else None
            elif isinstance(p, _plugin.PendingBatch):
                for h, out, e in zip(p.handles, p.outputs, p.wait()):
                    if e is None:
                        h._set(value=out)
                    else:
                        h._set(error=e)
                        p.error = p.error or e
            else:
                try:
                    outputs = p.wait()
                    if p.on_done:
                        p.on_done(outputs)
                    if p.handle is not None:
                        p.handle._set(value=outputs[0])
                except OpError as e:
                    p.error = e
                    for h in (p.handle, p.fail_handle):
                        if h is not None:
                            h._set(error=e)
            p.completed = True
        return self._retire(p)

    def _retire(self, p):
        with self._lock:
            if p in self._pending:
                self._pending.remove(p)
            if isinstance(p, AllreduceBatch):
                ranks = self._submitted.get(p.names_key)
                if ranks is not None:
                    ranks.discard(p.rank)
                    if not ranks:
                        self._submitted.pop(p.names_key, None)
                return p.error
            for name in p.node_names:
                ranks = self._submitted.get(name)
                if ranks is not None:
                    ranks.discard(p.rank)
                    if not ranks:
                        self._submitted.pop(name, None)
        return p.error

    def _check_all_ranks_submitted(self, batch):
        if self.real_rank is not None:
            return
        prepared = [p for p in batch if isinstance(p, AllreduceBatch) and not p.completed]
        for p in batch:
            if p.completed:
                continue
            if isinstance(p, AllreduceBatch) and len(self._submitted.get(p.names_key, ())) == self.size:
                continue            # every rank submitted this same set of nodes as one batch
            for name in p.node_names:
                ranks = set(self._submitted.get(name, ()))
                ranks.update(q.rank for q in prepared if name in q.name_set)
                if len(ranks) != self.size:
                    raise FailedPreconditionError(
                        "collective %r was submitted by ranks %s of %d; every rank must submit it "
                        "before the session runs" % (name, sorted(ranks), self.size))

    def _drain(self):
        first_error = None
        while True:
            with self._lock:
                batch = list(self._pending)
                if not batch:
                    break
                self._check_all_ranks_submitted(batch)
            self._flush()
            for p in batch:
                error = self._complete(p)          # every op is completed, also after a failure
                first_error = first_error or error
        if self.stream:
            ring_abi.stream_synchronize(self.stream)
        if first_error is not None:
            raise first_error

    def run(self, fetches=None, feed_dict=None):
        """Completes every submitted collective and returns `fetches` with each
        handle replaced by its torch tensor."""
        del feed_dict
        self._drain()
        return _resolve(fetches)


def _resolve(x):
    if isinstance(x, PendingTensor):
        return x.result()
    if isinstance(x, AllreduceBatch):
        return x.results()
    if isinstance(x, IndexedSlices):
        return IndexedSlices(_resolve(x.values), _resolve(x.indices), x.dense_shape)
    if isinstance(x, (list, tuple)):
        return type(x)(_resolve(v) for v in x)
    if isinstance(x, dict):
        return {k: _resolve(v) for k, v in x.items()}
    return x


def _div(session, handle):
    """tf.div(x, cast(size(), x.dtype)) applied to a collective's result: true
    division for float32, floor division for integers (__init__.py:160-164,
    math_ops.py:982-985), by the ring_scale kernel on the session's stream."""
    n = session.size

    def fn(t):
        if t.numel():
            # asynchronous on the session's stream; run() and wait() drain it
            ring_abi.scale(_TORCH2RING[t.dtype], t.data_ptr(), t.numel(), n, session.stream)
        return t

    session._after(handle, fn)
    return handle


def allreduce(tensor, average=True):
    """Perform an MPI allreduce on a torch.Tensor or an IndexedSlices.

    Arguments:
        tensor: torch.Tensor (on the GPU) or IndexedSlices to reduce. The
                shape of the input must be identical across all ranks.
        average: If True, computes the average over all ranks.
                 Otherwise, computes the sum over all ranks.

    This function performs a bandwidth-optimal ring allreduce on the input
    tensor. If the input is an IndexedSlices, the function instead does an
    allgather on the values and the indices, effectively doing an allreduce on
    the represented tensor.
    """
    session, _ = mpi_ops._current()
    # With every rank in this process the average's tf.div is fused into the
    # collective (the owner of a segment divides in its last accumulate). A
    # session with pre-staged peers keeps the reference's order, collective
    # then division, so that what is staged is the reference's wire traffic.
    fold = session.size if average and session.real_rank is None else 0
    if isinstance(tensor, IndexedSlices):
        # For IndexedSlices, do two allgathers instead of an allreduce.
        values = allgather(tensor.values, divisor=fold)
        indices = allgather(tensor.indices)
        # To make this operation into an average, divide all gathered values by the MPI size.
        new_values = _div(session, values) if average and not fold else values
        return IndexedSlices(new_values, indices, dense_shape=tensor.dense_shape)
    summed_tensor = _allreduce(tensor, divisor=fold)
    return _div(session, summed_tensor) if average and not fold else summed_tensor


def allreduce_batch(tensors, average=True):
    """allreduce() of every dense tensor of a list; returns the list of results
    (not in the reference, whose callers loop over allreduce).

    Each tensor is its own MPIAllreduce node, named, negotiated, validated and
    (with a fusion threshold) grouped exactly as the same calls made one by one
    would be; what changes is the cost of making them: one call into the plugin
    for all of them instead of several per tensor. This is what
    DistributedOptimizer.compute_gradients uses for the gradient set of a step."""
    session, r = mpi_ops._current()
    tensors = list(tensors)
    if session._immediate or not tensors:
        return [allreduce(t, average=average) for t in tensors]      # pre-staged peers / one rank: nothing to batch
    fold = session.size if average else 0
    return session._submit_batch(r, [None] * len(tensors), tensors, fold)


class _BatchResult(PendingTensor):
    """Result j of an AllreduceBatch: a handle like any other, whose tensor is
    the batch's output j after the latest submission."""

    def __init__(self, batch, index):
        self._batch, self._index = batch, index

    def _tensor(self):
        errors = self._batch.errors
        if errors and errors[self._index] is not None:
            raise errors[self._index]
        return self._batch.outputs[self._index]

    def result(self):
        if not self._batch.completed:
            self._batch.session.run()
        return self._tensor()

    def wait(self):
        self._batch.wait()
        return self._tensor()


class AllreduceBatch:
    """The allreduces of a list of dense tensors, built once and run every step.

    In the reference the graph is built once (one MPIAllreduce node per
    gradient, each with its name, __init__.py:195-205) and every session.run()
    executes the same nodes again. This is that graph fragment for one rank:
    construction names the nodes and creates their kernels; submit() runs each
    of them once more on the same tensors (new values, same memory), one call
    into the plugin for all of them; results are valid until the next submit().
    Every rank builds its batch in the same order, so the k-th node of each
    rank carries the same name.

      tensors: contiguous CUDA tensors; their memory is read at every submit.
      average: divide by the number of ranks (fused into the collective).
      inplace: the results replace the inputs' values instead of going to
               memory of their own (one allocation per element type, made once).
    """

    def __init__(self, tensors, average=True, inplace=False):
        session, r = mpi_ops._current()
        tensors = list(tensors)
        if session._immediate:
            raise InvalidArgumentError("a prepared batch needs a session that holds every rank")
        for t in tensors:
            if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous()):
                raise InvalidArgumentError("a prepared batch takes contiguous CUDA tensors")
        self.session, self.rank, self.inputs = session, r, tensors
        self.node_names = [session._node_name(r, 'MPIAllreduce', None) for _ in tensors]
        self.names_key = tuple(self.node_names)
        self.name_set = frozenset(self.node_names)
        if inplace:
            self.outputs = tensors
        else:
            self.outputs = [None] * len(tensors)
            by_dtype = {}
            for j, t in enumerate(tensors):
                by_dtype.setdefault((t.dtype, t.device), []).append(j)
            for (dtype, device), idx in by_dtype.items():
                flat = torch.empty(sum(tensors[j].numel() for j in idx), dtype=dtype, device=device)
                for j, piece in zip(idx, flat.split([tensors[j].numel() for j in idx])):
                    self.outputs[j] = piece.view(tensors[j].shape)
        self._c = _plugin.Batch(session._world, r, self.node_names, tensors, self.outputs,
                                session.size if average else 0)
        self.handles = [_BatchResult(self, j) for j in range(len(tensors))]
        self.lock = threading.Lock()
        self.completed = True          # nothing submitted yet
        self.error = None
        self.errors = None
        self.next_op = self.on_done = self.handle = self.fail_handle = None
        session._batches.append(self)

    def submit(self):
        """Runs the nodes once more. Returns the handles of the results (the
        same objects every time)."""
        session = self.session
        if session._world is None:
            raise FailedPreconditionError("the session of this batch is closed")
        if not self.completed:
            raise FailedPreconditionError("the batch's previous submission has not been completed; "
                                          "run the session first")
        session._order_after_producers(self.inputs[:1])
        self.error = self.errors = None
        self.completed = False
        try:
            self._c.submit()
        except OpError:
            self.completed = True
            raise
        with session._lock:
            session._submitted.setdefault(self.names_key, set()).add(self.rank)
            session._pending.append(self)
        return self.handles

    def wait(self):
        """Blocks until the submission has run (ranks driven from separate threads)."""
        self.session._flush()
        error = self.session._complete(self)
        if self.session.stream:
            ring_abi.stream_synchronize(self.session.stream)
        if error is not None:
            raise error

    def results(self):
        """The output tensors, running the session if the submission is still pending."""
        if not self.completed:
            self.session.run()
        if self.error is not None:
            raise self.error
        return self.outputs

    def close(self):
        self._c.close()
        if self in self.session._batches:
            self.session._batches.remove(self)

    def __del__(self):
        try:
            self._c.close(wait=False)
        except Exception:
            pass


def prepare_allreduce_batch(tensors, average=True, inplace=False):
    """An AllreduceBatch for the current rank (not in the reference, where
    building the graph once is what a TensorFlow program does anyway)."""
    return AllreduceBatch(tensors, average=average, inplace=inplace)


class DistributedOptimizer:
    """An optimizer that wraps a torch.optim.Optimizer, using an MPI allreduce
    to average gradient values before applying gradients to model weights
    (``__init__.py:167-234``).

    Args:
      optimizer: optimizer to use for applying updates.
      name: optional name prefix for the collectives this optimizer issues;
        defaults to "Distributed" followed by the optimizer's type.
      use_locking: accepted for signature compatibility.
      fusion: pack all dense float32 gradients into one fusion buffer and
        reduce them with a single ring allreduce (not in the reference, which
        issues one allreduce per gradient).
    """

    def __init__(self, optimizer, name=None, use_locking=False, fusion=False):
        if name is None:
            name = "Distributed{}".format(type(optimizer).__name__)
        self._optimizer = optimizer
        self._name = name
        self._use_locking = use_locking
        self._fusion = fusion
        self._fused = None      # (FusionPlan, fused buffer, grads) while a fused allreduce is in flight
        self._batch = None      # the dense gradients' allreduces, built once (AllreduceBatch)
        self._batch_key = None
        self._stale = []        # batches replaced while their last submission was still pending
        self._rebuilt = 0       # steps in a row that presented other gradient tensors than the step before

    @property
    def param_groups(self):
        return self._optimizer.param_groups

    def _params(self, var_list=None):
        if var_list is not None:
            return list(var_list)
        return [p for g in self._optimizer.param_groups for p in g["params"]]

    def compute_gradients(self, loss=None, var_list=None):
        """Gradients of all trainable variables, allreduced (averaged) across
        ranks. Calls loss.backward() when a loss is given; returns a list of
        (gradient handle, variable) pairs."""
        if loss is not None:
            loss.backward()
        params = [p for p in self._params(var_list) if p.grad is not None]
        if self._fusion:
            return self._compute_fused(params)
        # one MPIAllreduce per gradient, as in the reference (__init__.py:195-205); the dense ones
        # are submitted together
        dense = [p for p in params if not p.grad.is_sparse]
        reduced = dict(zip((id(p) for p in dense), self._reduce_dense([p.grad for p in dense])))
        out = []
        for p in params:
            g = p.grad
            if g.is_sparse:
                g = g.coalesce()
                slices = IndexedSlices(g.values().contiguous(), g.indices()[0].contiguous(), dense_shape=g.shape)
                out.append((allreduce(slices), p))
            else:
                out.append((reduced[id(p)], p))
        return out

    def _reduce_dense(self, grads):
        """Handles of the averaged dense gradients. A training loop presents the
        same gradient tensors every step, so their MPIAllreduce nodes are built
        once (the reference's graph) and run again while the tensors stay where
        they are; anything else goes through allreduce_batch."""
        session, _ = mpi_ops._current()
        if session._immediate or not grads or not all(g.is_cuda and g.is_contiguous() for g in grads):
            return allreduce_batch(grads)
        key = (id(session),) + tuple(g.data_ptr() for g in grads) + tuple(g.shape for g in grads)
        for old in [b for b in self._stale if b.completed]:
            old.close()
            self._stale.remove(old)
        if self._batch is not None and self._batch_key == key:
            self._rebuilt = 0
            return self._batch.submit()
        if self._batch is not None:
            # other tensors than last step's: the nodes built for those are of no further use
            if self._batch.completed:
                self._batch.close()
            else:
                self._stale.append(self._batch)
            self._batch = self._batch_key = None
            self._rebuilt += 1
        if self._rebuilt >= 2:
            # the gradients move every step (zero_grad(set_to_none=True) frees them): building nodes for
            # tensors that will not be seen again costs more than it saves, and would keep them alive
            return allreduce_batch(grads)
        # in place: the averaged gradient takes the gradient's memory (p.grad then holds the average
        # already when compute_gradients returns), so tensors that stay where they are between steps
        # (zero_grad(), whose default here is set_to_none=False) keep the batch valid
        self._batch, self._batch_key = AllreduceBatch(grads, inplace=True), key
        return self._batch.submit()

    def _compute_fused(self, params):
        session, _ = mpi_ops._current()
        dense = [p for p in params if not p.grad.is_sparse and p.grad.dtype == torch.float32]
        dense_ids = {id(p) for p in dense}
        rest = [p for p in params if id(p) not in dense_ids]
        grads = [p.grad.contiguous() for p in dense]
        plan = ring_abi.FusionPlan([g.data_ptr() if g.numel() else None for g in grads],
                                   [g.numel() for g in grads], ring_abi.F32)
        fused = torch.empty(plan.elements, dtype=torch.float32, device="cuda")
        torch.cuda.current_stream().synchronize()      # the gradients' producers
        plan.pack(fused.data_ptr(), session.stream)
        ring_abi.stream_synchronize(session.stream)
        handle = allreduce(fused, average=False)
        unpacked = {"done": False}

        def unpack(t):
            if not unpacked["done"]:
                # the average's divide (tf.div by the size) rides on the unpack
                plan.unpack_scaled(t.data_ptr(), session.size, session.stream)
                ring_abi.stream_synchronize(session.stream)
                unpacked["done"] = True
                plan.close()
            return t

        session._after(handle, unpack)
        out = [(_FusedGrad(handle, g), p) for g, p in zip(grads, dense)]
        for p in rest:
            out.append((allreduce(p.grad.contiguous()), p))
        return out

    def apply_gradients(self, grads_and_vars, global_step=None, name=None):
        """Stores the reduced gradients on their variables and steps the
        wrapped optimizer."""
        del global_step, name
        for g, p in grads_and_vars:
            g = _resolve(g.resolve() if isinstance(g, _FusedGrad) else g)
            if isinstance(g, IndexedSlices):
                idx = g.indices.reshape(1, -1)
                p.grad = torch.sparse_coo_tensor(idx, g.values, size=tuple(g.dense_shape)).coalesce()
            else:
                p.grad = g.reshape(p.shape)
        return self._optimizer.step()

    def minimize(self, loss, global_step=None, var_list=None):
        """compute_gradients followed by apply_gradients. In a session that holds
        several virtual ranks call the two halves yourself, with every rank's
        compute_gradients before the first apply_gradients."""
        return self.apply_gradients(self.compute_gradients(loss, var_list), global_step=global_step)

    def step(self, closure=None):
        if closure is not None:
            closure()
        return self.apply_gradients(self.compute_gradients())

    def zero_grad(self, set_to_none=False):
        """Clears the gradients. Unlike torch's own default the tensors are kept
        and zeroed: gradients that stay where they are let the next step run the
        allreduce nodes built for them again instead of building new ones."""
        return self._optimizer.zero_grad(set_to_none=set_to_none)

    def close(self):
        """Destroys the allreduce nodes this optimizer has built (a closing session does the same)."""
        for b in self._stale + ([self._batch] if self._batch is not None else []):
            if b.completed:
                b.close()
        self._stale, self._batch, self._batch_key = [], None, None

    def state_dict(self):
        return self._optimizer.state_dict()

    def load_state_dict(self, state):
        return self._optimizer.load_state_dict(state)


class _FusedGrad:
    """A gradient that comes back through the fusion buffer."""

    def __init__(self, handle, grad):
        self._handle, self._grad = handle, grad

    def resolve(self):
        self._handle.result()      # runs the unpack
        return self._grad
