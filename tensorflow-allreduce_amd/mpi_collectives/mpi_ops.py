"""Inter-process communication using (virtual) MPI ranks on one MI355X.

The op wrappers of tensorflow/contrib/mpi_collectives/mpi_ops.py:57-163 with
the same names and arguments, over torch tensors instead of graph tensors.
Each wrapper runs the registered op of the same name in the plugin library;
which virtual rank it runs as, and in which world, comes from the enclosing
`Session` (see the package docstring).
"""
import threading

import torch

from . import _plugin

# The ops the library must register, checked at load (mpi_ops.py:57-59).
MPI_LIB = None
_REQUIRED_OPS = ['MPISize', 'MPIRank', 'MPILocalRank', 'MPIAllgather', 'MPIAllreduce']


def _load_library(name, op_list=None):
    """Loads the plugin containing the specified operators.

    Raises NameError if one of the required ops is missing.
    """
    return _plugin.load_library(name, op_list)


def _mpi_lib():
    global MPI_LIB
    if MPI_LIB is None:
        MPI_LIB = _load_library('libmpi_collectives.so', _REQUIRED_OPS)
    return MPI_LIB


class _Scope(threading.local):
    def __init__(self):
        self.session = None
        self.rank = 0


_scope = _Scope()


def _current():
    _mpi_lib()
    if _scope.session is None:
        raise _plugin.FailedPreconditionError(
            "MPI has not been initialized; use tf.contrib.mpi.Session.")
    return _scope.session, _scope.rank


def _run(op, inputs, name, device=None, divisor=0):
    session, rank = _current()
    node_name = session._node_name(rank, op, name)
    if device is None:
        device = "GPU" if any(t.is_cuda for t in inputs) or not inputs else "CPU"
    return session._submit(rank, op, node_name, inputs, device, divisor)


def _scalar(op, name):
    pending = _run(op, [], name, device=_current()[0].device)
    return int(pending.wait()[0].item())


def size(name=None):
    """The number of MPI processes (MPI_Comm_size of MPI_COMM_WORLD): here the
    number of virtual ranks of the session. Returns a Python int."""
    return _scalar('MPISize', name)


def rank(name=None):
    """The MPI rank of the calling process: the virtual rank of the enclosing
    `Session.as_rank` scope."""
    return _scalar('MPIRank', name)


def init(name=None):
    """Initializes MPI on the device on which it is run. All future MPI ops
    must be run on the same device."""
    session, r = _current()
    pending = session._submit(r, 'MPIInit', session._node_name(r, 'MPIInit', name), [], session.device)
    pending.wait()


def local_rank(name=None):
    """The local MPI rank of the calling process within its node. All virtual
    ranks share one node, so this equals rank()."""
    return _scalar('MPILocalRank', name)


def _allreduce(tensor, name=None, divisor=0):
    """Sums `tensor` over all the MPI processes.

    The reduction is keyed by the name of the op. The tensor type and shape
    must be the same on all ranks for a given name. The reduction will not
    start until all ranks are ready to send and receive the tensor, so the
    returned tensor holds the sum once every rank has submitted the op and the
    session has run (immediately, in a session with pre-staged peers).

    divisor > 0 (not in the reference): the op delivers tf.div(sum, divisor),
    the consumer `allreduce(average=True)` appends, without a pass of its own.
    """
    tensor = tensor.contiguous()            # the ring works on the flat buffer
    pending = _run('MPIAllreduce', [tensor], name, device="GPU" if tensor.is_cuda else "CPU", divisor=divisor)
    return _current()[0]._result(pending)


def allgather(tensor, name=None, divisor=0):
    """Concatenates `tensor` with the same tensor on all other MPI processes
    along the first dimension, which may differ between ranks.

    As in the reference (mpi_ops.py:152-160) this is two collectives: a gather
    of every rank's first-dimension size, flagged by a scalar `sizes` input,
    whose result is the host-side `sizes` input of the gather proper.

    divisor > 0 (not in the reference): the gathered values arrive divided by
    it (tf.div), each rank dividing its own slice on the way into the ring.
    """
    session, r = _current()
    tensor = tensor.contiguous()
    if name is None:
        name = "allgather"
    sizing_name = "{}_sizing".format(name)
    dev = "GPU" if tensor.is_cuda else "CPU"
    sizes_flag = torch.zeros((), dtype=torch.int64)                       # scalar 0: sizing pass
    first = tensor.shape[0] if tensor.dim() > 0 else 0
    my_size = torch.tensor([first], dtype=torch.int64, device=tensor.device)
    sizing = _run('MPIAllgather', [my_size, sizes_flag], sizing_name, device=dev)
    return session._chain_allgather(r, sizing, tensor, name, dev, divisor)
