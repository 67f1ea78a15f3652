"""The ring over a transport (mpic_ring_allreduce_transport / _allgather_transport):
the reference's loop structure, MPI_Irecv / MPI_Send / MPI_Wait and MPI_Sendrecv
on device buffers, with the in-process loopback transport standing in for MPI.
Every virtual rank is driven by its own thread, as separate MPI processes would
be. Results are compared bit for bit with the CPU oracle's ring."""
import ctypes
import threading

import numpy as np
import pytest
import torch

import gpu_util as G
from gpu_util import ring_abi
from mpi_collectives import _plugin

pytestmark = pytest.mark.gpu

DT = {np.dtype(np.float32): _plugin.DT_FLOAT, np.dtype(np.int32): _plugin.DT_INT32,
      np.dtype(np.int64): _plugin.DT_INT64}
TIMEOUT = 20.0


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    G.require_gpu()


def cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def flags_of(chunks=1, divisor=0):
    return ((chunks - 1) << 4) | (divisor << 8)


def run_ranks(n, body, wrap=None):
    """body(r, transport, stream) on one thread per rank over a fresh loopback;
    returns the list of results, raising the first failure."""
    L = _plugin.load_library()
    h = ctypes.c_void_p()
    assert L.mpic_loopback_create(n, TIMEOUT, ctypes.byref(h)) == 0
    results, errors = [None] * n, [None] * n

    def worker(r):
        try:
            t = _plugin.Transport()
            assert L.mpic_loopback_endpoint(h.value, r, ctypes.byref(t)) == 0
            if wrap is not None:
                t = wrap(r, t)
            stream = ring_abi.stream_create()
            try:
                results[r] = body(r, t, stream)
            finally:
                ring_abi.stream_synchronize(stream)
                ring_abi.stream_destroy(stream)
        except BaseException as e:          # noqa: BLE001 - reported by the main thread
            errors[r] = e

    threads = [threading.Thread(target=worker, args=(r,)) for r in range(n)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(4 * TIMEOUT)
    alive = [t for t in threads if t.is_alive()]
    assert not alive, "rank threads did not finish"
    L.mpic_loopback_destroy(h.value)
    for e in errors:
        if e is not None:
            raise e
    return results


def allreduce_over_transport(ins, dtype, chunks, temp_factor, divisor=0, in_place=False, wrap=None):
    L = _plugin.load_library()
    n, count = len(ins), ins[0].size
    seg = ring_abi.temp_elements(count, n)
    tdt = G.NP2TORCH[np.dtype(dtype)]
    dins = [cuda(x) for x in ins]
    douts = [d if in_place else torch.zeros(count + 3, dtype=tdt, device="cuda")[:count] for d in dins]
    temps = [torch.zeros(max(temp_factor * seg, 1), dtype=tdt, device="cuda") for _ in range(n)]
    torch.cuda.synchronize()

    def body(r, t, stream):
        rc = L.mpic_ring_allreduce_transport(n, r, DT[np.dtype(dtype)], dins[r].data_ptr() if count else None,
                                             douts[r].data_ptr() if count else None, temps[r].data_ptr(),
                                             temp_factor * seg, count, ctypes.byref(t), stream,
                                             flags_of(chunks, divisor))
        assert rc == 0, L.mpic_last_error()
        return rc

    run_ranks(n, body, wrap)
    torch.cuda.synchronize()
    if not in_place:
        for r in range(n):
            assert torch.equal(dins[r], cuda(ins[r]))      # inputs are never written
    return [G.host(o) for o in douts]


def tf_div(x, n):
    with np.errstate(all="ignore"):
        return (x / np.float32(n) if x.dtype == np.float32 else x // x.dtype.type(n)).astype(x.dtype)


@pytest.mark.parametrize("dtype", G.DTYPES)
@pytest.mark.parametrize("chunks,temp_factor", [(1, 1), (4, 1), (4, 2), (16, 2)])
def test_allreduce_over_loopback_matches_oracle(oracle, dtype, chunks, temp_factor):
    for n, count in ((1, 11), (2, 7), (3, 2), (5, 4099), (8, 100_003), (4, 0)):
        ins = [G.random_array(np.random.default_rng(31 * n + r), count, dtype, wide=dtype == np.float32)
               for r in range(n)]
        want = oracle.ring_allreduce(ins)
        got = allreduce_over_transport(ins, dtype, chunks, temp_factor)
        for r in range(n):
            G.assert_same_bits(got[r], want[r], "transport ring n=%d count=%d rank %d chunks=%d temp x%d"
                               % (n, count, r, chunks, temp_factor))


def test_allreduce_in_place_and_with_the_average_folded_in(oracle):
    n, count = 6, 50_001
    for dtype in G.DTYPES:
        ins = [G.random_array(np.random.default_rng(77 + r), count, dtype) for r in range(n)]
        want = oracle.ring_allreduce(ins)[0]
        for chunks, temp_factor in ((1, 1), (3, 2)):
            got = allreduce_over_transport(ins, dtype, chunks, temp_factor, divisor=n, in_place=chunks == 3)
            for r in range(n):
                G.assert_same_bits(got[r], tf_div(want, n), "average over the transport, rank %d" % r)


def test_the_call_sequence_is_the_references():
    """Whole segments (chunks = 1): per reduce-scatter step MPI_Irecv from the
    left of the segment (r-i-1) into temp, MPI_Send to the right of segment
    (r-i), MPI_Wait; per allgather step a receive of (r-i) posted, (r-i+1)
    sent, all on tag 12 (ring.h:183-225). The deferred wait of the allgather is
    the only reordering."""
    n, count = 4, 1003
    sizes, _ = ring_abi.segment_table(count, n)
    logs = [[] for _ in range(n)]
    keep = []

    def wrap(r, inner):
        def irecv(user, buf, nbytes, source, tag, request):
            logs[r].append(("irecv", nbytes, source, tag))
            return inner.irecv(user, buf, nbytes, source, tag, request)

        def send(user, buf, nbytes, dest, tag):
            logs[r].append(("send", nbytes, dest, tag))
            return inner.send(user, buf, nbytes, dest, tag)

        def wait(user, request):
            logs[r].append(("wait",))
            return inner.wait(user, request)

        t = _plugin.Transport(inner.user, _plugin.Transport.IRECV(irecv), _plugin.Transport.SEND(send),
                              _plugin.Transport.WAIT(wait))
        keep.append((t, inner))
        return t

    ins = [np.full(count, r + 1, dtype=np.float32) for r in range(n)]
    got = allreduce_over_transport(ins, np.float32, 1, 1, wrap=wrap)
    for r in range(n):
        assert np.array_equal(got[r], np.full(count, 10, dtype=np.float32))
        left, right = (r - 1) % n, (r + 1) % n
        want = []
        for i in range(n - 1):
            want += [("irecv", 4 * sizes[(r - i - 1) % n], left, 12), ("send", 4 * sizes[(r - i) % n], right, 12),
                     ("wait",)]
        for i in range(n - 1):
            want.append(("irecv", 4 * sizes[(r - i) % n], left, 12))
            if i > 0:
                want.append(("wait",))
            want.append(("send", 4 * sizes[(r - i + 1) % n], right, 12))
        want.append(("wait",))
        assert logs[r] == want, "rank %d" % r


@pytest.mark.parametrize("chunks", [1, 5])
def test_allgather_over_loopback_matches_oracle(oracle, chunks):
    L = _plugin.load_library()
    for dtype in G.DTYPES:
        for rows in ([3], [2, 5], [0, 4, 1], [7, 0, 0, 2, 9, 1, 3], [1] * 8):
            n, epr = len(rows), 6
            parts = [G.random_array(np.random.default_rng(5 * n + r), rows[r] * epr, dtype) for r in range(n)]
            want = oracle.ring_allgather([p.reshape(rows[r], epr) for r, p in enumerate(parts)])
            dins = [cuda(p) for p in parts]
            total = sum(rows) * epr
            douts = [torch.zeros(max(total, 1), dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda") for _ in range(n)]
            rows_c = (ctypes.c_size_t * n)(*rows)
            torch.cuda.synchronize()

            def body(r, t, stream):
                rc = L.mpic_ring_allgather_transport(n, r, DT[np.dtype(dtype)],
                                                     dins[r].data_ptr() if rows[r] else None, rows_c, epr,
                                                     douts[r].data_ptr(), ctypes.byref(t), stream, flags_of(chunks))
                assert rc == 0, L.mpic_last_error()

            run_ranks(n, body)
            torch.cuda.synchronize()
            for r in range(n):
                G.assert_same_bits(G.host(douts[r])[:total], np.asarray(want[r]).reshape(-1),
                                   "allgather over the transport rows=%s rank %d" % (rows, r))


def test_a_missing_peer_ends_in_an_error_not_a_hang():
    """Rank 1 never joins: rank 0's send finds no posted receive and gives up
    after the loopback's timeout with the reference's MPI failure message."""
    L = _plugin.load_library()
    h = ctypes.c_void_p()
    assert L.mpic_loopback_create(2, 0.3, ctypes.byref(h)) == 0
    try:
        t = _plugin.Transport()
        assert L.mpic_loopback_endpoint(h.value, 0, ctypes.byref(t)) == 0
        x = torch.ones(64, device="cuda")
        out, temp = torch.empty(64, device="cuda"), torch.empty(32, device="cuda")
        rc = L.mpic_ring_allreduce_transport(2, 0, _plugin.DT_FLOAT, x.data_ptr(), out.data_ptr(), temp.data_ptr(),
                                             32, 64, ctypes.byref(t), None, 0)
        assert rc == _plugin.UNKNOWN
        assert L.mpic_last_error().decode().startswith("MPI operation failed unexpectedly.")
        assert "MPI_Send" in L.mpic_last_error().decode()
        torch.cuda.synchronize()
    finally:
        L.mpic_loopback_destroy(h.value)
