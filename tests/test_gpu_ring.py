"""GPU parity of the whole ring against the CPU oracle, through the op layer
(mpi_collectives.allreduce / allgather over virtual ranks) and through the
ring driver's C entry points, on the configurations of the benchmark plan:
float32 64 MiB at N=8, ragged int32/int64 at N=6, the ResNet-50 fusion set at
N=8, variable-row allgather at N=16 and 1 GiB float32 at N=64.

Bar: bit-exact for int32, int64 AND float32 (the ring fixes the order of the
additions per segment); NaNs only have to be NaNs."""
import ctypes
import itertools

import numpy as np
import pytest
import torch

import gpu_util as G
import mpi_collectives as mpi
from gpu_util import ring_abi
from mpi_collectives import _plugin

pytestmark = pytest.mark.gpu

DT = {np.dtype(np.float32): _plugin.DT_FLOAT, np.dtype(np.int32): _plugin.DT_INT32,
      np.dtype(np.int64): _plugin.DT_INT64}


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    G.require_gpu()


def cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_inputs(n, count, dtype, seed=0, wide=True):
    return [G.random_array(np.random.default_rng(seed + r), count, dtype, wide=wide and dtype == np.float32)
            for r in range(n)]


# ---- all ranks resident: the op layer --------------------------------------------------

@pytest.mark.parametrize("dtype", G.DTYPES)
@pytest.mark.parametrize("n", [1, 2, 3, 4, 6, 8])
def test_allreduce_all_ranks_matches_oracle(oracle, dtype, n):
    for count in sorted({0, 1, max(n - 1, 0), n, n + 1, 17, 4913, 1_000_003}):
        ins = make_inputs(n, count, dtype, seed=31 * n + count)
        want = oracle.ring_allreduce(ins)
        # the direct form (a world's default), then the lockstep ring without / with
        # the in->out copy as a launch of its own
        for direct, fuse in ((1, 1), (0, 1), (0, 0)):
            with mpi.Session(size=n) as session:
                session.set_option("direct", direct)
                session.set_option("fuse_copy", fuse)
                handles, dins = [], [cuda(x) for x in ins]
                for r in range(n):
                    with session.as_rank(r):
                        assert mpi.rank() == r
                        handles.append(mpi.allreduce(dins[r], average=False))
                outs = session.run(handles)
            for r in range(n):
                G.assert_same_bits(G.host(outs[r]), want[r], "allreduce %s n=%d count=%d rank %d direct=%d fuse=%d"
                                   % (dtype.__name__, n, count, r, direct, fuse))
                G.assert_same_bits(G.host(dins[r]), ins[r], "the input is never written")


@pytest.mark.parametrize("size", [1, 2, 3, 4, 7, 9, 12, 14])
def test_reference_allreduce_gpu_test(oracle, size):
    """mpi_ops_test.py:114-156 (and :84-112 for int32): every rank reduces the
    same [17]^dim tensor; the sum equals tensor*size, exactly for size <= 3
    (the reference's threshold 0). Above that the reference allows 1e-4 / 5e-4;
    here the result must in addition equal the oracle's bit for bit."""
    for dtype, dim in itertools.product((np.int32, np.float32), (1, 2, 3)):
        rng = np.random.default_rng(1234)
        t = rng.uniform(-100, 100, [17] * dim).astype(np.float32) if dtype == np.float32 \
            else rng.integers(-100, 100, [17] * dim).astype(np.int32)
        want = oracle.ring_allreduce([t] * size)[0]
        with mpi.Session(size=size) as session:
            hs = []
            for r in range(size):
                with session.as_rank(r):
                    hs.append(mpi.allreduce(cuda(t), average=False))
            outs = session.run(hs)
        for o in outs:
            assert list(o.shape) == [17] * dim
            G.assert_same_bits(G.host(o), want, "same-input allreduce size=%d dim=%d" % (size, dim))
            diff = np.max(np.abs(G.host(o) - t * dtype(size)))
            if size <= 3 or dtype == np.int32:
                assert diff == 0, "mpi.allreduce on GPU produces incorrect results"
            else:
                assert diff <= 1e-3


@pytest.mark.parametrize("n", [2, 3, 6])
def test_allreduce_average_is_tf_div(oracle, n):
    """allreduce(average=True) = sum then tf.div by the size: true division for
    float32, floor division for integers (__init__.py:160-164)."""
    for dtype in G.DTYPES:
        ins = make_inputs(n, 50_001, dtype, seed=5)
        summed = oracle.ring_allreduce(ins)[0]
        with np.errstate(all="ignore"):
            want = summed / np.float32(n) if dtype == np.float32 else summed // dtype(n)
        with mpi.Session(size=n) as session:
            hs = []
            for r in range(n):
                with session.as_rank(r):
                    hs.append(mpi.allreduce(cuda(ins[r])))            # average=True is the default
            outs = session.run(hs)
        for o in outs:
            G.assert_same_bits(G.host(o), want.astype(dtype), "average %s n=%d" % (dtype.__name__, n))


@pytest.mark.parametrize("direct", [1, 0])
@pytest.mark.parametrize("size", [1, 2, 3, 7, 16])
def test_reference_allgather_tests(size, direct):
    """mpi_ops_test.py:204-263: rank-stamped tensors, equal and variable first
    dimension, 1-3 dims, int32 and float32 (int64 added)."""
    tensor_sizes = ([17, 32, 81, 12, 15, 23, 22] * 5)[:size]
    for dtype, dim, variable in itertools.product((torch.int32, torch.float32, torch.int64), (1, 2, 3), (False, True)):
        rows = tensor_sizes if variable else [17] * size
        with mpi.Session(size=size) as session:
            session.set_option("direct", direct)        # every slice from its owner at once / the lockstep ring
            hs = []
            for r in range(size):
                with session.as_rank(r):
                    tensor = torch.ones([rows[r]] + [17] * (dim - 1), dtype=dtype, device="cuda") * r
                    hs.append(mpi.allgather(tensor))
            outs = session.run(hs)
        for gathered in outs:
            assert list(gathered.shape) == [sum(rows)] + [17] * (dim - 1)
            for i in range(size):
                part = gathered[sum(rows[:i]):sum(rows[:i + 1])]
                assert list(part.shape) == [rows[i]] + [17] * (dim - 1)
                assert bool((part == i).all()), "mpi.allgather produces incorrect gathered tensor"


@pytest.mark.parametrize("direct", [1, 0])
def test_allgather_variable_rows_n16_matches_oracle(oracle, direct):
    """Rank i contributes [rows_i, 1024] float32 with rows_i uniform in [1, 4096]."""
    n = 16
    rows = [int(np.random.default_rng(i).integers(1, 4097)) for i in range(n)]
    ins = [np.random.default_rng(100 + i).standard_normal((rows[i], 1024)).astype(np.float32) for i in range(n)]
    want = np.concatenate(ins, axis=0)
    assert np.array_equal(oracle.ring_allgather([x[:3] for x in ins])[5], np.concatenate([x[:3] for x in ins]))
    with mpi.Session(size=n) as session:
        session.set_option("direct", direct)
        hs = []
        for r in range(n):
            with session.as_rank(r):
                hs.append(mpi.allgather(cuda(ins[r]), name="rows"))
        outs = session.run(hs)
    for o in outs:
        assert list(o.shape) == [sum(rows), 1024]
    for r in (0, 7, 15):
        G.assert_same_bits(G.host(outs[r]), want, "allgather n=16 rank %d" % r)
    for r in range(n):       # all ranks hold the same bytes
        assert torch.equal(outs[r], outs[0])


@pytest.mark.parametrize("direct", [1, 0])
def test_allgather_with_empty_ranks_and_indexed_slices(oracle, direct):
    n = 4
    rows = [3, 0, 5, 1]
    vals = [np.random.default_rng(r).standard_normal((rows[r], 6)).astype(np.float32) for r in range(n)]
    idx = [np.arange(rows[r], dtype=np.int64) * 10 + r for r in range(n)]
    with mpi.Session(size=n) as session:
        session.set_option("direct", direct)
        hs = []
        for r in range(n):
            with session.as_rank(r):
                sl = mpi.IndexedSlices(cuda(vals[r]), cuda(idx[r]), dense_shape=(100, 6))
                hs.append(mpi.allreduce(sl))                        # two allgathers, values / n
        outs = session.run(hs)
    want_vals = np.concatenate(vals) / np.float32(n)
    want_idx = np.concatenate(idx)
    for o in outs:
        G.assert_same_bits(G.host(o.values), want_vals, "IndexedSlices values")
        assert np.array_equal(G.host(o.indices), want_idx)
        assert o.dense_shape == (100, 6)


# ---- ragged integers at N=6 (10,000,019 elements) -------------------------------------------

@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_ragged_integers_n6(oracle, dtype):
    n, count = 6, 10_000_019
    ins = [np.random.default_rng(r).integers(-1000, 1001, count).astype(dtype) for r in range(n)]
    want = oracle.ring_allreduce_lockstep(ins)[0]
    assert np.array_equal(want, sum(x.astype(np.int64) for x in ins).astype(dtype))   # integers: any order
    with mpi.Session(size=n) as session:
        hs = []
        for r in range(n):
            with session.as_rank(r):
                hs.append(mpi.allreduce(cuda(ins[r]), average=False))
        outs = session.run(hs)
    for r in range(n):
        G.assert_same_bits(G.host(outs[r]), want, "ragged %s rank %d" % (dtype.__name__, r))


# ---- one real rank, peers pre-staged: the measured per-rank path ---------------------------

def _prestaged(n, r, ins, rs, ag, flags, dtype):
    """mpic_ring_allreduce_prestaged for rank r; returns the output tensor."""
    L = _plugin.load_library()
    count = ins[r].size
    sizes, _ = ring_abi.segment_table(count, n)
    din = cuda(ins[r])
    dout = torch.zeros(count + 4, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda")[:count]
    keep = []
    rs_ptrs = (ctypes.c_void_p * max(n - 1, 1))()
    ag_ptrs = (ctypes.c_void_p * max(n - 1, 1))()
    for i in range(n - 1):
        rseg = ring_abi.schedule(ring_abi.PHASE_REDUCE_SCATTER, n, r, i)[1]
        aseg = ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i)[1]
        a = cuda(rs[r][i][:sizes[rseg]])
        b = cuda(ag[r][i][:sizes[aseg]])
        keep += [a, b]
        rs_ptrs[i] = a.data_ptr() if a.numel() else None
        ag_ptrs[i] = b.data_ptr() if b.numel() else None
    stream = torch.cuda.current_stream().cuda_stream
    rc = L.mpic_ring_allreduce_prestaged(n, r, DT[np.dtype(dtype)], din.data_ptr() if count else None,
                                         dout.data_ptr() if count else None, count, rs_ptrs, ag_ptrs, stream, flags)
    assert rc == 0, L.mpic_last_error()
    torch.cuda.synchronize()
    assert torch.equal(din, cuda(ins[r]))            # the input tensor is never written
    return dout


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_prestaged_rank_matches_oracle_small(oracle, dtype):
    for n, count in ((1, 9), (2, 7), (3, 3), (4, 2), (6, 4099), (8, 100_003), (5, 0)):
        ins = make_inputs(n, count, dtype, seed=n)
        outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
        for r in sorted({0, n // 2, n - 1}):
            for flags in (0, 1, 3):                  # per step; batched; batched + fused copy
                got = _prestaged(n, r, ins, rs, ag, flags, dtype)
                G.assert_same_bits(G.host(got), outs[r], "prestaged n=%d r=%d flags=%d" % (n, r, flags))


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_prestaged_ragged_integers_n6_full_size(oracle, dtype):
    """The ragged 10,000,019-element allreduce at N=6 through the per-rank
    step-table path the benchmark times (mpic_ring_allreduce_prestaged,
    batched, without and with the folded copy), peers' traffic from the
    oracle's ring."""
    n, count = 6, 10_000_019
    ins = [np.random.default_rng(r).integers(-1000, 1001, count).astype(dtype) for r in range(n)]
    outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
    assert np.array_equal(outs[0], sum(x.astype(np.int64) for x in ins).astype(dtype))
    for r in (0, 3, 5):
        for flags in (1, 3):
            got = _prestaged(n, r, ins, rs, ag, flags, dtype)
            G.assert_same_bits(G.host(got), outs[r], "prestaged ragged %s r=%d flags=%d" % (dtype.__name__, r, flags))


def _tf_div(x, n):
    with np.errstate(all="ignore"):
        return (x / np.float32(n) if x.dtype == np.float32 else x // x.dtype.type(n)).astype(x.dtype)


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_prestaged_rank_with_the_average_folded_in(oracle, dtype):
    """Divisor in the flags: the rank divides the segment it owns in its last
    accumulate and receives the other segments already divided (what its
    peers, doing the same, send): the output is tf.div(sum, divisor)."""
    for n, count, divisor in ((1, 9, 1), (1, 10, 3), (2, 7, 2), (3, 3, 3), (6, 4099, 6), (8, 100_003, 8), (4, 50, 7)):
        ins = make_inputs(n, count, dtype, seed=20 + n)
        outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
        sizes, _ = ring_abi.segment_table(count, n)
        ag_div = [[_tf_div(seg, divisor) for seg in per_rank] for per_rank in ag]
        for r in sorted({0, n // 2, n - 1}):
            for flags in (0, 1, 3):
                got = _prestaged(n, r, ins, rs, ag_div, flags | (divisor << 8), dtype)
                G.assert_same_bits(G.host(got), _tf_div(outs[r], divisor),
                                   "folded average n=%d r=%d flags=%d /%d" % (n, r, flags, divisor))


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_direct_form_for_one_rank_matches_the_ring(oracle, dtype):
    """mpic_ring_allreduce_direct_prestaged: the owner folds every rank's raw
    copy of its segment in ring order; the other segments arrive finished.
    Bit-identical to the oracle's ring, with and without the divide."""
    L = _plugin.load_library()
    for n, count, divisor in ((1, 9, 0), (2, 7, 0), (3, 2, 0), (6, 4099, 6), (8, 100_003, 0), (8, 50_000, 8), (5, 0, 0)):
        ins = make_inputs(n, count, dtype, seed=40 + n)
        want = oracle.ring_allreduce(ins)[0]
        if divisor:
            want = _tf_div(want, divisor)
        sizes, starts = ring_abi.segment_table(count, n)
        for r in sorted({0, n // 2, n - 1}):
            s = (r + 1) % n
            peers = [cuda(ins[(s + k) % n][starts[s]:starts[s] + sizes[s]]) for k in range(n - 1)]
            ag_segs = [ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i)[1] for i in range(n - 1)]
            ags = [cuda(want[starts[g]:starts[g] + sizes[g]]) for g in ag_segs]
            pp = (ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() if t.numel() else None for t in peers])
            ap = (ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() if t.numel() else None for t in ags])
            din = cuda(ins[r])
            for one_launch in (1, 0):
                dout = torch.zeros(count + 4, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda")[:count]
                rc = L.mpic_ring_allreduce_direct_prestaged(n, r, DT[np.dtype(dtype)], din.data_ptr() if count else None,
                                                            dout.data_ptr() if count else None, count, pp, ap,
                                                            torch.cuda.current_stream().cuda_stream,
                                                            one_launch | (divisor << 8))
                assert rc == 0, L.mpic_last_error()
                torch.cuda.synchronize()
                G.assert_same_bits(G.host(dout), want, "direct n=%d r=%d count=%d /%d one launch=%d"
                                   % (n, r, count, divisor, one_launch))


@pytest.mark.parametrize("n", [33, 64])
def test_direct_form_with_more_sources_than_one_launch_holds(oracle, n):
    """n*n source pointers exceed one fold launch's table: the rows are spread
    over several launches; float32 and int64 against the oracle."""
    L = _plugin.load_library()
    for dtype in (np.float32, np.int64):
        count = 10 * n + 7
        ins = make_inputs(n, count, dtype, seed=n)
        want = oracle.ring_allreduce_lockstep(ins)
        dins = [cuda(x) for x in ins]
        douts = [torch.zeros(count, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda") for _ in range(n)]
        ip = (ctypes.c_void_p * n)(*[t.data_ptr() for t in dins])
        op = (ctypes.c_void_p * n)(*[t.data_ptr() for t in douts])
        rc = L.mpic_ring_allreduce_all_ranks(n, DT[np.dtype(dtype)], ip, op, count,
                                             torch.cuda.current_stream().cuda_stream, 7)
        assert rc == 0, L.mpic_last_error()
        torch.cuda.synchronize()
        for r in range(n):
            G.assert_same_bits(G.host(douts[r]), want[r], "direct n=%d rank %d" % (n, r))


def test_average_costs_no_extra_launch():
    """allreduce(average=True) over resident ranks: as many kernel launches as
    the sum alone (the divide rides on the last reduce-scatter step)."""
    L = _plugin.load_library()
    n, count = 4, 10_000
    ins = [cuda(np.full(count, r + 1, dtype=np.float32)) for r in range(n)]
    outs = [torch.empty(count, device="cuda") for _ in range(n)]
    ip = (ctypes.c_void_p * n)(*[t.data_ptr() for t in ins])
    op = (ctypes.c_void_p * n)(*[t.data_ptr() for t in outs])
    stream = torch.cuda.current_stream().cuda_stream
    assert L.mpic_ring_allreduce_all_ranks(n, _plugin.DT_FLOAT, ip, op, count, stream, 1 | (n << 8)) == 0
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, torch.full((count,), 2.5, device="cuda"))     # (1+2+3+4)/4


def test_mismatched_divisors_are_refused():
    """Every rank must fuse the same division (FailedPrecondition otherwise)."""
    with mpi.Session(size=2) as session:
        hs = []
        for r in range(2):
            with session.as_rank(r):
                hs.append(mpi._allreduce(cuda(np.ones(8, dtype=np.float32)), name="x", divisor=2 if r else 0))
        with pytest.raises(mpi.FailedPreconditionError, match="Mismatched fused divisors"):
            session.run(hs)


def test_coordinator_fusion_with_average(oracle):
    """Averaged allreduces fused by the coordinator; sums and averages submitted
    together still form one group (each averaged tensor is divided after the
    unpack), a group of averages only has the divide ride on the unpack."""
    n = 3
    counts = [1000, 37, 5000, 64]
    per_rank = [[np.random.default_rng(10 * r + j).standard_normal(c).astype(np.float32) for j, c in enumerate(counts)]
                for r in range(n)]
    want = _expected_with_fusion(oracle, per_rank, [[0, 1, 2, 3]])
    for averaged in ((0, 1), (0, 1, 2, 3)):
        with mpi.Session(size=n, fusion_threshold=1 << 20) as session:
            hs = [[None] * 4 for _ in range(n)]
            for r in range(n):
                with session.as_rank(r):
                    for j in range(4):
                        hs[r][j] = mpi.allreduce(cuda(per_rank[r][j]), average=j in averaged)
            outs = session.run(hs)
        for r in range(n):
            for j in range(4):
                G.assert_same_bits(G.host(outs[r][j]), _tf_div(want[j], n) if j in averaged else want[j],
                                   "coordinator fusion + average %s: rank %d tensor %d" % (averaged, r, j))


def test_prestaged_64mib_float32_n8(oracle):
    """The headline shape: 16,777,216 float32, N=8, values N(0,1) from seed=rank,
    peers' segments staged from the oracle's full ring."""
    n, count = 8, 16_777_216
    ins = [np.random.default_rng(r).standard_normal(count, dtype=np.float32) for r in range(n)]
    outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
    assert np.array_equal(outs[0], outs[5])
    for r, flags in ((0, 1), (3, 3), (7, 0)):
        got = _prestaged(n, r, ins, rs, ag, flags, np.float32)
        G.assert_same_bits(G.host(got), outs[r], "64 MiB rank %d flags %d" % (r, flags))


def test_prestaged_through_the_op_layer(oracle):
    n, r, count = 4, 2, 70_001
    ins = make_inputs(n, count, np.float32, seed=9)
    outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
    sizes, _ = ring_abi.segment_table(count, n)
    for fuse in (0, 1):
        with mpi.Session(size=n, rank=r) as session:
            session.set_option("fuse_copy", fuse)
            assert mpi.rank() == r and mpi.size() == n
            rs_t = [cuda(rs[r][i][:sizes[ring_abi.schedule(0, n, r, i)[1]]]) for i in range(n - 1)]
            ag_t = [cuda(ag[r][i][:sizes[ring_abi.schedule(1, n, r, i)[1]]]) for i in range(n - 1)]
            session.stage_peers("MPIAllreduce", rs_t, ag_t)
            out = session.run(mpi.allreduce(cuda(ins[r]), average=False))
            G.assert_same_bits(G.host(out), outs[r], "op layer, prestaged, fuse=%d" % fuse)
            # nothing staged for the second call of that name
            with pytest.raises(mpi.FailedPreconditionError, match="No pre-staged peer segments"):
                session.run(mpi.allreduce(cuda(ins[r]), average=False))


def test_prestaged_1gib_float32_n64(oracle):
    """268,435,456 float32 (1 GiB), N=64: 63 + 63 steps on 16 MiB segments, one
    launch per phase. The reduce-scatter alone is checked against numpy on the
    host (every step is input + received on its own segment), the whole
    per-rank allreduce against the oracle's rank 37 run alone on the same
    incoming segments, and against what the schedule says of every segment."""
    n, r, count = 64, 37, 268_435_456
    seg = count // n
    gen = torch.Generator(device="cuda").manual_seed(r)
    din = torch.randn(count, device="cuda", generator=gen)
    rs = torch.randn(n - 1, seg, device="cuda", generator=gen)
    ag = torch.randn(n - 1, seg, device="cuda", generator=gen)
    dout = torch.empty(count, device="cuda")
    L = _plugin.load_library()
    rs_ptrs = (ctypes.c_void_p * (n - 1))(*[rs[i].data_ptr() for i in range(n - 1)])
    ag_ptrs = (ctypes.c_void_p * (n - 1))(*[ag[i].data_ptr() for i in range(n - 1)])
    stream = torch.cuda.current_stream().cuda_stream
    # reduce-scatter only first: n-1 rows through the step-table entry point
    ring_abi.copy_bytes(dout.data_ptr(), din.data_ptr(), count * 4, stream)
    rows = [(ring_abi.schedule(0, n, r, i)[1] * seg, rs[i].data_ptr(), seg) for i in range(n - 1)]
    steps, k = ring_abi.make_steps(rows)
    ring_abi.reduce_scatter_steps(dout.data_ptr(), steps, k, ring_abi.F32, stream)
    torch.cuda.synchronize()
    hin, hrs, hout = G.host(din), G.host(rs), G.host(dout)
    for i in range(n - 1):
        s = ring_abi.schedule(0, n, r, i)[1]
        G.assert_same_bits(hout[s * seg:(s + 1) * seg], hin[s * seg:(s + 1) * seg] + hrs[i], "RS step %d" % i)
    G.assert_same_bits(hout[r * seg:(r + 1) * seg], hin[r * seg:(r + 1) * seg], "own segment")
    # then the whole per-rank allreduce, batched and fused
    dout.zero_()
    rc = L.mpic_ring_allreduce_prestaged(n, r, _plugin.DT_FLOAT, din.data_ptr(), dout.data_ptr(), count,
                                         rs_ptrs, ag_ptrs, stream, 3)
    assert rc == 0, L.mpic_last_error()
    torch.cuda.synchronize()
    hout, hag = G.host(dout), G.host(ag)
    G.assert_same_bits(hout, oracle.ring_allreduce_rank_prestaged(n, r, hin, list(hrs), list(hag)),
                       "the oracle's rank %d alone on the same incoming segments" % r)
    owned = (r + 1) % n
    for i in range(n - 1):
        s = ring_abi.schedule(1, n, r, i)[1]
        G.assert_same_bits(hout[s * seg:(s + 1) * seg], hag[i], "AG step %d" % i)
    G.assert_same_bits(hout[owned * seg:(owned + 1) * seg],
                       hin[owned * seg:(owned + 1) * seg] + hrs[n - 2], "owned segment")


# ---- tensor fusion: the ResNet-50 gradient set at N=8 ------------------------------------------

def test_fused_resnet50_allreduce_matches_ring_on_the_packed_buffer(oracle):
    """161 float32 tensors ~N(0, 1e-3) packed into one buffer, ring-reduced at
    N=8, unpacked. Parity is with the reference ring applied to the packed 1-D
    buffer (fusion moves an element to another segment, hence another rotation
    of the sum, than 161 separate allreduces would)."""
    n = 8
    shapes = G.resnet50_shapes()
    counts = [int(np.prod(s)) for s in shapes]
    grads = [[(np.random.default_rng(1000 * r + j).standard_normal(c) * 1e-3).astype(np.float32)
              for j, c in enumerate(counts)] for r in range(n)]
    packed = [np.concatenate(g) for g in grads]
    want = oracle.ring_allreduce_lockstep(packed)[0]
    stream = torch.cuda.current_stream().cuda_stream
    dgrads = [[cuda(t) for t in g] for g in grads]
    plans = [ring_abi.FusionPlan([t.data_ptr() for t in g], counts, ring_abi.F32) for g in dgrads]
    fused_in = [torch.empty(sum(counts), device="cuda") for _ in range(n)]
    fused_out = [torch.empty(sum(counts), device="cuda") for _ in range(n)]
    for r in range(n):
        plans[r].pack(fused_in[r].data_ptr(), stream)
    L = _plugin.load_library()
    ins = (ctypes.c_void_p * n)(*[t.data_ptr() for t in fused_in])
    outs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in fused_out])
    rc = L.mpic_ring_allreduce_all_ranks(n, _plugin.DT_FLOAT, ins, outs, sum(counts), stream, 1)
    assert rc == 0, L.mpic_last_error()
    for r in range(n):
        plans[r].unpack(fused_out[r].data_ptr(), stream)
    torch.cuda.synchronize()
    for r in (0, 4, 7):
        at = 0
        for j, c in enumerate(counts):
            G.assert_same_bits(G.host(dgrads[r][j]), want[at:at + c], "fused rank %d tensor %d" % (r, j))
            at += c


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fused_allreduce_without_pack_and_unpack_passes(oracle, dtype):
    """mpic_ring_allreduce_fused_prestaged: the accumulates gather their local
    operand from the tensors, the finished segments scatter into them. Every
    tensor equals the oracle's ring on the packed buffer (then tf.div), and the
    wire buffer holds what the ring would send on."""
    L = _plugin.load_library()
    rng = np.random.default_rng(8)
    cases = [(8, [int(np.prod(s)) for s in G.resnet50_shapes()][:60], 8), (3, [5, 0, 4096, 1, 3, 8191, 2, 70_001], 0),
             (6, [int(c) for c in rng.integers(0, 50, 400)], 6), (1, [10, 20], 4), (4, [2], 0)]
    if dtype == np.float32:
        # the whole 161-tensor ResNet-50 set (25,557,032 elements) at N=8: the size the benchmark times
        cases.append((8, [int(np.prod(s)) for s in G.resnet50_shapes()], 8))
    for n, counts, divisor in cases:
        total = sum(counts)
        grads = [[G.random_array(np.random.default_rng(100 * r + j), c, dtype) for j, c in enumerate(counts)]
                 for r in range(n)]
        packed = [np.concatenate(g) for g in grads]
        outs, rs, ag = oracle.ring_allreduce(packed, tap=True)
        want = _tf_div(outs[0], divisor) if divisor else outs[0]
        sizes, starts = ring_abi.segment_table(total, n)
        for r in sorted({0, n // 2, n - 1}):
            dts = [G.dev(t, (j + r) % 4) for j, t in enumerate(grads[r])]
            plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(dts, counts)], counts,
                                       G.NP2ABI[np.dtype(dtype)])
            wire = torch.zeros(total + 4, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda")[1:total + 1]   # element-aligned only
            rs_seg = [ring_abi.schedule(ring_abi.PHASE_REDUCE_SCATTER, n, r, i)[1] for i in range(n - 1)]
            ag_seg = [ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i)[1] for i in range(n - 1)]
            rs_t = [cuda(rs[r][i][:sizes[g]]) for i, g in enumerate(rs_seg)]
            ag_t = [cuda(ag[r][i][:sizes[g]]) for i, g in enumerate(ag_seg)]
            rs_p = (ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() if t.numel() else None for t in rs_t])
            ag_p = (ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() if t.numel() else None for t in ag_t])
            rc = L.mpic_ring_allreduce_fused_prestaged(plan._h, n, r, wire.data_ptr(), rs_p, ag_p,
                                                       torch.cuda.current_stream().cuda_stream, divisor << 8)
            assert rc == 0, L.mpic_last_error()
            torch.cuda.synchronize()
            at = 0
            for j, c in enumerate(counts):
                G.assert_same_bits(G.host(dts[j][0]), want[at:at + c], "n=%d rank %d tensor %d /%d" % (n, r, j, divisor))
                at += c
            got_wire = G.host(wire)
            for i, g in enumerate(rs_seg):                      # partial sums, as sent on at the next step
                a, b = starts[g], starts[g] + sizes[g]
                with np.errstate(all="ignore"):
                    G.assert_same_bits(got_wire[a:b], (packed[r][a:b] + rs[r][i][:sizes[g]]).astype(dtype),
                                       "wire segment %d" % g)
            a, b = starts[r], starts[r] + sizes[r]
            G.assert_same_bits(got_wire[a:b], packed[r][a:b], "wire segment r (packed only)")
            # the direct form: raw copies of the owned segment from every peer, folded in ring order
            if n > 1:
                for t, g in zip(dts, grads[r]):
                    t[0].copy_(torch.from_numpy(g))
                own = (r + 1) % n
                raw_t = [cuda(packed[(own + k) % n][starts[own]:starts[own] + sizes[own]]) for k in range(n - 1)]
                fin_t = [cuda(outs[0][starts[g]:starts[g] + sizes[g]]) for g in ag_seg]
                raw_p = (ctypes.c_void_p * (n - 1))(*[t.data_ptr() if t.numel() else None for t in raw_t])
                fin_p = (ctypes.c_void_p * (n - 1))(*[t.data_ptr() if t.numel() else None for t in fin_t])
                rc = L.mpic_ring_allreduce_fused_prestaged(plan._h, n, r, wire.data_ptr(), raw_p, fin_p,
                                                           torch.cuda.current_stream().cuda_stream, 4 | (divisor << 8))
                assert rc == 0, L.mpic_last_error()
                torch.cuda.synchronize()
                at = 0
                for j, c in enumerate(counts):
                    G.assert_same_bits(G.host(dts[j][0]), want[at:at + c],
                                       "direct fused n=%d rank %d tensor %d /%d" % (n, r, j, divisor))
                    at += c
                # the owned segment of the wire buffer: the sum itself, as the rank sends it on
                a, b = starts[own], starts[own] + sizes[own]
                G.assert_same_bits(G.host(wire)[a:b], outs[0][a:b], "direct fused wire n=%d rank %d" % (n, r))
            plan.close()


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_direct_fused_form_split_at_the_exchange(oracle, dtype):
    """With a real exchange the direct form is two launches: the fold of the
    owned segment (ring_fusion_fold_scatter with no finished spans), whose sum
    the rank then sends, and, once the peers' finished segments have arrived,
    their scatter. Same tensors and the same wire segment as the one launch;
    also the argument checks of the entry point."""
    stream = torch.cuda.current_stream().cuda_stream
    abi = G.NP2ABI[np.dtype(dtype)]
    for n, counts, divisor in [(5, [3, 0, 9000, 17, 4096, 1, 5000], 5), (2, [70_001], 0), (33, [40] * 50, 3), (34, [40] * 50, 0)]:
        total = sum(counts)
        grads = [[G.random_array(np.random.default_rng(31 * r + j), c, dtype) for j, c in enumerate(counts)]
                 for r in range(n)]
        packed = [np.concatenate(g) for g in grads]
        summed = oracle.ring_allreduce(packed)[0]
        want = _tf_div(summed, divisor) if divisor else summed
        sizes, starts = ring_abi.segment_table(total, n)
        r = n - 2
        own = (r + 1) % n
        dts = [G.dev(t, (j + 1) % 4) for j, t in enumerate(grads[r])]
        plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(dts, counts)], counts, abi)
        wire = torch.zeros(sizes[own] + 2, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda")[1:sizes[own] + 1]
        raw = [cuda(packed[(own + k) % n][starts[own]:starts[own] + sizes[own]]) for k in range(n - 1)]
        fin = {g: cuda(summed[starts[g]:starts[g] + sizes[g]]) for g in range(n) if g != own}
        others = [(starts[g], sizes[g], fin[g].data_ptr(), None) for g in range(n) if g != own]
        if n - 1 > 32:
            with pytest.raises(ring_abi.RingError) as e:
                plan.fold_scatter(starts[own], sizes[own], [t.data_ptr() for t in raw], wire.data_ptr(),
                                  ring_abi.make_spans([]), divisor, stream)
            assert e.value.status == 5            # beyond the capacity of one launch
            plan.close()
            continue
        plan.fold_scatter(starts[own], sizes[own], [t.data_ptr() for t in raw], wire.data_ptr(),
                          ring_abi.make_spans([]), divisor, stream)
        torch.cuda.synchronize()
        G.assert_same_bits(G.host(wire), summed[starts[own]:starts[own] + sizes[own]], "wire after the fold")
        flat = np.concatenate([G.host(d[0]) for d in dts]) if total else np.zeros(0, dtype)
        a, b = starts[own], starts[own] + sizes[own]
        G.assert_same_bits(flat[a:b], want[a:b], "owned segment in the tensors")
        G.assert_same_bits(np.concatenate([flat[:a], flat[b:]]), np.concatenate([packed[r][:a], packed[r][b:]]),
                           "the other segments untouched by the fold")
        plan.scatter(ring_abi.make_spans(others), divisor, stream)
        torch.cuda.synchronize()
        G.assert_same_bits(np.concatenate([G.host(d[0]) for d in dts]), want, "tensors after the scatter")
        # a finished span that meets the fold span, a span beyond the plan, a null staged copy
        for bad in ([(starts[own], 1, fin[(own + 1) % n].data_ptr(), None)], [(total, 1, fin[(own + 1) % n].data_ptr(), None)]):
            with pytest.raises(ring_abi.RingError):
                plan.fold_scatter(starts[own], sizes[own], [t.data_ptr() for t in raw], wire.data_ptr(),
                                  ring_abi.make_spans(bad), divisor, stream)
        with pytest.raises(ring_abi.RingError):
            plan.fold_scatter(starts[own], sizes[own], [None] * (n - 1), wire.data_ptr(), ring_abi.make_spans([]),
                              divisor, stream)
        plan.close()


def test_distributed_optimizer_fused_and_unfused(oracle):
    """DistributedOptimizer.compute_gradients averages every gradient across
    ranks (__init__.py:195-205); with fusion=True through one fused buffer."""
    n = 3
    torch.manual_seed(0)
    base = torch.nn.Sequential(torch.nn.Linear(37, 19), torch.nn.Tanh(), torch.nn.Linear(19, 5)).cuda()
    for fusion in (False, True):
        replicas, opts, xs = [], [], []
        for r in range(n):
            m = torch.nn.Sequential(torch.nn.Linear(37, 19), torch.nn.Tanh(), torch.nn.Linear(19, 5)).cuda()
            m.load_state_dict(base.state_dict())
            replicas.append(m)
            opts.append(mpi.DistributedOptimizer(torch.optim.SGD(m.parameters(), lr=0.1), fusion=fusion))
            xs.append(torch.randn(11, 37, generator=torch.Generator().manual_seed(r)).cuda())
        local = []
        with mpi.Session(size=n) as session:
            gvs = []
            for r in range(n):
                with session.as_rank(r):
                    loss = replicas[r](xs[r]).square().mean()
                    loss.backward()
                    local.append([G.host(p.grad).reshape(-1).copy() for p in replicas[r].parameters()])
                    gvs.append(opts[r].compute_gradients())
            session.run()
            for r in range(n):
                with session.as_rank(r):
                    opts[r].apply_gradients(gvs[r])
        nparam = len(local[0])
        if fusion:
            summed = oracle.ring_allreduce([np.concatenate(local[r]) for r in range(n)])[0] / np.float32(n)
            want, at = [], 0
            for j in range(nparam):
                want.append(summed[at:at + local[0][j].size])
                at += local[0][j].size
        else:
            want = [oracle.ring_allreduce([local[r][j] for r in range(n)])[0] / np.float32(n) for j in range(nparam)]
        for r in range(n):
            for j, p in enumerate(replicas[r].parameters()):
                G.assert_same_bits(G.host(p.grad).reshape(-1), want[j], "fusion=%s rank %d param %d" % (fusion, r, j))
        # every replica took the same step
        for p0, p1 in zip(replicas[0].parameters(), replicas[n - 1].parameters()):
            assert torch.equal(p0, p1)
        assert not torch.equal(next(replicas[0].parameters()), next(base.parameters()))


def test_chained_allreduces_closed_form():
    """mpi_allreduce_test.py:40-112 at 2 ranks, one iteration: 13 dependent
    allreduces of a 1331x1331 matrix (odd element count, ragged segments)."""
    n, stages, side, spread = 2, 13, 1331, 100
    for average in (False, True):
        with mpi.Session(size=n) as session:
            state = [torch.full((side, side), 1.0 + r * spread, device="cuda") for r in range(n)]
            for i in range(stages):
                hs = []
                for r in range(n):
                    with session.as_rank(r):
                        hs.append(mpi.allreduce(state[r] + 2.0 ** (i + 1), average=average))
                state = session.run(hs)
        ours = 1.0
        for i in range(stages):
            cur = ours + 2.0 ** (i + 1)
            if average:
                ours = cur + (spread * (n - 1) / 2 if i == 0 else 0)
            else:
                ours = cur * n + (spread * n * (n - 1) / 2 if i == 0 else 0)
        for s in state:
            assert np.allclose(G.host(s), np.float32(ours))


def _expected_with_fusion(oracle, per_rank, groups):
    """Per-tensor results when the tensors of each group are reduced as one
    packed buffer (a group of one is a plain ring)."""
    n = len(per_rank)
    out = [None] * len(per_rank[0])
    for g in groups:
        packed = [np.concatenate([per_rank[r][j] for j in g]) for r in range(n)]
        red = oracle.ring_allreduce(packed)[0]
        at = 0
        for j in g:
            c = per_rank[0][j].size
            out[j] = red[at:at + c]
            at += c
    return out


@pytest.mark.parametrize("threshold,groups", [
    (8 << 20, [[0, 1, 2, 3, 4, 5, 6]]),                    # everything fits: one ring
    (20_000, [[0, 1, 2, 3], [4], [5, 6]]),                 # tensor 4 alone exceeds the buffer
])
def test_coordinator_fusion_matches_ring_on_packed_buffer(oracle, threshold, groups):
    """Allreduces submitted between two runs are fused by the coordinator, in
    submission order, up to the threshold; each tensor equals the reference
    ring applied to the packed buffer of its group."""
    n = 4
    counts = [5, 4099, 64, 0, 100_003, 17, 2048]
    per_rank = [[(np.random.default_rng(100 * r + j).standard_normal(c) * 10.0 ** (j - 3)).astype(np.float32)
                 for j, c in enumerate(counts)] for r in range(n)]
    want = _expected_with_fusion(oracle, per_rank, groups)
    with mpi.Session(size=n, fusion_threshold=threshold) as session:
        hs = [[None] * len(counts) for _ in range(n)]
        for r in range(n):
            with session.as_rank(r):
                for j in range(len(counts)):
                    hs[r][j] = mpi.allreduce(cuda(per_rank[r][j]), average=False)
        outs = session.run(hs)
    for r in range(n):
        for j in range(len(counts)):
            G.assert_same_bits(G.host(outs[r][j]), want[j], "fused by coordinator: rank %d tensor %d" % (r, j))


def test_coordinator_fusion_groups_by_dtype_and_keeps_other_ops_apart(oracle):
    n = 3
    f = [[np.random.default_rng(r * 10 + j).standard_normal(1000 + j).astype(np.float32) for j in range(4)]
         for r in range(n)]
    i32 = [np.random.default_rng(50 + r).integers(-1000, 1001, 777).astype(np.int32) for r in range(n)]
    rows = [2, 5, 1]
    g = [np.random.default_rng(70 + r).standard_normal((rows[r], 3)).astype(np.float32) for r in range(n)]
    with mpi.Session(size=n, fusion_threshold=1 << 20) as session:
        hs = []
        for r in range(n):
            with session.as_rank(r):
                hs.append([mpi.allreduce(cuda(f[r][0]), average=False), mpi.allreduce(cuda(f[r][1])),
                           mpi.allreduce(cuda(i32[r]), average=False), mpi.allgather(cuda(g[r])),
                           mpi.allreduce(cuda(f[r][2]), average=False), mpi.allreduce(cuda(f[r][3]), average=False)])
        outs = session.run(hs)
    first = _expected_with_fusion(oracle, [[f[r][0], f[r][1]] for r in range(n)], [[0, 1]])
    # the int32 allreduce and the allgather's sizing pass are ready between the two
    # float32 pairs, so each pair is its own group
    second = _expected_with_fusion(oracle, [[f[r][2], f[r][3]] for r in range(n)], [[0, 1]])
    ints = oracle.ring_allreduce(i32)[0]
    for r in range(n):
        G.assert_same_bits(G.host(outs[r][0]), first[0], "pair 1 a")
        G.assert_same_bits(G.host(outs[r][1]), first[1] / np.float32(n), "pair 1 b (averaged)")
        G.assert_same_bits(G.host(outs[r][2]), ints, "int32 between the groups")
        G.assert_same_bits(G.host(outs[r][3]), np.concatenate(g), "allgather between the groups")
        G.assert_same_bits(G.host(outs[r][4]), second[0], "pair 2 a")
        G.assert_same_bits(G.host(outs[r][5]), second[1], "pair 2 b")


def test_distributed_optimizer_over_coordinator_fusion(oracle):
    """The reference's DistributedOptimizer issues one allreduce per gradient
    (__init__.py:195-205); with a fusion threshold the coordinator reduces them
    all with one ring."""
    n = 3
    torch.manual_seed(1)
    base = torch.nn.Sequential(torch.nn.Linear(23, 31), torch.nn.ReLU(), torch.nn.Linear(31, 7)).cuda()
    replicas, opts, local = [], [], []
    with mpi.Session(size=n, fusion_threshold=1 << 20) as session:
        gvs = []
        for r in range(n):
            m = torch.nn.Sequential(torch.nn.Linear(23, 31), torch.nn.ReLU(), torch.nn.Linear(31, 7)).cuda()
            m.load_state_dict(base.state_dict())
            replicas.append(m)
            opts.append(mpi.DistributedOptimizer(torch.optim.SGD(m.parameters(), lr=0.05)))
            x = torch.randn(9, 23, generator=torch.Generator().manual_seed(40 + r)).cuda()
            with session.as_rank(r):
                m(x).square().mean().backward()
                local.append([G.host(p.grad).reshape(-1).copy() for p in m.parameters()])
                gvs.append(opts[r].compute_gradients())
        session.run()
        for r in range(n):
            with session.as_rank(r):
                opts[r].apply_gradients(gvs[r])
    k = len(local[0])
    want = _expected_with_fusion(oracle, local, [list(range(k))])
    for r in range(n):
        for j, p in enumerate(replicas[r].parameters()):
            G.assert_same_bits(G.host(p.grad).reshape(-1), want[j] / np.float32(n), "rank %d gradient %d" % (r, j))


def test_per_rank_path_replays_from_a_hip_graph(oracle):
    """The entry points only launch kernels (no allocation, no memset), so a
    caller can capture a rank's whole data path in a HIP graph. Every replay,
    with eager work and synchronisations in between, must reproduce the eager
    result."""
    n, r, count = 4, 1, 300_007
    ins = make_inputs(n, count, np.float32, seed=21)
    outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
    sizes, _ = ring_abi.segment_table(count, n)
    L = _plugin.load_library()
    din = cuda(ins[r])
    dout = torch.zeros(count, device="cuda")
    rs_t = [cuda(rs[r][i][:sizes[ring_abi.schedule(0, n, r, i)[1]]]) for i in range(n - 1)]
    ag_t = [cuda(ag[r][i][:sizes[ring_abi.schedule(1, n, r, i)[1]]]) for i in range(n - 1)]
    rs_p = (ctypes.c_void_p * (n - 1))(*[t.data_ptr() for t in rs_t])
    ag_p = (ctypes.c_void_p * (n - 1))(*[t.data_ptr() for t in ag_t])
    for flags in (1, 3):
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                rc = L.mpic_ring_allreduce_prestaged(n, r, _plugin.DT_FLOAT, din.data_ptr(), dout.data_ptr(), count,
                                                     rs_p, ag_p, torch.cuda.current_stream().cuda_stream, flags)
                assert rc == 0, L.mpic_last_error()
        torch.cuda.current_stream().wait_stream(side)
        for replay in range(4):
            dout.zero_()                              # eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            G.assert_same_bits(G.host(dout), outs[r], "graph replay %d flags %d" % (replay, flags))


def test_ranks_driven_from_separate_threads(oracle):
    """One thread per rank, as one MPI process per rank would run: every thread
    submits its collectives and blocks on its own results; the readiness table
    and the background thread see truly concurrent arrivals."""
    import threading
    n = 6
    ins = make_inputs(n, 123_457, np.float32, seed=77)
    ints = make_inputs(n, 1001, np.int64, seed=78)
    rows = [3, 1, 4, 1, 5, 9]
    parts = [np.random.default_rng(90 + r).standard_normal((rows[r], 7)).astype(np.float32) for r in range(n)]
    want_sum = oracle.ring_allreduce(ins)[0]
    want_int = oracle.ring_allreduce(ints)[0] // n
    want_cat = np.concatenate(parts)
    results, errors = [None] * n, []
    with mpi.Session(size=n) as session:
        def worker(r):
            try:
                with session.as_rank(r):
                    out = []
                    for rep in range(3):                       # the same ops again: node names must keep matching
                        a = mpi.allreduce(cuda(ins[r]), average=False).wait()
                        b = mpi.allreduce(cuda(ints[r])).wait()            # average: floor division
                        c = mpi.allgather(cuda(parts[r])).wait()
                        out.append((G.host(a), G.host(b), G.host(c)))
                    results[r] = out
            except Exception as e:                             # surfaced below, in the main thread
                errors.append((r, e))
        threads = [threading.Thread(target=worker, args=(r,)) for r in range(n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=60)
        assert not any(t.is_alive() for t in threads), "a rank is still waiting for its collective"
    assert not errors, errors
    for r in range(n):
        for a, b, c in results[r]:
            G.assert_same_bits(a, want_sum, "threaded allreduce rank %d" % r)
            G.assert_same_bits(b, want_int, "threaded averaged int64 rank %d" % r)
            G.assert_same_bits(c, want_cat, "threaded allgather rank %d" % r)


@pytest.mark.parametrize("fusion", [False, True])
def test_training_example_runs_and_learns(fusion, monkeypatch):
    """The data-parallel example: replicas stay bit-identical and the loss falls."""
    import importlib.util
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "tensorflow-allreduce_amd", "examples", "train_virtual_ranks.py")
    spec = importlib.util.spec_from_file_location("train_virtual_ranks", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    monkeypatch.setattr("sys.argv", ["train_virtual_ranks.py", "--ranks", "3", "--steps", "2"] + (["--fusion"] if fusion else []))
    first = mod.main()
    monkeypatch.setattr("sys.argv", ["train_virtual_ranks.py", "--ranks", "3", "--steps", "30"] + (["--fusion"] if fusion else []))
    last = mod.main()
    assert last < first


def test_reference_cpu_case_two_ranks_one_mebi_elements():
    """The reference's own CPU-runnable case: MPIAllreduce (sum) of one float32
    tensor of 1,048,576 elements at 2 ranks, values uniform[-1,1] from
    seed=1234+rank. With two ranks the sum is a single commutative add."""
    xs = [np.random.default_rng(1234 + r).uniform(-1, 1, 1_048_576).astype(np.float32) for r in range(2)]
    with mpi.Session(size=2) as session:
        hs = []
        for r in range(2):
            with session.as_rank(r):
                hs.append(mpi.allreduce(cuda(xs[r]), average=False))
        outs = session.run(hs)
    for o in outs:
        G.assert_same_bits(G.host(o), xs[0] + xs[1], "two-rank allreduce")


def test_non_contiguous_and_multi_dimensional_tensors(oracle):
    n = 3
    base = [np.random.default_rng(r).standard_normal((40, 50)).astype(np.float32) for r in range(n)]
    want = oracle.ring_allreduce([np.ascontiguousarray(b.T) for b in base])[0].reshape(50, 40)
    gathered = np.concatenate([np.ascontiguousarray(b.T) for b in base])
    with mpi.Session(size=n) as session:
        hs, gs = [], []
        for r in range(n):
            with session.as_rank(r):
                t = cuda(base[r]).t()                       # a transposed view: not contiguous
                assert not t.is_contiguous()
                hs.append(mpi.allreduce(t, average=False))
                gs.append(mpi.allgather(t))
        outs, cats = session.run([hs, gs])
    for o, c in zip(outs, cats):
        assert list(o.shape) == [50, 40] and list(c.shape) == [150, 40]
        G.assert_same_bits(G.host(o), want, "transposed input")
        G.assert_same_bits(G.host(c), gathered, "transposed gather")


@pytest.mark.parametrize("direct", [0, 1])
def test_committed_known_answer_vectors_on_the_gpu(direct):
    """tests/golden/ring_kats.json (order-sensitive inputs, expected values from
    a pure-Python mailbox simulation of the reference schedule) through the op
    layer, as the lockstep ring and in the direct form: every rank's output
    equals the committed answer bit for bit."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ring_kats.json")) as f:
        kats = json.load(f)["cases"]
    assert len(kats) >= 27
    for case in kats:
        if case["dtype"] == "f32":
            ins = [np.array(x, dtype=np.uint32).view(np.float32) for x in case["inputs"]]
            want = np.array(case["expected"], dtype=np.uint32).view(np.float32)
        else:
            dt = np.int32 if case["dtype"] == "i32" else np.int64
            ins = [np.array(x, dtype=dt) for x in case["inputs"]]
            want = np.array(case["expected"], dtype=dt)
        n = case["n"]
        with mpi.Session(size=n) as session:
            session.set_option("direct", direct)
            hs = []
            for r in range(n):
                with session.as_rank(r):
                    hs.append(mpi.allreduce(cuda(ins[r]), average=False))
            outs = session.run(hs)
        for r in range(n):
            G.assert_same_bits(G.host(outs[r]), want,
                               "KAT %s n=%d count=%d rank %d direct=%d" % (case["dtype"], n, case["count"], r, direct))


def test_inputs_still_being_produced_on_another_stream(oracle):
    """The producer hands its tensor to the ring without the host waiting: the
    inputs are written by a long chain of kernels on a side stream and the
    allreduce is submitted while that chain is still running; the world's
    stream waits for the producer on the device (ring_stream_wait_event), so
    the ring reads the finished values."""
    n, count, rounds = 4, 8 * 1024 * 1024, 60
    base = make_inputs(n, count, np.float32, seed=5, wide=False)
    side = torch.cuda.Stream()
    dins = [cuda(x) for x in base]
    ballast = torch.zeros(256 * 1024 * 1024, dtype=torch.float32, device="cuda")     # 1 GiB per pass
    torch.cuda.synchronize()
    with mpi.Session(size=n) as session:
        handles = []
        with torch.cuda.stream(side):
            # several milliseconds of work ahead of the producers on the same stream, so that
            # they are certainly still queued when the host reaches the submissions
            for _ in range(24):
                ballast.add_(1.0)
            for r in range(n):
                for _ in range(rounds):
                    dins[r].add_(1.0)                 # ~60 kernels per rank queued on the side stream
                with session.as_rank(r):
                    handles.append(mpi.allreduce(dins[r], average=False))
            still_running = not side.query()
        outs = session.run(handles)
    torch.cuda.synchronize()
    produced = [G.host(t) for t in dins]
    for r in range(n):          # what the producers finally wrote, rounded as the GPU rounded it
        acc = base[r].copy()
        for _ in range(rounds):
            acc = (acc + np.float32(1.0)).astype(np.float32)
        G.assert_same_bits(produced[r], acc, "producer chain rank %d" % r)
    want = oracle.ring_allreduce(produced)
    for r in range(n):
        G.assert_same_bits(G.host(outs[r]), want[r], "allreduce of inputs produced on a side stream, rank %d" % r)
    assert still_running, "the producers had already finished at submission: the test did not exercise the hand-off"


def test_more_ranks_than_the_direct_form_addresses(oracle):
    """A session of 257 virtual ranks with its default options: the direct form
    folds at most 256 copies of a segment, so the allreduce runs as the
    lockstep ring, which takes any number of ranks, with the same result."""
    n, count = 257, 1000
    ins = make_inputs(n, count, np.float32, seed=9, wide=False)
    want = oracle.ring_allreduce_lockstep(ins)[0]
    with mpi.Session(size=n) as session:
        handles = []
        for r in range(n):
            with session.as_rank(r):
                handles.append(mpi.allreduce(cuda(ins[r]), average=False))
        outs = session.run(handles)
    for r in (0, 1, 128, 256):
        G.assert_same_bits(G.host(outs[r]), want, "257 ranks, rank %d" % r)


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_recorded_steps_replay_with_the_eager_results(oracle, dtype):
    """Several per-rank steps recorded as one HIP graph through the C ABI
    (ring_graph_begin_capture ... ring_graph_end_capture) and replayed. Every
    replay, with the program's own eager work and synchronisations between
    them and new values in the same buffers, gives the oracle's result bit for
    bit on every recorded step."""
    L, R = _plugin.load_library(), ring_abi.lib()
    cases = ((8, 262_144, 1), (6, 100_003, 3), (3, 17, 3), (1, 9, 1))
    tdt = G.NP2TORCH[np.dtype(dtype)]
    bufs = []
    for n, count, flags in cases:
        sizes, _ = ring_abi.segment_table(count, n)
        r = n // 2
        rs_seg = [ring_abi.schedule(ring_abi.PHASE_REDUCE_SCATTER, n, r, i)[1] for i in range(n - 1)]
        ag_seg = [ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i)[1] for i in range(n - 1)]
        rs_t = [torch.zeros(sizes[g], dtype=tdt, device="cuda") for g in rs_seg]
        ag_t = [torch.zeros(sizes[g], dtype=tdt, device="cuda") for g in ag_seg]
        bufs.append(dict(n=n, r=r, count=count, flags=flags, sizes=sizes, rs_seg=rs_seg, ag_seg=ag_seg, rs_t=rs_t, ag_t=ag_t,
                         din=torch.zeros(count, dtype=tdt, device="cuda"), dout=torch.zeros(count, dtype=tdt, device="cuda"),
                         rs_p=(ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() if t.numel() else None for t in rs_t]),
                         ag_p=(ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() if t.numel() else None for t in ag_t])))
    stream = ring_abi.stream_create()
    graph = ctypes.c_void_p()
    try:
        torch.cuda.synchronize()
        ring_abi.check(R.ring_graph_begin_capture(stream), "begin capture")
        for b in bufs:
            rc = L.mpic_ring_allreduce_prestaged(b["n"], b["r"], DT[np.dtype(dtype)], b["din"].data_ptr(), b["dout"].data_ptr(),
                                                 b["count"], b["rs_p"], b["ag_p"], stream, b["flags"])
            assert rc == 0, L.mpic_last_error()
        ring_abi.check(R.ring_graph_end_capture(stream, ctypes.byref(graph)), "end capture")
        for replay in range(4):
            wants = []
            for b in bufs:      # eager work of the program itself between the replays
                ins = make_inputs(b["n"], b["count"], dtype, seed=40 * replay + b["n"])
                outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
                b["din"].copy_(torch.from_numpy(ins[b["r"]]))
                for i in range(b["n"] - 1):
                    b["rs_t"][i].copy_(torch.from_numpy(np.ascontiguousarray(rs[b["r"]][i][:b["sizes"][b["rs_seg"][i]]])))
                    b["ag_t"][i].copy_(torch.from_numpy(np.ascontiguousarray(ag[b["r"]][i][:b["sizes"][b["ag_seg"][i]]])))
                b["dout"].zero_()
                wants.append((outs[b["r"]], ins[b["r"]]))
            torch.cuda.synchronize()
            ring_abi.check(R.ring_graph_launch(graph, stream), "graph launch")
            ring_abi.stream_synchronize(stream)
            for b, (want, inp) in zip(bufs, wants):
                G.assert_same_bits(G.host(b["dout"]), want, "recorded step n=%d replay %d" % (b["n"], replay))
                G.assert_same_bits(G.host(b["din"]), inp, "the input is never written")
    finally:
        if graph.value:
            ring_abi.check(R.ring_graph_destroy(graph), "graph destroy")
        ring_abi.stream_destroy(stream)
    assert R.ring_graph_begin_capture(None) == 2        # the null stream cannot be recorded


def test_allreduce_batch_is_one_node_per_tensor(oracle):
    """mpi.allreduce_batch: every tensor is its own MPIAllreduce node (same
    results as a loop over mpi.allreduce, bit for bit, sum and average, mixed
    element types and shapes, an empty tensor among them), and a tensor whose
    shape differs between ranks fails alone, with the reference's message,
    while the others of the batch complete."""
    n = 4
    shapes = [(1000, 3), (0,), (70_001,), (5,), (128, 64)]
    dtypes = [np.float32, np.float32, np.int32, np.int64, np.float32]
    ins = [[G.random_array(np.random.default_rng(10 * r + j), int(np.prod(s)), dt).reshape(s)
            for j, (s, dt) in enumerate(zip(shapes, dtypes))] for r in range(n)]
    for average in (False, True):
        with mpi.Session(size=n) as session:
            handles = []
            for r in range(n):
                with session.as_rank(r):
                    handles.append(mpi.allreduce_batch([cuda(x) for x in ins[r]], average=average))
            outs = session.run(handles)
        for j in range(len(shapes)):
            want = oracle.ring_allreduce([ins[r][j].reshape(-1) for r in range(n)])
            for r in range(n):
                w = _tf_div(want[r], n) if average else want[r]
                assert tuple(outs[r][j].shape) == shapes[j]
                G.assert_same_bits(G.host(outs[r][j]).reshape(-1), w, "batch tensor %d rank %d average=%s" % (j, r, average))
    # one tensor's shape differs on one rank: that node fails on every rank, the rest complete
    with mpi.Session(size=n) as session:
        handles = []
        for r in range(n):
            with session.as_rank(r):
                xs = [cuda(ins[r][0]), cuda(ins[r][3] if r != 2 else np.zeros(6, np.int64)), cuda(ins[r][4])]
                handles.append(mpi.allreduce_batch(xs, average=False))
        with pytest.raises(mpi.FailedPreconditionError) as e:
            session.run()
        assert "Mismatched allreduce tensor shapes" in str(e.value)
        for r in range(n):
            G.assert_same_bits(G.host(handles[r][0].result()).reshape(-1),
                               oracle.ring_allreduce([ins[q][0].reshape(-1) for q in range(n)])[r], "first of the batch")
            with pytest.raises(mpi.FailedPreconditionError):
                handles[r][1].result()
            # the one behind the bad node was enqueued in the same tick and completes like the first
            G.assert_same_bits(G.host(handles[r][2].result()).reshape(-1),
                               oracle.ring_allreduce([ins[q][4].reshape(-1) for q in range(n)])[r], "last of the batch")


def test_prepared_batch_runs_the_same_nodes_every_step(oracle):
    """mpi.prepare_allreduce_batch: a rank's MPIAllreduce nodes built once (the
    reference builds its graph once) and run on new values every step, in memory
    of their own or in place; each step's results equal a loop over
    mpi.allreduce, bit for bit, with and without the coordinator's fusion."""
    n, steps = 4, 3
    shapes = [(1000, 3), (0,), (70_001,), (5,), (128, 64)]
    dtypes = [np.float32, np.float32, np.int32, np.int64, np.float32]

    def values(step, r):
        return [G.random_array(np.random.default_rng(1000 * step + 10 * r + j), int(np.prod(s)), dt).reshape(s)
                for j, (s, dt) in enumerate(zip(shapes, dtypes))]

    for inplace, fusion in ((False, 0), (True, 0), (False, 1 << 22), (True, 1 << 22)):
        with mpi.Session(size=n, fusion_threshold=fusion) as session:
            tensors = [[cuda(x) for x in values(0, r)] for r in range(n)]
            batches = []
            for r in range(n):
                with session.as_rank(r):
                    batches.append(mpi.prepare_allreduce_batch(tensors[r], average=True, inplace=inplace))
            assert batches[0].node_names == batches[n - 1].node_names
            for step in range(steps):
                ins = [values(step, r) for r in range(n)]
                for r in range(n):
                    for t, x in zip(tensors[r], ins[r]):
                        t.copy_(torch.from_numpy(x))
                handles = [b.submit() for b in batches]
                with pytest.raises(mpi.FailedPreconditionError):
                    batches[0].submit()                     # still pending
                outs = session.run(handles)
                for j in range(len(shapes)):
                    if fusion and dtypes[j] == np.float32:
                        continue        # fused float32 sums round as the ring over the packed buffer does (checked below)
                    want = oracle.ring_allreduce([ins[r][j].reshape(-1) for r in range(n)])
                    for r in range(n):
                        got = G.host(outs[r][j])
                        assert tuple(got.shape) == shapes[j]
                        G.assert_same_bits(got.reshape(-1), _tf_div(want[r], n),
                                           "step %d tensor %d rank %d inplace=%s fusion=%d" % (step, j, r, inplace, fusion))
                        if inplace:
                            assert outs[r][j].data_ptr() == tensors[r][j].data_ptr()
                if fusion:
                    f32 = [j for j in range(len(shapes)) if dtypes[j] == np.float32]
                    # consecutive ready allreduces of one type fuse: tensors 0 and 1; tensor 4 comes after the integers
                    want = _expected_with_fusion(oracle, [[ins[r][j].reshape(-1) for j in f32] for r in range(n)],
                                                 [[0, 1], [2]])
                    for r in range(n):
                        for k, j in enumerate(f32):
                            G.assert_same_bits(G.host(outs[r][j]).reshape(-1), want[k] / np.float32(n),
                                               "fused step %d tensor %d rank %d" % (step, j, r))


def test_prepared_batch_mixes_with_single_ops_and_reports_one_bad_node(oracle):
    """A prepared batch on some ranks and the same nodes submitted one by one on
    the others meet under their node names; a node whose shape differs on one
    rank fails alone, every step, with the reference's message."""
    n = 3
    xs = [[G.random_array(np.random.default_rng(7 * r + j), 5000 + j, np.float32) for j in range(3)] for r in range(n)]
    with mpi.Session(size=n) as session:
        handles = []
        with session.as_rank(0):
            batch = mpi.prepare_allreduce_batch([cuda(x) for x in xs[0]], average=False)
            handles.append(batch.submit())
        for r in (1, 2):
            with session.as_rank(r):
                handles.append([mpi.allreduce(cuda(x), average=False) for x in xs[r]])
        outs = session.run(handles)
        for j in range(3):
            want = oracle.ring_allreduce([xs[r][j] for r in range(n)])
            for r in range(n):
                G.assert_same_bits(G.host(outs[r][j]), want[r], "mixed submission tensor %d rank %d" % (j, r))
    with mpi.Session(size=n) as session:
        batches = []
        for r in range(n):
            with session.as_rank(r):
                ts = [cuda(xs[r][0]), cuda(xs[r][1] if r != 1 else xs[r][1][:17]), cuda(xs[r][2])]
                batches.append(mpi.prepare_allreduce_batch(ts, average=False))
        for step in range(2):
            handles = [b.submit() for b in batches]
            with pytest.raises(mpi.FailedPreconditionError) as e:
                session.run()
            assert "Mismatched allreduce tensor shapes" in str(e.value)
            for r in range(n):
                G.assert_same_bits(G.host(handles[r][0].result()), oracle.ring_allreduce([xs[q][0] for q in range(n)])[r],
                                   "good node of a batch with a bad one")
                with pytest.raises(mpi.FailedPreconditionError):
                    handles[r][1].result()
                G.assert_same_bits(G.host(handles[r][2].result()), oracle.ring_allreduce([xs[q][2] for q in range(n)])[r],
                                   "the node behind the bad one")
    with pytest.raises(mpi.FailedPreconditionError):
        batches[0].submit()                                 # its session is closed


def test_distributed_optimizer_builds_its_nodes_once(oracle):
    """DistributedOptimizer over gradients that stay where they are
    (zero_grad(set_to_none=False)): the allreduce nodes are built at the first
    step and run again at the next ones, in place; every step's gradients are
    the ring's averages and all replicas stay equal."""
    n, steps = 3, 3
    torch.manual_seed(3)
    base = torch.nn.Sequential(torch.nn.Linear(29, 17), torch.nn.Tanh(), torch.nn.Linear(17, 4)).cuda()
    replicas, opts = [], []
    for r in range(n):
        m = torch.nn.Sequential(torch.nn.Linear(29, 17), torch.nn.Tanh(), torch.nn.Linear(17, 4)).cuda()
        m.load_state_dict(base.state_dict())
        replicas.append(m)
        opts.append(mpi.DistributedOptimizer(torch.optim.SGD(m.parameters(), lr=0.1)))
    with mpi.Session(size=n) as session:
        built = []
        for step in range(steps):
            local, gvs = [], []
            for r in range(n):
                with session.as_rank(r):
                    opts[r].zero_grad(set_to_none=False)
                    x = torch.randn(13, 29, generator=torch.Generator().manual_seed(100 * step + r)).cuda()
                    replicas[r](x).square().mean().backward()
                    local.append([G.host(p.grad).reshape(-1).copy() for p in replicas[r].parameters()])
                    gvs.append(opts[r].compute_gradients())
            session.run()
            for r in range(n):
                with session.as_rank(r):
                    opts[r].apply_gradients(gvs[r])
            built.append([id(o._batch) for o in opts])
            for j in range(len(local[0])):
                want = oracle.ring_allreduce([local[r][j] for r in range(n)])[0] / np.float32(n)
                for r in range(n):
                    G.assert_same_bits(G.host(list(replicas[r].parameters())[j].grad).reshape(-1), want,
                                       "step %d rank %d gradient %d" % (step, r, j))
            for p0, p1 in zip(replicas[0].parameters(), replicas[n - 1].parameters()):
                assert torch.equal(p0, p1)
        assert built[1] == built[2], "the nodes were rebuilt although the gradients stayed in place"


@pytest.mark.parametrize("set_to_none", [None, True])
def test_distributed_optimizer_with_default_and_freed_gradients(oracle, set_to_none):
    """zero_grad() as a training loop calls it. The wrapper's default keeps the
    gradient tensors (set_to_none=False), so the nodes are built once; with
    set_to_none=True every backward allocates new gradients, and after two
    steps of rebuilding the optimizer stops building nodes for tensors it will
    not see again. Either way every step's gradients are the ring's averages,
    and the session's list of batches does not grow with the steps."""
    n, steps = 2, 5
    torch.manual_seed(5)
    base = torch.nn.Linear(11, 7).cuda()
    replicas, opts = [], []
    for r in range(n):
        m = torch.nn.Linear(11, 7).cuda()
        m.load_state_dict(base.state_dict())
        replicas.append(m)
        opts.append(mpi.DistributedOptimizer(torch.optim.SGD(m.parameters(), lr=0.05)))
    with mpi.Session(size=n) as session:
        live = []
        for step in range(steps):
            local, gvs = [], []
            for r in range(n):
                with session.as_rank(r):
                    if set_to_none is None:
                        opts[r].zero_grad()
                    else:
                        opts[r].zero_grad(set_to_none=set_to_none)
                    x = torch.randn(9, 11, generator=torch.Generator().manual_seed(10 * step + r)).cuda()
                    replicas[r](x).square().mean().backward()
                    local.append([G.host(p.grad).reshape(-1).copy() for p in replicas[r].parameters()])
                    gvs.append(opts[r].compute_gradients())
            session.run()
            for r in range(n):
                with session.as_rank(r):
                    opts[r].apply_gradients(gvs[r])
            live.append(len(session._batches))
            for j in range(len(local[0])):
                want = oracle.ring_allreduce([local[r][j] for r in range(n)])[0] / np.float32(n)
                for r in range(n):
                    G.assert_same_bits(G.host(list(replicas[r].parameters())[j].grad).reshape(-1), want,
                                       "step %d rank %d gradient %d" % (step, r, j))
        if set_to_none is None:
            assert live == [n] * steps, live                  # one batch per rank, built at the first step
        else:
            assert max(live) <= 2 * n and live[-1] <= n, live  # replaced, closed, and given up after two rebuilds
        for o in opts:
            o.close()
        assert session._batches == []


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fused_allreduce_of_resident_ranks_without_a_fused_buffer(oracle, dtype):
    """ring_fusion_allreduce_all: one launch over the tensors of all ranks gives
    every tensor what pack, the reference ring on the packed buffer and unpack
    give (tf.div included), into tensors of their own and in place; tensor sets
    with tiny, empty and misaligned tensors, ring segments that cut through
    tensors, and the full 161-tensor ResNet-50 set at N=8 for float32."""
    rng = np.random.default_rng(17)
    code = G.NP2ABI[np.dtype(dtype)]
    cases = [(3, [5, 0, 4099, 1, 64, 0, 3]), (8, [20_000, 64, 64, 36_864, 64, 64, 9_001, 2, 12_288]),
             (5, [int(c) for c in rng.integers(0, 40, 500)] + [9_000]), (16, [70_001]), (1, [100, 7])]
    if dtype == np.float32:
        cases.append((8, [int(np.prod(s)) for s in G.resnet50_shapes()]))
    for n, counts in cases:
        total = sum(counts)
        for divisor in (0, n):
            hosts = [[G.random_array(rng, c, dtype) for c in counts] for _ in range(n)]
            if dtype != np.float32:
                for r in range(n):
                    for h in hosts[r]:
                        h[: h.size // 2] = -np.abs(h[: h.size // 2])          # negative sums for the floor division
            ins = [[G.dev(h, (j + r) % 4) for j, h in enumerate(hosts[r])] for r in range(n)]
            outs = [[G.dev(np.zeros(c, dtype=dtype), (j + 2 * r + 1) % 4) for j, c in enumerate(counts)] for r in range(n)]
            in_plans = [ring_abi.FusionPlan([t[0].data_ptr() if c else None for t, c in zip(ins[r], counts)], counts, code)
                        for r in range(n)]
            out_plans = [ring_abi.FusionPlan([t[0].data_ptr() if c else None for t, c in zip(outs[r], counts)], counts, code)
                         for r in range(n)]
            packed = [np.concatenate(hosts[r]) if total else np.zeros(0, dtype=dtype) for r in range(n)]
            want = oracle.ring_allreduce(packed)[0] if total else packed[0]
            if divisor:
                want = _tf_div(want, divisor)
            ring_abi.fusion_allreduce_all(in_plans, out_plans, divisor, None)
            G.sync()
            for where, plans_in, tensors in (("fresh tensors", None, outs), ("in place", in_plans, ins)):
                if plans_in is not None:
                    ring_abi.fusion_allreduce_all(plans_in, plans_in, divisor, None)
                    G.sync()
                for r in range(n):
                    at = 0
                    for j, c in enumerate(counts):
                        G.assert_same_bits(G.host(tensors[r][j][0]), want[at:at + c],
                                           "n=%d /%d %s rank %d tensor %d of %d" % (n, divisor, where, r, j, len(counts)))
                        at += c
            for p in in_plans + out_plans:
                p.close()
