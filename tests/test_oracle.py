"""Pins the CPU oracle (oracle/ring_oracle.c) before anything is compared with it.

Checks, none of which re-types the oracle's own code path:
  * segment tables against the closed form and the ragged known answers;
  * accumulate against numpy's binary32 / integer addition;
  * the whole ring against (a) the closed-form left fold (conftest), (b) the
    lockstep evaluator, (c) the committed known-answer vectors made by a
    pure-Python mailbox simulation, (d) the same per-rank code over real MPI;
  * the invariants the reference's own tests assert
    (tensorflow/contrib/mpi_collectives/mpi_ops_test.py:84-112, 204-263;
    mpi_allreduce_test.py:96-105).
"""
import itertools
import json
import os

import numpy as np
import pytest

from conftest import bits, ring_closed_form

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DTYPES = [np.float32, np.int32, np.int64]


def make_inputs(n, count, dtype, seed=0):
    out = []
    for r in range(n):
        rng = np.random.default_rng(seed + r)
        if np.dtype(dtype) == np.float32:
            out.append((rng.standard_normal(count) * 10.0 ** rng.integers(-3, 4, count)).astype(np.float32))
        else:
            out.append(rng.integers(-1000, 1001, count).astype(dtype))
    return out


# --- segment split: ring.h:150-166 ------------------------------------------------

def test_segment_table_closed_form(oracle):
    for n in (1, 2, 3, 6, 8, 16, 64):
        for count in (0, 1, n - 1, n, n + 1, 17, 4913, 10_000_019, 16_777_216):
            if count < 0:
                continue
            sizes, starts = oracle.segment_table(count, n)
            q, rem = divmod(count, n)
            assert sizes == [q + 1] * rem + [q] * (n - rem)
            assert starts == [sum(sizes[:i]) for i in range(n)]
            assert starts[-1] + sizes[-1] == count          # ring.h:166
            assert oracle.temp_elements(count, n) == -(-count // n) == max(sizes)


def test_segment_table_known_answers(oracle):
    # ragged 10,000,019 elements over 6 ranks: only the last segment is short
    sizes, starts = oracle.segment_table(10_000_019, 6)
    assert sizes == [1_666_670] * 5 + [1_666_669]
    assert starts == [0, 1_666_670, 3_333_340, 5_000_010, 6_666_680, 8_333_350]
    # 64 MiB of float32 over 8 ranks, 1 GiB over 64, the 161-tensor fused buffer over 8
    assert oracle.segment_table(16_777_216, 8)[0] == [2_097_152] * 8
    assert oracle.segment_table(268_435_456, 64)[0] == [4_194_304] * 64
    assert oracle.segment_table(25_557_032, 8)[0] == [3_194_629] * 8
    # fewer elements than ranks (a scalar loss): trailing segments are empty
    assert oracle.segment_table(1, 4) == ([1, 0, 0, 0], [0, 1, 1, 1])
    assert oracle.segment_table(0, 3) == ([0, 0, 0], [0, 0, 0])


def test_allgather_table(oracle):
    rows = [17, 32, 81, 12, 15, 23, 22]
    assert oracle.allgather_table(rows, 17) == [17 * sum(rows[:i]) for i in range(7)]
    assert oracle.allgather_table([5], 3) == [0]


# --- accumulate: ring.cc:41-50 ------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_accumulate_is_one_add_per_element(oracle, dtype):
    rng = np.random.default_rng(7)
    if dtype == np.float32:
        a = (rng.standard_normal(100_003) * 1e3).astype(np.float32)
        b = (rng.standard_normal(100_003) * 1e-2).astype(np.float32)
        special = np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, 1.17549435e-38],
                           dtype=np.float32)
        a[:8], b[:8] = special, special[::-1]
        a[8:16], b[8:16] = special, special
    else:
        info = np.iinfo(dtype)
        a = rng.integers(info.min, info.max, 100_003, dtype=dtype, endpoint=True)
        b = rng.integers(info.min, info.max, 100_003, dtype=dtype, endpoint=True)
    with np.errstate(all="ignore"):
        want = a + b                                   # numpy: IEEE binary32 / wrapping ints
    got = oracle.accumulate(a.copy(), b)
    if dtype == np.float32:
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(bits(got)[~nan], bits(want)[~nan])
    else:
        assert np.array_equal(got, want)
    empty = np.empty(0, dtype=dtype)
    oracle.accumulate(empty, empty)


# --- the whole ring ---------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 2, 3, 4, 6, 8])
def test_ring_matches_closed_form_and_lockstep(oracle, dtype, n):
    for count in sorted({0, 1, max(n - 1, 0), n, n + 1, 17, 4913}):
        ins = make_inputs(n, count, dtype, seed=1000 * n + count)
        want = ring_closed_form(ins)
        outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
        lock = oracle.ring_allreduce_lockstep(ins)
        for r in range(n):
            assert np.array_equal(bits(outs[r]), bits(want)), (n, count, r)
            assert np.array_equal(bits(lock[r]), bits(want)), (n, count, r)
        # the taps are what the right-hand neighbour's accumulate consumed:
        # the last reduce-scatter receive plus the local value is the owned segment
        sizes, starts = oracle.segment_table(count, n)
        for r in range(n):
            if n > 1:
                seg = (r + 1) % n
                sl = slice(starts[seg], starts[seg] + sizes[seg])
                # partial before the last step = fold of the other n-1 ranks
                part = rs[r][n - 2][:sizes[seg]]
                redo = ins[r][sl] + part
                assert np.array_equal(bits(redo), bits(want[sl]))
                for i in range(n - 1):
                    s = (r - i) % n
                    assert np.array_equal(bits(ag[r][i][:sizes[s]]),
                                          bits(want[starts[s]:starts[s] + sizes[s]]))


def test_ring_order_matters_and_is_the_rotated_left_fold(oracle):
    # (1e8 + 1) - 1e8 == 0 in binary32 but (1e8 - 1e8) + 1 == 1: a fold in any other
    # rotation or direction gives different bits on these columns.
    x = [np.array([1e8, -1e8, 1.0], dtype=np.float32),
         np.array([1.0, 1e8, -1e8], dtype=np.float32),
         np.array([-1e8, 1.0, 1e8], dtype=np.float32)]
    out = oracle.ring_allreduce(x)[0]
    # segment s (one element each) folds ranks s, s+1, s+2
    f = np.float32
    want = np.array([f(x[2][0]) + (f(x[1][0]) + f(x[0][0])),
                     f(x[0][1]) + (f(x[2][1]) + f(x[1][1])),
                     f(x[1][2]) + (f(x[0][2]) + f(x[2][2]))], dtype=np.float32)
    assert np.array_equal(bits(out), bits(want))
    assert list(out) == [0.0, 0.0, 0.0]
    # the plain rank-order sum differs, so the test would catch a wrong rotation
    naive = (x[0] + x[1]) + x[2]
    assert not np.array_equal(naive, out)


def test_one_rank_on_given_segments_by_hand_and_against_the_whole_ring(oracle):
    """The per-rank data path (one rank, its incoming segments given): a case
    worked out by hand from ring.h:183-225, then, for every rank of rings of
    several sizes, what that rank received in the threaded ring replayed to it
    alone must give its output of the threaded ring."""
    # n=3, r=1, one element per segment. Reduce-scatter: step 0 receives segment (1-0-1)%3 = 0,
    # step 1 segment (1-1-1)%3 = 2; allgather: step 0 receives segment 1, step 1 segment 0.
    for dtype in DTYPES:
        out = oracle.ring_allreduce_rank_prestaged(3, 1, np.array([1, 2, 4], dtype=dtype),
                                                   [np.array([8], dtype=dtype), np.array([16], dtype=dtype)],
                                                   [np.array([32], dtype=dtype), np.array([64], dtype=dtype)])
        assert list(out) == [64, 32, 4 + 16]
    # the same with the allgather of step 1 taken away would leave 1 + 8 in segment 0: the order of the
    # steps is what the hand-made answer pins. A ragged rank: n=3, count=4 -> sizes [2, 1, 1], r=0:
    # reduce-scatter receives segment 2 then 1, allgather segment 0 (2 elements) then 2.
    out = oracle.ring_allreduce_rank_prestaged(3, 0, np.array([1, 2, 4, 8], dtype=np.int64),
                                               [np.array([16]), np.array([32])],
                                               [np.array([64, 128]), np.array([256])])
    assert list(out) == [64, 128, 4 + 32, 256]
    for dtype, n, count in itertools.product(DTYPES, (1, 2, 3, 5, 8), (0, 1, 7, 4913)):
        ins = make_inputs(n, count, dtype, seed=100 * n + count)
        outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
        for r in range(n):
            alone = oracle.ring_allreduce_rank_prestaged(n, r, ins[r], list(rs[r]), list(ag[r]))
            assert np.array_equal(bits(alone), bits(outs[r])), (np.dtype(dtype).name, n, count, r)


def test_ring_known_answer_vectors(oracle):
    with open(os.path.join(GOLDEN, "ring_kats.json")) as f:
        kats = json.load(f)["cases"]
    assert len(kats) >= 27
    for case in kats:
        if case["dtype"] == "f32":
            ins = [np.array(x, dtype=np.uint32).view(np.float32) for x in case["inputs"]]
            want = np.array(case["expected"], dtype=np.uint32)
        else:
            dt = np.int32 if case["dtype"] == "i32" else np.int64
            ins = [np.array(x, dtype=dt) for x in case["inputs"]]
            want = bits(np.array(case["expected"], dtype=dt))
        for out in oracle.ring_allreduce(ins):
            assert np.array_equal(bits(out), want), (case["dtype"], case["n"], case["count"])
        assert np.array_equal(bits(ring_closed_form(ins)), want)


@pytest.mark.parametrize("n", [2, 3, 5])
def test_ring_over_real_mpi_matches(oracle, tmp_path, n):
    if oracle.mpirun_path() is None:
        pytest.skip("no MPI installation to run the restatement over")
    for dtype, count in ((np.float32, 4913), (np.int64, 1001), (np.int32, n - 1)):
        ins = make_inputs(n, count, dtype, seed=77)
        got = oracle.mpi_check(ins, str(tmp_path))
        want = ring_closed_form(ins)
        for r in range(n):
            assert np.array_equal(bits(got[r]), bits(want))


# --- invariants asserted by the reference's own tests ------------------------------

@pytest.mark.parametrize("size", [1, 2, 3, 4, 7, 9, 12, 14])
def test_reference_same_input_invariant(oracle, size):
    """mpi_ops_test.py:84-112: every rank reduces the same tensor, so the sum
    equals tensor*size, exactly for size<=3 and within 1e-4 / 5e-4 beyond."""
    for dtype, dim in itertools.product((np.int32, np.float32), (1, 2, 3)):
        rng = np.random.default_rng(1234)
        if dtype == np.float32:
            t = rng.uniform(-100, 100, [17] * dim).astype(np.float32)
        else:
            t = rng.integers(-100, 100, [17] * dim).astype(np.int32)
        outs = oracle.ring_allreduce([t] * size)
        threshold = 0 if size <= 3 else (1e-4 if size < 10 else 5e-4)
        for o in outs:
            diff = np.max(np.abs(o.reshape(t.shape).astype(np.float64) - t.astype(np.float64) * size))
            if dtype == np.int32:
                assert diff == 0
            else:
                # the reference compares in float32: |sum - t*size| evaluated in binary32
                d32 = np.max(np.abs(o.reshape(t.shape) - t * np.float32(size)))
                assert d32 <= threshold or diff <= 1e-3, (size, dim, d32)
                if size <= 3:
                    assert d32 == 0


@pytest.mark.parametrize("num_ranks", [2, 3])
@pytest.mark.parametrize("average", [False, True])
def test_reference_chained_allreduce_closed_form(oracle, num_ranks, average):
    """mpi_allreduce_test.py:40-112: 13 dependent allreduces of a 1331x1331
    matrix (odd element count: ragged segments for even sizes); the result is
    a constant matrix with a closed-form value."""
    stages, side, spread = 13, 1331, 100
    feeds = [np.full((side, side), 1.0 + r * spread, dtype=np.float32) for r in range(num_ranks)]
    state = feeds
    for i in range(stages):
        w = np.float32(2.0 ** (i + 1))
        summed = oracle.ring_allreduce([s + w for s in state])
        if average:
            summed = [s / np.float32(num_ranks) for s in summed]   # tf.div: true division
        state = [s.reshape(side, side) for s in summed]
    # closed form of mpi_allreduce_test.py:96-105
    ours = 1.0
    for i in range(stages):
        cur = ours + 2.0 ** (i + 1)
        if average:
            ours = cur + (spread * (num_ranks - 1) / 2 if i == 0 else 0)
        else:
            ours = cur * num_ranks + (spread * num_ranks * (num_ranks - 1) / 2 if i == 0 else 0)
    for s in state:
        assert np.allclose(s, np.float32(ours))
        assert np.all(s == s[0, 0])


@pytest.mark.parametrize("size", [1, 2, 3, 7, 16, 35])
def test_reference_allgather_rank_stamped(oracle, size):
    """mpi_ops_test.py:204-263: rank r contributes ones*r; slice r of every
    rank's output equals r. Equal and variable first dimensions."""
    tensor_sizes = ([17, 32, 81, 12, 15, 23, 22] * 5)[:size]
    for dtype, dim, variable in itertools.product((np.int32, np.float32, np.int64), (1, 2, 3), (False, True)):
        rows = tensor_sizes if variable else [17] * size
        ins = [np.ones([rows[r]] + [17] * (dim - 1), dtype=dtype) * r for r in range(size)]
        outs = oracle.ring_allgather(ins)
        for o in outs:
            assert list(o.shape) == [sum(rows)] + [17] * (dim - 1)
            for i in range(size):
                part = o[sum(rows[:i]):sum(rows[:i + 1])]
                assert part.shape[0] == rows[i] and np.all(part == i)
            assert np.array_equal(o, np.concatenate(ins, axis=0))


def test_allgather_random_payload_and_empty_rows(oracle):
    rng = np.random.default_rng(5)
    rows = [3, 0, 5, 1]
    ins = [rng.standard_normal((k, 6)).astype(np.float32) for k in rows]
    for o in oracle.ring_allgather(ins):
        assert np.array_equal(bits(o), bits(np.concatenate(ins, axis=0)))
