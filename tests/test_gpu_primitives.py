"""GPU parity of the device primitives behind the C ABI against the CPU oracle:
accumulate (ring.cu.cc:48-69), copy (ring.cu.cc:41-45), the batched step
tables, the average divide and fusion pack/unpack. Integer and float32 results
must match bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

import gpu_util as G
from gpu_util import ring_abi

pytestmark = pytest.mark.gpu

COUNTS = [0, 1, 2, 3, 4, 5, 7, 8, 1023, 1024, 1025, 4096, 4097, 3 * 4096 + 7, 262_144, 1_000_003]


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    G.require_gpu()
    yield
    for k, v in (("unroll", 4), ("nontemporal", -1), ("blocks_per_cu", 0), ("paced_copy", -1), ("phased_copy", -1)):
        ring_abi.set_option(k, v)


def special_f32():
    return np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.1754942e-38,
                     1.17549435e-38, 3.4028235e38, -3.4028235e38, 1.0, 16777216.0, 1e-30],
                    dtype=np.float32)


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_accumulate_matches_oracle(oracle, dtype):
    rng = np.random.default_rng(11)
    for count in COUNTS:
        for doff, soff in ((0, 0), (1, 0), (0, 1), (3, 2), (2, 3), (1, 1)):
            a = G.random_array(rng, count, dtype, wide=True)
            b = G.random_array(rng, count, dtype, wide=True)
            if dtype == np.float32 and count >= 1024:
                sp = special_f32()
                k = sp.size
                for i in range(k):                      # every special against every special
                    a[i * k:(i + 1) * k] = sp[i]
                    b[i * k:(i + 1) * k] = sp
            da, keep_a = G.dev(a, doff)
            db, keep_b = G.dev(b, soff)
            ring_abi.accumulate(G.NP2ABI[np.dtype(dtype)], da.data_ptr(), db.data_ptr(), count, None)
            G.sync()
            want = oracle.accumulate(a.copy(), b)
            G.assert_same_bits(G.host(da), want, "accumulate %s n=%d off=%d/%d" % (dtype.__name__, count, doff, soff))
            # nothing outside the destination range moved, the source is untouched
            assert np.all(G.host(keep_a[:doff]) == 0) and np.all(G.host(keep_a[doff + count:]) == 0)
            G.assert_same_bits(G.host(db), b)


def test_more_than_2_pow_32_elements():
    """Counts are 64-bit end to end (the reference's CPU loop indexes with an
    `unsigned int`, ring.cc:44, and passes size_t counts to MPI as int)."""
    import torch
    count = (1 << 32) + 12_345
    gen = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randint(-2**31, 2**31 - 1, (count + 3,), dtype=torch.int32, device="cuda", generator=gen)
    b = torch.randint(-2**31, 2**31 - 1, (count + 1,), dtype=torch.int32, device="cuda", generator=gen)
    want = a[3:] + b[1:]                                  # wraps like the ring's integer add
    got = a.clone()
    ring_abi.accumulate(ring_abi.I32, got.data_ptr() + 12, b.data_ptr() + 4, count, None)
    G.sync()
    assert torch.equal(got[3:], want) and torch.equal(got[:3], a[:3])
    del want
    ring_abi.copy_bytes(got.data_ptr(), b.data_ptr() + 4, count * 4, None)
    G.sync()
    assert torch.equal(got[:count], b[1:]) and torch.equal(got[count:], (a[3:] + b[1:])[count - 3:])


def test_typed_entry_points_and_errors():
    L = ring_abi.lib()
    a, _ = G.dev(np.arange(10, dtype=np.float32))
    b, _ = G.dev(np.ones(10, dtype=np.float32))
    assert L.ring_accumulate_f32(a.data_ptr(), b.data_ptr(), 10, None) == 0
    ai, _ = G.dev(np.arange(10, dtype=np.int32))
    bi, _ = G.dev(np.full(10, 2**31 - 1, dtype=np.int32))
    assert L.ring_accumulate_i32(ai.data_ptr(), bi.data_ptr(), 10, None) == 0
    al, _ = G.dev(np.arange(10, dtype=np.int64))
    bl, _ = G.dev(np.full(10, -2**63, dtype=np.int64))
    assert L.ring_accumulate_i64(al.data_ptr(), bl.data_ptr(), 10, None) == 0
    G.sync()
    assert np.array_equal(G.host(a), np.arange(10, dtype=np.float32) + 1)
    with np.errstate(over="ignore"):
        assert np.array_equal(G.host(ai), np.arange(10, dtype=np.int32) + np.int32(2**31 - 1))
        assert np.array_equal(G.host(al), np.arange(10, dtype=np.int64) + np.int64(-2**63))
    # error behaviour: bad dtype, null with a size, misaligned element pointer
    assert L.ring_accumulate(7, a.data_ptr(), b.data_ptr(), 10, None) == 1
    assert ring_abi.status_string(1) == "Invalid tensor type passed."       # mpi_ops.cc:844
    assert L.ring_accumulate(0, None, b.data_ptr(), 10, None) == 2
    assert L.ring_accumulate(0, a.data_ptr() + 2, b.data_ptr(), 4, None) == 2
    assert L.ring_accumulate(0, None, None, 0, None) == 0                   # empty tensor: null, 0
    assert L.ring_copy_bytes(None, None, 0, None) == 0
    assert L.ring_copy_bytes(None, b.data_ptr(), 4, None) == 2


def test_copy_bytes():
    rng = np.random.default_rng(3)
    for nbytes in (0, 1, 3, 4, 5, 15, 16, 17, 4096, 65_536 + 4, 1_000_003, 4_000_012):
        for doff, soff in ((0, 0), (4, 0), (0, 8), (12, 4), (1, 0), (0, 3), (2, 2)):
            src = rng.integers(0, 256, nbytes + 32, dtype=np.uint8)
            import torch
            dsrc = torch.from_numpy(src).cuda()
            ddst = torch.zeros(nbytes + 64, dtype=torch.uint8, device="cuda")
            ring_abi.copy_bytes(ddst.data_ptr() + doff, dsrc.data_ptr() + soff, nbytes, None)
            G.sync()
            out = G.host(ddst)
            assert np.array_equal(out[doff:doff + nbytes], src[soff:soff + nbytes]), (nbytes, doff, soff)
            assert not out[:doff].any() and not out[doff + nbytes:].any()


def _random_table(rng, n_rows, dtype, max_count):
    """Disjoint destination ranges inside one buffer, at ragged offsets."""
    counts = [int(c) for c in rng.integers(0, max_count, n_rows)]
    counts[rng.integers(0, n_rows)] = 0
    gaps = [int(g) for g in rng.integers(0, 4, n_rows)]
    offs, at = [], int(rng.integers(0, 4))
    for c, g in zip(counts, gaps):
        offs.append(at)
        at += c + g
    order = rng.permutation(n_rows)            # rows need not be sorted by offset
    return [(offs[i], counts[i]) for i in order], at


def test_launch_timing_hook_times_the_armed_launches_in_order():
    """ring_time_next_launch / ring_event_elapsed_us (what bench.py's roofline
    figures are measured with): each armed pair times one launch, in order; a
    64 MiB copy takes longer than a 1 MiB one and both lie between what 8 TB/s
    and 0.2 TB/s would give; pairs beyond 8 are refused; null events disarm;
    the results of timed launches are the results of untimed ones."""
    stream = ring_abi.stream_create()
    try:
        big_n, small_n = 16 << 20, 256 << 10                      # float32 elements: 64 MiB and 1 MiB
        src = torch.arange(big_n, dtype=torch.float32, device="cuda")
        dst = torch.zeros(big_n, dtype=torch.float32, device="cuda")
        acc = torch.ones(small_n, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        events = [(ring_abi.event_create(), ring_abi.event_create()) for _ in range(9)]
        for _ in range(2):                                          # the first round warms up
            for pair in events[:3]:
                ring_abi.time_next_launch(*pair)
            ring_abi.copy_bytes(dst.data_ptr(), src.data_ptr(), big_n * 4, stream)
            ring_abi.copy_bytes(dst.data_ptr(), src.data_ptr(), small_n * 4, stream)
            ring_abi.accumulate(ring_abi.F32, acc.data_ptr(), src.data_ptr(), small_n, stream)
            ring_abi.stream_synchronize(stream)
        big, small, add = [ring_abi.event_elapsed_us(*pair) for pair in events[:3]]
        assert 2 * (64 << 20) / 8e6 < big < 2 * (64 << 20) / 0.2e6, big           # 16.8 us at 8 TB/s
        assert 0.5 < small < big / 4, (small, big)
        assert 0.5 < add < big / 4, (add, big)
        assert torch.equal(dst, src) and torch.equal(acc[:16], 1 + 2 * src[:16])
        # nine pairs ahead: the ninth is refused, two nulls drop the eight that wait
        for pair in events[:8]:
            ring_abi.time_next_launch(*pair)
        with pytest.raises(ring_abi.RingError):
            ring_abi.time_next_launch(*events[8])
        ring_abi.time_next_launch(None, None)
        ring_abi.copy_bytes(dst.data_ptr(), src.data_ptr(), small_n * 4, stream)   # not timed any more
        ring_abi.stream_synchronize(stream)
        assert ring_abi.event_elapsed_us(*events[0]) == big         # still what the first round's launch took
        for pair in events:
            for e in pair:
                ring_abi.event_destroy(e)
    finally:
        ring_abi.stream_destroy(stream)


def test_one_direction_probes_touch_what_they_say():
    """ring_probe_stream (the measurement hook behind bench.py's floors
    workloads): a write probe fills exactly the whole 16-byte vectors of every
    row with (1, 2, 3, lane) and nothing else, a read probe changes nothing,
    and rows it cannot take are refused."""
    counts = [1, 4, 21, 4096, 4099, 1_000_003, 3 * 1024 * 1024 + 2]      # float32 elements
    for mode in (0, 2, 1, 3):
        bufs = [torch.full((c + 8,), 7.0, dtype=torch.float32, device="cuda") for c in counts]
        rows = [(b[4:].data_ptr(), b[4:].data_ptr(), None, c) for b, c in zip(bufs, counts)]    # 16 bytes in: aligned
        ring_abi.probe_stream(rows, ring_abi.F32, mode, None)
        G.sync()
        for b, c in zip(bufs, counts):
            h = G.host(b)
            whole = c // 4
            if mode & 1:
                words = h[4:4 + 4 * whole].view(np.uint32).reshape(whole, 4)
                assert (words[:, 0] == 1).all() and (words[:, 1] == 2).all() and (words[:, 2] == 3).all()
                assert (words[:, 3] == np.arange(whole) % 256).all()
                assert (h[:4] == 7.0).all() and (h[4 + 4 * whole:] == 7.0).all(), "a write probe stays inside its whole vectors"
            else:
                assert (h == 7.0).all(), "a read probe leaves memory alone"
    x = torch.zeros(64, dtype=torch.float32, device="cuda")
    with pytest.raises(ring_abi.RingError):
        ring_abi.probe_stream([(x[1:].data_ptr(), x[1:].data_ptr(), None, 32)], ring_abi.F32, 0, None)   # misaligned
    with pytest.raises(ring_abi.RingError):
        ring_abi.probe_stream([(x.data_ptr(), x.data_ptr(), None, 32)] * 9, ring_abi.F32, 0, None)      # more than 8 rows
    with pytest.raises(ring_abi.RingError):
        ring_abi.probe_stream([(x.data_ptr(), x.data_ptr(), None, 32)], ring_abi.F32, 4, None)          # no such mode
    G.sync()


@pytest.mark.parametrize("dtype", G.DTYPES)
@pytest.mark.parametrize("n_rows", [1, 7, 63, 64, 65, 150])
def test_step_tables_match_oracle(oracle, dtype, n_rows):
    rng = np.random.default_rng(100 + n_rows)
    code = G.NP2ABI[np.dtype(dtype)]
    table, total = _random_table(rng, n_rows, dtype, 20_000 if n_rows < 100 else 3_000)
    for accumulate in (True, False):
        buf = G.random_array(rng, total + 5, dtype)
        dbuf, _ = G.dev(buf, int(rng.integers(0, 4)))
        srcs, rows, keep = [], [], []
        for off, cnt in table:
            s = G.random_array(rng, cnt, dtype)
            ds, base = G.dev(s, int(rng.integers(0, 4)))
            srcs.append(s)
            keep.append(base)
            rows.append((off, ds.data_ptr() if cnt else None, cnt))
        steps, n = ring_abi.make_steps(rows)
        want = buf.copy()
        for (off, cnt), s in zip(table, srcs):
            if accumulate:
                oracle.accumulate(want[off:off + cnt], s)
            else:
                want[off:off + cnt] = s
        fn = ring_abi.reduce_scatter_steps if accumulate else ring_abi.allgather_steps
        fn(dbuf.data_ptr(), steps, n, code, None)
        G.sync()
        G.assert_same_bits(G.host(dbuf), want, "table rows=%d acc=%s" % (n_rows, accumulate))


@pytest.mark.parametrize("dtype", G.DTYPES)
@pytest.mark.parametrize("paced", [1, 0])
def test_paced_allgather_copies_match(dtype, paced):
    """The allgather copies as one read phase and one write phase (32 KiB tiles that wait
    for all their loads and keep one store in flight), forced on for launches of any size
    and forced off: the same bytes either way, ragged rows at any alignment, rows shorter
    than a tile, a row of many tiles with a partial last one."""
    rng = np.random.default_rng(41 + paced)
    code = G.NP2ABI[np.dtype(dtype)]
    ring_abi.set_option("paced_copy", paced)
    try:
        for n_rows, max_count in ((1, 300_000), (7, 70_000), (16, 9_000), (64, 3_000)):
            table, total = _random_table(rng, n_rows, dtype, max_count)
            buf = G.random_array(rng, total + 5, dtype)
            dbuf, _ = G.dev(buf, int(rng.integers(0, 4)))
            want = buf.copy()
            rows, keep = [], []
            for off, cnt in table:
                src = G.random_array(rng, cnt, dtype)
                ds, base = G.dev(src, int(rng.integers(0, 4)))
                keep.append(base)
                rows.append((off, ds.data_ptr() if cnt else None, cnt))
                want[off:off + cnt] = src
            steps, n = ring_abi.make_steps(rows)
            ring_abi.allgather_steps(dbuf.data_ptr(), steps, n, code, None)
            G.sync()
            G.assert_same_bits(G.host(dbuf), want, "paced=%d rows=%d" % (paced, n_rows))
    finally:
        ring_abi.set_option("paced_copy", -1)


@pytest.mark.parametrize("dtype", G.DTYPES)
@pytest.mark.parametrize("phased", [1, 0, -1])
def test_phased_allgather_copies_match(dtype, phased):
    """The allgather copies with the whole payload in registers between one read
    phase and one write phase of the chip (rows of near-equal length, at most
    one workgroup per CU), forced on for every launch that fits and forced off:
    the same bytes either way, ragged segments at any alignment, counts from
    fewer elements than ranks up to all 112 vectors a lane has room for, and
    counts that just no longer fit (they must fall back, not truncate)."""
    rng = np.random.default_rng(43 + phased)
    code = G.NP2ABI[np.dtype(dtype)]
    vec = 16 // np.dtype(dtype).itemsize
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ring_abi.set_option("phased_copy", phased)
    try:
        stride = cus * 256 * vec                                  # elements the chip takes per round
        cases = [(8, 5), (6, 100_003), (8, 1_000_003), (3, 70_001), (64, 1_000_003), (2, 4_099), (9, 9_000_017),
                 (8, 8 * 16 * stride),                            # 7 rows of 16 rounds: all the registers
                 (8, 8 * (16 * stride + 128)),                    # a 17th round: must fall back, not truncate
                 (5, 5 * 28 * stride + 3), (2, 2 * 112 * stride + 1)]
        for n, count in cases:
            sizes, starts = ring_abi.segment_table(count, n)
            buf = G.random_array(rng, count + 5, dtype)
            dbuf, _ = G.dev(buf, int(rng.integers(0, 4)))
            want = buf.copy()
            rows, keep = [], []
            for g in range(1, n):                                 # n - 1 segments arrive, as in the allgather phase
                src = G.random_array(rng, sizes[g], dtype)
                ds, base = G.dev(src, int(rng.integers(0, 4)))
                keep.append(base)
                rows.append((starts[g], ds.data_ptr() if sizes[g] else None, sizes[g]))
                want[starts[g]:starts[g] + sizes[g]] = src
            steps, k = ring_abi.make_steps(rows)
            ring_abi.allgather_steps(dbuf.data_ptr(), steps, k, code, None)
            G.sync()
            G.assert_same_bits(G.host(dbuf), want, "phased=%d n=%d count=%d" % (phased, n, count))
    finally:
        ring_abi.set_option("phased_copy", -1)


@pytest.mark.parametrize("opt", [("unroll", 2), ("unroll", 8), ("nontemporal", 0),
                                 ("nontemporal", 1), ("nontemporal", 2), ("nontemporal", 3),
                                 ("blocks_per_cu", 1), ("blocks_per_cu", 8)])
def test_launch_options_do_not_change_results(oracle, opt):
    ring_abi.set_option(*opt)
    try:
        rng = np.random.default_rng(5)
        for dtype in G.DTYPES:
            for count in (5, 4097, 2_000_003):
                a = G.random_array(rng, count, dtype)
                b = G.random_array(rng, count, dtype)
                da, _ = G.dev(a, 1)
                db, _ = G.dev(b, 2)
                ring_abi.accumulate(G.NP2ABI[np.dtype(dtype)], da.data_ptr(), db.data_ptr(), count, None)
                dc, _ = G.dev(np.zeros(count, dtype=dtype), 3)
                ring_abi.copy_bytes(dc.data_ptr(), db.data_ptr(), count * a.itemsize, None)
                G.sync()
                G.assert_same_bits(G.host(da), oracle.accumulate(a.copy(), b), str(opt))
                G.assert_same_bits(G.host(dc), b, str(opt))
            _fusion_roundtrip([5, 0, 4096, 1, 0, 3, 8191, 2, 70_001], dtype, rng)
    finally:
        for k, v in (("unroll", 4), ("nontemporal", -1), ("blocks_per_cu", 0)):
            ring_abi.set_option(k, v)


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_rows_with_the_divide_folded_in(dtype):
    """ring_apply_rows_avg: flagged rows store (b + a) / n or a / n, the others
    b + a or a; equal to the accumulate followed by ring_scale's division,
    negative integers floored, any alignment, more rows than one table holds."""
    import torch
    rng = np.random.default_rng(77)
    code = G.NP2ABI[np.dtype(dtype)]
    for n_rows, divisor in ((1, 1), (4, 8), (7, 3), (70, 6)):
        counts = [int(c) for c in rng.integers(0, 9000, n_rows)]
        counts[0] = 20_011
        rows, wants, devs, flags = [], [], [], []
        for k, c in enumerate(counts):
            a = G.random_array(rng, c, dtype)
            b = G.random_array(rng, c, dtype)
            if dtype != np.float32 and c:
                a[: c // 2] = -np.abs(a[: c // 2])          # negative sums with remainders
                b[: c // 2] = -np.abs(b[: c // 2])
            da, _ = G.dev(a, k % 4)
            kind = k % 3                                        # in-place add, out-of-place add, copy
            flag = bool((k * 7 + 1) % 2)
            if kind == 0:
                db, _ = G.dev(b, (k + 1) % 4)
                dst, bptr = db, db.data_ptr()
            elif kind == 1:
                db, _ = G.dev(b, (k + 2) % 4)
                dst, _ = G.dev(np.zeros(c, dtype=dtype), (k + 3) % 4)
                bptr = db.data_ptr()
            else:
                db = None
                dst, _ = G.dev(np.zeros(c, dtype=dtype), (k + 1) % 4)
                bptr = None
            with np.errstate(all="ignore"):
                w = a if kind == 2 else (b + a).astype(dtype)
                if flag:
                    w = w / np.float32(divisor) if dtype == np.float32 else w // dtype(divisor)
            rows.append((dst.data_ptr() if c else None, da.data_ptr() if c else None, bptr if c else None, c))
            wants.append(np.asarray(w, dtype=dtype))
            devs.append((dst, da, db))
            flags.append(flag)
        ring_abi.apply_rows_avg(rows, flags, divisor, code, None)
        G.sync()
        for k, (dst, _, _) in enumerate(devs):
            G.assert_same_bits(G.host(dst), wants[k], "row %d of %d, /%d, flag %s" % (k, n_rows, divisor, flags[k]))
    # divide=None flags every row; divisor 0 is plain ring_apply_rows
    a = G.random_array(rng, 1000, dtype)
    da, _ = G.dev(a, 1)
    out, _ = G.dev(np.zeros(1000, dtype=dtype), 2)
    ring_abi.apply_rows_avg([(out.data_ptr(), da.data_ptr(), None, 1000)], None, 5, code, None)
    G.sync()
    with np.errstate(all="ignore"):
        G.assert_same_bits(G.host(out), (a / np.float32(5) if dtype == np.float32 else a // dtype(5)).astype(dtype), "all rows")
    ring_abi.apply_rows_avg([(out.data_ptr(), da.data_ptr(), None, 1000)], [True], 0, code, None)
    G.sync()
    G.assert_same_bits(G.host(out), a, "divisor 0")
    with pytest.raises(ring_abi.RingError):
        ring_abi.apply_rows_avg([(out.data_ptr(), da.data_ptr(), None, 1000)], None, -1, code, None)


def _fold_reference(srcs, divisor, dtype):
    """acc = s0; acc = s_k + acc, one rounded add per step, then tf.div."""
    acc = srcs[0].copy()
    with np.errstate(all="ignore"):
        for s in srcs[1:]:
            acc = (s + acc).astype(dtype)
        if divisor:
            acc = (acc / np.float32(divisor) if dtype == np.float32 else acc // dtype(divisor)).astype(dtype)
    return acc


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fold_rows_is_the_sequential_fold(dtype):
    """ring_fold_rows against a numpy fold in the same order: any number of
    sources, rows of equal and unequal length, any alignment, the divide, a
    destination that is one of the sources, more rows than one launch holds."""
    rng = np.random.default_rng(99)
    code = G.NP2ABI[np.dtype(dtype)]
    cases = [(1, 1, [10]), (2, 1, [4099]), (3, 2, [7, 0]), (8, 8, [30_011] * 8), (8, 3, [5, 9000, 123]),
             (9, 40, [int(c) for c in rng.integers(0, 3000, 40)]), (64, 2, [2049, 2049]), (256, 1, [1500])]
    for m, n_rows, counts in cases:
        for divisor in (0, 6):
            rows, wants, dsts, keep = [], [], [], []
            for k, c in enumerate(counts):
                hs = [G.random_array(rng, c, dtype, wide=dtype == np.float32) for _ in range(m)]
                if dtype != np.float32 and c:
                    hs[0][: c // 2] = -np.abs(hs[0][: c // 2]) - 7        # negative sums for the floor division
                ds = [G.dev(h, (k + j) % 4) for j, h in enumerate(hs)]
                keep.append(ds)
                in_place = k % 2 == 1                                     # dst is the last source
                if in_place:
                    dst = ds[-1][0]
                else:
                    dst, base = G.dev(np.zeros(c, dtype=dtype), (k + 2) % 4)
                    keep.append(base)
                rows.append((dst.data_ptr() if c else None, [d[0].data_ptr() if c else None for d in ds], c))
                wants.append(_fold_reference(hs, divisor, dtype))
                dsts.append(dst)
            ring_abi.fold_rows(rows, m, divisor, code, None)
            G.sync()
            for k in range(n_rows):
                G.assert_same_bits(G.host(dsts[k]), wants[k], "fold m=%d row %d of %d /%d" % (m, k, n_rows, divisor))
    x, _ = G.dev(np.ones(8, dtype=dtype), 0)
    with pytest.raises(ring_abi.RingError):
        ring_abi.fold_rows([(x.data_ptr(), [x.data_ptr()] * 257, 8)], 257, 0, code, None)
    with pytest.raises(ring_abi.RingError):
        ring_abi.fold_rows([(x.data_ptr(), [None, x.data_ptr()], 8)], 2, 0, code, None)
    with pytest.raises(ring_abi.RingError):
        ring_abi.fold_rows([(x.data_ptr(), [x.data_ptr()], 8)], 1, -1, code, None)


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fold_stored_to_every_rank(dtype):
    """ring_fold_to_all_rows: the numpy fold in the same order, stored to n_dst
    destinations of differing alignment; rows of unequal length, the divide, an
    allreduce in place (every destination is a source), more pointers than one
    launch's table holds, one source stored to several destinations."""
    rng = np.random.default_rng(7)
    code = G.NP2ABI[np.dtype(dtype)]
    for m, n_dst, counts in ((1, 1, [33]), (1, 4, [700, 3]), (2, 3, [4099, 0, 12]), (8, 8, [30_011] * 8), (5, 7, [9000, 5, 2049]),
                             (40, 40, [1500] * 6), (128, 129, [777])):
        for divisor in (0, 6):
            rows, checks, keep = [], [], []
            for k, c in enumerate(counts):
                hs = [G.random_array(rng, c, dtype, wide=dtype == np.float32) for _ in range(m)]
                if dtype != np.float32 and c:
                    hs[0][: c // 2] = -np.abs(hs[0][: c // 2]) - 7
                ds = [G.dev(h, (k + j) % 4) for j, h in enumerate(hs)]
                outs = [G.dev(np.zeros(c, dtype=dtype), (k + 3 * j + 1) % 4) for j in range(n_dst)]
                keep += [ds, outs]
                rows.append(([o[0].data_ptr() if c else None for o in outs], [d[0].data_ptr() if c else None for d in ds], c))
                want = _fold_reference(hs, divisor, dtype)
                checks += [(o[0], want, "row %d destination %d" % (k, j)) for j, o in enumerate(outs)]
            ring_abi.fold_to_all_rows(rows, m, n_dst, divisor, code, None)
            G.sync()
            for t, want, what in checks:
                G.assert_same_bits(G.host(t), want, "fold to all m=%d n_dst=%d /%d %s" % (m, n_dst, divisor, what))
    # in place: 6 ranks whose outputs are their inputs, two segments
    for divisor in (0, 6):
        hs = [[G.random_array(rng, c, dtype) for _ in range(6)] for c in (20_011, 4097)]
        ds = [[G.dev(h, j % 4) for j, h in enumerate(seg)] for seg in hs]
        rows = [([d[0].data_ptr() for d in seg], [d[0].data_ptr() for d in seg], seg[0][0].numel()) for seg in ds]
        ring_abi.fold_to_all_rows(rows, 6, 6, divisor, code, None)
        G.sync()
        for seg_h, seg_d in zip(hs, ds):
            want = _fold_reference(seg_h, divisor, dtype)
            for j, d in enumerate(seg_d):
                G.assert_same_bits(G.host(d[0]), want, "in place, rank %d /%d" % (j, divisor))
    x, _ = G.dev(np.ones(8, dtype=dtype), 0)
    with pytest.raises(ring_abi.RingError):
        ring_abi.fold_to_all_rows([([x.data_ptr()] * 129, [x.data_ptr()] * 129, 8)], 129, 129, 0, code, None)
    with pytest.raises(ring_abi.RingError):
        ring_abi.fold_to_all_rows([([None], [x.data_ptr()], 8)], 1, 1, 0, code, None)


def test_fold_and_average_on_special_float_values():
    """Denormals, signed zeros, infinities, NaN, the largest finite value: the
    fold, the add-and-divide row and the divided scatter give numpy's bits
    (denormal results of the division included; NaNs only have to be NaNs)."""
    sp = special_f32()
    pairs = np.array([(a, b) for a in sp for b in sp], dtype=np.float32)          # every pair of specials
    a, b = pairs[:, 0].copy(), pairs[:, 1].copy()
    c = np.resize(np.array([1e-38, -1e-38, 3e-39, 1.0, -0.0, 7e37], dtype=np.float32), a.size)
    for divisor in (0, 3, 8):
        da, db, dc = G.dev(a, 1), G.dev(b, 2), G.dev(c, 3)
        out, _ = G.dev(np.zeros(a.size, dtype=np.float32), 1)
        ring_abi.fold_rows([(out.data_ptr(), [da[0].data_ptr(), db[0].data_ptr(), dc[0].data_ptr()], a.size)], 3,
                           divisor, ring_abi.F32, None)
        G.sync()
        G.assert_same_bits(G.host(out), _fold_reference([a, b, c], divisor, np.float32), "fold of specials /%d" % divisor)
        if divisor:
            out2, _ = G.dev(np.zeros(a.size, dtype=np.float32), 2)
            ring_abi.apply_rows_avg([(out2.data_ptr(), da[0].data_ptr(), db[0].data_ptr(), a.size)], None, divisor,
                                    ring_abi.F32, None)
            G.sync()
            with np.errstate(all="ignore"):
                want = ((b + a).astype(np.float32) / np.float32(divisor)).astype(np.float32)
            G.assert_same_bits(G.host(out2), want, "add-and-divide of specials /%d" % divisor)
            t, _ = G.dev(np.zeros(a.size, dtype=np.float32), 3)
            plan = ring_abi.FusionPlan([t.data_ptr()], [a.size], ring_abi.F32)
            plan.scatter(ring_abi.make_spans([(0, a.size, da[0].data_ptr(), None)]), divisor, None)
            G.sync()
            with np.errstate(all="ignore"):
                G.assert_same_bits(G.host(t), (a / np.float32(divisor)).astype(np.float32), "scatter of specials /%d" % divisor)
            plan.close()


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fold_and_copy_rows_in_one_call(dtype):
    """Fold rows (divided) and plain copy rows (never divided) of one call; more
    source pointers and rows than one launch's table holds."""
    rng = np.random.default_rng(123)
    code = G.NP2ABI[np.dtype(dtype)]
    for m, fold_counts, copy_counts, divisor in ((8, [20_003], [5000, 7, 0, 9001, 4096, 33, 12_345], 8),
                                                 (100, [700, 1300, 5], [int(c) for c in rng.integers(0, 2000, 45)], 0),
                                                 (3, [], [10, 20], 4), (2, [9], [], 2)):
        keep, fold, copies, checks = [], [], [], []
        for k, c in enumerate(fold_counts):
            hs = [G.random_array(rng, c, dtype) for _ in range(m)]
            ds = [G.dev(h, (k + j) % 4) for j, h in enumerate(hs)]
            dst, base = G.dev(np.zeros(c, dtype=dtype), (k + 1) % 4)
            keep += [ds, base]
            fold.append((dst.data_ptr(), [d[0].data_ptr() for d in ds], c))
            checks.append((dst, _fold_reference(hs, divisor, dtype), "fold row %d" % k))
        for k, c in enumerate(copy_counts):
            h = G.random_array(rng, c, dtype)
            d, b1 = G.dev(h, k % 4)
            dst, b2 = G.dev(np.zeros(c, dtype=dtype), (k + 3) % 4)
            keep += [b1, b2]
            copies.append((dst.data_ptr() if c else None, d.data_ptr() if c else None, c))
            checks.append((dst, h, "copy row %d" % k))
        ring_abi.fold_and_copy_rows(fold, m, divisor, copies, code, None)
        G.sync()
        for dst, want, what in checks:
            G.assert_same_bits(G.host(dst), want, "%s (m=%d, /%d)" % (what, m, divisor))
    x, _ = G.dev(np.ones(8, dtype=dtype), 0)
    L = ring_abi.lib()
    bad = (ring_abi.Row * 1)()
    bad[0].dst, bad[0].a, bad[0].b, bad[0].count = x.data_ptr(), x.data_ptr(), x.data_ptr(), 8      # an add row
    assert L.ring_fold_and_copy_rows(None, 0, 1, 0, bad, 1, code, None) == 2      # RING_ERR_ARGUMENT


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_scale_is_tf_div(dtype):
    """allreduce(average=True) divides with tf.div (__init__.py:160-164): true
    division for float32, floor division for integers."""
    rng = np.random.default_rng(9)
    for n in (1, 2, 3, 6, 7, 8, 13, 64):
        for count, off in ((0, 0), (1, 0), (5, 1), (4099, 3), (300_001, 2)):
            x = G.random_array(rng, count, dtype, wide=True)
            if dtype == np.float32 and count > 100:
                x[:14] = special_f32()
            dx, keep = G.dev(x, off)
            ring_abi.scale(G.NP2ABI[np.dtype(dtype)], dx.data_ptr(), count, n, None)
            G.sync()
            with np.errstate(all="ignore"):
                want = x / np.float32(n) if dtype == np.float32 else x // dtype(n)
            G.assert_same_bits(G.host(dx), want.astype(dtype), "scale %s /%d n=%d" % (dtype.__name__, n, count))
            assert np.all(G.host(keep[:off]) == 0) and np.all(G.host(keep[off + count:]) == 0)


def _fusion_roundtrip(counts, dtype, rng, offsets=None, divisors=(6,)):
    code = G.NP2ABI[np.dtype(dtype)]
    hosts, devs, keep = [], [], []
    for j, c in enumerate(counts):
        h = G.random_array(rng, c, dtype)
        d, base = G.dev(h, (offsets[j] if offsets else int(rng.integers(0, 4))))
        hosts.append(h)
        devs.append(d)
        keep.append(base)
    plan = ring_abi.FusionPlan([d.data_ptr() if c else None for d, c in zip(devs, counts)], counts, code)
    total = sum(counts)
    assert plan.elements == total
    import torch
    fused = torch.zeros(total + 8, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda")
    plan.pack(fused.data_ptr(), None)
    G.sync()
    want = np.concatenate(hosts) if hosts else np.empty(0, dtype=dtype)
    G.assert_same_bits(G.host(fused)[:total], want, "pack")
    assert not G.host(fused)[total:].any()
    # unpack different data into zeroed tensors
    new = G.random_array(rng, total, dtype)
    fused[:total].copy_(torch.from_numpy(new))
    for base in keep:
        base.zero_()
    plan.unpack(fused.data_ptr(), None)
    G.sync()
    at = 0
    for j, (d, base, c) in enumerate(zip(devs, keep, counts)):
        G.assert_same_bits(G.host(d), new[at:at + c], "unpack tensor %d" % j)
        assert int(torch.count_nonzero(base)) == int(np.count_nonzero(new[at:at + c]))  # nothing outside
        at += c
    # unpack with the average folded in: tf.div by the number of ranks
    if np.dtype(dtype) != np.float32 and total:
        new[: total // 2] = -np.abs(new[: total // 2])               # negative values with remainders: floored
        fused[:total].copy_(torch.from_numpy(new))
    for divisor in divisors:
        for base in keep:
            base.zero_()
        plan.unpack_scaled(fused.data_ptr(), divisor, None)
        G.sync()
        with np.errstate(all="ignore"):
            want = new / np.float32(divisor) if np.dtype(dtype) == np.float32 else new // np.dtype(dtype).type(divisor)
        at = 0
        for j, (d, c) in enumerate(zip(devs, counts)):
            G.assert_same_bits(G.host(d), want[at:at + c].astype(dtype), "unpack_scaled /%d tensor %d" % (divisor, j))
            at += c
    plan.close()


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fusion_pack_unpack(dtype):
    rng = np.random.default_rng(21)
    _fusion_roundtrip([int(np.prod(s)) for s in G.resnet50_shapes()], dtype, rng)
    _fusion_roundtrip([], dtype, rng)
    _fusion_roundtrip([0, 0], dtype, rng)
    _fusion_roundtrip([1], dtype, rng)
    _fusion_roundtrip([5, 0, 4096, 1, 0, 3, 8191, 2], dtype, rng)
    # thousands of tiny tensors inside one tile: more than the LDS table holds
    _fusion_roundtrip([int(c) for c in rng.integers(0, 4, 3000)], dtype, rng)
    _fusion_roundtrip([int(c) for c in rng.integers(1, 200, 700)], dtype, rng)


@pytest.mark.parametrize("dtype", G.DTYPES)
@pytest.mark.parametrize("phased", [1, -1, 0])
def test_fusion_unpack_with_the_payload_in_registers(dtype, phased):
    """The unpack as one read phase and one write phase of the chip (every lane
    holds its share of the fused buffer in registers; rounds whose tile meets
    several tensors are stored lane by lane after a search of the offset
    table), forced on for every set it can take, left to the launcher (which
    takes it from 1 MiB, as two workgroups per CU up to 75 MiB and as one
    beyond) and off: the same bytes in the tensors and nothing outside them,
    with no divisor, with powers of two and with 6 and 3 (float32 divides by
    them in the form as two workgroups per CU; the integers and the larger
    float32 sets must leave them to the tiles), tensor ends that cut 16-byte
    groups, hundreds of tiny tensors, as many tensors as its table holds
    (1024) and one more, and a buffer of exactly and of just over the 112
    rounds a lane has registers for."""
    import torch
    rng = np.random.default_rng(51 + phased)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    vec = 16 // np.dtype(dtype).itemsize
    full = cus * 256 * 112 * vec                                     # elements of 112 rounds
    ring_abi.set_option("phased_copy", phased)
    try:
        _fusion_roundtrip([int(np.prod(s)) for s in G.resnet50_shapes()], dtype, rng, divisors=(8, 6))
        _fusion_roundtrip([5, 0, 4096, 1, 0, 3, 8191, 2, 70_001], dtype, rng, divisors=(1, 2, 6, 1024))
        _fusion_roundtrip([1], dtype, rng, divisors=(4,))
        _fusion_roundtrip([3, 2_000_003, 1, 1, 7, 999_999], dtype, rng, divisors=(8,))
        _fusion_roundtrip([int(c) for c in rng.integers(1, 200, 500)], dtype, rng, divisors=(4, 3))
        _fusion_roundtrip([int(c) for c in rng.integers(0, 9000, 512)], dtype, rng, divisors=(16,))
        _fusion_roundtrip([int(c) for c in rng.integers(1, 300, 1024)], dtype, rng, divisors=(8,))  # all its table holds
        _fusion_roundtrip([int(c) for c in rng.integers(1, 300, 1025)], dtype, rng, divisors=(8,))  # one too many
        if np.dtype(dtype).itemsize == 4:
            switch = cus * 300 * 1024 // 4                                                           # elements at the change of form
            _fusion_roundtrip([switch - 7, 7], dtype, rng, divisors=(2,))                           # two workgroups per CU, 38 rounds
            _fusion_roundtrip([switch - 7, 7 + 1024], dtype, rng, divisors=(2,))                    # one per CU
            _fusion_roundtrip([full - 5, 5], dtype, rng, divisors=(8,))                             # all the registers
            _fusion_roundtrip([full - 5, 5 + vec], dtype, rng, divisors=(8,))                       # a 113th round
    finally:
        ring_abi.set_option("phased_copy", -1)


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_fusion_gather_and_scatter_spans(dtype):
    """Spans of the fused element space: gather = tensors (+ incoming) into a
    linear buffer, scatter = incoming (/ divisor) into the tensors; spans that
    start and end inside tensors, cover many tiny tensors, leave gaps; against
    numpy on the concatenation."""
    import torch
    rng = np.random.default_rng(31)
    code = G.NP2ABI[np.dtype(dtype)]
    tdt = G.NP2TORCH[np.dtype(dtype)]
    for counts in ([int(np.prod(s)) for s in G.resnet50_shapes()][:40], [5, 0, 4096, 1, 0, 3, 8191, 2, 70_001],
                   [int(c) for c in rng.integers(0, 4, 3000)] + [10_000], [int(c) for c in rng.integers(1, 200, 700)]):
        hosts = [G.random_array(rng, c, dtype) for c in counts]
        devs = [G.dev(h, int(rng.integers(0, 4))) for h in hosts]
        plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(devs, counts)], counts, code)
        total = sum(counts)
        flat = np.concatenate(hosts)
        # 5 spans with gaps, boundaries anywhere
        cuts = sorted(int(c) for c in rng.integers(0, total + 1, 10))
        spans = [(cuts[2 * k], cuts[2 * k + 1] - cuts[2 * k]) for k in range(5)]
        incoming = [G.random_array(rng, c, dtype) for _, c in spans]
        d_in = [G.dev(x, k % 4) for k, x in enumerate(incoming)]
        d_out = [G.dev(np.zeros(c, dtype=dtype), (k + 1) % 4) for k, (_, c) in enumerate(spans)]
        with_in = [k % 2 == 0 for k in range(5)]                     # every other span is a plain pack
        ring_abi_spans = ring_abi.make_spans(
            [(b, c, d_in[k][0].data_ptr() if (with_in[k] and c) else None, d_out[k][0].data_ptr() if c else None)
             for k, (b, c) in enumerate(spans)])
        plan.gather(ring_abi_spans, None)
        G.sync()
        for k, (b, c) in enumerate(spans):
            with np.errstate(all="ignore"):
                want = (flat[b:b + c] + incoming[k]).astype(dtype) if with_in[k] else flat[b:b + c]
            G.assert_same_bits(G.host(d_out[k][0]), want, "gather span %d [%d,+%d)" % (k, b, c))
        for d, h in zip(devs, hosts):                               # gather never writes the tensors
            G.assert_same_bits(G.host(d[0]), h, "tensor after gather")
        for divisor in (0, 6):
            for d, h in zip(devs, hosts):
                d[0].copy_(torch.from_numpy(h))
            plan.scatter(ring_abi.make_spans([(b, c, d_in[k][0].data_ptr() if c else None, None)
                                              for k, (b, c) in enumerate(spans)]), divisor, None)
            G.sync()
            want = flat.copy()
            for k, (b, c) in enumerate(spans):
                with np.errstate(all="ignore"):
                    x = incoming[k]
                    if divisor:
                        x = (x / np.float32(divisor) if dtype == np.float32 else x // dtype(divisor)).astype(dtype)
                want[b:b + c] = x
            got = np.concatenate([G.host(d[0]) for d in devs]) if devs else np.empty(0, dtype=dtype)
            G.assert_same_bits(got, want, "scatter /%d" % divisor)
        # spans out of order, overlapping or beyond the plan are refused
        if total > 10:
            a = d_in[0][0].data_ptr()
            for bad in ([(5, 3, a, a), (2, 2, a, a)], [(0, 6, a, a), (5, 3, a, a)], [(total - 1, 2, a, a)]):
                with pytest.raises(ring_abi.RingError):
                    plan.gather(ring_abi.make_spans(bad), None)
            with pytest.raises(ring_abi.RingError):
                plan.scatter(ring_abi.make_spans([(0, 4, None, None)]), 0, None)
        plan.close()


@pytest.mark.parametrize("dtype", G.DTYPES)
def test_scatter_of_segments_received_in_place(dtype):
    """Finished segments that lie in one buffer, each at its own offset (received in
    place), are scattered by the unpack of that buffer, in registers where the
    unpack would be; segments in slots of their own, a gap, or a buffer that is not
    16-byte aligned take the tiles. Same tensors either way, against numpy on the
    concatenation: segment ends that cut 16-byte groups, the full ResNet-50 set at
    N=8 with the divide, a divisor the registers do not take."""
    import torch
    rng = np.random.default_rng(47)
    code = G.NP2ABI[np.dtype(dtype)]
    tdt = G.NP2TORCH[np.dtype(dtype)]
    esz = np.dtype(dtype).itemsize
    resnet = [int(np.prod(s)) for s in G.resnet50_shapes()]
    cases = [(resnet, 8, 8), (resnet[:60], 6, 0), ([100_003, 1, 2, 50_001, 0, 4096, 3, 1], 5, 2),
             ([7, 300_017, 64, 64, 99_991], 3, 4), (resnet[:100], 7, 6)]
    for counts, n, divisor in cases:
        total = sum(counts)
        hosts = [G.random_array(rng, c, dtype) for c in counts]
        if dtype != np.float32:
            for h in hosts:
                h[: h.size // 2] = -np.abs(h[: h.size // 2])              # negative values for the floor division
        devs = [G.dev(h, int(rng.integers(0, 4))) for h in hosts]
        plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(devs, counts)], counts, code)
        sizes, starts = ring_abi.segment_table(total, n)
        incoming = [G.random_array(rng, c, dtype) for c in sizes]
        want = np.concatenate(incoming)
        if divisor:
            with np.errstate(all="ignore"):
                want = (want / np.float32(divisor) if dtype == np.float32 else want // dtype(divisor)).astype(dtype)
        unpack_form = ring_abi.describe_unpack_launch(total, sum(1 for c in counts if c), code, divisor, 256)

        def form_of(spans):
            form = ctypes.c_int(-1)
            ring_abi.check(ring_abi.lib().ring_describe_scatter_launch(plan._h, spans[0], spans[1], divisor, 256,
                                                                        ctypes.byref(form)), "describe")
            return form.value

        def run(pointers, what, expect_form):
            spans = ring_abi.make_spans([(starts[g], sizes[g], pointers[g], None) for g in range(n)])
            assert form_of(spans) == expect_form, (what, form_of(spans), expect_form)
            for d in devs:
                d[0].zero_()
            plan.scatter(spans, divisor, None)
            G.sync()
            got = np.concatenate([G.host(d[0]) for d in devs])
            G.assert_same_bits(got, want, "%s: %d elements in %d tensors, %d segments, /%d" % (what, total, len(counts), n, divisor))

        buffer = torch.from_numpy(np.concatenate(incoming)).cuda()
        run([buffer.data_ptr() + starts[g] * esz for g in range(n)], "received in place", unpack_form)
        shifted = torch.zeros(total + 8, dtype=tdt, device="cuda")
        shifted[1:total + 1].copy_(buffer)
        run([shifted.data_ptr() + (starts[g] + 1) * esz for g in range(n)], "in place in a buffer an element off 16 bytes",
            ring_abi.FORM_TILES)
        slots = [G.dev(x, starts[g] % 32, pad=40) for g, x in enumerate(incoming)]
        run([s[0].data_ptr() for s in slots], "slots of their own", ring_abi.FORM_TILES)
        if n > 2:
            # a gap: the second piece is left out, and its elements keep their values
            spans = ring_abi.make_spans([(starts[g], sizes[g], buffer.data_ptr() + starts[g] * esz, None)
                                         for g in range(n) if g != 1])
            assert form_of(spans) == ring_abi.FORM_TILES
            for d, h in zip(devs, hosts):
                d[0].copy_(torch.from_numpy(h))
            plan.scatter(spans, divisor, None)
            G.sync()
            expect = want.copy()
            expect[starts[1]:starts[1] + sizes[1]] = np.concatenate(hosts)[starts[1]:starts[1] + sizes[1]]
            G.assert_same_bits(np.concatenate([G.host(d[0]) for d in devs]), expect, "a gap in the pieces")
        plan.close()


def test_fusion_errors():
    L = ring_abi.lib()
    h = ctypes.c_void_p()
    p = (ctypes.c_void_p * 1)(None)
    c = (ctypes.c_size_t * 1)(4)
    assert L.ring_fusion_plan_create(p, c, 1, 0, ctypes.byref(h)) == 2      # null tensor with a size
    assert L.ring_fusion_plan_create(p, c, 1, 9, ctypes.byref(h)) == 1      # bad dtype
    assert L.ring_fusion_plan_destroy(None) == 0
