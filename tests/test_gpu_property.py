"""Property tests on the GPU (hypothesis, derandomised): random ring sizes,
element counts, element types, buffer misalignments and step-table shapes,
always compared bit for bit with the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch
from hypothesis import HealthCheck, given, settings, strategies as st

import gpu_util as G
from gpu_util import ring_abi
from mpi_collectives import _plugin

pytestmark = pytest.mark.gpu

COMMON = dict(deadline=None, derandomize=True, suppress_health_check=list(HealthCheck))
DT = {np.dtype(np.float32): _plugin.DT_FLOAT, np.dtype(np.int32): _plugin.DT_INT32,
      np.dtype(np.int64): _plugin.DT_INT64}
counts = st.one_of(st.integers(0, 40), st.integers(0, 70_000), st.sampled_from([4095, 4096, 4097, 8191, 65_536]))


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    G.require_gpu()


@settings(max_examples=60, **COMMON)
@given(n=st.integers(1, 9), count=counts, dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31),
       offs=st.lists(st.integers(0, 3), min_size=2, max_size=2), divisor=st.sampled_from([0, 0, 1, 2, 3, 7, 8, 64]), fuse=st.booleans(),
       direct=st.booleans())
def test_all_ranks_ring_equals_oracle(oracle, n, count, dtype, seed, offs, divisor, fuse, direct):
    """Sum, or (divisor > 0) the average folded into the last accumulate:
    tf.div of the oracle's sum."""
    ins = [G.random_array(np.random.default_rng(seed + r), count, dtype, wide=True) for r in range(n)]
    want = oracle.ring_allreduce_lockstep(ins)
    if divisor:
        with np.errstate(all="ignore"):
            want = [(w / np.float32(divisor) if dtype == np.float32 else w // dtype(divisor)).astype(dtype) for w in want]
    L = _plugin.load_library()
    dins, douts, keep = [], [], []
    for r in range(n):
        a, ka = G.dev(ins[r], offs[0])
        b, kb = G.dev(np.zeros(count, dtype=dtype), offs[1])
        dins.append(a)
        douts.append(b)
        keep += [ka, kb]
    pin = (ctypes.c_void_p * n)(*[t.data_ptr() if count else None for t in dins])
    pout = (ctypes.c_void_p * n)(*[t.data_ptr() if count else None for t in douts])
    rc = L.mpic_ring_allreduce_all_ranks(n, DT[np.dtype(dtype)], pin, pout, count,
                                         torch.cuda.current_stream().cuda_stream, 1 | (2 if fuse else 0) | (4 if direct else 0) | (divisor << 8))
    assert rc == 0, L.mpic_last_error()
    torch.cuda.synchronize()
    for r in range(n):
        G.assert_same_bits(G.host(douts[r]), want[r],
                           "n=%d count=%d %s rank %d /%d fuse=%s direct=%s" % (n, count, dtype.__name__, r, divisor, fuse, direct))


@settings(max_examples=40, **COMMON)
@given(n=st.integers(2, 9), count=counts, dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31),
       r_pick=st.integers(0, 8), flags=st.sampled_from([0, 1, 3]))
def test_prestaged_rank_equals_oracle(oracle, n, count, dtype, seed, r_pick, flags):
    r = r_pick % n
    ins = [G.random_array(np.random.default_rng(seed + k), count, dtype, wide=True) for k in range(n)]
    outs, rs, ag = oracle.ring_allreduce(ins, tap=True)
    sizes, _ = ring_abi.segment_table(count, n)
    L = _plugin.load_library()
    din, _k1 = G.dev(ins[r], seed % 4)
    dout, _k2 = G.dev(np.zeros(count, dtype=dtype), (seed >> 2) % 4)
    keep = []
    rs_p = (ctypes.c_void_p * (n - 1))()
    ag_p = (ctypes.c_void_p * (n - 1))()
    for i in range(n - 1):
        a, ka = G.dev(rs[r][i][:sizes[ring_abi.schedule(0, n, r, i)[1]]], (seed + i) % 4)
        b, kb = G.dev(ag[r][i][:sizes[ring_abi.schedule(1, n, r, i)[1]]], (seed + 2 * i) % 4)
        keep += [ka, kb]
        rs_p[i] = a.data_ptr() if a.numel() else None
        ag_p[i] = b.data_ptr() if b.numel() else None
    rc = L.mpic_ring_allreduce_prestaged(n, r, DT[np.dtype(dtype)], din.data_ptr() if count else None,
                                         dout.data_ptr() if count else None, count, rs_p, ag_p,
                                         torch.cuda.current_stream().cuda_stream, flags)
    assert rc == 0, L.mpic_last_error()
    torch.cuda.synchronize()
    G.assert_same_bits(G.host(dout), outs[r], "n=%d r=%d count=%d flags=%d" % (n, r, count, flags))


@settings(max_examples=40, **COMMON)
@given(rows=st.lists(st.integers(0, 5000), min_size=1, max_size=12), epr=st.sampled_from([1, 3, 17, 256]),
       dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31), direct=st.booleans(),
       divisor=st.sampled_from([0, 0, 3, 8]))
def test_all_ranks_allgather_is_the_concatenation(rows, epr, dtype, seed, direct, divisor):
    n = len(rows)
    parts = [G.random_array(np.random.default_rng(seed + r), rows[r] * epr, dtype) for r in range(n)]
    want = np.concatenate(parts) if parts else np.empty(0, dtype=dtype)
    if divisor:
        with np.errstate(all="ignore"):
            want = (want / np.float32(divisor) if dtype == np.float32 else want // dtype(divisor)).astype(dtype)
    L = _plugin.load_library()
    dins = [G.dev(p, r % 4) for r, p in enumerate(parts)]
    douts = [G.dev(np.zeros(want.size, dtype=dtype), (r + 1) % 4) for r in range(n)]
    pin = (ctypes.c_void_p * n)(*[d[0].data_ptr() if d[0].numel() else None for d in dins])
    pout = (ctypes.c_void_p * n)(*[d[0].data_ptr() if want.size else None for d in douts])
    rows_c = (ctypes.c_size_t * n)(*rows)
    rc = L.mpic_ring_allgather_all_ranks(n, DT[np.dtype(dtype)], pin, rows_c, epr, pout,
                                         torch.cuda.current_stream().cuda_stream,
                                         1 | (4 if direct else 0) | (divisor << 8))
    assert rc == 0, L.mpic_last_error()
    torch.cuda.synchronize()
    for r in range(n):
        G.assert_same_bits(G.host(douts[r][0]), want,
                           "allgather rows=%r epr=%d rank %d direct=%s /%d" % (rows, epr, r, direct, divisor))


@settings(max_examples=40, **COMMON)
@given(lens=st.lists(st.one_of(st.integers(0, 40), st.integers(0, 300_000), st.sampled_from([65_536, 131_072, 262_147])),
                     min_size=1, max_size=9),
       gaps=st.lists(st.integers(0, 37), min_size=9, max_size=9), dtype=st.sampled_from(G.DTYPES),
       seed=st.integers(0, 2**31), phased=st.sampled_from([1, 1, -1, 0]), shift=st.integers(0, 3))
def test_allgather_copy_rows_of_any_shape_in_every_form(lens, gaps, dtype, seed, phased, shift):
    """The copies of an allgather phase through a step table whose rows have
    any length (empty ones included), start anywhere in the destination and
    read from sources at any element alignment: the form with the payload held
    in registers forced on wherever it fits (one to eight rows; nine fall back
    to tiles), left to the launcher, and off. Every byte outside the rows stays
    as it was."""
    rng = np.random.default_rng(seed)
    starts, at = [], 0
    for ln, gap in zip(lens, gaps):
        at += gap
        starts.append(at)
        at += ln
    buf = G.random_array(rng, at + 7, dtype)
    dbuf, _ = G.dev(buf, shift)
    want = buf.copy()
    rows, keep = [], []
    for ln, st_ in zip(lens, starts):
        src = G.random_array(rng, ln, dtype)
        ds, base = G.dev(src, int(rng.integers(0, 4)))
        keep.append(base)
        rows.append((st_, ds.data_ptr() if ln else None, ln))
        want[st_:st_ + ln] = src
    ring_abi.set_option("phased_copy", phased)
    try:
        steps, k = ring_abi.make_steps(rows)
        ring_abi.allgather_steps(dbuf.data_ptr(), steps, k, G.NP2ABI[np.dtype(dtype)], None)
        G.sync()
    finally:
        ring_abi.set_option("phased_copy", -1)
    G.assert_same_bits(G.host(dbuf), want, "rows %r at %r phased=%d" % (lens, starts, phased))


@settings(max_examples=30, **COMMON)
@given(sizes=st.lists(st.integers(0, 9000), min_size=0, max_size=40), dtype=st.sampled_from(G.DTYPES),
       seed=st.integers(0, 2**31), divisor=st.one_of(st.integers(1, 9), st.sampled_from([2, 4, 8, 64])),
       phased=st.sampled_from([-1, 1, 1]))
def test_fusion_pack_unpack_roundtrip(sizes, dtype, seed, divisor, phased):
    """pack, then unpack and divide, as tiles and (phased = 1) with the fused
    buffer held in registers between one read phase and one write phase, the
    form that takes no divisor but a power of two."""
    rng = np.random.default_rng(seed)
    hosts = [G.random_array(rng, c, dtype, wide=True) for c in sizes]
    devs = [G.dev(h, int(rng.integers(0, 4))) for h in hosts]
    plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(devs, sizes)], sizes,
                               G.NP2ABI[np.dtype(dtype)])
    total = sum(sizes)
    fused = torch.zeros(total + 4, dtype=G.NP2TORCH[np.dtype(dtype)], device="cuda")
    plan.pack(fused.data_ptr(), None)
    torch.cuda.synchronize()
    want = np.concatenate(hosts) if hosts else np.empty(0, dtype=dtype)
    G.assert_same_bits(G.host(fused)[:total], want, "pack")
    for d in devs:
        d[1].zero_()
    ring_abi.set_option("phased_copy", phased)
    try:
        plan.unpack_scaled(fused.data_ptr(), divisor, None)
        torch.cuda.synchronize()
    finally:
        ring_abi.set_option("phased_copy", -1)
    with np.errstate(all="ignore"):
        scaled = want / np.float32(divisor) if dtype == np.float32 else want // dtype(divisor)
    at = 0
    for d, c in zip(devs, sizes):
        G.assert_same_bits(G.host(d[0]), scaled[at:at + c].astype(dtype), "unpack_scaled")
        at += c
    plan.close()


@settings(max_examples=25, **COMMON)
@given(counts=st.lists(st.one_of(st.integers(0, 6), st.sampled_from([1023, 4095, 4096, 4097, 8192, 12_289]),
                                 st.integers(0, 20_000)), min_size=1, max_size=30),
       dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31), divisor=st.sampled_from([0, 5]),
       n_spans=st.integers(1, 6))
def test_fusion_spans_with_boundaries_on_tiles_and_tensors(counts, dtype, seed, divisor, n_spans):
    """Gather and scatter over spans whose ends fall on tensor boundaries, on
    multiples of the kernel's tile, one element either side of them, or
    anywhere; against numpy on the concatenation."""
    rng = np.random.default_rng(seed)
    total = sum(counts)
    hosts = [G.random_array(rng, c, dtype) for c in counts]
    devs = [G.dev(h, int(rng.integers(0, 4))) for h in hosts]
    plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(devs, counts)], counts,
                               G.NP2ABI[np.dtype(dtype)])
    flat = np.concatenate(hosts) if hosts else np.empty(0, dtype=dtype)
    tile = 4096 if np.dtype(dtype).itemsize == 4 else 2048
    marks = sorted({0, total} | {int(x) for x in np.cumsum(counts)} | set(range(0, total + 1, tile)))
    marks = sorted({min(max(m + d, 0), total) for m in marks for d in (-1, 0, 1)})
    cuts = sorted(int(rng.choice(marks)) if rng.random() < 0.7 else int(rng.integers(0, total + 1))
                  for _ in range(2 * n_spans))
    spans = [(cuts[2 * k], cuts[2 * k + 1] - cuts[2 * k]) for k in range(n_spans)]
    incoming = [G.random_array(rng, c, dtype) for _, c in spans]
    d_in = [G.dev(x, k % 4) for k, x in enumerate(incoming)]
    d_out = [G.dev(np.zeros(c, dtype=dtype), (k + 2) % 4) for k, (_, c) in enumerate(spans)]
    plan.gather(ring_abi.make_spans([(b, c, d_in[k][0].data_ptr() if c and k % 2 == 0 else None,
                                      d_out[k][0].data_ptr() if c else None) for k, (b, c) in enumerate(spans)]), None)
    torch.cuda.synchronize()
    for k, (b, c) in enumerate(spans):
        with np.errstate(all="ignore"):
            want = (flat[b:b + c] + incoming[k]).astype(dtype) if k % 2 == 0 else flat[b:b + c]
        G.assert_same_bits(G.host(d_out[k][0]), want, "gather span %d [%d,+%d) of %d" % (k, b, c, total))
    plan.scatter(ring_abi.make_spans([(b, c, d_in[k][0].data_ptr() if c else None, None)
                                      for k, (b, c) in enumerate(spans)]), divisor, None)
    torch.cuda.synchronize()
    want = flat.copy()
    for k, (b, c) in enumerate(spans):
        x = incoming[k]
        if divisor:
            with np.errstate(all="ignore"):
                x = (x / np.float32(divisor) if dtype == np.float32 else x // dtype(divisor)).astype(dtype)
        want[b:b + c] = x
    got = np.concatenate([G.host(d[0]) for d in devs]) if devs else np.empty(0, dtype=dtype)
    G.assert_same_bits(got, want, "scatter /%d spans %r" % (divisor, spans))
    plan.close()


@settings(max_examples=40, **COMMON)
@given(counts=st.lists(st.one_of(st.integers(0, 6), st.sampled_from([1023, 4095, 4096, 4097, 8192]),
                                 st.integers(0, 20_000)), min_size=1, max_size=24),
       dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31), divisor=st.sampled_from([0, 3, 8]),
       n=st.integers(1, 9), own_pick=st.integers(0, 8), with_others=st.booleans())
def test_fusion_fold_scatter_is_fold_then_scatter(counts, dtype, seed, divisor, n, own_pick, with_others):
    """ring_fusion_fold_scatter on any tensor set and ring size: the owned
    segment of the packed layout folded from n - 1 staged copies and the
    tensors (last), in that order; its sum in the send buffer, sum (/ divisor)
    in the tensors; the other segments scattered (/ divisor) or, without them,
    left untouched. Against numpy on the concatenation."""
    rng = np.random.default_rng(seed)
    total = sum(counts)
    hosts = [G.random_array(rng, c, dtype, wide=True) for c in counts]
    devs = [G.dev(h, int(rng.integers(0, 4))) for h in hosts]
    plan = ring_abi.FusionPlan([d[0].data_ptr() if c else None for d, c in zip(devs, counts)], counts,
                               G.NP2ABI[np.dtype(dtype)])
    flat = np.concatenate(hosts) if hosts else np.empty(0, dtype=dtype)
    sizes, starts = ring_abi.segment_table(total, n)
    own = own_pick % n
    a, b = starts[own], starts[own] + sizes[own]
    staged = [G.random_array(rng, sizes[own], dtype, wide=True) for _ in range(n - 1)]
    d_staged = [G.dev(x, (k + 1) % 4) for k, x in enumerate(staged)]
    with np.errstate(all="ignore"):
        acc = flat[a:b].copy() if n == 1 else staged[0].copy()
        for x in staged[1:]:
            acc = (x + acc).astype(dtype)
        if n > 1:
            acc = (flat[a:b] + acc).astype(dtype)

        def div(x):
            if not divisor:
                return x
            return (x / np.float32(divisor) if dtype == np.float32 else x // dtype(divisor)).astype(dtype)
        want = flat.copy()
        want[a:b] = div(acc)
        finished, keep = [], []
        if with_others:
            for g in range(n):
                if g == own or sizes[g] == 0:
                    continue
                x = G.random_array(rng, sizes[g], dtype, wide=True)
                d = G.dev(x, g % 4)
                keep.append(d)
                finished.append((starts[g], sizes[g], d[0].data_ptr(), None))
                want[starts[g]:starts[g] + sizes[g]] = div(x)
    wire = G.dev(np.zeros(sizes[own], dtype=dtype), 3)
    plan.fold_scatter(a, sizes[own], [d[0].data_ptr() if sizes[own] else d[1].data_ptr() for d in d_staged],
                      wire[0].data_ptr() if sizes[own] else wire[1].data_ptr(), ring_abi.make_spans(finished), divisor, None)
    torch.cuda.synchronize()
    G.assert_same_bits(G.host(wire[0]), acc, "send buffer n=%d own=%d" % (n, own))
    got = np.concatenate([G.host(d[0]) for d in devs]) if devs else np.empty(0, dtype=dtype)
    G.assert_same_bits(got, want, "tensors n=%d own=%d /%d others=%s" % (n, own, divisor, with_others))
    plan.close()


@settings(max_examples=30, **COMMON)
@given(m=st.integers(1, 12), count=counts, dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31),
       divisor=st.sampled_from([0, 0, 2, 7]), in_place=st.integers(-1, 11), n_copies=st.integers(0, 3))
def test_fold_rows_any_source_may_be_the_destination(m, count, dtype, seed, divisor, in_place, n_copies):
    """One fold row whose destination is a fresh buffer or any one of its own
    sources, with copy rows in the same launch; against a numpy fold in the
    same order."""
    rng = np.random.default_rng(seed)
    hs = [G.random_array(rng, count, dtype, wide=True) for _ in range(m)]
    ds = [G.dev(h, int(rng.integers(0, 4))) for h in hs]
    acc = hs[0].copy()
    with np.errstate(all="ignore"):
        for h in hs[1:]:
            acc = (h + acc).astype(dtype)
        if divisor:
            acc = (acc / np.float32(divisor) if dtype == np.float32 else acc // dtype(divisor)).astype(dtype)
    if 0 <= in_place < m:
        dst = ds[in_place][0]
    else:
        dst = G.dev(np.zeros(count, dtype=dtype), int(rng.integers(0, 4)))[0]
    copies_h = [G.random_array(rng, int(rng.integers(0, 5000)), dtype) for _ in range(n_copies)]
    copies_s = [G.dev(h, k % 4) for k, h in enumerate(copies_h)]
    copies_d = [G.dev(np.zeros(h.size, dtype=dtype), (k + 1) % 4) for k, h in enumerate(copies_h)]
    ring_abi.fold_and_copy_rows(
        [(dst.data_ptr() if count else None, [d[0].data_ptr() if count else None for d in ds], count)], m, divisor,
        [(d[0].data_ptr() if h.size else None, s[0].data_ptr() if h.size else None, h.size)
         for d, s, h in zip(copies_d, copies_s, copies_h)], G.NP2ABI[np.dtype(dtype)], None)
    torch.cuda.synchronize()
    G.assert_same_bits(G.host(dst), acc, "fold m=%d count=%d /%d in place %d" % (m, count, divisor, in_place))
    for k, h in enumerate(copies_h):
        G.assert_same_bits(G.host(copies_d[k][0]), h, "copy row %d" % k)
    for k, h in enumerate(hs):                       # the other sources are never written
        if k != in_place:
            G.assert_same_bits(G.host(ds[k][0]), h, "source %d untouched" % k)


@settings(max_examples=30, **COMMON)
@given(n=st.integers(1, 16), sizes=st.lists(st.one_of(st.integers(0, 40), st.integers(0, 9000)), min_size=1, max_size=40),
       dtype=st.sampled_from(G.DTYPES), seed=st.integers(0, 2**31), divisor=st.sampled_from([0, 0, 1, 3, 8]),
       in_place=st.booleans())
def test_fused_allreduce_of_all_ranks_is_the_ring_on_the_packed_buffer(oracle, n, sizes, dtype, seed, divisor, in_place):
    """ring_fusion_allreduce_all on random tensor sets: every tensor of every rank equals
    the oracle's ring over the concatenations, divided as tf.div divides."""
    rng = np.random.default_rng(seed)
    code = G.NP2ABI[np.dtype(dtype)]
    hosts = [[G.random_array(rng, c, dtype) for c in sizes] for _ in range(n)]
    ins = [[G.dev(h, int(rng.integers(0, 4))) for h in hosts[r]] for r in range(n)]
    outs = ins if in_place else [[G.dev(np.zeros(c, dtype=dtype), int(rng.integers(0, 4))) for c in sizes] for _ in range(n)]
    in_plans = [ring_abi.FusionPlan([t[0].data_ptr() if c else None for t, c in zip(ins[r], sizes)], sizes, code) for r in range(n)]
    out_plans = in_plans if in_place else [
        ring_abi.FusionPlan([t[0].data_ptr() if c else None for t, c in zip(outs[r], sizes)], sizes, code) for r in range(n)]
    total = sum(sizes)
    want = oracle.ring_allreduce([np.concatenate(h) for h in hosts])[0] if total else np.empty(0, dtype=dtype)
    if divisor and total:
        with np.errstate(all="ignore"):
            want = (want / np.float32(divisor)).astype(np.float32) if dtype == np.float32 else want // dtype(divisor)
    ring_abi.fusion_allreduce_all(in_plans, out_plans, divisor, None)
    torch.cuda.synchronize()
    for r in range(n):
        at = 0
        for j, c in enumerate(sizes):
            G.assert_same_bits(G.host(outs[r][j][0]), want[at:at + c].astype(dtype),
                               "n=%d sizes=%r /%d in_place=%s rank %d tensor %d" % (n, sizes, divisor, in_place, r, j))
            at += c
    for p in set(in_plans + out_plans):
        p.close()
