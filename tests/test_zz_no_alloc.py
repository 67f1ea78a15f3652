"""The allocation-free pack / unpack entry point (ring_fusion_run_static):
its offset table lives in a static device array instead of a plan's own
allocation. Checked bit for bit against the plan-based entry points
(ring_fusion_pack / ring_fusion_unpack / ring_fusion_unpack_scaled), on calls
in a row that reuse the array, the later ones with smaller inputs."""
import numpy as np
import pytest
import torch

from gpu_util import DTYPES, NP2ABI, NP2TORCH, assert_same_bits, host, random_array, require_gpu, resnet50_shapes, sync
from mpi_collectives import ring_abi

pytestmark = pytest.mark.gpu


def _tensor_set(rng, counts, dtype):
    """Device tensors at varying element offsets inside their allocations."""
    keep, views = [], []
    for j, c in enumerate(counts):
        base = torch.zeros(c + 8, dtype=NP2TORCH[np.dtype(dtype)], device="cuda")
        off = j % 4
        view = base[off:off + c]
        if c:
            view.copy_(torch.from_numpy(random_array(rng, c, dtype)))
        keep.append(base)
        views.append(view)
    return views, keep


def _check_pack_and_unpack(counts, dtype, divisor, seed):
    rng = np.random.default_rng(seed)
    code = NP2ABI[np.dtype(dtype)]
    tdt = NP2TORCH[np.dtype(dtype)]
    views, _keep = _tensor_set(rng, counts, dtype)
    ptrs = [v.data_ptr() if v.numel() else 0 for v in views]
    total = int(sum(counts))
    stream = ring_abi.stream_create()
    try:
        plan = ring_abi.FusionPlan(ptrs, counts, code)
        want_fused = torch.full((total + 4,), 7, dtype=tdt, device="cuda")
        got_fused = torch.full((total + 4,), 7, dtype=tdt, device="cuda")
        sync()
        plan.pack(want_fused.data_ptr(), stream)
        ring_abi.fusion_run_static(False, ptrs, counts, code, got_fused.data_ptr(), 0, stream)
        ring_abi.stream_synchronize(stream)
        assert_same_bits(host(got_fused), host(want_fused), "static pack vs plan pack")
        want_np = np.concatenate([host(v) for v in views]) if total else np.zeros(0, dtype)
        assert_same_bits(host(got_fused)[:total], want_np, "static pack vs concatenation")

        # unpack the packed buffer into two fresh tensor sets, one per entry point
        outs_a, _ka = _tensor_set(rng, counts, dtype)
        outs_b, _kb = _tensor_set(rng, counts, dtype)
        pa = [v.data_ptr() if v.numel() else 0 for v in outs_a]
        pb = [v.data_ptr() if v.numel() else 0 for v in outs_b]
        plan_a = ring_abi.FusionPlan(pa, counts, code)
        sync()
        if divisor:
            plan_a.unpack_scaled(want_fused.data_ptr(), divisor, stream)
        else:
            plan_a.unpack(want_fused.data_ptr(), stream)
        ring_abi.fusion_run_static(True, pb, counts, code, want_fused.data_ptr(), divisor, stream)
        ring_abi.stream_synchronize(stream)
        for j, (a, b) in enumerate(zip(outs_a, outs_b)):
            assert_same_bits(host(b), host(a), "static unpack vs plan unpack, tensor %d" % j)
        for j, (v, base) in enumerate(zip(outs_b, _kb)):   # nothing outside the tensors was written
            off = j % 4
            pad = torch.cat([base[:off], base[off + v.numel():]])
            assert not bool(pad.any()), "static unpack wrote outside tensor %d" % j
        plan.close()
        plan_a.close()
    finally:
        ring_abi.stream_destroy(stream)


def test_two_calls_in_a_row_second_smaller():
    """The ResNet-50 set (161 tensors, 6240 tiles), then a much smaller set on the
    same array: stale entries of the first call must not reach the second."""
    require_gpu()
    big = [int(np.prod(s)) for s in resnet50_shapes()]
    _check_pack_and_unpack(big, np.float32, 8, seed=1)
    _check_pack_and_unpack([5, 0, 4099, 1, 64, 0, 3], np.float32, 0, seed=2)
    _check_pack_and_unpack([17], np.float32, 3, seed=3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_types_and_divisors(dtype):
    require_gpu()
    rng = np.random.default_rng(11)
    counts = [int(c) for c in rng.integers(0, 9000, 300)] + [1_000_003, 2, 70_001]
    _check_pack_and_unpack(counts, dtype, 6, seed=4)
    _check_pack_and_unpack(counts[:130], dtype, 0, seed=5)       # more than one table chunk, then fewer tensors
    _check_pack_and_unpack([3] * 1024, dtype, 0, seed=6)         # the tensor limit itself


def test_limits_and_arguments():
    require_gpu()
    buf = torch.zeros(4096, device="cuda")
    small = torch.zeros(8, device="cuda")
    # 1025 non-empty tensors: refused, nothing launched
    with pytest.raises(ring_abi.RingError) as e:
        ring_abi.fusion_run_static(False, [small.data_ptr()] * 1025, [1] * 1025, ring_abi.F32, buf.data_ptr(), 0, None)
    assert e.value.status == 5 and "static device table" in str(e.value)
    # more than 65536 tiles (the pointers are never dereferenced: the call is refused first)
    with pytest.raises(ring_abi.RingError) as e:
        ring_abi.fusion_run_static(False, [small.data_ptr()], [65536 * 4096 + 1], ring_abi.F32, buf.data_ptr(), 0, None)
    assert e.value.status == 5
    with pytest.raises(ring_abi.RingError) as e:      # a divisor makes no sense for a pack
        ring_abi.fusion_run_static(False, [small.data_ptr()], [8], ring_abi.F32, buf.data_ptr(), 2, None)
    assert e.value.status == 2
    with pytest.raises(ring_abi.RingError) as e:      # fused buffer must be 16-byte aligned
        ring_abi.fusion_run_static(False, [small.data_ptr()], [8], ring_abi.F32, buf.data_ptr() + 4, 0, None)
    assert e.value.status == 2
    with pytest.raises(ring_abi.RingError) as e:
        ring_abi.fusion_run_static(False, [small.data_ptr()], [8], 9, buf.data_ptr(), 0, None)
    assert e.value.status == 1
    # empty inputs do nothing
    ring_abi.fusion_run_static(False, [], [], ring_abi.F32, 0, 0, None)
    ring_abi.fusion_run_static(True, [0, 0], [0, 0], ring_abi.I64, 0, 4, None)
    sync()


def test_calls_on_different_streams_are_ordered_and_nothing_is_allocated():
    """Two streams take turns on the one array with no synchronisation in between: every
    call's stream waits (on the device) for the call before it, so a table is never rewritten
    under a running pack. And the property the entry point exists for: free device memory is
    the same after warmed-up calls as before them."""
    require_gpu()
    rng = np.random.default_rng(21)
    big = [int(np.prod(s)) for s in resnet50_shapes()]
    small = [int(c) for c in rng.integers(1, 3000, 200)]
    sets = []
    for counts in (big, small):
        views, keep = _tensor_set(rng, counts, np.float32)
        ptrs = [v.data_ptr() for v in views]
        want = torch.cat([v.reshape(-1) for v in views])
        sets.append((counts, ptrs, want, keep))
    streams = [ring_abi.stream_create(), ring_abi.stream_create()]
    outs = [[torch.zeros(int(sum(c)), device="cuda") for _ in range(6)] for c, _, _, _ in sets]
    try:
        # warm-up: the array's address and the event exist from here on
        for which, (counts, ptrs, _w, _k) in enumerate(sets):
            ring_abi.fusion_run_static(False, ptrs, counts, ring_abi.F32, outs[which][0].data_ptr(), 0, streams[which])
        for s in streams:
            ring_abi.stream_synchronize(s)
        sync()
        free_before = torch.cuda.mem_get_info()[0]
        for i in range(6):
            for which, (counts, ptrs, _w, _k) in enumerate(sets):
                ring_abi.fusion_run_static(False, ptrs, counts, ring_abi.F32, outs[which][i].data_ptr(), 0, streams[which])
        for s in streams:
            ring_abi.stream_synchronize(s)
        assert torch.cuda.mem_get_info()[0] == free_before, "a call allocated or freed device memory"
        for which, (_c, _p, want, _k) in enumerate(sets):
            for i in range(6):
                assert torch.equal(outs[which][i], want), "pack %d of set %d, calls interleaved on two streams" % (i, which)
    finally:
        for s in streams:
            ring_abi.stream_destroy(s)
