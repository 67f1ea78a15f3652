"""Helpers shared by the GPU parity tests: device buffers at chosen element
offsets (to break 16-byte alignment the way ragged ring segments do), and the
loaded C ABI. torch is only the allocator here."""
import numpy as np
import torch

from mpi_collectives import ring_abi

NP2ABI = {np.dtype(np.float32): ring_abi.F32, np.dtype(np.int32): ring_abi.I32,
          np.dtype(np.int64): ring_abi.I64}
NP2TORCH = {np.dtype(np.float32): torch.float32, np.dtype(np.int32): torch.int32,
            np.dtype(np.int64): torch.int64}
DTYPES = [np.float32, np.int32, np.int64]


def require_gpu():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    ring_abi.lib()


def dev(array, offset=0, pad=8):
    """Copy a 1-D numpy array to the GPU, `offset` elements into a 256-byte
    aligned allocation. Returns (view tensor, keep-alive base)."""
    array = np.ascontiguousarray(array).reshape(-1)
    base = torch.zeros(array.size + offset + pad, dtype=NP2TORCH[array.dtype], device="cuda")
    view = base[offset:offset + array.size]
    if array.size:
        view.copy_(torch.from_numpy(array))
    return view, base


def host(t):
    return t.detach().cpu().numpy()


def random_array(rng, count, dtype, wide=False):
    if np.dtype(dtype) == np.float32:
        scale = 10.0 ** rng.integers(-3, 4, count) if wide else 1.0
        return (rng.standard_normal(count) * scale).astype(np.float32)
    if wide:
        info = np.iinfo(dtype)
        return rng.integers(info.min, info.max, count, dtype=dtype, endpoint=True)
    return rng.integers(-1000, 1001, count).astype(dtype)


def sync():
    torch.cuda.synchronize()


def assert_same_bits(got, want, what=""):
    """Bit-exact, except that NaNs only have to be NaNs (payloads differ
    between x86 and the GPU and the reference does not define them)."""
    got = np.ascontiguousarray(got).reshape(-1)
    want = np.ascontiguousarray(want).reshape(-1)
    assert got.dtype == want.dtype and got.size == want.size, what
    view = {4: np.uint32, 8: np.uint64}[got.dtype.itemsize]
    if got.dtype == np.float32:
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan), what
        ok = np.array_equal(got.view(view)[~nan], want.view(view)[~nan])
    else:
        ok = np.array_equal(got.view(view), want.view(view))
    if not ok:
        bad = np.flatnonzero(got.view(view) != want.view(view))
        raise AssertionError("%s: %d of %d elements differ, first at %d: got %r want %r"
                             % (what, bad.size, got.size, bad[0], got[bad[0]], want[bad[0]]))


def resnet50_shapes():
    """The 161 trainable tensors of ResNet-50 v1, in layer order."""
    shapes = [(7, 7, 3, 64), (64,), (64,)]
    cin = 64
    for width, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            shapes += [(1, 1, cin, width), (width,), (width,),
                       (3, 3, width, width), (width,), (width,),
                       (1, 1, width, 4 * width), (4 * width,), (4 * width,)]
            if b == 0:
                shapes += [(1, 1, cin, 4 * width), (4 * width,), (4 * width,)]
            cin = 4 * width
    shapes += [(2048, 1000), (1000,)]
    return shapes
