"""Shared pytest setup: markers, import paths, the closed-form ring evaluator."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_ROOT = os.path.join(ROOT, "tensorflow-allreduce_amd")
for p in (ROOT, PKG_ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def ring_closed_form(inputs):
    """What every rank holds after the reference ring allreduce, derived from
    the schedule rather than by running it: the element of segment s is the
    left fold x_s, then x_{s+1} + acc, ... x_{s+n-1 mod n} + acc, one rounding
    per add (tensorflow/contrib/mpi_collectives/ring.h:183-205 fixes the
    order; :150-166 the segments)."""
    n = len(inputs)
    flat = [np.ascontiguousarray(x).reshape(-1) for x in inputs]
    count = flat[0].size
    base, rem = divmod(count, n)
    out = np.empty_like(flat[0])
    start = 0
    for s in range(n):
        size = base + (1 if s < rem else 0)
        sl = slice(start, start + size)
        acc = flat[s][sl].copy()
        for k in range(1, n):
            with np.errstate(over="ignore", invalid="ignore"):
                acc = flat[(s + k) % n][sl] + acc
        out[sl] = acc
        start += size
    return out


def bits(a):
    """Integer view of an array, for exact comparison (NaN-safe, -0 != +0)."""
    a = np.ascontiguousarray(a)
    return a.view({4: np.uint32, 8: np.uint64}[a.dtype.itemsize])


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o
