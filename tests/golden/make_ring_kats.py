"""Writes tests/golden/ring_kats.json: small known-answer vectors for the ring.

The expected values are produced here by a third evaluation of the reference
schedule (tensorflow/contrib/mpi_collectives/ring.h:136-228), independent of
the C oracle and of the closed form used in the tests: a pure-Python
message-passing simulation, one mailbox per directed link, every add rounded
to binary32 through numpy scalars (or exact Python ints for the integer
types). Inputs are chosen so that the order of additions matters (large
cancelling terms next to small ones), so an oracle that folds in another
order fails on them.

Run from the repository root:  python tests/golden/make_ring_kats.py
"""
import json
import os
from collections import deque

import numpy as np


def split(count, n):
    base, rem = divmod(count, n)
    sizes = [base + (1 if i < rem else 0) for i in range(n)]
    starts = [sum(sizes[:i]) for i in range(n)]
    return sizes, starts


def add(a, b, kind):
    if kind == "f32":
        return np.float32(np.float32(a) + np.float32(b))
    bitsz = 32 if kind == "i32" else 64
    v = (int(a) + int(b)) & ((1 << bitsz) - 1)
    return v - (1 << bitsz) if v >> (bitsz - 1) else v


def simulate(inputs, kind):
    """Every rank's output; ranks advance one ring step at a time."""
    n = len(inputs)
    count = len(inputs[0])
    sizes, starts = split(count, n)
    buf = [list(x) for x in inputs]                   # ring.h:146-148
    link = [deque() for _ in range(n)]                # link[r]: messages to rank r
    for i in range(n - 1):                            # ring.h:183-205
        for r in range(n):
            s = (r - i) % n
            link[(r + 1) % n].append(buf[r][starts[s]:starts[s] + sizes[s]])
        for r in range(n):
            s = (r - i - 1) % n
            temp = link[r].popleft()
            for k in range(sizes[s]):
                buf[r][starts[s] + k] = add(buf[r][starts[s] + k], temp[k], kind)
    for i in range(n - 1):                            # ring.h:211-225
        for r in range(n):
            s = (r - i + 1) % n
            link[(r + 1) % n].append(buf[r][starts[s]:starts[s] + sizes[s]])
        for r in range(n):
            s = (r - i) % n
            buf[r][starts[s]:starts[s] + sizes[s]] = link[r].popleft()
    return buf


def f32_inputs(n, count, seed):
    rng = np.random.default_rng(seed)
    mags = np.array([1e8, 1.0, 3e-5, 7e3, 16777216.0, 0.1], dtype=np.float32)
    out = []
    for r in range(n):
        x = rng.standard_normal(count).astype(np.float32) * mags[rng.integers(0, len(mags), count)]
        out.append([float(v) for v in x])
    # exact cancellations that only one order resolves to a non-zero value
    if count >= 2 and n >= 3:
        out[0][0], out[1][0], out[2][0] = 1e8, 1.0, -1e8
        out[0][1], out[1][1], out[2][1] = 1.0, 1e8, -1e8
    return out


def int_inputs(n, count, seed, kind):
    rng = np.random.default_rng(seed)
    lo, hi = (-2**31, 2**31 - 1) if kind == "i32" else (-2**63, 2**63 - 1)
    out = []
    for r in range(n):
        x = [int(v) for v in rng.integers(-1000, 1001, count)]
        if count:
            x[0] = hi if r % 2 == 0 else lo          # wraps on overflow
        out.append(x)
    return out


def main():
    cases = []
    seed = 100
    for kind in ("f32", "i32", "i64"):
        for n, count in ((1, 5), (2, 7), (3, 3), (3, 10), (4, 2), (4, 9), (6, 19), (8, 8), (8, 37)):
            seed += 1
            ins = f32_inputs(n, count, seed) if kind == "f32" else int_inputs(n, count, seed, kind)
            outs = simulate(ins, kind)
            for r in range(1, n):
                assert [str(v) for v in outs[r]] == [str(v) for v in outs[0]]
            if kind == "f32":
                enc_in = [[int(np.float32(v).view(np.uint32)) for v in x] for x in ins]
                enc_out = [int(np.float32(v).view(np.uint32)) for v in outs[0]]
            else:
                enc_in = ins
                enc_out = [int(v) for v in outs[0]]
            cases.append({"dtype": kind, "n": n, "count": count,
                          "inputs": enc_in, "expected": enc_out})
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "ring_kats.json"), "w") as f:
        json.dump({"note": "f32 values are stored as uint32 bit patterns",
                   "cases": cases}, f)
    print("wrote %d cases" % len(cases))


if __name__ == "__main__":
    main()
