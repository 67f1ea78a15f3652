#!/usr/bin/env python3
"""Times one data-parallel step's gradient allreduce through the op layer.

Every virtual rank submits the 161 gradients of a ResNet-50 (25,557,032
float32) with mpi.allreduce, as the reference's DistributedOptimizer does
(tensorflow/contrib/mpi_collectives/__init__.py:195-205: one MPIAllreduce per
gradient), and session.run() completes them. Compared: one ring per gradient
(the reference's behaviour; there each op also waits for a coordinator tick of
at least 1 ms, mpi_ops.cc:635), the coordinator's tensor fusion, each of them
also with the gradients of a rank submitted by one call (mpi.allreduce_batch)
and with the nodes built once and run every step (mpi.prepare_allreduce_batch,
what DistributedOptimizer.compute_gradients does), and a single pre-packed
tensor. All ranks live on one GPU, so a ring step is one launch for
all ranks.

    python tensorflow-allreduce_amd/examples/bench_op_layer.py [--ranks 8] [--steps 5]
"""
import argparse
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch  # noqa: E402

import mpi_collectives as mpi  # noqa: E402


def resnet50_counts():
    counts = [7 * 7 * 3 * 64, 64, 64]
    cin = 64
    for width, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            counts += [cin * width, width, width, 9 * width * width, width, width,
                       width * 4 * width, 4 * width, 4 * width]
            if b == 0:
                counts += [cin * 4 * width, 4 * width, 4 * width]
            cin = 4 * width
    return counts + [2048 * 1000, 1000]


def step(session, grads, average=True, batch=False, prepared=None):
    """One step: every rank submits all its gradients, then the session runs."""
    t0 = time.perf_counter()
    handles = []
    if prepared is not None:
        for b in prepared:
            handles.append(b.submit())
    for r, gs in enumerate(grads if prepared is None else []):
        with session.as_rank(r):
            if batch:
                handles.append(mpi.allreduce_batch(gs, average=average))
            else:
                handles.append([mpi.allreduce(g, average=average) for g in gs])
    t1 = time.perf_counter()
    session.run()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    return t1 - t0, t2 - t1


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--steps", type=int, default=5)
    args = ap.parse_args()
    counts = resnet50_counts()
    total = sum(counts)
    gen = torch.Generator(device="cuda").manual_seed(0)
    grads = [[torch.randn(c, device="cuda", generator=gen) * 1e-3 for c in counts] for _ in range(args.ranks)]
    packed = [[torch.cat(gs)] for gs in grads]
    print("%d ranks x %d gradients, %d float32 (%.1f MB) per rank" % (args.ranks, len(counts), total, total * 4 / 1e6))
    for label, kwargs, data, batch in (
            ("one ring per gradient", {}, grads, False),
            ("one ring per gradient, submitted as a batch", {}, grads, True),
            ("one ring per gradient, nodes built once", {}, grads, "prepared"),
            ("coordinator fusion (128 MiB buffer per rank)", {"fusion_threshold": 128 << 20}, grads, False),
            ("coordinator fusion, submitted as a batch", {"fusion_threshold": 128 << 20}, grads, True),
            ("coordinator fusion, nodes built once", {"fusion_threshold": 128 << 20}, grads, "prepared"),
            ("one pre-packed tensor", {}, packed, False)):
        with mpi.Session(size=args.ranks, **kwargs) as session:
            prepared = None
            if batch == "prepared":
                prepared = []
                for r, gs in enumerate(data):
                    with session.as_rank(r):
                        prepared.append(mpi.prepare_allreduce_batch(gs))
            step(session, data, batch=batch, prepared=prepared)  # warm-up (fusion plans, allocator)
            submit, run = zip(*[step(session, data, batch=batch, prepared=prepared) for _ in range(args.steps)])
        print("%-46s submit %7.2f ms   run %7.2f ms   total %7.2f ms per step"
              % (label, 1e3 * min(submit), 1e3 * min(run), 1e3 * min(s + r for s, r in zip(submit, run))))


if __name__ == "__main__":
    main()
