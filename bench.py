#!/usr/bin/env python3
"""Benchmark of the per-rank ring-allreduce data path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the headline configuration): float32 allreduce of one 16,777,216
element (64 MiB) tensor at N=8 virtual ranks. One STEP is the complete
per-rank data path of one virtual rank, as the reference's RingAllreduce
performs it (tensorflow/contrib/mpi_collectives/ring.h:136-228): the in->out
copy, the 7 reduce-scatter accumulates on 2,097,152-element segments and the
7 allgather segment copies, with every incoming segment pre-staged in HBM
(values ~N(0,1), seed = rank). Successive steps rotate over the 8 virtual
ranks, each with its own input, output and staged buffers (1.9 GiB in all),
so no step finds its data in the 256 MB Infinity Cache.

Prints one JSON line. `value` = algorithmic bytes moved per second over the
timed region (copy 2x, accumulate 3x, allgather 2x the element bytes:
427,819,008 B per step). `roofline` is for the dominant kernel, the batched
reduce-scatter accumulate, from HIP events recorded around a sample of its
launches inside the timed region. `cpu_baseline` is the CPU restatement of the
reference ring (oracle/) timed on this machine's host cores on the same
workload; it is a reported baseline, not what the kernels are compared to.
"""
import argparse
import ctypes
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tensorflow-allreduce_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

N_RANKS = 8
COUNT = 16 * 1024 * 1024            # float32 elements: 64 MiB
SEG = COUNT // N_RANKS
ESZ = 4
BYTES_COPY = COUNT * ESZ * 2
BYTES_RS = (N_RANKS - 1) * SEG * ESZ * 3
BYTES_AG = (N_RANKS - 1) * SEG * ESZ * 2
BYTES_STEP = BYTES_COPY + BYTES_RS + BYTES_AG           # 427,819,008
BYTES_STEP_FUSED = BYTES_RS + SEG * ESZ * 2 + BYTES_AG  # copy folded into the accumulate
HBM_PEAK_GBS = 8000.0
SAMPLE_EVERY = 16                   # steps between event-bracketed launches
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "rows_kernel_f32_accumulate_64MiB_n8_pmc.txt")


def cpu_baseline():
    """The CPU restatement of the reference ring on the same workload (64 MiB
    float32, 8 ranks), over real MPI when one is installed, else over the
    in-process mailbox transport. Bounded: 3 warm-ups + 20 repetitions."""
    import numpy as np
    from oracle import oracle
    warm, reps = 3, 20
    cores = N_RANKS
    if oracle.mpirun_path():
        res = oracle.mpi_time(N_RANKS, oracle.F32, COUNT, warm, reps)
        secs, transport = res["secs"], "MPI point-to-point (%s), one process per rank" % os.path.basename(
            os.path.dirname(os.path.dirname(oracle.mpirun_path())))
    else:
        ins = [np.random.default_rng(1234 + r).uniform(-1, 1, COUNT).astype(np.float32) for r in range(N_RANKS)]
        secs, _ = oracle.time_allreduce_threads(ins, warm, reps)
        transport = "in-process mailbox transport, one thread per rank"
    med = statistics.median(secs)
    out = {
        "value": round(BYTES_STEP / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
        "ms_per_allreduce": round(med * 1e3, 3),
        "sample": "%d timed RingAllreduce calls (after %d warm-ups) of the same 64 MiB float32 tensor at %d "
                  "ranks on %d of %d host cores, %s; per-rank algorithmic bytes / median time of the slowest "
                  "rank; RingAllreduce only (no coordinator tick, no TensorFlow dispatch)"
                  % (reps, warm, N_RANKS, cores, os.cpu_count() or 0, transport),
    }
    # the reference's own CPU-runnable case: 1,048,576 float32 at 2 ranks
    try:
        if oracle.mpirun_path():
            s2 = oracle.mpi_time(2, oracle.F32, 1_048_576, 5, 50)["secs"]
        else:
            small = [np.random.default_rng(1234 + r).uniform(-1, 1, 1_048_576).astype(np.float32) for r in range(2)]
            s2, _ = oracle.time_allreduce_threads(small, 5, 50)
        out["np2_1Mi_float32"] = {"GB/s": round(18_874_368 / statistics.median(s2) / 1e9, 3),
                                  "ms_per_allreduce": round(statistics.median(s2) * 1e3, 4), "cores": 2}
    except Exception as e:   # the small case is extra information only
        out["np2_1Mi_float32"] = {"error": str(e)}
    return out


def measured_traffic():
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3
    counter summary (FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known
    size), or None when no such summary exists."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, re.M)
    return float(m.group(1)) if m else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures the per-rank data path on ONE GPU (the ring's N ranks are virtual); "
                 "--gpus %d is not supported" % args.gpus)

    import torch
    from mpi_collectives import _plugin, ring_abi
    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X; no GPU is visible")
    L = _plugin.load_library('libmpi_collectives.so', ['MPIAllreduce', 'MPIAllgather'])
    ring_abi.lib()

    # ---- synthetic data: per virtual rank, its tensor and what its left neighbour sends
    sets = []
    for r in range(N_RANKS):
        gen = torch.Generator(device="cuda").manual_seed(r)
        inp = torch.randn(COUNT, device="cuda", generator=gen)
        out = torch.empty(COUNT, device="cuda")
        left = torch.Generator(device="cuda").manual_seed(1000 + (r - 1) % N_RANKS)
        rs = torch.randn(N_RANKS - 1, SEG, device="cuda", generator=left)
        ag = torch.randn(N_RANKS - 1, SEG, device="cuda", generator=left)
        rs_ptrs = (ctypes.c_void_p * (N_RANKS - 1))(*[rs[i].data_ptr() for i in range(N_RANKS - 1)])
        ag_ptrs = (ctypes.c_void_p * (N_RANKS - 1))(*[ag[i].data_ptr() for i in range(N_RANKS - 1)])
        rs_steps = ring_abi.make_steps(
            [(ring_abi.schedule(ring_abi.PHASE_REDUCE_SCATTER, N_RANKS, r, i)[1] * SEG, rs[i].data_ptr(), SEG)
             for i in range(N_RANKS - 1)])
        ag_steps = ring_abi.make_steps(
            [(ring_abi.schedule(ring_abi.PHASE_ALLGATHER, N_RANKS, r, i)[1] * SEG, ag[i].data_ptr(), SEG)
             for i in range(N_RANKS - 1)])
        sets.append(dict(r=r, inp=inp, out=out, rs=rs, ag=ag, rs_ptrs=rs_ptrs, ag_ptrs=ag_ptrs,
                         rs_steps=rs_steps, ag_steps=ag_steps))
    torch.cuda.synchronize()

    # the dedicated stream every ring kernel is launched on (CudaStreamForMPI)
    stream = ring_abi.stream_create()
    R = ring_abi.lib()

    def step(k, fused=False, sample=None):
        """The per-rank data path of virtual rank k % 8. With `sample`, the three
        launches are issued one by one with events around the accumulate."""
        s = sets[k % N_RANKS]
        if sample is None:
            rc = L.mpic_ring_allreduce_prestaged(N_RANKS, s["r"], _plugin.DT_FLOAT, s["inp"].data_ptr(),
                                                 s["out"].data_ptr(), COUNT, s["rs_ptrs"], s["ag_ptrs"], stream,
                                                 3 if fused else 1)
            if rc != 0:
                raise RuntimeError("mpic_ring_allreduce_prestaged failed: %s" % L.mpic_last_error().decode())
            return
        # the same three launches through the C ABI, each carrying its own pair of
        # HIP events in the dispatch (on the stream the kernels run on)
        e = event_pool.pop()
        ring_abi.time_next_launch(e[0], e[1])
        ring_abi.check(R.ring_copy_bytes(s["out"].data_ptr(), s["inp"].data_ptr(), COUNT * ESZ, stream), "copy")
        ring_abi.time_next_launch(e[2], e[3])
        ring_abi.check(R.ring_reduce_scatter_steps(s["out"].data_ptr(), s["rs_steps"][0], s["rs_steps"][1],
                                                   ring_abi.F32, stream), "reduce-scatter")
        ring_abi.time_next_launch(e[4], e[5])
        ring_abi.check(R.ring_allgather_steps(s["out"].data_ptr(), s["ag_steps"][0], s["ag_steps"][1],
                                              ring_abi.F32, stream), "allgather")
        sample.append(e)

    # events are created before the timed region: creating them inside it would
    # let the queue drain and the sampled launches start on an idle GPU
    event_pool = [[ring_abi.event_create() for _ in range(6)] for _ in range(args.steps // SAMPLE_EVERY + 1)]

    def timed(steps, warmup, fused=False, with_samples=False):
        for k in range(warmup):
            step(k, fused)
        ring_abi.stream_synchronize(stream)
        torch.cuda.synchronize()
        samples = [] if with_samples else None
        t0 = time.perf_counter()
        for k in range(steps):
            if with_samples and k % SAMPLE_EVERY == SAMPLE_EVERY // 2:
                step(k, fused, samples)
            else:
                step(k, fused)
        ring_abi.stream_synchronize(stream)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, samples

    elapsed, samples = timed(args.steps, args.warmup, with_samples=True)
    ms_per_step = elapsed / args.steps * 1e3
    value = BYTES_STEP * args.steps / elapsed / 1e9

    def phase_us(i):
        ts = [ring_abi.event_elapsed_us(e[2 * i], e[2 * i + 1]) for e in samples]
        return statistics.mean(ts) if ts else float("nan")

    copy_us, rs_us, ag_us = phase_us(0), phase_us(1), phase_us(2)
    achieved = BYTES_RS / (rs_us * 1e-6) / 1e9 if samples else None

    # the same job with the copy folded into the accumulate (fewer bytes, same result)
    fused_elapsed, _ = timed(args.steps, min(args.warmup, 50), fused=True)

    # sanity: the last step's output is what the schedule says (copy, accumulate, overwrite)
    s = sets[(args.steps - 1) % N_RANKS]
    owned = (s["r"] + 1) % N_RANKS
    want = s["inp"][owned * SEG:(owned + 1) * SEG] + s["rs"][N_RANKS - 2]
    ok = torch.equal(s["out"][owned * SEG:(owned + 1) * SEG], want)
    for i in range(N_RANKS - 1):
        seg = ring_abi.schedule(ring_abi.PHASE_ALLGATHER, N_RANKS, s["r"], i)[1]
        ok = ok and torch.equal(s["out"][seg * SEG:(seg + 1) * SEG], s["ag"][i])
    if not ok:
        sys.exit("bench.py: the output of the timed path is wrong; refusing to report a number")

    result = {
        "metric": "per-rank ring allreduce GB/s & % of HBM peak, 64 MiB fp32, N=8 virtual ranks",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "float32 ring allreduce of one 16,777,216-element (64 MiB) tensor, N=8 virtual ranks: "
                        "in->out copy + 7 reduce-scatter accumulates + 7 allgather copies on 2,097,152-element "
                        "segments per step, peers pre-staged in HBM, buffers rotated over 8 virtual ranks (cold)",
            "bytes_per_step": BYTES_STEP,
            "launches_per_step": 3,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": {
            "bound": "hbm",
            "kernel": "rows_kernel<float, kAdd> (batched reduce-scatter accumulate, 7 x 2,097,152 elements)",
            "achieved": round(achieved, 1) if achieved else None,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4) if achieved else None,
            "traffic": measured_traffic(),
            "algorithmic_bytes_per_launch": BYTES_RS,
            "avg_launch_us": round(rs_us, 3),
            "launches_timed": len(samples),
        },
        "phases_us": {
            "copy_64MiB": round(copy_us, 3), "reduce_scatter": round(rs_us, 3), "allgather": round(ag_us, 3),
            "copy_GBps": round(BYTES_COPY / copy_us / 1e3, 1), "reduce_scatter_GBps": round(BYTES_RS / rs_us / 1e3, 1),
            "allgather_GBps": round(BYTES_AG / ag_us / 1e3, 1),
            "note": "HIP events carried by each launch of every %dth step of the timed region" % SAMPLE_EVERY,
        },
        "fused_copy": {
            "ms_per_step": round(fused_elapsed / args.steps * 1e3, 5),
            "bytes_per_step": BYTES_STEP_FUSED,
            "GBps": round(BYTES_STEP_FUSED * args.steps / fused_elapsed / 1e9, 1),
            "launches_per_step": 2,
            "note": "same allreduce with the in->out copy folded into the accumulate (out = in + received)",
        },
    }
    if not args.no_cpu_baseline:
        try:
            result["cpu_baseline"] = cpu_baseline()
        except Exception as e:
            result["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port",
                                      "sample": "failed: %s" % e}
    ring_abi.stream_destroy(stream)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
