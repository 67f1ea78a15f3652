#!/usr/bin/env python3
"""Benchmark of the per-rank ring-allreduce data path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Default workload (the headline configuration): float32 allreduce of one
16,777,216 element (64 MiB) tensor at N=8 virtual ranks. One STEP is the
complete per-rank data path of one virtual rank, as the reference's
RingAllreduce performs it (tensorflow/contrib/mpi_collectives/ring.h:136-228):
the in->out copy, the 7 reduce-scatter accumulates on 2,097,152-element
segments and the 7 allgather segment copies, with every incoming segment
pre-staged in HBM (values ~N(0,1), seed = rank). Successive steps rotate over
the 8 virtual ranks, each with its own input, output and staged buffers
(1.9 GiB in all), so no step finds its data in the 256 MB Infinity Cache.

Prints one JSON line. `value` = algorithmic bytes moved per second over the
timed region (copy 2x, accumulate 3x, allgather 2x the element bytes:
427,819,008 B per step). `roofline` is for the dominant kernel, the batched
reduce-scatter accumulate, from HIP events that travel in the dispatch of a
sample of its launches inside the timed region. `cpu_baseline` is the CPU
restatement of the reference ring (oracle/) timed on this machine's host cores
on the same workload; it is a reported baseline, not what the kernels are
compared to.

The other workloads (--workload) time the remaining benchmark configurations
the same way; they exist so that their profiles can be reproduced.
"""
import argparse
import gc
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

HBM_PEAK_GBS = 8000.0
FRESH_STAGING = False               # --fresh-staging: see coaligned()
REGIONS = 9                         # wall-clock regions of --steps steps each; ms_per_step is their median
SAMPLE_EVERY = 4                    # steps between launches that carry timing events (sampling pass only)
MIN_SAMPLES = 32                    # timed launches per phase, whatever --steps is
MAX_SAMPLES = 128
COLD_SAMPLES = 32                   # timed launches of the cold-operand accumulate
EXTRA_MIN_STEPS = 200               # the extras (hot, fused_copy, direct_form) run at least this many steps per region
EXTRA_REGIONS = 3
METRIC = "per-rank ring allreduce GB/s & % of HBM peak, 64 MiB fp32, N=8 virtual ranks"
# committed rocprofv3 counter summaries holding a `traffic_bytes_per_launch:` line for a workload's dominant kernel
TRAFFIC_PROFILES = {
    "allreduce_f32_64MiB_n8": "rows_kernel_f32_64MiB_n8_headline.txt",
    "allreduce_i32_10000019_n6": "rows_kernel_i32_10000019_n6.txt",
    "allreduce_i64_10000019_n6": "rows_kernel_i64_10000019_n6.txt",
    "allgather_f32_n16": "rows_kernel_allgather_f32_n16.txt",
    "allreduce_f32_1GiB_n64": "rows_kernel_f32_1GiB_n64.txt",
    "fused_resnet50_n8": "fusion_kernel_resnet50_161_tensors_n8.txt",
    "fused_resnet50_n8_no_passes": "fusion_span_kernel_resnet50_161_tensors_n8_no_passes.txt",
    "fused_resnet50_n8_no_passes_direct": "fusion_direct_kernel_resnet50_161_tensors_n8.txt",
    "allreduce_f32_64MiB_n8_direct": "fold_kernel_f32_64MiB_n8_direct.txt",
    "allreduce_f32_64MiB_all_ranks_n8": "fold_kernel_f32_64MiB_all_ranks_n8.txt",
    "fused_resnet50_all_ranks_n8": "fusion_allreduce_kernel_resnet50_161_tensors_all_ranks_n8.txt",
}


def resnet50_counts():
    """Element counts of the 161 trainable tensors of ResNet-50 v1, in layer
    order: conv kernels, BN gamma/beta after every conv, the 2048x1000 FC."""
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


def coaligned(torch, t, begin_bytes):
    """A copy of the finished segment `t` that lies in its allocation where it would lie in a neighbour's buffer:
    `begin_bytes` mod 128 behind a 128-byte line. The reference receives an allgather segment in place, at
    buffer + starts[segment] (ring.h:211-225), and a virtual rank copies it from the neighbour's buffer at that
    same offset, so the 128-byte lines of the source are the lines of the destination; staged at the start of a
    fresh allocation instead, a ragged segment's source is shifted against its destination and every 1 KiB a
    wave loads straddles one more line (1.5-4.5 % more bytes fetched, measured). --fresh-staging keeps the
    fresh allocations, for comparison. Reduce-scatter arrivals stay at the start of theirs, like the reference's
    temp tensor (ring.h:189-204)."""
    if FRESH_STAGING:
        return t
    esz = t.element_size()
    lead = (begin_bytes % 128) // esz
    room = torch.empty(t.numel() + 128 // esz, dtype=t.dtype, device=t.device)
    view = room[lead: lead + t.numel()]
    view.copy_(t)
    return view


class Workload:
    """A set of device buffers and the launches of one step over them.

    phases: [(name, algorithmic bytes, kernel description)], in launch order;
    `dominant` indexes the phase the roofline is reported for."""
    name = ""
    description = ""
    dtype = "f32"
    phases = ()
    dominant = 0
    nsets = 1

    def launch_step(self, k, stream, fused=False):
        raise NotImplementedError

    def launch_phase(self, k, i, stream):
        raise NotImplementedError

    def check(self, k):
        return True

    step_bytes = None    # algorithmic bytes of one step when it is not the sum of the phases
    step_launches = None  # kernel launches of one step when it is not one per phase

    @property
    def bytes_per_step(self):
        return self.step_bytes if self.step_bytes is not None else sum(p[1] for p in self.phases)


class RingAllreduce(Workload):
    """Per-rank RingAllreduce of a `count`-element tensor at n virtual ranks,
    peers pre-staged: copy, batched reduce-scatter accumulate, batched allgather."""

    def __init__(self, name, np_name, count, n, nsets, what):
        import torch
        from mpi_collectives import _plugin, ring_abi
        self.torch, self.ring_abi, self.plugin = torch, ring_abi, _plugin
        self.L = _plugin.load_library('libmpi_collectives.so', ['MPIAllreduce', 'MPIAllgather'])
        self.R = ring_abi.lib()
        tdt, self.code, self.pdt, self.esz = {
            "f32": (torch.float32, ring_abi.F32, _plugin.DT_FLOAT, 4),
            "i32": (torch.int32, ring_abi.I32, _plugin.DT_INT32, 4),
            "i64": (torch.int64, ring_abi.I64, _plugin.DT_INT64, 8)}[np_name]
        self.name, self.dtype, self.count, self.n, self.nsets = name, np_name, count, n, nsets
        self.sizes, self.starts = ring_abi.segment_table(count, n)
        esz = self.esz
        self.sets = []
        for s in range(nsets):
            r = s % n
            gen = torch.Generator(device="cuda").manual_seed(r)
            left = torch.Generator(device="cuda").manual_seed(1000 + (r - 1) % n)

            def rnd(numel, g):
                if np_name == "f32":
                    return torch.randn(numel, device="cuda", generator=g)
                return torch.randint(-1000, 1001, (numel,), dtype=tdt, device="cuda", generator=g)
            inp, out = rnd(count, gen), torch.empty(count, dtype=tdt, device="cuda")
            rs_seg = [ring_abi.schedule(ring_abi.PHASE_REDUCE_SCATTER, n, r, i)[1] for i in range(n - 1)]
            ag_seg = [ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i)[1] for i in range(n - 1)]
            rs = [rnd(self.sizes[g], left) for g in rs_seg]
            ag = [coaligned(torch, rnd(self.sizes[g], left), self.starts[g] * esz) for g in ag_seg]
            self.sets.append(dict(
                r=r, inp=inp, out=out, rs=rs, ag=ag, rs_seg=rs_seg, ag_seg=ag_seg,
                rs_ptrs=(ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() for t in rs]),
                ag_ptrs=(ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() for t in ag]),
                rs_steps=ring_abi.make_steps([(self.starts[g], t.data_ptr(), self.sizes[g]) for g, t in zip(rs_seg, rs)]),
                ag_steps=ring_abi.make_steps([(self.starts[g], t.data_ptr(), self.sizes[g]) for g, t in zip(ag_seg, ag)])))
        s0 = self.sets[0]
        rs_elems = sum(self.sizes[g] for g in s0["rs_seg"])
        ag_elems = sum(self.sizes[g] for g in s0["ag_seg"])
        tname = {"f32": "float", "i32": "unsigned int", "i64": "unsigned long"}[np_name]
        carrier = "unsigned long" if esz == 8 else "unsigned int"
        self.phases = (
            ("copy", count * esz * 2, "rows_kernel<%s, kCopy> (in->out copy, %d elements)" % (carrier, count)),
            ("reduce_scatter", rs_elems * esz * 3,
             "rows_kernel<%s, kAdd> (batched reduce-scatter accumulate, %d rows, %d elements)" % (tname, n - 1, rs_elems)),
            ("allgather", ag_elems * esz * 2,
             "rows_kernel<%s, kCopy> (batched allgather copies, %d rows, %d elements)" % (carrier, n - 1, ag_elems)))
        self.dominant = 1
        self.fused_bytes = rs_elems * esz * 3 + ag_elems * esz * 2
        self.description = what

    def launch_step(self, k, stream, fused=False):
        s = self.sets[k % self.nsets]
        rc = self.L.mpic_ring_allreduce_prestaged(self.n, s["r"], self.pdt, s["inp"].data_ptr(), s["out"].data_ptr(),
                                                  self.count, s["rs_ptrs"], s["ag_ptrs"], stream, 3 if fused else 1)
        if rc != 0:
            raise RuntimeError("mpic_ring_allreduce_prestaged failed: %s" % self.L.mpic_last_error().decode())

    def launch_phase(self, k, i, stream):
        s, A, R = self.sets[k % self.nsets], self.ring_abi, self.R
        if i == 0:
            A.check(R.ring_copy_bytes(s["out"].data_ptr(), s["inp"].data_ptr(), self.count * self.esz, stream), "copy")
        elif i == 1:
            A.check(R.ring_reduce_scatter_steps(s["out"].data_ptr(), s["rs_steps"][0], s["rs_steps"][1], self.code,
                                                stream), "reduce-scatter")
        else:
            A.check(R.ring_allgather_steps(s["out"].data_ptr(), s["ag_steps"][0], s["ag_steps"][1], self.code,
                                           stream), "allgather")

    def check(self, k):
        """The output of step k is what the schedule says: the owned segment is
        input + last received partial, every other segment the received one."""
        s, torch = self.sets[k % self.nsets], self.torch
        owned = (s["r"] + 1) % self.n
        a, b = self.starts[owned], self.starts[owned] + self.sizes[owned]
        ok = torch.equal(s["out"][a:b], s["inp"][a:b] + s["rs"][self.n - 2])
        for g, t in zip(s["ag_seg"], s["ag"]):
            ok = ok and torch.equal(s["out"][self.starts[g]:self.starts[g] + self.sizes[g]], t)
        return bool(ok)


class RingAllreducePerStep(RingAllreduce):
    """The same allreduce with one launch per ring step, the structure of the
    reference's loop (ring.h:183-225): copy, n-1 accumulates of one segment,
    n-1 copies of one segment, all asynchronous on the stream. The phases timed
    are single launches: the copy, one accumulate, one segment copy."""

    def __init__(self, *args):
        super().__init__(*args)
        self.step_bytes = sum(p[1] for p in self.phases)
        self.step_launches = 2 * self.n - 1
        seg = self.sizes[self.sets[0]["rs_seg"][0]]
        self.phases = (self.phases[0],
                       ("accumulate_one_step", seg * self.esz * 3, "rows_kernel<float, kAdd> (one segment, %d elements)" % seg),
                       ("copy_one_step", seg * self.esz * 2, "rows_kernel<unsigned int, kCopy> (one segment, %d elements)" % seg))

    def launch_step(self, k, stream, fused=False):
        s = self.sets[k % self.nsets]
        rc = self.L.mpic_ring_allreduce_prestaged(self.n, s["r"], self.pdt, s["inp"].data_ptr(), s["out"].data_ptr(),
                                                  self.count, s["rs_ptrs"], s["ag_ptrs"], stream, 0)
        if rc != 0:
            raise RuntimeError("mpic_ring_allreduce_prestaged failed: %s" % self.L.mpic_last_error().decode())

    def launch_phase(self, k, i, stream):
        s, A, R = self.sets[k % self.nsets], self.ring_abi, self.R
        if i == 0:
            return super().launch_phase(k, i, stream)
        # all n-1 launches of the phase, so that a sampled step does a whole step's
        # work; the armed events time the first of them
        for g, t in zip(s["rs_seg"], s["rs"]) if i == 1 else zip(s["ag_seg"], s["ag"]):
            dst = s["out"].data_ptr() + self.starts[g] * self.esz
            if i == 1:
                A.check(R.ring_accumulate(self.code, dst, t.data_ptr(), self.sizes[g], stream), "accumulate")
            else:
                A.check(R.ring_copy_bytes(dst, t.data_ptr(), self.sizes[g] * self.esz, stream), "copy")


class StreamFloors(Workload):
    """What the chip gives ONE direction at the sizes of an allreduce's two copy
    launches, next to the launches themselves: the copy source read and nothing
    written, the copy destination written and nothing read, the in->out copy;
    the same three for the rows of the allgather phase (up to 8 rows: a larger
    ring shows its allgather without the one-directional launches). A copy runs
    no faster than its two directions one after the other, so read-only +
    write-only is the floor of the copy at that size on this chip. Buffers
    rotate as in the allreduce workload; every phase is one launch
    (ring_probe_stream for the one-directional ones), timed by events in its
    dispatch."""

    def __init__(self, name, np_name, count, n, nsets, what):
        self.inner = r = RingAllreduce(name, np_name, count, n, nsets, what)
        self.name, self.dtype, self.count, self.n, self.nsets, self.esz = name, np_name, count, n, nsets, r.esz
        self.ring_abi, self.R = r.ring_abi, r.R
        esz = r.esz
        up = lambda p: (p + 15) & ~15       # the probe wants 16-byte aligned pointers; a ragged start loses < 16 bytes
        self.probe_rows = n - 1 <= 8
        for s in r.sets:
            out = s["out"].data_ptr()
            s["probe_copy"] = [(out, s["inp"].data_ptr(), None, count)]
            s["probe_ag"] = [(up(out + r.starts[g] * esz), up(t.data_ptr()), None, r.sizes[g] - 16 // esz)
                             for g, t in zip(s["ag_seg"], s["ag"])]
        ag_bytes = sum(r.sizes[g] for g in r.sets[0]["ag_seg"]) * esz
        # (what runs, phase of the inner workload or probe mode, rows)
        self.plan = [("probe", 0, "probe_copy"), ("probe", 1, "probe_copy"), ("phase", 0, None)]
        self.phases = [
            ("read_only_copy_source", count * esz, "stream_probe_kernel<read> (1 row, %d bytes)" % (count * esz)),
            ("write_only_copy_destination", count * esz, "stream_probe_kernel<write> (1 row, %d bytes)" % (count * esz)),
            r.phases[0]]
        if self.probe_rows:
            self.plan += [("probe", 0, "probe_ag"), ("probe", 1, "probe_ag")]
            self.phases += [
                ("read_only_allgather_sources", ag_bytes, "stream_probe_kernel<read> (%d rows, %d bytes)" % (n - 1, ag_bytes)),
                ("write_only_allgather_destinations", ag_bytes,
                 "stream_probe_kernel<write> (%d rows, %d bytes)" % (n - 1, ag_bytes))]
        self.plan.append(("phase", 2, None))
        self.phases = tuple(self.phases + [r.phases[2]])
        self.dominant = 2
        self.description = ("one direction at a time against the copy launches of: " + what)

    def launch_phase(self, k, i, stream):
        kind, arg, rows = self.plan[i]
        if kind == "phase":
            self.inner.launch_phase(k, arg, stream)
        else:
            # the probes work on another buffer set than the copies of the same step, so that no copy
            # finds in a cache what a probe has just touched
            s = self.inner.sets[(k + self.nsets // 2) % self.nsets]
            self.ring_abi.probe_stream(s[rows], self.inner.code, arg, stream)

    def launch_step(self, k, stream, fused=False):
        for i in range(len(self.plan)):
            self.launch_phase(k, i, stream)

    def check(self, k):
        s = self.inner.sets[k % self.nsets]
        ok = True
        for g, t in zip(s["ag_seg"], s["ag"]):
            a = self.inner.starts[g]
            ok = ok and self.inner.torch.equal(s["out"][a:a + self.inner.sizes[g]], t)
        return bool(ok)


class RingAllreduceDirect(Workload):
    """The direct form of the same allreduce for one rank of n: the n-1 peers'
    raw copies of the rank's own segment lie in staging slots (as peers pushing
    over their own links would leave them) and are folded with the rank's copy
    in ring order in ONE pass; the other n-1 segments arrive finished and are
    copied in. Same result as the ring, bit for bit."""

    def __init__(self, name, count, n, nsets, what):
        import torch
        from mpi_collectives import _plugin, ring_abi
        self.torch, self.ring_abi = torch, ring_abi
        self.L = _plugin.load_library('libmpi_collectives.so', ['MPIAllreduce', 'MPIAllgather'])
        self.R = ring_abi.lib()
        self.pdt = _plugin.DT_FLOAT
        self.name, self.dtype, self.count, self.n, self.nsets, self.esz = name, "f32", count, n, nsets, 4
        self.sizes, self.starts = ring_abi.segment_table(count, n)
        self.sets = []
        for s in range(nsets):
            r = s % n
            own = (r + 1) % n
            gen = torch.Generator(device="cuda").manual_seed(r)
            inp = torch.randn(count, device="cuda", generator=gen)
            out = torch.empty(count, device="cuda")
            peers = [torch.randn(self.sizes[own], device="cuda", generator=gen) for _ in range(n - 1)]
            ag_seg = [ring_abi.schedule(ring_abi.PHASE_ALLGATHER, n, r, i)[1] for i in range(n - 1)]
            ag = [torch.randn(self.sizes[g], device="cuda", generator=gen) for g in ag_seg]
            srcs = [t.data_ptr() for t in peers] + [inp.data_ptr() + self.starts[own] * 4]
            self.sets.append(dict(
                r=r, own=own, inp=inp, out=out, peers=peers, ag=ag, ag_seg=ag_seg, srcs=srcs,
                peer_ptrs=(ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() for t in peers]),
                ag_ptrs=(ctypes.c_void_p * max(n - 1, 1))(*[t.data_ptr() for t in ag]),
                ag_steps=ring_abi.make_steps([(self.starts[g], t.data_ptr(), self.sizes[g]) for g, t in zip(ag_seg, ag)])))
        seg = self.sizes[self.sets[0]["own"]]
        ag_elems = sum(self.sizes[g] for g in self.sets[0]["ag_seg"])
        self.phases = (
            ("fold_and_copies", seg * 4 * (n + 1) + ag_elems * 8,
             "fold_kernel<float> (1 row folding %d sources into %d elements + %d copy rows, %d elements)"
             % (n, seg, n - 1, ag_elems)),)
        self.dominant = 0
        self.description = what

    def launch_step(self, k, stream, fused=False):
        s = self.sets[k % self.nsets]
        rc = self.L.mpic_ring_allreduce_direct_prestaged(self.n, s["r"], self.pdt, s["inp"].data_ptr(),
                                                         s["out"].data_ptr(), self.count, s["peer_ptrs"], s["ag_ptrs"],
                                                         stream, 1)
        if rc != 0:
            raise RuntimeError("mpic_ring_allreduce_direct_prestaged failed: %s" % self.L.mpic_last_error().decode())

    def launch_phase(self, k, i, stream):
        s, A = self.sets[k % self.nsets], self.ring_abi
        own, out = s["own"], s["out"].data_ptr()
        A.fold_and_copy_rows([(out + self.starts[own] * 4, s["srcs"], self.sizes[own])], self.n, 0,
                             [(out + self.starts[g] * 4, t.data_ptr(), self.sizes[g]) for g, t in zip(s["ag_seg"], s["ag"])],
                             A.F32, stream)

    def check(self, k):
        s, torch = self.sets[k % self.nsets], self.torch
        a, b = self.starts[s["own"]], self.starts[s["own"]] + self.sizes[s["own"]]
        acc = s["peers"][0].clone()
        for t in s["peers"][1:]:
            acc = t + acc
        ok = torch.equal(s["out"][a:b], s["inp"][a:b] + acc)
        for g, t in zip(s["ag_seg"], s["ag"]):
            ok = ok and torch.equal(s["out"][self.starts[g]:self.starts[g] + self.sizes[g]], t)
        return bool(ok)


class FusedResnet50(Workload):
    """161 float32 gradients packed into one fusion buffer, ring-reduced in
    place at N=8 (peers pre-staged), unpacked with the average's divide."""

    def __init__(self, nsets=4):
        import torch
        from mpi_collectives import ring_abi
        self.torch, self.ring_abi, self.R = torch, ring_abi, ring_abi.lib()
        self.name, self.dtype, self.n, self.nsets = "fused_resnet50_n8", "f32", 8, nsets
        counts = resnet50_counts()
        total = sum(counts)
        assert len(counts) == 161 and total == 25_557_032
        self.total = total
        sizes, starts = ring_abi.segment_table(total, 8)
        self.sets = []
        for s in range(nsets):
            r = s % 8
            gen = torch.Generator(device="cuda").manual_seed(r)
            grads = [torch.randn(c, device="cuda", generator=gen) * 1e-3 for c in counts]
            plan = ring_abi.FusionPlan([g.data_ptr() for g in grads], counts, ring_abi.F32)
            fused = torch.empty(total, device="cuda")
            rs_seg = [ring_abi.schedule(0, 8, r, i)[1] for i in range(7)]
            ag_seg = [ring_abi.schedule(1, 8, r, i)[1] for i in range(7)]
            rs = [torch.randn(sizes[g], device="cuda", generator=gen) * 1e-3 for g in rs_seg]
            ag = [coaligned(torch, torch.randn(sizes[g], device="cuda", generator=gen) * 1e-3, starts[g] * 4) for g in ag_seg]
            self.sets.append(dict(grads=grads, plan=plan, fused=fused, rs=rs, ag=ag, r=r, rs_seg=rs_seg, ag_seg=ag_seg,
                                  rs_steps=ring_abi.make_steps([(starts[g], t.data_ptr(), sizes[g]) for g, t in zip(rs_seg, rs)]),
                                  ag_steps=ring_abi.make_steps([(starts[g], t.data_ptr(), sizes[g]) for g, t in zip(ag_seg, ag)])))
        self.counts, self.sizes, self.starts = counts, sizes, starts
        seg = total // 8
        self.phases = (
            ("pack", total * 8, "fusion_kernel<unsigned int, pack> (161 tensors, 25,557,032 elements)"),
            ("reduce_scatter", 7 * seg * 12, "rows_kernel<float, kAdd> (7 rows x 3,194,629 elements, in place)"),
            ("allgather", 7 * seg * 8, "rows_kernel<unsigned int, kCopy> (7 rows x 3,194,629 elements)"),
            ("unpack_scaled", total * 8, "unpack_phased_kernel<float, divide> (161 tensors, /8; fusion_kernel<float, unpack, divide> with phased_copy=0)"))
        self.dominant = 1
        self.description = ("tensor-fusion allreduce of a ResNet-50 v1 gradient set: 161 float32 tensors "
                            "(25,557,032 elements, values ~N(0,1e-3)) packed into one fusion buffer, ring-reduced in "
                            "place at N=8 virtual ranks (7 accumulates + 7 copies on 3,194,629-element segments, "
                            "peers pre-staged), unpacked with the divide by 8; 4 launches per step")

    def launch_phase(self, k, i, stream):
        s, A, R = self.sets[k % self.nsets], self.ring_abi, self.R
        if i == 0:
            s["plan"].pack(s["fused"].data_ptr(), stream)
        elif i == 1:
            A.check(R.ring_reduce_scatter_steps(s["fused"].data_ptr(), s["rs_steps"][0], s["rs_steps"][1], A.F32, stream), "rs")
        elif i == 2:
            A.check(R.ring_allgather_steps(s["fused"].data_ptr(), s["ag_steps"][0], s["ag_steps"][1], A.F32, stream), "ag")
        else:
            s["plan"].unpack_scaled(s["fused"].data_ptr(), 8, stream)

    def launch_step(self, k, stream, fused=False):
        for i in range(4):
            self.launch_phase(k, i, stream)

    def owned_sum(self, s, packed):
        """The finished owned segment: the rank's own values plus the partial sum
        that arrives at the last reduce-scatter step."""
        own = (s["r"] + 1) % 8
        a, b = self.starts[own], self.starts[own] + self.sizes[own]
        return packed[a:b] + s["rs"][6]

    def check(self, k, stream=None):
        """One more step of the timed path on set k from freshly drawn gradients
        (a step overwrites its own inputs), compared tensor by tensor with what
        the schedule says: the owned segment is the rank's values plus what it
        received last (the fold of the staged copies in the direct form), every
        other segment is the one received in the allgather phase, all divided
        by 8 (one IEEE add and one IEEE divide per element, as torch computes
        them)."""
        s, torch = self.sets[k % self.nsets], self.torch
        gen = torch.Generator(device="cuda").manual_seed(4242 + k)
        for g in s["grads"]:
            g.copy_(torch.randn(g.numel(), device="cuda", generator=gen) * 1e-3)
        packed = torch.cat(s["grads"])
        own = (s["r"] + 1) % 8
        want = torch.empty_like(packed)
        a, b = self.starts[own], self.starts[own] + self.sizes[own]
        want[a:b] = self.owned_sum(s, packed)
        for g, t in zip(s["ag_seg"], s["ag"]):
            want[self.starts[g]:self.starts[g] + self.sizes[g]] = t
        want = want / 8
        torch.cuda.synchronize()
        st = stream if stream is not None else self.ring_abi.stream_create()
        self.launch_step(k, st)
        self.ring_abi.stream_synchronize(st)
        if stream is None:
            self.ring_abi.stream_destroy(st)
        at, ok = 0, True
        for g in s["grads"]:
            ok = ok and torch.equal(g, want[at:at + g.numel()])
            at += g.numel()
        return bool(ok)


class FusedResnet50NoPasses(FusedResnet50):
    """The same fused allreduce without pack and unpack passes: the
    reduce-scatter's accumulates gather their local operand from the 161
    tensors (the segment that is only sent is packed alongside), the finished
    segments scatter straight into the tensors with the divide. Two launches."""

    def __init__(self, nsets=4):
        super().__init__(nsets)
        from mpi_collectives import _plugin
        self.L = _plugin.load_library('libmpi_collectives.so', ['MPIAllreduce', 'MPIAllgather'])
        self.name = "fused_resnet50_n8_no_passes"
        A = self.ring_abi
        sizes, starts = A.segment_table(self.total, 8)
        for s, st in enumerate(self.sets):
            r = s % 8
            rs_seg = [A.schedule(0, 8, r, i)[1] for i in range(7)]
            ag_seg = [A.schedule(1, 8, r, i)[1] for i in range(7)]
            rs_of = {g: t for g, t in zip(rs_seg, st["rs"])}
            ag_of = {g: t for g, t in zip(ag_seg, st["ag"])}
            own, wire = (r + 1) % 8, st["fused"].data_ptr()
            st["r"] = r
            st["rs_ptrs"] = (ctypes.c_void_p * 7)(*[t.data_ptr() for t in st["rs"]])
            st["ag_ptrs"] = (ctypes.c_void_p * 7)(*[t.data_ptr() for t in st["ag"]])
            st["gather"] = A.make_spans([(starts[g], sizes[g], rs_of[g].data_ptr() if g in rs_of else None,
                                          wire + starts[g] * 4) for g in range(8)])
            st["scatter"] = A.make_spans([(starts[g], sizes[g],
                                           wire + starts[g] * 4 if g == own else ag_of[g].data_ptr(), None)
                                          for g in range(8)])
        seg = self.total // 8
        self.phases = (
            ("gather_accumulate", 7 * seg * 12 + seg * 8,
             "fusion_span_kernel<float, gather> (7 segments tensors + received -> wire, 1 segment packed)"),
            ("scatter_scaled", 8 * seg * 8, "fusion_span_kernel<float, scatter, divide> (8 finished segments -> 161 tensors, /8)"))
        self.dominant = 0
        self.description = ("tensor-fusion allreduce of a ResNet-50 v1 gradient set (161 float32 tensors, 25,557,032 "
                            "elements, values ~N(0,1e-3)) at N=8 virtual ranks WITHOUT pack and unpack passes: the 7 "
                            "accumulates read their local operand from the tensors and write the wire buffer, the 8 "
                            "finished segments go straight into the tensors with the divide by 8; 2 launches per step")

    def launch_phase(self, k, i, stream):
        s = self.sets[k % self.nsets]
        if i == 0:
            s["plan"].gather(s["gather"], stream)
        else:
            s["plan"].scatter(s["scatter"], 8, stream)

    def launch_step(self, k, stream, fused=False):
        s = self.sets[k % self.nsets]
        rc = self.L.mpic_ring_allreduce_fused_prestaged(s["plan"]._h, 8, s["r"], s["fused"].data_ptr(), s["rs_ptrs"],
                                                        s["ag_ptrs"], stream, 8 << 8)
        if rc != 0:
            raise RuntimeError("mpic_ring_allreduce_fused_prestaged failed: %s" % self.L.mpic_last_error().decode())


class FusedResnet50NoPassesDirect(FusedResnet50NoPasses):
    """The same without passes in the direct form: the 7 peers' raw copies of the
    owned segment (packed layout) lie in staging slots; ONE launch folds them
    with the rank's own copy, read from the tensors, in ring order, leaves the
    sum in the wire buffer (what the rank sends on) and the quotient in the
    tensors, and scatters the 7 other finished segments into the tensors with
    the divide."""

    def __init__(self, nsets=4):
        super().__init__(nsets)
        self.name = "fused_resnet50_n8_no_passes_direct"
        A, torch = self.ring_abi, self.torch
        sizes, starts = A.segment_table(self.total, 8)
        for st in self.sets:
            own = (st["r"] + 1) % 8
            gen = torch.Generator(device="cuda").manual_seed(77 + st["r"])
            # the slots peers push their raw copies of the owned segment into are the receiver's to place
            st["raw"] = [coaligned(torch, torch.randn(sizes[own], device="cuda", generator=gen) * 1e-3, starts[own] * 4)
                         for _ in range(7)]
            st["raw_ptrs"] = (ctypes.c_void_p * 7)(*[t.data_ptr() for t in st["raw"]])
            st["own"], st["mine"] = own, st["fused"].data_ptr() + starts[own] * 4
            ag_of = {g: t for g, t in zip(st["ag_seg"], st["ag"])}
            st["others"] = A.make_spans([(starts[g], sizes[g], ag_of[g].data_ptr(), None) for g in range(8) if g != own])
        seg = self.total // 8
        self.phases = (
            ("fold_and_scatter", seg * 4 * 10 + 7 * seg * 8,
             "fusion_direct_kernel<float, divide> (owned segment: 7 staged copies + tensors -> wire and tensors/8; "
             "7 finished segments -> tensors/8)"),)
        self.dominant = 0
        self.description = ("tensor-fusion allreduce of a ResNet-50 v1 gradient set (161 float32 tensors, 25,557,032 "
                            "elements) at N=8 virtual ranks, DIRECT form in ONE launch: the owned 3,194,629-element "
                            "segment folded in ring order from the 7 peers' staged raw copies and the tensors (sum to "
                            "the wire buffer, sum/8 into the tensors), the 7 other finished segments scattered into "
                            "the tensors with the divide by 8")

    def owned_sum(self, s, packed):
        """The fold of the 7 staged raw copies and the rank's own copy, in ring order."""
        own = s["own"]
        a, b = self.starts[own], self.starts[own] + self.sizes[own]
        acc = s["raw"][0].clone()
        for t in s["raw"][1:]:
            acc = t + acc
        return packed[a:b] + acc

    def launch_phase(self, k, i, stream):
        s = self.sets[k % self.nsets]
        s["plan"].fold_scatter(self.starts[s["own"]], self.sizes[s["own"]], [t.data_ptr() for t in s["raw"]], s["mine"],
                               s["others"], 8, stream)

    def launch_step(self, k, stream, fused=False):
        s = self.sets[k % self.nsets]
        rc = self.L.mpic_ring_allreduce_fused_prestaged(s["plan"]._h, 8, s["r"], s["fused"].data_ptr(), s["raw_ptrs"],
                                                        s["ag_ptrs"], stream, 4 | (8 << 8))
        if rc != 0:
            raise RuntimeError("mpic_ring_allreduce_fused_prestaged failed: %s" % self.L.mpic_last_error().decode())

    def check(self, k, stream=None):
        """The tensors as the parent checks them, and the wire buffer: the owned
        segment's sum, undivided."""
        if not super().check(k, stream):
            return False
        s, torch = self.sets[k % self.nsets], self.torch
        a, b = self.starts[s["own"]], self.starts[s["own"]] + self.sizes[s["own"]]
        # the tensors now hold sum / 8 and the wire the sum: dividing the wire must give the tensors bit for bit
        return bool(torch.equal(s["fused"][a:b] / 8, torch.cat(s["grads"])[a:b]))


class AllgatherN16(Workload):
    """RingAllgather at N=16: rank i contributes [rows_i, 1024] float32,
    rows_i uniform in [1, 4096] from seed=i; one launch per step gathers the
    own slice and the 15 received segments."""

    def __init__(self, nsets=6):
        import numpy as np
        import torch
        from mpi_collectives import ring_abi
        self.torch, self.ring_abi, self.R = torch, ring_abi, ring_abi.lib()
        self.name, self.dtype, self.n, self.nsets = "allgather_f32_n16", "f32", 16, nsets
        rows = [int(np.random.default_rng(i).integers(1, 4097)) for i in range(16)]
        starts = ring_abi.allgather_table(rows, 1024)
        self.sets = []
        for s in range(nsets):
            r = s % 16
            gen = torch.Generator(device="cuda").manual_seed(r)
            parts = [torch.randn(rows[k] * 1024, device="cuda", generator=gen) for k in range(16)]
            out = torch.empty(sum(rows) * 1024, device="cuda")
            order = [r] + [ring_abi.schedule(ring_abi.PHASE_GATHER, 16, r, i)[1] for i in range(15)]
            steps = ring_abi.make_steps([(starts[g], parts[g].data_ptr(), rows[g] * 1024) for g in order])
            self.sets.append(dict(parts=parts, out=out, steps=steps))
        self.total_rows = sum(rows)
        self.phases = (("gather", sum(rows) * 1024 * 8,
                        "rows_kernel<unsigned int, kCopy> (16 rows of unequal length, %d x 1024 elements)" % sum(rows)),)
        self.description = ("MPIAllgather of variable-first-dim tensors at N=16 virtual ranks: rank i contributes "
                            "[rows_i, 1024] float32 with rows_i uniform in [1,4096] (seed=i, %d rows in all); own slice "
                            "and 15 pre-staged segments gathered in one launch per step" % sum(rows))

    def launch_phase(self, k, i, stream):
        s, A = self.sets[k % self.nsets], self.ring_abi
        A.check(self.R.ring_allgather_steps(s["out"].data_ptr(), s["steps"][0], s["steps"][1], A.F32, stream), "gather")

    def launch_step(self, k, stream, fused=False):
        self.launch_phase(k, 0, stream)

    def check(self, k):
        s = self.sets[k % self.nsets]
        return bool(self.torch.equal(s["out"], self.torch.cat(s["parts"])))


class AllRanksAllreduce(Workload):
    """All n ranks of the ring resident on the GPU (a world of virtual ranks): a
    step is the whole allreduce of all ranks, in the direct form one launch in
    which the owner of every segment folds the n copies in ring order and
    stores the result into every rank's output. With `counts` the ranks hold
    tensor sets and the same launch works on the tensors themselves (what pack,
    ring and unpack of a fused allreduce compute). Averaged (divided by n)."""

    def __init__(self, name, counts, n, nsets, what):
        import torch
        from mpi_collectives import _plugin, ring_abi
        self.torch, self.ring_abi = torch, ring_abi
        self.L = _plugin.load_library('libmpi_collectives.so', ['MPIAllreduce', 'MPIAllgather'])
        self.pdt = _plugin.DT_FLOAT
        self.name, self.dtype, self.n, self.nsets, self.counts = name, "f32", n, nsets, counts
        self.count = total = sum(counts)
        self.fused = len(counts) > 1
        self.sizes, self.starts = ring_abi.segment_table(total, n)
        self.sets = []
        for s in range(nsets):
            gen = torch.Generator(device="cuda").manual_seed(s)
            ins = [torch.randn(total, device="cuda", generator=gen) for _ in range(n)]
            outs = [torch.empty(total, device="cuda") for _ in range(n)]
            d = dict(ins=ins, outs=outs,
                     ip=(ctypes.c_void_p * n)(*[t.data_ptr() for t in ins]),
                     op=(ctypes.c_void_p * n)(*[t.data_ptr() for t in outs]))
            if self.fused:
                # every tensor its own allocation, as gradients are
                d["tin"] = [[t.clone() for t in x.split(counts)] for x in ins]
                d["tout"] = [[torch.empty(c, device="cuda") for c in counts] for _ in range(n)]
                d["in_plans"] = [ring_abi.FusionPlan([t.data_ptr() for t in ts], counts, ring_abi.F32) for ts in d["tin"]]
                d["out_plans"] = [ring_abi.FusionPlan([t.data_ptr() for t in ts], counts, ring_abi.F32) for ts in d["tout"]]
            self.sets.append(d)
        kernel = ("fusion_allreduce_kernel<float> (%d tensors per rank)" % len(counts) if self.fused
                  else "fold_kernel<float> (%d rows of %d sources and %d destinations)" % (n, n, n))
        self.phases = (("fold_to_all", 2 * n * total * 4, kernel),)
        self.dominant = 0
        self.description = what

    def launch_step(self, k, stream, fused=False):
        s = self.sets[k % self.nsets]
        if self.fused:
            self.ring_abi.fusion_allreduce_all(s["in_plans"], s["out_plans"], self.n, stream)
            return
        rc = self.L.mpic_ring_allreduce_all_ranks(self.n, self.pdt, s["ip"], s["op"], self.count, stream,
                                                  7 | (self.n << 8))
        if rc != 0:
            raise RuntimeError("mpic_ring_allreduce_all_ranks failed: %s" % self.L.mpic_last_error().decode())

    def launch_phase(self, k, i, stream):
        self.launch_step(k, stream)

    def check(self, k):
        s, torch, n = self.sets[k % self.nsets], self.torch, self.n
        want = torch.empty(self.count, device="cuda")
        for seg in range(n):
            a, b = self.starts[seg], self.starts[seg] + self.sizes[seg]
            acc = s["ins"][seg][a:b].clone()
            for j in range(1, n):
                acc = s["ins"][(seg + j) % n][a:b] + acc
            want[a:b] = acc / n
        if self.fused:
            return all(torch.equal(torch.cat(ts), want) for ts in s["tout"])
        return all(torch.equal(o, want) for o in s["outs"])


def make_workload(name):
    if name == "allreduce_f32_64MiB_all_ranks_n8":
        return AllRanksAllreduce(name, [16 * 1024 * 1024], 8, 3,
                                 "float32 averaged allreduce of a 64 MiB tensor per rank, all 8 virtual ranks resident: "
                                 "ONE launch, the owner of every segment folds the 8 copies in ring order and stores "
                                 "the result into all 8 outputs (8 reads + 8 writes per element); 3 buffer sets rotated")
    if name == "fused_resnet50_all_ranks_n8":
        return AllRanksAllreduce(name, resnet50_counts(), 8, 2,
                                 "float32 averaged allreduce of the 161 ResNet-50 gradients (25,557,032 elements) of all "
                                 "8 resident virtual ranks: ONE launch on the tensors themselves, every tensor equal to "
                                 "the ring on the packed buffer; 2 buffer sets rotated")
    if name == "allreduce_f32_64MiB_n8":
        return RingAllreduce(name, "f32", 16 * 1024 * 1024, 8, 8,
                             "float32 ring allreduce of one 16,777,216-element (64 MiB) tensor, N=8 virtual ranks: "
                             "in->out copy + 7 reduce-scatter accumulates + 7 allgather copies on 2,097,152-element "
                             "segments per step, peers pre-staged in HBM, buffers rotated over 8 virtual ranks (cold)")
    if name == "allreduce_f32_64MiB_n8_direct":
        return RingAllreduceDirect(name, 16 * 1024 * 1024, 8, 8,
                                   "float32 allreduce of one 64 MiB tensor, N=8 virtual ranks, DIRECT form: the rank's own "
                                   "2,097,152-element segment folded in ring order from the 7 peers' staged raw copies "
                                   "and its own (8 reads, 1 write per element) + 7 copies of finished segments, all in "
                                   "one launch; buffers rotated over 8 virtual ranks")
    if name == "allreduce_f32_1MiB_n8_direct":
        return RingAllreduceDirect(name, 262_144, 8, 8,
                                   "float32 allreduce of one 1 MiB tensor, N=8 virtual ranks, DIRECT form: the launch-bound "
                                   "size in ONE launch per allreduce (fold of the 8 copies of the rank's 128 KiB segment "
                                   "+ 7 copies of finished segments); buffers rotated over 8 virtual ranks")
    if name == "allreduce_f32_64MiB_n8_per_step":
        return RingAllreducePerStep(name, "f32", 16 * 1024 * 1024, 8, 8,
                                    "float32 ring allreduce of one 64 MiB tensor, N=8 virtual ranks, ONE LAUNCH PER RING "
                                    "STEP as in the reference's loop: copy + 7 accumulate launches + 7 copy launches "
                                    "(15 per step), peers pre-staged, buffers rotated over 8 virtual ranks")
    if name in ("allreduce_i32_10000019_n6", "allreduce_i64_10000019_n6"):
        dt = name.split("_")[1]
        return RingAllreduce(name, dt, 10_000_019, 6, 12,
                             "%s ring allreduce of a ragged 10,000,019-element tensor, N=6 virtual ranks (segments "
                             "1,666,670 x5 + 1,666,669): copy + 5 accumulates + 5 copies per step, peers pre-staged, "
                             "12 buffer sets rotated" % {"i32": "int32", "i64": "int64"}[dt])
    if name.startswith("floors_"):
        _, dt, size, ranks = name.split("_")
        count = {"64MiB": 16 * 1024 * 1024, "10000019": 10_000_019, "1GiB": 268_435_456}[size]
        n = int(ranks[1:])
        return StreamFloors(name, dt, count, n, {8: 8, 6: 12, 64: 2}[n],
                            "%s ring allreduce of %d elements at N=%d (in->out copy of %d bytes; allgather copies of %d rows)"
                            % (dt, count, n, count * (8 if dt == "i64" else 4), n - 1))
    if name == "allreduce_f32_1MiB_n8":
        return RingAllreduce(name, "f32", 262_144, 8, 8,
                             "float32 ring allreduce of one 262,144-element (1 MiB) tensor, N=8 virtual ranks: a "
                             "launch-bound step (copy + 7 accumulates + 7 copies on 128 KiB segments, 3 launches), "
                             "peers pre-staged, buffers rotated over 8 virtual ranks")
    if name == "allreduce_f32_1GiB_n64":
        return RingAllreduce(name, "f32", 268_435_456, 64, 2,
                             "float32 ring allreduce of one 268,435,456-element (1 GiB) tensor, N=64 virtual ranks: "
                             "copy + 63 accumulates + 63 copies on 4,194,304-element (16 MiB) segments per step, one "
                             "launch per phase, peers pre-staged, 2 buffer sets (8 GiB) rotated")
    if name == "fused_resnet50_n8":
        return FusedResnet50()
    if name == "fused_resnet50_n8_no_passes":
        return FusedResnet50NoPasses()
    if name == "fused_resnet50_n8_no_passes_direct":
        return FusedResnet50NoPassesDirect()
    if name == "allgather_f32_n16":
        return AllgatherN16()
    raise SystemExit("unknown workload %r" % name)


WORKLOADS = ("allreduce_f32_64MiB_n8", "allreduce_i32_10000019_n6", "allreduce_i64_10000019_n6",
             "fused_resnet50_n8", "allgather_f32_n16", "allreduce_f32_1GiB_n64", "allreduce_f32_64MiB_n8_per_step",
             "allreduce_f32_1MiB_n8", "allreduce_f32_1MiB_n8_direct",
             "allreduce_f32_64MiB_n8_direct", "fused_resnet50_n8_no_passes",
             "fused_resnet50_n8_no_passes_direct", "allreduce_f32_64MiB_all_ranks_n8",
             "fused_resnet50_all_ranks_n8",
             "floors_f32_64MiB_n8", "floors_i32_10000019_n6", "floors_i64_10000019_n6", "floors_f32_1GiB_n64")


def cpu_baseline(w):
    """The CPU restatement of the reference ring on the same allreduce (same
    element type, count and ranks), over real MPI when one is installed, else
    over the in-process mailbox transport. Bounded to a few seconds."""
    import numpy as np
    from oracle import oracle
    code = {"f32": oracle.F32, "i32": oracle.I32, "i64": oracle.I64}[w.dtype]
    n, count = w.n, w.count
    warm, reps = 3, 20
    host_cores = os.cpu_count() or 1
    if n > host_cores or count * w.esz * n * 3 > 24 << 30:
        return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port",
                "sample": "not run: %d ranks of %d bytes do not fit %d host cores / the memory bound" % (
                    n, count * w.esz, host_cores)}
    if oracle.mpirun_path():
        secs = oracle.mpi_time(n, code, count, warm, reps)["secs"]
        transport = "MPICH point-to-point, one process per rank"
    else:
        npdt = {"f32": np.float32, "i32": np.int32, "i64": np.int64}[w.dtype]
        ins = [(np.random.default_rng(1234 + r).uniform(-1, 1, count) * 1000).astype(npdt) for r in range(n)]
        secs, _ = oracle.time_allreduce_threads(ins, warm, reps)
        transport = "in-process mailbox transport, one thread per rank"
    med = statistics.median(secs)
    out = {
        "value": round(w.bytes_per_step / med / 1e9, 3), "unit": "GB/s", "cores": n, "kind": "port",
        "ms_per_allreduce": round(med * 1e3, 3),
        "sample": "%d timed RingAllreduce calls (after %d warm-ups) of the same tensor (%s, %d elements) at %d ranks "
                  "on %d of %d host cores, %s; per-rank algorithmic bytes / median time of the slowest rank; "
                  "RingAllreduce only (no coordinator tick, no TensorFlow dispatch)"
                  % (reps, warm, w.dtype, count, n, n, host_cores, transport),
    }
    if w.name == "allreduce_f32_64MiB_n8":
        # the reference's own CPU-runnable case: 1,048,576 float32 at 2 ranks
        try:
            if oracle.mpirun_path():
                s2 = oracle.mpi_time(2, oracle.F32, 1_048_576, 5, 50)["secs"]
            else:
                small = [np.random.default_rng(1234 + r).uniform(-1, 1, 1_048_576).astype(np.float32) for r in range(2)]
                s2, _ = oracle.time_allreduce_threads(small, 5, 50)
            out["np2_1Mi_float32"] = {"GB/s": round(18_874_368 / statistics.median(s2) / 1e9, 3),
                                      "ms_per_allreduce": round(statistics.median(s2) * 1e3, 4), "cores": 2}
        except Exception as e:   # extra information only
            out["np2_1Mi_float32"] = {"error": str(e)}
    return out


def measured_traffic(workload):
    """HBM bytes per launch of the workload's dominant kernel from the committed
    rocprofv3 counter summary (FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel
    of known size), or None when no such summary exists."""
    name = TRAFFIC_PROFILES.get(workload)
    if name is None:
        return None
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, re.M)
    return float(m.group(1)) if m else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default=WORKLOADS[0], choices=WORKLOADS)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--fresh-staging", action="store_true",
                    help="stage every finished (allgather) segment at the start of a fresh allocation instead of "
                         "where it lies in a neighbour's buffer (see coaligned())")
    ap.add_argument("--variant", choices=("all", "reference", "fused"), default="all",
                    help="all: the reference-shaped path (the reported value), then the extras: the same job with "
                         "the in->out copy folded into the accumulate, and the hot (one buffer set) rate. "
                         "reference / fused: that path alone, for kernel traces (kernel names do not tell the two "
                         "accumulates apart, and the extras would mix into the per-kernel averages)")
    ap.add_argument("--recorded", type=int, default=0, metavar="STEPS",
                    help="allreduce workloads: record this many consecutive steps as ONE HIP graph (ring_graph_*) and "
                         "time its replays; for launch-bound sizes. --steps is rounded down to a multiple of it")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="launch option of the kernel library (unroll, blocks_per_cu, nontemporal[_copy|_accumulate|"
                         "_allgather|_pack|_unpack], paced_copy, phased_copy, dry_launch, flat_grid), "
                         "for comparing launch shapes under a profiler")
    args = ap.parse_args()
    global FRESH_STAGING
    FRESH_STAGING = args.fresh_staging
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures the per-rank data path on ONE GPU (the ring's N ranks are virtual); "
                 "--gpus %d is not supported" % args.gpus)
    big = args.workload in ("allreduce_f32_1GiB_n64", "floors_f32_1GiB_n64")
    steps = args.steps if args.steps is not None else (200 if big else 2000)
    warmup = args.warmup if args.warmup is not None else (20 if big else 200)

    import torch
    from mpi_collectives import ring_abi
    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X; no GPU is visible")
    ring_abi.lib()
    options = {}
    for item in args.option:
        name, _, value = item.partition("=")
        ring_abi.set_option(name, int(value))
        options[name] = int(value)
    w = make_workload(args.workload)
    if args.recorded and (not isinstance(w, RingAllreduce) or isinstance(w, RingAllreducePerStep)):
        sys.exit("bench.py: --recorded applies to the allreduce workloads")
    if options.get("dry_launch"):
        # the kernels return at entry: what is timed is the launches themselves, and there is no output to check
        w.check = lambda k: True
    torch.cuda.synchronize()

    # the dedicated stream every ring kernel is launched on (CudaStreamForMPI)
    stream = ring_abi.stream_create()
    nph = len(w.phases)
    # events are created ahead of the passes that use them: creating them between launches
    # would let the queue drain and the sampled launches start on an idle GPU
    # (a set = one pair per launch of the sampled step and one per launch of the step before it)
    npairs = max(nph, 2)
    n_samples = max(MIN_SAMPLES, min(steps // 16, MAX_SAMPLES))
    event_pool = [[ring_abi.event_create() for _ in range(4 * npairs)]
                  for _ in range(n_samples + 1 + COLD_SAMPLES)]

    def launcher(hot):
        # hot: the same buffer set every step (what fits stays in the last-level
        # cache); otherwise the sets rotate and every step starts cold
        if hot:
            return lambda k, stream, fused: w.launch_step(0, stream, fused)
        return w.launch_step

    def region(nsteps, nwarm, fused=False, hot=False, first=0, streams=None):
        """Wall-clock seconds of `nsteps` steps, bracketed by a synchronize on both sides,
        after `nwarm` untimed steps. Nothing inside the region carries an event: a dispatch
        that carries one ends only when its stores have drained, which serialises it against
        the launch behind it. `streams`: the steps go to these streams in turn (successive
        steps work on different virtual ranks' buffers and do not depend on one another);
        the default is the one dedicated stream."""
        launch_step = launcher(hot)
        streams = streams or (stream,)
        ns = len(streams)
        for k in range(first, first + nwarm):
            launch_step(k, streams[k % ns], fused)
        for st in streams:
            ring_abi.stream_synchronize(st)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(first + nwarm, first + nwarm + nsteps):
            launch_step(k, streams[k % ns], fused)
        for st in streams:
            ring_abi.stream_synchronize(st)
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    def regions(count, nsteps, nwarm, **kw):
        """`count` such regions back to back, each behind its own `nwarm` warm-up steps;
        returns their seconds per step, in the order measured. The interpreter's garbage is
        collected once, ahead of the first region, and the collector is off until the last
        has ended: a collection in the middle of a region stalls the launching thread for
        tens of milliseconds (a step that is one short launch has no queue of launches ahead
        of the GPU to hide that behind), and one between two regions leaves the GPU idle for
        as long, after which a region of a millisecond runs 5 % slower from its first step to
        its last than the same steps do in a longer one."""
        out, first = [], 0
        gc.collect()
        gc.disable()
        try:
            for _ in range(count):
                out.append(region(nsteps, nwarm, first=first, **kw) / nsteps)
                first += nsteps + nwarm
        finally:
            gc.enable()
        return out

    def sampling_pass(count):
        """Per-launch durations, outside every wall-clock region: the same steps on the same
        rotating buffers, every SAMPLE_EVERY-th one launched phase by phase, each launch
        carrying its own pair of HIP events in the dispatch (on the stream the kernels run
        on). The step before a sampled one carries (unused) events too: a timed dispatch ends
        when its stores have drained, so the sampled step's first launch does not pay for its
        predecessor's, as under a profiler's kernel trace, where every dispatch is timed."""
        samples = []
        for k in range(8):
            w.launch_step(k, stream)
        for k in range(8, 8 + count * SAMPLE_EVERY):
            if k % SAMPLE_EVERY == SAMPLE_EVERY - 2:
                spare = event_pool[-1]
                for i in range(nph):
                    ring_abi.time_next_launch(spare[2 * (npairs + i)], spare[2 * (npairs + i) + 1])
                w.launch_step(k, stream)
                ring_abi.time_next_launch(None, None)       # a step of fewer launches leaves none armed
            elif k % SAMPLE_EVERY == SAMPLE_EVERY - 1:
                e = event_pool.pop()
                for i in range(nph):
                    ring_abi.time_next_launch(e[2 * i], e[2 * i + 1])
                    w.launch_phase(k, i, stream)
                samples.append(e)
            else:
                w.launch_step(k, stream)
        ring_abi.stream_synchronize(stream)
        torch.cuda.synchronize()
        return samples

    if args.recorded:
        # `recorded` consecutive steps (rotating over the buffer sets) as one HIP graph, replayed
        fused = args.variant == "fused"
        L = ring_abi.lib()
        for k in range(8):
            w.launch_step(k, stream, fused)
        ring_abi.stream_synchronize(stream)
        ring_abi.check(L.ring_graph_begin_capture(stream), "ring_graph_begin_capture")
        for k in range(args.recorded):
            w.launch_step(k, stream, fused)
        graph = ctypes.c_void_p()
        ring_abi.check(L.ring_graph_end_capture(stream, ctypes.byref(graph)), "ring_graph_end_capture")
        replays = max(steps // args.recorded, 1)
        for _ in range(max(warmup // args.recorded, 1)):
            ring_abi.check(L.ring_graph_launch(graph, stream), "ring_graph_launch")
        ring_abi.stream_synchronize(stream)
        t0 = time.perf_counter()
        for _ in range(replays):
            ring_abi.check(L.ring_graph_launch(graph, stream), "ring_graph_launch")
        ring_abi.stream_synchronize(stream)
        elapsed = time.perf_counter() - t0
        ok = all(w.check(k) for k in range(min(args.recorded, w.nsets)))
        ring_abi.check(L.ring_graph_destroy(graph), "ring_graph_destroy")
        if not ok:
            sys.exit("bench.py: the output of the replayed graph is wrong; refusing to report a number")
        nsteps = replays * args.recorded
        nbytes = w.fused_bytes if fused else w.bytes_per_step
        print(json.dumps({"metric": "per-rank ring data path GB/s, %s, %d steps per replayed HIP graph" % (w.name, args.recorded),
                          "value": round(nbytes * nsteps / elapsed / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
                          "steps": nsteps, "warmup": warmup, "ms_per_step": round(elapsed / nsteps * 1e3, 5),
                          "higher_is_better": True, "dtype": w.dtype, "data": "synthetic",
                          "config": {"workload": w.description, "name": w.name, "bytes_per_step": nbytes,
                                     "launches_per_step": 2 if fused else 3,
                                     "steps_per_recorded_hip_graph": args.recorded}}))
        return
    if args.variant == "fused":
        if not isinstance(w, RingAllreduce) or isinstance(w, RingAllreducePerStep):
            sys.exit("bench.py: --variant fused applies to the allreduce workloads")
        per_step = regions(REGIONS, steps, warmup, fused=True)
        fused_elapsed = statistics.median(per_step) * steps
        if not w.check(REGIONS * (steps + warmup) - 1):
            sys.exit("bench.py: the output of the fused-copy path is wrong; refusing to report a number")
        print(json.dumps({"metric": "per-rank ring data path GB/s, %s, in->out copy folded into the accumulate" % w.name,
                          "value": round(w.fused_bytes * steps / fused_elapsed / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
                          "steps": steps, "warmup": warmup, "ms_per_step": round(fused_elapsed / steps * 1e3, 5),
                          "higher_is_better": True, "dtype": w.dtype, "data": "synthetic",
                          "config": {"workload": w.description, "name": w.name, "bytes_per_step": w.fused_bytes,
                                     "launches_per_step": 2}}))
        return
    per_step = regions(REGIONS, steps, warmup)
    if not w.check(REGIONS * (steps + warmup) - 1):
        sys.exit("bench.py: the output of the timed path is wrong; refusing to report a number")
    ms_per_step = statistics.median(per_step) * 1e3
    value = w.bytes_per_step / statistics.median(per_step) / 1e9
    samples = sampling_pass(n_samples)
    phase_times = [[ring_abi.event_elapsed_us(e[2 * i], e[2 * i + 1]) for e in samples] for i in range(nph)]
    phase_us = [statistics.mean(t) for t in phase_times]
    dom = w.phases[w.dominant]
    dom_median = statistics.median(phase_times[w.dominant])
    achieved = dom[1] / dom_median / 1e3

    # the same accumulate on operands nothing has touched before it: the step with the in->out copy
    # folded in (out = in + received), every 4th step timed
    cold = None
    if isinstance(w, RingAllreduce) and not isinstance(w, RingAllreducePerStep) and args.variant == "all":
        for k in range(8):
            w.launch_step(k, stream, True)
        cold_events = []
        for k in range(COLD_SAMPLES * 4):
            if k % 4 == 1:
                # the step before, timed too (see sampling_pass())
                spare = event_pool[-1]
                for i in range(2):
                    ring_abi.time_next_launch(spare[2 * (npairs + i)], spare[2 * (npairs + i) + 1])
            if k % 4 == 2:
                # the driver's own step; the events ride on its two launches, accumulate and allgather
                e = event_pool.pop()
                for i in range(2):
                    ring_abi.time_next_launch(e[2 * i], e[2 * i + 1])
                cold_events.append(e)
            w.launch_step(k, stream, True)
            ring_abi.time_next_launch(None, None)
        ring_abi.stream_synchronize(stream)
        cold_acc = [ring_abi.event_elapsed_us(e[0], e[1]) for e in cold_events]
        cold_ag = [ring_abi.event_elapsed_us(e[2], e[3]) for e in cold_events]
        cold = {"accumulate_median_us": round(statistics.median(cold_acc), 3),
                "accumulate_mean_us": round(statistics.mean(cold_acc), 3),
                "allgather_behind_it_median_us": round(statistics.median(cold_ag), 3),
                "launches_timed": len(cold_events)}

    result = {
        "metric": METRIC if args.workload == WORKLOADS[0] else "per-rank ring data path GB/s, " + w.name,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 5),
        "regions": {"count": REGIONS, "steps_each": steps, "warmup_before_each": warmup,
                    "ms_per_step_each": [round(t * 1e3, 5) for t in per_step],
                    "min_ms_per_step": round(min(per_step) * 1e3, 5),
                    "note": "ms_per_step and value are the MEDIAN of %d wall-clock regions of %d steps each, run back "
                            "to back, every region bracketed by a stream synchronize on both sides and free of "
                            "event-carrying launches" % (REGIONS, steps)},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.dtype,
        "data": "synthetic",
        "config": {"workload": w.description, "name": w.name, "bytes_per_step": w.bytes_per_step,
                   "launches_per_step": w.step_launches or nph, **({"launch_options": options} if options else {}),
                   **({"steps_per_recorded_hip_graph": args.recorded} if args.recorded else {})},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": {
            "bound": "hbm",
            "kernel": dom[2],
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic(args.workload),
            "algorithmic_bytes_per_launch": dom[1],
            "median_launch_us": round(dom_median, 3),
            "avg_launch_us": round(phase_us[w.dominant], 3),
            "launches_timed": len(samples),
            "launches_timed_inside_the_wall_clock_region": 0,
            "note": "achieved = algorithmic bytes / median launch duration (HIP events carried in the dispatch)."
                    + (" In the reference-shaped step the accumulate reads the buffer the in->out copy has just "
                       "written with ordinary stores, so part of its reads are served by the last-level cache: `frac` "
                       "is that LLC-assisted figure. `frac_cold` is the same kernel where no operand was touched "
                       "before it (the step with the copy folded in, out = in + received): the HBM figure."
                       if cold is not None else
                       " Buffer sets are rotated, so no operand of a launch was left in the last-level cache by the "
                       "launch before it."),
        },
        "phases": {p[0]: {"us": round(t, 3), "median_us": round(statistics.median(phase_times[i]), 3),
                          "min_us": round(min(phase_times[i]), 3), "GBps": round(p[1] / t / 1e3, 1),
                          "bytes": p[1]}
                   for i, (p, t) in enumerate(zip(w.phases, phase_us))},
        "phases_note": "HIP events carried by each launch of every %dth step of a sampling pass of %d steps that "
                       "follows the wall-clock regions (none of their launches carries an event); us = mean"
                       % (SAMPLE_EVERY, n_samples * SAMPLE_EVERY),
    }
    if cold is not None:
        result["roofline"]["frac_cold"] = round(dom[1] / cold["accumulate_median_us"] / 1e3 / HBM_PEAK_GBS, 4)
        result["roofline"]["achieved_cold"] = round(dom[1] / cold["accumulate_median_us"] / 1e3, 1)
        result["roofline"]["cold"] = cold
    # the same steps on ONE buffer set: at the headline size the working set fits the
    # last-level cache, so this is the cache-resident rate, not the HBM one
    if args.variant == "all":
        extra_steps = max(steps, EXTRA_MIN_STEPS)
        hot_steps = extra_steps
        hot_elapsed = statistics.median(regions(EXTRA_REGIONS, hot_steps, min(max(warmup, 20), 50), hot=True)) * hot_steps
        result["hot"] = {"ms_per_step": round(hot_elapsed / hot_steps * 1e3, 5),
                         "GBps": round(w.bytes_per_step * hot_steps / hot_elapsed / 1e9, 1),
                         "note": "every step on the same buffers (%.0f MiB touched per step); `value` is the cold "
                                 "rate, buffer sets rotated" % (w.bytes_per_step / 2**20)}
    if args.variant == "all" and w.nsets >= 2 and not options.get("dry_launch") and not isinstance(w, StreamFloors):
        # the same steps issued to two streams in turn: successive steps work on different virtual ranks'
        # buffers, so the start of one step's launches fills the chip while the step before it drains
        # (not the floors workload: its write probes fill another set's output, which only stream order
        # keeps apart from that set's own step)
        second = ring_abi.stream_create()
        two = statistics.median(regions(EXTRA_REGIONS, extra_steps, min(max(warmup, 20), 50), streams=(stream, second)))
        ok = all(w.check(k) for k in range(min(w.nsets, 2))) if not isinstance(w, FusedResnet50) else True
        ring_abi.stream_destroy(second)
        if not ok:
            sys.exit("bench.py: the output of the two-stream run is wrong; refusing to report a number")
        result["two_streams"] = {
            "ms_per_step": round(two * 1e3, 5), "steps": extra_steps, "regions": EXTRA_REGIONS,
            "GBps": round(w.bytes_per_step / two / 1e9, 1),
            "note": "the same steps, even ones on the dedicated stream and odd ones on a second stream (the C ABI takes the "
                    "stream per call): throughput of independent allreduces in flight together, not the latency of one; "
                    "`value` is the one-stream figure"}
    if isinstance(w, RingAllreduce) and not isinstance(w, RingAllreducePerStep):
        # the same job with the in->out copy folded into the accumulate (fewer bytes, same result)
        if args.variant == "all":
            fwarm = min(max(warmup, 20), 50)
            fused_per_step = statistics.median(regions(EXTRA_REGIONS, extra_steps, fwarm, fused=True))
            if not w.check(EXTRA_REGIONS * (extra_steps + fwarm) - 1):
                sys.exit("bench.py: the output of the fused-copy path is wrong; refusing to report a number")
            result["fused_copy"] = {
                "ms_per_step": round(fused_per_step * 1e3, 5),
                "steps": extra_steps, "regions": EXTRA_REGIONS,
                "bytes_per_step": w.fused_bytes,
                "GBps": round(w.fused_bytes / fused_per_step / 1e9, 1),
                "launches_per_step": 2,
                "note": "same allreduce with the in->out copy folded into the accumulate (out = in + received; the "
                        "segment that is only sent is written by the first allgather step and never copied)",
            }
        if args.variant == "all" and w.name == WORKLOADS[0] and not options.get("dry_launch"):
            # the same allreduce in the direct form (one fold pass over pushed copies + copies, one launch)
            d = make_workload("allreduce_f32_64MiB_n8_direct")
            for k in range(50):
                d.launch_step(k, stream)
            direct = []
            for _ in range(EXTRA_REGIONS):
                ring_abi.stream_synchronize(stream)
                t0 = time.perf_counter()
                for k in range(extra_steps):
                    d.launch_step(k, stream)
                ring_abi.stream_synchronize(stream)
                direct.append((time.perf_counter() - t0) / extra_steps)
            if not d.check(extra_steps - 1):
                sys.exit("bench.py: the output of the direct form is wrong; refusing to report a number")
            direct_per_step = statistics.median(direct)
            result["direct_form"] = {
                "ms_per_step": round(direct_per_step * 1e3, 5),
                "steps": extra_steps, "regions": EXTRA_REGIONS,
                "bytes_per_step": d.bytes_per_step,
                "GBps": round(d.bytes_per_step / direct_per_step / 1e9, 1),
                "launches_per_step": 1,
                "note": "same tensor and ranks, peers push raw copies of the owned segment instead of passing partial "
                        "sums round: the owner folds the 8 copies in ring order in one pass and copies the 7 finished "
                        "segments in, one launch; output bit-identical to the ring's (--workload "
                        "allreduce_f32_64MiB_n8_direct)",
            }
            del d
        if not args.no_cpu_baseline:
            try:
                result["cpu_baseline"] = cpu_baseline(w)
            except Exception as e:
                result["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port",
                                          "sample": "failed: %s" % e}
    elif not args.no_cpu_baseline:
        result["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port",
                                  "sample": "not run for this workload (the reference has no fusion buffer, no "
                                            "direct form and no ranks that share a device, and its allgather moves "
                                            "bytes only): the default workload carries the CPU baseline"}
    ring_abi.stream_destroy(stream)
    try:
        # what this process started and has not reaped (the cpu_baseline's mpirun legs run in process
        # groups of their own, which are ended when each returns)
        import psutil
        result["child_processes_at_exit"] = len(psutil.Process().children(recursive=True))
    except Exception:
        result["child_processes_at_exit"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
