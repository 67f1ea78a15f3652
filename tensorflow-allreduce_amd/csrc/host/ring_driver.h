// Host side of the ring: segmenting, step schedule and step tables for one
// rank (or for all virtual ranks at once), issued through the C ABI of
// ring_abi.h. The counterpart of RingAllreduce / RingAllgather in
// tensorflow/contrib/mpi_collectives/ring.h:136-301 with the MPI
// point-to-point calls replaced by segments that are already addressable in
// device memory.
#ifndef MPIC_RING_DRIVER_H_
#define MPIC_RING_DRIVER_H_

#include <cstddef>
#include <vector>

#include "framework.h"
#include "ring_abi.h"

namespace mpic {

// Most copies of a segment one fold launch can address (ring_fold_rows): the
// direct forms are limited to rings of this many ranks.
constexpr int kMaxDirectRanks = 256;
// Most peers whose staged copies the one-launch direct form of a fused
// allreduce takes (ring_fusion_fold_scatter); larger rings run it as three launches.
constexpr int kMaxOneLaunchDirectRanks = 32;

struct RingOptions {
  // One launch per ring phase (all n-1 steps of a rank) instead of one per
  // step. Steps of one rank write disjoint segments, so the order inside a
  // phase does not matter and the result is bit-identical.
  bool batched = true;
  // Fold the in->out copy (ring.h:146-148) into the reduce-scatter:
  // out[seg] = in[seg] + received, the same single add per element.
  bool fuse_copy = false;
  // > 0: the result is tf.div(result, divisor), the average of
  // allreduce(average=True) (__init__.py:160-164, 153-157 of the reference),
  // computed where a value becomes final instead of in a pass of its own: the
  // owner of a segment divides in its last reduce-scatter accumulate (the
  // owner of an allgather slice, when it copies the slice into its output), and
  // what then travels round the ring is already divided. Pre-staged allgather
  // segments are therefore expected divided, as a peer would send them.
  int divisor = 0;
  // Where every rank's copy of a segment is addressable at once: its owner
  // folds the n copies in ring order in one pass instead of n-1 accumulate
  // steps. A rank with pre-staged peers then copies each finished segment
  // straight from where it was pushed; ranks that share the GPU get the result
  // stored into all their outputs by the fold itself (ring_fold_to_all_rows).
  // Same additions in the same order, so the same bits; 1 launch (2 beyond 128
  // ranks) instead of 2(n-1)+1.
  bool direct = false;
  // Transport-driven rings only: pieces a segment travels in (1..16).
  int chunks = 1;
  static RingOptions FromFlags(int flags) {
    RingOptions o;
    o.batched = (flags & 1) != 0;
    o.fuse_copy = (flags & 2) != 0;
    o.direct = (flags & 4) != 0;
    o.chunks = ((flags >> 4) & 15) + 1;
    o.divisor = (flags >> 8) & 0x7fffff;
    return o;
  }
};

// ring.cu.cc:14-20 / mpi_ops.cc:836-847: the three supported element types.
// Sets *ring_dtype to the ring_abi.h code.
Status RingDataType(DataType dt, int* ring_dtype);

// ring.h:136-228 for rank r of n. rs_recv[i] / ag_recv[i]: device pointers to
// the segment the left neighbour sends at reduce-scatter / allgather step i
// (n-1 each). Asynchronous on `stream`.
Status RingAllreducePrestaged(int n, int r, DataType dt, const void* input, void* output, size_t count,
                              const void* const* rs_recv, const void* const* ag_recv, void* stream,
                              const RingOptions& opts);

// The direct form for rank r of n, which owns segment s = (r+1) mod n: peers[k]
// (k = 0..n-2) is rank (s+k) mod n's copy of segment s, as that rank would push
// it into this rank's staging slot; they and the rank's own copy are folded in
// ring order into output[s]. ag_recv[i]: the finished segment (r-i) mod n, as
// its owner would push it. Bit-identical to RingAllreducePrestaged fed with
// the ring's own traffic.
Status RingAllreduceDirectPrestaged(int n, int r, DataType dt, const void* input, void* output, size_t count,
                                    const void* const* peers, const void* const* ag_recv, void* stream,
                                    const RingOptions& opts);

// A fused allreduce for rank r of n without pack and unpack passes. `plan`
// (ring_fusion_plan_create) lists the rank's tensors; the packed buffer exists
// only as `wire`, plan-elements long, where the sums a ring sends on are left.
// Reduce-scatter: wire[seg] = tensors[seg] + rs_recv[i] for the n-1 received
// segments, and segment r, which is only sent, is packed (one launch, the local
// operand read straight from the tensors). Allgather: every finished segment,
// ag_recv[i] or the rank's own in `wire`, goes straight into the tensors,
// divided when opts.divisor > 0 (one launch). Each tensor ends up as the
// reference ring applied to the packed buffer would leave it.
Status RingAllreduceFusedPrestaged(const ring_fusion_plan* plan, int n, int r, void* wire,
                                   const void* const* rs_recv, const void* const* ag_recv, void* stream,
                                   const RingOptions& opts);

// ring.h:236-301 for rank r of n. recv[i]: the segment received at step i
// (segment (r-i-1) mod n).
Status RingAllgatherPrestaged(int n, int r, DataType dt, const void* input, const std::vector<size_t>& rows,
                              size_t elems_per_row, void* output, const void* const* recv, void* stream,
                              const RingOptions& opts);

// All n ranks on this GPU, advancing in lockstep: at every step each rank
// reads its left neighbour's buffer where MPI would have delivered a copy
// (the neighbour does not write that segment during the step).
Status RingAllreduceAllRanks(int n, DataType dt, const void* const* inputs, void* const* outputs, size_t count,
                             void* stream, const RingOptions& opts);
Status RingAllgatherAllRanks(int n, DataType dt, const void* const* inputs, const std::vector<size_t>& rows,
                             size_t elems_per_row, void* const* outputs, void* stream, const RingOptions& opts);

}  // namespace mpic
#endif  // MPIC_RING_DRIVER_H_
