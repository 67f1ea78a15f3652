#include "ring_driver.h"

#include <memory>
#include <string>

#include "ring_abi.h"

namespace mpic {
namespace {

// A call's small tables (segment sizes, step rows, pointers): on the stack up
// to N items, which covers a ring of 64 ranks, on the heap beyond. The driver
// runs once per collective on the thread that feeds the stream; at small
// tensors a step costs what that thread spends, and a handful of heap
// allocations per call were a measurable part of it.
template <typename T, size_t N>
class Table {
 public:
  explicit Table(size_t capacity) : data_(stack_) {
    if (capacity > N) {
      heap_.reset(new T[capacity]);
      data_ = heap_.get();
    }
  }
  Table(size_t n, const T& fill) : Table(n) {
    for (size_t i = 0; i < n; i++) data_[i] = fill;
    size_ = n;
  }
  void push_back(const T& v) { data_[size_++] = v; }  // within the capacity given at construction
  T* data() { return data_; }
  const T* data() const { return data_; }
  size_t size() const { return size_; }
  T& operator[](size_t i) { return data_[i]; }
  const T& operator[](size_t i) const { return data_[i]; }

 private:
  T stack_[N];
  std::unique_ptr<T[]> heap_;
  T* data_;
  size_t size_ = 0;
};
constexpr size_t kStackRanks = 64;
constexpr size_t kStackPointers = 256;  // the n x n tables of resident ranks: 16 ranks on the stack

// The reference's MPI_REQUIRES_OK (ring.h:36-39) for the device layer.
Status FromRing(int rc, const char* what) {
  if (rc == RING_OK) return Status::OK();
  std::string msg = std::string(what) + ": " + ring_status_string(rc);
  if (rc == RING_ERR_HIP) msg += " (hipError " + std::to_string(ring_last_hip_error()) + ")";
  if (rc == RING_ERR_DTYPE) return errors::FailedPrecondition(ring_status_string(rc));
  return errors::Unknown(msg);
}
#define RING_RETURN_IF_ERROR(call, what)      \
  do {                                        \
    Status s_ = FromRing((call), (what));     \
    if (!s_.ok()) return s_;                  \
  } while (0)

inline const char* at(const void* base, size_t elems, size_t esz) {
  return static_cast<const char*>(base) + elems * esz;
}
inline char* at(void* base, size_t elems, size_t esz) { return static_cast<char*>(base) + elems * esz; }

int Seg(int phase, int n, int r, int step, bool recv) {
  int s = 0, v = 0;
  ring_schedule(phase, n, r, step, &s, &v);
  return recv ? v : s;
}

}  // namespace

Status RingDataType(DataType dt, int* ring_dtype) {
  switch (dt) {
    case DT_FLOAT: *ring_dtype = RING_F32; return Status::OK();
    case DT_INT32: *ring_dtype = RING_I32; return Status::OK();
    case DT_INT64: *ring_dtype = RING_I64; return Status::OK();
    default: return errors::FailedPrecondition("Invalid tensor type passed.");
  }
}

Status RingAllreducePrestaged(int n, int r, DataType dt, const void* input, void* output, size_t count,
                              const void* const* rs_recv, const void* const* ag_recv, void* stream,
                              const RingOptions& opts) {
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1 || r < 0 || r >= n) return errors::InvalidArgument("rank out of range for the ring");
  const size_t esz = ring_dtype_size(code);
  if (count == 0) return Status::OK();
  if (!input || !output) return errors::InvalidArgument("null tensor with a non-zero element count");
  if (n > 1 && (!rs_recv || !ag_recv)) return errors::InvalidArgument("no staged peer segments");

  Table<size_t, kStackRanks> sizes(static_cast<size_t>(n), 0), starts(static_cast<size_t>(n), 0);
  RING_RETURN_IF_ERROR(ring_segment_table(count, n, sizes.data(), starts.data()), "ring_segment_table");

  const int divisor = opts.divisor;
  if (divisor < 0) return errors::InvalidArgument("negative divisor");
  if (n == 1) {  // ring.h:146-148 is all there is; a lone rank owns every element
    if (divisor > 0) {
      ring_row row{output, input, nullptr, count};
      RING_RETURN_IF_ERROR(ring_apply_rows_avg(&row, 1, nullptr, divisor, code, stream), "ring_apply_rows_avg");
    } else if (input != output) {
      RING_RETURN_IF_ERROR(ring_copy_bytes(output, input, count * esz, stream), "ring_copy_bytes");
    }
    return Status::OK();
  }
  const bool fuse = opts.fuse_copy && opts.batched && input != output;
  if (!fuse && input != output)  // ring.h:146-148
    RING_RETURN_IF_ERROR(ring_copy_bytes(output, input, count * esz, stream), "ring_copy_bytes");
  // the segment whose sum completes at the last step (n-2) is the one this rank
  // owns and sends first in the allgather: the only one it divides
  Table<unsigned char, kStackRanks> divide(static_cast<size_t>(n), 0);
  divide[static_cast<size_t>(n - 2)] = 1;

  // ring.h:183-205: step i receives segment (r-i-1) and adds it into the buffer
  if (fuse) {
    Table<ring_row, kStackRanks> rows(static_cast<size_t>(n));
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_REDUCE_SCATTER, n, r, i, true));
      rows.push_back(ring_row{at(output, starts[seg], esz), rs_recv[i], at(input, starts[seg], esz), sizes[seg]});
    }
    // Segment r is only ever sent, never accumulated, and the first allgather
    // step overwrites it with its final value (ring.h:211-225 receives segment
    // r at step 0): a transport would send it from the input, nothing copies it.
    RING_RETURN_IF_ERROR(ring_apply_rows_avg(rows.data(), static_cast<int>(rows.size()), divide.data(), divisor,
                                             code, stream),
                         "ring_apply_rows_avg");
  } else if (opts.batched && divisor > 0) {
    Table<ring_row, kStackRanks> rows(static_cast<size_t>(n));
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_REDUCE_SCATTER, n, r, i, true));
      char* dst = at(output, starts[seg], esz);
      rows.push_back(ring_row{dst, rs_recv[i], dst, sizes[seg]});
    }
    RING_RETURN_IF_ERROR(ring_apply_rows_avg(rows.data(), n - 1, divide.data(), divisor, code, stream),
                         "ring_apply_rows_avg");
  } else if (opts.batched) {
    Table<ring_step, kStackRanks> steps(static_cast<size_t>(n));
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_REDUCE_SCATTER, n, r, i, true));
      steps.push_back(ring_step{starts[seg], rs_recv[i], sizes[seg]});
    }
    RING_RETURN_IF_ERROR(ring_reduce_scatter_steps(output, steps.data(), n - 1, code, stream),
                         "ring_reduce_scatter_steps");
  } else {
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_REDUCE_SCATTER, n, r, i, true));
      if (divisor > 0 && i == n - 2) {
        char* dst = at(output, starts[seg], esz);
        ring_row row{dst, rs_recv[i], dst, sizes[seg]};
        RING_RETURN_IF_ERROR(ring_apply_rows_avg(&row, 1, nullptr, divisor, code, stream), "ring_apply_rows_avg");
      } else {
        RING_RETURN_IF_ERROR(ring_accumulate(code, at(output, starts[seg], esz), rs_recv[i], sizes[seg], stream),
                             "ring_accumulate");
      }
    }
  }

  // ring.h:211-225: step i receives segment (r-i) straight into the buffer
  if (opts.batched) {
    Table<ring_step, kStackRanks> steps(static_cast<size_t>(n));
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_ALLGATHER, n, r, i, true));
      steps.push_back(ring_step{starts[seg], ag_recv[i], sizes[seg]});
    }
    RING_RETURN_IF_ERROR(ring_allgather_steps(output, steps.data(), n - 1, code, stream), "ring_allgather_steps");
  } else {
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_ALLGATHER, n, r, i, true));
      // a one-row step table rather than ring_copy_bytes: a received segment is
      // touched once, while the in->out copy's output is read again at once
      const ring_step step{starts[seg], ag_recv[i], sizes[seg]};
      RING_RETURN_IF_ERROR(ring_allgather_steps(output, &step, 1, code, stream), "ring_allgather_steps");
    }
  }
  return Status::OK();
}

Status RingAllreduceDirectPrestaged(int n, int r, DataType dt, const void* input, void* output, size_t count,
                                    const void* const* peers, const void* const* ag_recv, void* stream,
                                    const RingOptions& opts) {
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1 || r < 0 || r >= n) return errors::InvalidArgument("rank out of range for the ring");
  if (n > kMaxDirectRanks)
    return errors::InvalidArgument("the direct form folds at most 256 copies of a segment; use the ring form for " +
                                   std::to_string(n) + " ranks");
  if (opts.divisor < 0) return errors::InvalidArgument("negative divisor");
  const size_t esz = ring_dtype_size(code);
  if (count == 0) return Status::OK();
  if (!input || !output) return errors::InvalidArgument("null tensor with a non-zero element count");
  if (n > 1 && (!peers || !ag_recv)) return errors::InvalidArgument("no staged peer segments");
  Table<size_t, kStackRanks> sizes(static_cast<size_t>(n), 0), starts(static_cast<size_t>(n), 0);
  RING_RETURN_IF_ERROR(ring_segment_table(count, n, sizes.data(), starts.data()), "ring_segment_table");

  // the owned segment: x_s, x_{s+1}, ..., x_{s+n-1} = this rank's own, folded in that order
  const size_t own = static_cast<size_t>((r + 1) % n);
  Table<const void*, kStackRanks> srcs(static_cast<size_t>(n));
  for (int k = 0; k < n - 1; k++) {
    if (sizes[own] && !peers[k]) return errors::InvalidArgument("null staged peer segment");
    srcs.push_back(peers[k]);
  }
  srcs.push_back(at(input, starts[own], esz));
  ring_fold_row fold{at(output, starts[own], esz), srcs.data(), sizes[own]};
  // every other segment arrives finished (ring.h:211-225 delivers the same values step by step)
  Table<ring_row, kStackRanks> copies(static_cast<size_t>(n));
  for (int i = 0; i < n - 1; i++) {
    const size_t seg = static_cast<size_t>(Seg(RING_PHASE_ALLGATHER, n, r, i, true));
    copies.push_back(ring_row{at(output, starts[seg], esz), ag_recv[i], nullptr, sizes[seg]});
  }
  if (opts.batched) {
    // fold and copies write disjoint segments: one launch
    RING_RETURN_IF_ERROR(ring_fold_and_copy_rows(&fold, 1, n, opts.divisor, copies.data(), n - 1, code, stream),
                         "ring_fold_and_copy_rows");
  } else {
    RING_RETURN_IF_ERROR(ring_fold_rows(&fold, 1, n, opts.divisor, code, stream), "ring_fold_rows");
    RING_RETURN_IF_ERROR(ring_apply_rows(copies.data(), n - 1, code, stream), "ring_apply_rows");
  }
  return Status::OK();
}

Status RingAllreduceFusedPrestaged(const ring_fusion_plan* plan, int n, int r, void* wire,
                                   const void* const* rs_recv, const void* const* ag_recv, void* stream,
                                   const RingOptions& opts) {
  if (!plan) return errors::InvalidArgument("no fusion plan");
  const int code = ring_fusion_plan_dtype(plan);
  if (n < 1 || r < 0 || r >= n) return errors::InvalidArgument("rank out of range for the ring");
  if (opts.divisor < 0) return errors::InvalidArgument("negative divisor");
  const size_t count = ring_fusion_plan_elements(plan);
  if (count == 0) return Status::OK();
  if (!wire) return errors::InvalidArgument("no wire buffer");
  if (n > 1 && (!rs_recv || !ag_recv)) return errors::InvalidArgument("no staged peer segments");
  const size_t esz = ring_dtype_size(code);
  Table<size_t, kStackRanks> sizes(static_cast<size_t>(n), 0), starts(static_cast<size_t>(n), 0);
  RING_RETURN_IF_ERROR(ring_segment_table(count, n, sizes.data(), starts.data()), "ring_segment_table");

  const size_t own = static_cast<size_t>((r + 1) % n);
  if (opts.direct && n > kMaxDirectRanks)
    return errors::InvalidArgument("the direct form folds at most 256 copies of a segment; use the ring form for " +
                                   std::to_string(n) + " ranks");
  if (opts.direct && n > 1) {
    // Direct form: rs_recv[k] is rank (own+k)'s raw copy of the owned segment
    // (packed layout). The rank packs its own copy of that segment into the
    // wire buffer, folds the n copies there in ring order, and scatters the
    // finished segments into the tensors.
    Table<const void*, kStackRanks> ag_direct(static_cast<size_t>(n), nullptr);
    for (int i = 0; i < n - 1; i++)
      ag_direct[static_cast<size_t>(Seg(RING_PHASE_ALLGATHER, n, r, i, true))] = ag_recv[i];
    char* mine = at(wire, starts[own], esz);
    if (n - 1 <= kMaxOneLaunchDirectRanks) {
      // one launch: the owned segment folded from the staged copies and the
      // tensors, its sum left in the wire buffer, everything scattered
      Table<const void*, kStackRanks> staged(static_cast<size_t>(n));
      for (int k = 0; k < n - 1; k++) {
        if (sizes[own] && !rs_recv[k]) return errors::InvalidArgument("null staged peer segment");
        staged.push_back(rs_recv[k]);
      }
      Table<ring_fusion_span, kStackRanks> others(static_cast<size_t>(n));
      for (size_t seg = 0; seg < static_cast<size_t>(n); seg++) {
        if (seg == own) continue;
        if (sizes[seg] && !ag_direct[seg]) return errors::InvalidArgument("null staged peer segment");
        others.push_back(ring_fusion_span{starts[seg], sizes[seg], ag_direct[seg], nullptr});
      }
      RING_RETURN_IF_ERROR(ring_fusion_fold_scatter(plan, starts[own], sizes[own], staged.data(), n - 1, mine,
                                                    others.data(), n - 1, opts.divisor, stream),
                           "ring_fusion_fold_scatter");
      return Status::OK();
    }
    ring_fusion_span pack{starts[own], sizes[own], nullptr, mine};
    RING_RETURN_IF_ERROR(ring_fusion_gather(plan, &pack, 1, stream), "ring_fusion_gather");
    Table<const void*, kStackRanks> srcs(static_cast<size_t>(n));
    for (int k = 0; k < n - 1; k++) {
      if (sizes[own] && !rs_recv[k]) return errors::InvalidArgument("null staged peer segment");
      srcs.push_back(rs_recv[k]);
    }
    srcs.push_back(mine);
    ring_fold_row fold{mine, srcs.data(), sizes[own]};
    RING_RETURN_IF_ERROR(ring_fold_rows(&fold, 1, n, 0, code, stream), "ring_fold_rows");
    Table<ring_fusion_span, kStackRanks> finished(static_cast<size_t>(n));
    for (size_t seg = 0; seg < static_cast<size_t>(n); seg++) {
      const void* from = seg == own ? static_cast<const void*>(mine) : ag_direct[seg];
      if (sizes[seg] && !from) return errors::InvalidArgument("null staged peer segment");
      finished.push_back(ring_fusion_span{starts[seg], sizes[seg], from, nullptr});
    }
    RING_RETURN_IF_ERROR(ring_fusion_scatter(plan, finished.data(), n, opts.divisor, stream), "ring_fusion_scatter");
    return Status::OK();
  }

  // what arrives for each segment in either phase (ring.h:183-205, :211-225)
  Table<const void*, kStackRanks> rs_of(static_cast<size_t>(n), nullptr), ag_of(static_cast<size_t>(n), nullptr);
  for (int i = 0; i < n - 1; i++) {
    rs_of[static_cast<size_t>(Seg(RING_PHASE_REDUCE_SCATTER, n, r, i, true))] = rs_recv[i];
    ag_of[static_cast<size_t>(Seg(RING_PHASE_ALLGATHER, n, r, i, true))] = ag_recv[i];
  }
  Table<ring_fusion_span, kStackRanks> gather(static_cast<size_t>(n)), scatter(static_cast<size_t>(n));
  for (size_t seg = 0; seg < static_cast<size_t>(n); seg++) {
    // segment r has no arrival in the reduce-scatter: packed, as the first send needs it
    gather.push_back(ring_fusion_span{starts[seg], sizes[seg], rs_of[seg], at(wire, starts[seg], esz)});
    const void* finished = (seg == own || n == 1) ? at(static_cast<const void*>(wire), starts[seg], esz) : ag_of[seg];
    if (sizes[seg] && !finished) return errors::InvalidArgument("null staged peer segment");
    scatter.push_back(ring_fusion_span{starts[seg], sizes[seg], finished, nullptr});
  }
  for (size_t seg = 0; seg < static_cast<size_t>(n); seg++)
    if (sizes[seg] && n > 1 && seg != static_cast<size_t>(r) && !rs_of[seg])
      return errors::InvalidArgument("null staged peer segment");
  RING_RETURN_IF_ERROR(ring_fusion_gather(plan, gather.data(), n, stream), "ring_fusion_gather");
  RING_RETURN_IF_ERROR(ring_fusion_scatter(plan, scatter.data(), n, opts.divisor, stream), "ring_fusion_scatter");
  return Status::OK();
}

Status RingAllgatherPrestaged(int n, int r, DataType dt, const void* input, const std::vector<size_t>& rows,
                              size_t elems_per_row, void* output, const void* const* recv, void* stream,
                              const RingOptions& opts) {
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1 || r < 0 || r >= n || rows.size() != static_cast<size_t>(n))
    return errors::InvalidArgument("rank or sizes do not match the ring");
  const size_t esz = ring_dtype_size(code);
  Table<size_t, kStackRanks> starts(static_cast<size_t>(n), 0);
  RING_RETURN_IF_ERROR(ring_allgather_table(rows.data(), n, elems_per_row, starts.data()), "ring_allgather_table");

  // ring.h:263-266: own slice to its offset
  const size_t own = elems_per_row * rows[static_cast<size_t>(r)];
  if (own && (!input || !output)) return errors::InvalidArgument("null tensor with a non-zero element count");
  if (n > 1 && !recv) return errors::InvalidArgument("no staged peer segments");

  // ring.h:279-298: step i receives segment (r-i-1) in place. With a step table
  // the own-slice copy is one more row of the same launch.
  if (opts.divisor < 0) return errors::InvalidArgument("negative divisor");
  if (opts.batched && opts.divisor > 0) {
    Table<ring_row, kStackRanks> table(static_cast<size_t>(n));
    Table<unsigned char, kStackRanks> divide(static_cast<size_t>(n), 0);
    divide[0] = 1;  // the own slice; what arrives was divided by its owner
    table.push_back(ring_row{own ? at(output, starts[static_cast<size_t>(r)], esz) : nullptr, input, nullptr, own});
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_GATHER, n, r, i, true));
      const size_t cnt = elems_per_row * rows[seg];
      table.push_back(ring_row{cnt ? at(output, starts[seg], esz) : nullptr, recv[i], nullptr, cnt});
    }
    RING_RETURN_IF_ERROR(ring_apply_rows_avg(table.data(), n, divide.data(), opts.divisor, code, stream),
                         "ring_apply_rows_avg");
  } else if (opts.batched) {
    Table<ring_step, kStackRanks> steps(static_cast<size_t>(n));
    steps.push_back(ring_step{starts[static_cast<size_t>(r)], input, own});
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_GATHER, n, r, i, true));
      steps.push_back(ring_step{starts[seg], recv[i], elems_per_row * rows[seg]});
    }
    RING_RETURN_IF_ERROR(ring_allgather_steps(output, steps.data(), n, code, stream), "ring_allgather_steps");
  } else {
    if (opts.divisor > 0) {
      ring_row row{own ? at(output, starts[static_cast<size_t>(r)], esz) : nullptr, input, nullptr, own};
      RING_RETURN_IF_ERROR(ring_apply_rows_avg(&row, 1, nullptr, opts.divisor, code, stream), "ring_apply_rows_avg");
    } else {
      const ring_step mine{starts[static_cast<size_t>(r)], input, own};
      RING_RETURN_IF_ERROR(ring_allgather_steps(output, &mine, 1, code, stream), "ring_allgather_steps");
    }
    for (int i = 0; i < n - 1; i++) {
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_GATHER, n, r, i, true));
      const ring_step step{starts[seg], recv[i], elems_per_row * rows[seg]};
      RING_RETURN_IF_ERROR(ring_allgather_steps(output, &step, 1, code, stream), "ring_allgather_steps");
    }
  }
  return Status::OK();
}

Status RingAllreduceAllRanks(int n, DataType dt, const void* const* inputs, void* const* outputs, size_t count,
                             void* stream, const RingOptions& opts) {
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1) return errors::InvalidArgument("empty ring");
  if (opts.divisor < 0) return errors::InvalidArgument("negative divisor");
  if (count == 0) return Status::OK();
  const size_t esz = ring_dtype_size(code);
  Table<size_t, kStackRanks> sizes(static_cast<size_t>(n), 0), starts(static_cast<size_t>(n), 0);
  RING_RETURN_IF_ERROR(ring_segment_table(count, n, sizes.data(), starts.data()), "ring_segment_table");

  Table<ring_row, kStackRanks> rows(static_cast<size_t>(n), ring_row{nullptr, nullptr, nullptr, 0});
  for (int r = 0; r < n; r++)
    if (!inputs[r] || !outputs[r]) return errors::InvalidArgument("null tensor with a non-zero element count");

  // The fold kernel carries at most kMaxDirectRanks source pointers per launch; a
  // larger ring runs the lockstep form below, which handles any n (ring.h:136-228).
  if (opts.direct && 2 * n - 1 <= kMaxDirectRanks) {
    // One launch for the whole allreduce: the owner of every segment folds the n
    // copies in ring order and stores the result into every rank's output. Rank
    // (seg-1) owns segment seg; its own output leads the destinations.
    const size_t un = static_cast<size_t>(n);
    Table<const void*, kStackPointers> srcs(un * un);  // row j's n sources at [j * n, (j + 1) * n)
    Table<void*, kStackPointers> dsts(un * un);
    Table<ring_fold_to_all_row, kStackRanks> folds(un);
    for (int j = 0; j < n; j++) {
      const size_t seg = static_cast<size_t>((j + 1) % n);
      for (int k = 0; k < n; k++) {
        srcs.push_back(at(inputs[(static_cast<int>(seg) + k) % n], starts[seg], esz));
        dsts.push_back(at(outputs[(j + k) % n], starts[seg], esz));
      }
      folds.push_back(ring_fold_to_all_row{dsts.data() + static_cast<size_t>(j) * un,
                                           srcs.data() + static_cast<size_t>(j) * un, sizes[seg]});
    }
    if (!(n == 1 && inputs[0] == outputs[0] && opts.divisor == 0))
      RING_RETURN_IF_ERROR(ring_fold_to_all_rows(folds.data(), n, n, n, opts.divisor, code, stream),
                           "ring_fold_to_all_rows");
    return Status::OK();
  }
  if (opts.direct && n <= kMaxDirectRanks) {
    // More ranks than one row's pointers hold twice over: the owner of every
    // segment folds the n copies in ring order (one launch) ...
    const size_t un = static_cast<size_t>(n);
    Table<const void*, kStackPointers> srcs(un * un);
    Table<ring_fold_row, kStackRanks> folds(un);
    for (int j = 0; j < n; j++) {
      const size_t seg = static_cast<size_t>((j + 1) % n);
      for (int k = 0; k < n; k++)
        srcs.push_back(at(inputs[(static_cast<int>(seg) + k) % n], starts[seg], esz));
      folds.push_back(ring_fold_row{at(outputs[j], starts[seg], esz), srcs.data() + static_cast<size_t>(j) * un, sizes[seg]});
    }
    RING_RETURN_IF_ERROR(ring_fold_rows(folds.data(), n, n, opts.divisor, code, stream), "ring_fold_rows");
    // ... and every rank copies each finished segment from its owner (one more).
    Table<ring_row, kStackPointers> copies(un * un);
    for (int r = 0; r < n; r++) {
      for (int seg = 0; seg < n; seg++) {
        const int owner = (seg - 1 + n) % n;
        if (owner == r) continue;
        const size_t sg = static_cast<size_t>(seg);
        copies.push_back(ring_row{at(outputs[r], starts[sg], esz),
                                  at(static_cast<const void*>(outputs[owner]), starts[sg], esz), nullptr, sizes[sg]});
      }
    }
    RING_RETURN_IF_ERROR(ring_apply_rows(copies.data(), static_cast<int>(copies.size()), code, stream),
                         "ring_apply_rows");
    return Status::OK();
  }
  // Without the in->out copy (ring.h:146-148): every segment of a rank's output
  // is written by one of the 2(n-1) steps anyway (the reduce-scatter writes all
  // but segment r, the allgather all but segment r+1), and a rank accumulates
  // into each segment once, so the local operand of that add is still the
  // untouched input: out[seg] = in[seg] + received is the same single add. What
  // is received at step 0 is the neighbour's own segment, which it never
  // accumulates into: its input. n == 1 has no steps and keeps the copy.
  const bool fuse = opts.fuse_copy && n > 1;
  if (!fuse) {
    for (int r = 0; r < n; r++) {
      // a rank reducing in place (a fusion buffer) has nothing to copy
      const bool nothing = inputs[r] == outputs[r] && !(n == 1 && opts.divisor > 0);
      rows[static_cast<size_t>(r)] = ring_row{outputs[r], inputs[r], nullptr, nothing ? 0 : count};
    }
    // a lone rank owns every element: its copy is where the divide happens
    RING_RETURN_IF_ERROR(ring_apply_rows_avg(rows.data(), n, nullptr, n == 1 ? opts.divisor : 0, code, stream),
                         "ring_apply_rows");
  }

  // ring.h:183-205: at step i rank r adds its left neighbour's segment (r-i-1)
  for (int i = 0; i < n - 1; i++) {
    for (int r = 0; r < n; r++) {
      const int left = (r - 1 + n) % n;
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_REDUCE_SCATTER, n, r, i, true));
      char* dst = at(outputs[r], starts[seg], esz);
      const void* local = fuse ? static_cast<const void*>(at(inputs[r], starts[seg], esz)) : dst;
      const void* received = (fuse && i == 0) ? at(inputs[left], starts[seg], esz)
                                              : at(static_cast<const void*>(outputs[left]), starts[seg], esz);
      rows[static_cast<size_t>(r)] = ring_row{dst, received, local, sizes[seg]};
    }
    // the last step completes every rank's owned segment: all of its rows divide
    RING_RETURN_IF_ERROR(ring_apply_rows_avg(rows.data(), n, nullptr, i == n - 2 ? opts.divisor : 0, code, stream),
                         "ring_apply_rows");
  }
  // ring.h:211-225: at step i rank r receives segment (r-i) from the left
  for (int i = 0; i < n - 1; i++) {
    for (int r = 0; r < n; r++) {
      const int left = (r - 1 + n) % n;
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_ALLGATHER, n, r, i, true));
      rows[static_cast<size_t>(r)] = ring_row{at(outputs[r], starts[seg], esz),
                                              at(static_cast<const void*>(outputs[left]), starts[seg], esz), nullptr, sizes[seg]};
    }
    RING_RETURN_IF_ERROR(ring_apply_rows(rows.data(), n, code, stream), "ring_apply_rows");
  }
  return Status::OK();
}

Status RingAllgatherAllRanks(int n, DataType dt, const void* const* inputs, const std::vector<size_t>& rows_per_rank,
                             size_t elems_per_row, void* const* outputs, void* stream, const RingOptions& opts) {
  if (opts.divisor < 0) return errors::InvalidArgument("negative divisor");
  int code = 0;
  Status s = RingDataType(dt, &code);
  if (!s.ok()) return s;
  if (n < 1 || rows_per_rank.size() != static_cast<size_t>(n)) return errors::InvalidArgument("sizes do not match the ring");
  const size_t esz = ring_dtype_size(code);
  Table<size_t, kStackRanks> starts(static_cast<size_t>(n), 0);
  RING_RETURN_IF_ERROR(ring_allgather_table(rows_per_rank.data(), n, elems_per_row, starts.data()), "ring_allgather_table");

  if (opts.direct) {
    // Every slice straight from its owner's input into every rank's output, one
    // launch: the values a ring allgather delivers after n-1 steps (it only
    // moves bytes). A divisor divides every copy, which gives each rank what
    // the owner's one division would have sent round.
    Table<ring_row, kStackPointers> all(static_cast<size_t>(n) * static_cast<size_t>(n));
    for (int r = 0; r < n; r++) {
      for (int k = 0; k < n; k++) {
        const size_t cnt = elems_per_row * rows_per_rank[static_cast<size_t>(k)];
        if (cnt == 0) continue;
        if (!inputs[k] || !outputs[r]) return errors::InvalidArgument("null tensor with a non-zero element count");
        all.push_back(ring_row{at(outputs[r], starts[static_cast<size_t>(k)], esz), inputs[k], nullptr, cnt});
      }
    }
    RING_RETURN_IF_ERROR(ring_apply_rows_avg(all.data(), static_cast<int>(all.size()), nullptr, opts.divisor, code,
                                             stream),
                         "ring_apply_rows");
    return Status::OK();
  }

  Table<ring_row, kStackRanks> rows(static_cast<size_t>(n), ring_row{nullptr, nullptr, nullptr, 0});
  for (int r = 0; r < n; r++) {  // ring.h:263-266
    const size_t own = elems_per_row * rows_per_rank[static_cast<size_t>(r)];
    if (own && (!inputs[r] || !outputs[r])) return errors::InvalidArgument("null tensor with a non-zero element count");
    rows[static_cast<size_t>(r)] = ring_row{own ? at(outputs[r], starts[static_cast<size_t>(r)], esz) : nullptr, inputs[r], nullptr, own};
  }
  // every rank divides its own slice on the way into its output
  RING_RETURN_IF_ERROR(ring_apply_rows_avg(rows.data(), n, nullptr, opts.divisor, code, stream), "ring_apply_rows");
  for (int i = 0; i < n - 1; i++) {  // ring.h:279-298
    for (int r = 0; r < n; r++) {
      const int left = (r - 1 + n) % n;
      const size_t seg = static_cast<size_t>(Seg(RING_PHASE_GATHER, n, r, i, true));
      const size_t cnt = elems_per_row * rows_per_rank[seg];
      rows[static_cast<size_t>(r)] = ring_row{cnt ? at(outputs[r], starts[seg], esz) : nullptr,
                                              cnt ? at(static_cast<const void*>(outputs[left]), starts[seg], esz) : nullptr, nullptr, cnt};
    }
    RING_RETURN_IF_ERROR(ring_apply_rows(rows.data(), n, code, stream), "ring_apply_rows");
  }
  return Status::OK();
}

}  // namespace mpic
