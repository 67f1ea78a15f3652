// The MPI ops of tensorflow/contrib/mpi_collectives (mpi_ops.cc) for virtual
// ranks on one MI355X: op registrations, OpKernels, the per-op record, the
// readiness table with its validation messages, the background thread that
// performs every collective, and the C interface of include/mpi_collectives.h.
//
// What differs from the reference, on purpose:
//   * ranks are virtual (one process, one GPU), so the coordinator's MPI
//     messages (mpi_ops.cc:666-790) become in-process queue entries; the
//     request/response records and the validation rules are kept;
//   * the background thread sleeps on a condition variable instead of polling
//     every millisecond (mpi_ops.cc:635), and initialisation waits on a
//     predicate (the reference's cv.wait at :816-818 can miss its wake-up);
//   * there is no temp tensor: where MPI_Irecv would fill one (ring.h:189-200)
//     the incoming segment is read in place, from the neighbour's buffer or
//     from a pre-staged one;
//   * collectives only have GPU kernels. A CPU tensor is an error, not a
//     silent host path.
#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <thread>
#include <unordered_map>

#include "framework.h"
#include "mpi_collectives.h"
#include "ring_abi.h"
#include "ring_driver.h"
#include "transport.h"
#include "wire.h"

namespace mpic {
namespace {

using CPUDevice = struct CPUDeviceTag {};
using GPUDevice = struct GPUDeviceTag {};
template <typename T> bool IsGPUDevice();
template <> bool IsGPUDevice<GPUDevice>() { return true; }
template <> bool IsGPUDevice<CPUDevice>() { return false; }

// What ends a rank's part of a collective (mpi_ops.cc:119-121: a function of the
// status; here the two things every op's callback does, mpi_ops.cc:1084-1087,
// held in place: a std::function over them would allocate for every request).
struct CommunicationDoneCallback {
  OpKernelContext* context = nullptr;
  AsyncOpKernel::DoneCallback done;
  void operator()(const Status& status) const {
    context->SetStatus(status);
    done();
  }
};

// mpi_ops.cc:123-153
struct CollectiveOpRecord {
  int rank = 0;                   // the (virtual) rank performing this piece of the op
  // node name: the key collectives are matched by. The kernel's own string (the node outlives its
  // execution, op_kernel.h:187-189), not a copy per execution.
  const std::string* name = nullptr;
  OpKernelContext* context = nullptr;
  MPIDataType dtype = TF_MPI_INVALID_TYPE;
  const Tensor* in_t = nullptr;
  std::vector<size_t> sizes_vec;  // allgather: per-rank first-dimension sizes
  size_t temp_elements = 0;       // what the reference's temp tensor would hold (mpi_ops.cc:1073-1077)
  Tensor* out_t = nullptr;
  bool on_gpu = false;
  int divisor = 0;                // > 0: deliver tf.div(result, divisor) (a fused consumer)
  CommunicationDoneCallback callback;
};

struct StagedPeers {
  std::vector<const void*> rs, ag;
};

// The records of one collective, one per rank that lives in this process, in
// rank order: the contents of a map from rank to record, in one array.
class RankRecords {
 public:
  typedef std::pair<int, CollectiveOpRecord> value_type;
  typedef std::vector<value_type>::iterator iterator;
  typedef std::vector<value_type>::const_iterator const_iterator;
  iterator begin() { return v_.begin(); }
  iterator end() { return v_.end(); }
  const_iterator begin() const { return v_.begin(); }
  const_iterator end() const { return v_.end(); }
  size_t size() const { return v_.size(); }
  bool empty() const { return v_.empty(); }
  void clear() { v_.clear(); }
  void reserve(size_t n) { v_.reserve(n); }
  CollectiveOpRecord& operator[](int rank) {
    auto it = std::lower_bound(v_.begin(), v_.end(), rank, [](const value_type& e, int r) { return e.first < r; });
    if (it == v_.end() || it->first != rank) it = v_.emplace(it, rank, CollectiveOpRecord());
    return it->second;
  }
  // the record of a rank that is known to have one
  const CollectiveOpRecord& at(int rank) const {
    auto it = std::lower_bound(v_.begin(), v_.end(), rank, [](const value_type& e, int r) { return e.first < r; });
    return it->second;
  }

 private:
  std::vector<value_type> v_;
};

typedef std::unordered_map<std::string, RankRecords> TensorTable;
typedef std::unordered_map<std::string, std::vector<MPIRequest>> MessageTable;

}  // namespace
}  // namespace mpic

// mpi_ops.cc:165-240 (MPIGlobalState), one per world instead of one per process.
struct mpic_batch;
// Links between worlds and the batches built on them (either may be destroyed first).
static std::mutex g_batch_registry_mu;
// The batches built on a world outlive it as objects (their owner destroys them), but can no
// longer be submitted: mpic_batch_submit answers FAILED_PRECONDITION once this has run.
static void DetachBatches(mpic_world* w);

struct mpic_world {
  std::atomic_flag initialized_flag = ATOMIC_FLAG_INIT;
  std::condition_variable cv;       // initialisation
  std::condition_variable work_cv;  // requests for the background thread
  bool initialization_done = false;
  mpic::Status init_status;
  std::mutex mu;
  mpic::TensorTable tensor_table;
  // requests on their way to the coordinator, in wire format (the bytes a rank
  // in another process would send), each behind its length
  std::string message_bytes;
  std::thread background_thread;
  bool shut_down = false;
  mpic::MessageTable message_table;  // coordinator side
  std::unordered_map<std::string, mpic::StagedPeers> staged;
  int size = 1;
  int real_rank = -1;  // -1: every rank lives in this process
  int device = -1;     // -1 for no GPU
  void* stream = nullptr;
  // a world folds the in->out copy into the reduce-scatter unless told otherwise
  // (same results, a third fewer bytes)
  mpic::RingOptions ring_options = [] { mpic::RingOptions o; o.fuse_copy = true; o.direct = true; return o; }();
  bool sync_on_done = true;
  // Tensor fusion in the coordinator: allreduces that are ready in the same
  // tick are packed, per rank, into that rank's slice of this caller-owned
  // device buffer and reduced by one ring. Off while fusion_bytes == 0.
  void* fusion_buffer = nullptr;
  size_t fusion_bytes = 0;     // per rank
  bool flush_requested = false;  // with fusion on, a tick starts when the embedder asks
  std::map<std::string, ring_fusion_plan*> fusion_plans;  // keyed by the tensors' addresses and sizes
  // the batches built on this world (mpic_batch_create), so that destroying the world can tell them:
  // guarded by g_batch_registry_mu, not by mu
  std::vector<mpic_batch*> batches;

  int expected_requests() const { return real_rank >= 0 ? 1 : size; }
};

namespace mpic {
namespace {

// mpi_ops.cc:255-269
bool IncrementTensorCount(MessageTable* table, const MPIRequest& msg, int expected) {
  std::vector<MPIRequest>& v = (*table)[msg.tensor_name];
  if (v.empty()) v.reserve(static_cast<size_t>(expected));
  // the table's key is the name: the stored requests do not repeat it
  v.emplace_back();
  MPIRequest& stored = v.back();
  stored.request_rank = msg.request_rank;
  stored.request_type = msg.request_type;
  stored.tensor_type = msg.tensor_type;
  stored.tensor_shape = msg.tensor_shape;
  return static_cast<int>(v.size()) == expected;
}

TensorShape ShapeOf(const MPIRequest& r) { return TensorShape(r.tensor_shape); }

// mpi_ops.cc:277-432: all the cross-rank checks, with the reference's messages.
MPIResponse ConstructMPIResponse(MessageTable* table, const std::string& name) {
  bool error = false;
  const std::vector<MPIRequest>& requests = (*table)[name];
  std::string message;  // of the first check that fails
  auto fail = [&error, &message](std::string text) {
    error = true;
    message = std::move(text);
  };

  const MPIDataType data_type = requests[0].tensor_type;
  for (size_t i = 1; i < requests.size(); i++) {
    if (data_type != requests[i].tensor_type) {
      fail(std::string("Mismatched data types: One rank had type ") + MPIDataType_Name(data_type) +
           ", but another rank had type " + MPIDataType_Name(requests[i].tensor_type) + ".");
      break;
    }
  }

  const MPIRequest::RequestType message_type = requests[0].request_type;
  for (size_t i = 1; i < requests.size() && !error; i++) {
    if (message_type != requests[i].request_type) {
      fail("Mismatched MPI operations: One rank did an " + std::to_string(static_cast<int>(message_type)) +
           ", but another rank did an " + std::to_string(static_cast<int>(requests[i].request_type)) + ".");
    }
  }

  if (message_type == MPIRequest::ALLREDUCE) {
    for (size_t i = 1; i < requests.size() && !error; i++) {
      if (requests[0].tensor_shape != requests[i].tensor_shape) {
        fail("Mismatched allreduce tensor shapes: One rank reduced a tensor of shape " +
             ShapeOf(requests[0]).DebugString() + ", but another rank sent a tensor of shape " +
             ShapeOf(requests[i]).DebugString() + ".");
      }
    }
  }

  if (message_type == MPIRequest::ALLGATHER) {
    const TensorShape tensor_shape = ShapeOf(requests[0]);
    if (tensor_shape.dims() == 0 && !error) fail("Rank zero tried to gather a rank-zero tensor.");
    for (size_t i = 1; i < requests.size() && !error; i++) {
      const TensorShape request_shape = ShapeOf(requests[i]);
      if (tensor_shape.dims() != request_shape.dims()) {
        fail("Mismatched allgather tensor shapes: One rank gathered a tensor of rank " +
             std::to_string(tensor_shape.dims()) + ", but another rank sent a tensor of rank " +
             std::to_string(request_shape.dims()) + ".");
        break;
      }
      for (int dim = 1; dim < tensor_shape.dims(); dim++) {
        if (tensor_shape.dim_size(dim) != request_shape.dim_size(dim)) {
          fail("Mismatched allgather tensor shapes: One rank gathered a tensor with dimension " +
               std::to_string(dim) + " equal to " + std::to_string(tensor_shape.dim_size(dim)) +
               ", but another rank sent a tensor with dimension " + std::to_string(dim) + " equal to " +
               std::to_string(request_shape.dim_size(dim)) + ".");
          break;
        }
      }
    }
  }

  MPIResponse response;
  response.tensor_name = name;
  if (error) {
    response.response_type = MPIResponse::ERROR;
    response.error_message = std::move(message);
  } else {
    response.response_type =
        message_type == MPIRequest::ALLREDUCE ? MPIResponse::ALLREDUCE : MPIResponse::ALLGATHER;
  }
  table->erase(name);
  return response;
}

// The options an embedder may change while the background thread runs, read
// once per collective under the world's mutex.
struct WorldOptions {
  RingOptions ring;
  bool sync_on_done = true;
  void* fusion_buffer = nullptr;
  size_t fusion_bytes = 0;
};
WorldOptions SnapshotOptions(mpic_world* w) {
  std::lock_guard<std::mutex> guard(w->mu);
  WorldOptions o;
  o.ring = w->ring_options;
  o.sync_on_done = w->sync_on_done;
  o.fusion_buffer = w->fusion_buffer;
  o.fusion_bytes = w->fusion_bytes;
  return o;
}

// mpi_ops.cc:435-515: run the collective for every rank that lives here, then
// resume their ops.
// The end of a collective: its records are released BEFORE the waiting ops are
// told. A thread that is told starts its next step at once, and what this
// thread still had to free (several allocations per record, made by those
// threads) would then compete with it for the allocator: measured on 8 x 161
// gradients, the next step's submission took 1.6 ms instead of 0.4.
template <typename Records>
void FinishRecords(Records* records, std::vector<CommunicationDoneCallback>* callbacks, const Status& status) {
  records->clear();
  for (auto& done : *callbacks) {
    done(status);
    done = CommunicationDoneCallback();  // and its captured state, while the waiters still wait for the last ones
  }
}

// A collective whose launches are on the stream and whose ops wait for the
// stream to be synchronised.
struct EnqueuedCollective {
  RankRecords records;
  std::vector<CommunicationDoneCallback> callbacks;
};

// With `enqueued`, a collective that has been launched is left there for the
// caller to synchronise and finish (one synchronisation for all the collectives
// of a tick instead of one each); without, it is finished here.
void PerformCollectiveOp(mpic_world* w, const MPIResponse& response, std::vector<EnqueuedCollective>* enqueued) {
  const WorldOptions opt = SnapshotOptions(w);
  RankRecords records;
  StagedPeers peers;
  bool have_peers = false;
  {
    std::lock_guard<std::mutex> guard(w->mu);
    auto it = w->tensor_table.find(response.tensor_name);
    if (it == w->tensor_table.end()) return;
    records = std::move(it->second);
    w->tensor_table.erase(it);
    auto st = w->staged.find(response.tensor_name);
    if (st != w->staged.end()) {
      peers = std::move(st->second);
      w->staged.erase(st);
      have_peers = true;
    }
  }
  if (records.empty()) return;

  Status status;
  const CollectiveOpRecord& first = records.begin()->second;
  const DataType dtype = first.in_t->dtype();
  const int n = w->size;
  bool on_gpu = true, same_divisor = true;
  for (auto& kv : records) {
    on_gpu = on_gpu && kv.second.on_gpu;
    same_divisor = same_divisor && kv.second.divisor == first.divisor;
  }
  RingOptions ring = opt.ring;
  ring.divisor = first.divisor;

  if (response.response_type == MPIResponse::ERROR) {
    status = errors::FailedPrecondition(response.error_message);
  } else if (!same_divisor) {
    status = errors::FailedPrecondition("Mismatched fused divisors: ranks asked for different divisions of " +
                                        response.tensor_name + ".");
  } else if (dtype != DT_FLOAT && dtype != DT_INT32 && dtype != DT_INT64) {
    status = errors::Unknown(response.response_type == MPIResponse::ALLGATHER
                                 ? "Invalid tensor type for MPI allgather."
                                 : "Invalid tensor type for MPI allreduce.");
  } else if (!on_gpu) {
    status = errors::FailedPrecondition("MPI collectives have GPU kernels only; the tensor is in host memory.");
  } else if (w->real_rank >= 0) {
    const int r = w->real_rank;
    if (n > 1 && !have_peers) {
      status = errors::FailedPrecondition("No pre-staged peer segments for " + response.tensor_name + ".");
    } else if (n > 1 && (peers.ag.size() != static_cast<size_t>(n - 1) ||
                         (response.response_type == MPIResponse::ALLREDUCE &&
                          peers.rs.size() != static_cast<size_t>(n - 1)))) {
      status = errors::FailedPrecondition("Pre-staged peer segments for " + response.tensor_name +
                                          " do not cover the ring's n-1 steps.");
    } else if (response.response_type == MPIResponse::ALLREDUCE) {
      status = RingAllreducePrestaged(n, r, dtype, first.in_t->data(), first.out_t->data(),
                                      static_cast<size_t>(first.in_t->NumElements()), peers.rs.data(),
                                      peers.ag.data(), w->stream, ring);
    } else {
      size_t epr = 1;
      for (int i = 1; i < first.in_t->shape().dims(); i++) epr *= static_cast<size_t>(first.in_t->dim_size(i));
      status = RingAllgatherPrestaged(n, r, dtype, first.in_t->data(), first.sizes_vec, epr, first.out_t->data(),
                                      peers.ag.data(), w->stream, ring);
    }
  } else {
    std::vector<const void*> ins(static_cast<size_t>(n));
    std::vector<void*> outs(static_cast<size_t>(n));
    for (auto& kv : records) {
      ins[static_cast<size_t>(kv.first)] = kv.second.in_t->data();
      outs[static_cast<size_t>(kv.first)] = kv.second.out_t->data();
    }
    if (response.response_type == MPIResponse::ALLREDUCE) {
      status = RingAllreduceAllRanks(n, dtype, ins.data(), outs.data(),
                                     static_cast<size_t>(first.in_t->NumElements()), w->stream, ring);
    } else {
      size_t epr = 1;
      for (int i = 1; i < first.in_t->shape().dims(); i++) epr *= static_cast<size_t>(first.in_t->dim_size(i));
      // every rank computed the same sizes from the sizing gather; the first
      // dimension each one actually submitted must agree with them
      for (auto& kv : records) {
        if (kv.second.sizes_vec != first.sizes_vec ||
            static_cast<size_t>(kv.second.in_t->dim_size(0)) != first.sizes_vec[static_cast<size_t>(kv.first)]) {
          status = errors::FailedPrecondition("Allgather sizes do not match the gathered tensors' first dimensions.");
          break;
        }
      }
      if (status.ok())
        status = RingAllgatherAllRanks(n, dtype, ins.data(), first.sizes_vec, epr, outs.data(), w->stream,
                                       ring);
    }
  }

  std::vector<CommunicationDoneCallback> callbacks;
  callbacks.reserve(records.size());
  for (auto& kv : records) callbacks.push_back(std::move(kv.second.callback));
  if (status.ok() && opt.sync_on_done && response.response_type != MPIResponse::ERROR) {
    if (enqueued) {
      enqueued->push_back(EnqueuedCollective{std::move(records), std::move(callbacks)});
      return;
    }
    const int rc = ring_stream_synchronize(w->stream);
    if (rc != RING_OK) status = errors::Unknown("MPI operation failed unexpectedly.");  // ring.h:36-39
  }
  FinishRecords(&records, &callbacks, status);
}

constexpr size_t kMaxCachedFusionPlans = 256;
void DropFusionPlans(mpic_world* w) {
  ring_stream_synchronize(w->stream);  // launches in flight still read the plans' device tables
  for (auto& kv : w->fusion_plans) ring_fusion_plan_destroy(kv.second);
  w->fusion_plans.clear();
}

// A fusion plan for these tensors, created on first use. Training loops reduce
// the same gradient buffers every step, so plans are found again by the
// tensors' addresses and sizes; the table is dropped when it grows large.
ring_fusion_plan* FusionPlanFor(mpic_world* w, const std::vector<const void*>& ptrs,
                                const std::vector<size_t>& counts, int ring_dtype) {
  std::string key(reinterpret_cast<const char*>(ptrs.data()), ptrs.size() * sizeof(void*));
  key.append(reinterpret_cast<const char*>(counts.data()), counts.size() * sizeof(size_t));
  key.push_back(static_cast<char>(ring_dtype));
  auto it = w->fusion_plans.find(key);
  if (it != w->fusion_plans.end()) return it->second;
  if (w->fusion_plans.size() >= kMaxCachedFusionPlans) DropFusionPlans(w);
  ring_fusion_plan* plan = nullptr;
  if (ring_fusion_plan_create(ptrs.data(), counts.data(), static_cast<int>(ptrs.size()), ring_dtype, &plan) != RING_OK)
    return nullptr;
  w->fusion_plans[key] = plan;
  return plan;
}

// ring_fusion_allreduce_all addresses this many ranks' tensor tables in one launch
constexpr int kMaxFusedDirectRanks = 16;

// Tensor fusion (no counterpart in the reference, where every gradient is its
// own collective and its own negotiation round, __init__.py:195-205): the
// allreduces `names`, all ready and valid, of one element type, are packed per
// rank into that rank's fusion buffer in the order given, reduced by ONE ring
// in place, and unpacked into each op's output. The result of each tensor is
// the reference ring applied to the packed buffer.
void PerformFusedAllreduce(mpic_world* w, const std::vector<std::string>& names, const WorldOptions& opt) {
  const int n = w->size;
  std::vector<RankRecords> records;
  records.reserve(names.size());
  {
    std::lock_guard<std::mutex> guard(w->mu);
    for (const std::string& name : names) {
      auto it = w->tensor_table.find(name);
      records.push_back(std::move(it->second));
      w->tensor_table.erase(it);
    }
  }
  Status status;
  int code = 0;
  const DataType dtype = records[0].begin()->second.in_t->dtype();
  status = RingDataType(dtype, &code);
  std::vector<size_t> counts;
  size_t total = 0;
  for (auto& rec : records) {
    counts.push_back(static_cast<size_t>(rec.begin()->second.in_t->NumElements()));
    total += counts.back();
  }
  // fused tf.div consumers: when the whole group asks for the same division it
  // rides on the unpack, otherwise each tensor that asks for one is divided
  // after the unpack
  int divisor = records[0].begin()->second.divisor;
  bool uniform = true;
  for (auto& rec : records) {
    for (auto& kv : rec) {
      if (kv.second.divisor != rec.begin()->second.divisor)
        status = errors::FailedPrecondition("Mismatched fused divisors: ranks asked for different divisions of " +
                                            *kv.second.name + ".");
    }
    uniform = uniform && rec.begin()->second.divisor == divisor;
  }
  if (!uniform) divisor = 0;

  // Direct form: the ranks share the GPU, so the ring over the packed buffers is
  // computed on the tensors themselves, one launch, no fusion buffer (each
  // tensor still equals the reference ring applied to the packed buffer).
  if (status.ok() && opt.ring.direct && uniform && n <= kMaxFusedDirectRanks) {
    // all the plans of this launch must be alive together: make room first, so
    // that looking one up cannot drop the table under the ones already taken
    if (w->fusion_plans.size() + 2 * static_cast<size_t>(n) > kMaxCachedFusionPlans) DropFusionPlans(w);
    std::vector<const ring_fusion_plan*> in_plans, out_plans;
    for (int r = 0; r < n; r++) {
      std::vector<const void*> ins, outs;
      ins.reserve(records.size());
      outs.reserve(records.size());
      for (auto& rec : records) {
        ins.push_back(rec.at(r).in_t->data());
        outs.push_back(rec.at(r).out_t->data());
      }
      in_plans.push_back(FusionPlanFor(w, ins, counts, code));
      out_plans.push_back(ins == outs ? in_plans.back() : FusionPlanFor(w, outs, counts, code));
      if (!in_plans.back() || !out_plans.back()) status = errors::Unknown("MPI operation failed unexpectedly.");
    }
    if (status.ok() &&
        ring_fusion_allreduce_all(in_plans.data(), out_plans.data(), n, divisor, w->stream) != RING_OK)
      status = errors::Unknown("MPI operation failed unexpectedly.");
    if (status.ok() && opt.sync_on_done && ring_stream_synchronize(w->stream) != RING_OK)
      status = errors::Unknown("MPI operation failed unexpectedly.");
    std::vector<CommunicationDoneCallback> callbacks;
    callbacks.reserve(records.size() * static_cast<size_t>(n));
    for (auto& rec : records)
      for (auto& kv : rec) callbacks.push_back(std::move(kv.second.callback));
    FinishRecords(&records, &callbacks, status);
    return;
  }

  std::vector<void*> bufs(static_cast<size_t>(n));
  for (int r = 0; r < n && status.ok(); r++) {
    bufs[static_cast<size_t>(r)] = static_cast<char*>(opt.fusion_buffer) + static_cast<size_t>(r) * opt.fusion_bytes;
    std::vector<const void*> ins;
    for (auto& rec : records) ins.push_back(rec.at(r).in_t->data());
    ring_fusion_plan* plan = FusionPlanFor(w, ins, counts, code);
    if (!plan || ring_fusion_pack(plan, bufs[static_cast<size_t>(r)], w->stream) != RING_OK)
      status = errors::Unknown("MPI operation failed unexpectedly.");
  }
  if (status.ok()) {
    std::vector<const void*> ins(bufs.begin(), bufs.end());
    status = RingAllreduceAllRanks(n, dtype, ins.data(), bufs.data(), total, w->stream, opt.ring);
  }
  for (int r = 0; r < n && status.ok(); r++) {
    std::vector<const void*> outs;
    for (auto& rec : records) outs.push_back(rec.at(r).out_t->data());
    ring_fusion_plan* plan = FusionPlanFor(w, outs, counts, code);
    if (!plan || (divisor > 0 ? ring_fusion_unpack_scaled(plan, bufs[static_cast<size_t>(r)], divisor, w->stream)
                              : ring_fusion_unpack(plan, bufs[static_cast<size_t>(r)], w->stream)) != RING_OK)
      status = errors::Unknown("MPI operation failed unexpectedly.");
    for (auto& rec : records) {
      const CollectiveOpRecord& op = rec.at(r);
      if (uniform || op.divisor <= 0 || !status.ok()) continue;
      if (ring_scale(code, op.out_t->data(), static_cast<size_t>(op.out_t->NumElements()), op.divisor, w->stream) !=
          RING_OK)
        status = errors::Unknown("MPI operation failed unexpectedly.");
    }
  }
  if (status.ok() && opt.sync_on_done && ring_stream_synchronize(w->stream) != RING_OK)
    status = errors::Unknown("MPI operation failed unexpectedly.");
  std::vector<CommunicationDoneCallback> callbacks;
  for (auto& rec : records)
    for (auto& kv : rec) callbacks.push_back(std::move(kv.second.callback));
  FinishRecords(&records, &callbacks, status);
}

// One tick's ready collectives, in the order they became ready. With fusion on,
// runs of consecutive valid allreduces of one element type that fit the fusion
// buffer together are reduced as one; everything else goes one by one.
void PerformReady(mpic_world* w, const std::vector<std::string>& ready) {
  // Each response goes through its wire form, as it would to ranks in other
  // processes (mpi_ops.cc:727-739).
  std::vector<MPIResponse> responses;
  responses.reserve(ready.size());
  for (const std::string& name : ready) {
    MPIResponse received;
    if (received.ParseFromString(ConstructMPIResponse(&w->message_table, name).SerializeAsString()))
      responses.push_back(std::move(received));
  }
  const WorldOptions opt = SnapshotOptions(w);
  const bool fusing = opt.fusion_bytes > 0 && opt.fusion_buffer && w->real_rank < 0 && w->size > 1;
  // The reference synchronises the stream inside every device primitive
  // (ring.cu.cc:41-45, 60-69). Here a tick's collectives are all enqueued first
  // and the stream is synchronised once, before any of their ops is told: an op
  // still completes only when its result is there, and a tick of 161 small
  // gradients waits for the GPU once instead of 161 times.
  std::vector<EnqueuedCollective> enqueued;
  size_t i = 0;
  while (i < responses.size()) {
    std::vector<std::string> group;
    if (fusing && responses[i].response_type == MPIResponse::ALLREDUCE) {
      size_t bytes = 0;
      DataType group_dtype = DT_INVALID;
      size_t j = i;
      std::lock_guard<std::mutex> guard(w->mu);
      for (; j < responses.size() && responses[j].response_type == MPIResponse::ALLREDUCE; j++) {
        auto it = w->tensor_table.find(responses[j].tensor_name);
        if (it == w->tensor_table.end() || static_cast<int>(it->second.size()) != w->size) break;
        const CollectiveOpRecord& rec = it->second.begin()->second;
        bool on_gpu = true;
        for (auto& kv : it->second) on_gpu = on_gpu && kv.second.on_gpu;
        const DataType dt = rec.in_t->dtype();
        if (!on_gpu || DataTypeSize(dt) == 0 || dt == DT_DOUBLE) break;
        if (group.empty()) group_dtype = dt;
        // each tensor starts 16-byte aligned inside the buffer only by luck; the
        // pack/unpack kernels handle any element alignment, so bytes just add up
        if (dt != group_dtype || bytes + rec.in_t->TotalBytes() > opt.fusion_bytes) break;
        bytes += rec.in_t->TotalBytes();
        group.push_back(responses[j].tensor_name);
      }
    }
    if (group.size() >= 2) {
      PerformFusedAllreduce(w, group, opt);
      i += group.size();
    } else {
      PerformCollectiveOp(w, responses[i], &enqueued);
      i++;
    }
  }
  if (!enqueued.empty()) {
    Status status;
    if (ring_stream_synchronize(w->stream) != RING_OK)
      status = errors::Unknown("MPI operation failed unexpectedly.");  // ring.h:36-39
    for (EnqueuedCollective& e : enqueued) e.records.clear();  // all of them, before any waiter is told
    for (EnqueuedCollective& e : enqueued) FinishRecords(&e.records, &e.callbacks, status);
  }
}

// mpi_ops.cc:572-795. Ticks are driven by arrivals, not by a 1 ms sleep.
void BackgroundThreadLoop(mpic_world* w) {
  Status init;
  if (w->device >= 0) {
    // the dedicated stream (mpi_ops.cc:582-583)
    const int rc = ring_stream_create(&w->stream);
    if (rc != RING_OK)
      init = errors::Unknown(std::string("Could not create the MPI stream: ") + ring_status_string(rc));
  }
  {
    std::lock_guard<std::mutex> guard(w->mu);
    w->init_status = init;
    w->initialization_done = true;
  }
  w->cv.notify_all();
  if (!init.ok()) return;

  bool should_shut_down = false;
  // this tick's requests; the buffer goes back to the ranks at the next swap, so
  // that neither side allocates per request
  std::string message_bytes;
  do {
    message_bytes.clear();
    {
      std::unique_lock<std::mutex> lock(w->mu);
      // With fusion on a tick starts when the embedder asks for one (so the set of
      // tensors fused together, and with it the rounding of the sums, does not
      // depend on timing); otherwise every arrival starts one. (Counting the
      // requests while the ranks still submit them, ahead of the flush, was
      // measured and not kept: the two threads then compete for the allocator
      // and the queue, and a step's submission slows by more than its tick gains.)
      w->work_cv.wait(lock, [w] {
        const bool hold = w->fusion_bytes > 0 && !w->flush_requested;
        return w->shut_down || (!w->message_bytes.empty() && !hold);
      });
      std::swap(message_bytes, w->message_bytes);
      w->flush_requested = false;
      should_shut_down = w->shut_down;
    }
    std::vector<std::string> ready_to_reduce;
    size_t at = 0, size = 0;
    const char* data = nullptr;
    MPIRequest message;  // one for the whole tick: the storage of its name is reused
    while (NextRequestFrame(message_bytes, &at, &data, &size)) {
      if (message.ParseFromArray(data, size) &&
          IncrementTensorCount(&w->message_table, message, w->expected_requests()))
        ready_to_reduce.push_back(message.tensor_name);
    }
    PerformReady(w, ready_to_reduce);
  } while (!should_shut_down);

  // ops still waiting for absent ranks can never run: fail them
  TensorTable leftover;
  {
    std::lock_guard<std::mutex> guard(w->mu);
    leftover.swap(w->tensor_table);
  }
  for (auto& named : leftover)
    for (auto& kv : named.second) kv.second.callback(errors::Unknown("MPI was shut down before the collective ran."));
  if (w->stream) ring_stream_synchronize(w->stream);
  for (auto& kv : w->fusion_plans) ring_fusion_plan_destroy(kv.second);
  w->fusion_plans.clear();
  if (w->stream) {
    ring_stream_destroy(w->stream);
    w->stream = nullptr;
  }
}

// mpi_ops.cc:799-824
Status InitializeMPIOnce(mpic_world* w, bool gpu) {
  if (w->initialized_flag.test_and_set()) {
    std::unique_lock<std::mutex> lock(w->mu);
    w->cv.wait(lock, [w] { return w->initialization_done; });
    return w->init_status;
  }
  w->device = gpu ? 0 : -1;
  w->background_thread = std::thread(BackgroundThreadLoop, w);
  std::unique_lock<std::mutex> lock(w->mu);
  w->cv.wait(lock, [w] { return w->initialization_done; });
  return w->init_status;
}

// mpi_ops.cc:827-833
Status IsMPIInitialized(mpic_world* w) {
  std::lock_guard<std::mutex> guard(w->mu);
  if (!w->initialization_done)
    return errors::FailedPrecondition("MPI has not been initialized; use tf.contrib.mpi.Session.");
  return w->init_status;
}

// mpi_ops.cc:836-847
Status DataTypeToMPIType(DataType tf_dtype, MPIDataType* mpi_dtype) {
  if (tf_dtype == DT_FLOAT) *mpi_dtype = TF_MPI_FLOAT32;
  else if (tf_dtype == DT_INT32) *mpi_dtype = TF_MPI_INT32;
  else if (tf_dtype == DT_INT64) *mpi_dtype = TF_MPI_INT64;
  else return errors::FailedPrecondition("Invalid tensor type passed.");
  return Status::OK();
}

// mpi_ops.cc:853-868
void EnqueueTensorCollective(mpic_world* w, CollectiveOpRecord record, MPIRequest::RequestType rtype) {
  bool wake;
  {
    std::lock_guard<std::mutex> guard(w->mu);
    // the MPIRequest of mpi_ops.cc:855-863, written straight into its wire form
    AppendRequestFrame(&w->message_bytes, record.rank, rtype, record.dtype, *record.name,
                       record.in_t->shape().dim_sizes());
    RankRecords& by_rank = w->tensor_table[*record.name];
    if (by_rank.empty()) by_rank.reserve(static_cast<size_t>(w->expected_requests()));
    const int rank = record.rank;
    by_rank[rank] = std::move(record);
    // with fusion on, requests wait for a flush: waking the thread for each
    // would only have it look at the queue and go back to sleep
    wake = !(w->fusion_bytes > 0 && !w->flush_requested);
  }
  if (wake) w->work_cv.notify_one();
}

// Dimensions that come from outside (an embedder's tensors, an allgather's
// sizes): none negative, and a byte size that fits 63 bits (8-byte elements at
// most), so that no size computed from them wraps.
bool DimsFit(const int64_t* dims, int ndims) {
  uint64_t elements = 1;
  for (int i = 0; i < ndims; i++) {
    if (dims[i] < 0) return false;
    const uint64_t d = static_cast<uint64_t>(dims[i]);
    if (d != 0 && elements > (static_cast<uint64_t>(INT64_MAX) / 8) / d) return false;
    elements *= d;
  }
  return true;
}

mpic_world* WorldOf(OpKernelContext* context) { return static_cast<mpic_world*>(context->world()); }

// ---- ops -------------------------------------------------------------------------

// mpi_ops.cc:880-907
template <typename Device>
class MPIInitOp : public OpKernel {
 public:
  explicit MPIInitOp(OpKernelConstruction* context) : OpKernel(context) {}
  void Compute(OpKernelContext* context) override {
    OP_REQUIRES_OK(context, InitializeMPIOnce(WorldOf(context), IsGPUDevice<Device>()));
  }
};
REGISTER_KERNEL_BUILDER(Name("MPIInit").Device(DEVICE_CPU), MPIInitOp<CPUDevice>);
REGISTER_KERNEL_BUILDER(Name("MPIInit").Device(DEVICE_GPU), MPIInitOp<GPUDevice>);
REGISTER_OP("MPIInit").Doc(R"doc(
Initialize MPI for the current process.

If this is run on a GPU, then that GPU must be used for all future MPI
operations. If it is run on CPU, then all future MPI operations must also
run on CPU.
)doc");

// A scalar int32 in host memory (the GPU kernels of these three ops pin their
// output to the host, mpi_ops.cc:933, 975, 1018-1020).
void ScalarOutput(OpKernelContext* context, int value) {
  OP_REQUIRES_OK(context, IsMPIInitialized(WorldOf(context)));
  Tensor* output = nullptr;
  OP_REQUIRES_OK(context, context->allocate_output(0, TensorShape(), DT_INT32, true, &output));
  *static_cast<int32_t*>(output->data()) = value;
}

// mpi_ops.cc:910-950
template <typename Device>
class MPISizeOp : public OpKernel {
 public:
  explicit MPISizeOp(OpKernelConstruction* context) : OpKernel(context) {}
  void Compute(OpKernelContext* context) override { ScalarOutput(context, WorldOf(context)->size); }
};
REGISTER_KERNEL_BUILDER(Name("MPISize").Device(DEVICE_CPU), MPISizeOp<CPUDevice>);
REGISTER_KERNEL_BUILDER(Name("MPISize").Device(DEVICE_GPU).HostMemory("size"), MPISizeOp<GPUDevice>);
REGISTER_OP("MPISize")
    .Output("size: int32")
    .SetShapeFn([](const std::vector<int64_t>&, std::vector<int64_t>* out) { out->clear(); return Status::OK(); })
    .Doc(R"doc(
Returns the number of running MPI processes.

More precisely, returns the number of MPI processes in the group associated
with the MPI_COMM_WORLD communicator.

size:   Size of the MPI group.
)doc");

// mpi_ops.cc:953-992
template <typename Device>
class MPIRankOp : public OpKernel {
 public:
  explicit MPIRankOp(OpKernelConstruction* context) : OpKernel(context) {}
  void Compute(OpKernelContext* context) override { ScalarOutput(context, context->rank()); }
};
REGISTER_KERNEL_BUILDER(Name("MPIRank").Device(DEVICE_CPU), MPIRankOp<CPUDevice>);
REGISTER_KERNEL_BUILDER(Name("MPIRank").Device(DEVICE_GPU).HostMemory("rank"), MPIRankOp<GPUDevice>);
REGISTER_OP("MPIRank")
    .Output("rank: int32")
    .SetShapeFn([](const std::vector<int64_t>&, std::vector<int64_t>* out) { out->clear(); return Status::OK(); })
    .Doc(R"doc(
Returns the index of the current process in the MPI group.

More precisely, returns the rank of the calling process in the MPI_COMM_WORLD
communicator.

rank:   Rank of the calling process.
)doc");

// mpi_ops.cc:996-1037. All virtual ranks share one node, so the local rank is
// the rank.
template <typename Device>
class MPILocalRankOp : public OpKernel {
 public:
  explicit MPILocalRankOp(OpKernelConstruction* context) : OpKernel(context) {}
  void Compute(OpKernelContext* context) override { ScalarOutput(context, context->rank()); }
};
REGISTER_KERNEL_BUILDER(Name("MPILocalRank").Device(DEVICE_CPU), MPILocalRankOp<CPUDevice>);
REGISTER_KERNEL_BUILDER(Name("MPILocalRank").Device(DEVICE_GPU).HostMemory("rank"), MPILocalRankOp<GPUDevice>);
REGISTER_OP("MPILocalRank")
    .Output("rank: int32")
    .SetShapeFn([](const std::vector<int64_t>&, std::vector<int64_t>* out) { out->clear(); return Status::OK(); })
    .Doc(R"doc(
Returns the index of the current process in the node it is on.

More precisely, returns the rank of the calling process in communicator that
only spans the MPI processes running on that node.

rank:   Rank of the calling process on the node it is on.
)doc");

// mpi_ops.cc:1039-1139
template <typename Device>
class MPIAllreduceOp : public AsyncOpKernel {
 public:
  explicit MPIAllreduceOp(OpKernelConstruction* context) : AsyncOpKernel(context) {}
  // ComputeAsync only files a record for the background thread.
  bool IsExpensive() override { return false; }

  void ComputeAsync(OpKernelContext* context, DoneCallback done) override {
    mpic_world* world = WorldOf(context);
    OP_REQUIRES_OK_ASYNC(context, IsMPIInitialized(world), done);
    OP_REQUIRES_OK_ASYNC(context,
                         context->num_inputs() == 1 ? Status::OK()
                                                    : errors::InvalidArgument("MPIAllreduce takes one input."),
                         done);
    const Tensor* input_tensor = &context->input(0);

    CollectiveOpRecord record;
    record.dtype = TF_MPI_INVALID_TYPE;
    OP_REQUIRES_OK_ASYNC(context, DataTypeToMPIType(input_tensor->dtype(), &record.dtype), done);

    Tensor* output_tensor = nullptr;
    OP_REQUIRES_OK_ASYNC(
        context, context->allocate_output(0, input_tensor->shape(), input_tensor->dtype(), false, &output_tensor),
        done);

    record.rank = context->rank();
    record.name = &name();
    record.context = context;
    record.in_t = input_tensor;
    record.out_t = output_tensor;
    record.on_gpu = IsGPUDevice<Device>() && !input_tensor->host_memory();
    record.temp_elements = ring_temp_elements(static_cast<size_t>(input_tensor->NumElements()), world->size);
    record.divisor = context->fused_divisor();
    record.callback.context = context;
    record.callback.done = done;
    // The caller's producer work is ordered before the collective by the
    // embedding framework (the reference defers this call with a stream host
    // callback, mpi_ops.cc:1099-1105).
    EnqueueTensorCollective(world, std::move(record), MPIRequest::ALLREDUCE);
  }
};
REGISTER_KERNEL_BUILDER(Name("MPIAllreduce").Device(DEVICE_GPU), MPIAllreduceOp<GPUDevice>);
REGISTER_OP("MPIAllreduce")
    .Attr("T: {int32, int64, float32}")
    .Input("tensor: T")
    .Output("sum: T")
    .SetShapeFn([](const std::vector<int64_t>& in, std::vector<int64_t>* out) { *out = in; return Status::OK(); })
    .Doc(R"doc(
Perform an MPI Allreduce on a tensor. All other processes that do a reduction
on a tensor with the same name must have the same dimension for that tensor.
Tensors are reduced with other tensors that have the same node name for the
allreduce.

Arguments
    tensor:     A tensor to reduce.

Output
    sum:        A tensor with the same shape as `tensor`, summed across all
                MPI processes.
)doc");

// mpi_ops.cc:1141-1270
template <typename Device>
class MPIAllgatherOp : public AsyncOpKernel {
 public:
  explicit MPIAllgatherOp(OpKernelConstruction* context) : AsyncOpKernel(context) {}
  bool IsExpensive() override { return false; }

  void ComputeAsync(OpKernelContext* context, DoneCallback done) override {
    mpic_world* world = WorldOf(context);
    OP_REQUIRES_OK_ASYNC(context, IsMPIInitialized(world), done);
    OP_REQUIRES_OK_ASYNC(context,
                         context->num_inputs() == 2 ? Status::OK()
                                                    : errors::InvalidArgument("MPIAllgather takes two inputs."),
                         done);
    const Tensor* input_tensor = &context->input(0);
    const Tensor* sizing_tensor = &context->input(1);

    CollectiveOpRecord record;
    record.rank = context->rank();
    record.name = &name();
    record.context = context;
    record.in_t = input_tensor;
    record.on_gpu = IsGPUDevice<Device>() && !input_tensor->host_memory();

    // A scalar sizing tensor means one element per rank (the sizing pre-pass,
    // mpi_ops.cc:1167-1173); otherwise it lists every rank's first dimension
    // and lives in host memory (:1176-1183).
    size_t output_first_dim = 0;
    if (sizing_tensor->shape().dims() == 0) {
      output_first_dim = static_cast<size_t>(world->size);
      record.sizes_vec.assign(static_cast<size_t>(world->size), 1);
    } else {
      OP_REQUIRES_OK_ASYNC(
          context,
          (sizing_tensor->host_memory() && sizing_tensor->dtype() == DT_INT64 &&
           sizing_tensor->NumElements() >= world->size)
              ? Status::OK()
              : errors::InvalidArgument("sizes must be an int64 host tensor with one entry per rank."),
          done);
      const int64_t* sizing_array = static_cast<const int64_t*>(sizing_tensor->data());
      bool sizes_fit = true;
      for (int i = 0; i < world->size; i++) {
        sizes_fit = sizes_fit && sizing_array[i] >= 0 &&
                    static_cast<uint64_t>(sizing_array[i]) <= static_cast<uint64_t>(INT64_MAX) / 8 - output_first_dim;
        if (!sizes_fit) break;
        record.sizes_vec.push_back(static_cast<size_t>(sizing_array[i]));
        output_first_dim += static_cast<size_t>(sizing_array[i]);
      }
      OP_REQUIRES_OK_ASYNC(
          context,
          sizes_fit ? Status::OK()
                    : errors::InvalidArgument("sizes must be non-negative and add up to a tensor's first dimension."),
          done);
    }

    record.dtype = TF_MPI_INVALID_TYPE;
    OP_REQUIRES_OK_ASYNC(context, DataTypeToMPIType(input_tensor->dtype(), &record.dtype), done);

    TensorShape output_shape;
    output_shape.AddDim(static_cast<int64_t>(output_first_dim));
    for (int i = 1; i < input_tensor->shape().dims(); i++) output_shape.AddDim(input_tensor->dim_size(i));
    OP_REQUIRES_OK_ASYNC(context,
                         DimsFit(output_shape.dim_sizes().data(), output_shape.dims())
                             ? Status::OK()
                             : errors::InvalidArgument("the gathered tensor is too large."),
                         done);
    Tensor* output_tensor = nullptr;
    OP_REQUIRES_OK_ASYNC(context,
                         context->allocate_output(0, output_shape, input_tensor->dtype(), false, &output_tensor), done);
    record.out_t = output_tensor;
    record.divisor = context->fused_divisor();
    record.callback.context = context;
    record.callback.done = done;
    EnqueueTensorCollective(world, std::move(record), MPIRequest::ALLGATHER);
  }
};
REGISTER_OP("MPIAllgather")
    .Attr("T: {int32, int64, float32}")
    .Attr("S: {int64}")
    .Input("tensor: T")
    .Input("sizes: S")
    .Output("gathered: T")
    .SetShapeFn([](const std::vector<int64_t>& in, std::vector<int64_t>* out) {
      if (in.empty()) return errors::InvalidArgument("Shape must be at least rank 1 but is rank 0");
      *out = in;
      (*out)[0] = -1;  // ReplaceDim(input, 0, UnknownDim)
      return Status::OK();
    })
    .Doc(R"doc(
Perform an MPI Allgather on a tensor. All other processes that do a gather on a
tensor with the same name must have the same rank for that tensor, and have the
same dimension on all but the first dimension.

Arguments
    tensor:     A tensor to gather.
    sizes:      A tensor containing the first-dimension sizes of tensors to be
                gathered from other ranks

Output
    gathered:   A tensor with the same shape as `tensor` except for the first
                dimension, which is the sum of dimensions in `sizes`.
)doc");
REGISTER_KERNEL_BUILDER(Name("MPIAllgather").Device(DEVICE_GPU).HostMemory("sizes"), MPIAllgatherOp<GPUDevice>);

thread_local std::string g_last_error;
int Fail(const Status& s) {
  g_last_error = s.error_message();
  return static_cast<int>(s.code());
}

}  // namespace
}  // namespace mpic

// =============================================================================
// C interface
// =============================================================================
struct mpic_context {
  std::unique_ptr<mpic::OpKernelContext> ctx;
  std::unique_ptr<mpic::OpKernel> kernel;
  std::mutex mu;
  std::condition_variable cv;
  bool started = false;
  bool done = false;
};

using mpic::OpRegistry;

extern "C" {

int mpic_op_count(void) { return static_cast<int>(OpRegistry::Global()->op_names().size()); }

const char* mpic_op_name(int index) {
  const auto& names = OpRegistry::Global()->op_names();
  if (index < 0 || static_cast<size_t>(index) >= names.size()) return nullptr;
  return names[static_cast<size_t>(index)].c_str();
}

const char* mpic_op_signature(const char* op) {
  static thread_local std::string text;
  const mpic::OpDef* def = op ? OpRegistry::Global()->LookUp(op) : nullptr;
  if (!def) return nullptr;
  text = def->Signature();
  return text.c_str();
}

const char* mpic_op_doc(const char* op) {
  const mpic::OpDef* def = op ? OpRegistry::Global()->LookUp(op) : nullptr;
  return def ? def->doc.c_str() : nullptr;
}

int mpic_op_has_kernel(const char* op, const char* device) {
  return op && device && OpRegistry::Global()->FindKernel(op, device) ? 1 : 0;
}

int mpic_op_infer_shape(const char* op, int ndims, const int64_t* dims, int64_t* out_dims) {
  const mpic::OpDef* def = op ? OpRegistry::Global()->LookUp(op) : nullptr;
  if (!def || !def->shape_fn || def->outputs.empty() || ndims < 0) return -1;
  std::vector<int64_t> in(dims, dims + ndims), out;
  if (!def->shape_fn(in, &out).ok()) return -1;
  for (size_t i = 0; i < out.size(); i++) out_dims[i] = out[i];
  return static_cast<int>(out.size());
}

static int world_create(int size, int rank, mpic_world** world) {
  if (!world || size < 1 || rank >= size) return MPIC_INVALID_ARGUMENT;
  mpic_world* w = new mpic_world();
  w->size = size;
  w->real_rank = rank;
  *world = w;
  return MPIC_OK;
}

int mpic_world_create(int size, mpic_world** world) { return world_create(size, -1, world); }

int mpic_world_create_prestaged(int size, int rank, mpic_world** world) {
  if (rank < 0) return MPIC_INVALID_ARGUMENT;
  return world_create(size, rank, world);
}

int mpic_world_destroy(mpic_world* w) {
  if (!w) return MPIC_OK;
  if (w->background_thread.joinable()) {
    {
      std::lock_guard<std::mutex> guard(w->mu);
      w->shut_down = true;
    }
    w->work_cv.notify_all();
    w->background_thread.join();
  }
  DetachBatches(w);
  delete w;
  return MPIC_OK;
}

int mpic_world_size(const mpic_world* w) { return w ? w->size : 0; }
void* mpic_world_stream(const mpic_world* w) { return w ? w->stream : nullptr; }

int mpic_world_set_option(mpic_world* w, const char* name, int value) {
  if (!w || !name) return MPIC_INVALID_ARGUMENT;
  std::lock_guard<std::mutex> guard(w->mu);
  if (!strcmp(name, "batched")) w->ring_options.batched = value != 0;
  else if (!strcmp(name, "fuse_copy")) w->ring_options.fuse_copy = value != 0;
  else if (!strcmp(name, "direct")) w->ring_options.direct = value != 0;
  else if (!strcmp(name, "sync")) w->sync_on_done = value != 0;
  else return MPIC_INVALID_ARGUMENT;
  return MPIC_OK;
}

int mpic_world_set_fusion_buffer(mpic_world* w, void* buffer, size_t bytes_per_rank) {
  if (!w || (bytes_per_rank > 0 && (!buffer || (reinterpret_cast<uintptr_t>(buffer) & 15u) || (bytes_per_rank & 15u))))
    return MPIC_INVALID_ARGUMENT;
  {
    std::lock_guard<std::mutex> guard(w->mu);
    w->fusion_buffer = bytes_per_rank ? buffer : nullptr;
    w->fusion_bytes = bytes_per_rank;
  }
  w->work_cv.notify_all();
  return MPIC_OK;
}

int mpic_world_flush(mpic_world* w) {
  if (!w) return MPIC_INVALID_ARGUMENT;
  {
    std::lock_guard<std::mutex> guard(w->mu);
    w->flush_requested = true;
  }
  w->work_cv.notify_all();
  return MPIC_OK;
}

int mpic_stage_peers(mpic_world* w, const char* name, const void* const* rs_segments,
                     const void* const* ag_segments) {
  if (!w || !name || w->real_rank < 0 || (w->size > 1 && !ag_segments)) return MPIC_INVALID_ARGUMENT;
  mpic::StagedPeers peers;
  for (int i = 0; i < w->size - 1; i++) {
    if (rs_segments) peers.rs.push_back(rs_segments[i]);
    peers.ag.push_back(ag_segments[i]);
  }
  std::lock_guard<std::mutex> guard(w->mu);
  w->staged[name] = std::move(peers);
  return MPIC_OK;
}

int mpic_context_create(mpic_world* world, int rank, const char* op, const char* node_name, const char* device,
                        mpic_alloc_fn alloc, void* user, mpic_context** out) {
  if (!world || !op || !device || !out) return MPIC_INVALID_ARGUMENT;
  if (rank < 0 || rank >= world->size || (world->real_rank >= 0 && rank != world->real_rank))
    return MPIC_INVALID_ARGUMENT;
  if (!OpRegistry::Global()->LookUp(op)) return MPIC_NOT_FOUND;
  const mpic::KernelDef* kdef = OpRegistry::Global()->FindKernel(op, device);
  if (!kdef) return MPIC_NOT_FOUND;  // "No OpKernel was registered to support Op ... on this device"
  mpic_context* c = new mpic_context();
  mpic::OpKernelConstruction construction(node_name && *node_name ? node_name : op);
  c->kernel.reset(kdef->factory(&construction));
  mpic::OutputAllocator allocator;
  if (alloc) {
    allocator = [alloc, user](mpic::DataType dt, const mpic::TensorShape& shape, bool host) -> void* {
      return alloc(user, static_cast<int>(dt), shape.dims(), shape.dim_sizes().data(), host ? 1 : 0);
    };
  }
  c->ctx.reset(new mpic::OpKernelContext(world, rank, !strcmp(device, "GPU"), allocator));
  *out = c;
  return MPIC_OK;
}

int mpic_context_add_input(mpic_context* c, int dtype, int ndims, const int64_t* dims, const void* data,
                           int host_memory) {
  if (!c || c->started || ndims < 0 || ndims > 8 || (ndims > 0 && !dims)) return MPIC_INVALID_ARGUMENT;
  if (!mpic::DimsFit(dims, ndims)) return MPIC_INVALID_ARGUMENT;
  std::vector<int64_t> d(dims, dims + ndims);
  c->ctx->AddInput(mpic::Tensor(static_cast<mpic::DataType>(dtype), mpic::TensorShape(d), const_cast<void*>(data),
                                host_memory != 0));
  return MPIC_OK;
}

int mpic_context_set_divisor(mpic_context* c, int divisor) {
  if (!c || c->started || divisor < 0) return MPIC_INVALID_ARGUMENT;
  c->ctx->set_fused_divisor(divisor);
  return MPIC_OK;
}

int mpic_context_compute(mpic_context* c) {
  if (!c || c->started) return MPIC_INVALID_ARGUMENT;
  c->started = true;
  auto done = [c] {
    // notify under the lock: the waiter may destroy the context as soon as it
    // sees `done`, so nothing of the context is touched after the unlock
    std::lock_guard<std::mutex> guard(c->mu);
    c->done = true;
    c->cv.notify_all();
  };
  if (c->kernel->IsAsync()) {
    static_cast<mpic::AsyncOpKernel*>(c->kernel.get())->ComputeAsync(c->ctx.get(), done);
  } else {
    c->kernel->Compute(c->ctx.get());
    done();
  }
  return MPIC_OK;
}

int mpic_context_wait(mpic_context* c) {
  if (!c || !c->started) return MPIC_INVALID_ARGUMENT;
  std::unique_lock<std::mutex> lock(c->mu);
  c->cv.wait(lock, [c] { return c->done; });
  return static_cast<int>(c->ctx->status().code());
}

const char* mpic_context_message(const mpic_context* c) {
  return c ? c->ctx->status().error_message().c_str() : "";
}

int mpic_context_num_outputs(const mpic_context* c) { return c ? c->ctx->num_outputs() : 0; }

int mpic_context_output(const mpic_context* c, int index, int* dtype, int* ndims, int64_t* dims, void** data) {
  if (!c || index < 0 || index >= c->ctx->num_outputs()) return MPIC_INVALID_ARGUMENT;
  const mpic::Tensor* t = c->ctx->output(index);
  if (!t) return MPIC_INVALID_ARGUMENT;
  if (dtype) *dtype = static_cast<int>(t->dtype());
  if (ndims) *ndims = t->shape().dims();
  if (dims) for (int i = 0; i < t->shape().dims() && i < 8; i++) dims[i] = t->dim_size(i);
  if (data) *data = t->data();
  return MPIC_OK;
}

int mpic_context_done(mpic_context* c) {
  if (!c) return 1;
  if (!c->started) return 1;
  std::lock_guard<std::mutex> lock(c->mu);
  return c->done ? 1 : 0;
}

int mpic_context_destroy(mpic_context* c) {
  if (!c) return MPIC_OK;
  if (c->started) {  // never free a context the background thread may still call back into
    std::unique_lock<std::mutex> lock(c->mu);
    c->cv.wait(lock, [c] { return c->done; });
  }
  delete c;
  return MPIC_OK;
}

// ---- many MPIAllreduce nodes in one call ------------------------------------------------

int mpic_allreduce_batch(mpic_world* world, int rank, int k, const char* const* node_names, const int* dtypes,
                         const int* ndims, const int64_t* dims, const void* const* inputs, void* const* outputs,
                         int divisor, mpic_context** contexts) {
  if (!world || k < 0 || divisor < 0) return MPIC_INVALID_ARGUMENT;
  if (k > 0 && (!node_names || !dtypes || !ndims || !inputs || !outputs || !contexts)) return MPIC_INVALID_ARGUMENT;
  if (rank < 0 || rank >= world->size || (world->real_rank >= 0 && rank != world->real_rank))
    return MPIC_INVALID_ARGUMENT;
  const mpic::KernelDef* kdef = OpRegistry::Global()->FindKernel("MPIAllreduce", "GPU");
  if (!kdef) return MPIC_NOT_FOUND;
  size_t at = 0;
  for (int j = 0; j < k; j++) {
    if (ndims[j] < 0 || ndims[j] > 8 || (ndims[j] > 0 && !dims) || !node_names[j] ||
        !mpic::DimsFit(dims + at, ndims[j])) {
      for (int i = 0; i < j; i++) { delete contexts[i]; contexts[i] = nullptr; }
      return MPIC_INVALID_ARGUMENT;
    }
    mpic_context* c = new mpic_context();
    mpic::OpKernelConstruction construction(*node_names[j] ? node_names[j] : "MPIAllreduce");
    c->kernel.reset(kdef->factory(&construction));
    void* out = outputs[j];
    // the node's one output has the input's shape: the caller supplies its memory
    mpic::OutputAllocator allocator = [out](mpic::DataType, const mpic::TensorShape&, bool) -> void* { return out; };
    c->ctx.reset(new mpic::OpKernelContext(world, rank, true, allocator));
    std::vector<int64_t> d(dims + at, dims + at + ndims[j]);
    at += static_cast<size_t>(ndims[j]);
    c->ctx->AddInput(mpic::Tensor(static_cast<mpic::DataType>(dtypes[j]), mpic::TensorShape(d),
                                  const_cast<void*>(inputs[j]), false));
    c->ctx->set_fused_divisor(divisor);
    contexts[j] = c;
  }
  for (int j = 0; j < k; j++) mpic_context_compute(contexts[j]);
  return MPIC_OK;
}

int mpic_context_wait_batch(mpic_context** contexts, int k, int destroy_ok, int* codes) {
  if (k < 0 || (k > 0 && !contexts)) return MPIC_INVALID_ARGUMENT;
  int first = MPIC_OK;
  for (int j = 0; j < k; j++) {
    if (!contexts[j]) continue;
    const int code = mpic_context_wait(contexts[j]);
    if (codes) codes[j] = code;
    if (code != MPIC_OK && first == MPIC_OK) first = code;
    if (code == MPIC_OK && destroy_ok) {
      mpic_context_destroy(contexts[j]);
      contexts[j] = nullptr;
    }
  }
  return first;
}

// ---- a rank's MPIAllreduce nodes, built once and run every step ---------------------------

struct mpic_batch {
  // null once the world has been destroyed: the nodes' contexts still point at it, so the batch
  // may only be waited for and destroyed from then on
  std::atomic<mpic_world*> world{nullptr};
  int rank = 0;
  // the graph's nodes: kernels are constructed once, as a TensorFlow graph's are,
  // and every submission is one execution of each
  std::vector<std::unique_ptr<mpic::OpKernel>> kernels;
  std::vector<std::unique_ptr<mpic::OpKernelContext>> contexts;
  std::mutex mu;
  std::condition_variable cv;
  int outstanding = 0;  // nodes of the current submission that have not called done()
};

}  // extern "C"
static void DetachBatches(mpic_world* w) {
  std::lock_guard<std::mutex> registry(g_batch_registry_mu);
  for (mpic_batch* b : w->batches) b->world.store(nullptr);
  w->batches.clear();
}
extern "C" {

int mpic_batch_create(mpic_world* world, int rank, int k, const char* const* node_names, const int* dtypes,
                      const int* ndims, const int64_t* dims, const void* const* inputs, void* const* outputs,
                      int divisor, mpic_batch** batch) {
  if (!world || !batch || k < 0 || divisor < 0) return MPIC_INVALID_ARGUMENT;
  if (k > 0 && (!node_names || !dtypes || !ndims || !inputs || !outputs)) return MPIC_INVALID_ARGUMENT;
  if (rank < 0 || rank >= world->size || (world->real_rank >= 0 && rank != world->real_rank))
    return MPIC_INVALID_ARGUMENT;
  const mpic::KernelDef* kdef = OpRegistry::Global()->FindKernel("MPIAllreduce", "GPU");
  if (!kdef) return MPIC_NOT_FOUND;
  std::unique_ptr<mpic_batch> b(new mpic_batch());
  b->world = world;
  b->rank = rank;
  size_t at = 0;
  for (int j = 0; j < k; j++) {
    if (ndims[j] < 0 || ndims[j] > 8 || (ndims[j] > 0 && !dims) || !node_names[j] || !mpic::DimsFit(dims + at, ndims[j]))
      return MPIC_INVALID_ARGUMENT;
    mpic::OpKernelConstruction construction(*node_names[j] ? node_names[j] : "MPIAllreduce");
    b->kernels.emplace_back(kdef->factory(&construction));
    void* out = outputs[j];
    mpic::OutputAllocator allocator = [out](mpic::DataType, const mpic::TensorShape&, bool) -> void* { return out; };
    b->contexts.emplace_back(new mpic::OpKernelContext(world, rank, true, allocator));
    std::vector<int64_t> d(dims + at, dims + at + ndims[j]);
    at += static_cast<size_t>(ndims[j]);
    b->contexts.back()->AddInput(mpic::Tensor(static_cast<mpic::DataType>(dtypes[j]), mpic::TensorShape(d),
                                              const_cast<void*>(inputs[j]), false));
    b->contexts.back()->set_fused_divisor(divisor);
  }
  {
    std::lock_guard<std::mutex> registry(g_batch_registry_mu);
    world->batches.push_back(b.get());
  }
  *batch = b.release();
  return MPIC_OK;
}

int mpic_batch_size(const mpic_batch* b) { return b ? static_cast<int>(b->kernels.size()) : 0; }

int mpic_batch_submit(mpic_batch* b) {
  if (!b) return MPIC_INVALID_ARGUMENT;
  if (b->world.load() == nullptr) {
    mpic::g_last_error = "the world this batch was built on has been destroyed";
    return MPIC_FAILED_PRECONDITION;
  }
  {
    std::lock_guard<std::mutex> guard(b->mu);
    if (b->outstanding != 0) {
      mpic::g_last_error = "the batch's previous submission has not finished";
      return MPIC_FAILED_PRECONDITION;
    }
    b->outstanding = static_cast<int>(b->kernels.size());
  }
  auto done = [b] {
    // notify under the lock: the waiter may destroy the batch as soon as it sees zero
    std::lock_guard<std::mutex> guard(b->mu);
    if (--b->outstanding == 0) b->cv.notify_all();
  };
  for (size_t j = 0; j < b->kernels.size(); j++) {
    b->contexts[j]->Reset();
    static_cast<mpic::AsyncOpKernel*>(b->kernels[j].get())->ComputeAsync(b->contexts[j].get(), done);
  }
  return MPIC_OK;
}

int mpic_batch_wait(mpic_batch* b, int* codes) {
  if (!b) return MPIC_INVALID_ARGUMENT;
  {
    std::unique_lock<std::mutex> lock(b->mu);
    b->cv.wait(lock, [b] { return b->outstanding == 0; });
  }
  int first = MPIC_OK;
  for (size_t j = 0; j < b->contexts.size(); j++) {
    const int code = static_cast<int>(b->contexts[j]->status().code());
    if (codes) codes[j] = code;
    if (code != MPIC_OK && first == MPIC_OK) first = code;
  }
  return first;
}

const char* mpic_batch_message(const mpic_batch* b, int index) {
  if (!b || index < 0 || static_cast<size_t>(index) >= b->contexts.size()) return "";
  return b->contexts[static_cast<size_t>(index)]->status().error_message().c_str();
}

int mpic_batch_busy(mpic_batch* b) {
  if (!b) return 0;
  std::lock_guard<std::mutex> guard(b->mu);
  return b->outstanding != 0;
}

int mpic_batch_destroy(mpic_batch* b) {
  if (!b) return MPIC_OK;
  {  // never free nodes the background thread may still call back into
    std::unique_lock<std::mutex> lock(b->mu);
    b->cv.wait(lock, [b] { return b->outstanding == 0; });
  }
  {
    std::lock_guard<std::mutex> registry(g_batch_registry_mu);
    if (mpic_world* w = b->world.load()) {
      auto it = std::find(w->batches.begin(), w->batches.end(), b);
      if (it != w->batches.end()) w->batches.erase(it);
    }
  }
  delete b;
  return MPIC_OK;
}

// ---- the ring driver without the op layer --------------------------------------------

int mpic_ring_allreduce_prestaged(int n, int r, int dtype, const void* input, void* output, size_t count,
                                  const void* const* rs_segments, const void* const* ag_segments, void* stream,
                                  int flags) {
  mpic::Status s = mpic::RingAllreducePrestaged(n, r, static_cast<mpic::DataType>(dtype), input, output, count,
                                                rs_segments, ag_segments, stream, mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allreduce_direct_prestaged(int n, int r, int dtype, const void* input, void* output, size_t count,
                                         const void* const* peer_segments, const void* const* ag_segments,
                                         void* stream, int flags) {
  mpic::Status s = mpic::RingAllreduceDirectPrestaged(n, r, static_cast<mpic::DataType>(dtype), input, output, count,
                                                      peer_segments, ag_segments, stream,
                                                      mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allreduce_fused_prestaged(const struct ring_fusion_plan* plan, int n, int r, void* wire,
                                        const void* const* rs_segments, const void* const* ag_segments, void* stream,
                                        int flags) {
  mpic::Status s = mpic::RingAllreduceFusedPrestaged(plan, n, r, wire, rs_segments, ag_segments, stream,
                                                     mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allgather_prestaged(int n, int r, int dtype, const void* input, const size_t* rows,
                                  size_t elems_per_row, void* output, const void* const* segments, void* stream,
                                  int flags) {
  if (n < 1 || !rows) return MPIC_INVALID_ARGUMENT;
  std::vector<size_t> rv(rows, rows + n);
  mpic::Status s = mpic::RingAllgatherPrestaged(n, r, static_cast<mpic::DataType>(dtype), input, rv, elems_per_row,
                                                output, segments, stream, mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allreduce_transport(int n, int r, int dtype, const void* input, void* output, void* temp,
                                  size_t temp_elements, size_t count, const mpic_transport* transport, void* stream,
                                  int flags) {
  mpic::Status s = mpic::RingAllreduceTransport(n, r, static_cast<mpic::DataType>(dtype), input, output, temp,
                                                temp_elements, count, transport, stream,
                                                mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allgather_transport(int n, int r, int dtype, const void* input, const size_t* rows,
                                  size_t elems_per_row, void* output, const mpic_transport* transport, void* stream,
                                  int flags) {
  if (n < 1 || !rows) return MPIC_INVALID_ARGUMENT;
  std::vector<size_t> rv(rows, rows + n);
  mpic::Status s = mpic::RingAllgatherTransport(n, r, static_cast<mpic::DataType>(dtype), input, rv, elems_per_row,
                                                output, transport, stream, mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allreduce_all_ranks(int n, int dtype, const void* const* inputs, void* const* outputs, size_t count,
                                  void* stream, int flags) {
  if (n < 1 || !inputs || !outputs) return MPIC_INVALID_ARGUMENT;
  mpic::Status s = mpic::RingAllreduceAllRanks(n, static_cast<mpic::DataType>(dtype), inputs, outputs, count, stream,
                                               mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

int mpic_ring_allgather_all_ranks(int n, int dtype, const void* const* inputs, const size_t* rows,
                                  size_t elems_per_row, void* const* outputs, void* stream, int flags) {
  if (n < 1 || !inputs || !outputs || !rows) return MPIC_INVALID_ARGUMENT;
  std::vector<size_t> rv(rows, rows + n);
  mpic::Status s = mpic::RingAllgatherAllRanks(n, static_cast<mpic::DataType>(dtype), inputs, rv, elems_per_row,
                                               outputs, stream, mpic::RingOptions::FromFlags(flags));
  return s.ok() ? MPIC_OK : mpic::Fail(s);
}

const char* mpic_last_error(void) { return mpic::g_last_error.c_str(); }

}  // extern "C"
