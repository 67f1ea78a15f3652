// The small slice of an op framework the MPI ops need when no TensorFlow is
// linked in: Status, DataType, TensorShape, Tensor views over caller memory,
// an op registry with REGISTER_OP / REGISTER_KERNEL_BUILDER, OpKernel /
// AsyncOpKernel and an OpKernelContext. Names and meanings follow the
// TensorFlow interfaces the reference plugin is written against
// (tensorflow/core/framework/op.h, op_kernel.h:181-198, 803-832, 1517-1525),
// so the op source reads like the reference's mpi_ops.cc; nothing here is a
// TensorFlow re-implementation beyond what those ops touch.
#ifndef MPIC_FRAMEWORK_H_
#define MPIC_FRAMEWORK_H_

#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "dims.h"

namespace mpic {

// ---- Status (tensorflow/core/lib/core/status.h, error_codes.proto) ----------
namespace error {
enum Code { OK = 0, UNKNOWN = 2, INVALID_ARGUMENT = 3, NOT_FOUND = 5, FAILED_PRECONDITION = 9, INTERNAL = 13 };
}

class Status {
 public:
  Status() : code_(error::OK) {}
  Status(error::Code code, std::string msg) : code_(code), msg_(std::move(msg)) {}
  static Status OK() { return Status(); }
  bool ok() const { return code_ == error::OK; }
  error::Code code() const { return code_; }
  const std::string& error_message() const { return msg_; }

 private:
  error::Code code_;
  std::string msg_;
};

namespace errors {
inline Status Unknown(const std::string& m) { return Status(error::UNKNOWN, m); }
inline Status FailedPrecondition(const std::string& m) { return Status(error::FAILED_PRECONDITION, m); }
inline Status InvalidArgument(const std::string& m) { return Status(error::INVALID_ARGUMENT, m); }
inline Status NotFound(const std::string& m) { return Status(error::NOT_FOUND, m); }
inline Status Internal(const std::string& m) { return Status(error::INTERNAL, m); }
}  // namespace errors

// ---- DataType (numbering of tensorflow/core/framework/types.proto) ------------
enum DataType { DT_INVALID = 0, DT_FLOAT = 1, DT_DOUBLE = 2, DT_INT32 = 3, DT_INT64 = 9 };
const char* DataTypeString(DataType dt);
size_t DataTypeSize(DataType dt);  // 0 for types the MPI ops do not handle

// ---- TensorShape ----------------------------------------------------------------
class TensorShape {
 public:
  TensorShape() {}
  explicit TensorShape(Dims dims) : dims_(std::move(dims)) {}  // also from a std::vector<int64_t>
  void AddDim(int64_t d) { dims_.push_back(d); }
  int dims() const { return static_cast<int>(dims_.size()); }
  int64_t dim_size(int i) const { return dims_[static_cast<size_t>(i)]; }
  int64_t num_elements() const {
    int64_t n = 1;
    for (int64_t d : dims_) n *= d;
    return n;
  }
  const Dims& dim_sizes() const { return dims_; }
  std::string DebugString() const;  // "[17,17,17]"
  bool operator==(const TensorShape& o) const { return dims_ == o.dims_; }
  bool operator!=(const TensorShape& o) const { return dims_ != o.dims_; }

 private:
  Dims dims_;
};

// A view of memory owned by the embedding framework (device memory unless
// host_memory). The op layer never frees it.
class Tensor {
 public:
  Tensor() : dtype_(DT_INVALID), data_(nullptr), host_(false) {}
  Tensor(DataType dt, TensorShape shape, void* data, bool host_memory)
      : dtype_(dt), shape_(std::move(shape)), data_(data), host_(host_memory) {}
  DataType dtype() const { return dtype_; }
  const TensorShape& shape() const { return shape_; }
  int64_t NumElements() const { return shape_.num_elements(); }
  int64_t dim_size(int i) const { return shape_.dim_size(i); }
  size_t TotalBytes() const { return static_cast<size_t>(NumElements()) * DataTypeSize(dtype_); }
  void* data() const { return data_; }
  bool host_memory() const { return host_; }

 private:
  DataType dtype_;
  TensorShape shape_;
  void* data_;
  bool host_;
};

// ---- op definitions and the registry ----------------------------------------------
extern const char* const DEVICE_CPU;
extern const char* const DEVICE_GPU;

// Shape function: output shape from input 0's shape; -1 = unknown dimension.
typedef std::function<Status(const std::vector<int64_t>& in, std::vector<int64_t>* out)> ShapeFn;

struct OpDef {
  std::string name;
  std::vector<std::string> attrs;    // "T: {int32, int64, float32}"
  std::vector<std::string> inputs;   // "tensor: T"
  std::vector<std::string> outputs;  // "sum: T"
  std::string doc;
  ShapeFn shape_fn;
  std::string Signature() const;
};

class OpDefBuilder {
 public:
  explicit OpDefBuilder(const char* name) { def_.name = name; }
  OpDefBuilder& Attr(const char* spec) { def_.attrs.push_back(spec); return *this; }
  OpDefBuilder& Input(const char* spec) { def_.inputs.push_back(spec); return *this; }
  OpDefBuilder& Output(const char* spec) { def_.outputs.push_back(spec); return *this; }
  OpDefBuilder& SetShapeFn(ShapeFn fn) { def_.shape_fn = std::move(fn); return *this; }
  OpDefBuilder& Doc(const char* text) { def_.doc = text; return *this; }
  const OpDef& def() const { return def_; }

 private:
  OpDef def_;
};

class OpKernel;
class OpKernelConstruction {
 public:
  explicit OpKernelConstruction(std::string node_name) : node_name_(std::move(node_name)) {}
  const std::string& node_name() const { return node_name_; }

 private:
  std::string node_name_;
};

struct KernelDef {
  std::string op;
  std::string device;
  std::vector<std::string> host_memory_args;
  std::function<OpKernel*(OpKernelConstruction*)> factory;
};

class KernelDefBuilder {
 public:
  explicit KernelDefBuilder(const char* op) { def_.op = op; }
  KernelDefBuilder& Device(const char* device) { def_.device = device; return *this; }
  KernelDefBuilder& HostMemory(const char* arg) { def_.host_memory_args.push_back(arg); return *this; }
  KernelDef def_;
};
inline KernelDefBuilder Name(const char* op) { return KernelDefBuilder(op); }

class OpRegistry {
 public:
  static OpRegistry* Global();
  void Register(const OpDef& def);
  void RegisterKernel(KernelDef def);
  const OpDef* LookUp(const std::string& name) const;
  const KernelDef* FindKernel(const std::string& op, const std::string& device) const;
  const std::vector<std::string>& op_names() const { return order_; }

 private:
  std::map<std::string, OpDef> ops_;
  std::vector<std::string> order_;
  std::vector<KernelDef> kernels_;
};

namespace register_detail {
struct OpRegistrar {
  OpRegistrar(const OpDefBuilder& b) { OpRegistry::Global()->Register(b.def()); }  // NOLINT: implicit on purpose
};
struct KernelRegistrar {
  KernelRegistrar(KernelDefBuilder b, std::function<OpKernel*(OpKernelConstruction*)> f) {
    b.def_.factory = std::move(f);
    OpRegistry::Global()->RegisterKernel(std::move(b.def_));
  }
};
}  // namespace register_detail

#define MPIC_CONCAT_IMPL(a, b) a##b
#define MPIC_CONCAT(a, b) MPIC_CONCAT_IMPL(a, b)
#define REGISTER_OP(name) \
  static ::mpic::register_detail::OpRegistrar MPIC_CONCAT(register_op_, __COUNTER__) = ::mpic::OpDefBuilder(name)
#define REGISTER_KERNEL_BUILDER(builder, ...)                                                  \
  static ::mpic::register_detail::KernelRegistrar MPIC_CONCAT(register_kernel_, __COUNTER__)(  \
      builder, [](::mpic::OpKernelConstruction* c) -> ::mpic::OpKernel* { return new __VA_ARGS__(c); })

// ---- kernels and their context ------------------------------------------------------

// allocate_output of the embedding framework: memory for (dtype, shape), on the
// host if host_memory. Returns nullptr on failure.
typedef std::function<void*(DataType, const TensorShape&, bool host_memory)> OutputAllocator;

class OpKernelContext {
 public:
  OpKernelContext(void* world, int rank, bool on_gpu, OutputAllocator alloc)
      : world_(world), rank_(rank), on_gpu_(on_gpu), alloc_(std::move(alloc)) {}

  void AddInput(Tensor t) { inputs_.push_back(std::move(t)); }
  int num_inputs() const { return static_cast<int>(inputs_.size()); }
  const Tensor& input(int i) const { return inputs_[static_cast<size_t>(i)]; }

  // op_kernel.h:803-832. host_memory: the kernel registration pinned this
  // output to host memory.
  Status allocate_output(int index, const TensorShape& shape, DataType dt, bool host_memory, Tensor** out);
  int num_outputs() const { return static_cast<int>(outputs_.size()); }
  const Tensor* output(int i) const { return outputs_[static_cast<size_t>(i)].get(); }

  // For a node that runs again with the same inputs (a step of a training
  // loop): forgets the last run's outputs and status.
  void Reset() {
    for (auto& t : outputs_) spare_.push_back(std::move(t));  // their objects serve the next run's outputs
    outputs_.clear();
    status_ = Status();
  }

  void SetStatus(const Status& s) { if (status_.ok()) status_ = s; }
  const Status& status() const { return status_; }

  void* world() const { return world_; }
  int rank() const { return rank_; }
  bool on_gpu() const { return on_gpu_; }

  // Set by an executor that has fused the graph's tf.div(output, n) consumer
  // into this node (the reference's allreduce(average=True) is MPIAllreduce
  // followed by tf.div, __init__.py:160-164): the kernel then delivers
  // output / n. 0: no consumer fused.
  void set_fused_divisor(int n) { fused_divisor_ = n; }
  int fused_divisor() const { return fused_divisor_; }

 private:
  int fused_divisor_ = 0;
  void* world_;
  int rank_;
  bool on_gpu_;
  OutputAllocator alloc_;
  std::vector<Tensor> inputs_;
  std::vector<std::unique_ptr<Tensor>> outputs_;
  std::vector<std::unique_ptr<Tensor>> spare_;  // Tensor objects of earlier runs, reused by allocate_output
  Status status_;
};

class OpKernel {
 public:
  explicit OpKernel(OpKernelConstruction* c) : name_(c->node_name()) {}
  virtual ~OpKernel() {}
  virtual void Compute(OpKernelContext* context) = 0;
  virtual bool IsExpensive() { return true; }
  virtual bool IsAsync() const { return false; }
  const std::string& name() const { return name_; }  // the graph node name

 private:
  std::string name_;
};

class AsyncOpKernel : public OpKernel {
 public:
  typedef std::function<void()> DoneCallback;
  explicit AsyncOpKernel(OpKernelConstruction* c) : OpKernel(c) {}
  virtual void ComputeAsync(OpKernelContext* context, DoneCallback done) = 0;
  void Compute(OpKernelContext*) override {}
  bool IsAsync() const override { return true; }
};

// op_kernel.h:1502-1525
#define OP_REQUIRES_OK(CTX, ...)                     \
  do {                                               \
    ::mpic::Status _s(__VA_ARGS__);                  \
    if (!_s.ok()) { (CTX)->SetStatus(_s); return; }  \
  } while (0)
#define OP_REQUIRES_OK_ASYNC(CTX, STATUS, CALLBACK)                 \
  do {                                                              \
    ::mpic::Status _s(STATUS);                                      \
    if (!_s.ok()) { (CTX)->SetStatus(_s); (CALLBACK)(); return; }   \
  } while (0)

}  // namespace mpic
#endif  // MPIC_FRAMEWORK_H_
