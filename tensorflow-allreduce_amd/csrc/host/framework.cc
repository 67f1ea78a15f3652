#include "framework.h"

#include <sstream>

namespace mpic {

const char* const DEVICE_CPU = "CPU";
const char* const DEVICE_GPU = "GPU";

const char* DataTypeString(DataType dt) {
  switch (dt) {
    case DT_FLOAT: return "float32";
    case DT_DOUBLE: return "float64";
    case DT_INT32: return "int32";
    case DT_INT64: return "int64";
    default: return "invalid";
  }
}

size_t DataTypeSize(DataType dt) {
  switch (dt) {
    case DT_FLOAT: return 4;
    case DT_INT32: return 4;
    case DT_INT64: return 8;
    case DT_DOUBLE: return 8;
    default: return 0;
  }
}

std::string TensorShape::DebugString() const {
  std::ostringstream os;
  os << "[";
  for (size_t i = 0; i < dims_.size(); i++) os << (i ? "," : "") << dims_[i];
  os << "]";
  return os.str();
}

std::string OpDef::Signature() const {
  std::ostringstream os;
  os << name << "(";
  for (size_t i = 0; i < inputs.size(); i++) os << (i ? ", " : "") << inputs[i];
  os << ")";
  if (!outputs.empty()) {
    os << " -> (";
    for (size_t i = 0; i < outputs.size(); i++) os << (i ? ", " : "") << outputs[i];
    os << ")";
  }
  for (const std::string& a : attrs) os << "; " << a;
  return os.str();
}

OpRegistry* OpRegistry::Global() {
  static OpRegistry* registry = new OpRegistry();
  return registry;
}

void OpRegistry::Register(const OpDef& def) {
  if (ops_.emplace(def.name, def).second) order_.push_back(def.name);
}

void OpRegistry::RegisterKernel(KernelDef def) { kernels_.push_back(std::move(def)); }

const OpDef* OpRegistry::LookUp(const std::string& name) const {
  auto it = ops_.find(name);
  return it == ops_.end() ? nullptr : &it->second;
}

const KernelDef* OpRegistry::FindKernel(const std::string& op, const std::string& device) const {
  for (const KernelDef& k : kernels_)
    if (k.op == op && k.device == device) return &k;
  return nullptr;
}

Status OpKernelContext::allocate_output(int index, const TensorShape& shape, DataType dt,
                                        bool host_memory, Tensor** out) {
  if (index < 0) return errors::InvalidArgument("negative output index");
  // An empty tensor is still allocated (the embedder owns an object for it);
  // its data pointer may be null.
  void* mem = alloc_ ? alloc_(dt, shape, host_memory) : nullptr;
  if (!mem && shape.num_elements() > 0)
    return errors::Internal("allocate_output failed for a tensor of shape " + shape.DebugString());
  if (outputs_.size() <= static_cast<size_t>(index)) outputs_.resize(static_cast<size_t>(index) + 1);
  std::unique_ptr<Tensor>& slot = outputs_[static_cast<size_t>(index)];
  if (!slot && !spare_.empty()) {
    slot = std::move(spare_.back());
    spare_.pop_back();
  }
  if (slot) *slot = Tensor(dt, shape, mem, host_memory);
  else slot.reset(new Tensor(dt, shape, mem, host_memory));
  *out = outputs_[static_cast<size_t>(index)].get();
  return Status::OK();
}

}  // namespace mpic
