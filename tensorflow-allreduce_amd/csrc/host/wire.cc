#include "wire.h"

#include <cstring>

namespace mpic {
namespace {

constexpr uint32_t kRequestMagic = 0x5149504du;   // "MPIQ"
constexpr uint32_t kResponseMagic = 0x5249504du;  // "MPIR"
constexpr uint8_t kVersion = 1;
constexpr uint32_t kMaxDims = 254;  // TensorFlow's limit on a shape's rank

template <typename T>
void Put(std::string* out, T v) {
  char buf[sizeof(T)];
  for (size_t i = 0; i < sizeof(T); i++) buf[i] = static_cast<char>((static_cast<uint64_t>(v) >> (8 * i)) & 0xff);
  out->append(buf, sizeof(T));
}

void PutBytes(std::string* out, const std::string& s) {
  Put<uint32_t>(out, static_cast<uint32_t>(s.size()));
  out->append(s);
}

class Reader {
 public:
  explicit Reader(const std::string& s) : p_(s.data()), end_(s.data() + s.size()) {}
  Reader(const char* data, size_t size) : p_(data), end_(data + size) {}
  template <typename T>
  bool Get(T* v) {
    if (static_cast<size_t>(end_ - p_) < sizeof(T)) return false;
    uint64_t x = 0;
    for (size_t i = 0; i < sizeof(T); i++) x |= static_cast<uint64_t>(static_cast<unsigned char>(p_[i])) << (8 * i);
    *v = static_cast<T>(x);
    p_ += sizeof(T);
    return true;
  }
  bool GetBytes(std::string* s) {
    uint32_t n = 0;
    if (!Get(&n) || static_cast<size_t>(end_ - p_) < n) return false;
    s->assign(p_, n);
    p_ += n;
    return true;
  }
  bool AtEnd() const { return p_ == end_; }

 private:
  const char* p_;
  const char* end_;
};

}  // namespace

const char* MPIDataType_Name(MPIDataType t) {
  switch (t) {
    case TF_MPI_FLOAT32: return "TF_MPI_FLOAT32";
    case TF_MPI_INT32: return "TF_MPI_INT32";
    case TF_MPI_INT64: return "TF_MPI_INT64";
    default: return "TF_MPI_INVALID_TYPE";
  }
}

void MPIRequest::AppendTo(std::string* out, int32_t rank, RequestType type, MPIDataType dtype,
                          const std::string& name, const Dims& shape) {
  Put<uint32_t>(out, kRequestMagic);
  Put<uint8_t>(out, kVersion);
  Put<int32_t>(out, rank);
  Put<uint8_t>(out, static_cast<uint8_t>(type));
  Put<uint8_t>(out, static_cast<uint8_t>(dtype));
  PutBytes(out, name);
  Put<uint32_t>(out, static_cast<uint32_t>(shape.size()));
  for (int64_t d : shape) Put<int64_t>(out, d);
}

std::string MPIRequest::SerializeAsString() const {
  std::string out;
  out.reserve(4 + 1 + 4 + 1 + 1 + 4 + tensor_name.size() + 4 + 8 * tensor_shape.size());  // one allocation
  AppendTo(&out, request_rank, request_type, tensor_type, tensor_name, tensor_shape);
  return out;
}

void AppendRequestFrame(std::string* stream, int32_t rank, MPIRequest::RequestType type, MPIDataType dtype,
                        const std::string& name, const Dims& shape) {
  const size_t at = stream->size();
  Put<uint32_t>(stream, 0);
  MPIRequest::AppendTo(stream, rank, type, dtype, name, shape);
  const uint32_t size = static_cast<uint32_t>(stream->size() - at - 4);
  for (size_t i = 0; i < 4; i++) (*stream)[at + i] = static_cast<char>((size >> (8 * i)) & 0xff);
}

bool NextRequestFrame(const std::string& stream, size_t* at, const char** data, size_t* size) {
  if (*at > stream.size() || stream.size() - *at < 4) return false;
  uint32_t n = 0;
  for (size_t i = 0; i < 4; i++) n |= static_cast<uint32_t>(static_cast<unsigned char>(stream[*at + i])) << (8 * i);
  if (stream.size() - *at - 4 < n) return false;
  *data = stream.data() + *at + 4;
  *size = n;
  *at += 4 + static_cast<size_t>(n);
  return true;
}

bool MPIRequest::ParseFromString(const std::string& bytes) { return ParseFromArray(bytes.data(), bytes.size()); }

bool MPIRequest::ParseFromArray(const char* data, size_t size) {
  Reader r(data, size);
  uint32_t magic = 0, ndims = 0;
  uint8_t version = 0, rtype = 0, dtype = 0;
  if (!r.Get(&magic) || magic != kRequestMagic || !r.Get(&version) || version != kVersion) return false;
  if (!r.Get(&request_rank) || !r.Get(&rtype) || !r.Get(&dtype) || rtype > ALLGATHER || dtype > TF_MPI_INT64)
    return false;
  request_type = static_cast<RequestType>(rtype);
  tensor_type = static_cast<MPIDataType>(dtype);
  if (!r.GetBytes(&tensor_name) || !r.Get(&ndims) || ndims > kMaxDims) return false;
  tensor_shape.resize(ndims);
  for (uint32_t i = 0; i < ndims; i++)
    if (!r.Get(&tensor_shape[i])) return false;
  return r.AtEnd();
}

std::string MPIResponse::SerializeAsString() const {
  std::string out;
  out.reserve(4 + 1 + 1 + 4 + tensor_name.size() + 4 + error_message.size());
  Put<uint32_t>(&out, kResponseMagic);
  Put<uint8_t>(&out, kVersion);
  Put<uint8_t>(&out, static_cast<uint8_t>(response_type));
  PutBytes(&out, tensor_name);
  PutBytes(&out, error_message);
  return out;
}

bool MPIResponse::ParseFromString(const std::string& bytes) {
  Reader r(bytes);
  uint32_t magic = 0;
  uint8_t version = 0, type = 0;
  if (!r.Get(&magic) || magic != kResponseMagic || !r.Get(&version) || version != kVersion) return false;
  if (!r.Get(&type) || type > SHUTDOWN) return false;
  response_type = static_cast<ResponseType>(type);
  return r.GetBytes(&tensor_name) && r.GetBytes(&error_message) && r.AtEnd();
}

}  // namespace mpic
