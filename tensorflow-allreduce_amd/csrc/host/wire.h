// Wire format of the coordinator's messages: MPIRequest (a rank announces a
// collective it is ready for) and MPIResponse (the coordinator tells the ranks
// what to run), the records of tensorflow/contrib/mpi_collectives/
// mpi_message.proto:12-63 without protobuf.
//
// Every message is a length-delimited byte string with explicit field sizes,
// so nothing depends on NUL termination: the reference sends
// SerializeToString().c_str() and rebuilds std::string from a char*
// (mpi_ops.cc:668-669, 703, 731-734, 773), which truncates at the first zero
// byte - and a zero-sized dimension, rank 0 or type 0 all encode as zero bytes.
// Element counts and dimensions are 64-bit.
//
// Layout (little endian):
//   u32 magic 'MPIQ' / 'MPIR', u8 version,
//   request:  i32 rank, u8 request_type, u8 tensor_type, u32 name_len, name bytes,
//             u32 ndims, i64 dims[ndims]
//   response: u8 response_type, u32 name_len, name bytes, u32 error_len, error bytes
#ifndef MPIC_WIRE_H_
#define MPIC_WIRE_H_

#include <cstdint>
#include <string>
#include <vector>

#include "dims.h"

namespace mpic {

// mpi_message.proto:12-17
enum MPIDataType { TF_MPI_INVALID_TYPE = 0, TF_MPI_FLOAT32 = 1, TF_MPI_INT32 = 2, TF_MPI_INT64 = 3 };
const char* MPIDataType_Name(MPIDataType t);

// mpi_message.proto:22-40
struct MPIRequest {
  enum RequestType { ALLREDUCE = 0, ALLGATHER = 1 };
  int32_t request_rank = 0;
  RequestType request_type = ALLREDUCE;
  MPIDataType tensor_type = TF_MPI_INVALID_TYPE;
  std::string tensor_name;
  Dims tensor_shape;

  std::string SerializeAsString() const;
  bool ParseFromString(const std::string& bytes);
  bool ParseFromArray(const char* data, size_t size);
  // The bytes SerializeAsString gives for a request of these fields, appended to
  // `out` without building the request.
  static void AppendTo(std::string* out, int32_t rank, RequestType type, MPIDataType dtype, const std::string& name,
                       const Dims& shape);
};

// A stream of requests, each behind its length (u32, little endian): how the
// requests of one process travel to its coordinator thread, in one buffer that
// is filled, handed over and reused, instead of one string per request.
void AppendRequestFrame(std::string* stream, int32_t rank, MPIRequest::RequestType type, MPIDataType dtype,
                        const std::string& name, const Dims& shape);
// The frame that starts at *at: its bytes, and *at moved behind it. False at
// the end of the stream or when the stream is cut short inside a frame.
bool NextRequestFrame(const std::string& stream, size_t* at, const char** data, size_t* size);

// mpi_message.proto:49-63
struct MPIResponse {
  enum ResponseType { ALLREDUCE = 0, ALLGATHER = 1, ERROR = 2, DONE = 3, SHUTDOWN = 4 };
  ResponseType response_type = DONE;
  std::string tensor_name;
  std::string error_message;

  std::string SerializeAsString() const;
  bool ParseFromString(const std::string& bytes);
};

}  // namespace mpic
#endif  // MPIC_WIRE_H_
