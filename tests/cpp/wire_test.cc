// Unit tests of the coordinator's wire format (csrc/host/wire.{h,cc}) and of
// the small framework types it travels with. Built and run by
// tests/test_host_cpp.py with g++; prints "ok" and exits 0 on success.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <utility>
#include <vector>

#include "framework.h"
#include "wire.h"

#define CHECK(cond)                                                       \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                       \
    }                                                                     \
  } while (0)

using namespace mpic;

int main() {
  // every field that encodes as zero bytes, and a name with zero bytes inside:
  // what the reference's c_str() round trip (mpi_ops.cc:703, 773) cannot carry
  MPIRequest q;
  q.request_rank = 0;
  q.request_type = MPIRequest::ALLREDUCE;
  q.tensor_type = TF_MPI_INVALID_TYPE;
  q.tensor_name = std::string("grad\0ient/0", 11);
  q.tensor_shape = {0, 5, 0};
  MPIRequest back;
  CHECK(back.ParseFromString(q.SerializeAsString()));
  CHECK(back.request_rank == 0 && back.request_type == MPIRequest::ALLREDUCE);
  CHECK(back.tensor_type == TF_MPI_INVALID_TYPE);
  CHECK(back.tensor_name.size() == 11 && back.tensor_name == q.tensor_name);
  CHECK(back.tensor_shape == q.tensor_shape);

  // 64-bit dimensions, a scalar (no dims), every enum value
  q.request_rank = 63;
  q.request_type = MPIRequest::ALLGATHER;
  q.tensor_type = TF_MPI_INT64;
  q.tensor_name = "allgather_sizing";
  q.tensor_shape = {int64_t(1) << 40, 3};
  CHECK(back.ParseFromString(q.SerializeAsString()));
  CHECK(back.request_rank == 63 && back.request_type == MPIRequest::ALLGATHER && back.tensor_type == TF_MPI_INT64);
  CHECK(back.tensor_shape.size() == 2 && back.tensor_shape[0] == (int64_t(1) << 40));
  q.tensor_shape.clear();
  q.tensor_name.clear();
  CHECK(back.ParseFromString(q.SerializeAsString()));
  CHECK(back.tensor_shape.empty() && back.tensor_name.empty());

  // malformed input is rejected, never read past its end
  const std::string good = q.SerializeAsString();
  for (size_t cut = 0; cut < good.size(); cut++) CHECK(!back.ParseFromString(good.substr(0, cut)));
  CHECK(!back.ParseFromString(good + "x"));                       // trailing bytes
  std::string bad = good;
  bad[0] ^= 1;                                                    // wrong magic
  CHECK(!back.ParseFromString(bad));
  bad = good;
  bad[4] = 9;                                                     // unknown version
  CHECK(!back.ParseFromString(bad));
  MPIRequest huge;
  huge.tensor_shape.assign(300, 1);                               // more dims than a shape may have
  CHECK(!back.ParseFromString(huge.SerializeAsString()));
  MPIResponse not_a_request;
  CHECK(!back.ParseFromString(not_a_request.SerializeAsString()));

  // responses: every type, empty and non-empty strings, zero bytes inside
  for (int t = MPIResponse::ALLREDUCE; t <= MPIResponse::SHUTDOWN; t++) {
    MPIResponse r, rb;
    r.response_type = static_cast<MPIResponse::ResponseType>(t);
    r.tensor_name = t == MPIResponse::DONE ? "" : std::string("a\0b", 3);
    r.error_message = t == MPIResponse::ERROR ? "Mismatched data types: One rank had type TF_MPI_INT32." : "";
    CHECK(rb.ParseFromString(r.SerializeAsString()));
    CHECK(rb.response_type == r.response_type && rb.tensor_name == r.tensor_name && rb.error_message == r.error_message);
    const std::string bytes = r.SerializeAsString();
    for (size_t cut = 0; cut < bytes.size(); cut++) CHECK(!rb.ParseFromString(bytes.substr(0, cut)));
  }
  CHECK(std::string(MPIDataType_Name(TF_MPI_FLOAT32)) == "TF_MPI_FLOAT32");
  CHECK(std::string(MPIDataType_Name(TF_MPI_INVALID_TYPE)) == "TF_MPI_INVALID_TYPE");

  // the framework types the messages are checked with
  CHECK(TensorShape({17, 17, 17}).DebugString() == "[17,17,17]");
  CHECK(TensorShape().DebugString() == "[]" && TensorShape().num_elements() == 1);
  CHECK(TensorShape({0, 5}).num_elements() == 0);
  CHECK(TensorShape({2, 3}) != TensorShape({3, 2}) && TensorShape({2, 3}) == TensorShape({2, 3}));
  CHECK(DataTypeSize(DT_FLOAT) == 4 && DataTypeSize(DT_INT64) == 8 && DataTypeSize(DT_INVALID) == 0);

  // Dims: values survive every move between the in-place array and the heap
  {
    Dims d;
    CHECK(d.empty() && d.size() == 0 && d == Dims());
    for (int64_t i = 0; i < 20; i++) {
      d.push_back(100 + i);
      CHECK(d.size() == static_cast<size_t>(i + 1));
      for (int64_t j = 0; j <= i; j++) CHECK(d[static_cast<size_t>(j)] == 100 + j);
    }
    Dims copy = d;
    CHECK(copy == d && copy.size() == 20);
    d.resize(3);                                       // back into the array
    CHECK(d.size() == 3 && d[0] == 100 && d[2] == 102 && d != copy);
    d.resize(6);                                       // new ones are zero, old ones kept
    CHECK(d[2] == 102 && d[3] == 0 && d[5] == 0);
    d.resize(12);                                      // array to heap
    CHECK(d[2] == 102 && d[5] == 0 && d[11] == 0);
    Dims moved = std::move(copy);
    CHECK(moved.size() == 20 && moved[19] == 119 && copy.empty());
    copy = std::move(moved);
    CHECK(copy.size() == 20 && copy[8] == 108 && moved.empty());
    copy.assign(9, 7);
    CHECK(copy.size() == 9 && copy[0] == 7 && copy[8] == 7);
    copy = {1, 2};
    CHECK(copy == Dims({1, 2}) && copy != Dims({1, 2, 0}) && copy != Dims({2, 1}));
    std::vector<int64_t> v = {4, 5, 6};
    CHECK(Dims(v) == Dims({4, 5, 6}) && TensorShape(v).num_elements() == 120);
    int64_t sum = 0;
    for (int64_t x : Dims({1, 2, 3})) sum += x;
    CHECK(sum == 6);
    // the bytes of a request do not depend on whether it was built first
    MPIRequest nine;
    nine.request_rank = 3;
    nine.tensor_name = "n";
    nine.tensor_type = TF_MPI_INT64;
    nine.request_type = MPIRequest::ALLGATHER;
    nine.tensor_shape.assign(9, 2);                    // more than Dims holds in place
    std::string appended = "x";
    MPIRequest::AppendTo(&appended, 3, MPIRequest::ALLGATHER, TF_MPI_INT64, "n", nine.tensor_shape);
    CHECK(appended == "x" + nine.SerializeAsString());
    MPIRequest nine_back;
    CHECK(nine_back.ParseFromString(nine.SerializeAsString()) && nine_back.tensor_shape == nine.tensor_shape);
    CHECK(nine_back.ParseFromString(q.SerializeAsString()) && nine_back.tensor_shape == q.tensor_shape);  // 9 dims -> 3

    // a stream of requests, each behind its length: every frame comes back as it went in,
    // an empty stream has none, and a stream cut short inside a frame stops there
    std::string stream;
    size_t at = 0, size = 0;
    const char* data = nullptr;
    CHECK(!NextRequestFrame(stream, &at, &data, &size));
    AppendRequestFrame(&stream, 3, MPIRequest::ALLGATHER, TF_MPI_INT64, "n", nine.tensor_shape);
    AppendRequestFrame(&stream, q.request_rank, q.request_type, q.tensor_type, q.tensor_name, q.tensor_shape);
    AppendRequestFrame(&stream, 0, MPIRequest::ALLREDUCE, TF_MPI_FLOAT32, "", Dims());
    MPIRequest f;  // one object for all frames, as the coordinator parses
    CHECK(NextRequestFrame(stream, &at, &data, &size) && std::string(data, size) == nine.SerializeAsString());
    CHECK(f.ParseFromArray(data, size) && f.tensor_shape == nine.tensor_shape && f.request_rank == 3);
    CHECK(NextRequestFrame(stream, &at, &data, &size) && f.ParseFromArray(data, size));
    CHECK(f.tensor_name == q.tensor_name && f.tensor_shape == q.tensor_shape && f.tensor_type == q.tensor_type);
    CHECK(NextRequestFrame(stream, &at, &data, &size) && f.ParseFromArray(data, size));
    CHECK(f.tensor_name.empty() && f.tensor_shape.empty() && f.tensor_type == TF_MPI_FLOAT32);
    CHECK(at == stream.size() && !NextRequestFrame(stream, &at, &data, &size));
    for (size_t cut = 1; cut < 8; cut++) {
      const std::string shorter = stream.substr(0, stream.size() - cut);
      size_t frames = 0;
      at = 0;
      while (NextRequestFrame(shorter, &at, &data, &size)) frames++;
      CHECK(frames == 2);
    }
  }
  Status s = errors::FailedPrecondition("x");
  CHECK(!s.ok() && s.code() == error::FAILED_PRECONDITION && s.error_message() == "x" && Status::OK().ok());
  OpDef def = OpDefBuilder("Demo").Attr("T: {int32}").Input("a: T").Input("b: T").Output("c: T").def();
  CHECK(def.Signature() == "Demo(a: T, b: T) -> (c: T); T: {int32}");
  std::printf("ok\n");
  return 0;
}
