// Concurrency test of the plugin's host code without a GPU: worlds are
// initialised on the CPU device, several threads play the ranks and submit
// collectives whose cross-rank checks fail (so nothing reaches a device), and
// every op must come back with the coordinator's verdict. Built with
// -fsanitize=thread by tests/test_host_cpp.py; prints "ok" on success.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "mpi_collectives.h"

#define CHECK(cond)                                                                 \
  do {                                                                              \
    if (!(cond)) {                                                                  \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                                 \
    }                                                                               \
  } while (0)

static void* host_alloc(void*, int, int ndims, const int64_t* dims, int) {
  size_t n = 1;
  for (int i = 0; i < ndims; i++) n *= static_cast<size_t>(dims[i]);
  return std::calloc(n ? n : 1, 8);  // leaked on purpose: lifetime of the test
}

static int run_scalar(mpic_world* w, int rank, const char* op) {
  mpic_context* c = nullptr;
  CHECK(mpic_context_create(w, rank, op, op, "CPU", host_alloc, nullptr, &c) == MPIC_OK);
  CHECK(mpic_context_compute(c) == MPIC_OK);
  CHECK(mpic_context_wait(c) == MPIC_OK);
  int value = -1;
  if (mpic_context_num_outputs(c) == 1) {
    void* data = nullptr;
    CHECK(mpic_context_output(c, 0, nullptr, nullptr, nullptr, &data) == MPIC_OK);
    value = *static_cast<int32_t*>(data);
  }
  CHECK(mpic_context_destroy(c) == MPIC_OK);
  return value;
}

int main() {
  const int kRanks = 4, kRounds = 200;
  CHECK(mpic_op_count() == 6);
  mpic_world* w = nullptr;
  CHECK(mpic_world_create(kRanks, &w) == MPIC_OK);
  // ops before init fail (mpi_ops.cc:827-833)
  {
    mpic_context* c = nullptr;
    CHECK(mpic_context_create(w, 0, "MPISize", "MPISize", "CPU", host_alloc, nullptr, &c) == MPIC_OK);
    CHECK(mpic_context_compute(c) == MPIC_OK);
    CHECK(mpic_context_wait(c) == MPIC_FAILED_PRECONDITION);
    CHECK(std::strstr(mpic_context_message(c), "MPI has not been initialized") != nullptr);
    mpic_context_destroy(c);
  }
  // all ranks race to initialise; exactly one background thread results
  {
    std::vector<std::thread> ts;
    for (int r = 0; r < kRanks; r++) ts.emplace_back([w, r] { run_scalar(w, r, "MPIInit"); });
    for (auto& t : ts) t.join();
  }
  for (int r = 0; r < kRanks; r++) {
    CHECK(run_scalar(w, r, "MPISize") == kRanks);
    CHECK(run_scalar(w, r, "MPIRank") == r);
    CHECK(run_scalar(w, r, "MPILocalRank") == r);
  }

  std::atomic<int> verdicts{0};
  std::vector<std::thread> ts;
  for (int r = 0; r < kRanks; r++) {
    ts.emplace_back([w, r, &verdicts] {
      std::vector<float> data(64, 1.0f);
      for (int k = 0; k < kRounds; k++) {
        // rank r announces a [4 + r]-element tensor: shapes differ between ranks
        const std::string name = "t" + std::to_string(k);
        const int64_t dims[1] = {4 + r};
        mpic_context* c = nullptr;
        CHECK(mpic_context_create(w, r, "MPIAllreduce", name.c_str(), "GPU", host_alloc, nullptr, &c) == MPIC_OK);
        CHECK(mpic_context_add_input(c, MPIC_DT_FLOAT, 1, dims, data.data(), 1) == MPIC_OK);
        CHECK(mpic_context_compute(c) == MPIC_OK);
        CHECK(mpic_context_wait(c) == MPIC_FAILED_PRECONDITION);
        CHECK(std::strstr(mpic_context_message(c), "Mismatched allreduce tensor shapes") != nullptr);
        CHECK(mpic_context_destroy(c) == MPIC_OK);
        verdicts++;
      }
    });
  }
  for (auto& t : ts) t.join();
  CHECK(verdicts == kRanks * kRounds);

  // an op that can never complete is failed by the shutdown, not left hanging
  mpic_context* lonely = nullptr;
  const int64_t dims[1] = {8};
  float buf[8] = {0};
  CHECK(mpic_context_create(w, 1, "MPIAllreduce", "lonely", "GPU", host_alloc, nullptr, &lonely) == MPIC_OK);
  CHECK(mpic_context_add_input(lonely, MPIC_DT_FLOAT, 1, dims, buf, 1) == MPIC_OK);
  CHECK(mpic_context_compute(lonely) == MPIC_OK);
  CHECK(mpic_world_destroy(w) == MPIC_OK);
  CHECK(mpic_context_wait(lonely) == MPIC_UNKNOWN);
  CHECK(mpic_context_destroy(lonely) == MPIC_OK);

  // fusion switched on holds requests until a flush; errors still come back
  CHECK(mpic_world_create(2, &w) == MPIC_OK);
  run_scalar(w, 0, "MPIInit");
  static char fusion_area[4096] __attribute__((aligned(16)));
  CHECK(mpic_world_set_fusion_buffer(w, fusion_area, 2048) == MPIC_OK);
  mpic_context* cs[2];
  for (int r = 0; r < 2; r++) {
    const int64_t d[1] = {4 + r};
    CHECK(mpic_context_create(w, r, "MPIAllreduce", "held", "GPU", host_alloc, nullptr, &cs[r]) == MPIC_OK);
    CHECK(mpic_context_add_input(cs[r], MPIC_DT_FLOAT, 1, d, buf, 1) == MPIC_OK);
    CHECK(mpic_context_compute(cs[r]) == MPIC_OK);
  }
  CHECK(mpic_world_flush(w) == MPIC_OK);
  for (int r = 0; r < 2; r++) {
    CHECK(mpic_context_wait(cs[r]) == MPIC_FAILED_PRECONDITION);
    mpic_context_destroy(cs[r]);
  }
  CHECK(mpic_world_destroy(w) == MPIC_OK);

  // a rank's nodes built once and run again and again (mpic_batch_*): two ranks on two threads, shapes
  // that differ in the second node, so each run ends with one OK-less node and its message; the
  // nodes' done() calls race with the waiters
  CHECK(mpic_world_create(2, &w) == MPIC_OK);
  run_scalar(w, 0, "MPIInit");
  {
    mpic_batch* bs[2] = {nullptr, nullptr};
    const char* names[3] = {"g0", "g1", "g2"};
    const int dts[3] = {MPIC_DT_FLOAT, MPIC_DT_FLOAT, MPIC_DT_FLOAT}, nd[3] = {1, 1, 0};
    for (int r = 0; r < 2; r++) {
      const int64_t d[2] = {0, 3 + r};        // g0: empty on both ranks; g1: 3 against 4 elements; g2: a scalar
      const void* ins[3] = {nullptr, buf, buf};
      void* outs[3] = {nullptr, buf, buf};
      CHECK(mpic_batch_create(w, r, 3, names, dts, nd, d, ins, outs, 0, &bs[r]) == MPIC_OK);
      CHECK(mpic_batch_size(bs[r]) == 3);
    }
    CHECK(mpic_batch_create(w, 2, 3, names, dts, nd, nullptr, nullptr, nullptr, 0, &bs[0]) == MPIC_INVALID_ARGUMENT);
    for (int round = 0; round < 50; round++) {
      std::vector<std::thread> ts;
      for (int r = 0; r < 2; r++) {
        ts.emplace_back([&bs, r] {
          CHECK(mpic_batch_submit(bs[r]) == MPIC_OK);
          int codes[3] = {-1, -1, -1};
          CHECK(mpic_batch_wait(bs[r], codes) != MPIC_OK);      // (without a GPU the valid nodes fail too, in their own way)
          CHECK(codes[0] != -1 && codes[2] != -1 && codes[1] == MPIC_FAILED_PRECONDITION);
          CHECK(std::strstr(mpic_batch_message(bs[r], 1), "Mismatched allreduce tensor shapes") != nullptr);
        });
      }
      for (auto& t : ts) t.join();
    }
    // a submission nobody answers: the second submit is refused, destroying the world ends the first
    CHECK(mpic_batch_submit(bs[0]) == MPIC_OK);
    CHECK(mpic_batch_submit(bs[0]) == MPIC_FAILED_PRECONDITION);
    CHECK(mpic_world_destroy(w) == MPIC_OK);
    CHECK(mpic_batch_wait(bs[0], nullptr) == MPIC_UNKNOWN);
    for (int r = 0; r < 2; r++) CHECK(mpic_batch_destroy(bs[r]) == MPIC_OK);
  }

  // the in-process transport under concurrent ranks: every rank posts its
  // receives, sends to the right and waits, as the ring's steps do (zero-byte
  // messages: no device is touched)
  {
    mpic_loopback* lb = nullptr;
    CHECK(mpic_loopback_create(kRanks, 30.0, &lb) == MPIC_OK);
    std::atomic<int> exchanged{0};
    std::vector<std::thread> ranks;
    for (int r = 0; r < kRanks; r++) {
      ranks.emplace_back([lb, r, kRanks, &exchanged] {
        mpic_transport t;
        CHECK(mpic_loopback_endpoint(lb, r, &t) == MPIC_OK);
        const int left = (r - 1 + kRanks) % kRanks, right = (r + 1) % kRanks;
        for (int step = 0; step < 300; step++) {
          void* reqs[3];
          for (int c = 0; c < 3; c++) CHECK(t.irecv(t.user, nullptr, 0, left, 12, &reqs[c]) == 0);
          for (int c = 0; c < 3; c++) CHECK(t.send(t.user, nullptr, 0, right, 12) == 0);
          for (int c = 0; c < 3; c++) CHECK(t.wait(t.user, reqs[c]) == 0);
          exchanged++;
        }
      });
    }
    for (auto& t : ranks) t.join();
    CHECK(exchanged == kRanks * 300);
    CHECK(mpic_loopback_destroy(lb) == MPIC_OK);
  }
  std::printf("ok\n");
  return 0;
}
