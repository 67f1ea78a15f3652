// What a launch-bound allreduce step costs, driven from C++ (no interpreter).
//
// A float32 tensor of 1 MiB (or the element count given as the first argument)
// at N=8 virtual ranks, peers pre-staged, 8 buffer sets rotated. Each form of
// the per-rank step is run 4000 times back to back on the ring's stream and
// timed with the host clock: how long the host needs to enqueue the steps, and
// how long until the stream has drained.
//
//   the reference-shaped step, 3 launches (copy, 7 accumulates, 7 copies)
//   the same with the in->out copy folded into the accumulates, 2 launches
//   the direct form, 1 launch (fold of the 8 copies of the owned segment + 7 copies)
//   the first two recorded as HIP graphs of 8 and 32 steps and replayed
//
//   g++ -O2 -std=c++17 -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -I include launch_bound_steps.cc \
//       -L lib -lmpi_collectives -lring_hip -L/opt/rocm/lib -lamdhip64
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "mpi_collectives.h"
#include "ring_abi.h"

#define HIP_OK(x)                                                                \
  do {                                                                           \
    hipError_t e_ = (x);                                                         \
    if (e_ != hipSuccess) {                                                      \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
      exit(1);                                                                   \
    }                                                                            \
  } while (0)
#define RING_OK_OR_DIE(x)                                                        \
  do {                                                                           \
    int rc_ = (x);                                                               \
    if (rc_) {                                                                   \
      printf("error %d at line %d: %s\n", rc_, __LINE__, mpic_last_error());     \
      exit(1);                                                                   \
    }                                                                            \
  } while (0)

using Clock = std::chrono::steady_clock;
static double us_since(Clock::time_point t0) {
  return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
}

int main(int argc, char** argv) {
  const int n = 8, kSets = 8, kSteps = 4000;
  const size_t count = argc > 1 ? static_cast<size_t>(atol(argv[1])) : 262144;
  std::vector<size_t> sizes(n), starts(n);
  RING_OK_OR_DIE(ring_segment_table(count, n, sizes.data(), starts.data()));
  struct Set {
    float *in, *out;
    std::vector<const void*> rs, ag, raw;
  };
  std::vector<Set> sets(kSets);
  auto segment = [&]() {
    void* p;
    HIP_OK(hipMalloc(&p, (sizes[0] + 1) * 4));
    HIP_OK(hipMemset(p, 0, (sizes[0] + 1) * 4));
    return p;
  };
  for (auto& s : sets) {
    HIP_OK(hipMalloc(&s.in, count * 4));
    HIP_OK(hipMalloc(&s.out, count * 4));
    HIP_OK(hipMemset(s.in, 0, count * 4));
    for (int i = 0; i < n - 1; i++) {
      s.rs.push_back(segment());
      s.ag.push_back(segment());
      s.raw.push_back(segment());
    }
  }
  void* stream;
  RING_OK_OR_DIE(ring_stream_create(&stream));
  printf("float32, %zu elements (%.2f MiB), N=%d, %d steps per figure\n", count, count * 4 / 1048576.0, n, kSteps);

  auto step = [&](int it, int flags) {
    Set& s = sets[it % kSets];
    if (flags < 0)
      RING_OK_OR_DIE(mpic_ring_allreduce_direct_prestaged(n, it % n, MPIC_DT_FLOAT, s.in, s.out, count, s.raw.data(),
                                                          s.ag.data(), stream, 1));
    else
      RING_OK_OR_DIE(mpic_ring_allreduce_prestaged(n, it % n, MPIC_DT_FLOAT, s.in, s.out, count, s.rs.data(),
                                                   s.ag.data(), stream, flags));
  };
  auto eager = [&](const char* name, int flags) {
    for (int pass = 0; pass < 2; pass++) {  // the first pass warms up
      const auto t0 = Clock::now();
      for (int it = 0; it < kSteps; it++) step(it, flags);
      const double host = us_since(t0);
      RING_OK_OR_DIE(ring_stream_synchronize(stream));
      const double all = us_since(t0);
      if (pass) printf("%-58s %6.2f us per step (the host enqueues one in %5.2f us)\n", name, all / kSteps, host / kSteps);
    }
  };
  eager("3 launches per step, one by one", 1);
  eager("copy folded in, 2 launches per step, one by one", 3);
  eager("direct form, 1 launch per step, one by one", -1);

  for (int per : {8, 32}) {
    for (int flags : {1, 3}) {
      void* graph;
      RING_OK_OR_DIE(ring_graph_begin_capture(stream));
      for (int it = 0; it < per; it++) step(it, flags);
      RING_OK_OR_DIE(ring_graph_end_capture(stream, &graph));
      for (int pass = 0; pass < 2; pass++) {
        const auto t0 = Clock::now();
        for (int it = 0; it < kSteps / per; it++) RING_OK_OR_DIE(ring_graph_launch(graph, stream));
        RING_OK_OR_DIE(ring_stream_synchronize(stream));
        if (pass)
          printf("%d launches per step, %2d steps recorded as one HIP graph        %6.2f us per step\n", flags == 1 ? 3 : 2,
                 per, us_since(t0) / (kSteps / per * per));
      }
      RING_OK_OR_DIE(ring_graph_destroy(graph));
    }
  }
  return 0;
}
