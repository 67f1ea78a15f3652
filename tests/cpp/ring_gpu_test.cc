// End-to-end GPU test of the C ABI without Python or torch: plain HIP runtime
// for memory, libring_hip.so for the data path, libmpi_collectives.so for the
// ring driver, and the C oracle (oracle/ring_oracle.c) as the checker.
// Built by tensorflow-allreduce_amd/build.py into tests/cpp/build/, run on the
// GPU by tests/test_gpu_cpp.py. Prints "ok" and exits 0 when every comparison
// is bit-exact.
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <random>
#include <thread>
#include <vector>

#include "mpi_collectives.h"
#include "ring_abi.h"
#include "ring_oracle.h"

#define CHECK(cond)                                                                 \
  do {                                                                              \
    if (!(cond)) {                                                                  \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                                 \
    }                                                                               \
  } while (0)
#define HIP_OK(call) CHECK((call) == hipSuccess)

template <typename T>
static T* to_device(const std::vector<T>& v, size_t pad_front = 0) {
  char* d = nullptr;
  HIP_OK(hipMalloc(reinterpret_cast<void**>(&d), (v.size() + pad_front + 4) * sizeof(T)));
  if (!v.empty()) HIP_OK(hipMemcpy(d + pad_front * sizeof(T), v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return reinterpret_cast<T*>(d) + pad_front;
}

template <typename T>
static std::vector<T> to_host(const T* d, size_t n) {
  std::vector<T> v(n);
  if (n) HIP_OK(hipMemcpy(v.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
  return v;
}

template <typename T> struct Code;
template <> struct Code<float> { enum { ring = RING_F32, oracle = ORACLE_F32, mpic = MPIC_DT_FLOAT }; };
template <> struct Code<int32_t> { enum { ring = RING_I32, oracle = ORACLE_I32, mpic = MPIC_DT_INT32 }; };
template <> struct Code<int64_t> { enum { ring = RING_I64, oracle = ORACLE_I64, mpic = MPIC_DT_INT64 }; };

template <typename T>
static void fill(std::vector<T>& v, unsigned seed) {
  std::mt19937_64 gen(seed);
  for (auto& x : v) {
    const int64_t r = static_cast<int64_t>(gen() % 2000001) - 1000000;
    x = std::is_floating_point<T>::value ? static_cast<T>(static_cast<double>(r) * 1e-3 * ((gen() & 7) ? 1.0 : 1e4)) : static_cast<T>(r);
  }
}

template <typename T>
static void ring_case(int n, size_t count, void* stream) {
  // inputs of every rank, the oracle's result and what each rank receives
  std::vector<std::vector<T>> in(n, std::vector<T>(count)), want(n, std::vector<T>(count));
  const size_t slot = oracle_temp_elements(count, n);
  std::vector<std::vector<T>> rs(n, std::vector<T>(slot * (n > 1 ? n - 1 : 1))), ag = rs;
  std::vector<const void*> in_p(n);
  std::vector<void*> out_p(n);
  std::vector<oracle_tap> taps(n);
  for (int r = 0; r < n; r++) {
    fill(in[r], 1000u * n + r);
    in_p[r] = in[r].data();
    out_p[r] = want[r].data();
    taps[r] = oracle_tap{rs[r].data(), ag[r].data(), slot};
  }
  CHECK(oracle_ring_allreduce_threads(n, Code<T>::oracle, count, in_p.data(), out_p.data(), taps.data()) == 0);

  std::vector<size_t> sizes(n), starts(n);
  CHECK(ring_segment_table(count, n, sizes.data(), starts.data()) == RING_OK);

  // (1) one real rank at a time against pre-staged peers, through the step tables
  for (int r = 0; r < n; r += (n > 3 ? n - 1 : 1)) {
    T* d_in = to_device(in[r], r % 4);   // deliberately misaligned allocations
    T* d_out = to_device(std::vector<T>(count), (r + 1) % 4);
    std::vector<T*> d_rs, d_ag;
    std::vector<ring_step> rs_steps, ag_steps;
    for (int i = 0; i < n - 1; i++) {
      int snd, rcv;
      CHECK(ring_schedule(RING_PHASE_REDUCE_SCATTER, n, r, i, &snd, &rcv) == RING_OK);
      d_rs.push_back(to_device(std::vector<T>(rs[r].begin() + i * slot, rs[r].begin() + i * slot + sizes[rcv]), i % 3));
      rs_steps.push_back(ring_step{starts[rcv], d_rs.back(), sizes[rcv]});
      CHECK(ring_schedule(RING_PHASE_ALLGATHER, n, r, i, &snd, &rcv) == RING_OK);
      d_ag.push_back(to_device(std::vector<T>(ag[r].begin() + i * slot, ag[r].begin() + i * slot + sizes[rcv]), (i + 1) % 3));
      ag_steps.push_back(ring_step{starts[rcv], d_ag.back(), sizes[rcv]});
    }
    CHECK(ring_copy_bytes(d_out, d_in, count * sizeof(T), stream) == RING_OK);
    CHECK(ring_reduce_scatter_steps(d_out, rs_steps.data(), n - 1, Code<T>::ring, stream) == RING_OK);
    CHECK(ring_allgather_steps(d_out, ag_steps.data(), n - 1, Code<T>::ring, stream) == RING_OK);
    CHECK(ring_stream_synchronize(stream) == RING_OK);
    CHECK(std::memcmp(to_host(d_out, count).data(), want[r].data(), count * sizeof(T)) == 0);
    // the same through the ring driver, copy folded into the accumulate
    std::vector<const void*> rs_p(d_rs.begin(), d_rs.end()), ag_p(d_ag.begin(), d_ag.end());
    // on the ring's own stream: a memset on the null stream is not ordered with a non-blocking stream
    HIP_OK(hipMemsetAsync(d_out, 0, count * sizeof(T), static_cast<hipStream_t>(stream)));
    CHECK(mpic_ring_allreduce_prestaged(n, r, Code<T>::mpic, d_in, d_out, count, rs_p.data(), ag_p.data(), stream, 3) == MPIC_OK);
    CHECK(ring_stream_synchronize(stream) == RING_OK);
    CHECK(std::memcmp(to_host(d_out, count).data(), want[r].data(), count * sizeof(T)) == 0);
    // the direct form: every peer's raw copy of the owned segment, folded in ring order in one pass
    const int own = (r + 1) % n;
    std::vector<const void*> raw;
    for (int k = 0; k < n - 1; k++) {
      const std::vector<T>& peer = in[(own + k) % n];
      raw.push_back(to_device(std::vector<T>(peer.begin() + starts[own], peer.begin() + starts[own] + sizes[own]), k % 4));
    }
    // on the ring's own stream: a memset on the null stream is not ordered with a non-blocking stream
    HIP_OK(hipMemsetAsync(d_out, 0, count * sizeof(T), static_cast<hipStream_t>(stream)));
    CHECK(mpic_ring_allreduce_direct_prestaged(n, r, Code<T>::mpic, d_in, d_out, count, raw.data(), ag_p.data(), stream,
                                               r % 2) == MPIC_OK);
    CHECK(ring_stream_synchronize(stream) == RING_OK);
    CHECK(std::memcmp(to_host(d_out, count).data(), want[r].data(), count * sizeof(T)) == 0);
  }

  // (2) all ranks resident: the neighbour's buffer is the transport
  std::vector<const void*> d_ins(n);
  std::vector<void*> d_outs(n);
  for (int r = 0; r < n; r++) {
    d_ins[r] = to_device(in[r]);
    d_outs[r] = to_device(std::vector<T>(count));
  }
  CHECK(mpic_ring_allreduce_all_ranks(n, Code<T>::mpic, d_ins.data(), d_outs.data(), count, stream, (n % 2) ? 1 : 3) == MPIC_OK);
  CHECK(ring_stream_synchronize(stream) == RING_OK);
  for (int r = 0; r < n; r++)
    CHECK(std::memcmp(to_host(static_cast<T*>(d_outs[r]), count).data(), want[r].data(), count * sizeof(T)) == 0);

  // (3) one thread per rank, segments exchanged through the loopback transport
  // in 4 pieces with a two-segment temp: the reference's loop, pipelined
  mpic_loopback* lb = nullptr;
  CHECK(mpic_loopback_create(n, 30.0, &lb) == MPIC_OK);
  std::vector<T*> d_temp(n);
  for (int r = 0; r < n; r++) {
    HIP_OK(hipMemset(d_outs[r], 0, count * sizeof(T)));
    d_temp[r] = to_device(std::vector<T>(2 * slot + 1));
  }
  HIP_OK(hipDeviceSynchronize());
  std::atomic<int> failures{0};
  std::vector<std::thread> threads;
  for (int r = 0; r < n; r++) {
    threads.emplace_back([&, r] {
      mpic_transport t;
      void* own_stream = nullptr;
      if (mpic_loopback_endpoint(lb, r, &t) != MPIC_OK || ring_stream_create(&own_stream) != RING_OK) {
        failures++;
        return;
      }
      if (mpic_ring_allreduce_transport(n, r, Code<T>::mpic, d_ins[r], d_outs[r], d_temp[r], 2 * slot, count, &t,
                                        own_stream, (4 - 1) << 4) != MPIC_OK) {
        std::fprintf(stderr, "rank %d: %s\n", r, mpic_last_error());
        failures++;
      }
      ring_stream_destroy(own_stream);
    });
  }
  for (auto& th : threads) th.join();
  CHECK(failures == 0);
  CHECK(mpic_loopback_destroy(lb) == MPIC_OK);
  for (int r = 0; r < n; r++)
    CHECK(std::memcmp(to_host(static_cast<T*>(d_outs[r]), count).data(), want[r].data(), count * sizeof(T)) == 0);
}

int main() {
  int devices = 0;
  HIP_OK(hipGetDeviceCount(&devices));
  CHECK(devices >= 1);
  CHECK(ring_abi_version() == RING_ABI_VERSION);
  void* stream = nullptr;
  CHECK(ring_stream_create(&stream) == RING_OK);
  const size_t counts[] = {0, 1, 5, 4099, 1000003};
  const int ranks[] = {1, 2, 3, 6, 8};
  for (int n : ranks)
    for (size_t count : counts) {
      ring_case<float>(n, count, stream);
      ring_case<int32_t>(n, count, stream);
      ring_case<int64_t>(n, count, stream);
    }
  CHECK(ring_stream_destroy(stream) == RING_OK);
  std::printf("ok\n");
  return 0;
}
