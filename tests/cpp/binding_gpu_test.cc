// GPU test of the reference-side binding
// (tensorflow-allreduce_amd/integration/ring_hip_binding.cc): the seam of
// tensorflow/contrib/mpi_collectives/ring.h:44-51, CopyTensorData<GPUDevice> and
// AccumulateTensorData<GPUDevice, T>, called the way ring.h calls it, with the
// reference's synchronous contract (nothing here synchronises a stream: a
// result read back right after a call must be complete), against the C oracle.
// Then the reference's own loop structure (ring.h:170-225: receive into temp,
// accumulate, receive in place) for n ranks resident on the GPU, a plain
// device-to-device copy standing in for each MPI transfer, against the
// oracle's ring. Built by tensorflow-allreduce_amd/build.py, run on the GPU by
// tests/test_gpu_cpp.py. Prints "ok" when every comparison is bit-exact.
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "ring_abi.h"
#include "ring_oracle.h"

namespace Eigen {
struct GpuDevice;
}
namespace tensorflow {
namespace contrib {
namespace mpi {
template <typename Device> void CopyTensorData(void* destination, void* source, size_t size);
template <typename Device, typename T> void AccumulateTensorData(T* destination, T* source, size_t size);
int RingDeviceStatusTake();

// What the patched mpi_ops.cc provides (mpi_ops.cc:213-230 the stream member, :582-583 its creation on the
// background thread after the device has been made current, :872-876 the accessor ring.h:55-57 declares):
// here the test is the owner of the stream.
static void* g_stream_for_mpi = nullptr;
void* CudaStreamForMPI() { return g_stream_for_mpi; }
static bool CreateStreamForMPI() {
  int device = -1;
  return ring_get_device(&device) == RING_OK && ring_set_device(device) == RING_OK &&
         ring_stream_create(&g_stream_for_mpi) == RING_OK && g_stream_for_mpi != nullptr;
}
}  // namespace mpi
}  // namespace contrib
}  // namespace tensorflow
using tensorflow::contrib::mpi::AccumulateTensorData;
using tensorflow::contrib::mpi::CopyTensorData;
using GPUDevice = Eigen::GpuDevice;

#define CHECK(cond)                                                                 \
  do {                                                                              \
    if (!(cond)) {                                                                  \
      std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond); \
      std::exit(1);                                                                 \
    }                                                                               \
  } while (0)
#define HIP_OK(call) CHECK((call) == hipSuccess)

template <typename T> struct OracleCode;
template <> struct OracleCode<float> { enum { value = ORACLE_F32 }; };
template <> struct OracleCode<int> { enum { value = ORACLE_I32 }; };
template <> struct OracleCode<long long> { enum { value = ORACLE_I64 }; };

template <typename T>
static void fill(std::vector<T>& v, unsigned seed) {
  std::mt19937_64 gen(seed);
  for (auto& x : v) {
    const long long r = static_cast<long long>(gen() % 2000001) - 1000000;
    x = std::is_floating_point<T>::value ? static_cast<T>(static_cast<double>(r) * 1e-3) : static_cast<T>(r);
  }
}

template <typename T>
static T* device_copy(const std::vector<T>& v, size_t lead) {
  char* d = nullptr;
  HIP_OK(hipMalloc(reinterpret_cast<void**>(&d), (v.size() + lead + 4) * sizeof(T)));
  if (!v.empty()) HIP_OK(hipMemcpy(d + lead * sizeof(T), v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return reinterpret_cast<T*>(d) + lead;
}

template <typename T>
static void primitives() {
  const size_t counts[] = {0, 1, 5, 1024, 4097, 1000003};
  for (size_t count : counts)
    for (size_t lead = 0; lead < 4; lead += 3) {
      std::vector<T> a(count), b(count);
      fill(a, 7 + static_cast<unsigned>(count));
      fill(b, 9 + static_cast<unsigned>(count));
      T* da = device_copy(a, lead);
      T* db = device_copy(b, (lead + 1) % 4);
      AccumulateTensorData<GPUDevice, T>(da, db, count);       // ring.h:203-204
      std::vector<T> got(count), want(a);
      if (count) HIP_OK(hipMemcpy(got.data(), da, count * sizeof(T), hipMemcpyDeviceToHost));
      oracle_accumulate(OracleCode<T>::value, want.data(), b.data(), count);
      CHECK(std::memcmp(got.data(), want.data(), count * sizeof(T)) == 0);
      std::vector<T> zero(count, T());
      T* dc = device_copy(zero, lead);
      CopyTensorData<GPUDevice>(dc, db, count * sizeof(T));      // ring.h:146-148
      if (count) HIP_OK(hipMemcpy(got.data(), dc, count * sizeof(T), hipMemcpyDeviceToHost));
      oracle_copy(want.data(), b.data(), count * sizeof(T));
      CHECK(std::memcmp(got.data(), want.data(), count * sizeof(T)) == 0);
      HIP_OK(hipFree(reinterpret_cast<char*>(da) - lead * sizeof(T)));
      HIP_OK(hipFree(reinterpret_cast<char*>(db) - ((lead + 1) % 4) * sizeof(T)));
      HIP_OK(hipFree(reinterpret_cast<char*>(dc) - lead * sizeof(T)));
    }
}

// RingAllreduce of ring.h:136-228 for n ranks in lockstep, every rank's buffers on this GPU.
template <typename T>
static void reference_loop(int n, size_t count) {
  std::vector<std::vector<T>> in(n, std::vector<T>(count));
  std::vector<T*> input(n), buffer(n), temp(n);
  std::vector<size_t> sizes(n), starts(n);
  CHECK(ring_segment_table(count, n, sizes.data(), starts.data()) == RING_OK);
  const size_t temp_elems = ring_temp_elements(count, n);
  for (int r = 0; r < n; r++) {
    fill(in[r], 100 + r);
    input[r] = device_copy(in[r], 0);
    buffer[r] = device_copy(std::vector<T>(count, T()), 0);
    temp[r] = device_copy(std::vector<T>(temp_elems, T()), 0);
    CopyTensorData<GPUDevice>(buffer[r], input[r], count * sizeof(T));                     // ring.h:146-148
  }
  auto mod = [n](int x) { return ((x % n) + n) % n; };
  for (int i = 0; i < n - 1; i++) {                                                        // ring.h:183-205
    for (int r = 0; r < n; r++) {   // MPI_Irecv into temp / MPI_Send of segment (r-i) to r+1
      const int send = mod(r - i), to = mod(r + 1);
      HIP_OK(hipMemcpy(temp[to], buffer[r] + starts[send], sizes[send] * sizeof(T), hipMemcpyDeviceToDevice));
    }
    // a device-to-device hipMemcpy may return before the copy has run, and the binding's stream does
    // not wait for the null stream: the "receive" is complete (MPI_Wait, ring.h:200) only after this
    HIP_OK(hipDeviceSynchronize());
    for (int r = 0; r < n; r++) {
      const int recv = mod(r - i - 1);
      AccumulateTensorData<GPUDevice, T>(buffer[r] + starts[recv], temp[r], sizes[recv]);
    }
  }
  for (int i = 0; i < n - 1; i++) {                                                        // ring.h:211-225
    std::vector<std::vector<T>> wire(n);
    for (int r = 0; r < n; r++) {   // MPI_Sendrecv: segment (r-i+1) goes to r+1, in place
      const int send = mod(r - i + 1);
      wire[r].resize(sizes[send]);
      if (sizes[send]) HIP_OK(hipMemcpy(wire[r].data(), buffer[r] + starts[send], sizes[send] * sizeof(T), hipMemcpyDeviceToHost));
    }
    for (int r = 0; r < n; r++) {
      const int from = mod(r - 1), recv = mod(r - i);
      if (sizes[recv]) HIP_OK(hipMemcpy(buffer[r] + starts[recv], wire[from].data(), sizes[recv] * sizeof(T), hipMemcpyHostToDevice));
    }
  }
  std::vector<const void*> ins(n);
  std::vector<std::vector<T>> want(n, std::vector<T>(count));
  std::vector<void*> outs(n);
  for (int r = 0; r < n; r++) { ins[r] = in[r].data(); outs[r] = want[r].data(); }
  CHECK(oracle_ring_allreduce_lockstep(n, OracleCode<T>::value, count, ins.data(), outs.data()) == 0);
  for (int r = 0; r < n; r++) {
    std::vector<T> got(count);
    if (count) HIP_OK(hipMemcpy(got.data(), buffer[r], count * sizeof(T), hipMemcpyDeviceToHost));
    CHECK(std::memcmp(got.data(), want[r].data(), count * sizeof(T)) == 0);
    HIP_OK(hipFree(input[r])); HIP_OK(hipFree(buffer[r])); HIP_OK(hipFree(temp[r]));
  }
}

// A failed device call is not dropped (the reference's seam is void and drops them): the first status is
// kept for the thread and handed out once.
static void failures_are_remembered() {
  using tensorflow::contrib::mpi::RingDeviceStatusTake;
  CHECK(RingDeviceStatusTake() == RING_OK);
  std::vector<float> a(64, 1.f);
  float* da = device_copy(a, 0);
  AccumulateTensorData<GPUDevice, float>(nullptr, da, 64);                        // no destination
  AccumulateTensorData<GPUDevice, float>(da, da, 64);                             // a good call does not clear it
  CHECK(RingDeviceStatusTake() == RING_ERR_ARGUMENT);
  CHECK(RingDeviceStatusTake() == RING_OK);
  CopyTensorData<GPUDevice>(nullptr, da, 16);
  CHECK(RingDeviceStatusTake() == RING_ERR_ARGUMENT);
  HIP_OK(hipFree(da));
}

int main() {
  CHECK(tensorflow::contrib::mpi::CreateStreamForMPI());
  failures_are_remembered();
  primitives<float>();
  primitives<int>();
  primitives<long long>();
  reference_loop<float>(3, 10007);
  reference_loop<float>(8, 1000003);
  reference_loop<int>(6, 100019);
  reference_loop<long long>(5, 4099);
  reference_loop<float>(4, 2);       // fewer elements than ranks: empty segments
  CHECK(tensorflow::contrib::mpi::RingDeviceStatusTake() == RING_OK);
  std::printf("ok\n");
  return 0;
}
