// A CPU stand-in for the few pieces of the HIP runtime that
// csrc/ring_kernels.hip uses. TEST INFRASTRUCTURE ONLY: it lets the kernel
// library be compiled as plain C++ (clang++ -fsanitize=address,undefined) so
// that every index a kernel computes is bounds- and alignment-checked on the
// CPU before the same code runs on a GPU. The product never sees this header:
// the package builds the library with hipcc against the real runtime.
//
// Model: launches run one at a time, whichever host thread makes them; a launch
// runs its workgroups one after the other; the threads of a
// workgroup are real OS threads (a pool of up to 1024) so that __syncthreads()
// is a real barrier; __shared__ variables are function-local statics, shared by
// the threads of the running workgroup. Streams and events do nothing: every
// launch has finished when the launch call returns. Device memory is host
// memory.
#ifndef HIP_CPU_SHIM_RUNTIME_H_
#define HIP_CPU_SHIM_RUNTIME_H_

#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

#define __device__
#define __global__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))
// what the kernel library lets a build for another target define: nothing to wait for on the
// CPU (every access has completed when the statement returns), and no occupancy attribute
#define RING_WAIT_VMEM() do {} while (0)
#define RING_WAVES_PER_SIMD(n)

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1 };
typedef struct shim_stream* hipStream_t;
typedef struct shim_event* hipEvent_t;
enum { hipStreamNonBlocking = 1, hipMemcpyHostToDevice = 1, hipDeviceAttributeMultiprocessorCount = 1 };

namespace hip_cpu_shim {

struct Idx { unsigned x, y, z; };
inline thread_local Idx t_thread = {0, 0, 0};
inline Idx g_block = {0, 0, 0};
inline Idx g_grid = {1, 1, 1};
inline Idx g_block_dim = {1, 1, 1};

// A pool of workgroup threads with a reusable barrier.
class Pool {
 public:
  static Pool& get() { static Pool p; return p; }
  // Runs fn on threads 0..n-1 (threadIdx.x) and waits for all of them.
  void run(unsigned n, const std::function<void()>& fn) {
    grow(n);
    {
      std::lock_guard<std::mutex> lock(mu_);
      fn_ = &fn;
      active_ = n;
      done_ = 0;
      barrier_count_ = 0;
      generation_++;
    }
    cv_.notify_all();
    std::unique_lock<std::mutex> lock(mu_);
    done_cv_.wait(lock, [&] { return done_ == n; });
  }
  void barrier() {
    std::unique_lock<std::mutex> lock(mu_);
    const uint64_t phase = barrier_phase_;
    if (++barrier_count_ == active_) {
      barrier_count_ = 0;
      barrier_phase_++;
      barrier_cv_.notify_all();
    } else {
      barrier_cv_.wait(lock, [&] { return barrier_phase_ != phase; });
    }
  }

 private:
  Pool() {}
  ~Pool() {
    {
      std::lock_guard<std::mutex> lock(mu_);
      stop_ = true;
      generation_++;
    }
    cv_.notify_all();
    for (auto& t : threads_) t.join();
  }
  void grow(unsigned n) {
    while (threads_.size() < n) {
      const unsigned id = static_cast<unsigned>(threads_.size());
      uint64_t seen;
      {
        std::lock_guard<std::mutex> lock(mu_);
        seen = generation_;
      }
      threads_.emplace_back([this, id, seen]() mutable {
        t_thread = {id, 0, 0};
        for (;;) {
          const std::function<void()>* fn;
          {
            std::unique_lock<std::mutex> lock(mu_);
            cv_.wait(lock, [&] { return generation_ != seen; });
            seen = generation_;
            if (stop_) return;
            if (id >= active_) continue;
            fn = fn_;
          }
          (*fn)();
          {
            std::lock_guard<std::mutex> lock(mu_);
            done_++;
          }
          done_cv_.notify_all();
        }
      });
    }
  }
  std::mutex mu_;
  std::condition_variable cv_, done_cv_, barrier_cv_;
  std::vector<std::thread> threads_;
  const std::function<void()>* fn_ = nullptr;
  unsigned active_ = 0, done_ = 0, barrier_count_ = 0;
  uint64_t generation_ = 0, barrier_phase_ = 0;
  bool stop_ = false;
};

// One device: launches from several host threads (one per rank of a ring over a
// transport) run one after the other, each to its end.
inline std::mutex g_device;

template <typename Kernel, typename... Args>
void launch(Kernel kernel, dim3 grid, dim3 block, Args... args) {
  std::lock_guard<std::mutex> device(g_device);
  g_grid = {grid.x, grid.y, grid.z};
  g_block_dim = {block.x, block.y, block.z};
  const std::function<void()> body = [&]() { kernel(args...); };
  for (unsigned z = 0; z < grid.z; z++)
    for (unsigned y = 0; y < grid.y; y++)
      for (unsigned x = 0; x < grid.x; x++) {
        g_block = {x, y, z};
        Pool::get().run(block.x, body);
      }
}

}  // namespace hip_cpu_shim

#define threadIdx (hip_cpu_shim::t_thread)
#define blockIdx (hip_cpu_shim::g_block)
#define gridDim (hip_cpu_shim::g_grid)
#define blockDim (hip_cpu_shim::g_block_dim)
inline void __syncthreads() { hip_cpu_shim::Pool::get().barrier(); }

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
  hip_cpu_shim::launch(kernel, grid, block, ##__VA_ARGS__)
#define hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, e0, e1, flags, ...) \
  hip_cpu_shim::launch(kernel, grid, block, ##__VA_ARGS__)

inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
inline hipError_t hipSetDevice(int dev) { return dev == 0 ? hipSuccess : hipErrorInvalidValue; }
inline hipError_t hipDeviceGetAttribute(int* value, int, int) { *value = 4; return hipSuccess; }
// exact-size heap blocks: an access one byte outside is an AddressSanitizer error
inline hipError_t hipMalloc(void** p, size_t bytes) { *p = malloc(bytes ? bytes : 1); return *p ? hipSuccess : hipErrorInvalidValue; }
template <typename T> inline hipError_t hipMalloc(T** p, size_t bytes) { return hipMalloc(reinterpret_cast<void**>(p), bytes); }
inline hipError_t hipFree(void* p) { free(p); return hipSuccess; }
inline hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, int) { memcpy(dst, src, bytes); return hipSuccess; }
// a stream is an address of its own (code above the library tells "no stream yet" from a stream by it)
inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) { *s = reinterpret_cast<hipStream_t>(malloc(1)); return hipSuccess; }
inline hipError_t hipStreamDestroy(hipStream_t s) { free(s); return hipSuccess; }
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
enum { hipEventDisableTiming = 2 };
enum hipStreamCaptureStatus { hipStreamCaptureStatusNone = 0, hipStreamCaptureStatusActive = 1 };
inline hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* status) { *status = hipStreamCaptureStatusNone; return hipSuccess; }
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { *e = reinterpret_cast<hipEvent_t>(malloc(1)); return hipSuccess; }
inline hipError_t hipEventCreate(hipEvent_t* e) { *e = reinterpret_cast<hipEvent_t>(malloc(1)); return hipSuccess; }
inline hipError_t hipEventDestroy(hipEvent_t e) { free(e); return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
// graphs are not modelled: capture fails, so nothing can be taken for recorded that in fact ran
typedef struct shim_graph* hipGraph_t;
typedef struct shim_graph_exec* hipGraphExec_t;
enum { hipStreamCaptureModeThreadLocal = 1 };
inline hipError_t hipStreamBeginCapture(hipStream_t, int) { return hipErrorInvalidValue; }
inline hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t*) { return hipErrorInvalidValue; }
inline hipError_t hipGraphInstantiate(hipGraphExec_t*, hipGraph_t, void*, void*, size_t) { return hipErrorInvalidValue; }
inline hipError_t hipGraphDestroy(hipGraph_t) { return hipSuccess; }
inline hipError_t hipGraphLaunch(hipGraphExec_t, hipStream_t) { return hipErrorInvalidValue; }
inline hipError_t hipGraphExecDestroy(hipGraphExec_t) { return hipSuccess; }
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 0.f; return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }

#endif  // HIP_CPU_SHIM_RUNTIME_H_
