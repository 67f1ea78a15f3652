// ring_hip_binding.cc — what a maintainer of the reference puts in the place of
// tensorflow/contrib/mpi_collectives/ring.cu.cc to run its ring on an MI355X.
//
// The reference keeps one seam between the ring algorithm and the device
// (ring.h:44-57): CopyTensorData<Device>, AccumulateTensorData<Device, T> and
// the dedicated stream. ring.cu.cc:41-69 implements it with cudaMemcpyAsync,
// elemwise_accum<<<32, 256>>> and a stream synchronisation after every call.
// This file implements the same three template specialisations (plus the MPI
// type map ring.cu.cc:14-20 defines, which ring.h's RingAllreduce needs) over
// the C ABI of include/ring_abi.h. It is plain C++: no hipcc, only -lring_hip.
// RingAllreduce<GPUDevice, T> / RingAllgather<GPUDevice, T> of ring.h then run
// unchanged, with the same results bit for bit (one IEEE add per element per
// step), and the contract stays the reference's: every call has finished when
// it returns.
//
// The dedicated stream is NOT this file's: as in the reference, ring.h declares
// the accessor (ring.h:55-57) and mpi_ops.cc, which owns the stream, defines it
// (mpi_ops.cc:213-230 the member, :582-583 its creation on the background
// thread, :872-876 the accessor). integration/mpi_ops_hip.patch holds those
// edits for a ROCm build, where the accessor returns the opaque stream of
// ring_stream_create instead of a cudaStream_t.
//
// The seam is void and the reference drops CUDA errors (ring.cu.cc:41-69 checks
// no return code). Here a failed call is remembered per thread, the first one
// wins, and RingDeviceStatusTake() hands it to the caller and clears it: the
// patched PerformCollectiveOp turns it into the op's status after RingAllreduce /
// RingAllgather have returned. Inside a TensorFlow tree it is logged as well.
//
// Inside a TensorFlow tree the seam's declarations come from ring.h itself.
// Outside one (this repository's own GPU test of the file) they are declared
// here exactly as ring.h:44-57 declares them (as patched), with Eigen::GpuDevice
// as an incomplete type: the specialisations never touch a device object.
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "ring_abi.h"

#if defined(__has_include)
#if __has_include("tensorflow/contrib/mpi_collectives/ring.h")
#define RING_BINDING_IN_TENSORFLOW_TREE 1
#endif
#endif

#ifdef RING_BINDING_IN_TENSORFLOW_TREE
// (no EIGEN_USE_GPU: this file is compiled by the host compiler, and ring.h needs
// Eigen::GpuDevice as a name only, which Eigen forward-declares)
#include "tensorflow/contrib/mpi_collectives/ring.h"
#include "tensorflow/core/platform/logging.h"
#else
namespace Eigen {
struct GpuDevice;
}
namespace tensorflow {
namespace contrib {
namespace mpi {
template <typename Device>
void CopyTensorData(void* destination, void* source, size_t size);               // ring.h:44-45
template <typename Device, typename T>
void AccumulateTensorData(T* destination, T* source, size_t size);               // ring.h:50-51
void* CudaStreamForMPI();                                                        // ring.h:55-57, as patched for ROCm
}  // namespace mpi
}  // namespace contrib
}  // namespace tensorflow
#endif

namespace tensorflow {
namespace contrib {
namespace mpi {

using GPUDevice = Eigen::GpuDevice;

#ifdef RING_BINDING_IN_TENSORFLOW_TREE
// ring.cu.cc:14-20: declared extern in ring.cc, defined in the GPU translation unit.
template <> MPI_Datatype MPIType<float>() { return MPI_FLOAT; };
template <> MPI_Datatype MPIType<int>() { return MPI_INT; };
template <> MPI_Datatype MPIType<long long>() { return MPI_LONG_LONG; };
template <> DataType TensorFlowDataType<float>() { return DT_FLOAT; };
template <> DataType TensorFlowDataType<int>() { return DT_INT32; };
template <> DataType TensorFlowDataType<long long>() { return DT_INT64; };
#endif

namespace {
thread_local int g_device_status = RING_OK;  // first failed ring_abi call of this thread since the last take

inline void Remember(int rc, const char* what) {
  if (rc == RING_OK) return;
  if (g_device_status == RING_OK) g_device_status = rc;
#ifdef RING_BINDING_IN_TENSORFLOW_TREE
  LOG(ERROR) << what << " failed: " << ring_status_string(rc)
             << (rc == RING_ERR_HIP ? " (hipError " + std::to_string(ring_last_hip_error()) + ")" : std::string());
#else
  (void)what;
#endif
}
}  // namespace

// The first ring_abi status other than RING_OK that a call of this seam met on
// the calling thread since the last call of this function (RING_OK if none);
// ring_status_string() names it. The ring runs on one thread (the background
// thread, mpi_ops.cc:572), which is the thread that asks.
int RingDeviceStatusTake() {
  const int rc = g_device_status;
  g_device_status = RING_OK;
  return rc;
}

// ring.cu.cc:41-45: copy on the dedicated stream, then wait for it.
template <>
void CopyTensorData<GPUDevice>(void* dst, void* src, size_t size) {
  void* stream = CudaStreamForMPI();
  Remember(ring_copy_bytes(dst, src, size, stream), "ring_copy_bytes");
  Remember(ring_stream_synchronize(stream), "ring_stream_synchronize");
}

// ring.cu.cc:48-69: dst[i] += src[i] on the dedicated stream, then wait for it.
template <>
void AccumulateTensorData<GPUDevice, float>(float* dst, float* src, size_t size) {
  void* stream = CudaStreamForMPI();
  Remember(ring_accumulate_f32(dst, src, size, stream), "ring_accumulate_f32");
  Remember(ring_stream_synchronize(stream), "ring_stream_synchronize");
}
template <>
void AccumulateTensorData<GPUDevice, int>(int* dst, int* src, size_t size) {
  void* stream = CudaStreamForMPI();
  Remember(ring_accumulate_i32(dst, src, size, stream), "ring_accumulate_i32");
  Remember(ring_stream_synchronize(stream), "ring_stream_synchronize");
}
template <>
void AccumulateTensorData<GPUDevice, long long>(long long* dst, long long* src, size_t size) {
  void* stream = CudaStreamForMPI();
  Remember(ring_accumulate_i64(reinterpret_cast<int64_t*>(dst), reinterpret_cast<const int64_t*>(src), size, stream),
           "ring_accumulate_i64");
  Remember(ring_stream_synchronize(stream), "ring_stream_synchronize");
}

#ifdef RING_BINDING_IN_TENSORFLOW_TREE
// mpi_ops.cc:86-96 declares the GPU instantiations of the two ring templates
// extern: the GPU translation unit provides them (ring.cu.cc:21-37), after the
// specialisations above so that the loops of ring.h bind to them.
#define RING_BINDING_INSTANTIATE(T)                                                                      \
  template Status RingAllreduce<GPUDevice, T>(OpKernelContext*, const Tensor*, Tensor*, Tensor*);       \
  template Status RingAllgather<GPUDevice, T>(OpKernelContext*, const Tensor*, const std::vector<size_t>&, Tensor*);
RING_BINDING_INSTANTIATE(int)
RING_BINDING_INSTANTIATE(long long)
RING_BINDING_INSTANTIATE(float)
#undef RING_BINDING_INSTANTIATE
#endif

}  // namespace mpi
}  // namespace contrib
}  // namespace tensorflow
