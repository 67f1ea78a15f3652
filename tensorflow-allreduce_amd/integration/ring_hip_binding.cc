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
// Inside a TensorFlow tree the seam's declarations come from ring.h itself.
// Outside one (this repository's own GPU test of the file) they are declared
// here exactly as ring.h:44-51 declares them, with Eigen::GpuDevice as an
// incomplete type: the specialisations never touch a device object.
#include <stddef.h>
#include <stdint.h>

#include "ring_abi.h"

#if defined(__has_include)
#if __has_include("tensorflow/contrib/mpi_collectives/ring.h")
#define RING_BINDING_IN_TENSORFLOW_TREE 1
#endif
#endif

#ifdef RING_BINDING_IN_TENSORFLOW_TREE
#define EIGEN_USE_GPU
#include "tensorflow/contrib/mpi_collectives/ring.h"
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

// The dedicated stream (CudaStreamForMPI, mpi_ops.cc:213-230, 872-876): one
// non-default stream for every copy and accumulate of the ring, created on
// first use by the background thread that runs the collectives.
void* HipStreamForMPI() {
  static void* stream = nullptr;
  if (!stream && ring_stream_create(&stream) != RING_OK) stream = nullptr;
  return stream;
}

// ring.cu.cc:41-45: copy on the dedicated stream, then wait for it.
template <>
void CopyTensorData<GPUDevice>(void* dst, void* src, size_t size) {
  void* stream = HipStreamForMPI();
  ring_copy_bytes(dst, src, size, stream);
  ring_stream_synchronize(stream);
}

// ring.cu.cc:48-69: dst[i] += src[i] on the dedicated stream, then wait for it.
template <>
void AccumulateTensorData<GPUDevice, float>(float* dst, float* src, size_t size) {
  void* stream = HipStreamForMPI();
  ring_accumulate_f32(dst, src, size, stream);
  ring_stream_synchronize(stream);
}
template <>
void AccumulateTensorData<GPUDevice, int>(int* dst, int* src, size_t size) {
  void* stream = HipStreamForMPI();
  ring_accumulate_i32(dst, src, size, stream);
  ring_stream_synchronize(stream);
}
template <>
void AccumulateTensorData<GPUDevice, long long>(long long* dst, long long* src, size_t size) {
  void* stream = HipStreamForMPI();
  ring_accumulate_i64(reinterpret_cast<int64_t*>(dst), reinterpret_cast<const int64_t*>(src), size, stream);
  ring_stream_synchronize(stream);
}

}  // namespace mpi
}  // namespace contrib
}  // namespace tensorflow
