/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the reference ring (tensorflow/contrib/mpi_collectives):
 * the checker the HIP data path is compared against, and the "port" CPU
 * baseline of the benchmark. Nothing in the product library may include,
 * link or call this; only tests, the smoke check and the benchmark's
 * cpu_baseline leg do.
 *
 * The reference itself cannot be compiled outside a TensorFlow build
 * (ring.h pulls the TF + Eigen header closure and generated protobuf
 * headers), so there is no build of the original sources next to this file.
 *
 * Every function below names the reference lines it follows; paths are
 * relative to tensorflow/contrib/mpi_collectives/ in the reference tree.
 */
#ifndef RING_ORACLE_H_
#define RING_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The three element types the reference dispatches on
 * (ring.cu.cc:14-20, mpi_ops.cc:478-508, mpi_ops.cc:836-847). */
enum { ORACLE_F32 = 0, ORACLE_I32 = 1, ORACLE_I64 = 2 };

/* sizeof(T) for a dtype code, 0 for an unknown code. */
size_t oracle_dtype_size(int dtype);

/* ring.h:150-166 — n segments of count/n elements, the first count%n get
 * one more; starts are the exclusive prefix sum. */
void oracle_segment_table(size_t count, int n, size_t* sizes, size_t* starts);

/* mpi_ops.cc:1073-1077 — elements of the temp tensor: ceil(count / n). */
size_t oracle_temp_elements(size_t count, int n);

/* ring.h:255-259 — allgather segment starts (in elements) from per-rank
 * first-dimension sizes and the elements per row. */
void oracle_allgather_table(const size_t* rows, int n, size_t elems_per_row,
                            size_t* starts);

/* ring.cc:36-38 — CopyTensorData<CPUDevice>: memcpy. */
void oracle_copy(void* dst, const void* src, size_t bytes);

/* ring.cc:41-50 — AccumulateTensorData<CPUDevice,T>: scalar dst[i] += src[i].
 * (The reference indexes with `unsigned int`; this uses size_t, identical for
 * every count below 2^32.) */
void oracle_accumulate_f32(float* dst, const float* src, size_t count);
void oracle_accumulate_i32(int32_t* dst, const int32_t* src, size_t count);
void oracle_accumulate_i64(int64_t* dst, const int64_t* src, size_t count);
void oracle_accumulate(int dtype, void* dst, const void* src, size_t count);

/* Point-to-point transport seen by one rank: the four MPI calls the ring
 * makes (ring.h:189-200, 221-224, 293-297), on bytes. Return 0 on success. */
typedef struct oracle_transport {
  void* self;
  int (*irecv)(void* self, void* buf, size_t bytes, int from);
  int (*send)(void* self, const void* buf, size_t bytes, int to);
  int (*wait)(void* self);
  int (*sendrecv)(void* self, const void* sbuf, size_t sbytes, int to,
                  void* rbuf, size_t rbytes, int from);
} oracle_transport;

/* Optional record of what one rank receives, step by step: slot i of
 * rs_recv holds the segment received at reduce-scatter step i and slot i of
 * ag_recv the one received at allgather step i; slots are `slot_elems`
 * elements apart. Either pointer may be NULL. */
typedef struct oracle_tap {
  void* rs_recv;
  void* ag_recv;
  size_t slot_elems;
} oracle_tap;

/* ring.h:136-228 — RingAllreduce for rank r of n, over raw buffers.
 * `temp` holds oracle_temp_elements(count, n) elements. Returns 0, or the
 * transport's error (the reference's errors::Unknown, ring.h:36-39). */
int oracle_ring_allreduce_rank(int n, int r, int dtype, const void* input,
                               void* temp, void* output, size_t count,
                               oracle_transport* tp, oracle_tap* tap);

/* ring.h:136-228 for one rank alone: rs_segments[i] is what the rank receives
 * at reduce-scatter step i, ag_segments[i] at allgather step i (n-1 of each,
 * of the sizes the segment table gives those steps); what it sends is
 * dropped. The per-rank data path on pre-staged peer segments. */
int oracle_ring_allreduce_rank_prestaged(int n, int r, int dtype,
                                         const void* input, void* output,
                                         size_t count,
                                         const void* const* rs_segments,
                                         const void* const* ag_segments);

/* ring.h:236-301 — RingAllgather for rank r of n. `rows[k]` is rank k's first
 * dimension, `input` holds rows[r]*elems_per_row elements, `output` the
 * concatenation. */
int oracle_ring_allgather_rank(int n, int r, int dtype, const void* input,
                               const size_t* rows, size_t elems_per_row,
                               void* output, oracle_transport* tp);

/* Run all n ranks of the allreduce in this process, one thread per rank over
 * an in-memory mailbox transport with MPI's ordering (one FIFO per directed
 * link). inputs[k]/outputs[k] are rank k's tensors; taps may be NULL or an
 * array of n taps. Returns 0 on success. */
int oracle_ring_allreduce_threads(int n, int dtype, size_t count,
                                  const void* const* inputs,
                                  void* const* outputs, oracle_tap* taps);

int oracle_ring_allgather_threads(int n, int dtype, const void* const* inputs,
                                  const size_t* rows, size_t elems_per_row,
                                  void* const* outputs);

/* Second, independent evaluation of the same schedule without threads or a
 * transport: all ranks advance in lockstep, step by step. Used to cross-check
 * the per-rank restatement above and for sizes where n threads with private
 * mailboxes would not fit. outputs[k] must not alias inputs. */
int oracle_ring_allreduce_lockstep(int n, int dtype, size_t count,
                                   const void* const* inputs,
                                   void* const* outputs);

/* Wall-clock timing of the threaded run: `reps` timed allreduces after
 * `warmup` untimed ones, all ranks released together by a barrier each rep;
 * seconds of the slowest rank per rep are written to secs[reps]. Only
 * RingAllreduce is inside the timed region. */
int oracle_time_allreduce_threads(int n, int dtype, size_t count,
                                  const void* const* inputs,
                                  void* const* outputs, int warmup, int reps,
                                  double* secs);

#ifdef __cplusplus
}
#endif
#endif /* RING_ORACLE_H_ */
