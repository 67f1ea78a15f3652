/*
 * mpi_collectives.h — C interface of the plugin library (libmpi_collectives.so),
 * the counterpart of the reference's mpi_collectives.so
 * (tensorflow/contrib/mpi_collectives/mpi_ops.cc, ring.h): the op registry
 * with the six MPI ops, their OpKernels, the readiness table / background
 * thread, and the host-side ring driver. It contains no GPU code; every
 * device operation goes through the C ABI of ring_abi.h.
 *
 * The reference is loaded into TensorFlow with tf.load_op_library() and driven
 * by the TF executor (mpi_ops.py:30-59). Without TensorFlow the same ops are
 * driven through the `mpic_context_*` calls below, which play the part of
 * OpKernelContext / AsyncOpKernel::ComputeAsync(ctx, done)
 * (tensorflow/core/framework/op_kernel.h:181-198).
 *
 * Ranks are VIRTUAL: one process, one GPU. A world either holds all `size`
 * ranks (each submits its own tensor under the same node name, as separate
 * MPI processes would) or a single real rank whose peers' incoming segments
 * were staged in device memory beforehand.
 *
 * Status codes are TensorFlow's (tensorflow/core/lib/core/error_codes.proto):
 * 0 OK, 2 UNKNOWN, 3 INVALID_ARGUMENT, 5 NOT_FOUND, 9 FAILED_PRECONDITION,
 * 13 INTERNAL. Data types use TensorFlow's DataType numbering
 * (tensorflow/core/framework/types.proto): 1 float32, 3 int32, 9 int64; any
 * other value is rejected with "Invalid tensor type passed." (mpi_ops.cc:844).
 */
#ifndef MPI_COLLECTIVES_H_
#define MPI_COLLECTIVES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum mpic_code {
  MPIC_OK = 0, MPIC_UNKNOWN = 2, MPIC_INVALID_ARGUMENT = 3, MPIC_NOT_FOUND = 5,
  MPIC_FAILED_PRECONDITION = 9, MPIC_INTERNAL = 13
};
enum mpic_dtype { MPIC_DT_INVALID = 0, MPIC_DT_FLOAT = 1, MPIC_DT_DOUBLE = 2, MPIC_DT_INT32 = 3, MPIC_DT_INT64 = 9 };

typedef struct mpic_world mpic_world;
typedef struct mpic_context mpic_context;

/* ---- op registry: what REGISTER_OP / REGISTER_KERNEL_BUILDER recorded at load
 * time (mpi_ops.cc:900-907, 937-950, 979-992, 1024-1037, 1119-1139, 1233-1259).
 * The Python loader checks the op list as mpi_ops.py:57-59 does. ------------ */
int mpic_op_count(void);
const char* mpic_op_name(int index);
/* One-line signature, e.g. "MPIAllreduce(tensor: T) -> (sum: T); T: {int32, int64, float32}";
 * NULL if the op is not registered. */
const char* mpic_op_signature(const char* op);
const char* mpic_op_doc(const char* op);
/* 1 if a kernel is registered for (op, device), device = "CPU" or "GPU". */
int mpic_op_has_kernel(const char* op, const char* device);
/* Shape function of the op (mpi_ops.cc:1123-1126, 1239-1245): writes the
 * output shape for input 0's shape; unknown dimensions are -1. Returns the
 * output rank, or -1 if the op has no outputs / is unknown. */
int mpic_op_infer_shape(const char* op, int ndims, const int64_t* dims, int64_t* out_dims);

/* ---- worlds (MPIGlobalState, mpi_ops.cc:165-240) ------------------------- */

/* All `size` ranks live in this process and share the current GPU. A
 * collective starts when every rank has submitted it (mpi_ops.cc:255-269). */
int mpic_world_create(int size, mpic_world** world);
/* Only `rank` is real; what its neighbour would send is staged with
 * mpic_stage_* before the op runs. */
int mpic_world_create_prestaged(int size, int rank, mpic_world** world);
/* Stops the background thread (SHUTDOWN, mpi_ops.cc:744-753) and frees the
 * world. Pending ops fail with UNKNOWN. */
int mpic_world_destroy(mpic_world* world);
int mpic_world_size(const mpic_world* world);
/* The dedicated stream of the world (CudaStreamForMPI, mpi_ops.cc:872-876), as
 * a hipStream_t. Valid after MPIInit has run. */
void* mpic_world_stream(const mpic_world* world);
/* Options: "batched" (1: one launch per ring phase, 0: one launch per ring
 * step as in ring.h:183-225; default 1), "fuse_copy" (1: fold the in->out copy
 * of ring.h:146-148 into the reduce-scatter, out[seg] = in[seg] + received, the
 * same single add; default 1), "direct" (worlds that hold all ranks: 1 = the
 * direct form of mpic_ring_allreduce_all_ranks, default; 0 = the lockstep
 * ring), "sync" (1: done() is called after
 * the stream has drained, 0: as soon as the work is enqueued). */
int mpic_world_set_option(mpic_world* world, const char* name, int value);

/* Tensor fusion in the coordinator (no counterpart in the reference, which runs
 * one collective and one negotiation round per gradient, __init__.py:195-205).
 * `buffer` is caller-owned device memory of size()*bytes_per_rank bytes, 16-byte
 * aligned, rank r using slice r; bytes_per_rank (a multiple of 16) is the
 * fusion threshold, 0 switches fusion off. While it is on, submitted
 * collectives wait for mpic_world_flush(); at a flush, consecutive ready
 * allreduces of one element type that fit the buffer together are packed per
 * rank, reduced by ONE ring in place and unpacked into each op's output. Each
 * tensor's result is then the reference ring applied to the packed buffer,
 * which for float32 rounds differently from a ring per tensor (an element
 * lands in another segment); grouping depends only on submission order and
 * flush points, not on timing. Worlds with pre-staged peers never fuse. In
 * the direct form (option "direct", the default) a group of up to 16 ranks
 * whose tensors ask for the same divisor is reduced on the tensors themselves
 * by one launch (ring_fusion_allreduce_all), with the same results, and the
 * buffer only bounds the size of a group. */
int mpic_world_set_fusion_buffer(mpic_world* world, void* buffer, size_t bytes_per_rank);
/* Start a tick now: everything submitted so far is negotiated and run. */
int mpic_world_flush(mpic_world* world);

/* Pre-staged peers for the op with node name `name`, consumed by the next
 * collective of that name: rs_segments[i] / ag_segments[i] are device pointers
 * to what the left neighbour sends at reduce-scatter / allgather step i
 * (n-1 each; sizes follow ring_segment_table). For an allgather pass
 * rs_segments = NULL and ag_segments[i] = the segment received at step i. */
int mpic_stage_peers(mpic_world* world, const char* name,
                     const void* const* rs_segments, const void* const* ag_segments);

/* ---- running one op instance (OpKernelContext + ComputeAsync) -------------- */

/* Output allocator supplied by the embedding framework (allocate_output,
 * op_kernel.h:803-832): returns memory for a tensor of the given type and
 * shape, on the host if `host_memory`, else on the GPU; NULL on failure. */
typedef void* (*mpic_alloc_fn)(void* user, int dtype, int ndims, const int64_t* dims, int host_memory);

/* `op`: registered op name; `node_name`: the graph node name collectives are
 * matched by across ranks (mpi_ops.cc:1062, 1127-1131); `device`: "CPU"/"GPU". */
int mpic_context_create(mpic_world* world, int rank, const char* op, const char* node_name,
                        const char* device, mpic_alloc_fn alloc, void* user, mpic_context** ctx);
/* An input tensor: at most 8 dimensions, none negative, and a size in bytes that
 * fits 63 bits (INVALID_ARGUMENT otherwise, here and for the tensors of
 * mpic_allreduce_batch / mpic_batch_create). */
int mpic_context_add_input(mpic_context* ctx, int dtype, int ndims, const int64_t* dims,
                           const void* data, int host_memory);
/* Fuses the graph's tf.div(output, divisor) consumer into this node: the
 * reference's allreduce(average=True) is MPIAllreduce followed by
 * tf.div(summed_tensor, size()) (__init__.py:160-164; :153-157 divides the
 * gathered values of an IndexedSlices). With a divisor > 0 an MPIAllreduce /
 * MPIAllgather node delivers exactly that quotient (true division for float32,
 * floor division for the integers) without a pass of its own: the divide rides
 * on the last accumulate of each segment (on the unpack for fused tensors, on
 * the own-slice copy of an allgather). Every rank must ask for the same
 * divisor. In a world with pre-staged peers the allgather-phase segments are
 * what a peer would send: already divided. Call before mpic_context_compute. */
int mpic_context_set_divisor(mpic_context* ctx, int divisor);
/* Runs Compute / ComputeAsync on the calling thread and returns. */
int mpic_context_compute(mpic_context* ctx);
/* Blocks until the op's done() ran; returns its status code. */
int mpic_context_wait(mpic_context* ctx);
const char* mpic_context_message(const mpic_context* ctx);
int mpic_context_num_outputs(const mpic_context* ctx);
int mpic_context_output(const mpic_context* ctx, int index, int* dtype, int* ndims,
                        int64_t* dims /* room for 8 */, void** data);
/* 1 when the op's done() has run (or the op was never started), else 0: whether
 * mpic_context_destroy would return at once. */
int mpic_context_done(mpic_context* ctx);
/* Waits for a started op's done() before it frees the context. */
int mpic_context_destroy(mpic_context* ctx);

/* k MPIAllreduce nodes of one rank in one call: what k rounds of
 * mpic_context_create / add_input / set_divisor / compute do, for callers that
 * reduce a whole gradient set per step (the reference's DistributedOptimizer
 * issues one MPIAllreduce per gradient, __init__.py:195-205, and so does this
 * call: every tensor is its own node, negotiated and validated under its own
 * node name, and the coordinator's tensor fusion groups them as it would
 * group separately submitted ones). Tensor j has element type dtypes[j]
 * (mpic_dtype) and ndims[j] dimensions, taken in order from `dims` (all
 * tensors' dimensions back to back); inputs[j] is its device memory and
 * outputs[j] device memory of the same size for the result (the caller
 * supplies it where a single node asks its allocator). divisor as
 * mpic_context_set_divisor, for every node. contexts[j] receives node j's
 * context: wait / message / destroy as for any other. */
int mpic_allreduce_batch(mpic_world* world, int rank, int k, const char* const* node_names, const int* dtypes,
                         const int* ndims, const int64_t* dims, const void* const* inputs, void* const* outputs,
                         int divisor, mpic_context** contexts);
/* Waits for every context of the array (NULL entries are skipped); codes[j],
 * when given, receives node j's status code. With destroy_ok, contexts that
 * ended OK are destroyed and their entries set to NULL, so that what is left
 * are the failed ones, whose message can still be read. Returns the first
 * status that is not OK. */
int mpic_context_wait_batch(mpic_context** contexts, int k, int destroy_ok, int* codes);

/* The same k nodes built ONCE and run every step, the way a TensorFlow graph's
 * nodes are constructed once and executed by every session.run() (the
 * reference's MPIAllreduceOp objects live as long as the graph; only its
 * OpKernelContext is per step, mpi_ops.cc:1039-1117). Arguments as
 * mpic_allreduce_batch; the tensors' memory must stay where it is for the life
 * of the batch. mpic_batch_submit files one MPIAllreduce request per node, as
 * k executions of the kernels would (FAILED_PRECONDITION while the previous
 * submission is still running); mpic_batch_wait blocks until all of them have
 * finished, returns the first status that is not OK and fills codes[j] (when
 * given) with node j's; mpic_batch_message(batch, j) is node j's message
 * until the next submit. mpic_batch_destroy waits for a running submission
 * (mpic_batch_busy: 1 while one is running). Lifetime: a batch may be
 * destroyed before or after its world; once mpic_world_destroy has returned
 * (which fails whatever was still running), mpic_batch_submit answers
 * FAILED_PRECONDITION and only mpic_batch_wait / _message / _destroy remain
 * meaningful. The contexts handed out by mpic_allreduce_batch follow the rule
 * of single contexts: wait for them, or destroy the world first. */
typedef struct mpic_batch mpic_batch;
int mpic_batch_create(mpic_world* world, int rank, int k, const char* const* node_names, const int* dtypes,
                      const int* ndims, const int64_t* dims, const void* const* inputs, void* const* outputs,
                      int divisor, mpic_batch** batch);
int mpic_batch_size(const mpic_batch* batch);
int mpic_batch_submit(mpic_batch* batch);
int mpic_batch_wait(mpic_batch* batch, int* codes);
const char* mpic_batch_message(const mpic_batch* batch, int index);
int mpic_batch_busy(mpic_batch* batch);
int mpic_batch_destroy(mpic_batch* batch);

/* ---- the ring driver, callable without the op layer ------------------------
 * RingAllreduce (ring.h:136-228) for rank r of n whose incoming segments are
 * already in device memory. `flags`: bit 0 = batched, bit 1 = fuse the
 * in->out copy, bits 8-30 = divisor (0: none; see mpic_context_set_divisor).
 * Asynchronous on `stream`. `dtype` is an mpic_dtype.
 * The calls only enqueue kernels, so any number of them can be recorded
 * between ring_graph_begin_capture and ring_graph_end_capture (ring_abi.h)
 * and replayed with ring_graph_launch: for launch-bound tensors (up to a few
 * MiB) a graph of 8 or more steps costs half of what the same steps cost
 * launched one by one; a graph of a single step costs more than the step.
 *
 * WHO DIVIDES, when a divisor is given, differs between the entry points, so
 * the same staged traffic must not be fed to both kinds:
 *   - mpic_ring_allreduce_prestaged and mpic_ring_allreduce_direct_prestaged:
 *     THE OWNER DIVIDES. The rank divides only the segment it owns (in the
 *     accumulate / fold that completes it) and copies ag_segments verbatim:
 *     ag_segments must hold quotients, what peers that do the same send round.
 *   - mpic_ring_allreduce_fused_prestaged: THE RECEIVER DIVIDES. Every finished
 *     segment, ag_segments included, is divided on its way into the tensors:
 *     ag_segments must hold undivided sums, and `wire` is left undivided (it is
 *     what a ring of such ranks sends on). */
int mpic_ring_allreduce_prestaged(int n, int r, int dtype, const void* input, void* output,
                                  size_t count, const void* const* rs_segments,
                                  const void* const* ag_segments, void* stream, int flags);
/* The same allreduce where every rank's copy of a segment can be addressed at
 * once (peers push into staging slots over their own links instead of passing
 * partial sums round the ring): rank r owns segment s = (r+1) mod n;
 * peer_segments[k], k = 0..n-2, is rank (s+k) mod n's copy of segment s, and
 * they are folded with the rank's own copy in ring order, one pass
 * (ring_fold_rows), into output[s]; ag_segments[i] is the finished segment
 * (r-i) mod n. The output is bit-identical to mpic_ring_allreduce_prestaged
 * fed with the ring's traffic. `flags`: bit 0 = fold and copies in one launch
 * (they write disjoint segments), bits 8-30 = divisor. At most 256 ranks (the
 * copies one fold launch can address); more is refused with INVALID_ARGUMENT.
 * No counterpart in the reference. */
int mpic_ring_allreduce_direct_prestaged(int n, int r, int dtype, const void* input, void* output,
                                         size_t count, const void* const* peer_segments,
                                         const void* const* ag_segments, void* stream, int flags);
/* A fused (tensor-fusion) allreduce for rank r without pack and unpack passes.
 * `plan` is a ring_fusion_plan (ring_abi.h) over the rank's tensors; the packed
 * buffer exists only as `wire` (plan-elements long, device memory), where the
 * sums a ring sends on are left. rs_segments / ag_segments as for
 * mpic_ring_allreduce_prestaged, on the packed layout. Two launches: the
 * reduce-scatter's accumulates read their local operand straight from the
 * tensors (the segment that is only sent is packed alongside), and every
 * finished segment goes straight into the tensors, divided when bits 8-30 of
 * `flags` hold a divisor. Each tensor ends up exactly as pack, ring, unpack
 * (and tf.div) would leave it. With bit 2 of `flags` (the direct form)
 * rs_segments[k] is rank (r+1+k) mod n's raw copy of the segment this rank
 * owns, in the packed layout: the rank packs its own copy of that segment into
 * `wire`, folds the n copies there in ring order and scatters the finished
 * segments (3 launches). No counterpart in the reference. */
struct ring_fusion_plan;
int mpic_ring_allreduce_fused_prestaged(const struct ring_fusion_plan* plan, int n, int r, void* wire,
                                        const void* const* rs_segments, const void* const* ag_segments,
                                        void* stream, int flags);
/* RingAllgather (ring.h:236-301) for rank r: rows[k] = rank k's first
 * dimension, segments[i] = what arrives at step i. */
int mpic_ring_allgather_prestaged(int n, int r, int dtype, const void* input, const size_t* rows,
                                  size_t elems_per_row, void* output,
                                  const void* const* segments, void* stream, int flags);
/* All n ranks resident on this GPU: inputs[k] / outputs[k] are rank k's
 * tensors; a neighbour's buffer is read in place of a transfer. `flags` bit 2:
 * the direct form: every segment folded by its owner in ring order and the
 * result stored into every rank's output by the same pass, ONE launch for the
 * whole allreduce (up to 128 ranks; from 129 to 256 the fold and the copies of
 * the finished segments are two launches); for the allgather, every slice
 * copied from its owner's input into every output in one launch. inputs[k] may
 * be outputs[k] (an allreduce in place). An allreduce of more than 256 ranks
 * runs the lockstep ring whatever bit 2 says (a fold launch addresses at most
 * 256 pointers). */
int mpic_ring_allreduce_all_ranks(int n, int dtype, const void* const* inputs,
                                  void* const* outputs, size_t count, void* stream, int flags);
int mpic_ring_allgather_all_ranks(int n, int dtype, const void* const* inputs, const size_t* rows,
                                  size_t elems_per_row, void* const* outputs, void* stream, int flags);
/* ---- the ring over a real transport ------------------------------------------
 * The reference's loops exchange segments with MPI_Irecv / MPI_Send / MPI_Wait
 * (reduce-scatter, ring.h:189-200) and MPI_Sendrecv (allgather, ring.h:221-224,
 * 291-295) on tag TAG_TENSOR (ring.h:19). A transport supplies those calls for
 * DEVICE buffers (GPU-aware MPI, a peer-to-peer copy engine, ...): each returns
 * 0 on success, and all are host-blocking in MPI's sense, i.e. when `send`
 * returns the buffer may be reused and when `wait` returns the data is in
 * `buf`, visible to work enqueued on any stream afterwards. MPI_Sendrecv is
 * irecv + send + wait. `wait` consumes the request whether it succeeds or not.
 * `cancel` (MPI_Cancel + MPI_Request_free; may be NULL) abandons a request that
 * will not be waited for: when a collective ends early with an error the
 * driver cancels what it had posted, and after the call the transport must no
 * longer write to that receive's buffer. */
typedef struct mpic_transport {
  void* user;
  int (*irecv)(void* user, void* buf, size_t bytes, int source, int tag, void** request);
  int (*send)(void* user, const void* buf, size_t bytes, int dest, int tag);
  int (*wait)(void* user, void* request);
  int (*cancel)(void* user, void* request);
} mpic_transport;

/* RingAllreduce (ring.h:136-228) for rank r of n over `transport`. `temp` is
 * the reference's temp tensor (mpi_ops.cc:1073-1077): device memory for
 * temp_elements elements, at least ring_temp_elements(count, n). `flags`:
 * bits 4-7 = chunks-1 (0: every segment travels whole, the reference's
 * structure, with the stream synchronised before each send as ring.cu.cc:69
 * does); with 2..16 chunks a segment travels in pieces, the accumulate of a
 * piece is enqueued as soon as it has arrived and a piece is forwarded as soon
 * as ITS accumulate has finished, so transfers overlap the accumulates of the
 * other pieces. When temp_elements holds two segments the pieces of successive
 * steps alternate between the halves (a receive is posted without waiting for
 * the previous step's accumulates). Bits 8-30 = divisor
 * (mpic_context_set_divisor). The per-element additions and their order are
 * those of the reference for any chunk count. Blocks the calling thread; the
 * output is complete on return. */
int mpic_ring_allreduce_transport(int n, int r, int dtype, const void* input, void* output, void* temp,
                                  size_t temp_elements, size_t count, const mpic_transport* transport,
                                  void* stream, int flags);
/* RingAllgather (ring.h:236-301) over `transport`; `flags` as above (chunks,
 * divisor: the own slice is divided before it is first sent). */
int mpic_ring_allgather_transport(int n, int r, int dtype, const void* input, const size_t* rows,
                                  size_t elems_per_row, void* output, const mpic_transport* transport,
                                  void* stream, int flags);

/* A transport between the virtual ranks of ONE process, each driven by its own
 * thread, all on the current GPU: a send blocks until the matching receive was
 * posted, then copies device to device. Messages between one pair of ranks on
 * one tag match in order, as MPI's do. Every blocking call gives up after
 * timeout_seconds (a peer that died) and returns non-zero. It stands in for
 * xGMI / MPI where there is one GPU; it is not a fast path. */
typedef struct mpic_loopback mpic_loopback;
int mpic_loopback_create(int n, double timeout_seconds, mpic_loopback** loopback);
int mpic_loopback_destroy(mpic_loopback* loopback);
/* Fills *transport with rank `rank`'s endpoint (owned by the loopback). Call on
 * the thread that will drive the rank, with the GPU current. */
int mpic_loopback_endpoint(mpic_loopback* loopback, int rank, mpic_transport* transport);

/* Message of the last failing mpic_ring_* call on this thread. */
const char* mpic_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* MPI_COLLECTIVES_H_ */
