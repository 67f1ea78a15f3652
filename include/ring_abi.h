/*
 * ring_abi.h — C ABI of the MI355X (gfx950) per-rank data path of the ring
 * allreduce / allgather of tensorflow/contrib/mpi_collectives.
 *
 * This is the seam the reference keeps inside its plugin between the ring
 * algorithm (ring.h) and the device primitives (ring.cc / ring.cu.cc):
 *
 *     template <typename Device>
 *     void CopyTensorData(void* dst, void* src, size_t size);        ring.h:44-45
 *     template <typename Device, typename T>
 *     void AccumulateTensorData(T* dst, T* src, size_t size);        ring.h:50-51
 *     cudaStream_t CudaStreamForMPI();                               ring.h:55-57
 *
 * restated as plain C: pointers, sizes, an opaque stream handle, an int
 * status. Differences from the reference seam, all deliberate:
 *   - every device entry point is ASYNCHRONOUS on the stream it is given; the
 *     caller synchronises (the reference blocks the host after every call,
 *     ring.cu.cc:41-45, :60-66);
 *   - every entry point returns a status (the reference returns void and
 *     drops CUDA errors);
 *   - a whole phase of the ring (all n-1 accumulates, all n-1 allgather
 *     copies) can be issued as ONE launch from a step table, because the
 *     steps of one rank write disjoint segments (ring.h:183-205, :211-225);
 *   - nothing allocates device memory unless its name says "create" (host
 *     memory: a table of more than 64 rows takes a heap buffer for the call).
 *
 * Conventions: `count` is in elements, `bytes` in bytes; a count of 0 with
 * null pointers is valid and does nothing (an empty tensor reaches the
 * reference's primitives the same way); pointers are device pointers unless
 * the parameter is documented as host; element offsets may be any multiple of
 * the element size (ragged segments break 16-byte alignment and the kernels
 * handle it). `stream` is a hipStream_t passed as void* (NULL = the default
 * stream). One thread per stream.
 */
#ifndef RING_ABI_H_
#define RING_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RING_ABI_VERSION 1

/* Element types: exactly the three the reference registers and dispatches on
 * (mpi_ops.cc:1120 `Attr("T: {int32, int64, float32}")`, ring.cu.cc:14-20,
 * mpi_ops.cc:478-508). */
enum ring_dtype { RING_F32 = 0, RING_I32 = 1, RING_I64 = 2 };

/* Status codes. RING_ERR_HIP: ring_last_hip_error() has the hipError_t. */
enum ring_status {
  RING_OK = 0,
  RING_ERR_DTYPE = 1,    /* not one of ring_dtype ("Invalid tensor type", mpi_ops.cc:844) */
  RING_ERR_ARGUMENT = 2, /* null pointer with a non-zero size, n < 1, rank out of range ... */
  RING_ERR_HIP = 3,      /* a HIP runtime call failed */
  RING_ERR_NO_DEVICE = 4, /* no usable GPU */
  RING_ERR_LIMIT = 5      /* beyond a stated fixed capacity (ring_fusion_run_static) */
};

int ring_abi_version(void);
const char* ring_status_string(int status);
/* hipError_t of the most recent failing HIP call on this thread (0 if none). */
int ring_last_hip_error(void);
/* sizeof(T) for a ring_dtype, 0 if the code is not one. */
size_t ring_dtype_size(int dtype);

/* Launch-shape knobs for measurement runs (process-wide; not needed for
 * normal use; may be set from one thread while others launch: every launch
 * reads the options once, at entry): "unroll" = 16-byte vectors per lane per tile (2, 4, 8),
 * "blocks_per_cu" = 0 for one workgroup per tile, k > 0 for a persistent grid
 * of CUs x k workgroups that stride over the tiles. Cache policy per kind of
 * launch: "nontemporal_copy" (ring_copy_bytes), "nontemporal_accumulate"
 * (accumulates, reduce-scatter tables, row tables, scale),
 * "nontemporal_allgather" (copy tables), "nontemporal_pack",
 * "nontemporal_unpack", "nontemporal_fold", "nontemporal_fold_all" (a fold
 * stored to every rank), "nontemporal_broadcast" (copy
 * rows of one call that share a source); value bit 0 = non-temporal stores,
 * bit 1 = non-temporal loads, -1 = the default: 3, except ordinary stores
 * where the next kernel reads the output (copy, pack, fold), ordinary loads
 * for a source several rows share (broadcast), and loads by size for the copy.
 * "nontemporal" sets all eight. "paced_copy": the copies of an allgather
 * phase as one read phase and one write phase (every workgroup waits for all
 * its loads, then keeps one store in flight per wave): 1 always, 0 never,
 * -1 (default) when every tile of the launch is on the chip at the same time
 * (between 2 and 7 tiles of 32 KiB per CU). "phased_copy": the same copies
 * with the whole payload of the launch held in registers between the two
 * phases (one or two workgroups per CU, up to 8 rows and 112 MiB): 1 whenever
 * the launch fits, 0 never, -1 (default) above 56 MiB per side, and from
 * 31 MiB when the paced tiles would not fill the chip's CUs evenly. The same
 * option governs the unpack of a fused buffer (ring_fusion_unpack,
 * _unpack_scaled and the unpack of ring_fusion_run_static), which runs in that
 * form by default between 1 and 112 MiB when the set has at most 1024
 * non-empty tensors and the divisor, if any, is a power of two (float32: any
 * divisor up to 64 MiB).
 * "dry_launch" = 1 makes the step-table / copy /
 * accumulate kernels return at entry: what is then timed is what a launch of
 * that grid costs by itself. "flat_grid" = 1 gives rows of equal length the
 * 1-D grid of unequal rows (a workgroup finds its row by counting) instead of
 * the 2-D grid (tiles, rows). No counterpart in the reference, whose launch
 * shape is the constant <<<32, 256>>> (ring.cu.cc:64). */
int ring_set_option(const char* name, int value);

/* Timing of single launches, for benchmarks (no counterpart in the
 * reference): events created here, and ring_time_next_launch(start, stop)
 * makes the NEXT step-table / copy / accumulate kernel this thread launches
 * record its own begin and end into them (the events travel in the dispatch,
 * so their difference is the kernel's execution time and nothing else). Read
 * with ring_event_elapsed_us after the stream has been synchronised. Each
 * call arms one more launch, in order, up to 8 ahead (RING_ERR_LIMIT beyond):
 * a call that needs several launches is timed launch by launch by arming as
 * many pairs before it. Two null events disarm whatever is still queued.
 * A timed dispatch signals its own completion, so it ends only when its
 * stores have drained, and one that follows an untimed dispatch also waits
 * for that one's: durations agree with a profiler's kernel trace (where
 * every dispatch is timed) when the launch before is timed as well. */
int ring_event_create(void** event);
int ring_event_destroy(void* event);
int ring_event_elapsed_us(void* start, void* stop, double* us);
int ring_time_next_launch(void* start_event, void* stop_event);
/* Ordering between the stream and the host at a finer grain than
 * ring_stream_synchronize: record marks the work enqueued on `stream` so far,
 * synchronize blocks the host until that work has finished. A ring driver
 * that hands a freshly accumulated chunk to a host-driven transport (the
 * reference synchronises the whole stream after every kernel, ring.cu.cc:69)
 * waits for that chunk only. */
int ring_event_record(void* event, void* stream);
int ring_event_synchronize(void* event);
/* Ordering between two streams without the host: work enqueued on `stream`
 * after this call starts only when the work `event` marked (ring_event_record
 * on the producer's stream, or any hipEvent_t the embedding framework
 * recorded there) has finished. This is how a producer hands a tensor to the
 * ring's non-blocking stream: the reference defers its enqueue with a host
 * callback on the producer's stream, stream->ThenDoHostCallback
 * (mpi_ops.cc:1099-1105), so that the executor thread never blocks; here the
 * dependency stays on the device and no thread blocks at all. */
int ring_stream_wait_event(void* stream, void* event);

/* HIP graphs, for steps that are bound by launches rather than bytes (a small
 * tensor's allreduce is 2-3 launches of 4-5 us each whatever it moves): what
 * is enqueued on `stream` between begin and end is recorded instead of run,
 * end returns an executable graph, and launch replays it as one submission.
 * A replay has a fixed cost of its own (about 12 us), so it pays from about
 * four steps per graph: the allreduces of a whole gradient set, say. The
 * recorded launches carry their kernel arguments, pointers included, so a
 * graph is only good for the buffers it was recorded with. `stream` must not
 * be the null stream. No counterpart in the reference. */
int ring_graph_begin_capture(void* stream);
int ring_graph_end_capture(void* stream, void** graph_exec);
int ring_graph_launch(void* graph_exec, void* stream);
int ring_graph_destroy(void* graph_exec);

/* ---- host-side tables (no GPU involved) ---------------------------------- */

/* Segment split of a `count`-element tensor over n ranks — ring.h:150-166:
 * count/n each, the first count%n segments one more, starts = exclusive
 * prefix sum. sizes/starts: host arrays of n. */
int ring_segment_table(size_t count, int n, size_t* sizes, size_t* starts);

/* Elements of the receive buffer an allreduce needs — mpi_ops.cc:1073-1077:
 * ceil(count / n). */
size_t ring_temp_elements(size_t count, int n);

/* Allgather segment starts, in elements — ring.h:255-259. rows[k] is rank k's
 * first dimension; starts: host array of n. RING_ERR_ARGUMENT when the gathered
 * tensor's element count does not fit size_t (the reference's table wraps). */
int ring_allgather_table(const size_t* rows, int n, size_t elems_per_row,
                         size_t* starts);

/* Which segments rank r sends / receives at step i (0 <= i < n-1):
 *   reduce-scatter  send (r-i),   recv (r-i-1)    ring.h:184-185
 *   allreduce's allgather  send (r-i+1), recv (r-i)   ring.h:212-213
 *   standalone allgather   send (r-i),   recv (r-i-1) ring.h:280-281
 * all modulo n. Neighbours are fixed: receive from r-1, send to r+1
 * (ring.h:171-174). */
enum ring_phase { RING_PHASE_REDUCE_SCATTER = 0, RING_PHASE_ALLGATHER = 1, RING_PHASE_GATHER = 2 };
int ring_schedule(int phase, int n, int r, int step, int* send_seg, int* recv_seg);

/* The GPU of the calling thread, for host code that includes no HIP header:
 * the reference remembers the device MPI was initialised on (cudaGetDevice,
 * mpi_ops.cc:805-809) and makes it current on its background thread before it
 * creates the stream there (cudaSetDevice, mpi_ops.cc:582). */
int ring_get_device(int* device);
int ring_set_device(int device);

/* ---- the dedicated stream — CudaStreamForMPI(), mpi_ops.cc:213-230, 582-583,
 * 872-876: one non-default stream for all ring copies and accumulates, so a
 * wait on it never waits for unrelated compute. Default priority. The stream
 * is non-blocking: work on the null stream (a plain hipMemset, say) is NOT
 * ordered with it, so whatever prepares a buffer for these calls runs on the
 * same stream or is synchronised first. ---------------------------------------- */
int ring_stream_create(void** stream);
int ring_stream_destroy(void* stream);
int ring_stream_synchronize(void* stream);

/* ---- device primitives ---------------------------------------------------- */

/* CopyTensorData<GPUDevice> — ring.cu.cc:41-45 (call sites ring.h:146-148,
 * 263-266). Device-to-device byte copy by a hand-written kernel; dst and src
 * must not overlap. */
int ring_copy_bytes(void* dst, const void* src, size_t bytes, void* stream);

/* AccumulateTensorData<GPUDevice,T> + elemwise_accum<T> — ring.cu.cc:48-69
 * (call site ring.h:203-204): dst[i] += src[i], one IEEE binary32 add (or one
 * wrapping integer add) per element. dst and src must not overlap. */
int ring_accumulate_f32(float* dst, const float* src, size_t count, void* stream);
int ring_accumulate_i32(int32_t* dst, const int32_t* src, size_t count, void* stream);
int ring_accumulate_i64(int64_t* dst, const int64_t* src, size_t count, void* stream);
int ring_accumulate(int dtype, void* dst, const void* src, size_t count, void* stream);

/* The divide of allreduce(average=True) — __init__.py:160-164
 * `tf.div(summed, cast(size(), dtype))`: in place data[i] = data[i] / divisor,
 * true (correctly rounded) division for float32, floor division for the
 * integer types (math_ops.py:982-985). divisor >= 1. */
int ring_scale(int dtype, void* data, size_t count, int divisor, void* stream);

/* One row of a step table: the segment received at one ring step. `src` is
 * where the incoming segment lies in device memory (the reference's `temp`
 * after MPI_Wait, ring.h:189-200, or the neighbour's send buffer itself when
 * it is directly addressable); `dst_offset` is segment_starts[recv_seg]. */
typedef struct ring_step {
  uint64_t dst_offset; /* elements from the start of `buffer` */
  const void* src;     /* device pointer, any multiple of the element size */
  uint64_t count;      /* elements; 0 is allowed */
} ring_step;

/* All the accumulates of a rank's reduce-scatter (ring.h:183-205) in one
 * launch: for every row, buffer[dst_offset + i] += src[i]. `steps` is a HOST
 * array of n_steps rows whose destination ranges are pairwise disjoint and
 * disjoint from every src (true for the n-1 steps of one rank). Any n_steps
 * >= 0; tables longer than one launch can carry are split internally. */
int ring_reduce_scatter_steps(void* buffer, const ring_step* steps, int n_steps,
                              int dtype, void* stream);

/* The same reduce-scatter with the in->out copy of ring.h:146-148 folded in:
 * for every row, buffer[dst_offset + i] = input[dst_offset + i] + src[i].
 * `input` is the rank's unmodified tensor, `buffer` its output; the sum is the
 * same single add, so results are bit-identical to copy-then-accumulate while
 * the accumulated segments are never copied (12 instead of 20 bytes moved
 * per element). The one segment no step touches (segment r) is not written;
 * the caller copies it if it needs it before the allgather phase fills it.
 * input == buffer degenerates to ring_reduce_scatter_steps. */
int ring_reduce_scatter_steps_from(const void* input, void* buffer,
                                   const ring_step* steps, int n_steps,
                                   int dtype, void* stream);

/* All the receives of a rank's allgather phase (ring.h:211-225, and
 * ring.h:279-298 for the standalone allgather) in one launch: for every row,
 * buffer[dst_offset + i] = src[i]. Same table rules. */
int ring_allgather_steps(void* buffer, const ring_step* steps, int n_steps,
                         int dtype, void* stream);

/* The general form the step tables reduce to, for callers whose rows live in
 * different buffers (all ranks of a virtual ring advancing one step in a
 * single launch): for every row, dst[i] = a[i] when b is NULL, else
 * dst[i] = b[i] + a[i]. b may be dst itself (in-place accumulate); otherwise
 * no operand of a row may overlap a destination of the same call. `rows` is a
 * HOST array. */
typedef struct ring_row {
  void* dst;
  const void* a;
  const void* b;
  uint64_t count; /* elements */
} ring_row;
int ring_apply_rows(const ring_row* rows, int n_rows, int dtype, void* stream);
/* The same launch with the divide of allreduce(average=True) folded in
 * (the reference divides in a separate graph op after the collective,
 * __init__.py:160-164 `tf.div(summed_tensor, size())`): rows with divide[k] != 0
 * (all rows when `divide` is NULL) store (b[i] + a[i]) / divisor, or
 * a[i] / divisor without b, with ring_scale's division (true division for
 * float32, floor division for the integers) applied to the already rounded
 * sum, so the result equals the two passes done one after the other. A ring
 * divides once, where a segment's sum becomes complete: at the last
 * reduce-scatter step of the rank that owns it. divisor 0 = ring_apply_rows.
 * `rows` and `divide` are HOST arrays. */
int ring_apply_rows_avg(const ring_row* rows, int n_rows, const unsigned char* divide, int divisor,
                        int dtype, void* stream);

/* Which form a launch takes, as a query that needs no GPU (no counterpart in
 * the reference, whose one launch shape is the constant <<<32, 256>>>,
 * ring.cu.cc:64). The copies of an allgather phase and the unpack of a fused
 * buffer run in one of several forms, chosen from the shape of the launch and
 * the number of compute units; every form gives the same bytes, so only this
 * query (and a profiler) tells which one a shape takes, and a test can pin
 * the choice for the shapes that were measured.
 * ring_describe_rows_launch: `rows` as ring_apply_rows takes them (pointers
 * are looked at for their alignment only, never dereferenced), `role` the
 * entry point they come from: RING_ROLE_COPY (ring_copy_bytes),
 * RING_ROLE_ACCUMULATE (accumulates, reduce-scatter tables, row tables) or
 * RING_ROLE_ALLGATHER (ring_allgather_steps: the only one with a choice).
 * ring_describe_unpack_launch: a fused buffer of `total_elements` elements in
 * `n_tensors` non-empty tensors, unpacked with `divisor` (0: no divide).
 * `cus`: compute units of the GPU (256 on an MI355X). Both answer for the
 * options currently set (ring_set_option). */
enum ring_form {
  RING_FORM_TILES = 0,       /* one workgroup per tile of 16 KiB */
  RING_FORM_PACED = 1,       /* tiles of 32 KiB: all loads, one wait, then one store in flight per wave */
  RING_FORM_REGISTERS_2 = 2, /* the launch's payload in registers, two workgroups per CU */
  RING_FORM_REGISTERS_1 = 3  /* the same, one workgroup per CU (one wave per SIMD, 112 vectors per lane) */
};
enum ring_role { RING_ROLE_COPY = 0, RING_ROLE_ACCUMULATE = 1, RING_ROLE_ALLGATHER = 2 };
int ring_describe_rows_launch(const ring_row* rows, int n_rows, int dtype, int role, int cus, int* form);
int ring_describe_unpack_launch(uint64_t total_elements, int n_tensors, int dtype, int divisor, int cus,
                                int* form);

/* Measurement only (no counterpart in the reference): ONE direction of a copy
 * launch in the tile shape and grid of the step-table kernel. mode 0: every
 * row's `a` is read (non-temporal loads) and nothing is written; mode 1:
 * every row's `dst` is written (non-temporal stores) and nothing is read;
 * modes 2 and 3: the same with the ordinary cache policy. Up to 8 rows;
 * the pointer used must be 16-byte aligned; counts are rounded down to whole
 * 16-byte vectors. A copy runs no faster than its two directions one after
 * the other, so these two launches give the floor of a copy of that shape.
 * Timed like any other launch (ring_time_next_launch). */
int ring_probe_stream(const ring_row* rows, int n_rows, int dtype, int mode, void* stream);

/* A segment reduced in one pass. After its n-1 reduce-scatter steps the ring
 * holds in segment s the left fold over the ranks in ring order,
 *   acc = x_s; acc = x_{s+1} + acc; ...; acc = x_{s+n-1} + acc
 * (ring.h:183-205: at step i rank r adds what it received, the running sum of
 * segment (r-i-1), into its own copy). Where every rank's copy of the segment
 * is addressable at once, the owner computes that fold directly: for every
 * row, dst[i] = srcs[m-1][i] + (... + (srcs[1][i] + srcs[0][i])), the same
 * additions in the same order, with m reads and one write per element instead
 * of 3(m-1) accesses. divisor > 0: the fold is divided as ring_scale divides
 * (the average) before it is stored. dst may be one of the row's own sources.
 * `rows` and each `srcs` are HOST arrays; every row has m sources, 1 <= m <=
 * 256. No counterpart in the reference. */
typedef struct ring_fold_row {
  void* dst;
  const void* const* srcs; /* m device pointers, in fold order */
  uint64_t count;          /* elements */
} ring_fold_row;
int ring_fold_rows(const ring_fold_row* rows, int n_rows, int m, int divisor, int dtype, void* stream);
/* The fold rows and, in the SAME launch, plain copy rows (b must be NULL; never
 * divided): a rank's whole direct step, its own segment folded from the
 * pushed copies while the other ranks' finished segments are copied in. The
 * two kinds of row write disjoint memory, so one launch saves the start-up and
 * drain of a second. */
int ring_fold_and_copy_rows(const ring_fold_row* fold_rows, int n_fold, int m, int divisor,
                            const ring_row* copy_rows, int n_copy, int dtype, void* stream);
/* The fold of a row stored to n_dst destinations at once: where the ranks of a
 * ring share a GPU (or an owner can write into its peers' memory), the owner
 * of a segment hands the finished segment to every rank in the pass that
 * reduces it, instead of each rank copying it from the owner afterwards
 * (ring.h:211-225 moves the same values round the ring in n-1 steps). n reads
 * and n_dst writes per element, one launch for a whole allreduce of all
 * ranks. dsts[0] is the destination whose alignment the vector stores follow;
 * the others need only be element-aligned. Any destination may be one of the
 * row's own sources (an allreduce in place): a lane reads every source of its
 * elements before it stores them. m + n_dst - 1 <= 256. `rows`, `dsts` and
 * `srcs` are HOST arrays. No counterpart in the reference. */
typedef struct ring_fold_to_all_row {
  void* const* dsts;       /* n_dst device pointers */
  const void* const* srcs; /* m device pointers, in fold order */
  uint64_t count;          /* elements */
} ring_fold_to_all_row;
int ring_fold_to_all_rows(const ring_fold_to_all_row* rows, int n_rows, int m, int n_dst, int divisor, int dtype,
                          void* stream);

/* ---- tensor fusion (no counterpart in the reference, which issues one
 * MPIAllreduce per gradient, __init__.py:195-205): k tensors are packed back
 * to back, in order, without padding, into one buffer that is ring-reduced
 * as a single tensor and unpacked again. -------------------------------- */

typedef struct ring_fusion_plan ring_fusion_plan;

/* Builds the device-resident offset table for k tensors (`tensors[j]` device
 * pointer to counts[j] elements; both HOST arrays). Allocates a few KiB of
 * device memory owned by the plan and copies the table synchronously. Tensor
 * pointers must stay valid while the plan is used. */
int ring_fusion_plan_create(const void* const* tensors, const size_t* counts,
                            int k, int dtype, ring_fusion_plan** plan);
int ring_fusion_plan_destroy(ring_fusion_plan* plan);
/* The plan's ring_dtype (-1 for a null plan). */
int ring_fusion_plan_dtype(const ring_fusion_plan* plan);
/* Total elements of the fused buffer (sum of counts). */
size_t ring_fusion_plan_elements(const ring_fusion_plan* plan);
/* fused[offset_j + i] = tensors[j][i] for all j. `fused` must be 16-byte
 * aligned (tensors need only element alignment). */
int ring_fusion_pack(const ring_fusion_plan* plan, void* fused, void* stream);
/* tensors[j][i] = fused[offset_j + i] for all j. */
int ring_fusion_unpack(const ring_fusion_plan* plan, const void* fused, void* stream);
/* tensors[j][i] = fused[offset_j + i] / divisor, with ring_scale's division
 * (the average of a fused allreduce folded into the unpack). divisor >= 1. */
int ring_fusion_unpack_scaled(const ring_fusion_plan* plan, const void* fused, int divisor,
                              void* stream);

/* Pack / unpack WITHOUT a plan and without any allocation. No counterpart in
 * the reference; for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * unpack == 0: fused[offset_j + i] = tensors[j][i] (divisor must be 0), as
 * ring_fusion_pack; unpack != 0: tensors[j][i] = fused[offset_j + i], divided
 * by divisor when divisor >= 1, as ring_fusion_unpack[_scaled]. `tensors` and
 * `counts` are HOST arrays of k entries, read before the call returns. The
 * offset table a plan keeps in an allocation of its own is built, by small
 * kernels on `stream` ahead of the pack / unpack kernel, in a static device
 * array of 1,064,968 bytes that every GPU the library runs on holds until the
 * process ends. Limits: 1024 non-empty tensors and 268,435,456 four-byte
 * (134,217,728 eight-byte) elements per call, beyond which the call returns
 * RING_ERR_LIMIT and launches nothing. All calls on one GPU share that GPU's
 * array. Calls on the same stream are ordered by it; a call on another stream
 * than the call before it on that GPU makes its stream wait, on the device,
 * for an event recorded behind that call's kernels, so eager calls from
 * several streams (one per rank, say) are safe, one after the other. A call
 * on a stream that is being captured neither waits nor records (a wait would
 * pull the other stream into the graph, and replays run whenever their owner
 * launches them): whoever captures a call orders its replays against calls on
 * other streams. Calls no hipMalloc / hipFree / hipMemcpy; the first call on
 * a device looks up the array's address and creates the one event. */
int ring_fusion_run_static(int unpack, const void* const* tensors, const size_t* counts, int k, int dtype,
                           void* fused, int divisor, void* stream);

/* Fusion without passes of its own. A span is `count` elements of the plan's
 * fused element space starting at `begin` (a ring segment of the packed
 * buffer). Gather: out[i] = tensor_element(begin + i) + incoming[i], or a plain
 * pack of the span when incoming is NULL: the first accumulate of a segment
 * takes its local operand straight from the tensors and leaves the sum in the
 * wire buffer the next rank is sent from. Scatter: tensor_element(begin + i) =
 * incoming[i], divided by divisor when divisor > 0: a finished segment goes
 * straight to the tensors. Elements outside the spans are not touched. Spans
 * must be sorted by `begin` and disjoint; `spans` is a HOST array. Together
 * the two calls do what pack, n-1 accumulates, and unpack do, minus one read
 * and one write of the whole set. `incoming` and `out` need only be aligned
 * to an element. The kernels align their stores to the tensors; a wave's
 * loads of `incoming` cover whole 128-byte lines as well when the arrival is
 * shifted against the fused space by a multiple of 128 bytes, i.e. when
 * (address of incoming - begin * element size) is a multiple of 128, as it is
 * for a segment received in place at wire + begin in a 128-byte aligned wire
 * buffer (where ring.h:211-225 receives it). A slot at the start of a fresh
 * allocation instead costs a ragged segment 3.6 % more bytes fetched (every
 * 1 KiB a wave loads straddles one more line) and 1.5 % of the launch. */
typedef struct ring_fusion_span {
  uint64_t begin;       /* first element in the fused space */
  uint64_t count;       /* elements */
  const void* incoming; /* element 0 of the span's incoming data */
  void* out;            /* gather: element 0 of the span's destination; scatter: unused */
} ring_fusion_span;
int ring_fusion_gather(const ring_fusion_plan* plan, const ring_fusion_span* spans, int n_spans, void* stream);
/* The form (enum ring_form) ring_fusion_scatter takes for these spans on a GPU
 * of `cus` compute units, without a GPU. Finished segments that were received
 * in place lie in one buffer, each at its own offset (every `incoming` less
 * `begin` elements is the same 16-byte aligned address, and the spans, empty
 * ones aside, cover the fused space end to end): the scatter is then the
 * unpack of that buffer and takes the unpack's launch
 * (ring_describe_unpack_launch: in registers from 1 to 112 MiB). Segments in
 * slots of their own are scattered as tiles (RING_FORM_TILES). Same results
 * either way. */
int ring_describe_scatter_launch(const ring_fusion_plan* plan, const ring_fusion_span* spans, int n_spans,
                                 int divisor, int cus, int* form);
int ring_fusion_scatter(const ring_fusion_plan* plan, const ring_fusion_span* spans, int n_spans, int divisor,
                        void* stream);

/* The direct form of a fused allreduce for one rank, in one launch. The
 * rank's own ring segment is the `fold_count` elements of the fused space from
 * `fold_begin`: `staged[0..m)` are the peers' raw copies of it (packed layout,
 * element 0 = element fold_begin), listed in the ring's order for that
 * segment, and the rank's own copy, which comes last in that order, is read
 * from the plan's tensors. The fold `staged[0], staged[1] + ., ..., tensors + .`
 * is stored to `wire` (element 0 = element fold_begin: what the rank sends to
 * its peers, a sum) and, divided by `divisor` when that is > 0 (tf.div), into
 * the tensors. `finished` are the other segments, as ring_fusion_scatter takes
 * them (sorted, disjoint, none meeting the fold span; sums, divided on the way
 * into the tensors). Bit-identical to ring_fusion_gather of the owned segment,
 * ring_fold_rows over the m + 1 copies and ring_fusion_scatter of all
 * segments, which read and write the owned segment three times where this
 * reads and writes it once. m and n_finished at most 32 (RING_ERR_LIMIT
 * beyond). No counterpart in the reference (its ring passes partial sums
 * round, ring.h:183-205). */
int ring_fusion_fold_scatter(const ring_fusion_plan* plan, uint64_t fold_begin, uint64_t fold_count,
                             const void* const* staged, int m, void* wire, const ring_fusion_span* finished,
                             int n_finished, int divisor, void* stream);

/* The fused allreduce of n ranks that share the GPU, without a fused buffer:
 * in_plans[k] / out_plans[k] are plans over rank k's input and output tensors
 * (the same plan for an allreduce in place), all with the same element type
 * and the same tensor sizes in the same order, i.e. one fused element space.
 * One launch computes what pack, the ring over the packed buffers and unpack
 * compute: element e of the space lies in ring segment s of the packed layout
 * (ring_segment_table of the total), every rank's tensor receives the ring's
 * fold of the n values in the order s, s+1, ..., s+n-1 (mod n), divided by
 * `divisor` when it is > 0 (tf.div, as ring_fusion_unpack_scaled). Each
 * tensor's result is bit-identical to the reference ring applied to the packed
 * buffer; the tensors are read once and written once. 1 <= n <= 16
 * (RING_ERR_LIMIT beyond). `in_plans` and `out_plans` are HOST arrays. No
 * counterpart in the reference. */
int ring_fusion_allreduce_all(const ring_fusion_plan* const* in_plans, const ring_fusion_plan* const* out_plans, int n,
                              int divisor, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RING_ABI_H_ */
