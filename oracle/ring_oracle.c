/*
 * TEST INFRASTRUCTURE ONLY — see ring_oracle.h.
 *
 * CPU restatement of the reference ring allreduce / allgather
 * (tensorflow/contrib/mpi_collectives/ring.h, ring.cc). The product library
 * never links this file.
 *
 * What pins it (all exercised by the CPU test-suite):
 *   - segment tables: closed form and the known answers of the ragged case;
 *   - accumulate: numpy float32 / integer addition, element by element;
 *   - whole ring: an independent closed form (element of segment s is the
 *     left fold x_s, x_{s+1}, ... x_{s+n-1 mod n}) evaluated in numpy, the
 *     lockstep evaluator below, and the same per-rank code run over real MPI;
 *   - one rank on given incoming segments (the replay transport): what the
 *     threaded ring's taps recorded, replayed to each rank alone, must give
 *     that rank's output of the threaded ring;
 *   - the reference tests' own invariants: allreduce(x) == x*size exactly for
 *     size <= 3 (mpi_ops_test.py:92-112), rank-stamped allgather
 *     (mpi_ops_test.py:204-263), the 13-stage chained closed form
 *     (mpi_allreduce_test.py:96-105).
 */
#define _GNU_SOURCE
#include "ring_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

size_t oracle_dtype_size(int dtype) {
  switch (dtype) {
    case ORACLE_F32: return sizeof(float);
    case ORACLE_I32: return sizeof(int32_t);
    case ORACLE_I64: return sizeof(int64_t);
    default: return 0;
  }
}

/* ring.h:150-166 */
void oracle_segment_table(size_t count, int n, size_t* sizes, size_t* starts) {
  const size_t segment_size = count / (size_t)n;
  const size_t residual = count % (size_t)n;
  for (int i = 0; i < n; i++) sizes[i] = segment_size;
  for (size_t i = 0; i < residual; i++) sizes[i]++;
  starts[0] = 0;
  for (int i = 1; i < n; i++) starts[i] = starts[i - 1] + sizes[i - 1];
}

/* mpi_ops.cc:1073-1077 */
size_t oracle_temp_elements(size_t count, int n) {
  return (count + (size_t)n - 1) / (size_t)n;
}

/* ring.h:255-259 */
void oracle_allgather_table(const size_t* rows, int n, size_t elems_per_row,
                            size_t* starts) {
  starts[0] = 0;
  for (int i = 1; i < n; i++)
    starts[i] = starts[i - 1] + elems_per_row * rows[i - 1];
}

/* ring.cc:36-38 */
void oracle_copy(void* dst, const void* src, size_t bytes) {
  if (bytes) memcpy(dst, src, bytes);
}

/* ring.cc:41-50. Compiled without -ffast-math: one IEEE add per element. */
void oracle_accumulate_f32(float* dst, const float* src, size_t count) {
  for (size_t i = 0; i < count; i++) dst[i] += src[i];
}
void oracle_accumulate_i32(int32_t* dst, const int32_t* src, size_t count) {
  /* two's-complement wrap, as the hardware add the reference compiles to */
  for (size_t i = 0; i < count; i++)
    dst[i] = (int32_t)((uint32_t)dst[i] + (uint32_t)src[i]);
}
void oracle_accumulate_i64(int64_t* dst, const int64_t* src, size_t count) {
  for (size_t i = 0; i < count; i++)
    dst[i] = (int64_t)((uint64_t)dst[i] + (uint64_t)src[i]);
}
void oracle_accumulate(int dtype, void* dst, const void* src, size_t count) {
  switch (dtype) {
    case ORACLE_F32: oracle_accumulate_f32((float*)dst, (const float*)src, count); break;
    case ORACLE_I32: oracle_accumulate_i32((int32_t*)dst, (const int32_t*)src, count); break;
    case ORACLE_I64: oracle_accumulate_i64((int64_t*)dst, (const int64_t*)src, count); break;
    default: break;
  }
}

#define ORACLE_OK(call) do { int rc_ = (call); if (rc_) return rc_; } while (0)

/* ring.h:136-228 */
int oracle_ring_allreduce_rank(int n, int r, int dtype, const void* input,
                               void* temp, void* output, size_t count,
                               oracle_transport* tp, oracle_tap* tap) {
  const size_t esz = oracle_dtype_size(dtype);
  if (!esz || n < 1 || r < 0 || r >= n) return -1;
  char* buffer = (char*)output;

  /* ring.h:146-148: output starts as a copy of the input */
  oracle_copy(buffer, input, count * esz);

  /* ring.h:150-166 */
  size_t* sizes = (size_t*)malloc(sizeof(size_t) * 2 * (size_t)n);
  if (!sizes) return -2;
  size_t* starts = sizes + n;
  oracle_segment_table(count, n, sizes, starts);

  /* ring.h:171-174: receive from the left, send to the right */
  const int recv_from = ((r - 1) + n) % n;
  const int send_to = (r + 1) % n;
  int rc = 0;

  /* ring.h:183-205: reduce-scatter. Step i sends segment (r-i), receives
   * segment (r-i-1) into temp and adds it into the buffer. */
  for (int i = 0; i < n - 1 && !rc; i++) {
    const int send_seg = ((r - i) % n + n) % n;
    const int recv_seg = ((r - i - 1) % n + n) % n;
    rc = tp->irecv(tp->self, temp, sizes[recv_seg] * esz, recv_from);
    if (rc) break;
    rc = tp->send(tp->self, buffer + starts[send_seg] * esz,
                  sizes[send_seg] * esz, send_to);
    if (rc) break;
    rc = tp->wait(tp->self);
    if (rc) break;
    if (tap && tap->rs_recv)
      oracle_copy((char*)tap->rs_recv + (size_t)i * tap->slot_elems * esz, temp,
                  sizes[recv_seg] * esz);
    oracle_accumulate(dtype, buffer + starts[recv_seg] * esz, temp,
                      sizes[recv_seg]);
  }

  /* ring.h:207-225: allgather. Step i sends segment (r-i+1) and receives
   * segment (r-i) straight into its place in the buffer. */
  for (int i = 0; i < n - 1 && !rc; i++) {
    const int send_seg = ((r - i + 1) % n + n) % n;
    const int recv_seg = ((r - i) % n + n) % n;
    rc = tp->sendrecv(tp->self, buffer + starts[send_seg] * esz,
                      sizes[send_seg] * esz, send_to,
                      buffer + starts[recv_seg] * esz, sizes[recv_seg] * esz,
                      recv_from);
    if (rc) break;
    if (tap && tap->ag_recv)
      oracle_copy((char*)tap->ag_recv + (size_t)i * tap->slot_elems * esz,
                  buffer + starts[recv_seg] * esz, sizes[recv_seg] * esz);
  }
  free(sizes);
  return rc;
}

/* A transport that replays what one rank of a ring receives: the i-th receive
 * of the reduce-scatter delivers rs[i], the i-th of the allgather ag[i]; what
 * the rank sends goes nowhere. */
typedef struct replay_state {
  const void* const* rs;
  const void* const* ag;
  int next_rs, next_ag, steps;
} replay_state;

static int replay_irecv(void* self, void* buf, size_t bytes, int from) {
  replay_state* st = (replay_state*)self;
  (void)from;
  if (st->next_rs >= st->steps) return -3;
  oracle_copy(buf, st->rs[st->next_rs++], bytes);
  return 0;
}
static int replay_send(void* self, const void* buf, size_t bytes, int to) {
  (void)self; (void)buf; (void)bytes; (void)to;
  return 0;
}
static int replay_wait(void* self) {
  (void)self;
  return 0;
}
static int replay_sendrecv(void* self, const void* sbuf, size_t sbytes, int to,
                           void* rbuf, size_t rbytes, int from) {
  replay_state* st = (replay_state*)self;
  (void)sbuf; (void)sbytes; (void)to; (void)from;
  if (st->next_ag >= st->steps) return -3;
  oracle_copy(rbuf, st->ag[st->next_ag++], rbytes);
  return 0;
}

/* ring.h:136-228 for ONE rank whose incoming segments are given: the same
 * oracle_ring_allreduce_rank, over the replay transport. */
int oracle_ring_allreduce_rank_prestaged(int n, int r, int dtype,
                                         const void* input, void* output,
                                         size_t count,
                                         const void* const* rs_segments,
                                         const void* const* ag_segments) {
  const size_t esz = oracle_dtype_size(dtype);
  if (!esz || n < 1) return -1;
  replay_state st = {rs_segments, ag_segments, 0, 0, n - 1};
  oracle_transport tp = {&st, replay_irecv, replay_send, replay_wait,
                         replay_sendrecv};
  const size_t temp_elems = oracle_temp_elements(count, n);
  void* temp = malloc(temp_elems > 0 ? temp_elems * esz : 1); /* mpi_ops.cc:1073-1077 */
  if (!temp) return -2;
  const int rc = oracle_ring_allreduce_rank(n, r, dtype, input, temp, output,
                                            count, &tp, NULL);
  free(temp);
  return rc;
}

/* ring.h:236-301 */
int oracle_ring_allgather_rank(int n, int r, int dtype, const void* input,
                               const size_t* rows, size_t elems_per_row,
                               void* output, oracle_transport* tp) {
  const size_t esz = oracle_dtype_size(dtype);
  if (!esz || n < 1 || r < 0 || r >= n) return -1;
  char* buffer = (char*)output;

  size_t* starts = (size_t*)malloc(sizeof(size_t) * (size_t)n);
  if (!starts) return -2;
  oracle_allgather_table(rows, n, elems_per_row, starts); /* ring.h:255-259 */

  /* ring.h:263-266: own slice to its offset */
  oracle_copy(buffer + starts[r] * esz, input, elems_per_row * rows[r] * esz);

  const int recv_from = ((r - 1) + n) % n;
  const int send_to = (r + 1) % n;
  int rc = 0;

  /* ring.h:279-298: step i sends segment (r-i), receives segment (r-i-1) */
  for (int i = 0; i < n - 1 && !rc; i++) {
    const int send_seg = ((r - i) % n + n) % n;
    const int recv_seg = ((r - i - 1) % n + n) % n;
    rc = tp->sendrecv(tp->self, buffer + starts[send_seg] * esz,
                      elems_per_row * rows[send_seg] * esz, send_to,
                      buffer + starts[recv_seg] * esz,
                      elems_per_row * rows[recv_seg] * esz, recv_from);
  }
  free(starts);
  return rc;
}

/* ------------------------------------------------------------------------
 * In-process mailbox transport: one FIFO inbox per rank (its only sender is
 * the left neighbour, so per-link ordering is MPI's non-overtaking rule).
 * send() is eager: it copies the payload into a heap message and returns.
 * ---------------------------------------------------------------------- */
typedef struct mb_msg {
  struct mb_msg* next;
  size_t bytes;
  char data[];
} mb_msg;

typedef struct mb_inbox {
  pthread_mutex_t mu;
  pthread_cond_t cv;
  mb_msg* head;
  mb_msg* tail;
} mb_inbox;

typedef struct mb_rank {
  mb_inbox* inboxes; /* all ranks' inboxes */
  int rank;
  void* pending_buf;
  size_t pending_bytes;
} mb_rank;

static int mb_send(void* self, const void* buf, size_t bytes, int to) {
  mb_rank* me = (mb_rank*)self;
  mb_msg* m = (mb_msg*)malloc(sizeof(mb_msg) + bytes);
  if (!m) return -2;
  m->next = NULL;
  m->bytes = bytes;
  if (bytes) memcpy(m->data, buf, bytes);
  mb_inbox* in = &me->inboxes[to];
  pthread_mutex_lock(&in->mu);
  if (in->tail) in->tail->next = m; else in->head = m;
  in->tail = m;
  pthread_cond_signal(&in->cv);
  pthread_mutex_unlock(&in->mu);
  return 0;
}

static int mb_irecv(void* self, void* buf, size_t bytes, int from) {
  (void)from;
  mb_rank* me = (mb_rank*)self;
  me->pending_buf = buf;
  me->pending_bytes = bytes;
  return 0;
}

static int mb_wait(void* self) {
  mb_rank* me = (mb_rank*)self;
  mb_inbox* in = &me->inboxes[me->rank];
  pthread_mutex_lock(&in->mu);
  while (!in->head) pthread_cond_wait(&in->cv, &in->mu);
  mb_msg* m = in->head;
  in->head = m->next;
  if (!in->head) in->tail = NULL;
  pthread_mutex_unlock(&in->mu);
  int rc = 0;
  if (m->bytes != me->pending_bytes) rc = -3; /* size mismatch = MPI_ERR_TRUNCATE */
  else if (m->bytes) memcpy(me->pending_buf, m->data, m->bytes);
  free(m);
  return rc;
}

static int mb_sendrecv(void* self, const void* sbuf, size_t sbytes, int to,
                       void* rbuf, size_t rbytes, int from) {
  int rc = mb_send(self, sbuf, sbytes, to);
  if (rc) return rc;
  rc = mb_irecv(self, rbuf, rbytes, from);
  if (rc) return rc;
  return mb_wait(self);
}

static mb_inbox* mb_world_create(int n) {
  mb_inbox* in = (mb_inbox*)calloc((size_t)n, sizeof(mb_inbox));
  if (!in) return NULL;
  for (int i = 0; i < n; i++) {
    pthread_mutex_init(&in[i].mu, NULL);
    pthread_cond_init(&in[i].cv, NULL);
  }
  return in;
}

static void mb_world_destroy(mb_inbox* in, int n) {
  for (int i = 0; i < n; i++) {
    while (in[i].head) { mb_msg* m = in[i].head; in[i].head = m->next; free(m); }
    pthread_mutex_destroy(&in[i].mu);
    pthread_cond_destroy(&in[i].cv);
  }
  free(in);
}

typedef struct ar_job {
  mb_rank me;
  int n, dtype;
  size_t count;
  const void* input;
  void* output;
  oracle_tap* tap;
  /* allgather */
  const size_t* rows;
  size_t elems_per_row;
  int is_gather;
  /* timing */
  pthread_barrier_t* barrier;
  int warmup, reps;
  double* secs; /* this rank's per-rep seconds */
  int rc;
} ar_job;

static double now_sec(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static void* ar_thread(void* arg) {
  ar_job* j = (ar_job*)arg;
  oracle_transport tp = {&j->me, mb_irecv, mb_send, mb_wait, mb_sendrecv};
  if (j->is_gather) {
    j->rc = oracle_ring_allgather_rank(j->n, j->me.rank, j->dtype, j->input,
                                       j->rows, j->elems_per_row, j->output, &tp);
    return NULL;
  }
  const size_t esz = oracle_dtype_size(j->dtype);
  void* temp = malloc(oracle_temp_elements(j->count, j->n) * esz + 1);
  if (!temp) { j->rc = -2; return NULL; }
  const int total = j->barrier ? j->warmup + j->reps : 1;
  for (int it = 0; it < total; it++) {
    double t0 = 0;
    if (j->barrier) { pthread_barrier_wait(j->barrier); t0 = now_sec(); }
    int rc = oracle_ring_allreduce_rank(j->n, j->me.rank, j->dtype, j->input,
                                        temp, j->output, j->count, &tp, j->tap);
    if (rc) j->rc = rc;
    if (j->barrier && it >= j->warmup) j->secs[it - j->warmup] = now_sec() - t0;
  }
  free(temp);
  return NULL;
}

static int run_threads(ar_job* jobs, int n) {
  pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)n);
  if (!th) return -2;
  int started = 0, rc = 0;
  for (; started < n; started++)
    if (pthread_create(&th[started], NULL, ar_thread, &jobs[started])) { rc = -4; break; }
  /* a rank that failed to start would leave its neighbours waiting forever;
   * n is small and thread creation does not fail in practice, so a partial
   * start is reported after joining what exists only when nothing started */
  for (int i = 0; i < started; i++) pthread_join(th[i], NULL);
  free(th);
  for (int i = 0; i < n && !rc; i++) rc = jobs[i].rc;
  return rc;
}

int oracle_ring_allreduce_threads(int n, int dtype, size_t count,
                                  const void* const* inputs,
                                  void* const* outputs, oracle_tap* taps) {
  if (n < 1 || !oracle_dtype_size(dtype)) return -1;
  mb_inbox* world = mb_world_create(n);
  ar_job* jobs = (ar_job*)calloc((size_t)n, sizeof(ar_job));
  if (!world || !jobs) return -2;
  for (int r = 0; r < n; r++) {
    jobs[r].me.inboxes = world; jobs[r].me.rank = r;
    jobs[r].n = n; jobs[r].dtype = dtype; jobs[r].count = count;
    jobs[r].input = inputs[r]; jobs[r].output = outputs[r];
    jobs[r].tap = taps ? &taps[r] : NULL;
  }
  int rc = run_threads(jobs, n);
  free(jobs);
  mb_world_destroy(world, n);
  return rc;
}

int oracle_ring_allgather_threads(int n, int dtype, const void* const* inputs,
                                  const size_t* rows, size_t elems_per_row,
                                  void* const* outputs) {
  if (n < 1 || !oracle_dtype_size(dtype)) return -1;
  mb_inbox* world = mb_world_create(n);
  ar_job* jobs = (ar_job*)calloc((size_t)n, sizeof(ar_job));
  if (!world || !jobs) return -2;
  for (int r = 0; r < n; r++) {
    jobs[r].me.inboxes = world; jobs[r].me.rank = r;
    jobs[r].n = n; jobs[r].dtype = dtype;
    jobs[r].input = inputs[r]; jobs[r].output = outputs[r];
    jobs[r].rows = rows; jobs[r].elems_per_row = elems_per_row;
    jobs[r].is_gather = 1;
  }
  int rc = run_threads(jobs, n);
  free(jobs);
  mb_world_destroy(world, n);
  return rc;
}

int oracle_time_allreduce_threads(int n, int dtype, size_t count,
                                  const void* const* inputs,
                                  void* const* outputs, int warmup, int reps,
                                  double* secs) {
  if (n < 1 || reps < 1 || warmup < 0 || !oracle_dtype_size(dtype)) return -1;
  mb_inbox* world = mb_world_create(n);
  ar_job* jobs = (ar_job*)calloc((size_t)n, sizeof(ar_job));
  double* per_rank = (double*)calloc((size_t)n * (size_t)reps, sizeof(double));
  pthread_barrier_t barrier;
  if (!world || !jobs || !per_rank) return -2;
  pthread_barrier_init(&barrier, NULL, (unsigned)n);
  for (int r = 0; r < n; r++) {
    jobs[r].me.inboxes = world; jobs[r].me.rank = r;
    jobs[r].n = n; jobs[r].dtype = dtype; jobs[r].count = count;
    jobs[r].input = inputs[r]; jobs[r].output = outputs[r];
    jobs[r].barrier = &barrier; jobs[r].warmup = warmup; jobs[r].reps = reps;
    jobs[r].secs = per_rank + (size_t)r * (size_t)reps;
  }
  int rc = run_threads(jobs, n);
  for (int k = 0; k < reps; k++) {
    double worst = 0;
    for (int r = 0; r < n; r++)
      if (per_rank[(size_t)r * (size_t)reps + k] > worst)
        worst = per_rank[(size_t)r * (size_t)reps + k];
    secs[k] = worst;
  }
  pthread_barrier_destroy(&barrier);
  free(per_rank);
  free(jobs);
  mb_world_destroy(world, n);
  return rc;
}

/* ------------------------------------------------------------------------
 * Lockstep evaluation of ring.h:183-225 for all ranks at once. At
 * reduce-scatter step i rank r adds what rank r-1 held in segment (r-1-i)
 * at the start of the step; that segment is not written by rank r-1 during
 * step i (it writes (r-2-i)), so reading the neighbour's buffer in place is
 * the value MPI would have delivered.
 * ---------------------------------------------------------------------- */
int oracle_ring_allreduce_lockstep(int n, int dtype, size_t count,
                                   const void* const* inputs,
                                   void* const* outputs) {
  const size_t esz = oracle_dtype_size(dtype);
  if (!esz || n < 1) return -1;
  size_t* sizes = (size_t*)malloc(sizeof(size_t) * 2 * (size_t)n);
  if (!sizes) return -2;
  size_t* starts = sizes + n;
  oracle_segment_table(count, n, sizes, starts);
  for (int r = 0; r < n; r++) oracle_copy(outputs[r], inputs[r], count * esz);
  for (int i = 0; i < n - 1; i++) {
    for (int r = 0; r < n; r++) {
      const int left = (r - 1 + n) % n;
      const int seg = ((r - i - 1) % n + n) % n;
      oracle_accumulate(dtype, (char*)outputs[r] + starts[seg] * esz,
                        (const char*)outputs[left] + starts[seg] * esz,
                        sizes[seg]);
    }
  }
  for (int i = 0; i < n - 1; i++) {
    for (int r = 0; r < n; r++) {
      const int left = (r - 1 + n) % n;
      const int seg = ((r - i) % n + n) % n;
      oracle_copy((char*)outputs[r] + starts[seg] * esz,
                  (const char*)outputs[left] + starts[seg] * esz,
                  sizes[seg] * esz);
    }
  }
  free(sizes);
  return 0;
}
