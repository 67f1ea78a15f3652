/*
 * TEST INFRASTRUCTURE ONLY — see ring_oracle.h.
 *
 * The per-rank restatement of the reference ring (ring_oracle.c) run over a
 * real MPI library, one process per rank, with the reference's own calls:
 * MPI_Irecv / MPI_Send / MPI_Wait in the reduce-scatter (ring.h:189-200) and
 * MPI_Sendrecv in the allgather (ring.h:221-224), tag 12 (ring.h:19).
 *
 * Two uses:
 *   check mode:  ring_mpi check <dtype> <count> <dir>
 *       rank r reads <dir>/in_<r>.bin, writes <dir>/out_<r>.bin; the tests
 *       compare these with the threaded and lockstep evaluations.
 *   time mode:   ring_mpi time <dtype> <count> <warmup> <reps>
 *       rank r fills its tensor from a fixed generator, times RingAllreduce
 *       only (MPI_Wtime around the call, barrier before each rep) and rank 0
 *       prints one JSON line with the per-rep maxima over ranks.
 */
#include <mpi.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ring_oracle.h"

#define TAG_TENSOR 12 /* ring.h:19 */

typedef struct mpi_rank_state {
  MPI_Request req;
} mpi_rank_state;

static int tp_irecv(void* self, void* buf, size_t bytes, int from) {
  mpi_rank_state* st = (mpi_rank_state*)self;
  return MPI_Irecv(buf, (int)bytes, MPI_BYTE, from, TAG_TENSOR, MPI_COMM_WORLD,
                   &st->req) != MPI_SUCCESS;
}
static int tp_send(void* self, const void* buf, size_t bytes, int to) {
  (void)self;
  return MPI_Send((void*)buf, (int)bytes, MPI_BYTE, to, TAG_TENSOR,
                  MPI_COMM_WORLD) != MPI_SUCCESS;
}
static int tp_wait(void* self) {
  mpi_rank_state* st = (mpi_rank_state*)self;
  MPI_Status status;
  return MPI_Wait(&st->req, &status) != MPI_SUCCESS;
}
static int tp_sendrecv(void* self, const void* sbuf, size_t sbytes, int to,
                       void* rbuf, size_t rbytes, int from) {
  (void)self;
  MPI_Status status;
  return MPI_Sendrecv((void*)sbuf, (int)sbytes, MPI_BYTE, to, TAG_TENSOR, rbuf,
                      (int)rbytes, MPI_BYTE, from, TAG_TENSOR, MPI_COMM_WORLD,
                      &status) != MPI_SUCCESS;
}

static int dtype_code(const char* s) {
  if (!strcmp(s, "f32")) return ORACLE_F32;
  if (!strcmp(s, "i32")) return ORACLE_I32;
  if (!strcmp(s, "i64")) return ORACLE_I64;
  return -1;
}

/* uniform [-1,1) floats / small integers from a 64-bit LCG; values only need
 * to be ordinary (no denormals, no overflow), the timing does not depend on
 * them */
static void fill(int dtype, void* p, size_t count, unsigned long long seed) {
  unsigned long long s = seed * 6364136223846793005ULL + 1442695040888963407ULL;
  for (size_t i = 0; i < count; i++) {
    s = s * 6364136223846793005ULL + 1442695040888963407ULL;
    unsigned v = (unsigned)(s >> 40); /* 24 bits */
    if (dtype == ORACLE_F32) ((float*)p)[i] = (float)v / 8388608.0f - 1.0f;
    else if (dtype == ORACLE_I32) ((int32_t*)p)[i] = (int32_t)(v % 2001u) - 1000;
    else ((int64_t*)p)[i] = (int64_t)(v % 2001u) - 1000;
  }
}

int main(int argc, char** argv) {
  MPI_Init(&argc, &argv);
  int n, r;
  MPI_Comm_size(MPI_COMM_WORLD, &n);
  MPI_Comm_rank(MPI_COMM_WORLD, &r);
  int rc = 2;
  if (argc >= 5) {
    const int dtype = dtype_code(argv[2]);
    const size_t count = (size_t)strtoull(argv[3], NULL, 10);
    const size_t esz = oracle_dtype_size(dtype);
    if (esz) {
      void* in = malloc(count * esz + 1);
      void* out = malloc(count * esz + 1);
      void* temp = malloc(oracle_temp_elements(count, n) * esz + 1);
      mpi_rank_state st;
      oracle_transport tp = {&st, tp_irecv, tp_send, tp_wait, tp_sendrecv};
      if (!strcmp(argv[1], "check")) {
        char path[4096];
        snprintf(path, sizeof path, "%s/in_%d.bin", argv[4], r);
        FILE* f = fopen(path, "rb");
        rc = 3;
        if (f && fread(in, esz, count, f) == count) {
          fclose(f);
          rc = oracle_ring_allreduce_rank(n, r, dtype, in, temp, out, count, &tp, NULL);
          snprintf(path, sizeof path, "%s/out_%d.bin", argv[4], r);
          f = fopen(path, "wb");
          if (!f || fwrite(out, esz, count, f) != count) rc = 4;
          if (f) fclose(f);
        }
      } else if (!strcmp(argv[1], "time") && argc >= 6) {
        const int warmup = atoi(argv[4]);
        const int reps = atoi(argv[5]);
        fill(dtype, in, count, 1234ULL + (unsigned long long)r);
        double* mine = (double*)calloc((size_t)reps, sizeof(double));
        double* worst = (double*)calloc((size_t)reps, sizeof(double));
        rc = 0;
        for (int it = 0; it < warmup + reps; it++) {
          MPI_Barrier(MPI_COMM_WORLD);
          double t0 = MPI_Wtime();
          rc |= oracle_ring_allreduce_rank(n, r, dtype, in, temp, out, count, &tp, NULL);
          double t1 = MPI_Wtime();
          if (it >= warmup) mine[it - warmup] = t1 - t0;
        }
        MPI_Reduce(mine, worst, reps, MPI_DOUBLE, MPI_MAX, 0, MPI_COMM_WORLD);
        if (r == 0) {
          printf("{\"transport\": \"mpi\", \"ranks\": %d, \"dtype\": \"%s\", "
                 "\"count\": %zu, \"secs\": [", n, argv[2], count);
          for (int k = 0; k < reps; k++) printf("%s%.9f", k ? ", " : "", worst[k]);
          printf("]}\n");
        }
        free(mine);
        free(worst);
      }
      free(in); free(out); free(temp);
    }
  }
  if (rc == 2 && r == 0)
    fprintf(stderr, "usage: ring_mpi check <f32|i32|i64> <count> <dir> | "
                    "time <f32|i32|i64> <count> <warmup> <reps>\n");
  MPI_Finalize();
  return rc;
}
