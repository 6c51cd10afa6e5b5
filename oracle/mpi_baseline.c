/*
 * CPU baseline: the reference's MPI-backend host combine.
 *
 * Al::Allreduce<MPIBackend>(send, recv, count, sum, comm) is a direct call of
 * MPI_Allreduce on a duplicated communicator
 * (reference: include/aluminum/mpi_impl.hpp:141-167 ->
 * include/aluminum/mpi/allreduce.hpp:38-44).  This program makes that call
 * with the reference benchmark's method (barrier before each iteration,
 * steady clock, warm-up then timed iterations;
 * benchmark/benchmark_ops.cpp:143-195) and prints one JSON line.
 * TEST / BENCH INFRASTRUCTURE ONLY.
 *
 * usage: mpiexec -n 4 ./mpi_baseline [count_per_rank] [warmup] [iters] [root]
 * With a root >= 0 the call is MPI_Reduce to that rank instead
 * (include/aluminum/mpi/reduce.hpp:41-49) and the checksum is the root's.
 */
#include <mpi.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

#include "oracle.h"

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static int cmp_double(const void *a, const void *b) {
  double x = *(const double *)a, y = *(const double *)b;
  return (x > y) - (x < y);
}

int main(int argc, char **argv) {
  MPI_Init(&argc, &argv);
  MPI_Comm comm;
  MPI_Comm_dup(MPI_COMM_WORLD, &comm);
  int rank, P;
  MPI_Comm_rank(comm, &rank);
  MPI_Comm_size(comm, &P);
  size_t n = argc > 1 ? (size_t)atoll(argv[1]) : (size_t)1 << 20;
  int warm = argc > 2 ? atoi(argv[2]) : 10, iters = argc > 3 ? atoi(argv[3]) : 100;
  int root = argc > 4 ? atoi(argv[4]) : -1;
  if (root >= P) root = P - 1;
  alo_set_num_threads(1);
  float *in = (float *)malloc(n * sizeof(float)), *out = (float *)malloc(n * sizeof(float));
  double *t = (double *)malloc(sizeof(double) * (size_t)iters);
  alo_fill(in, n, ALO_F32, ALO_DIST_UNIFORM_PM1, 1000u + (unsigned)rank, 0);
  for (int it = 0; it < warm + iters; it++) {
    MPI_Barrier(comm);
    double t0 = now_s();
    if (root < 0) MPI_Allreduce(in, out, (int)n, MPI_FLOAT, MPI_SUM, comm);
    else MPI_Reduce(in, out, (int)n, MPI_FLOAT, MPI_SUM, root, comm);
    double dt = now_s() - t0, mx;
    MPI_Reduce(&dt, &mx, 1, MPI_DOUBLE, MPI_MAX, 0, comm);
    if (it >= warm) t[it - warm] = mx;
  }
  unsigned long long cs = alo_checksum(out, n * sizeof(float));
  if (root > 0) { /* the root's result is the one that counts; rank 0 prints */
    if (rank == root) MPI_Send(&cs, 1, MPI_UNSIGNED_LONG_LONG, 0, 9, comm);
    if (rank == 0) MPI_Recv(&cs, 1, MPI_UNSIGNED_LONG_LONG, root, 9, comm, MPI_STATUS_IGNORE);
  }
  if (rank == 0) {
    qsort(t, (size_t)iters, sizeof(double), cmp_double);
    double med = t[iters / 2], mn = t[0];
    double bytes = (double)(P + 1) * (double)n * 4.0;
    printf("{\"ranks\": %d, \"count\": %zu, \"iters\": %d, \"median_ms\": %.6f, \"min_ms\": %.6f, "
           "\"gbps_median\": %.4f, \"checksum\": \"%016llx\"}\n",
           P, n, iters, med * 1e3, mn * 1e3, bytes / med * 1e-9, cs);
  }
  free(in); free(out); free(t);
  MPI_Comm_free(&comm);
  MPI_Finalize();
  return 0;
}
