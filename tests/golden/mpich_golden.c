/*
 * Golden-vector generator for the host combine that the reference performs.
 *
 * The reference's MPI backend forwards Al::Allreduce / Al::Reduce_scatter
 * straight to the MPI library (include/aluminum/mpi/allreduce.hpp:38-44,
 * include/aluminum/mpi/reduce_scatter.hpp:40-46), so the values it produces
 * are those of MPI_Allreduce / MPI_Reduce_scatter_block in the MPI it was
 * built with; Al::Reduce and Al::Reduce_scatterv likewise end in MPI_Reduce and
 * MPI_Reduce_scatter (include/aluminum/mpi/reduce.hpp:41-49,
 * include/aluminum/ht/reduce.hpp:72-82, ht/reduce_scatterv.hpp:75-79).  This program makes exactly those calls against the image's
 * MPICH and prints one JSON document (inputs and outputs as hex strings) that
 * is committed next to it as a fixture.  It runs nothing from the reference.
 *
 * Build and run: see make_mpich_golden.sh.
 */
#include <mpi.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../oracle/oracle.h"

static int rank_, P_;

static const char *dt_name[] = {"i8", "u8", "i16", "u16", "i32", "u32", "i64",
                                "u64", "f16", "bf16", "f32", "f64"};
static const char *op_name[] = {"sum", "prod", "min", "max", "lor", "land",
                                "lxor", "bor", "band", "bxor"};

static MPI_Datatype mpi_type(int dt) {
  switch (dt) {
  case ALO_I8: return MPI_SIGNED_CHAR;
  case ALO_U8: return MPI_UNSIGNED_CHAR;
  case ALO_I16: return MPI_SHORT;
  case ALO_U16: return MPI_UNSIGNED_SHORT;
  case ALO_I32: return MPI_INT;
  case ALO_U32: return MPI_UNSIGNED;
  case ALO_I64: return MPI_LONG;
  case ALO_U64: return MPI_UNSIGNED_LONG;
  case ALO_F16: case ALO_BF16: return MPI_SHORT;
  case ALO_F32: return MPI_FLOAT;
  case ALO_F64: return MPI_DOUBLE;
  default: return MPI_DATATYPE_NULL;
  }
}

static MPI_Op mpi_op(int op) {
  static MPI_Op t[10];
  t[0] = MPI_SUM; t[1] = MPI_PROD; t[2] = MPI_MIN; t[3] = MPI_MAX; t[4] = MPI_LOR;
  t[5] = MPI_LAND; t[6] = MPI_LXOR; t[7] = MPI_BOR; t[8] = MPI_BAND; t[9] = MPI_BXOR;
  return t[op];
}

/* The reference's own reduction functions for fp16 / bf16 (src/mpi_impl.cpp:61-145) are registered
 * as commutative user-defined operations on MPI_SHORT (src/mpi_impl.cpp:190-204,
 * include/aluminum/mpi/utils.hpp:59-67).  The same is done here with the oracle's step as the
 * function body: these cases pin the ORDER in which the MPI library applies a user-defined
 * commutative operation, not the step's arithmetic (which other tests pin). */
static int user_dt, user_op;
static void user_fn(void *in, void *inout, int *len, MPI_Datatype *type) {
  (void)type;
  alo_step(inout, in, (size_t)*len, user_dt, user_op);
}
static MPI_Op user_mpi_op = MPI_OP_NULL;
static int is_half(int dt) { return dt == ALO_F16 || dt == ALO_BF16; }

/* The operation to pass to MPI for (dt, op). */
static MPI_Op op_for(int dt, int op) {
  if (!is_half(dt)) return mpi_op(op);
  user_dt = dt;
  user_op = op;
  if (user_mpi_op == MPI_OP_NULL) MPI_Op_create(&user_fn, 1, &user_mpi_op);
  return user_mpi_op;
}

/* 1 if `mine` is nonzero on every rank. */
static int on_all(int mine) {
  int all = 0;
  MPI_Allreduce(&mine, &all, 1, MPI_INT, MPI_LAND, MPI_COMM_WORLD);
  return all;
}

/* The host-transfer backend makes the non-blocking, in-place form of every call
 * (include/aluminum/ht/allreduce.hpp:76-79, ht/reduce.hpp:72-82, ht/reduce_scatter.hpp:71-74,
 * ht/reduce_scatterv.hpp:76-79); every case records whether that form returned the same bytes, and
 * what it returned where it did not ("out_nonblocking": MPI_Ireduce and MPI_Iallreduce cut a long
 * message into blocks differently from MPI_Reduce and MPI_Allreduce, which shows where a float
 * min / max meets a tie or a NaN and the count is not a multiple of the power of two of ranks). */
static void emit_nb(int same) {
  if (rank_ == 0) printf(", \"nonblocking_in_place_same\": %s", same ? "true" : "false");
}

static void print_hex(const unsigned char *p, size_t nbytes) {
  putchar('"');
  for (size_t i = 0; i < nbytes; i++) printf("%02x", p[i]);
  putchar('"');
}

static int first_case = 1;
/* 32 ranks and more: an allreduce keeps rank 0's output only (and records that every rank received the
 * same bytes), and no case repeats its inputs. */
static int lean_ = 0;
/* Set while cases are made whose inputs, the generator's, need not be repeated whatever their size. */
static int no_inputs_ = 0;

/* Gather `nbytes` from every rank to rank 0 and print as a JSON list. */
static void emit_list(const char *key, const void *mine, size_t nbytes) {
  unsigned char *all = NULL;
  if (rank_ == 0) all = (unsigned char *)malloc(nbytes * (size_t)P_);
  MPI_Gather(mine, (int)nbytes, MPI_BYTE, all, (int)nbytes, MPI_BYTE, 0, MPI_COMM_WORLD);
  if (rank_ == 0) {
    printf(", \"%s\": [", key);
    for (int r = 0; r < P_; r++) {
      if (r) printf(", ");
      print_hex(all + (size_t)r * nbytes, nbytes);
    }
    printf("]");
    free(all);
  }
}

static void emit_sums(const char *key, const void *mine, size_t nbytes) {
  unsigned long long cs = alo_checksum(mine, nbytes), *all = NULL;
  if (rank_ == 0) all = (unsigned long long *)malloc(sizeof(*all) * (size_t)P_);
  MPI_Gather(&cs, 1, MPI_UNSIGNED_LONG_LONG, all, 1, MPI_UNSIGNED_LONG_LONG, 0, MPI_COMM_WORLD);
  if (rank_ == 0) {
    printf(", \"%s\": [", key);
    for (int r = 0; r < P_; r++) printf("%s\"%016llx\"", r ? ", " : "", all[r]);
    printf("]");
    free(all);
  }
}

static void head(const char *coll, int dt, int op, size_t n, int dist,
                 unsigned long long seed, const char *note) {
  if (rank_ != 0) return;
  printf("%s\n  {\"coll\": \"%s\", \"P\": %d, \"dtype\": \"%s\", \"op\": \"%s\", "
         "\"n\": %zu, \"dist\": %d, \"seed_base\": %llu, \"note\": \"%s\"",
         first_case ? "" : ",", coll, P_, dt_name[dt], op_name[op], n, dist, seed, note);
}

static void tail(void) {
  if (rank_ == 0) { printf("}"); fflush(stdout); }
  first_case = 0;
}

/* Special values planted over the start of a float buffer (P = 2 only):
 * element i of rank 0 meets element i of rank 1.  NaN against numbers on
 * either side, signed-zero ties both ways, infinities, denormals. */
static void plant_specials_many(void *buf, size_t n, int dt);

static void plant_specials(void *buf, size_t n, int dt) {
  if (P_ != 2) { plant_specials_many(buf, n, dt); return; }
  static const unsigned r0[] = {0x7fc00000u, 0xbf800000u, 0x7fc00000u, 0x00000000u, 0x80000000u,
                                0x7f800000u, 0xff800000u, 0x00000001u, 0x80000001u, 0x3f800000u,
                                0x7f7fffffu, 0x00800000u, 0x00000000u, 0x80000000u, 0x7f800000u,
                                0x00400000u};
  static const unsigned r1[] = {0x7f800000u, 0x7fc00000u, 0x7fc00000u, 0x80000000u, 0x00000000u,
                                0xff800000u, 0x7f800000u, 0x80000001u, 0x00000001u, 0x3f800000u,
                                0x7f7fffffu, 0x00800001u, 0x00000000u, 0x80000000u, 0x7f800000u,
                                0x00400000u};
  const size_t cnt = sizeof(r0) / sizeof(r0[0]);
  for (size_t i = 0; i < n && i < cnt; i++) {
    unsigned u = rank_ == 0 ? r0[i] : r1[i];
    float f;
    memcpy(&f, &u, 4);
    if (dt == ALO_F32) ((float *)buf)[i] = f;
    else ((double *)buf)[i] = (double)f; /* exact widening keeps the class */
  }
}

/* More than two ranks: every element of every rank is drawn from a pool of
 * special values (and two ordinary ones) by a fixed rule, so that NaNs, zeros
 * of both signs and infinities meet in every position of the combine order. */
/* (tests/util.py restates this rule, so that long cases need not repeat their inputs) */
static void plant_specials_many(void *buf, size_t n, int dt) {
  static const unsigned pool[] = {0x7fc00000u, 0xbf800000u, 0x00000000u, 0x80000000u, 0x7f800000u,
                                  0xff800000u, 0x00000001u, 0x80000001u, 0x3f800000u, 0x7f7fffffu,
                                  0x00800000u, 0x00400000u, 0x3e99999au};
  const size_t cnt = sizeof(pool) / sizeof(pool[0]);
  for (size_t i = 0; i < n; i++) {
    unsigned long long h = alo_mix64(77, (unsigned long long)i * 64u + (unsigned long long)rank_);
    unsigned u = pool[(size_t)(h % cnt)];
    if (i % 4 == 0 && (h >> 32) % 3 == 0) u = 0x80000000u;      /* plenty of zero ties */
    else if (i % 4 == 0) u = 0x00000000u;
    float f;
    memcpy(&f, &u, 4);
    if (dt == ALO_F32) ((float *)buf)[i] = f;
    else if (dt == ALO_F64) ((double *)buf)[i] = (double)f;
    else if (dt == ALO_BF16) ((unsigned short *)buf)[i] = alo_f32_to_bf16(f);
    else ((unsigned short *)buf)[i] = alo_f32_to_f16(f);
  }
}

static void case_allreduce(int dt, int op, size_t n, int dist, int specials,
                           const char *note) {
  const unsigned long long seed = 1000;
  size_t es = alo_dtype_size(dt);
  void *in = malloc(n * es), *out = malloc(n * es);
  alo_fill(in, n, dt, dist, seed + (unsigned long long)rank_, 0);
  if (specials) plant_specials(in, n, dt);
  MPI_Allreduce(in, out, (int)n, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD);
  void *nb = malloc(n * es);
  MPI_Request req;
  memcpy(nb, in, n * es);
  MPI_Iallreduce(MPI_IN_PLACE, nb, (int)n, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD, &req);
  MPI_Wait(&req, MPI_STATUS_IGNORE);
  int same = on_all(memcmp(nb, out, n * es) == 0);
  head("allreduce", dt, op, n, dist, seed, note);
  emit_nb(same);
  if (!same) { /* rank 0's, and whether every rank received those bytes */
    void *nb0 = malloc(n * es);
    memcpy(nb0, nb, n * es);
    MPI_Bcast(nb0, (int)(n * es), MPI_BYTE, 0, MPI_COMM_WORLD);
    int nb_same = on_all(memcmp(nb0, nb, n * es) == 0);
    if (rank_ == 0) {
      printf(", \"nonblocking_all_ranks_same\": %s, \"out_nonblocking\": ", nb_same ? "true" : "false");
      print_hex((unsigned char *)nb, n * es);
    }
    free(nb0);
  }
  if (lean_) {
    memcpy(nb, out, n * es);
    MPI_Bcast(nb, (int)(n * es), MPI_BYTE, 0, MPI_COMM_WORLD);
    int all_same = on_all(memcmp(nb, out, n * es) == 0);
    if (rank_ == 0) {
      printf(", \"all_ranks_same\": %s, \"out\": [", all_same ? "true" : "false");
      print_hex((unsigned char *)out, n * es);
      printf("]");
    }
  } else {
    /* inputs are repeated for short messages; the others are the generator's, or planted by rule */
    if (n * es <= 2048 && (specials || !is_half(dt)) && !no_inputs_) emit_list("in", in, n * es);
    emit_list("out", out, n * es);
  }
  tail();
  free(in); free(out); free(nb);
}

/* count = elements per rank; send buffer holds P*count. */
static void case_reduce_scatter_x(int dt, int op, size_t count, int dist, int full, int specials,
                                  const char *note) {
  const unsigned long long seed = 1000;
  size_t es = alo_dtype_size(dt), n = count * (size_t)P_;
  void *in = malloc(n * es), *out = malloc(count * es);
  alo_fill(in, n, dt, dist, seed + (unsigned long long)rank_, 0);
  if (specials) plant_specials(in, n, dt);
  MPI_Reduce_scatter_block(in, out, (int)count, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD);
  void *nb = malloc(n * es);
  MPI_Request req;
  memcpy(nb, in, n * es);
  MPI_Ireduce_scatter_block(MPI_IN_PLACE, nb, (int)count, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD, &req);
  MPI_Wait(&req, MPI_STATUS_IGNORE);
  int same = on_all(memcmp(nb, out, count * es) == 0);
  free(nb);
  head("reduce_scatter", dt, op, count, dist, seed, note);
  emit_nb(same);
  if (full) {
    if ((!is_half(dt) || specials) && !lean_) emit_list("in", in, n * es);
    emit_list("out", out, count * es);
  } else {
    emit_sums("out_checksum", out, count * es);
    emit_list("out_head", out, 8 * es);
  }
  tail();
  free(in); free(out);
}

static void case_reduce_scatter(int dt, int op, size_t count, int dist, int full, const char *note) {
  case_reduce_scatter_x(dt, op, count, dist, full, 0, note);
}

/* MPI_Reduce_scatter with uneven counts: rank b receives 3 + 2*((b*5) % 4) elements, rank 1 none. */
static void case_reduce_scatterv(int dt, int op, int dist, const char *note) {
  const unsigned long long seed = 1000;
  size_t es = alo_dtype_size(dt), n = 0;
  int *counts = (int *)malloc(sizeof(int) * (size_t)P_);
  for (int b = 0; b < P_; b++) { counts[b] = b == 1 ? 0 : 3 + 2 * ((b * 5) % 4); n += (size_t)counts[b]; }
  void *in = malloc(n * es), *out = malloc(16 * es);
  memset(out, 0, 16 * es);
  alo_fill(in, n, dt, dist, seed + (unsigned long long)rank_, 0);
  MPI_Reduce_scatter(in, out, counts, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD);
  void *nb = malloc((n ? n : 1) * es);
  MPI_Request req;
  memcpy(nb, in, n * es);
  MPI_Ireduce_scatter(MPI_IN_PLACE, nb, counts, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD, &req);
  MPI_Wait(&req, MPI_STATUS_IGNORE);
  int same = on_all(memcmp(nb, out, (size_t)counts[rank_] * es) == 0);
  free(nb);
  head("reduce_scatterv", dt, op, n, dist, seed, note);
  emit_nb(same);
  if (rank_ == 0) {
    printf(", \"counts\": [");
    for (int b = 0; b < P_; b++) printf("%s%d", b ? ", " : "", counts[b]);
    printf("]");
  }
  if (!is_half(dt)) emit_list("in", in, n * es);
  emit_list("out", out, 16 * es); /* first counts[rank] elements are significant */
  tail();
  free(in); free(out); free(counts);
}

/* MPI_Reduce to `root`; only the root's output is significant. */
static void case_reduce(int dt, int op, size_t n, int dist, int root, int specials, const char *note) {
  const unsigned long long seed = 1000;
  size_t es = alo_dtype_size(dt);
  void *in = malloc(n * es), *out = malloc(n * es);
  memset(out, 0, n * es);
  alo_fill(in, n, dt, dist, seed + (unsigned long long)rank_, 0);
  if (specials) plant_specials(in, n, dt);
  MPI_Reduce(in, out, (int)n, mpi_type(dt), op_for(dt, op), root, MPI_COMM_WORLD);
  void *nb = malloc(n * es);
  MPI_Request req;
  memcpy(nb, in, n * es);
  if (rank_ == root) MPI_Ireduce(MPI_IN_PLACE, nb, (int)n, mpi_type(dt), op_for(dt, op), root, MPI_COMM_WORLD, &req);
  else MPI_Ireduce(nb, NULL, (int)n, mpi_type(dt), op_for(dt, op), root, MPI_COMM_WORLD, &req);
  MPI_Wait(&req, MPI_STATUS_IGNORE);
  int same = on_all(rank_ != root || memcmp(nb, out, n * es) == 0);
  if (root != 0) { /* bring the root's results to rank 0, which prints */
    if (rank_ == root) MPI_Send(out, (int)(n * es), MPI_BYTE, 0, 7, MPI_COMM_WORLD);
    if (rank_ == 0) MPI_Recv(out, (int)(n * es), MPI_BYTE, root, 7, MPI_COMM_WORLD, MPI_STATUS_IGNORE);
    if (rank_ == root) MPI_Send(nb, (int)(n * es), MPI_BYTE, 0, 8, MPI_COMM_WORLD);
    if (rank_ == 0) MPI_Recv(nb, (int)(n * es), MPI_BYTE, root, 8, MPI_COMM_WORLD, MPI_STATUS_IGNORE);
  }
  head("reduce", dt, op, n, dist, seed, note);
  if (rank_ == 0) printf(", \"root\": %d", root);
  emit_nb(same);
  if (!same && rank_ == 0) {
    if (n <= 1024) { printf(", \"out_nonblocking\": "); print_hex((unsigned char *)nb, n * es); }
    else printf(", \"out_nonblocking_checksum\": \"%016llx\"", (unsigned long long)alo_checksum(nb, n * es));
  }
  free(nb);
  if (n <= 1024) {
    /* inputs are repeated for short messages; the others are the generator's, or planted by rule */
    if (specials && !lean_ && n * es <= 2048) emit_list("in", in, n * es);
    if (rank_ == 0) { printf(", \"out\": "); print_hex((unsigned char *)out, n * es); }
  } else if (rank_ == 0) {
    printf(", \"out_checksum\": \"%016llx\", \"out_head\": ", (unsigned long long)alo_checksum(out, n * es));
    print_hex((unsigned char *)out, 8 * es);
  }
  tail();
  free(in); free(out);
}

/* MPI_Reduce_scatter with uneven counts whose total reaches 512 KiB (the size
 * from which the block variant changes algorithm): rank b receives
 * base + 1000*((b*5) % 4) + b elements, rank 1 none.  Outputs as checksums. */
static void case_reduce_scatterv_long(int dt, int op, int dist, const char *note) {
  const unsigned long long seed = 1000;
  size_t es = alo_dtype_size(dt), n = 0;
  int *counts = (int *)malloc(sizeof(int) * (size_t)P_);
  const int base = (int)((size_t)(1u << 20) / (size_t)P_ / es);
  for (int b = 0; b < P_; b++) { counts[b] = b == 1 ? 0 : base + 1000 * ((b * 5) % 4) + b; n += (size_t)counts[b]; }
  void *in = malloc(n * es), *out = malloc(((size_t)base + 4096) * es);
  memset(out, 0, ((size_t)base + 4096) * es);
  alo_fill(in, n, dt, dist, seed + (unsigned long long)rank_, 0);
  MPI_Reduce_scatter(in, out, counts, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD);
  void *nb = malloc(n * es);
  MPI_Request req;
  memcpy(nb, in, n * es);
  MPI_Ireduce_scatter(MPI_IN_PLACE, nb, counts, mpi_type(dt), op_for(dt, op), MPI_COMM_WORLD, &req);
  MPI_Wait(&req, MPI_STATUS_IGNORE);
  int same = on_all(memcmp(nb, out, (size_t)counts[rank_] * es) == 0);
  free(nb);
  head("reduce_scatterv", dt, op, n, dist, seed, note);
  emit_nb(same);
  if (rank_ == 0) {
    printf(", \"counts\": [");
    for (int b = 0; b < P_; b++) printf("%s%d", b ? ", " : "", counts[b]);
    printf("]");
  }
  emit_sums("out_checksum", out, (size_t)counts[rank_] * es);
  emit_list("out_head", out, 8 * es);
  tail();
  free(in); free(out); free(counts);
}

int main(int argc, char **argv) {
  MPI_Init(&argc, &argv);
  MPI_Comm_rank(MPI_COMM_WORLD, &rank_);
  MPI_Comm_size(MPI_COMM_WORLD, &P_);
  alo_set_num_threads(1);
  int big = argc > 1 && !strcmp(argv[1], "big");

  if (rank_ == 0) {
    char ver[MPI_MAX_LIBRARY_VERSION_STRING];
    int len;
    MPI_Get_library_version(ver, &len);
    for (char *c = ver; *c; c++) if (*c == '\n' || *c == '\t' || *c == '"') *c = ' ';
    ver[60] = 0;
    printf("{\"mpi\": \"%s\", \"P\": %d, \"cases\": [", ver, P_);
  }

  if (P_ >= 32) {
    /* Many ranks (the tree orders over 32 slots and over two halves of 32; pre-folds of up to 31 pairs): a
     * small set, outputs only.  Inputs are the generator's, or planted by rule. */
    lean_ = 1;
    const size_t nlong = 2048 / 4 + 8;
    const int roots[3] = {0, 1, P_ - 1};
    case_allreduce(ALO_F32, ALO_SUM, 16, ALO_DIST_UNIFORM_PM1, 0, "short message");
    case_allreduce(ALO_F32, ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, 0, "long message");
    case_allreduce(ALO_F32, ALO_PROD, nlong, ALO_DIST_UNIFORM_09_11, 0, "long message");
    case_allreduce(ALO_F64, ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, 0, "long message");
    case_allreduce(ALO_BF16, ALO_SUM, 2 * nlong, ALO_DIST_UNIFORM_PM1, 0, "long message");
    case_allreduce(ALO_F32, ALO_MIN, nlong + 3, ALO_DIST_UNIFORM_PM1, 1, "specials");
    case_allreduce(ALO_F32, ALO_MAX, 96, ALO_DIST_UNIFORM_PM1, 1, "specials");
    for (int k = 0; k < 3; k++) {
      case_reduce(ALO_F32, ALO_SUM, 16, ALO_DIST_UNIFORM_PM1, roots[k], 0, "short message");
      case_reduce(ALO_F32, ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, roots[k], 0, "long message");
      case_reduce(ALO_BF16, ALO_SUM, 2 * nlong, ALO_DIST_UNIFORM_PM1, roots[k], 0, "long message");
      case_reduce(ALO_F32, ALO_MAX, nlong + 3, ALO_DIST_UNIFORM_PM1, roots[k], 1, "specials");
    }
    case_reduce_scatter(ALO_F32, ALO_SUM, 8, ALO_DIST_UNIFORM_PM1, 1, "short message");
    case_reduce_scatter_x(ALO_F32, ALO_MIN, 8, ALO_DIST_UNIFORM_PM1, 1, 1, "specials");
    if (big)
      case_reduce_scatter(ALO_F32, ALO_SUM, (size_t)(1u << 20) / (size_t)P_ / 4 + 64, ALO_DIST_UNIFORM_PM1, 0,
                          "long message");
    if (rank_ == 0) printf("\n]}\n");
    MPI_Finalize();
    return 0;
  }

  /* fp sum / prod: 16 elements (<= 2048 bytes) and just over 2048 bytes. */
  const int fdt[2] = {ALO_F32, ALO_F64};
  for (int d = 0; d < 2; d++) {
    const size_t nlong = 2048 / alo_dtype_size(fdt[d]) + 8;
    case_allreduce(fdt[d], ALO_SUM, 16, ALO_DIST_UNIFORM_PM1, 0, "short message");
    case_allreduce(fdt[d], ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, 0, "long message");
    case_allreduce(fdt[d], ALO_PROD, 16, ALO_DIST_UNIFORM_09_11, 0, "short message");
    case_allreduce(fdt[d], ALO_PROD, nlong, ALO_DIST_UNIFORM_09_11, 0, "long message");
    case_allreduce(fdt[d], ALO_MIN, 48, ALO_DIST_UNIFORM_PM1, 0, "");
    case_allreduce(fdt[d], ALO_MAX, 48, ALO_DIST_UNIFORM_PM1, 0, "");
    if (P_ == 2) { /* the two-operand step, special values, seen from both ranks */
      for (int op = ALO_SUM; op <= ALO_MAX; op++)
        case_allreduce(fdt[d], op, 48, ALO_DIST_UNIFORM_PM1, 1, "specials");
    }
    if (P_ == 3 || P_ == 4 || P_ == 7 || P_ == 8 || P_ == 16) { /* special values under a whole order; every rank's output is kept */
      for (int op = ALO_SUM; op <= ALO_MAX; op++) {
        case_allreduce(fdt[d], op, 96, ALO_DIST_UNIFORM_PM1, 1, "specials");
        case_allreduce(fdt[d], op, nlong + 3, ALO_DIST_UNIFORM_PM1, 1, "specials"); /* not a multiple of 2^k */
      }
    }
    /* rooted reduce: first, second and last rank as root, below and above 2048 bytes */
    const int roots[3] = {0, 1, P_ - 1};
    for (int k = 0; k < 3; k++) {
      if (k == 2 && roots[k] <= 1) break;
      case_reduce(fdt[d], ALO_SUM, 16, ALO_DIST_UNIFORM_PM1, roots[k], 0, "short message");
      case_reduce(fdt[d], ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, roots[k], 0, "long message");
      case_reduce(fdt[d], ALO_PROD, 16, ALO_DIST_UNIFORM_09_11, roots[k], 0, "short message");
      case_reduce(fdt[d], ALO_PROD, nlong, ALO_DIST_UNIFORM_09_11, roots[k], 0, "long message");
      if (big) case_reduce(fdt[d], ALO_SUM, (size_t)(1u << 18) + 3, ALO_DIST_UNIFORM_PM1, roots[k], 0, "1 MiB and more");
      if ((P_ == 3 || P_ == 4 || P_ == 7 || P_ == 8 || P_ == 16) && (d == 0 || k == 1))
        for (int op = ALO_MIN; op <= ALO_MAX; op++) {
          case_reduce(fdt[d], op, 96, ALO_DIST_UNIFORM_PM1, roots[k], 1, "specials");
          case_reduce(fdt[d], op, nlong + 3, ALO_DIST_UNIFORM_PM1, roots[k], 1, "specials");
        }
    }
    case_reduce_scatter(fdt[d], ALO_SUM, 8, ALO_DIST_UNIFORM_PM1, 1, "short message");
    case_reduce_scatterv(fdt[d], ALO_SUM, ALO_DIST_UNIFORM_PM1, "uneven counts");
    if (big) { /* >= 512 KiB in total selects the pairwise exchange */
      case_reduce_scatter(fdt[d], ALO_SUM, (size_t)(1u << 20) / (size_t)P_ / alo_dtype_size(fdt[d]) + 64,
                          ALO_DIST_UNIFORM_PM1, 0, "long message");
      case_reduce_scatterv_long(fdt[d], ALO_SUM, ALO_DIST_UNIFORM_PM1, "uneven counts, long message");
    }
    /* the sizes at which the library changes algorithm, exactly: 2048 bytes (still the short-message
     * tree; 5 and 7 ranks, where the two trees differ in shape) and 512 KiB in all (already the pairwise
     * exchange), with one element less or more beside them */
    no_inputs_ = 1;
    if (P_ == 5 || P_ == 7) {
      const size_t edge = 2048 / alo_dtype_size(fdt[d]);
      for (size_t n = edge - 1; n <= edge + 1; n++) {
        case_allreduce(fdt[d], ALO_SUM, n, ALO_DIST_UNIFORM_PM1, 0, "at 2048 bytes");
        case_reduce(fdt[d], ALO_SUM, n, ALO_DIST_UNIFORM_PM1, P_ - 1, 0, "at 2048 bytes");
      }
    }
    if (big && P_ == 4 && d == 0) {
      const size_t edge = (size_t)(512u << 10) / 4 / alo_dtype_size(fdt[d]);
      for (size_t n = edge - 1; n <= edge + 1; n++)
        case_reduce_scatter(fdt[d], ALO_SUM, n, ALO_DIST_UNIFORM_PM1, 0, "at 512 KiB");
    }
    no_inputs_ = 0;
  }

  /* fp16 / bf16 through user-defined commutative operations on MPI_SHORT, as the reference
   * registers them: which order does the library apply such an operation in?  Inputs are the
   * generator's and are not repeated here. */
  const int hdt[2] = {ALO_F16, ALO_BF16};
  for (int d = 0; d < 2; d++) {
    const size_t nlong = 2048 / 2 + 8;
    case_allreduce(hdt[d], ALO_SUM, 16, ALO_DIST_UNIFORM_PM1, 0, "short message");
    case_allreduce(hdt[d], ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, 0, "long message");
    case_allreduce(hdt[d], ALO_PROD, nlong, ALO_DIST_UNIFORM_09_11, 0, "long message");
    const int roots[3] = {0, 1, P_ - 1};
    for (int k = 0; k < 3; k++) {
      if (k == 2 && roots[k] <= 1) break;
      case_reduce(hdt[d], ALO_SUM, 16, ALO_DIST_UNIFORM_PM1, roots[k], 0, "short message");
      case_reduce(hdt[d], ALO_SUM, nlong, ALO_DIST_UNIFORM_PM1, roots[k], 0, "long message");
      if (big) case_reduce(hdt[d], ALO_SUM, (size_t)(1u << 19) + 3, ALO_DIST_UNIFORM_PM1, roots[k], 0, "1 MiB and more");
    }
    case_reduce_scatter(hdt[d], ALO_SUM, 8, ALO_DIST_UNIFORM_PM1, 1, "short message");
    case_reduce_scatterv(hdt[d], ALO_SUM, ALO_DIST_UNIFORM_PM1, "uneven counts");
    if (big) {
      case_reduce_scatter(hdt[d], ALO_SUM, (size_t)(1u << 20) / (size_t)P_ / 2 + 64, ALO_DIST_UNIFORM_PM1, 0,
                          "long message");
      case_reduce_scatterv_long(hdt[d], ALO_SUM, ALO_DIST_UNIFORM_PM1, "uneven counts, long message");
    }
  }

  /* operand roles of the reduce-scatter orders and of the 16-bit user-defined operations: special values
   * planted in every position (long cases keep checksums; their inputs follow plant_specials_many) */
  if (P_ == 3 || P_ == 4 || P_ == 8) {
    for (int op = ALO_MIN; op <= ALO_MAX; op++) {
      case_reduce_scatter_x(ALO_F32, op, 24, ALO_DIST_UNIFORM_PM1, 1, 1, "specials");
      case_reduce_scatter_x(ALO_BF16, op, 24, ALO_DIST_UNIFORM_PM1, 1, 1, "specials");
      if (big)
        case_reduce_scatter_x(ALO_F32, op, (size_t)(1u << 20) / (size_t)P_ / 4 + 64, ALO_DIST_UNIFORM_PM1, 0, 1,
                              "specials");
      case_allreduce(ALO_BF16, op, 96, ALO_DIST_UNIFORM_PM1, 1, "specials");
      case_allreduce(ALO_F16, op, 96, ALO_DIST_UNIFORM_PM1, 1, "specials");
      case_allreduce(ALO_BF16, op, 2048 / 2 + 8, ALO_DIST_UNIFORM_PM1, 1, "specials");
    }
  }

  /* integer types: every op, full-range bits (logical ops see arbitrary
   * nonzero values as true) and {0,1} inputs. */
  if (P_ == 2 || P_ == 5) {
    for (int dt = ALO_I8; dt <= ALO_U64; dt++)
      for (int op = ALO_SUM; op <= ALO_BXOR; op++) {
        case_allreduce(dt, op, 12, ALO_DIST_FULLRANGE, 0, "");
        if (op >= ALO_LOR && op <= ALO_LXOR)
          case_allreduce(dt, op, 12, ALO_DIST_BOOL01, 0, "");
        if (op == ALO_SUM || op == ALO_PROD)
          case_allreduce(dt, op, 12, ALO_DIST_SMALLINT, 0, "");
      }
    case_reduce_scatter(ALO_I32, ALO_SUM, 8, ALO_DIST_FULLRANGE, 1, "");
    case_reduce_scatter(ALO_U64, ALO_BXOR, 8, ALO_DIST_FULLRANGE, 1, "");
    case_reduce(ALO_I32, ALO_SUM, 12, ALO_DIST_FULLRANGE, P_ - 1, 0, "");
    case_reduce(ALO_U8, ALO_LXOR, 12, ALO_DIST_FULLRANGE, 1, 0, "");
  }

  if (rank_ == 0) printf("\n]}\n");
  MPI_Finalize();
  return 0;
}
