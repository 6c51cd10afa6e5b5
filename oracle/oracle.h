/*
 * CPU oracle for the Aluminum combine hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is the checker, never the product: only the test-suite, the
 * smoke check and the bench's CPU-baseline leg may link or load it.  The GPU
 * library must never call into it.
 *
 * It restates, in plain C, the host-side arithmetic that the reference
 * performs for Al::Allreduce / Reduce_scatter / Allgather:
 *   - native C types are combined by the MPI library's predefined ops
 *     (reference: include/aluminum/mpi/utils.hpp:169-233 maps
 *     ReductionOperator -> MPI_SUM ... MPI_BXOR; the call sites are
 *     include/aluminum/mpi/allreduce.hpp:38-44 and
 *     include/aluminum/ht/allreduce.hpp:75-79).  The MPI library is a
 *     third-party dependency that is not part of the reference tree (this
 *     image: MPICH 3.3.2).  Its published per-element rules are
 *     `b[i] = OP(b[i], a[i])` with a = invec, b = inoutvec and
 *       SUM b+a, PROD b*a, MIN (b<a)?b:a, MAX (b>a)?b:a, LAND b&&a, LOR b||a,
 *       LXOR (b&&!a)||(!b&&a), BAND b&a, BOR b|a, BXOR b^a
 *     (for min/max a tie or a NaN on either side yields the invec element;
 *     checked against MPICH with NaN and signed-zero operands).
 *   - fp16 / bf16 are combined by the reference's own user ops
 *     (src/mpi_impl.cpp:61-145): widen both operands to fp32, one fp32
 *     operation, narrow round-to-nearest-even; min/max use std::min/std::max
 *     with (invec, inoutvec) argument order.
 *
 * Pin status (what checks each function against something other than itself):
 *   alo_step (int / f32 / f64), the TREE_BINOMIAL / TREE_RSG /
 *     TREE_RSG_SPREAD / TREE_DBL / TREE_HALV / PAIRWISE_DESC schedules: MPICH
 *     3.3.2 golden vectors in tests/golden (MPI_Allreduce, MPI_Reduce to the
 *     first, second and last rank, MPI_Reduce_scatter_block, MPI_Reduce_scatter
 *     with uneven counts, and their non-blocking in-place forms; the exact
 *     calls the reference makes; 2 to 64 ranks; fp32 / fp64 and, as
 *     user-defined operations on MPI_SHORT the way the reference registers
 *     them, fp16 / bf16), numpy closed forms for the order-free integer ops.
 *     The vectors with NaN, signed zeros and infinities planted in every
 *     operand position (3 to 64 ranks) pin which operand of every pair is
 *     the inoutvec, i.e. which one a tie or a NaN lets through, and how the
 *     blocking and the non-blocking calls cut a long message into blocks.
 *   alo_step (f16 / bf16): numpy float16 and torch bfloat16 arithmetic
 *     (library round-to-nearest-even narrowing), exhaustive over all 2^16
 *     values for widening, sampled + edge cases for narrowing.
 *   RANK_ASC / RING folds: brute-force Python loops on tiny inputs, exact
 *     integer-valued inputs, numpy cumulative folds.
 *   Ring RS+AG emulation: moved literally chunk by chunk here and compared
 *     with the closed-form rotated fold, plus invariants (all ranks equal,
 *     chunk size does not change a bit).
 *   alo_divide (avg): numpy / torch division of the same sums (float32,
 *     float64, float16 and bfloat16 arithmetic; Python integers for the
 *     truncating integer division), closed forms (equal contributions).  The
 *     rounding rule itself is this build's: the reference hands avg to NCCL
 *     and holds no vectors for it, so against the reference avg is "parity
 *     unpinned".
 *   Halo pack/unpack: numpy slicing of the same grid.
 *   NaN payload bits are outside every parity claim (tests compare NaN-ness).
 */
#ifndef ALO_ORACLE_H
#define ALO_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types.  Same numbering as the GPU library's dtype enum. */
enum {
  ALO_I8 = 0, ALO_U8, ALO_I16, ALO_U16, ALO_I32, ALO_U32, ALO_I64, ALO_U64,
  ALO_F16, ALO_BF16, ALO_F32, ALO_F64, ALO_NUM_DTYPES
};

/* Same numbering as Al::ReductionOperator (include/aluminum/base.hpp:103-105). */
enum {
  ALO_SUM = 0, ALO_PROD, ALO_MIN, ALO_MAX, ALO_LOR, ALO_LAND, ALO_LXOR,
  ALO_BOR, ALO_BAND, ALO_BXOR, ALO_AVG
};

/* Named combine orders.  `s` is the `start` argument of the calls below. */
enum {
  ALO_ORDER_RANK_ASC = 0,      /* ((x0 . x1) . x2) ...                        */
  ALO_ORDER_TREE_DBL = 1,      /* pairwise tree, distance 1,2,4,...; the lower
                                  rank of a pair keeps the result            */
  ALO_ORDER_TREE_HALV = 2,     /* pairwise tree, distance P/2,...,1, for rank
                                  s: of a pair, the rank on s's side keeps
                                  the result (recursive-halving
                                  reduce-scatter, block of rank s)           */
  ALO_ORDER_PAIRWISE_DESC = 3, /* ((x_s . x_{s-1}) . x_{s-2}) ... with wrap   */
  ALO_ORDER_RING = 4,          /* ((x_s . x_{s+1}) . x_{s+2}) ... with wrap,
                                  the running partial is the `in` operand    */
  ALO_ORDER_TREE_BINOMIAL = 5, /* binomial tree to rank s over the ranks
                                  counted from s with wrap (rooted reduce)   */
  ALO_ORDER_TREE_RSG = 6,      /* reduce-scatter + gather (MPI_Ireduce and
                                  MPI_Iallreduce of long messages): the tree
                                  of TREE_DBL, but which rank of a pair keeps
                                  the result depends on the element's block;
                                  s must be 0 (in alo_schedule: the block's
                                  owner among the survivors)                 */
  ALO_ORDER_TREE_RSG_SPREAD = 7 /* the same with the blocks that MPI_Reduce and
                                  MPI_Allreduce cut: what count / 2^k leaves
                                  over goes one element each to the first
                                  blocks, not to the last block              */
};

/* Input distributions of the counter-based generator. */
enum {
  ALO_DIST_UNIFORM_PM1 = 0,   /* uniform [-1, 1)                              */
  ALO_DIST_UNIFORM_09_11 = 1, /* uniform [0.9, 1.1)                           */
  ALO_DIST_UNIFORM_01 = 2,    /* uniform [0, 1)                               */
  ALO_DIST_FULLRANGE = 3,     /* integers: all bits random; floats: as PM1    */
  ALO_DIST_BOOL01 = 4,        /* values in {0, 1}                             */
  ALO_DIST_NORMAL = 5,        /* ~normal(0,1): sum of 12 uniforms minus 6     */
  ALO_DIST_SMALLINT = 6       /* integers in [-8, 7] (exactly summable)       */
};

size_t alo_dtype_size(int dtype);
/* 0 if `op` is defined for `dtype`: the pairs of the reference's MPI / HT path
 * (include/aluminum/mpi/utils.hpp:169-233) plus avg for every type (the
 * reference has it on its NCCL path only, include/aluminum/nccl_impl.hpp:176),
 * else nonzero. */
int alo_check_op(int dtype, int op);

/* Counter-based generator: element `idx` of stream `seed`. */
uint64_t alo_mix64(uint64_t seed, uint64_t idx);
void alo_fill(void *dst, size_t n, int dtype, int dist, uint64_t seed,
              uint64_t idx0);

/* 16-bit float conversions (round-to-nearest-even narrowing). */
uint16_t alo_f32_to_bf16(float f);
float alo_bf16_to_f32(uint16_t h);
uint16_t alo_f32_to_f16(float f);
float alo_f16_to_f32(uint16_t h);
void alo_f32_to_bf16_array(uint16_t *dst, const float *src, size_t n);
void alo_f32_to_f16_array(uint16_t *dst, const float *src, size_t n);
void alo_bf16_to_f32_array(float *dst, const uint16_t *src, size_t n);
void alo_f16_to_f32_array(float *dst, const uint16_t *src, size_t n);

/* One pairwise step with the MPI user-op signature:
 * inout[i] = in[i] OP inout[i].  Returns 0, or nonzero for an undefined
 * (dtype, op) pair. */
int alo_step(void *inout, const void *in, size_t n, int dtype, int op);

/* The division that ends an avg: x[i] = x[i] / ranks.  fp32 / fp64: IEEE
 * division; fp16 / bf16: widen, fp32 division, round-to-nearest-even
 * narrowing; integers: C division (truncation toward zero).  With op =
 * ALO_AVG every combine below is the sum in the named order (rounded or wrapped
 * after every step as for sum) followed by this division by P. */
int alo_divide(void *x, size_t n, int dtype, int ranks);

/* The schedule of a named order over P operands: `pairs` receives up to P-1
 * (inout_slot, in_slot) pairs, executed in sequence; the result ends in
 * slot *result.  Returns the number of pairs, or -1 on bad arguments. */
int alo_schedule(int P, int order, int start, int *pairs, int *result);

/* TREE_RSG (spread = 0) and TREE_RSG_SPREAD (spread = 1): the blocks the n
 * elements are cut into, and the survivor that ends up owning block k (what
 * alo_schedule takes as `start`). */
int alo_rsg_blocks(int P);
void alo_rsg_block(int P, size_t n, int k, int spread, size_t *lo, size_t *hi, int *owner);
/* The `start` a Reduce_scatter passes for the block that rank b receives. */
int alo_order_start(int order, int b);

/* out[i] = fold of in[0..P-1][i] in the named order.  `out` must not alias
 * an input. */
int alo_combine(void *out, const void *const *in, int P, size_t n, int dtype,
                int op, int order, int start);

/* As alo_combine, with the inputs produced on the fly: logical rank r's
 * element i is element (idx0 + i) of stream (seed_base + r) under `dist`. */
int alo_combine_generated(void *out, int P, size_t n, int dtype, int op,
                          int order, int start, int dist, uint64_t seed_base,
                          uint64_t idx0);

/* MPI_Reduce_scatter_block over P logical ranks: send[r] holds P*count
 * elements; recv[r] receives block r, folded in `order` with start = r
 * (layout: include/aluminum/ht/reduce_scatter.hpp:45-74). */
int alo_reduce_scatter(void *const *recv, const void *const *send, int P,
                       size_t count, int dtype, int op, int order);

/* MPI_Allgather over P logical ranks: recv[r][q*count + i] = send[q][i]
 * (layout: include/aluminum/ht/allgather.hpp:48-81). */
int alo_allgather(void *const *recv, const void *const *send, int P,
                  size_t count, int dtype);

/* MPI_Reduce_scatter with per-rank counts: send[r] holds sum(counts)
 * elements; recv[b] receives counts[b] elements, the fold of elements
 * [displ_b, displ_b + counts[b]) with start = b
 * (layout: include/aluminum/ht/reduce_scatterv.hpp:40-87). */
int alo_reduce_scatterv(void *const *recv, const void *const *send, int P,
                        const size_t *counts, int dtype, int op, int order);

/* MPI_Allgatherv: recv[r][displs[q] + i] = send[q][i], i < counts[q]
 * (layout: include/aluminum/ht/allgatherv.hpp:38-100). */
int alo_allgatherv(void *const *recv, const void *const *send, int P,
                   const size_t *counts, const size_t *displs, int dtype);

/* Segment s of an n-element buffer split over P ranks. */
void alo_ring_segment(size_t n, int P, int s, size_t *offset, size_t *len);

/* Literal emulation of a P-rank ring allreduce, in place on P buffers of n
 * elements: P-1 reduce-scatter steps then P-1 allgather steps, every
 * segment moved in chunks of `chunk_elems`.  At reduce-scatter step t rank r
 * receives segment (r-t-1) mod P from rank r-1 and applies
 * local = received OP local (received = invec, local = inoutvec, the operand
 * roles of src/mpi_impl.cpp:106-114). */
int alo_ring_allreduce(void *const *bufs, int P, size_t n, int dtype, int op,
                       size_t chunk_elems);
int alo_ring_reduce_scatter(void *const *bufs, int P, size_t n, int dtype,
                            int op, size_t chunk_elems);
int alo_ring_allgather(void *const *bufs, int P, size_t n, int dtype,
                       size_t chunk_elems);

/* Halo faces of a 3-D grid, x fastest.  Interior nx*ny*nz, halo width h on
 * all six sides, allocation (nx+2h)(ny+2h)(nz+2h).  Faces: 0 -x, 1 +x,
 * 2 -y, 3 +y, 4 -z, 5 +z.  A face excludes edges and corners; its buffer
 * keeps the grid's index order (x fastest).  pack reads the interior
 * boundary slab of the face, unpack writes the ghost slab of the face. */
size_t alo_halo_face_elems(size_t nx, size_t ny, size_t nz, size_t h, int face);
int alo_halo_pack(void *buf, const void *grid, size_t nx, size_t ny, size_t nz,
                  size_t h, int face, size_t elem_size);
int alo_halo_unpack(void *grid, const void *buf, size_t nx, size_t ny,
                    size_t nz, size_t h, int face, size_t elem_size);

/* Order-dependent 64-bit checksum of a byte buffer. */
uint64_t alo_checksum(const void *buf, size_t nbytes);

/* Number of OpenMP threads the array functions use. */
int alo_num_threads(void);
void alo_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
