/*
 * aluminum_amd - MI355X (gfx950) on-device combine engine for the
 * Al::Allreduce / Reduce_scatter / Allgather hot path of Aluminum.
 *
 * C ABI.  No C++ or HIP types cross this boundary: streams are passed as
 * `void *` (a hipStream_t; NULL is the default stream), buffers as device
 * pointers.  Every call that takes a stream only enqueues work on it and
 * returns (the set-up calls alamd_reserve_scratch / alamd_release_scratch
 * aside; the one collective that may need memory of the library's own says so:
 * alamd_reduce_scatterv); buffers are caller-owned and must stay valid until
 * the stream has passed the call (reference contract: docs/comm.rst:18,
 * docs/index.rst:33-40).
 * Calls return ALAMD_OK or a small positive status code; the message of
 * the last error on the calling thread is alamd_last_error().  The library is
 * thread-compatible: concurrent calls are fine as long as they do not share a
 * stream or output buffers.
 *
 * The reference has no C ABI; its boundary is a compile-time backend policy
 * class (include/aluminum/ht_impl.hpp:125-1111).  The header-only C++ shim
 * include/aluminum_amd/Al.hpp maps that class interface onto the functions
 * below, turning error codes into Al::al_exception.
 *
 * Entry points that replace nothing in the reference and exist for tests and
 * benchmarks only (input generator, the 16-bit float conversions on their own)
 * are declared in aluminum_amd_support.h, not here.
 */
#ifndef ALUMINUM_AMD_H
#define ALUMINUM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ALAMD_VERSION_MAJOR 0
#define ALAMD_VERSION_MINOR 1

/* Largest number of logical ranks one call can combine, under every order. */
#define ALAMD_MAX_RANKS 64

typedef enum {
  ALAMD_OK = 0,
  ALAMD_ERR_INVALID_ARG = 1,     /* null pointer, bad count, bad rank count        */
  ALAMD_ERR_UNSUPPORTED_OP = 2,  /* "Reduction operator not supported"
                                    (include/aluminum/mpi/utils.hpp:192-194)       */
  ALAMD_ERR_UNSUPPORTED_TYPE = 3,
  ALAMD_ERR_INVALID_ALGO = 4,    /* "Invalid algorithm" (ht_impl.hpp:156-158)      */
  ALAMD_ERR_OVERLAP = 5,         /* partially overlapping buffers
                                    (include/aluminum/debug_helpers.hpp:117-135)   */
  ALAMD_ERR_HIP = 6,             /* a HIP runtime call failed                      */
  ALAMD_ERR_TIMEOUT = 7,         /* a bounded wait expired                         */
  ALAMD_ERR_UNSUPPORTED = 8      /* feature not available on this device           */
} alamd_status;

/* Element types: the arithmetic types of mpi::TypeMap<T>
 * (include/aluminum/mpi/utils.hpp:43-67) by width and signedness, plus the
 * two 16-bit float types of include/aluminum/datatypes.hpp:37-56. */
typedef enum {
  ALAMD_I8 = 0, ALAMD_U8 = 1, ALAMD_I16 = 2, ALAMD_U16 = 3, ALAMD_I32 = 4,
  ALAMD_U32 = 5, ALAMD_I64 = 6, ALAMD_U64 = 7, ALAMD_F16 = 8, ALAMD_BF16 = 9,
  ALAMD_F32 = 10, ALAMD_F64 = 11, ALAMD_NUM_DTYPES = 12
} alamd_dtype;

/* Numerically identical to Al::ReductionOperator
 * (include/aluminum/base.hpp:103-105), so the C++ shim casts.
 * avg (the reference has it on its NCCL backend only,
 * include/aluminum/nccl_impl.hpp:176; its MPI and host-transfer backends throw,
 * include/aluminum/mpi/utils.hpp:192-194) is defined for every type as the sum
 * in the call's order, rounded or wrapped after every step exactly as for
 * ALAMD_SUM, followed by one division by the number of ranks P in the element
 * type's own arithmetic: IEEE division for fp32 / fp64; for fp16 / bf16 the
 * sum is widened, divided in fp32 and narrowed round-to-nearest-even; for the
 * integer types C division, which truncates toward zero.  Parity unpinned: the
 * reference holds no values for avg, and the library its NCCL backend hands it
 * to may scale every contribution by 1/P before summing instead, so float
 * results need not agree with Al::NCCLBackend bit for bit. */
typedef enum {
  ALAMD_SUM = 0, ALAMD_PROD = 1, ALAMD_MIN = 2, ALAMD_MAX = 3, ALAMD_LOR = 4,
  ALAMD_LAND = 5, ALAMD_LXOR = 6, ALAMD_BOR = 7, ALAMD_BAND = 8, ALAMD_BXOR = 9,
  ALAMD_AVG = 10
} alamd_op;

/* Named combine orders.  One pairwise step is always
 *   result = OP(inout, in)
 * with the operand roles of an MPI reduction function (for fp16 / bf16:
 * src/mpi_impl.cpp:61-145); the order names which operand plays which role
 * and in what sequence the P contributions meet.
 *   RANK_ASC       acc = x0; acc = step(in = x_k, inout = acc), k = 1..P-1
 *   PAIRWISE_DESC  acc = x_s; acc = step(in = x_{s-k}, inout = acc)  (wrap)
 *   RING           acc = x_s; acc = step(in = acc, inout = x_{s+k})  (wrap)
 *   TREE_BINOMIAL  binomial tree to rank s: with y_i = x_{(s+i) mod P},
 *                  distance d = 1,2,4..: y_i = step(in = y_{i+d}, inout = y_i)
 *                  for every i that is a multiple of 2d with i+d < P
 *   TREE_DBL       the first 2*(P - 2^k) ranks fold pairwise
 *                  (step(in = x_{2j}, inout = x_{2j+1})), the 2^k survivors
 *                  then pair at distance 1,2,4,..., the lower one keeping the
 *                  result (the inout operand)
 *   TREE_HALV      the same pre-fold, survivors pair at distance 2^k/2,...,1;
 *                  of a pair, the survivor on the side of rank s keeps the
 *                  result: the order in which a recursive-halving
 *                  reduce-scatter makes the block that rank s receives
 *   TREE_RSG       reduce-scatter by recursive halving of the data, then
 *                  gather: the first 2*(P - 2^k) ranks fold pairwise, the even
 *                  one keeping the result (step(in = x_{2j+1}, inout = x_{2j}));
 *                  the survivors pair at distance 1,2,4,... as under TREE_DBL,
 *                  but which one of a pair keeps the result depends on where
 *                  the element lies: the count elements are cut into 2^k blocks
 *                  of count / 2^k (the last one takes the remainder), block b
 *                  ends up on survivor bit_reverse(b), and at distance d the
 *                  survivor whose bit d equals that survivor's bit d keeps.
 *                  For sum and prod this gives the bits of TREE_DBL; it differs
 *                  where a float min / max meets a tie (+0 / -0) or a NaN.
 *   TREE_RSG_SPREAD  the same, but what count / 2^k leaves over goes one
 *                  element each to the first blocks instead of to the last one.
 * Which of two operands is the inout one only shows in float min / max (a tie
 * or a NaN lets the in operand through); every other result depends on the
 * shape of the tree alone.
 * With MPICH 3.3.2 on one host the reference's MPI and host-transfer backends
 * produce: Allreduce and Reduce of native types - TREE_BINOMIAL with s = root
 * (Allreduce: 0) up to 2048 bytes or when count < 2^k; above that, whatever the
 * root, TREE_RSG where the backend calls MPI_Ireduce / MPI_Iallreduce (the
 * host-transfer backend always, the MPI backend in its non-blocking calls) and
 * TREE_RSG_SPREAD where it calls MPI_Reduce / MPI_Allreduce (the MPI backend's
 * blocking calls); of fp16 / bf16, which are user-defined operations to the MPI
 * library - TREE_BINOMIAL at every size; Reduce_scatter, with equal or unequal
 * counts - TREE_HALV with s = receiving rank below 512 KiB in total,
 * PAIRWISE_DESC with s = receiving rank from there on. */
typedef enum {
  ALAMD_ORDER_RANK_ASC = 0,
  ALAMD_ORDER_TREE_DBL = 1,
  ALAMD_ORDER_TREE_HALV = 2,
  ALAMD_ORDER_PAIRWISE_DESC = 3,
  ALAMD_ORDER_RING = 4,
  ALAMD_ORDER_TREE_BINOMIAL = 5,
  ALAMD_ORDER_TREE_RSG = 6,
  ALAMD_ORDER_TREE_RSG_SPREAD = 7
} alamd_order;

/* ---- library ---------------------------------------------------------- */

/* Text of the last error raised on the calling thread ("" if none). */
const char *alamd_last_error(void);
/* major * 100 + minor */
int alamd_version(void);
/* Bytes per element, 0 for an unknown dtype. */
size_t alamd_dtype_size(int dtype);
/* ALAMD_OK if `op` is defined for `dtype`
 * (include/aluminum/mpi/utils.hpp:169-269: sum, prod, min, max for every type;
 * MPI defines the logical and bitwise ops for integers only; avg for every
 * type, see alamd_op). */
int alamd_check_op(int dtype, int op);
/* Set-up for the current device, once per device (calling it again is cheap):
 * checks that the device is a gfx950, caches its compute-unit count, allocates
 * one line of pinned host memory (where a bounded wait that gives up leaves
 * its mark, see alamd_reduce_scatterv_wait_expired), looks up the address of
 * the fixed scratch array of alamd_reduce_scatterv_noalloc and creates the
 * event that guards it.  Required before alamd_reduce_scatterv_noalloc, which
 * may not allocate; every other entry point works without it.  (Replaces
 * internal::cuda::init, src/cuda/cuda.cpp:52-78.) */
int alamd_init(void);

/* The order (and its start rank) under which the reference's result comes
 * about for a collective over P ranks when its MPI library is MPICH 3.3.2 and
 * all ranks share one host - what an `automatic` algorithm should pick to give
 * the reference's bits.  The reference hands the call to MPI_(I)allreduce,
 * MPI_(I)reduce, MPI_(I)reduce_scatter_block and MPI_(I)reduce_scatter
 * (include/aluminum/mpi/allreduce.hpp:38-44, mpi/reduce.hpp:41-49,
 * mpi/reduce_scatter.hpp:40-46, include/aluminum/ht/allreduce.hpp:76-79,
 * ht/reduce.hpp:72-82, ht/reduce_scatter.hpp:71-74, ht/reduce_scatterv.hpp:76-79);
 * the table was read off that library's results for 2 to 64 ranks.
 * ALAMD_COLL_ALLREDUCE and ALAMD_COLL_REDUCE stand for the non-blocking MPI
 * calls (every call of the host-transfer backend), the _BLOCKING ones for
 * MPI_Allreduce and MPI_Reduce (the MPI backend's blocking calls), which differ
 * in how a long message is cut into blocks; a reduce-scatter is the same in both.
 * `count`: elements per rank for an allreduce or reduce, elements in a whole
 * send buffer for ALAMD_COLL_REDUCE_SCATTER (with equal or unequal counts).
 * `root` is ignored except for a reduce.  *start is what alamd_combine takes;
 * alamd_reduce_scatter(v) add the receiving rank themselves. */
typedef enum {
  ALAMD_COLL_ALLREDUCE = 0,
  ALAMD_COLL_REDUCE = 1,
  ALAMD_COLL_REDUCE_SCATTER = 2,
  ALAMD_COLL_ALLREDUCE_BLOCKING = 3,
  ALAMD_COLL_REDUCE_BLOCKING = 4
} alamd_collective;
int alamd_reference_order(int collective, int P, size_t count, int dtype, int root, int *order, int *start);

/* ---- combine: the element-wise fold of P rank contributions ----------- */

/* outs[j][i] = fold over r of ins[r][i], i in [0, count), for each of the
 * `nout` output buffers.  This is the arithmetic the reference delegates to
 * MPI_Iallreduce on a pinned host copy
 * (include/aluminum/ht/allreduce.hpp:41-79) or to MPI_Allreduce
 * (include/aluminum/mpi/allreduce.hpp:38-44); nout = 1 is a Reduce
 * (include/aluminum/ht/reduce.hpp:72-82), nout = P an Allreduce over P
 * logical ranks.  An output may be identical to an input (in-place), but
 * must not overlap one partially.  `start` is the rank s of the orders that
 * have one and must be 0 otherwise.  Here and in every entry point below a
 * buffer must be aligned to its element type (ALAMD_ERR_INVALID_ARG if not);
 * no wider alignment is needed.
 * Outside every parity claim: the payload bits of a NaN result. */
int alamd_combine(void *const *outs, int nout, const void *const *ins, int P,
                  size_t count, int dtype, int op, int order, int start,
                  void *stream);

/* Reduce_scatter over P logical ranks: sends[r] holds P*count elements;
 * recvs[b] receives count elements, the fold of block b of every sends[r],
 * with start = b under PAIRWISE_DESC, RING and TREE_HALV (TREE_BINOMIAL: 0;
 * TREE_RSG, TREE_RSG_SPREAD: every block is a message of its own).  In-place form
 * (recvs[b] == sends[b]) puts the result at the start of the buffer.
 * Replaces MPI_Ireduce_scatter_block on the host copy
 * (include/aluminum/ht/reduce_scatter.hpp:45-74; layout docs/comm.rst:284-285). */
int alamd_reduce_scatter(void *const *recvs, const void *const *sends, int P,
                         size_t count, int dtype, int op, int order,
                         void *stream);

/* Allgather over P logical ranks: recvs[r][q*count + i] = sends[q][i].
 * In-place form: sends[q] == recvs[q] + q*count elements
 * (include/aluminum/ht/allgather.hpp:48-81; docs/comm.rst:152). */
int alamd_allgather(void *const *recvs, const void *const *sends, int P,
                    size_t count, int dtype, void *stream);

/* Reduce_scatterv: sends[r] holds sum(counts) elements; recvs[b] receives
 * counts[b] elements, the fold of elements [displ_b, displ_b + counts[b]) of
 * every sends[r], displ_b = counts[0] + ... + counts[b-1], with start = b as
 * for alamd_reduce_scatter.  In-place form (recvs[b] == sends[b]) puts the
 * result at the start of the buffer; any counts are accepted, as by the
 * reference.  A block that is in place and starts fewer elements into its own
 * buffer than it is long is read and overwritten at a displacement: in two
 * launches no longer than the displacement where they suffice, else in one
 * launch whose workgroups order themselves through a ticket counter and one
 * flag per tile in device scratch memory of the library's own, kept per
 * stream.  That scratch is the one thing a collective here may have to
 * allocate: the first such launch on a stream calls hipMalloc (4 bytes per
 * 4 KiB of the block, at least 256 KiB) unless alamd_reserve_scratch has been
 * called for the stream; a stream that is being captured into a graph never
 * allocates, and the call then fails with ALAMD_ERR_INVALID_ARG if nothing was
 * reserved.  Everything the launch needs cleared is cleared by a small kernel
 * on the stream itself.
 * Replaces MPI_Ireduce_scatter on the host copy
 * (include/aluminum/ht/reduce_scatterv.hpp:40-87). */
int alamd_reduce_scatterv(void *const *recvs, const void *const *sends, int P,
                          const size_t *counts, int dtype, int op, int order,
                          void *stream);

/* Set-up calls, not stream-ordered work.  alamd_reserve_scratch makes sure that
 * `stream` (on the current device) owns scratch for in-place Reduce_scatterv
 * blocks of up to max_block_bytes that overlap their own input, allocating it
 * now if need be, so that no later alamd_reduce_scatterv on that stream
 * allocates and the call can be captured into a graph.  alamd_release_scratch
 * synchronises the stream and frees what it holds (call it before destroying a
 * stream whose scratch should not outlive it).  No counterpart in the
 * reference, whose host-transfer backend draws staging memory from a pool
 * (include/aluminum/mempool.hpp) inside the call. */
int alamd_reserve_scratch(void *stream, size_t max_block_bytes);
int alamd_release_scratch(void *stream);

/* The waits inside a chained in-place launch (see alamd_reduce_scatterv) are
 * bounded, so that a device that loses a workgroup cannot hang the stream; a
 * wait that gives up lets its workgroup go on, and the block's result is then
 * not valid.  This returns 1, once, if that has happened since the last call
 * (meaningful once the streams concerned have been synchronised); the next
 * alamd_reduce_scatterv / _noalloc call reports it too, with
 * ALAMD_ERR_TIMEOUT, and does nothing else.  No counterpart in the reference,
 * whose collectives wait without bound. */
int alamd_reduce_scatterv_wait_expired(void);

/* alamd_reduce_scatterv for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same arguments, same
 * results, and no hipMalloc, hipFree or other allocating call is made: the
 * ticket counter and tile flags that an in-place block needs when it overlaps
 * its own input (see alamd_reduce_scatterv) live in a fixed array of
 * ALAMD_NOALLOC_SCRATCH_BYTES that is part of the library's code object (every
 * device the library runs on holds its copy until the process ends).  Limit:
 * such a block may be at most ALAMD_NOALLOC_MAX_BLOCK_BYTES long unless it
 * starts at least a 32nd of its length into its buffer (then up to 32 plain
 * launches do; ALAMD_ERR_INVALID_ARG otherwise; blocks that do not overlap their own
 * input, and separate receive buffers, have no limit).  alamd_init must have
 * run on the device (ALAMD_ERR_INVALID_ARG otherwise): it looks the array up.
 * All calls on one device share the array, which keeps the last call's
 * contents (every call clears what it uses): calls that overlap in time on one
 * device would race, so keep them on one stream.  A call made on another
 * stream while the last chained launch that used the array is still running is
 * refused (ALAMD_ERR_INVALID_ARG); launches recorded into a graph are not
 * tracked that way, and what runs beside a replay is the caller's to order. */
#define ALAMD_NOALLOC_SCRATCH_BYTES ((size_t)1 << 20)
#define ALAMD_NOALLOC_MAX_BLOCK_BYTES (((ALAMD_NOALLOC_SCRATCH_BYTES - 256) / 4) * 4096)
int alamd_reduce_scatterv_noalloc(void *const *recvs, const void *const *sends, int P,
                                  const size_t *counts, int dtype, int op, int order,
                                  void *stream);

/* Allgatherv: recvs[r][displs[q] + i] = sends[q][i], i < counts[q].
 * In-place form: sends[q] == recvs[q] + displs[q] elements
 * (include/aluminum/ht/allgatherv.hpp:38-100). */
int alamd_allgatherv(void *const *recvs, const void *const *sends, int P,
                     const size_t *counts, const size_t *displs, int dtype,
                     void *stream);

/* ---- ring reduce-scatter + allgather over P logical ranks ------------- */

typedef enum {
  /* one launch per ring step; every byte a real ring moves is moved */
  ALAMD_RING_STEPWISE = 0,
  /* each segment is folded in registers in ring order, written once and
   * (allreduce) copied once to every other rank: same bits, fewer bytes */
  ALAMD_RING_FUSED = 1
} alamd_ring_mode;

/* In place on bufs[0..P-1], each `count` elements.  Segment s is
 * [s*q + min(s, m), ...) with q = count / P, m = count % P, and the first m
 * segments one element longer.  Reduce-scatter step t = 0..P-2: rank r
 * receives segment (r-t-1) mod P from rank r-1 and applies
 * local = step(in = received, inout = local); afterwards rank r holds the
 * fully reduced segment (r+1) mod P.  Allgather step t: rank r receives
 * segment (r-t) mod P from rank r-1.  Segments move in chunks of
 * `chunk_bytes` (a multiple of the element size; the chunk is the unit of
 * work of one workgroup pass and does not change any bit of the result).
 * The reference names the algorithm (mpi_impl.hpp:83-90 `mpi_ring`) but
 * carries no implementation of it. */
int alamd_ring_allreduce(void *const *bufs, int P, size_t count, int dtype,
                         int op, size_t chunk_bytes, int mode, void *stream);
/* The same allreduce with the contributions read from sends[r] (each identical
 * to recvs[r] or overlapping no receive buffer), as Al::Allreduce's form with
 * separate send and receive buffers (include/Al.hpp:118-152).  The fused mode
 * reads them where they are; the step-by-step mode copies each into its
 * receive buffer first. */
int alamd_ring_allreduce_from(void *const *recvs, const void *const *sends, int P,
                              size_t count, int dtype, int op, size_t chunk_bytes,
                              int mode, void *stream);
int alamd_ring_reduce_scatter(void *const *bufs, int P, size_t count, int dtype,
                              int op, size_t chunk_bytes, int mode, void *stream);
int alamd_ring_allgather(void *const *bufs, int P, size_t count, int dtype,
                         size_t chunk_bytes, void *stream);
/* Offset and length (in elements) of ring segment s. */
int alamd_ring_segment(size_t count, int P, int s, size_t *offset, size_t *len);

/* ---- halo faces -------------------------------------------------------- */

/* A 3-D grid, x fastest: interior dims[0] x dims[1] x dims[2], halo width
 * `halo` on all six sides, allocation (dims[d] + 2*halo) per axis.  Faces:
 * 0 -x, 1 +x, 2 -y, 3 +y, 4 -z, 5 +z; a face excludes edges and corners and
 * its buffer keeps the grid's index order (x fastest).  pack copies the
 * interior boundary slab of each selected face into its send buffer; unpack
 * copies each receive buffer into the ghost slab of its face.  `face_mask`
 * selects faces (bit f); bufs[f] is ignored for unselected faces.  All
 * selected faces are handled by one launch.  These produce the contiguous
 * buffers that Al::ext::Put moves (include/aluminum/mpi_cuda/rma_ipc.hpp:287-301,
 * test/test_rma_halo_exchange.cpp:171-197); the reference itself has no
 * strided faces. */
int alamd_halo_pack(void *const bufs[6], const void *grid, const size_t dims[3],
                    size_t halo, size_t elem_size, unsigned face_mask, void *stream);
int alamd_halo_unpack(void *grid, const void *const bufs[6], const size_t dims[3],
                      size_t halo, size_t elem_size, unsigned face_mask, void *stream);
/* Elements in the buffer of `face`. */
size_t alamd_halo_face_elems(const size_t dims[3], size_t halo, int face);

/* ---- stream flags ------------------------------------------------------ */

/* One int32 synchronisation word in pinned, device-mapped host memory on its
 * own 128-byte line, taken from a pool of pinned slabs that live until the
 * process ends (include/aluminum/cuda/sync_memory.hpp:46-63).  Destroy a flag
 * only when no stream can still wait on it or write to it. */
typedef struct alamd_flag alamd_flag;

typedef enum {
  ALAMD_FLAG_AUTO = 0,   /* stream memory operation if the device has them  */
  ALAMD_FLAG_MEMOP = 1,  /* hipStreamWaitValue32 / hipStreamWriteValue32    */
  ALAMD_FLAG_KERNEL = 2  /* single-lane spin kernel / store kernel          */
} alamd_flag_mode;

int alamd_flag_create(alamd_flag **flag, int32_t initial);
int alamd_flag_destroy(alamd_flag *flag);
/* Host address of the word. */
volatile int32_t *alamd_flag_host_ptr(alamd_flag *flag);
/* 1 if stream memory operations are usable on the current device
 * (internal::cuda::stream_memory_operations_supported, src/cuda/cuda.cpp:52-88). */
int alamd_stream_memops_supported(void);
/* Blocks `stream` until the word equals `value`
 * (launch_wait_kernel / spin_wait_kernel, src/cuda/helper_kernels.cu:42-71;
 * GPUWait::wait, src/cuda/gpu_wait.cpp:64-70).  In ALAMD_FLAG_KERNEL mode
 * `max_spins` bounds the number of polls (0 = unbounded, as the reference);
 * a wait that gives up stores 1 to the word returned by
 * alamd_flag_timed_out(). */
int alamd_stream_wait_flag(void *stream, alamd_flag *flag, int32_t value,
                           int mode, uint64_t max_spins);
/* Has `stream` store `value` into the word when it gets there
 * (GPUStatusFlag::record, src/cuda/gpu_status_flag.cpp:65-82). */
int alamd_stream_write_flag(void *stream, alamd_flag *flag, int32_t value, int mode);
/* Host-side atomic store / load (GPUWait::signal, src/cuda/gpu_wait.cpp:72-74;
 * GPUStatusFlag::query, src/cuda/gpu_status_flag.cpp:84-87). */
int alamd_flag_signal(alamd_flag *flag, int32_t value);
int32_t alamd_flag_query(alamd_flag *flag);
/* 1 if a bounded kernel wait on this flag has expired since creation. */
int alamd_flag_timed_out(alamd_flag *flag);

/* ---- plain copy ---------------------------------------------------------- */

/* dst[i] = src[i] for `bytes` bytes on `stream`, with the load / store path of
 * the combine kernels (any alignment; the ranges must not overlap).  This is
 * what a Put between two logical ranks of one GPU is
 * (ConnectionSelf::put, include/aluminum/mpi_cuda/rma_self.hpp:57-70, there a
 * cudaMemcpyAsync), and the copy that precedes an out-of-place ring allreduce;
 * it is also the practical 1-read + 1-write bandwidth ceiling that counter
 * readings of the other kernels are scaled by. */
int alamd_copy(void *dst, const void *src, size_t bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif
