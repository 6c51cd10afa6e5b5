// Ring reduce-scatter + allgather over P logical ranks held in one GPU's HBM.
//
// STEPWISE: one launch per ring step.  In reduce-scatter step t every rank r
// (blockIdx.y) folds the segment it "receives" from rank r-1 into its own
// copy; in allgather step t it copies the segment.  A segment is worked
// through chunk by chunk: a chunk is a run of tiles, no tile crosses a chunk
// boundary.
// FUSED: the fold kernels walk each segment once in ring order; an allreduce
// then spreads every folded segment from its owner to the other ranks.
#include "alamd_dispatch.h"
#include "alamd_tile.h"

namespace alamd {

namespace {

// (A ring step keeps tiles of 256 threads x 8 vectors: on C3, whose segments the previous step has just
// written, the streaming shape of the fold kernels gains nothing - 1358 us per allreduce against 1349.)
constexpr int kThreads = 256;

struct RingParams {
  char *buf[ALAMD_MAX_RANKS];
  unsigned long long seg_base, seg_rem;
  unsigned long long chunk_accesses;  // 128-bit vectors per chunk
  int P;
  int t;              // ring step
  unsigned tiles_per_chunk;  // workgroups (tiles) per chunk
  Divisor div;        // avg: the number of ranks as a divisor
};

__device__ __forceinline__ void ring_seg(const RingParams &p, int seg, size_t &off, size_t &len) {
  const unsigned long long sg = (unsigned long long)seg;
  off = sg * p.seg_base + (sg < p.seg_rem ? sg : p.seg_rem);
  len = p.seg_base + (sg < p.seg_rem ? 1u : 0u);
}

// A chunk is a run of tiles_per_chunk tiles; no tile crosses a chunk boundary.
// OP < 0: plain copy (allgather step).  FIN: the last reduce-scatter step of an
// avg, which ends with the division by the number of ranks.
constexpr int kRingU = 8;
template <typename T, int OP, bool FIN>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 2)))
ring_step_vec_kernel(const RingParams p) {
  using TL = Tile<kRingU, kThreads>;
  const TL tl;
  const int P = p.P, r = blockIdx.y;
  int seg = (OP >= 0 ? r - p.t - 1 : r - p.t) % P;
  if (seg < 0) seg += P;
  const int from = r == 0 ? P - 1 : r - 1;
  size_t off, len;
  ring_seg(p, seg, off, len);
  char *local = p.buf[r] + off * sizeof(T);
  const char *recv = p.buf[from] + off * sizeof(T);
  constexpr size_t N = 16 / sizeof(T);
  const size_t head = head_elems<T>(local, recv, len);
  const size_t vlen = len - head;
  // the head elements and the vlen % N elements after the last whole vector, one per thread of the
  // segment's first workgroup
  if (blockIdx.x == 0 && threadIdx.x < head + vlen % N) {
    const size_t e = threadIdx.x < head ? threadIdx.x : (vlen / N) * N + threadIdx.x;
    const T a = ld_elem<T>(recv + e * sizeof(T));
    if constexpr (OP >= 0) {
      const T b = ld_elem<T>(local + e * sizeof(T));
      T v = Step<T, (OP >= 0 ? OP : 0)>::apply(a, b);
      if constexpr (FIN) v = finish_elem<T, OP>(v, p.div);
      st_elem<T>(local + e * sizeof(T), v);
    } else {
      st_elem<T>(local + e * sizeof(T), a);
    }
  }
  local += head * sizeof(T);
  recv += head * sizeof(T);
  const size_t seg_bytes = (vlen / N) * 16;  // whole vectors
  const size_t chunk_bytes = (size_t)p.chunk_accesses * 16;
  const size_t c = blockIdx.x / p.tiles_per_chunk, ti = blockIdx.x % p.tiles_per_chunk;
  const size_t c0 = c * chunk_bytes;
  if (c0 >= seg_bytes) return;
  const size_t c1 = c0 + chunk_bytes < seg_bytes ? c0 + chunk_bytes : seg_bytes;
  const size_t tb = c0 + ti * TL::BYTES;
  if (tb >= c1) return;
  const int nrec = c1 - tb > TL::BYTES ? (int)TL::BYTES : (int)(c1 - tb);
  const auto rr = TL::rsrc(recv + tb, nrec);
  const auto rl = TL::rsrc(local + tb, nrec);
  u32x4 a[kRingU], b[kRingU];
#pragma unroll
  for (int u = 0; u < kRingU; ++u) a[u] = tl.load(rr, u);
  if constexpr (OP >= 0) {
#pragma unroll
    for (int u = 0; u < kRingU; ++u) b[u] = tl.load(rl, u);
#pragma unroll
    for (int u = 0; u < kRingU; ++u) {
      u32x4 v = step_vec<T, (OP >= 0 ? OP : 0)>(a[u], b[u]);
      if constexpr (FIN) v = finish_vec<T, OP>(v, p.div);
      tl.store(rl, u, v);
    }
  } else {
#pragma unroll
    for (int u = 0; u < kRingU; ++u) tl.store(rl, u, a[u]);
  }
}

struct RingPlan {
  RingParams rp;
  unsigned gx;
  size_t es;
};

int make_plan(RingPlan &pl, void *const *bufs, int P, size_t count, int dtype, size_t chunk_bytes) {
  if (P < 1 || P > ALAMD_MAX_RANKS)
    return set_error(ALAMD_ERR_INVALID_ARG, "number of ranks %d outside [1, %d]", P, ALAMD_MAX_RANKS);
  pl.es = alamd_dtype_size(dtype);
  if (pl.es == 0) return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);
  if (!bufs) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  if (chunk_bytes == 0 || chunk_bytes % pl.es != 0)
    return set_error(ALAMD_ERR_INVALID_ARG, "chunk size %zu is not a positive multiple of the element size", chunk_bytes);
  const size_t bytes = count * pl.es;
  for (int r = 0; r < ALAMD_MAX_RANKS; ++r) pl.rp.buf[r] = nullptr;
  for (int r = 0; r < P; ++r) {
    if (!bufs[r] && count) return set_error(ALAMD_ERR_INVALID_ARG, "buffer %d is null", r);
    pl.rp.buf[r] = static_cast<char *>(bufs[r]);
    if (!aligned_to(bufs[r], pl.es))
      return set_error(ALAMD_ERR_INVALID_ARG, "buffer %d is not aligned to its element type", r);
    for (int k = 0; k < r; ++k) {
      const uintptr_t x = reinterpret_cast<uintptr_t>(bufs[r]), y = reinterpret_cast<uintptr_t>(bufs[k]);
      if (count && x < y + bytes && y < x + bytes)
        return set_error(ALAMD_ERR_OVERLAP, "rank buffers %d and %d overlap", k, r);
    }
  }
  pl.rp.P = P;
  pl.rp.div = make_divisor(P);
  pl.rp.seg_base = count / (size_t)P;
  pl.rp.seg_rem = count % (size_t)P;
  pl.rp.t = 0;
  // a chunk is a whole number of 128-bit vectors (chunking never changes a bit: the step is element-wise)
  size_t cn = chunk_bytes / 16;
  if (cn < 1) cn = 1;
  pl.rp.chunk_accesses = cn;
  const size_t seg_max = pl.rp.seg_base + (pl.rp.seg_rem ? 1 : 0);
  const size_t n = seg_max / (16 / pl.es);  // whole vectors of the longest segment
  size_t nchunks = (n + cn - 1) / cn;
  if (nchunks < 1) nchunks = 1;
  const size_t tile_vecs = Tile<kRingU, kThreads>::BYTES / 16;
  const size_t tpc = ((cn < n ? cn : (n ? n : 1)) + tile_vecs - 1) / tile_vecs;
  if (nchunks * tpc * kThreads > 0xffffffffull)
    return set_error(ALAMD_ERR_INVALID_ARG, "too many chunks for one launch");
  pl.rp.tiles_per_chunk = (unsigned)tpc;
  pl.gx = (unsigned)(nchunks * tpc);
  return ALAMD_OK;
}

// last: the final reduce-scatter step, after which every rank holds its fully reduced segment
int launch_step(const RingPlan &pl, int dtype, int op, bool reduce, bool last, hipStream_t stream) {
  const dim3 grid(pl.gx, pl.rp.P, 1), block(kThreads, 1, 1);
  if (!reduce) {
    // a copy only needs the element size
    void (*kern)(const RingParams) = nullptr;
    switch (pl.es) {
    case 1: kern = ring_step_vec_kernel<uint8_t, -1, false>; break;
    case 2: kern = ring_step_vec_kernel<uint16_t, -1, false>; break;
    case 4: kern = ring_step_vec_kernel<uint32_t, -1, false>; break;
    default: kern = ring_step_vec_kernel<uint64_t, -1, false>; break;
    }
    hipLaunchKernelGGL(kern, grid, block, 0, stream, pl.rp);
    ALAMD_HIP(hipGetLastError());
    return ALAMD_OK;
  }
  return dispatch_any(dtype, op, [&](auto tt, auto ot) -> int {
    using T = typename decltype(tt)::type;
    constexpr int OP = decltype(ot)::value;
    void (*kern)(const RingParams) = ring_step_vec_kernel<T, OP, false>;
    if constexpr (OP == ALAMD_AVG) {
      if (last) kern = ring_step_vec_kernel<T, OP, true>;
    }
    hipLaunchKernelGGL(kern, grid, block, 0, stream, pl.rp);
    ALAMD_HIP(hipGetLastError());
    return ALAMD_OK;
  });
}

// ins[r] is bufs[r] itself (in place) or a buffer that overlaps none of bufs.
int fused_fold(void *const *bufs, const void *const *ins, int P, size_t count, int dtype, int op, bool all,
               hipStream_t stream) {
  FoldParams fp;
  for (int r = 0; r < ALAMD_MAX_RANKS; ++r) {
    fp.in[r] = r < P ? static_cast<const char *>(ins[r]) : nullptr;
    fp.out[r] = r < P ? static_cast<char *>(bufs[r]) : nullptr;
  }
  fp.P = P;
  fp.seg = make_seg(count / (size_t)P, count % (size_t)P, 1, all ? OUT_ALL : OUT_OWNER, P);
  fp.seg.owner_shift = P - 1;
  fp.start0 = 0;
  fp.start_stride = 1;
  fp.dir = 1;
  const size_t max_len = fp.seg.seg_base + (fp.seg.seg_rem ? 1 : 0);
  if (max_len == 0) return ALAMD_OK;
  const size_t es = alamd_dtype_size(dtype);
  if (!all || (size_t)P < tunables().two_step_min_outputs || count * es * (size_t)P < tunables().two_step_min_total_bytes)
    return launch_fold(fp, (unsigned)P, max_len, dtype, op, true, stream);
  // Large allreduce.  Writing each result tile to all P buffers from the fold
  // kernel interleaves P write streams; instead every segment is folded into
  // its owner's buffer (what the reduce-scatter leaves there) and then spread
  // from the owner to the other ranks.
  auto seg_off = [&](int s) {
    const size_t sg = (size_t)s, rem = (size_t)fp.seg.seg_rem;
    return (sg * fp.seg.seg_base + (sg < rem ? sg : rem)) * es;
  };
  auto seg_len = [&](int s) { return fp.seg.seg_base + ((size_t)s < fp.seg.seg_rem ? 1 : 0); };
  // piece by piece: fold the same range of every segment (P reads + 1 write), then spread it
  // (the fold's launches over the piece, then one pass of spread launches)
  const size_t tile_elems = 16384 / es;  // pieces are multiples of 16 KiB
  const size_t piece_bytes = tunables().ring_piece_bytes;
  size_t piece = piece_bytes / (size_t)P / es / tile_elems * tile_elems;
  if (piece == 0) piece = tile_elems;
  for (size_t e0 = 0, pn; e0 < max_len; e0 += pn) {
    pn = max_len - e0 < piece + piece / 2 ? max_len - e0 : piece;  // no short last piece
    FoldParams fo = fp;
    fo.seg.out_mode = OUT_OWNER;
    fo.seg.ragged = 1;
    FoldParams sp;
    sp.seg = make_seg(0, 0, 0, OUT_ALL, 0);
    sp.P = P;
    for (int r = 0; r < ALAMD_MAX_RANKS; ++r) {
      sp.in[r] = nullptr;
      sp.out[r] = r < P ? static_cast<char *>(bufs[r]) : nullptr;
    }
    size_t longest = 0;
    for (int s = 0; s < P; ++s) {
      const size_t len = seg_len(s) > e0 ? (seg_len(s) - e0 < pn ? seg_len(s) - e0 : pn) : 0;
      const size_t off = seg_off(s) + e0 * es;
      fo.seg.seg_off[s] = off / es;
      fo.seg.seg_len[s] = len;
      sp.in[s] = static_cast<const char *>(bufs[(s + P - 1) % P]) + off;
      sp.seg.seg_off[s] = off;
      sp.seg.seg_len[s] = len * es;
      if (len > longest) longest = len;
    }
    int rc = launch_fold(fo, (unsigned)P, longest, dtype, op, true, stream);
    if (rc) return rc;
    if ((rc = launch_spread_table(sp, P, false, stream))) return rc;
  }
  return ALAMD_OK;
}

}  // namespace
}  // namespace alamd

using namespace alamd;

extern "C" {

int alamd_ring_segment(size_t count, int P, int s, size_t *offset, size_t *len) {
  if (P < 1 || s < 0 || s >= P || !offset || !len)
    return set_error(ALAMD_ERR_INVALID_ARG, "bad ring segment query");
  const size_t base = count / (size_t)P, rem = count % (size_t)P;
  *offset = (size_t)s * base + ((size_t)s < rem ? (size_t)s : rem);
  *len = base + ((size_t)s < rem ? 1 : 0);
  return ALAMD_OK;
}

int alamd_ring_reduce_scatter(void *const *bufs, int P, size_t count, int dtype, int op,
                              size_t chunk_bytes, int mode, void *stream) {
  RingPlan pl;
  int rc = make_plan(pl, bufs, P, count, dtype, chunk_bytes);
  if (rc) return rc;
  if ((rc = check_type_op(dtype, op))) return rc;
  if (mode != ALAMD_RING_STEPWISE && mode != ALAMD_RING_FUSED)
    return set_error(ALAMD_ERR_INVALID_ALGO, "Invalid algorithm");
  if (count == 0 || P == 1) return ALAMD_OK;
  if (mode == ALAMD_RING_FUSED) return fused_fold(bufs, bufs, P, count, dtype, op, false, as_stream(stream));
  for (int t = 0; t < P - 1; ++t) {
    pl.rp.t = t;
    if ((rc = launch_step(pl, dtype, op, true, t == P - 2, as_stream(stream)))) return rc;
  }
  return ALAMD_OK;
}

int alamd_ring_allgather(void *const *bufs, int P, size_t count, int dtype, size_t chunk_bytes,
                         void *stream) {
  RingPlan pl;
  int rc = make_plan(pl, bufs, P, count, dtype, chunk_bytes);
  if (rc) return rc;
  if (count == 0 || P == 1) return ALAMD_OK;
  for (int t = 0; t < P - 1; ++t) {
    pl.rp.t = t;
    if ((rc = launch_step(pl, dtype, 0, false, false, as_stream(stream)))) return rc;
  }
  return ALAMD_OK;
}

int alamd_ring_allreduce(void *const *bufs, int P, size_t count, int dtype, int op, size_t chunk_bytes,
                         int mode, void *stream) {
  RingPlan pl;
  int rc = make_plan(pl, bufs, P, count, dtype, chunk_bytes);
  if (rc) return rc;
  if ((rc = check_type_op(dtype, op))) return rc;
  if (mode != ALAMD_RING_STEPWISE && mode != ALAMD_RING_FUSED)
    return set_error(ALAMD_ERR_INVALID_ALGO, "Invalid algorithm");
  if (count == 0 || P == 1) return ALAMD_OK;
  if (mode == ALAMD_RING_FUSED) return fused_fold(bufs, bufs, P, count, dtype, op, true, as_stream(stream));
  rc = alamd_ring_reduce_scatter(bufs, P, count, dtype, op, chunk_bytes, mode, stream);
  if (rc) return rc;
  return alamd_ring_allgather(bufs, P, count, dtype, chunk_bytes, stream);
}

int alamd_ring_allreduce_from(void *const *recvs, const void *const *sends, int P, size_t count, int dtype, int op,
                              size_t chunk_bytes, int mode, void *stream) {
  RingPlan pl;
  int rc = make_plan(pl, recvs, P, count, dtype, chunk_bytes);
  if (rc) return rc;
  if ((rc = check_type_op(dtype, op))) return rc;
  if (mode != ALAMD_RING_STEPWISE && mode != ALAMD_RING_FUSED)
    return set_error(ALAMD_ERR_INVALID_ALGO, "Invalid algorithm");
  if (!sends) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  if (count == 0) return ALAMD_OK;
  const size_t bytes = count * pl.es;
  bool in_place = true;
  for (int r = 0; r < P; ++r) {
    if (!sends[r]) return set_error(ALAMD_ERR_INVALID_ARG, "send buffer %d is null", r);
    if (!aligned_to(sends[r], pl.es))
      return set_error(ALAMD_ERR_INVALID_ARG, "send buffer %d is not aligned to its element type", r);
    in_place = in_place && sends[r] == recvs[r];
    for (int k = 0; k < P; ++k) {
      if (k == r && sends[r] == recvs[k]) continue;  // this rank in place
      const uintptr_t x = reinterpret_cast<uintptr_t>(sends[r]), y = reinterpret_cast<uintptr_t>(recvs[k]);
      if (x < y + bytes && y < x + bytes)
        return set_error(ALAMD_ERR_OVERLAP, "receive buffer %d overlaps send buffer %d", k, r);
    }
  }
  if (in_place) return alamd_ring_allreduce(recvs, P, count, dtype, op, chunk_bytes, mode, stream);
  // the fused form reads the contributions where they are; the step-by-step form moves them first,
  // as a rank of a ring would copy its send buffer before the first step
  if (mode == ALAMD_RING_FUSED && P > 1)
    return fused_fold(recvs, sends, P, count, dtype, op, true, as_stream(stream));
  for (int r = 0; r < P; ++r)
    if (sends[r] != recvs[r] && (rc = alamd_copy(recvs[r], sends[r], bytes, stream))) return rc;
  return alamd_ring_allreduce(recvs, P, count, dtype, op, chunk_bytes, mode, stream);
}

}  // extern "C"
