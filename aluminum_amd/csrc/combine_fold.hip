// The fold kernels: out[i] = (((x_s . x_s+-1) . x_s+-2) ...)[i] over P rank
// contributions resident in HBM.  Bandwidth-bound: every input byte is read
// once with 128-bit non-temporal loads, all P loads of a lane are issued
// before the first use, and the result is written once per output.
#include "alamd_dispatch.h"

namespace alamd {

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ void seg_range(const SegParams &s, unsigned seg, size_t &off, size_t &len) {
  const unsigned long long sg = seg;
  off = sg * s.seg_base + (sg < s.seg_rem ? sg : s.seg_rem);
  len = s.seg_base + (sg < s.seg_rem ? 1u : 0u);
}

// Which outputs a segment writes, and at which byte offset.
__device__ __forceinline__ void out_select(const SegParams &s, int P, unsigned seg, size_t off_bytes,
                                           int &j0, int &nj, size_t &out_bytes) {
  if (s.out_mode == OUT_ALL) { j0 = 0; nj = s.nout; out_bytes = s.in_blocked ? off_bytes : 0; }
  else if (s.out_mode == OUT_SEG) { j0 = (int)seg; nj = 1; out_bytes = 0; }
  else { j0 = ((int)seg + s.owner_shift) % P; nj = 1; out_bytes = off_bytes; }
}

__device__ __forceinline__ int next_rank(int idx, int dir, int P) {
  idx += dir;
  if (idx >= P) idx -= P;
  if (idx < 0) idx += P;
  return idx;
}

// One tile: U accesses per thread, spaced one workgroup apart so that every
// wave-wide access is a run of contiguous 128-bit vectors.
template <typename T, int OP, bool ACC_IS_IN, bool VECTOR, int PT, int U, bool GUARD>
__device__ __forceinline__ void fold_tile(const FoldParams &p, int P, int s, size_t in_bytes,
                                          int j0, int nj, size_t out_bytes, size_t i0, size_t n) {
  using L = Lane<T, VECTOR>;
  using V = typename L::V;
  V acc[U];
  bool act[U];
#pragma unroll
  for (int u = 0; u < U; ++u) act[u] = !GUARD || (i0 + (size_t)u * kThreads < n);

  if constexpr (PT > 0) {
    V x[PT][U];
    int idx = s;
#pragma unroll
    for (int k = 0; k < PT; ++k) {
      const char *pk = p.in[idx] + in_bytes;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (act[u]) x[k][u] = L::ld(pk, i0 + (size_t)u * kThreads);
      idx = next_rank(idx, p.dir, PT);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (!act[u]) continue;
      acc[u] = x[0][u];
#pragma unroll
      for (int k = 1; k < PT; ++k)
        acc[u] = ACC_IS_IN ? L::template step<OP>(acc[u], x[k][u]) : L::template step<OP>(x[k][u], acc[u]);
    }
  } else {
    constexpr int B = 4;  // loads in flight per access between uses
    int idx = s;
    {
      const char *p0 = p.in[idx] + in_bytes;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (act[u]) acc[u] = L::ld(p0, i0 + (size_t)u * kThreads);
    }
    for (int k = 1; k < P; k += B) {
      V x[B][U];
      int id = idx;
#pragma unroll
      for (int b = 0; b < B; ++b) {
        if (k + b < P) {
          id = next_rank(id, p.dir, P);
          const char *pk = p.in[id] + in_bytes;
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (act[u]) x[b][u] = L::ld(pk, i0 + (size_t)u * kThreads);
        }
      }
#pragma unroll
      for (int b = 0; b < B; ++b) {
        if (k + b < P) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (act[u])
              acc[u] = ACC_IS_IN ? L::template step<OP>(acc[u], x[b][u]) : L::template step<OP>(x[b][u], acc[u]);
        }
      }
      idx = id;
    }
  }

  for (int j = j0; j < j0 + nj; ++j) {
    char *po = p.out[j] + out_bytes;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (act[u]) L::st(po, i0 + (size_t)u * kThreads, acc[u]);
  }
}

template <typename T, int OP, bool ACC_IS_IN, bool VECTOR, int PT>
__global__ void __launch_bounds__(kThreads) fold_kernel(const FoldParams p) {
  using L = Lane<T, VECTOR>;
  constexpr int U = VECTOR ? 2 : 4;
  constexpr size_t TILE = (size_t)kThreads * U;
  const int P = PT ? PT : p.P;
  const unsigned seg = blockIdx.y;
  size_t off, len;
  seg_range(p.seg, seg, off, len);
  const size_t off_bytes = off * sizeof(T);
  const size_t in_bytes = p.seg.in_blocked ? off_bytes : 0;
  const int s = (p.start0 + (int)seg * p.start_stride) % P;
  int j0, nj;
  size_t out_bytes;
  out_select(p.seg, P, seg, off_bytes, j0, nj, out_bytes);

  const size_t n = len / L::N;  // accesses in this segment
  const size_t ntiles = (n + TILE - 1) / TILE;
  for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t i0 = t * TILE + threadIdx.x;
    if ((t + 1) * TILE <= n)
      fold_tile<T, OP, ACC_IS_IN, VECTOR, PT, U, false>(p, P, s, in_bytes, j0, nj, out_bytes, i0, n);
    else
      fold_tile<T, OP, ACC_IS_IN, VECTOR, PT, U, true>(p, P, s, in_bytes, j0, nj, out_bytes, i0, n);
  }

  if constexpr (VECTOR) {
    // the len % N trailing elements, one per thread of the first workgroup
    const size_t e = n * L::N + threadIdx.x;
    if (blockIdx.x == 0 && e < len)
      fold_tile<T, OP, ACC_IS_IN, false, 0, 1, false>(p, P, s, in_bytes, j0, nj, out_bytes, e, len);
  }
}

}  // namespace

unsigned stream_grid(size_t work_items, size_t per_block, int waves) {
  const int cus = device_cus();
  size_t need = (work_items + per_block - 1) / per_block;
  size_t cap = (size_t)(cus > 0 ? cus : 256) * (size_t)(waves > 0 ? waves : 1);
  if (need < 1) need = 1;
  return (unsigned)(need < cap ? need : cap);
}

int launch_fold(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op,
                bool acc_is_in, bool vector, hipStream_t stream) {
  // operand roles only matter where a tie or a NaN can pick a side
  const bool roles = acc_is_in && is_float_dtype(dtype) && (op == ALAMD_MIN || op == ALAMD_MAX);
  return dispatch_any(dtype, op, [&](auto tt, auto ot) -> int {
    using T = typename decltype(tt)::type;
    constexpr int OP = decltype(ot)::value;
    constexpr bool FP_MINMAX = (std::is_same<T, float>::value || std::is_same<T, double>::value ||
                                std::is_same<T, f16_t>::value || std::is_same<T, bf16_t>::value) &&
                               (OP == ALAMD_MIN || OP == ALAMD_MAX);
    const size_t per_access = vector ? 16 / sizeof(T) : 1;
    const size_t tile = (size_t)kThreads * (vector ? 2 : 4) * per_access;
    unsigned gx = stream_grid(max_len, tile, 8);
    if (nseg > 1) {
      unsigned per_seg = (stream_grid((size_t)-1 / 2, 1, 8) + nseg - 1) / nseg;
      if (per_seg < 1) per_seg = 1;
      if (gx > per_seg) gx = per_seg;
    }
    dim3 grid(gx, nseg, 1), block(kThreads, 1, 1);
    void (*kern)(const FoldParams) = nullptr;
    if (vector) {
      if (p.P == 8) {
        if constexpr (FP_MINMAX) kern = roles ? fold_kernel<T, OP, true, true, 8> : fold_kernel<T, OP, false, true, 8>;
        else kern = fold_kernel<T, OP, false, true, 8>;
      } else {
        if constexpr (FP_MINMAX) kern = roles ? fold_kernel<T, OP, true, true, 0> : fold_kernel<T, OP, false, true, 0>;
        else kern = fold_kernel<T, OP, false, true, 0>;
      }
    } else {
      if constexpr (FP_MINMAX) kern = roles ? fold_kernel<T, OP, true, false, 0> : fold_kernel<T, OP, false, false, 0>;
      else kern = fold_kernel<T, OP, false, false, 0>;
    }
    hipLaunchKernelGGL(kern, grid, block, 0, stream, p);
    ALAMD_HIP(hipGetLastError());
    return ALAMD_OK;
  });
}

}  // namespace alamd
