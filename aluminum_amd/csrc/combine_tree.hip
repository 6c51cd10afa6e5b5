// The tree kernels: balanced pairwise combine of up to 32 slots held in
// registers.  Used for floating-point types under the TREE_* orders, where
// the pairing decides the rounding; integer types never need it.
#include "alamd_dispatch.h"

namespace alamd {

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ void seg_range(const SegParams &s, unsigned seg, size_t &off, size_t &len) {
  const unsigned long long sg = seg;
  off = sg * s.seg_base + (sg < s.seg_rem ? sg : s.seg_rem);
  len = s.seg_base + (sg < s.seg_rem ? 1u : 0u);
}

template <typename T, int OP, int SLOTS, bool VECTOR, int U, bool GUARD>
__device__ __forceinline__ void tree_tile(const TreeParams &p, size_t in_bytes, int j0, int nj,
                                          size_t out_bytes, size_t i0, size_t n) {
  using L = Lane<T, VECTOR>;
  using V = typename L::V;
  const int nvalid = p.nvalid;
  bool act[U];
#pragma unroll
  for (int u = 0; u < U; ++u) act[u] = !GUARD || (i0 + (size_t)u * kThreads < n);

  V v[SLOTS][U];
#pragma unroll
  for (int j = 0; j < SLOTS; ++j) {
    if (j < nvalid) {
      const char *pa = p.a[j] + in_bytes;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (act[u]) v[j][u] = L::ld(pa, i0 + (size_t)u * kThreads);
    }
  }
  // pre-folded slots: the odd rank keeps step(in = even rank, inout = odd rank)
#pragma unroll
  for (int j = 0; j < SLOTS; ++j) {
    if (j < nvalid && p.b[j] != nullptr) {
      const char *pb = p.b[j] + in_bytes;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (act[u]) v[j][u] = L::template step<OP>(v[j][u], L::ld(pb, i0 + (size_t)u * kThreads));
    }
  }
#pragma unroll
  for (int d = 1; d < SLOTS; d *= 2) {
#pragma unroll
    for (int i = 0; i + d < SLOTS; i += 2 * d) {
      if (i + d < nvalid) {
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (act[u]) v[i][u] = L::template step<OP>(v[i + d][u], v[i][u]);
      }
    }
  }
  for (int j = j0; j < j0 + nj; ++j) {
    char *po = p.out[j] + out_bytes;
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (act[u]) L::st(po, i0 + (size_t)u * kThreads, v[0][u]);
  }
}

template <typename T, int OP, int SLOTS, bool VECTOR>
__global__ void __launch_bounds__(kThreads) tree_kernel(const TreeParams p) {
  using L = Lane<T, VECTOR>;
  constexpr int U = VECTOR ? (SLOTS <= 8 ? 2 : 1) : (SLOTS <= 8 ? 4 : 2);
  constexpr size_t TILE = (size_t)kThreads * U;
  const unsigned seg = blockIdx.y;
  size_t off, len;
  seg_range(p.seg, seg, off, len);
  const size_t off_bytes = off * sizeof(T);
  const size_t in_bytes = p.seg.in_blocked ? off_bytes : 0;
  int j0, nj;
  size_t out_bytes;
  if (p.seg.out_mode == OUT_ALL) { j0 = 0; nj = p.seg.nout; out_bytes = in_bytes; }
  else if (p.seg.out_mode == OUT_SEG) { j0 = (int)seg; nj = 1; out_bytes = 0; }
  else { j0 = ((int)seg + p.seg.owner_shift) % p.P; nj = 1; out_bytes = off_bytes; }

  const size_t n = len / L::N;
  const size_t ntiles = (n + TILE - 1) / TILE;
  for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t i0 = t * TILE + threadIdx.x;
    if ((t + 1) * TILE <= n) tree_tile<T, OP, SLOTS, VECTOR, U, false>(p, in_bytes, j0, nj, out_bytes, i0, n);
    else tree_tile<T, OP, SLOTS, VECTOR, U, true>(p, in_bytes, j0, nj, out_bytes, i0, n);
  }
  if constexpr (VECTOR) {
    const size_t e = n * L::N + threadIdx.x;
    if (blockIdx.x == 0 && e < len)
      tree_tile<T, OP, SLOTS, false, 1, false>(p, in_bytes, j0, nj, out_bytes, e, len);
  }
}

template <typename T, int OP, int SLOTS>
void (*pick_tree(bool vector))(const TreeParams) {
  return vector ? tree_kernel<T, OP, SLOTS, true> : tree_kernel<T, OP, SLOTS, false>;
}

}  // namespace

int launch_tree(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int dtype,
                int op, bool vector, hipStream_t stream) {
  return dispatch_float(dtype, op, [&](auto tt, auto ot) -> int {
    using T = typename decltype(tt)::type;
    constexpr int OP = decltype(ot)::value;
    const size_t per_access = vector ? 16 / sizeof(T) : 1;
    const int u = vector ? (slots <= 8 ? 2 : 1) : (slots <= 8 ? 4 : 2);
    const size_t tile = (size_t)kThreads * (size_t)u * per_access;
    unsigned gx = stream_grid(max_len, tile, 8);
    if (nseg > 1) {
      unsigned per_seg = (stream_grid((size_t)-1 / 2, 1, 8) + nseg - 1) / nseg;
      if (per_seg < 1) per_seg = 1;
      if (gx > per_seg) gx = per_seg;
    }
    void (*kern)(const TreeParams) = nullptr;
    switch (slots) {
    case 2: kern = pick_tree<T, OP, 2>(vector); break;
    case 4: kern = pick_tree<T, OP, 4>(vector); break;
    case 8: kern = pick_tree<T, OP, 8>(vector); break;
    case 16: kern = pick_tree<T, OP, 16>(vector); break;
    case 32: kern = pick_tree<T, OP, 32>(vector); break;
    default: return set_error(ALAMD_ERR_INVALID_ARG, "tree combine: bad slot count %d", slots);
    }
    hipLaunchKernelGGL(kern, dim3(gx, nseg, 1), dim3(kThreads, 1, 1), 0, stream, p);
    ALAMD_HIP(hipGetLastError());
    return ALAMD_OK;
  });
}

}  // namespace alamd
