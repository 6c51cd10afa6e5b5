// The tree kernels: balanced pairwise combine of up to 32 slots held in
// registers (64 slots as two halves of 32).  Used for floating-point types under the TREE_* orders, where
// the pairing decides the rounding; integer types never need it.
#include "alamd_dispatch.h"
#include "alamd_tile.h"

namespace alamd {

namespace {

// The tree over one element position, one element per access.  HALVES = 2: 2 * SLOTS slots, the
// two halves reduced one after the other and combined by the tree's top level.
template <typename T, int OP, int SLOTS, int HALVES>
__device__ __forceinline__ void tree_elem(const TreeParams &p, size_t in_bytes, int j0, int nj,
                                          size_t out_bytes, size_t e) {
  T res;
#pragma unroll
  for (int h = 0; h < HALVES; ++h) {
    const int base = h * SLOTS;
    const int nvalid = p.nvalid - base;
    if (h > 0 && nvalid <= 0) break;
    T v[SLOTS];
#pragma unroll
    for (int j = 0; j < SLOTS; ++j)
      if (j < nvalid) v[j] = ld_elem<T>(p.a[base + j] + in_bytes + e * sizeof(T));
#pragma unroll
    for (int j = 0; j < SLOTS; ++j)
      if (j < nvalid && p.b[base + j] != nullptr)
        v[j] = Step<T, OP>::apply(v[j], ld_elem<T>(p.b[base + j] + in_bytes + e * sizeof(T)));
#pragma unroll
    for (int d = 1; d < SLOTS; d *= 2) {
#pragma unroll
      for (int i = 0; i + d < SLOTS; i += 2 * d)
        if (i + d < nvalid) v[i] = Step<T, OP>::apply(v[i + d], v[i]);
    }
    res = h == 0 ? v[0] : Step<T, OP>::apply(v[0], res);
  }
  res = finish_elem<T, OP>(res, p.div);
  for (int j = j0; j < j0 + nj; ++j) st_elem<T>(p.out[j] + out_bytes + e * sizeof(T), res);
}

// Kernel variants: every slot occupied and none pre-folded (P a power of two:
// straight-line code, no uniform branches between the loads and their uses);
// some slots empty (binomial order, P not a power of two); some slots
// pre-folded from a second rank (doubling / halving orders, P not a power of
// two), which needs room for up to twice as many loads in flight.
enum { TREE_FULL = 0, TREE_PARTIAL = 1, TREE_PREFOLD = 2 };

template <typename T, int OP, int SLOTS, int MODE> struct TreeShape {
  static constexpr bool heavy = sizeof(T) <= 2;
  static constexpr int budget = heavy ? 32 : 64;  // 128-bit loads in flight per lane
  static constexpr int streams = MODE == TREE_PREFOLD ? 2 * SLOTS : SLOTS;
  static constexpr int U = budget / streams >= 8 ? (heavy ? 4 : 8) : (budget / streams >= 1 ? budget / streams : 1);
  static constexpr int THREADS = U == 8 ? 128 : 256;
};

__host__ __device__ inline void tree_out_select(const TreeParams &p, unsigned seg, size_t off_bytes,
                                                size_t in_bytes, int &j0, int &nj, size_t &out_bytes) {
  if (p.seg.out_mode == OUT_ALL) { j0 = 0; nj = p.seg.nout; out_bytes = in_bytes; }
  else if (p.seg.out_mode == OUT_SEG) { j0 = (int)seg; nj = 1; out_bytes = 0; }
  else { j0 = ((int)seg + p.seg.owner_shift) % p.P; nj = 1; out_bytes = off_bytes; }
}

// HEAD = false: no segment has leading elements to handle one by one (see the fold kernel).
// HALVES = 2: 2 * SLOTS slots (33 to 64 ranks under the binomial order, 64 under the other two).  The
// top level of a tree over 2 * SLOTS slots combines slot 0 with slot SLOTS, each the root of a tree
// over SLOTS slots, so the two halves are loaded and reduced one after the other with the registers
// of one.
template <typename T, int OP, int SLOTS, int MODE, bool HEAD, int HALVES>
__global__ void __launch_bounds__((TreeShape<T, OP, SLOTS, MODE>::THREADS)) __attribute__((amdgpu_waves_per_eu(1, 2)))
tree_vec_kernel(const TreeParams p) {
  constexpr int U = TreeShape<T, OP, SLOTS, MODE>::U, THREADS = TreeShape<T, OP, SLOTS, MODE>::THREADS;
  constexpr int N = 16 / sizeof(T);
  static_assert(HALVES == 1 || MODE != TREE_PREFOLD, "a pre-fold never meets more than 32 slots");
  using TL = Tile<U, THREADS>;
  const TL tl;
  const unsigned seg = seg_of(p.seg, blockIdx.y + p.seg.seg0);
  size_t off, len;
  seg_range(p.seg, seg, off, len);
  const size_t off_bytes = off * sizeof(T);
  const size_t in_bytes = p.seg.in_blocked ? off_bytes : 0;
  int j0, nj;
  size_t out_bytes;
  tree_out_select(p, seg, off_bytes, in_bytes, j0, nj, out_bytes);

  const size_t head = HEAD ? p.seg.seg_head[seg] : 0;
  const size_t vlen = len - head;
  const size_t vin = in_bytes + head * sizeof(T), vout = out_bytes + head * sizeof(T);
  const size_t vec_bytes = (vlen / N) * 16;
  const size_t tb = ((size_t)p.seg.tile0 + blockIdx.x) * TL::BYTES;
  if (tb < vec_bytes) {
    const size_t rem = vec_bytes - tb;
    const int nrec = rem > TL::BYTES ? (int)TL::BYTES : (int)rem;
    u32x4 res[U];
#pragma unroll
    for (int h = 0; h < HALVES; ++h) {
      const int base = h * SLOTS;
      const int nvalid = MODE == TREE_FULL ? SLOTS : p.nvalid - base;
      if (h > 0 && nvalid <= 0) break;
      u32x4 v[SLOTS][U];
#pragma unroll
      for (int j = 0; j < SLOTS; ++j) {
        if (j < nvalid) {
          const auto r = TL::rsrc(p.a[base + j] + vin + tb, nrec);
#pragma unroll
          for (int u = 0; u < U; ++u) v[j][u] = tl.load(r, u);
        }
      }
      if constexpr (MODE == TREE_PREFOLD) {
        // pre-folded slots: the odd rank keeps step(in = even rank, inout = odd rank); all of
        // their loads are issued before the first use, like the slots' own
        u32x4 w[SLOTS][U];
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
          if (j < nvalid && p.b[j] != nullptr) {
            const auto r = TL::rsrc(p.b[j] + vin + tb, nrec);
#pragma unroll
            for (int u = 0; u < U; ++u) w[j][u] = tl.load(r, u);
          }
        }
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
          if (j < nvalid && p.b[j] != nullptr) {
#pragma unroll
            for (int u = 0; u < U; ++u) v[j][u] = step_vec<T, OP>(v[j][u], w[j][u]);
          }
        }
      }
#pragma unroll
      for (int d = 1; d < SLOTS; d *= 2) {
#pragma unroll
        for (int i = 0; i + d < SLOTS; i += 2 * d) {
          if (i + d < nvalid) {
#pragma unroll
            for (int u = 0; u < U; ++u) v[i][u] = step_vec<T, OP>(v[i + d][u], v[i][u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) res[u] = h == 0 ? v[0][u] : step_vec<T, OP>(v[0][u], res[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) res[u] = finish_vec<T, OP>(res[u], p.div);
    for (int j = j0; j < j0 + nj; ++j) {
      const auto r = TL::rsrc(p.out[j] + vout + tb, nrec);
#pragma unroll
      for (int u = 0; u < U; ++u) tl.store(r, u, res[u]);
    }
  }
  // the head elements and the vlen % N elements behind the last whole vector
  if (p.seg.tile0 == 0 && blockIdx.x == 0 && threadIdx.x < head + vlen % N) {
    const size_t e = threadIdx.x < head ? threadIdx.x : (vlen / N) * N + threadIdx.x;
    tree_elem<T, OP, SLOTS, HALVES>(p, in_bytes, j0, nj, out_bytes, e);
  }
}


template <typename T, int OP, int SLOTS, int MODE, int HALVES = 1>
int launch_tree_mode(const TreeParams &p, unsigned nseg, size_t max_len, hipStream_t stream) {
  using S = TreeShape<T, OP, SLOTS, MODE>;
  const size_t tile_elems = Tile<S::U, S::THREADS>::BYTES / sizeof(T);
  const size_t per_launch = launch_tiles(p.P, Tile<S::U, S::THREADS>::BYTES);
  TreeParams q = p;
  q.div = make_divisor(p.P);
  for (unsigned sg = 0; sg < nseg; ++sg) {
    size_t off, len, out_bytes;
    int j0, nj;
    seg_range(p.seg, sg, off, len);
    const size_t in_bytes = p.seg.in_blocked ? off * sizeof(T) : 0;
    tree_out_select(p, sg, off * sizeof(T), in_bytes, j0, nj, out_bytes);
    q.seg.seg_head[sg] = (unsigned char)head_count(sizeof(T), p.out[j0] + out_bytes, p.a[0] + in_bytes, len);
    if (q.seg.seg_head[sg]) q.seg.any_head = 1;
  }
  void (*kern)(const TreeParams) =
      q.seg.any_head ? tree_vec_kernel<T, OP, SLOTS, MODE, true, HALVES> : tree_vec_kernel<T, OP, SLOTS, MODE, false, HALVES>;
  plan_launches(q.seg, nseg, max_len, tile_elems, per_launch, [&](size_t t0, size_t nt, unsigned s0, unsigned ns) {
    q.seg.tile0 = t0;
    q.seg.seg0 = s0;
    hipLaunchKernelGGL(kern, dim3((unsigned)nt, ns, 1), dim3(S::THREADS, 1, 1), 0, stream, q);
  });
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

template <typename T, int OP, int SLOTS>
int launch_tree_slots(const TreeParams &p, unsigned nseg, size_t max_len, hipStream_t stream) {
  bool prefold = false;
  for (int j = 0; j < SLOTS; ++j) prefold = prefold || p.b[j] != nullptr;
  if (prefold) return launch_tree_mode<T, OP, SLOTS, TREE_PREFOLD>(p, nseg, max_len, stream);
  if (p.nvalid == SLOTS) return launch_tree_mode<T, OP, SLOTS, TREE_FULL>(p, nseg, max_len, stream);
  return launch_tree_mode<T, OP, SLOTS, TREE_PARTIAL>(p, nseg, max_len, stream);
}

// 33 to 64 slots: two halves of 32.
template <typename T, int OP>
int launch_tree_two_halves(const TreeParams &p, unsigned nseg, size_t max_len, hipStream_t stream) {
  for (int j = 0; j < 64; ++j)
    if (p.b[j] != nullptr) return set_error(ALAMD_ERR_INVALID_ARG, "tree combine: pre-fold beyond 32 slots");
  if (p.nvalid == 64) return launch_tree_mode<T, OP, 32, TREE_FULL, 2>(p, nseg, max_len, stream);
  return launch_tree_mode<T, OP, 32, TREE_PARTIAL, 2>(p, nseg, max_len, stream);
}

}  // namespace

int launch_tree(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int dtype, int op,
                hipStream_t stream) {
  return dispatch_float(dtype, op, [&](auto tt, auto ot) -> int {
    using T = typename decltype(tt)::type;
    constexpr int OP = decltype(ot)::value;
    switch (slots) {
    case 2: return launch_tree_slots<T, OP, 2>(p, nseg, max_len, stream);
    case 4: return launch_tree_slots<T, OP, 4>(p, nseg, max_len, stream);
    case 8: return launch_tree_slots<T, OP, 8>(p, nseg, max_len, stream);
    case 16: return launch_tree_slots<T, OP, 16>(p, nseg, max_len, stream);
    case 32: return launch_tree_slots<T, OP, 32>(p, nseg, max_len, stream);
    case 64: return launch_tree_two_halves<T, OP>(p, nseg, max_len, stream);
    default: return set_error(ALAMD_ERR_INVALID_ARG, "tree combine: bad slot count %d", slots);
    }
  });
}

}  // namespace alamd
