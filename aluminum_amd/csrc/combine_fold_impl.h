// The fold kernels (included by the translation units that build them, one per
// group of element types): out[i] = (((x_s . x_s+-1) . x_s+-2) ...)[i] over P rank
// contributions resident in HBM.  Bandwidth-bound: every input byte is read
// once, every output byte written once.
//
// One workgroup per tile, all loads of a lane issued before the first use,
// buffer instructions with per-tile descriptors (see alamd_tile.h); buffers
// need only be aligned to their element type.  The len % N elements behind the
// last whole vector of a segment are folded one per thread.
#pragma once

#include "alamd_dispatch.h"
#include "alamd_tile.h"

namespace alamd {

namespace {

__device__ __forceinline__ int next_rank(int idx, int dir, int P) {
  idx += dir;
  if (idx >= P) idx -= P;
  if (idx < 0) idx += P;
  return idx;
}

// The fold of one element position, one element per access.
template <typename T, int OP, bool ACC_IS_IN>
__device__ __forceinline__ T fold_elem_value(const FoldParams &p, int P, int s, size_t in_bytes, size_t e) {
  int idx = s;
  T acc = ld_elem<T>(p.in[idx] + in_bytes + e * sizeof(T));
  for (int k = 1; k < P; ++k) {
    idx = next_rank(idx, p.dir, P);
    const T x = ld_elem<T>(p.in[idx] + in_bytes + e * sizeof(T));
    acc = ACC_IS_IN ? Step<T, OP>::apply(acc, x) : Step<T, OP>::apply(x, acc);
  }
  return finish_elem<T, OP>(acc, p.div);
}
template <typename T, int OP, bool ACC_IS_IN>
__device__ __forceinline__ void fold_elem(const FoldParams &p, int P, int s, size_t in_bytes, int j0, int nj,
                                          size_t out_bytes, size_t e) {
  const T acc = fold_elem_value<T, OP, ACC_IS_IN>(p, P, s, in_bytes, e);
  for (int j = j0; j < j0 + nj; ++j) st_elem<T>(p.out[j] + out_bytes + e * sizeof(T), acc);
}

// Tile shape: 128 threads x 8 vectors per stream for every type (byte sums and
// products, the most arithmetic per byte, are done a dword at a time and keep up).
template <typename T, int OP> struct Shape {
  static constexpr int U = 8;
  static constexpr int THREADS = 128;
  // P = 8 body: streams whose loads are issued before the first use (0: left to the compiler, which
  // keeps as many in flight as the registers hold).  bf16 spends seven instructions per dword and
  // step where the other types spend one; with everything requested up front the compiler ends up
  // with a schedule that asks for 36 vectors, works through 27 of them and only then asks for the
  // rest.  Two streams up front and one more requested for every one consumed is worth 0.3 to 0.5
  // points to bf16 (6253 against 6227 GB/s, and 6250 against 6210, on buffers that are not reused)
  // and nothing to fp32 (6144 / 6122, 6179 / 6173); three to seven streams up front, or more than
  // two waves per SIMD with two, lose 1 to 5 points for both.
  static constexpr int FRONT = std::is_same<T, bf16_t>::value ? 2 : 0;
};

// amdgpu_waves_per_eu(1, 2): the loads in flight are the point of this kernel;
// the register allocator must not trade them away for more resident waves.
// HEAD = false: no segment has leading elements to handle one by one (every buffer on a 64-byte
// boundary).  With the head a compile-time zero the fp32 fold runs 1.6 points faster (83.8 % of the HBM
// peak against 82.2 %) and the fp32 tree 2.8; both bodies in one kernel behind a uniform branch ran slower
// than either (82.7 %, bf16 80.8 % against 82.2 %), so there are two kernels and the host picks.
// (The body must stay in the kernel itself: moved into an inlined device function it was compiled
// with 161 instead of 249 VGPRs, i.e. with fewer loads in flight, and lost 1.5 points.)
// CHAIN: the output overlaps one of the inputs at a displacement; tiles come from a ticket counter and
// a tile's stores wait for the loads of the tiles that read what it writes (see ChainParams).  Always
// with HEAD = false (no leading elements: the vectors start at the output's first element) and one
// segment with one output.
template <typename T, int OP, bool ACC_IS_IN, int PT, bool HEAD, bool CHAIN = false>
__global__ void __launch_bounds__((Shape<T, OP>::THREADS)) __attribute__((amdgpu_waves_per_eu(1, 2)))
fold_vec_kernel(const FoldParams p) {
  static_assert(!(CHAIN && HEAD), "a chained launch has no head");
  constexpr int U = Shape<T, OP>::U, THREADS = Shape<T, OP>::THREADS;
  constexpr int N = 16 / sizeof(T);
  using TL = Tile<U, THREADS>;
  const TL tl;
  const int P = PT ? PT : p.P;
  // The general case looks its segment up in several tables, one dependent scalar load after the
  // other; a launch over one whole segment into one output needs none of that.
  unsigned seg = 0;
  size_t off = 0, len = p.seg.seg_base, in_bytes = 0, out_bytes = 0;
  int s = p.start0, j0 = 0, nj = 1;
  if (!p.seg.simple) {
    seg = seg_of(p.seg, blockIdx.y + p.seg.seg0);
    seg_range(p.seg, seg, off, len);
    const size_t off_bytes = off * sizeof(T);
    in_bytes = p.seg.in_blocked ? off_bytes : 0;
    s = (p.start0 + (int)seg * p.start_stride) % P;
    out_select(p.seg, P, seg, off_bytes, j0, nj, out_bytes);
  }

  const size_t head = HEAD ? p.seg.seg_head[seg] : 0;
  const size_t vlen = len - head;
  const size_t vin = in_bytes + head * sizeof(T), vout = out_bytes + head * sizeof(T);
  const size_t vec_bytes = (vlen / N) * 16;
  unsigned bx = blockIdx.x;
  if constexpr (CHAIN) bx = chain_take_tile(p.chain);
  const size_t tb = ((size_t)p.seg.tile0 + bx) * TL::BYTES;
  if (tb < vec_bytes) {
    const size_t rem = vec_bytes - tb;
    const int nrec = rem > TL::BYTES ? (int)TL::BYTES : (int)rem;
    u32x4 acc[U];
    if constexpr (PT == 8 && Shape<T, OP>::FRONT >= 2) {
      // FRONT streams have their loads issued before the first use; every vector consumed then frees
      // four registers, which the same vector of the next stream not yet requested takes.
      constexpr int FRONT = Shape<T, OP>::FRONT;
      u32x4 x[PT][U];
      __amdgpu_buffer_rsrc_t r[PT];
      int idx = s;
#pragma unroll
      for (int k = 0; k < PT; ++k) {
        r[k] = TL::rsrc(p.in[idx] + vin + tb, nrec);
        idx = next_rank(idx, p.dir, PT);
      }
#pragma unroll
      for (int k = 0; k < FRONT; ++k) {
#pragma unroll
        for (int u = 0; u < U; ++u) x[k][u] = tl.load(r[k], u);
      }
      __builtin_amdgcn_sched_barrier(0);
      // a later load takes its offset from an empty asm statement that reads the step's result, so
      // that it cannot be issued earlier
      auto load_after = [&](__amdgpu_buffer_rsrc_t rs, int u, const u32x4 &after) {
        unsigned vo = tl.vo;
        asm volatile("" : "+v"(vo) : "v"(after));
        return __builtin_amdgcn_raw_buffer_load_b128(rs, vo + (unsigned)u * 1024u, 0, kAuxLoadStream);
      };
#pragma unroll
      for (int k = 1; k < PT; ++k) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const u32x4 a = k == 1 ? x[0][u] : acc[u];
          acc[u] = ACC_IS_IN ? step_vec<T, OP>(a, x[k][u]) : step_vec<T, OP>(x[k][u], a);
          const int nx = FRONT + k - 1;  // the stream requested next
          if (nx < PT) x[nx < PT ? nx : 0][u] = load_after(r[nx < PT ? nx : 0], u, acc[u]);
        }
        // an empty asm statement per accumulator: the steps of stream k can neither sink below it nor
        // mix with those of stream k + 1
#pragma unroll
        for (int u = 0; u < U; ++u) asm volatile("" : "+v"(acc[u]));
      }
    } else if constexpr (PT > 0) {
      u32x4 x[PT][U];
      int idx = s;
#pragma unroll
      for (int k = 0; k < PT; ++k) {
        const auto r = TL::rsrc(p.in[idx] + vin + tb, nrec);
#pragma unroll
        for (int u = 0; u < U; ++u) x[k][u] = tl.load(r, u);
        idx = next_rank(idx, p.dir, PT);
      }
      // stream-major, the order the loads were issued in (they return in
      // order): every accumulator advances as soon as a stream has arrived
#pragma unroll
      for (int u = 0; u < U; ++u) acc[u] = x[0][u];
#pragma unroll
      for (int k = 1; k < PT; ++k) {
#pragma unroll
        for (int u = 0; u < U; ++u)
          acc[u] = ACC_IS_IN ? step_vec<T, OP>(acc[u], x[k][u]) : step_vec<T, OP>(x[k][u], acc[u]);
      }
    } else {
      // Run-time rank count: the streams are taken in batches of a compile-time size - the pointers
      // of a batch, then all its loads, then all its steps, no branch in between - so that up to
      // seven ranks have every stream in flight at once, like the P = 8 body above.  (With one
      // branch per stream the compiler fetched each stream's pointer, waited for it and only then
      // issued that stream's loads: 1.5 % slower at P = 12 and 16, and for 16-bit and 8-bit types
      // at P = 4.  A compile-time P = 4 body gains another 0.5 to 1 %, not worth its kernels.)
      int idx = s;
      auto batch = [&](auto rc, auto first_c) {
        constexpr int R = decltype(rc)::value;
        constexpr bool FIRST = decltype(first_c)::value;  // the batch starts the fold
        const char *src[R];
#pragma unroll
        for (int b = 0; b < R; ++b) {
          if (!(FIRST && b == 0)) idx = next_rank(idx, p.dir, P);
          src[b] = p.in[idx];
        }
        u32x4 x[R][U];
#pragma unroll
        for (int b = 0; b < R; ++b) {
          const auto r = TL::rsrc(src[b] + vin + tb, nrec);
#pragma unroll
          for (int u = 0; u < U; ++u) x[b][u] = tl.load(r, u);
        }
        if constexpr (FIRST) {
#pragma unroll
          for (int u = 0; u < U; ++u) acc[u] = x[0][u];
        }
#pragma unroll
        for (int b = FIRST ? 1 : 0; b < R; ++b) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            acc[u] = ACC_IS_IN ? step_vec<T, OP>(acc[u], x[b][u]) : step_vec<T, OP>(x[b][u], acc[u]);
        }
      };
      using Yes = std::true_type;
      using No = std::false_type;
      // Up to seven streams in one batch; beyond that a first batch that leaves a multiple of six.
      // For 8- and 16-bit types, whose arithmetic needs registers as well, the kernel then no longer
      // fits two waves per SIMD.  Batches of five and four, which do, ran 1 to 3 % slower all the
      // same - except in a chained launch, where the second wave hides the waits for the
      // neighbouring tile (bf16, a block one element into its buffer: 5.2 TB/s against 4.5).
      constexpr bool kTwoWaves = CHAIN && sizeof(T) <= 2;
      constexpr int B0 = kTwoWaves ? 5 : 7, B = kTwoWaves ? 4 : 6;
      int left = P;
      switch (P <= B0 ? P : (P - 1) % B + 1) {
      case 7: if constexpr (B0 >= 7) { batch(std::integral_constant<int, 7>{}, Yes{}); left -= 7; } break;
      case 6: if constexpr (B0 >= 6) { batch(std::integral_constant<int, 6>{}, Yes{}); left -= 6; } break;
      case 5: batch(std::integral_constant<int, 5>{}, Yes{}); left -= 5; break;
      case 4: batch(std::integral_constant<int, 4>{}, Yes{}); left -= 4; break;
      case 3: batch(std::integral_constant<int, 3>{}, Yes{}); left -= 3; break;
      case 2: batch(std::integral_constant<int, 2>{}, Yes{}); left -= 2; break;
      default: batch(std::integral_constant<int, 1>{}, Yes{}); left -= 1; break;
      }
      for (; left >= B; left -= B) batch(std::integral_constant<int, B>{}, No{});
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc[u] = finish_vec<T, OP>(acc[u], p.div);
    if constexpr (CHAIN) chain_gate(p.chain, bx, tb, (unsigned long long)nrec, (unsigned)TL::BYTES);
    for (int j = j0; j < j0 + nj; ++j) {
      const auto r = TL::rsrc(p.out[j] + vout + tb, nrec);
#pragma unroll
      for (int u = 0; u < U; ++u) tl.store(r, u, acc[u]);
    }
  }
  if constexpr (CHAIN) {
    // the vlen % N elements behind the last whole vector are the last ticket
    if (bx == p.chain.nvec_tiles) {
      const bool mine = threadIdx.x < vlen % N;
      const size_t e = (vlen / N) * N + threadIdx.x;
      T val = T();
      if (mine) val = fold_elem_value<T, OP, ACC_IS_IN>(p, P, s, in_bytes, e);
      chain_gate(p.chain, bx, vec_bytes, (vlen % N) * sizeof(T), (unsigned)TL::BYTES);
      if (mine) st_elem<T>(p.out[j0] + out_bytes + e * sizeof(T), val);
    }
  } else {
    // the head elements and the vlen % N elements behind the last whole vector, one per thread of the
    // segment's first workgroup
    if (p.seg.tile0 == 0 && blockIdx.x == 0 && threadIdx.x < head + vlen % N) {
      const size_t e = threadIdx.x < head ? threadIdx.x : (vlen / N) * N + threadIdx.x;
      fold_elem<T, OP, ACC_IS_IN>(p, P, s, in_bytes, j0, nj, out_bytes, e);
    }
  }
}


// The launches of one (type, operator) pair.  roles: the running result is the `in` operand of every
// step (only matters where a tie or a NaN can pick a side: float min / max).
template <typename T, int OP>
int launch_fold_typed(const FoldParams &p, unsigned nseg, size_t max_len, bool roles, hipStream_t stream,
                      const ChainScratch *chain, size_t displ_bytes) {
  {
    constexpr bool FP_MINMAX = (std::is_same<T, float>::value || std::is_same<T, double>::value ||
                                std::is_same<T, f16_t>::value || std::is_same<T, bf16_t>::value) &&
                               (OP == ALAMD_MIN || OP == ALAMD_MAX);
    const size_t tile_elems = Tile<Shape<T, OP>::U, Shape<T, OP>::THREADS>::BYTES / sizeof(T);
    FoldParams q = p;
    q.div = make_divisor(p.P);
    q.chain = ChainParams{nullptr, nullptr, nullptr, 0, 0, 0};
    q.seg.simple = 0;
    if (chain) {
      // one segment, one output, every tile in one launch, tiles handed out by the ticket counter
      if (nseg != 1) return set_error(ALAMD_ERR_INVALID_ARG, "a chained fold has one segment");
      constexpr size_t N = 16 / sizeof(T);
      const size_t nvec = (max_len / N * 16 + Tile<Shape<T, OP>::U, Shape<T, OP>::THREADS>::BYTES - 1) /
                          Tile<Shape<T, OP>::U, Shape<T, OP>::THREADS>::BYTES;
      const size_t tickets = nvec + (max_len % N ? 1 : 0);
      if (nvec > chain->max_tiles || tickets > 0x7fffffffull)
        return set_error(ALAMD_ERR_INVALID_ARG, "in-place block of %zu elements needs %zu tile flags, the scratch holds %zu",
                         max_len, nvec, chain->max_tiles);
      int rc = chain_clear(*chain, nvec, stream);
      if (rc) return rc;
      q.chain = ChainParams{chain->ticket, chain->flags, chain->error, displ_bytes, (unsigned)nvec, chain->max_polls};
      q.seg.tile0 = 0;
      q.seg.seg0 = 0;
      q.seg.mapped = 0;
      void (*ck)(const FoldParams) = nullptr;
      // Always the run-time-P body: with the gate in it the P = 8 body no longer fits two waves per SIMD,
      // and a second wave is what hides a tile's wait for its neighbour (a block one element into its
      // buffer: 3 to 11 % faster than with the P = 8 body; from a few MiB in, 3 % slower).
      if constexpr (FP_MINMAX) ck = roles ? fold_vec_kernel<T, OP, true, 0, false, true> : fold_vec_kernel<T, OP, false, 0, false, true>;
      else ck = fold_vec_kernel<T, OP, false, 0, false, true>;
      hipLaunchKernelGGL(ck, dim3((unsigned)tickets, 1, 1), dim3(Shape<T, OP>::THREADS, 1, 1), 0, stream, q);
      ALAMD_HIP(hipGetLastError());
      return ALAMD_OK;
    }
    for (unsigned sg = 0; sg < nseg; ++sg) {
      size_t off, len, out_bytes;
      int j0, nj;
      seg_range(p.seg, sg, off, len);
      out_select(p.seg, p.P, sg, off * sizeof(T), j0, nj, out_bytes);
      const int first = (p.start0 + (int)sg * p.start_stride) % p.P;
      q.seg.seg_head[sg] = (unsigned char)head_count(sizeof(T), p.out[j0] + out_bytes,
                                                     p.in[first] + (p.seg.in_blocked ? off * sizeof(T) : 0), len);
      if (q.seg.seg_head[sg]) q.seg.any_head = 1;
    }
    q.seg.simple = nseg == 1 && !q.seg.ragged && q.seg.seg_rem == 0 && !q.seg.in_blocked && q.seg.out_mode == OUT_ALL && q.seg.nout == 1 &&
                   !q.seg.any_head && p.start0 >= 0 && p.start0 < p.P;
    auto pick = [&](auto acc_is_in_t, auto pt_t) -> void (*)(const FoldParams) {
      constexpr bool A = decltype(acc_is_in_t)::value;
      constexpr int PT = decltype(pt_t)::value;
      return q.seg.any_head ? fold_vec_kernel<T, OP, A, PT, true> : fold_vec_kernel<T, OP, A, PT, false>;
    };
    using No = std::false_type;
    using Yes = std::true_type;
    using P8 = std::integral_constant<int, 8>;
    using PN = std::integral_constant<int, 0>;
    void (*kern)(const FoldParams) = nullptr;
    if (p.P == 8) {
      if constexpr (FP_MINMAX) kern = roles ? pick(Yes{}, P8{}) : pick(No{}, P8{});
      else kern = pick(No{}, P8{});
    } else {
      if constexpr (FP_MINMAX) kern = roles ? pick(Yes{}, PN{}) : pick(No{}, PN{});
      else kern = pick(No{}, PN{});
    }
    const size_t per_launch = launch_tiles(p.P, Tile<Shape<T, OP>::U, Shape<T, OP>::THREADS>::BYTES, tunables().launch_bytes);
    plan_launches(q.seg, nseg, max_len, tile_elems, per_launch, [&](size_t t0, size_t nt, unsigned s0, unsigned ns) {
      q.seg.tile0 = t0;
      q.seg.seg0 = s0;
      hipLaunchKernelGGL(kern, dim3((unsigned)nt, ns, 1), dim3(Shape<T, OP>::THREADS, 1, 1), 0, stream, q);
    });
    ALAMD_HIP(hipGetLastError());
    return ALAMD_OK;
  }
}

// Defines `NAME`, the launcher of one group of element types.
#define ALAMD_FOLD_GROUP(NAME, ...)                                                                     \
  int NAME(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool roles,           \
           hipStream_t stream, const ChainScratch *chain, size_t displ_bytes) {                         \
    auto run = [&](auto tt, auto ot) -> int {                                                           \
      using T = typename decltype(tt)::type;                                                            \
      constexpr int OP = decltype(ot)::value;                                                           \
      return launch_fold_typed<T, OP>(p, nseg, max_len, roles, stream, chain, displ_bytes);             \
    };                                                                                                  \
    switch (dtype) {                                                                                    \
      __VA_ARGS__                                                                                       \
    default: return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);                   \
    }                                                                                                   \
  }

}  // namespace
}  // namespace alamd
