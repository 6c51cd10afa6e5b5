// The fold kernels (included by the translation units that build them, one per
// group of element types): out[i] = (((x_s . x_s+-1) . x_s+-2) ...)[i] over P rank
// contributions resident in HBM.  Bandwidth-bound: every input byte is read
// once, every output byte written once.
//
// One workgroup per tile, a bounded number of loads in flight per wave (see Shape),
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

// Shape of a launch.
//
// A large or a small launch streams: one wave per workgroup, one 128-bit vector per lane and stream (1 KiB per
// wave and stream), FRONT streams requested before the first use and one more for every stream consumed
// (so FRONT - 1 loads of a wave are in flight once the fold is under way), and a number of waves per CU
// that the host sets per launch (see stream_lds_bytes and stream_wgs_per_cu in alamd_tile.h, which also
// hold the measurements).  Workgroups of two or four waves with the same amount in flight run 2 to 4
// points lower, and so does every shape that asks for all of a lane's vectors up front (128 threads x
// 8 vectors x 8 streams, two waves per SIMD: 79 % of the HBM peak where this shape reaches 85 %).
//
// The block shape keeps tiles of 16 KiB per stream, 128 threads x 8 vectors, all of a batch of streams
// requested up front, two waves per SIMD.  A launch of middling size takes it (see use_block_shape in
// alamd_dispatch.h and the measurements above Tile in alamd_tile.h): sixteen times fewer workgroups to hand out, each done after one trip to memory instead
// of P / FRONT of them, which is what counts while a launch lasts tens of microseconds and much of what
// it reads sits in the caches.  A chained launch (see KIND below) takes it as well: its tiles are handed
// out by a counter and wait for one another through one flag per tile, which small tiles would make
// sixteen times as many of.
template <typename T, int OP, bool BLOCK = false> struct Shape {
  static constexpr int U = BLOCK ? 8 : 1;
  static constexpr int THREADS = BLOCK ? 128 : 64;
  static constexpr int WAVES = BLOCK ? 2 : kStreamMaxWaves;  // compiled for; see stream_lds_bytes
};
// Ordinary launches are built with FRONT = 2 and FRONT = 3; the host takes three from this many ranks on
// (P = 8: 84 against 84 %, P = 12: 82 and 82, P = 16: 84 against 81, P = 64: 82 against 79).
constexpr int kFront3FromRanks = 12;

// HEAD = false: no segment has leading elements to handle one by one (see stream_head_count); two
// kernels, and the host picks, so that the usual case carries no trace of the other.
// FRONT: see Shape (0 in the block shape).
// KIND: FOLD_STREAM, FOLD_BLOCK (built with HEAD = true only: its few workgroups do not feel the lookup),
// or FOLD_CHAINED: the output overlaps one of the inputs at a displacement; tiles in the block shape come
// from a ticket counter and a tile's stores wait for the loads of the tiles that read what it writes
// (see ChainParams).  Always with HEAD = false (no leading elements: the vectors start at the output's
// first element) and one segment with one output.
template <typename T, int OP, bool ACC_IS_IN, int FRONT, bool HEAD, int KIND = FOLD_STREAM>
__global__ void __launch_bounds__((Shape<T, OP, KIND != FOLD_STREAM>::THREADS))
__attribute__((amdgpu_waves_per_eu(1, Shape<T, OP, KIND != FOLD_STREAM>::WAVES)))
fold_vec_kernel(const FoldParams p) {
  constexpr bool CHAIN = KIND == FOLD_CHAINED, BLOCK = KIND != FOLD_STREAM;
  static_assert(!(CHAIN && HEAD), "a chained launch has no head");
  static_assert(BLOCK ? FRONT == 0 : (FRONT >= 2 && FRONT <= 4), "streams requested up front");
  constexpr int U = Shape<T, OP, BLOCK>::U, THREADS = Shape<T, OP, BLOCK>::THREADS;
  constexpr int N = 16 / sizeof(T);
  using TL = Tile<U, THREADS>;
  const TL tl;
  const int P = p.P;
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

  const size_t head = HEAD ? arg_u16(p.seg.seg_head, seg) : 0;
  const size_t vlen = len - head;
  const size_t vin = in_bytes + head * sizeof(T), vout = out_bytes + head * sizeof(T);
  const size_t vec_bytes = (vlen / N) * 16;
  unsigned bx = blockIdx.x;
  if constexpr (HEAD && !BLOCK) { if (p.seg.xcd_run_log2) bx = xcd_run_tile(bx, gridDim.x, (unsigned)p.seg.xcd_run_log2); }
  if constexpr (CHAIN) bx = chain_take_tile(p.chain);
  const size_t tb = ((size_t)p.seg.tile0 + bx) * TL::BYTES;
  if (tb < vec_bytes) {
    const size_t rem = vec_bytes - tb;
    const int nrec = rem > TL::BYTES ? (int)TL::BYTES : (int)rem;
    u32x4 acc[U];
    // (a logical operator on 8- or 16-bit elements: the running result is made 0 / 1 per element once,
    // and every step then only looks at the stream it adds; with one rank there is no step, and the
    // result is the input as it is)
    constexpr bool TRUTH = narrow_logical<T, OP>();
    if constexpr (!BLOCK) {
      static_assert(U == 1, "the streaming body holds one vector per lane and stream");
      // Stream k lives in x[k % FRONT].  A later load takes its offset from an empty asm statement that
      // reads the result of the step before it, so that it cannot be issued any earlier; the empty
      // statement on the accumulator keeps the steps themselves in order.
      u32x4 x[FRONT];
      // the rank whose stream is requested next, and its buffer: the pointer is fetched one request
      // ahead, so that its scalar load is not part of the chain from one request to the next
      int req = s;
      const char *next_in = p.in[req];
#pragma unroll
      for (int j = 0; j < FRONT; ++j) {
        if (j < P) {
          x[j] = tl.load(TL::rsrc(next_in + vin + tb, nrec), 0);
          req = next_rank(req, p.dir, P);
          next_in = p.in[req];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      auto load_after = [&](__amdgpu_buffer_rsrc_t rs, const u32x4 &after) {
        unsigned vo = tl.vo;
        asm volatile("" : "+v"(vo) : "v"(after));
        return __builtin_amdgcn_raw_buffer_load_b128(rs, vo, 0, kAuxLoadStream);
      };
      acc[0] = x[0];
      if constexpr (TRUTH) { if (P >= 2) acc[0] = truth_vec<T>(acc[0]); }
      for (int base = 0; base < P; base += FRONT) {
#pragma unroll
        for (int j = 0; j < FRONT; ++j) {
          const int k = base + j;
          if (k >= 1 && k < P) {
            acc[0] = ACC_IS_IN ? step_vec<T, OP>(acc[0], x[j]) : step_vec<T, OP, TRUTH>(x[j], acc[0]);
            if (k + FRONT - 1 < P) {
              x[(j + FRONT - 1) % FRONT] = load_after(TL::rsrc(next_in + vin + tb, nrec), acc[0]);
              req = next_rank(req, p.dir, P);
              next_in = p.in[req];
            }
            asm volatile("" : "+v"(acc[0]));
          }
        }
      }
    } else {
      // The streams are taken in batches of a compile-time size - the pointers of a batch, then all its
      // loads, then all its steps, no branch in between.
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
          if constexpr (TRUTH) {
            if (P >= 2) {
#pragma unroll
              for (int u = 0; u < U; ++u) acc[u] = truth_vec<T>(acc[u]);
            }
          }
        }
#pragma unroll
        for (int b = FIRST ? 1 : 0; b < R; ++b) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            acc[u] = ACC_IS_IN ? step_vec<T, OP>(acc[u], x[b][u]) : step_vec<T, OP, TRUTH>(x[b][u], acc[u]);
        }
      };
      using Yes = std::true_type;
      using No = std::false_type;
      // Up to eight streams in one batch; beyond that a first batch that leaves a multiple of six.
      // For 8- and 16-bit types, whose arithmetic needs registers as well, the kernel then no longer
      // fits two waves per SIMD, and the second wave is what hides the waits for the neighbouring
      // tile (bf16, a block one element into its buffer: 5.2 TB/s against 4.5): batches of five and four.
      constexpr bool kSmall = sizeof(T) <= 2;
      constexpr int B0 = kSmall ? 5 : 8, B = kSmall ? 4 : 6;
      int left = P;
      switch (P <= B0 ? P : (P - 1) % B + 1) {
      case 8: if constexpr (B0 >= 8) { batch(std::integral_constant<int, 8>{}, Yes{}); left -= 8; } break;
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
    if constexpr (BLOCK) {
      // (one buffer after the other: with store_to_outputs the compiler keeps fewer of the loads above in
      // flight, 194 instead of 254 registers in the fp32 tree over eight slots)
      for (int j = j0; j < j0 + nj; ++j) {
        const auto r = TL::rsrc(p.out[j] + vout + tb, nrec);
#pragma unroll
        for (int u = 0; u < U; ++u) tl.store(r, u, acc[u]);
      }
    } else {
      store_to_outputs<TL, U>(tl, p.out, j0, nj, vout + tb, nrec, acc);
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
    // the head elements and the vlen % N elements behind the last whole vector (up to 1 KiB's worth and
    // 15 of them), one per thread of the segment's first workgroups
    const size_t loose = head + vlen % N;
    if (loose) {
      const size_t ntiles = vec_bytes ? (vec_bytes + TL::BYTES - 1) / TL::BYTES : 1, mine = (size_t)p.seg.tile0 + blockIdx.x;
      if (mine < ntiles) {
        for (size_t t = mine * THREADS + threadIdx.x; t < loose; t += ntiles * THREADS) {
          const size_t e = t < head ? t : (vlen / N) * N + t;
          fold_elem<T, OP, ACC_IS_IN>(p, P, s, in_bytes, j0, nj, out_bytes, e);
        }
      }
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
    using Stream = Shape<T, OP, false>;
    using Chained = Shape<T, OP, true>;
    static_assert(Tile<Stream::U, Stream::THREADS>::BYTES == kStreamTileBytes && Tile<Chained::U, Chained::THREADS>::BYTES == kBlockTileBytes,
                  "alamd_planned_launches counts in these tiles");
    const size_t total_bytes = (size_t)nseg * max_len * sizeof(T) * (size_t)(p.P + (p.seg.out_mode == OUT_ALL ? p.seg.nout : 1));
    constexpr size_t kBlockTile = Tile<Chained::U, Chained::THREADS>::BYTES;
    const size_t block_tiles = (size_t)nseg * ((max_len * sizeof(T) + kBlockTile - 1) / kBlockTile);
    // (the number of CUs only matters to launches of few rounds: the others do not ask for it)
    const size_t stream_tiles = (size_t)nseg * ((max_len * sizeof(T) + kStreamTileBytes - 1) / kStreamTileBytes);
    const int cus = stream_tiles <= kFewRoundsTiles ? device_cus() : 0;
    const bool block = !chain && use_block_shape(total_bytes, p.P, p.seg.out_mode == OUT_ALL ? p.seg.nout : 1, false, block_tiles, cus);
    const size_t tile_bytes = block ? kBlockTile : Tile<Stream::U, Stream::THREADS>::BYTES;
    const size_t tile_elems = tile_bytes / sizeof(T);
    FoldParams q = p;
    q.div = make_divisor(p.P);
    q.chain = ChainParams{nullptr, nullptr, nullptr, 0, 0, 0};
    q.seg.simple = 0;
    if (chain) {
      // one segment, one output, every tile in one launch, tiles handed out by the ticket counter
      if (nseg != 1) return set_error(ALAMD_ERR_INVALID_ARG, "a chained fold has one segment");
      constexpr size_t N = 16 / sizeof(T);
      constexpr size_t kChainTile = Tile<Chained::U, Chained::THREADS>::BYTES;
      const size_t nvec = (max_len / N * 16 + kChainTile - 1) / kChainTile;
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
      if constexpr (FP_MINMAX) ck = roles ? fold_vec_kernel<T, OP, true, 0, false, FOLD_CHAINED> : fold_vec_kernel<T, OP, false, 0, false, FOLD_CHAINED>;
      else ck = fold_vec_kernel<T, OP, false, 0, false, FOLD_CHAINED>;
      hipLaunchKernelGGL(ck, dim3((unsigned)tickets, 1, 1), dim3(Chained::THREADS, 1, 1), 0, stream, q);
      ALAMD_HIP(hipGetLastError());
      return ALAMD_OK;
    }
    for (unsigned sg = 0; sg < nseg; ++sg) {
      size_t off, len, out_bytes;
      int j0, nj;
      seg_range(p.seg, sg, off, len);
      out_select(p.seg, p.P, sg, off * sizeof(T), j0, nj, out_bytes);
      const int first = (p.start0 + (int)sg * p.start_stride) % p.P;
      const size_t in_bytes = p.seg.in_blocked ? off * sizeof(T) : 0;
      const bool by_output = !block && tiles_by_output(sizeof(T), p.out[j0] + out_bytes, len, p.P, [&](int k) { return p.in[k] + in_bytes; });
      q.seg.seg_head[sg] = (unsigned short)stream_head_count(sizeof(T), p.out[j0] + out_bytes, p.in[first] + in_bytes, len, by_output);
      if (by_output) q.seg.xcd_run_log2 = kXcdRunLog2;
      if (q.seg.seg_head[sg] || by_output) q.seg.any_head = 1;
    }
    q.seg.simple = nseg == 1 && !q.seg.ragged && q.seg.seg_rem == 0 && !q.seg.in_blocked && q.seg.out_mode == OUT_ALL && q.seg.nout == 1 &&
                   p.start0 >= 0 && p.start0 < p.P;
    auto pick = [&](auto acc_is_in_t, auto front_t) -> void (*)(const FoldParams) {
      constexpr bool A = decltype(acc_is_in_t)::value;
      constexpr int FRONT = decltype(front_t)::value;
      return q.seg.any_head ? fold_vec_kernel<T, OP, A, FRONT, true> : fold_vec_kernel<T, OP, A, FRONT, false>;
    };
    using No = std::false_type;
    using Yes = std::true_type;
    using F2 = std::integral_constant<int, 2>;
    using F3 = std::integral_constant<int, 3>;
    void (*kern)(const FoldParams) = nullptr;
    const size_t front3 = tunables().fold_front3_ranks;
    if ((size_t)p.P >= (front3 ? front3 : (size_t)kFront3FromRanks)) {
      if constexpr (FP_MINMAX) kern = roles ? pick(Yes{}, F3{}) : pick(No{}, F3{});
      else kern = pick(No{}, F3{});
    } else {
      if constexpr (FP_MINMAX) kern = roles ? pick(Yes{}, F2{}) : pick(No{}, F2{});
      else kern = pick(No{}, F2{});
    }
    const size_t per_launch = launch_tiles(p.P, tile_bytes, tunables().launch_bytes);
    const size_t wgs = tunables().stream_wgs_per_cu;
    unsigned lds = stream_lds_bytes(wgs ? (int)wgs : stream_wgs_per_cu(false, p.P, p.seg.out_mode == OUT_ALL ? p.seg.nout : 1, total_bytes,
                                                                           stream_tiles, cus));
    unsigned threads = Stream::THREADS;
    if (block) {
      if constexpr (FP_MINMAX) kern = roles ? fold_vec_kernel<T, OP, true, 0, true, FOLD_BLOCK> : fold_vec_kernel<T, OP, false, 0, true, FOLD_BLOCK>;
      else kern = fold_vec_kernel<T, OP, false, 0, true, FOLD_BLOCK>;
      lds = 0;
      threads = Chained::THREADS;
    }
    plan_launches(q.seg, nseg, max_len, tile_elems, per_launch, [&](size_t t0, size_t nt, unsigned s0, unsigned ns) {
      q.seg.tile0 = t0;
      q.seg.seg0 = s0;
      hipLaunchKernelGGL(kern, dim3((unsigned)nt, ns, 1), dim3(threads, 1, 1), lds, stream, q);
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
