// The tree kernels (included by the translation units that build them, one per
// element type): balanced pairwise combine of up to 32 slots held in
// registers (64 slots as two halves of 32).  Used for floating-point types under the TREE_* orders, where
// the pairing decides the rounding; integer types never need it.
#pragma once

#include "alamd_dispatch.h"
#include "alamd_tile.h"

namespace alamd {

namespace {

// The tree over one element position, one element per access.  HALVES = 2: 2 * SLOTS slots, the
// two halves reduced one after the other and combined by the tree's top level.
// Float min / max: the kernels that honour TreeParams::role_mode.
template <int OP> constexpr bool op_has_roles() { return OP == ALAMD_MIN || OP == ALAMD_MAX; }

// w: slot j reads what slot j ^ w holds (see TreeParams).
template <typename T, int OP, int SLOTS, int HALVES>
__device__ __forceinline__ T tree_elem_value(const TreeParams &p, size_t in_bytes, size_t e, unsigned w = 0) {
  T res;
  // (rolled: unrolled over 64 slots, the table lookups below make the compiler copy the whole argument
  // structure into scratch memory for every wave)
#pragma unroll 1
  for (int h = 0; h < HALVES; ++h) {
    const int base = h * SLOTS;
    const int nvalid = p.nvalid - base;
    if (h > 0 && nvalid <= 0) break;
    T v[SLOTS];
#pragma unroll
    for (int j = 0; j < SLOTS; ++j)
      if (j < nvalid) v[j] = ld_elem<T>(p.a[(base + j) ^ w] + in_bytes + e * sizeof(T));
#pragma unroll
    for (int j = 0; j < SLOTS; ++j)
      if (j < nvalid && p.b[(base + j) ^ w] != nullptr)
        v[j] = Step<T, OP>::apply(v[j], ld_elem<T>(p.b[(base + j) ^ w] + in_bytes + e * sizeof(T)));
#pragma unroll
    for (int d = 1; d < SLOTS; d *= 2) {
#pragma unroll
      for (int i = 0; i + d < SLOTS; i += 2 * d)
        if (i + d < nvalid) v[i] = Step<T, OP>::apply(v[i + d], v[i]);
    }
    res = h == 0 ? v[0] : Step<T, OP>::apply(v[0], res);
  }
  return finish_elem<T, OP>(res, p.div);
}
template <typename T, int OP, int SLOTS, int HALVES>
__device__ __forceinline__ void tree_elem(const TreeParams &p, size_t in_bytes, int j0, int nj,
                                          size_t out_bytes, size_t e, unsigned w = 0) {
  const T res = tree_elem_value<T, OP, SLOTS, HALVES>(p, in_bytes, e, w);
  for (int j = j0; j < j0 + nj; ++j) st_elem<T>(p.out[j] + out_bytes + e * sizeof(T), res);
}

// The elements [lo, hi) of a segment one by one, a workgroup's threads side by side.  per_block: the
// mask changes from block to block of the message (ROLE_PER_BLOCK); the range is then walked block by
// block, so that the mask is the same in every lane and may index the argument tables.
template <typename T, int OP, int SLOTS, int HALVES, int THREADS>
__device__ __forceinline__ void tree_elems(const TreeParams &p, size_t len, size_t in_bytes, int j0, int nj,
                                           size_t out_bytes, size_t lo, size_t hi, unsigned w, bool per_block,
                                           size_t first = threadIdx.x, size_t stride = THREADS) {
  if (!per_block) {
    for (size_t e = lo + first; e < hi; e += stride) tree_elem<T, OP, SLOTS, HALVES>(p, in_bytes, j0, nj, out_bytes, e, w);
    return;
  }
  size_t e0 = lo;
  while (e0 < hi) {
    unsigned long long block_end;
    const unsigned m = (unsigned)__builtin_amdgcn_readfirstlane((int)role_mask_of_elem(p, len, e0, &block_end));
    const size_t stop = block_end < hi ? (size_t)block_end : hi;
    for (size_t e = e0 + first; e < stop; e += stride) tree_elem<T, OP, SLOTS, HALVES>(p, in_bytes, j0, nj, out_bytes, e, m);
    e0 = stop;
  }
}

// Kernel variants: every slot occupied and none pre-folded (P a power of two:
// straight-line code, no uniform branches between the loads and their uses);
// some slots empty (binomial order, P not a power of two); some slots
// pre-folded from a second rank (doubling / halving orders, P not a power of
// two), which needs room for up to twice as many loads in flight.
enum { TREE_FULL = 0, TREE_PARTIAL = 1, TREE_PREFOLD = 2 };

// A large or a small launch streams like the fold does (see Shape there): one wave per workgroup, one vector per
// lane and slot, the two slots of a pair requested together and the next pair as soon as a pair has been
// combined, partial results combined as soon as both halves of a subtree are there; the waves per CU
// are the host's choice per launch (stream_wgs_per_cu in alamd_tile.h).  A second pair requested ahead
// changes nothing; every slot requested up front (128 threads x 8 vectors) runs 5 points lower.
// The block shape (launches of middling size and chained launches: see the fold) keeps tiles of 4 to
// 16 KiB per slot with every load issued up front.
template <typename T, int OP, int SLOTS, int MODE, bool BLOCK = false> struct TreeShape {
  static constexpr bool heavy = sizeof(T) <= 2;
  static constexpr int budget = heavy ? 32 : 64;  // block shape: 128-bit loads in flight per lane
  static constexpr int streams = MODE == TREE_PREFOLD ? 2 * SLOTS : SLOTS;
  static constexpr int block_u = budget / streams >= 8 ? (heavy ? 4 : 8) : (budget / streams >= 1 ? budget / streams : 1);
  static constexpr int U = BLOCK ? block_u : 1;
  static constexpr int THREADS = BLOCK ? (block_u == 8 ? 128 : 256) : 64;
  static constexpr int WAVES = BLOCK ? 2 : kStreamMaxWaves;  // compiled for; see stream_lds_bytes
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
// KIND: FOLD_STREAM, FOLD_BLOCK (built with HEAD = true only) or FOLD_CHAINED: the output overlaps one of
// the inputs at a displacement (see ChainParams and the fold kernel).
template <typename T, int OP, int SLOTS, int MODE, bool HEAD, int HALVES, int KIND = FOLD_STREAM>
__global__ void __launch_bounds__((TreeShape<T, OP, SLOTS, MODE, KIND != FOLD_STREAM>::THREADS))
__attribute__((amdgpu_waves_per_eu(1, TreeShape<T, OP, SLOTS, MODE, KIND != FOLD_STREAM>::WAVES)))
tree_vec_kernel(const TreeParams p) {
  constexpr bool CHAIN = KIND == FOLD_CHAINED, BLOCK = KIND != FOLD_STREAM;
  static_assert(!(CHAIN && HEAD), "a chained launch has no head");
  constexpr int U = TreeShape<T, OP, SLOTS, MODE, BLOCK>::U, THREADS = TreeShape<T, OP, SLOTS, MODE, BLOCK>::THREADS;
  constexpr int N = 16 / sizeof(T);
  static_assert(HALVES == 1 || MODE != TREE_PREFOLD, "a pre-fold never meets more than 32 slots");
  using TL = Tile<U, THREADS>;
  const TL tl;
  // (a launch over one whole segment into one output skips the lookups: see the fold kernel)
  unsigned seg = 0;
  size_t off = 0, len = p.seg.seg_base, in_bytes = 0, out_bytes = 0;
  int j0 = 0, nj = 1;
  if (!p.seg.simple) {
    seg = seg_of(p.seg, blockIdx.y + p.seg.seg0);
    seg_range(p.seg, seg, off, len);
    const size_t off_bytes = off * sizeof(T);
    in_bytes = p.seg.in_blocked ? off_bytes : 0;
    tree_out_select(p, seg, off_bytes, in_bytes, j0, nj, out_bytes);
  }

  const size_t head = HEAD ? arg_u16(p.seg.seg_head, seg) : 0;
  const size_t vlen = len - head;
  const size_t vin = in_bytes + head * sizeof(T), vout = out_bytes + head * sizeof(T);
  const size_t vec_bytes = (vlen / N) * 16;
  unsigned bx = blockIdx.x;
  if constexpr (HEAD && !BLOCK) { if (p.seg.xcd_run_log2) bx = xcd_run_tile(bx, gridDim.x, (unsigned)p.seg.xcd_run_log2); }
  if constexpr (CHAIN) bx = chain_take_tile(p.chain);
  const size_t tb = ((size_t)p.seg.tile0 + bx) * TL::BYTES;
  // float min / max: the slot mask of this tile (uniform), or, where a tile straddles two blocks of a
  // TREE_RSG message, one mask per element
  constexpr bool ROLES = op_has_roles<OP>();
  unsigned w = 0;
  bool mixed = false;
  if constexpr (ROLES) {
    if (p.role_mode == ROLE_PER_SEGMENT) {
      w = role_mask_of_rank(p, (p.role_start0 + (int)seg * p.role_stride) % p.P);
    } else if (p.role_mode == ROLE_PER_BLOCK && tb < vec_bytes) {
      const size_t rem = vec_bytes - tb, nb = rem > TL::BYTES ? TL::BYTES : rem;
      const size_t e0 = head + tb / sizeof(T);
      unsigned long long block_end;
      w = role_mask_of_elem(p, len, e0, &block_end);
      mixed = e0 + nb / sizeof(T) > block_end;
    }
    // (the same in every lane; said explicitly, because it indexes the argument tables)
    w = (unsigned)__builtin_amdgcn_readfirstlane((int)w);
  }
  if (ROLES && !CHAIN && mixed) {
    // one element per access, block by block (never in a chained launch: the host refuses that
    // combination)
    const size_t rem = vec_bytes - tb, nb = rem > TL::BYTES ? TL::BYTES : rem;
    const size_t e0 = head + tb / sizeof(T), ne = nb / sizeof(T);
    tree_elems<T, OP, SLOTS, HALVES, THREADS>(p, len, in_bytes, j0, nj, out_bytes, e0, e0 + ne, w, true);
  } else if (tb < vec_bytes) {
    const size_t rem = vec_bytes - tb;
    const int nrec = rem > TL::BYTES ? (int)TL::BYTES : (int)rem;
    u32x4 res[U];
    if constexpr (!BLOCK) {
      static_assert(U == 1, "the streaming body holds one vector per lane and slot");
      // a later load takes its offset from an empty asm statement that reads the result of the pair
      // before it, so that it cannot be issued any earlier
      auto load_after = [&](const char *base, const u32x4 &after) {
        unsigned vo = tl.vo;
        asm volatile("" : "+v"(vo) : "v"(after));
        return __builtin_amdgcn_raw_buffer_load_b128(TL::rsrc(base + vin + tb, nrec), vo, 0, kAuxLoadStream);
      };
      // (the two halves of 33 to 64 slots run through the same code one after the other: unrolled, the
      // body outgrows what the compiler will unroll of the loop over the slots, and the arrays below
      // end up in scratch memory)
#pragma unroll 1
      for (int h = 0; h < HALVES; ++h) {
        const int base = h * SLOTS;
        const int nvalid = MODE == TREE_FULL ? SLOTS : p.nvalid - base;
        if (h > 0 && nvalid <= 0) break;
        // la / lb: what slot j and the rank pre-folded into it have sent; v: the partial results
        u32x4 la[SLOTS], lb[SLOTS], v[SLOTS];
        // the buffers of slot j (with a mask in play their table index is only known here): fetched a
        // pair ahead of their request, so that no scalar load sits between one request and the next
        const char *pa[SLOTS], *pb[SLOTS];
        auto fetch = [&](int j) {
          if (j < SLOTS && j < nvalid) {
            const int sl = ROLES ? (base + j) ^ (int)w : base + j;
            pa[j] = p.a[sl];
            if constexpr (MODE == TREE_PREFOLD) pb[j] = p.b[sl];
          }
        };
        auto request = [&](int j, const u32x4 &after, bool first) {
          if (j < nvalid) {
            la[j] = first ? tl.load(TL::rsrc(pa[j] + vin + tb, nrec), 0) : load_after(pa[j], after);
            if constexpr (MODE == TREE_PREFOLD) {
              if (pb[j] != nullptr) lb[j] = first ? tl.load(TL::rsrc(pb[j] + vin + tb, nrec), 0) : load_after(pb[j], after);
            }
          }
        };
        // the leaf of slot j: its own data, with the pre-folded rank's combined in (the odd rank keeps
        // step(in = even rank, inout = odd rank))
        auto leaf = [&](int j) {
          u32x4 x = la[j];
          if constexpr (MODE == TREE_PREFOLD) {
            if (pb[j] != nullptr) x = step_vec<T, OP>(x, lb[j]);
          }
          return x;
        };
        const u32x4 none = {0u, 0u, 0u, 0u};
        fetch(0);
        fetch(1);
        request(0, none, true);
        request(1, none, true);
        fetch(2);
        fetch(3);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < SLOTS; j += 2) {
          if (j < nvalid) {
            v[j] = leaf(j);
            if (j + 1 < nvalid) v[j] = step_vec<T, OP>(leaf(j + 1), v[j]);
            if (j + 2 < SLOTS) request(j + 2, v[j], false);
            if (j + 3 < SLOTS) request(j + 3, v[j], false);
            fetch(j + 4);
            fetch(j + 5);
            asm volatile("" : "+v"(v[j]));
          }
          // the subtrees that end with this pair: distance 2, 4, ...
#pragma unroll
          for (int d = 2; d < SLOTS; d *= 2) {
            if ((j + 2) % (2 * d) != 0) break;
            const int i = j + 2 - 2 * d;
            if (i + d < nvalid) {
              v[i] = step_vec<T, OP>(v[i + d], v[i]);
              asm volatile("" : "+v"(v[i]));
            }
          }
        }
        res[0] = h == 0 ? v[0] : step_vec<T, OP>(v[0], res[0]);
      }
    } else {
#pragma unroll
    for (int h = 0; h < HALVES; ++h) {
      const int base = h * SLOTS;
      const int nvalid = MODE == TREE_FULL ? SLOTS : p.nvalid - base;
      if (h > 0 && nvalid <= 0) break;
      u32x4 v[SLOTS][U];
#pragma unroll
      for (int j = 0; j < SLOTS; ++j) {
        if (j < nvalid) {
          const auto r = TL::rsrc(p.a[ROLES ? (base + j) ^ w : base + j] + vin + tb, nrec);
#pragma unroll
          for (int u = 0; u < U; ++u) v[j][u] = tl.load(r, u);
        }
      }
      if constexpr (MODE == TREE_PREFOLD) {
        // pre-folded slots: the odd rank keeps step(in = even rank, inout = odd rank); all of
        // their loads are issued before the first use, like the slots' own
        u32x4 pre[SLOTS][U];
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
          if (j < nvalid && p.b[ROLES ? j ^ w : j] != nullptr) {
            const auto r = TL::rsrc(p.b[ROLES ? j ^ w : j] + vin + tb, nrec);
#pragma unroll
            for (int u = 0; u < U; ++u) pre[j][u] = tl.load(r, u);
          }
        }
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
          if (j < nvalid && p.b[ROLES ? j ^ w : j] != nullptr) {
#pragma unroll
            for (int u = 0; u < U; ++u) v[j][u] = step_vec<T, OP>(v[j][u], pre[j][u]);
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
    }
#pragma unroll
    for (int u = 0; u < U; ++u) res[u] = finish_vec<T, OP>(res[u], p.div);
    if constexpr (CHAIN) chain_gate(p.chain, bx, tb, (unsigned long long)nrec, (unsigned)TL::BYTES);
    if constexpr (BLOCK) {
      // (one buffer after the other: with store_to_outputs the compiler keeps fewer of the loads above in
      // flight, 194 instead of 254 registers in the fp32 tree over eight slots)
      for (int j = j0; j < j0 + nj; ++j) {
        const auto r = TL::rsrc(p.out[j] + vout + tb, nrec);
#pragma unroll
        for (int u = 0; u < U; ++u) tl.store(r, u, res[u]);
      }
    } else {
      store_to_outputs<TL, U>(tl, p.out, j0, nj, vout + tb, nrec, res);
    }
  }
  if constexpr (CHAIN) {
    // the vlen % N elements behind the last whole vector are the last ticket
    if (bx == p.chain.nvec_tiles) {
      const bool mine = threadIdx.x < vlen % N;
      const size_t e = (vlen / N) * N + threadIdx.x;
      T val = T();
      // (never with a mask per block: the host refuses that combination)
      if (mine) val = tree_elem_value<T, OP, SLOTS, HALVES>(p, in_bytes, e, w);
      chain_gate(p.chain, bx, vec_bytes, (vlen % N) * sizeof(T), (unsigned)TL::BYTES);
      if (mine) st_elem<T>(p.out[j0] + out_bytes + e * sizeof(T), val);
    }
  } else {
    // the head elements and the vlen % N elements behind the last whole vector, spread over the
    // segment's first workgroups
    if (head + vlen % N) {
      const size_t ntiles = vec_bytes ? (vec_bytes + TL::BYTES - 1) / TL::BYTES : 1, mine = (size_t)p.seg.tile0 + blockIdx.x;
      if (mine < ntiles) {
        const bool per_block = ROLES && p.role_mode == ROLE_PER_BLOCK;
        const size_t tail = head + (vlen / N) * N, first = mine * THREADS + threadIdx.x, stride = ntiles * THREADS;
        tree_elems<T, OP, SLOTS, HALVES, THREADS>(p, len, in_bytes, j0, nj, out_bytes, 0, head, w, per_block, first, stride);
        tree_elems<T, OP, SLOTS, HALVES, THREADS>(p, len, in_bytes, j0, nj, out_bytes, tail, tail + vlen % N, w, per_block, first, stride);
      }
    }
  }
}


struct ChainArgs { const ChainScratch *scratch; size_t displ_bytes; };

template <typename T, int OP, int SLOTS, int MODE, int HALVES = 1>
int launch_tree_mode(const TreeParams &p, unsigned nseg, size_t max_len, hipStream_t stream, ChainArgs chain) {
  using S = TreeShape<T, OP, SLOTS, MODE, false>;
  using C = TreeShape<T, OP, SLOTS, MODE, true>;
  static_assert(Tile<S::U, S::THREADS>::BYTES == kStreamTileBytes, "the tile of a streaming launch");
  const size_t total_bytes = (size_t)nseg * max_len * sizeof(T) * (size_t)(p.P + (p.seg.out_mode == OUT_ALL ? p.seg.nout : 1));
  constexpr size_t kBlockTile = Tile<C::U, C::THREADS>::BYTES;
  const size_t block_tiles = (size_t)nseg * ((max_len * sizeof(T) + kBlockTile - 1) / kBlockTile);
  const size_t stream_tiles = (size_t)nseg * ((max_len * sizeof(T) + kStreamTileBytes - 1) / kStreamTileBytes);
  const int cus = stream_tiles <= kFewRoundsTiles ? device_cus() : 0;
  const bool block = !chain.scratch && use_block_shape(total_bytes, p.P, p.seg.out_mode == OUT_ALL ? p.seg.nout : 1, true, block_tiles, cus, kBlockTile);
  const size_t tile_bytes = block ? kBlockTile : Tile<S::U, S::THREADS>::BYTES;
  const size_t tile_elems = tile_bytes / sizeof(T);
  const size_t per_launch = launch_tiles(p.P, tile_bytes, tunables().launch_bytes);
  TreeParams q = p;
  q.div = make_divisor(p.P);
  q.chain = ChainParams{nullptr, nullptr, nullptr, 0, 0, 0};
  q.seg.simple = 0;
  q.role_n = q.role_blk = 0;
  q.role_inv_blk = q.role_inv_blk1 = 0.0;
  if (p.role_mode == ROLE_PER_BLOCK) {
    // the message every segment belongs to, if it is the same for all and short enough for exact doubles
    const unsigned long long n = p.role_count ? p.role_count : (!p.seg.ragged && p.seg.seg_rem == 0 ? p.seg.seg_base : 0);
    if (n != 0 && n < (1ull << 52)) {
      q.role_n = n;
      q.role_blk = n >> p.role_bits;
      q.role_inv_blk = q.role_blk ? 1.0 / (double)q.role_blk : 0.0;
      q.role_inv_blk1 = 1.0 / (double)(q.role_blk + 1);
    }
  }
  if (chain.scratch) {
    if (nseg != 1) return set_error(ALAMD_ERR_INVALID_ARG, "a chained combine has one segment");
    if (op_has_roles<OP>() && p.role_mode == ROLE_PER_BLOCK)
      return set_error(ALAMD_ERR_INVALID_ALGO, "a float min / max under the reduce-scatter + gather order is not available "
                       "for an in-place block that overlaps its own input");
    constexpr size_t N = 16 / sizeof(T);
    const size_t tile_bytes = Tile<C::U, C::THREADS>::BYTES;
    const size_t nvec = (max_len / N * 16 + tile_bytes - 1) / tile_bytes;
    const size_t tickets = nvec + (max_len % N ? 1 : 0);
    if (nvec > chain.scratch->max_tiles || tickets > 0x7fffffffull)
      return set_error(ALAMD_ERR_INVALID_ARG, "in-place block of %zu elements needs %zu tile flags, the scratch holds %zu",
                       max_len, nvec, chain.scratch->max_tiles);
    int rc = chain_clear(*chain.scratch, nvec, stream);
    if (rc) return rc;
    q.chain = ChainParams{chain.scratch->ticket, chain.scratch->flags, chain.scratch->error, chain.displ_bytes,
                          (unsigned)nvec, chain.scratch->max_polls};
    q.seg.tile0 = 0;
    q.seg.seg0 = 0;
    q.seg.mapped = 0;
    // only the most general variants are built for chained launches
    if constexpr (MODE == TREE_PREFOLD || (HALVES == 2 && MODE == TREE_PARTIAL)) {
      hipLaunchKernelGGL((tree_vec_kernel<T, OP, SLOTS, MODE, false, HALVES, FOLD_CHAINED>), dim3((unsigned)tickets, 1, 1),
                         dim3(C::THREADS, 1, 1), 0, stream, q);
      ALAMD_HIP(hipGetLastError());
      return ALAMD_OK;
    } else {
      return set_error(ALAMD_ERR_INVALID_ARG, "tree combine: no chained variant of this mode");
    }
  }
  for (unsigned sg = 0; sg < nseg; ++sg) {
    size_t off, len, out_bytes;
    int j0, nj;
    seg_range(p.seg, sg, off, len);
    const size_t in_bytes = p.seg.in_blocked ? off * sizeof(T) : 0;
    tree_out_select(p, sg, off * sizeof(T), in_bytes, j0, nj, out_bytes);
    const bool by_output = !block && tiles_by_output(sizeof(T), p.out[j0] + out_bytes, len, 2 * SLOTS * HALVES, [&](int k) {
      const char *in = k < SLOTS * HALVES ? p.a[k] : p.b[k - SLOTS * HALVES];
      return in ? in + in_bytes : nullptr;
    });
    q.seg.seg_head[sg] = (unsigned short)stream_head_count(sizeof(T), p.out[j0] + out_bytes, p.a[0] + in_bytes, len, by_output);
    if (by_output) q.seg.xcd_run_log2 = kXcdRunLog2;
    if (q.seg.seg_head[sg] || by_output) q.seg.any_head = 1;
  }
  q.seg.simple = nseg == 1 && !q.seg.ragged && q.seg.seg_rem == 0 && !q.seg.in_blocked && q.seg.out_mode == OUT_ALL && q.seg.nout == 1;
  const size_t wgs = tunables().stream_wgs_per_cu;
  unsigned lds = stream_lds_bytes(wgs ? (int)wgs : stream_wgs_per_cu(true, SLOTS * HALVES, p.seg.out_mode == OUT_ALL ? p.seg.nout : 1, total_bytes,
                                                                         stream_tiles, cus));
  unsigned threads = S::THREADS;
  void (*kern)(const TreeParams) =
      q.seg.any_head ? tree_vec_kernel<T, OP, SLOTS, MODE, true, HALVES> : tree_vec_kernel<T, OP, SLOTS, MODE, false, HALVES>;
  if (block) {
    kern = tree_vec_kernel<T, OP, SLOTS, MODE, true, HALVES, FOLD_BLOCK>;
    lds = 0;
    threads = C::THREADS;
  }
  plan_launches(q.seg, nseg, max_len, tile_elems, per_launch, [&](size_t t0, size_t nt, unsigned s0, unsigned ns) {
    q.seg.tile0 = t0;
    q.seg.seg0 = s0;
    hipLaunchKernelGGL(kern, dim3((unsigned)nt, ns, 1), dim3(threads, 1, 1), lds, stream, q);
  });
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

template <typename T, int OP, int SLOTS>
int launch_tree_slots(const TreeParams &p, unsigned nseg, size_t max_len, hipStream_t stream, ChainArgs chain) {
  bool prefold = false;
  for (int j = 0; j < SLOTS; ++j) prefold = prefold || p.b[j] != nullptr;
  // a chained launch takes the most general variant whatever the slots hold: fewer kernels to build
  if (prefold || chain.scratch) return launch_tree_mode<T, OP, SLOTS, TREE_PREFOLD>(p, nseg, max_len, stream, chain);
  if (p.nvalid == SLOTS) return launch_tree_mode<T, OP, SLOTS, TREE_FULL>(p, nseg, max_len, stream, chain);
  return launch_tree_mode<T, OP, SLOTS, TREE_PARTIAL>(p, nseg, max_len, stream, chain);
}

// 33 to 64 slots: two halves of 32.
template <typename T, int OP>
int launch_tree_two_halves(const TreeParams &p, unsigned nseg, size_t max_len, hipStream_t stream, ChainArgs chain) {
  for (int j = 0; j < 64; ++j)
    if (p.b[j] != nullptr) return set_error(ALAMD_ERR_INVALID_ARG, "tree combine: pre-fold beyond 32 slots");
  if (p.nvalid == 64 && !chain.scratch) return launch_tree_mode<T, OP, 32, TREE_FULL, 2>(p, nseg, max_len, stream, chain);
  return launch_tree_mode<T, OP, 32, TREE_PARTIAL, 2>(p, nseg, max_len, stream, chain);
}

// The launches of one element type.
template <typename T>
int launch_tree_of(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int op, hipStream_t stream,
                   const ChainScratch *scratch, size_t displ_bytes) {
  const ChainArgs chain = {scratch, displ_bytes};
  return dispatch_fp_op<T>(op, [&](auto tt, auto ot) -> int {
    using TT = typename decltype(tt)::type;
    constexpr int OP = decltype(ot)::value;
    switch (slots) {
    case 2: return launch_tree_slots<TT, OP, 2>(p, nseg, max_len, stream, chain);
    case 4: return launch_tree_slots<TT, OP, 4>(p, nseg, max_len, stream, chain);
    case 8: return launch_tree_slots<TT, OP, 8>(p, nseg, max_len, stream, chain);
    case 16: return launch_tree_slots<TT, OP, 16>(p, nseg, max_len, stream, chain);
    case 32: return launch_tree_slots<TT, OP, 32>(p, nseg, max_len, stream, chain);
    case 64: return launch_tree_two_halves<TT, OP>(p, nseg, max_len, stream, chain);
    default: return set_error(ALAMD_ERR_INVALID_ARG, "tree combine: bad slot count %d", slots);
    }
  });
}

}  // namespace
}  // namespace alamd
