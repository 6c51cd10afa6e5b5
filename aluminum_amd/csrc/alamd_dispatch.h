// Run-time (dtype, op) -> compile-time <T, OP> dispatch shared by the kernel
// translation units.
#pragma once

#include "alamd_common.h"
#include "alamd_tile.h"

namespace alamd {

template <typename T> struct TypeTag { using type = T; };
template <int OP> struct OpTag { static constexpr int value = OP; };

// Integer ops other than min / max do not depend on signedness, so signed
// types share the kernels of the unsigned type of the same width.
template <typename S, typename F> int dispatch_int_op(int op, F &&f) {
  using U = typename unsigned_of<S>::type;
  switch (op) {
  case ALAMD_SUM: return f(TypeTag<U>{}, OpTag<ALAMD_SUM>{});
  case ALAMD_PROD: return f(TypeTag<U>{}, OpTag<ALAMD_PROD>{});
  case ALAMD_MIN: return f(TypeTag<S>{}, OpTag<ALAMD_MIN>{});
  case ALAMD_MAX: return f(TypeTag<S>{}, OpTag<ALAMD_MAX>{});
  case ALAMD_LOR: return f(TypeTag<U>{}, OpTag<ALAMD_LOR>{});
  case ALAMD_LAND: return f(TypeTag<U>{}, OpTag<ALAMD_LAND>{});
  case ALAMD_LXOR: return f(TypeTag<U>{}, OpTag<ALAMD_LXOR>{});
  case ALAMD_BOR: return f(TypeTag<U>{}, OpTag<ALAMD_BOR>{});
  case ALAMD_BAND: return f(TypeTag<U>{}, OpTag<ALAMD_BAND>{});
  case ALAMD_BXOR: return f(TypeTag<U>{}, OpTag<ALAMD_BXOR>{});
  case ALAMD_AVG: return f(TypeTag<S>{}, OpTag<ALAMD_AVG>{});  // the final division depends on the sign
  default: return set_error(ALAMD_ERR_UNSUPPORTED_OP, "Reduction operator not supported");
  }
}

template <typename T, typename F> int dispatch_fp_op(int op, F &&f) {
  switch (op) {
  case ALAMD_SUM: return f(TypeTag<T>{}, OpTag<ALAMD_SUM>{});
  case ALAMD_PROD: return f(TypeTag<T>{}, OpTag<ALAMD_PROD>{});
  case ALAMD_MIN: return f(TypeTag<T>{}, OpTag<ALAMD_MIN>{});
  case ALAMD_MAX: return f(TypeTag<T>{}, OpTag<ALAMD_MAX>{});
  case ALAMD_AVG: return f(TypeTag<T>{}, OpTag<ALAMD_AVG>{});
  default: return set_error(ALAMD_ERR_UNSUPPORTED_OP, "Reduction operator not supported");
  }
}

// Calls f(TypeTag<T>, OpTag<OP>) for the kernel types of a float dtype.
template <typename F> int dispatch_float(int dtype, int op, F &&f) {
  switch (dtype) {
  case ALAMD_F16: return dispatch_fp_op<f16_t>(op, f);
  case ALAMD_BF16: return dispatch_fp_op<bf16_t>(op, f);
  case ALAMD_F32: return dispatch_fp_op<float>(op, f);
  case ALAMD_F64: return dispatch_fp_op<double>(op, f);
  default: return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);
  }
}

template <typename F> int dispatch_any(int dtype, int op, F &&f) {
  switch (dtype) {
  case ALAMD_I8: return dispatch_int_op<int8_t>(op, f);
  case ALAMD_U8: return dispatch_int_op<uint8_t>(op, f);
  case ALAMD_I16: return dispatch_int_op<int16_t>(op, f);
  case ALAMD_U16: return dispatch_int_op<uint16_t>(op, f);
  case ALAMD_I32: return dispatch_int_op<int32_t>(op, f);
  case ALAMD_U32: return dispatch_int_op<uint32_t>(op, f);
  case ALAMD_I64: return dispatch_int_op<int64_t>(op, f);
  case ALAMD_U64: return dispatch_int_op<uint64_t>(op, f);
  default: return dispatch_float(dtype, op, f);
  }
}

// Whether a fold / tree launch takes the block shape (the measurements are in alamd_tile.h, above Tile).
// total_bytes: what it reads and writes in all; streams: ranks it reads; outputs: buffers every tile goes
// to; tiles: how many block-shaped tiles it would have; cus: compute units of the device (<= 0: unknown).
// With the two sizes at their defaults the rule is finer than the window between them:
//  - three and more outputs: always (a streaming wave would write its KiB to every buffer in turn);
//  - otherwise only if the tiles deal out evenly.  A CU gets through block-shaped tiles one at a time
//    (one tile's loads are about what a CU can have in flight), so a launch of t tiles per CU lasts as
//    long as ceil(t) of them: P = 32 fold, 140 / 186 / 279 / 372 / 558 tiles: 13.9 / 15.7 / 30.5 / 34.0 /
//    53.2 us, where streaming takes 17.7 / 19.6 / 23.9 / 31.0 / 47.0 us; P = 8, 21.3 MiB per rank, 5.33
//    tiles per CU: 31.5 us in blocks against 30.0 us streaming; 32 MiB per rank, 8 per CU: 45.7 against
//    47.4.  Up to one tile per CU, or with up to 4 % of the CUs idle in the last round, it is taken.
//    Powers of two from 4 MiB per rank on always deal out evenly;
//  - up to four ranks into one or two buffers: never (every load up front buys little where there are few
//    streams to wait for: P = 4, 8 / 16 / 32 MiB per rank: 12.5 / 23.2 / 48.0 us in blocks against 11.4 /
//    22.0 / 46.9 us);
//  - a tree whose block-shaped tiles are smaller than 16 KiB per slot (from 16 pre-folded slots or 32 slots
//    on, where a lane's loads in flight are used up by the slots): never (48 ranks, 144 MiB in all: 29.0 us
//    in blocks of 4 KiB against 23.0 us);
//  - a fold over 24 ranks and more from half the size on (a streaming wave walks through its streams two
//    or three at a time, P / 2 trips to memory one after the other: 64 ranks, 20 MiB in all: 20.0 us in
//    blocks against 21.0 us, 96 MiB: 23.6 against 31.6).
enum { FOLD_STREAM = 0, FOLD_BLOCK = 1, FOLD_CHAINED = 2 };  // the KIND of a fold / tree kernel
inline bool use_block_shape(size_t total_bytes, int streams, int outputs, bool tree, size_t tiles, int cus,
                            size_t tile_bytes = kBlockTileBytes) {
  const size_t from = tunables().block_shape_from_bytes, below = tunables().block_shape_below_bytes;
  const bool defaults = from == kBlockShapeFromBytes && below == kBlockShapeBelowBytes;
  const bool many = streams >= 24;
  if (total_bytes >= below) return false;
  if (total_bytes < (defaults && many && !tree ? from / 2 : from)) return false;
  if (!defaults) return true;
  if (tile_bytes < kBlockTileBytes) return false;
  if (outputs >= 3) return true;
  if (streams <= 4) return false;
  if (cus <= 0 || tiles <= (size_t)cus) return true;
  const size_t per_cu = (tiles + (size_t)cus - 1) / (size_t)cus;  // ceil(t)
  return (per_cu * (size_t)cus - tiles) * 25 <= per_cu * (size_t)cus;  // idle share <= 4 %
}

// ---- parameters of the two combine kernel families -------------------------

// Work is a grid of segments (blockIdx.y) x tiles (blockIdx.x).  Segment s
// covers elements [s*seg_base + min(s, seg_rem), +seg_base + (s < seg_rem)),
// or, when `ragged` is set, [seg_off[s], +seg_len[s]).
struct SegParams {
  unsigned long long seg_base;
  unsigned long long seg_rem;
  unsigned long long tile0;  // index of the first tile of this launch
  unsigned seg0;             // position of the first segment of this launch
  int mapped;                // 1: the segment at position i is order[i], 0: it is i
  alignas(4) unsigned char order[ALAMD_MAX_RANKS];
  // leading elements of each segment handled one by one (see stream_head_count); the host fills this
  // in, so that no workgroup has to wait for the output pointer before it can issue its loads
  alignas(4) unsigned short seg_head[ALAMD_MAX_RANKS];
  int any_head;              // 0: every seg_head is zero (all buffers 1 KiB aligned: the usual case)
  int in_blocked;   // 1: inputs are read at the segment's offset, 0: at 0
  int out_mode;     // OUT_ALL / OUT_SEG / OUT_OWNER
  int owner_shift;  // OUT_OWNER: output index is (segment + owner_shift) mod P
  int nout;         // OUT_ALL: number of outputs written
  int simple;       // 1: one segment from element 0, one output (the kernels then skip the lookups)
  int xcd_run_log2; // > 0: runs of 2^k consecutive tiles go to one XCD (kernels with HEAD only; see tiles_by_output)
  int ragged;       // 1: segments are given by the two tables below
  unsigned long long seg_off[ALAMD_MAX_RANKS];
  unsigned long long seg_len[ALAMD_MAX_RANKS];
};
enum { OUT_ALL = 0, OUT_SEG = 1, OUT_OWNER = 2 };

// Equal segments (the first seg_rem of them one element longer), everything else zero.
inline SegParams make_seg(size_t seg_base, size_t seg_rem, int in_blocked, int out_mode, int nout) {
  SegParams s = {};
  s.seg_base = seg_base;
  s.seg_rem = seg_rem;
  s.in_blocked = in_blocked;
  s.out_mode = out_mode;
  s.nout = nout;
  return s;
}

// The segment a workgroup works on: launches walk positions, which the host may have sorted by length.
// (These lookups are a chain of dependent scalar loads, one branch per mode.  Reading every table
// whatever the mode and choosing afterwards shortens the chain but ran 2 to 3 % slower for a
// Reduce_scatter; the launches that need no lookup at all skip them instead: SegParams::simple.)
// Entry i of a table of bytes or of 16-bit numbers in the kernel's arguments, i the same in every lane:
// read as the dword it lies in, which is a scalar load; read as what it is, it would be a vector load
// (there are no scalar loads of less than a dword), i.e. a round trip through the memory pipeline that
// a workgroup's first requests would wait for.  Both tables start on a dword.
__device__ __forceinline__ unsigned arg_u8(const unsigned char *table, unsigned i) {
  return (reinterpret_cast<const unsigned *>(table)[i >> 2] >> ((i & 3u) * 8u)) & 0xffu;
}
__device__ __forceinline__ unsigned arg_u16(const unsigned short *table, unsigned i) {
  return (reinterpret_cast<const unsigned *>(table)[i >> 1] >> ((i & 1u) * 16u)) & 0xffffu;
}
// Workgroup i of a launch of n -> tile, so that runs of 2^rl consecutive tiles fall to one XCD (workgroups
// are dealt to the eight XCDs round-robin); the workgroups behind the last whole group of 8 * 2^rl keep
// their own index.
__host__ __device__ __forceinline__ unsigned xcd_run_tile(unsigned i, unsigned n, unsigned rl) {
  const unsigned span = 8u << rl, full = n & ~(span - 1u);
  if (i >= full) return i;
  const unsigned w = i & (span - 1u);
  return (i & ~(span - 1u)) + ((w & 7u) << rl) + (w >> 3);
}
__device__ __forceinline__ unsigned seg_of(const SegParams &s, unsigned pos) {
  return s.mapped ? arg_u8(s.order, pos) : pos;
}

__host__ __device__ inline void seg_range(const SegParams &s, unsigned seg, size_t &off, size_t &len) {
  if (s.ragged) {
    off = s.seg_off[seg];
    len = s.seg_len[seg];
  } else {
    const unsigned long long sg = seg;
    off = sg * s.seg_base + (sg < s.seg_rem ? sg : s.seg_rem);
    len = s.seg_base + (sg < s.seg_rem ? 1u : 0u);
  }
}

// Which outputs a segment writes (out[j0 .. j0 + nj)), and at which byte offset.
__host__ __device__ inline void out_select(const SegParams &s, int P, unsigned seg, size_t off_bytes, int &j0, int &nj,
                                           size_t &out_bytes) {
  if (s.out_mode == OUT_ALL) { j0 = 0; nj = s.nout; out_bytes = s.in_blocked ? off_bytes : 0; }
  else if (s.out_mode == OUT_SEG) { j0 = (int)seg; nj = 1; out_bytes = 0; }
  else { j0 = ((int)seg + s.owner_shift) % P; nj = 1; out_bytes = off_bytes; }
}

// ---- a fold whose output overlaps one of its inputs at a displacement ---------
//
// An in-place Reduce_scatterv writes block b's result to elements [0, n) of
// rank b's buffer while that rank's contribution is read from [displ, displ + n)
// of the same buffer: with 0 < displ < n the tile that writes a range must not
// store before the tiles that read that range have loaded it.  One launch does
// this without any order among workgroups being assumed:
//  - a workgroup takes its tile from a ticket counter, so every tile with a
//    lower number is held by a workgroup that is already running;
//  - when the loads of a tile have landed (values in registers) its workgroup
//    sets the tile's flag, and only then waits for the flags of the (at most
//    two) lower-numbered tiles whose reads overlap its own writes; a flag is set
//    before any wait, so no wait can be circular;
//  - the elements behind the last whole vector are one more ticket, handled
//    the same way.
// The counter and the flags are scratch memory in HBM, cleared on the stream
// before the launch.  A wait is bounded: if it expires (it cannot, unless the
// device loses a workgroup) the error word, which the host can read, is set and
// the workgroup goes on.
struct ChainParams {
  unsigned *ticket;                 // next tile; null: not a chained launch
  unsigned *flags;                  // flags[t] != 0: tile t has loaded its inputs
  unsigned *error;                  // set to 1 by a wait that expired
  unsigned long long displ_bytes;   // the overlapping input starts this far behind the output
  unsigned nvec_tiles;              // whole-vector tiles (the tail is ticket nvec_tiles)
  unsigned max_polls;               // polls of one flag before a wait gives up
};
constexpr unsigned kChainDefaultPolls = 1u << 24;

__device__ __forceinline__ unsigned chain_take_tile(const ChainParams &c) {
  __shared__ unsigned s_tile;
  if (threadIdx.x == 0) s_tile = __hip_atomic_fetch_add(c.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  return s_tile;
}

// Called by every thread of the workgroup that holds tile `self`, between the last use of the loaded
// values and the first store to bytes [w0, w0 + wlen) of the output.
__device__ __forceinline__ void chain_gate(const ChainParams &c, unsigned self, unsigned long long w0,
                                           unsigned long long wlen, unsigned tile_bytes) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's loads have returned
  __syncthreads();                                  // ... and every other wave's of the workgroup
  if (threadIdx.x == 0) {
    // Nothing this workgroup wrote has to become visible with the flag, and a waiting workgroup reads nothing
    // that this one wrote: the flag only says "my loads are done".  Relaxed accesses that go past the caches
    // are therefore enough; release / acquire would add a write-back and an invalidation of the L2 per tile.
    if (self < c.nvec_tiles) __hip_atomic_store(&c.flags[self], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    // tiles t that read output bytes [w0, w0 + wlen): displ + t*TB < w0 + wlen and displ + (t+1)*TB > w0
    const long long tb = (long long)tile_bytes;
    const long long a0 = (long long)w0 - (long long)c.displ_bytes, a1 = a0 + (long long)wlen;
    if (a1 > 0 && self > 0) {
      long long lo = a0 <= 0 ? 0 : a0 / tb;            // floor
      long long hi = (a1 + tb - 1) / tb - 1;           // ceil - 1
      if (hi > (long long)self - 1) hi = (long long)self - 1;
      if (hi > (long long)c.nvec_tiles - 1) hi = (long long)c.nvec_tiles - 1;
      // max_polls == 0 (a test's setting): a wait that the tiling calls for gives up without looking
      if (c.max_polls == 0 && lo <= hi) __hip_atomic_store(c.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      for (long long t = lo; t <= hi && c.max_polls != 0; ++t) {
        unsigned spins = 0;
        while (__hip_atomic_load(&c.flags[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) == 0u) {
          __builtin_amdgcn_s_sleep(2);
          if (++spins >= c.max_polls) {
            __hip_atomic_store(c.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            break;
          }
        }
      }
    }
  }
  __syncthreads();
}

// Left fold over a rotated rank sequence.
struct FoldParams {
  const char *in[ALAMD_MAX_RANKS];
  char *out[ALAMD_MAX_RANKS];
  SegParams seg;
  int P;
  int start0;        // first operand of segment s is rank (start0 + s*start_stride) mod P
  int start_stride;
  int dir;           // +1: next operand is rank+1, -1: rank-1 (with wrap)
  Divisor div;       // avg: the number of ranks as a divisor
  ChainParams chain; // set for a chained launch only
};

// Balanced pairwise tree over up to 64 slots.  Slot j holds a[j], or
// step(in = a[j], inout = b[j]) when b[j] is set (only among the first 32: a
// pre-fold leaves at most 32 slots); slots >= nvalid are empty.
// Level d = 1,2,4..: slot i (multiple of 2d) = step(in = slot i+d, inout = slot i).
//
// Operand roles (which of the two partial results of a pair is the inoutvec) only show in the bits of
// a float min / max, where a tie or a NaN lets the invec through.  Two orders let them depend on
// where the result goes: TREE_HALV (a recursive-halving reduce-scatter: at every level the half that
// holds the receiving rank keeps its own data) and TREE_RSG (reduce-scatter by recursive halving of
// the data plus gather: the same, per block of the message).  In both, the side that keeps is the same
// for every pair of a level, so the tree with fixed roles gives the right bits once slot j reads what
// slot j ^ w would have read, w being the slot of the survivor the result is for: the min / max
// kernels apply that mask (role_mode), the others ignore it.
enum { ROLE_FIXED = 0, ROLE_PER_SEGMENT = 1, ROLE_PER_BLOCK = 2 };
struct TreeParams {
  const char *a[ALAMD_MAX_RANKS];
  const char *b[ALAMD_MAX_RANKS];
  char *out[ALAMD_MAX_RANKS];
  SegParams seg;
  int P;        // number of ranks (for OUT_OWNER)
  int nvalid;   // occupied slots
  Divisor div;  // avg: the number of ranks as a divisor
  ChainParams chain;  // set for a chained launch only
  int role_mode;                     // ROLE_*
  int role_rem, role_bits;           // P = 2^role_bits + role_rem
  int role_start0, role_stride;      // ROLE_PER_SEGMENT: segment s is for rank (role_start0 + s * role_stride) mod P
  unsigned long long role_base;      // ROLE_PER_BLOCK: element 0 of a segment is element role_base of the message,
  unsigned long long role_count;     // which has role_count elements (0: the segment is the message)
  int role_spread;                   // ROLE_PER_BLOCK: how the message is cut into blocks, see role_mask_of_elem
  // ROLE_PER_BLOCK, filled in by the launcher when every segment's message has the same known length:
  // that length, its block length and the reciprocals of the two block lengths there are, so that a
  // workgroup finds its block without a 64-bit division
  unsigned long long role_n, role_blk;
  double role_inv_blk, role_inv_blk1;
};

__host__ __device__ inline unsigned role_bit_reverse(unsigned v, int bits) {
  unsigned r = 0;
  for (int b = 0; b < bits; ++b) r |= ((v >> b) & 1u) << (bits - 1 - b);
  return r;
}
// ROLE_PER_SEGMENT: the slot mask of the segment whose result is for `rank` (the halving tree lists the
// survivors in bit-reversed order).
__host__ __device__ inline unsigned role_mask_of_rank(const TreeParams &p, int rank) {
  const int o = rank < 2 * p.role_rem ? rank / 2 : rank - p.role_rem;
  return role_bit_reverse((unsigned)o, p.role_bits);
}
// ROLE_PER_BLOCK: the message is cut into 2^role_bits blocks of count >> role_bits elements; what that
// leaves over goes to the last block (TREE_RSG) or, role_spread, one element each to the first blocks
// (TREE_RSG_SPREAD).  Block k ends up on survivor bit_reverse(k).
// x / d from the reciprocal of d (x < 2^53, d > 0): the rounded product is within one of the quotient.
__host__ __device__ inline unsigned long long role_div(unsigned long long x, unsigned long long d, double inv) {
  unsigned long long q = (unsigned long long)((double)x * inv);
  if (q * d > x) --q;
  else if ((q + 1) * d <= x) ++q;
  return q;
}
// *end: the element of the segment at which that block ends (for the last block: beyond every element).
__host__ __device__ inline unsigned role_mask_of_elem(const TreeParams &p, size_t seg_len, size_t e,
                                                      unsigned long long *end = nullptr) {
  const bool fast = p.role_n != 0;
  const unsigned long long n = fast ? p.role_n : (p.role_count ? p.role_count : seg_len);
  const unsigned long long blk = fast ? p.role_blk : n >> p.role_bits;
  const unsigned long long last = (1ull << p.role_bits) - 1, x = p.role_base + e;
  unsigned long long k, stop;
  if (p.role_spread) {
    const unsigned long long longer = n & last, cut = longer * (blk + 1);  // `longer` blocks of blk + 1 come first
    if (x < cut) k = fast ? role_div(x, blk + 1, p.role_inv_blk1) : x / (blk + 1);
    else k = blk ? longer + (fast ? role_div(x - cut, blk, p.role_inv_blk) : (x - cut) / blk) : last;
    if (k > last) k = last;
    stop = k * blk + (k < longer ? k : longer) + blk + (k < longer ? 1 : 0);
  } else {
    k = blk ? (fast ? role_div(x, blk, p.role_inv_blk) : x / blk) : last;
    if (k > last) k = last;
    stop = (k + 1) * blk;
  }
  if (end) *end = k == last ? ~0ull : stop - p.role_base;
  return role_bit_reverse((unsigned)k, p.role_bits);
}

// The launches of a kernel whose grid is (tiles, segments): `launch(tile0, ntiles, seg0, nsegs)` is
// called for each.  About `per_launch` workgroups per launch (see launch_tiles), whatever the number of
// segments: small work goes in one launch; otherwise up to four consecutive segments of similar
// length run side by side (blockIdx.y), more when they are short enough for one launch to hold
// them (eight long ones side by side run 0.5 to 1 point lower on untouched buffers, one or two the
// same), and a segment much longer than its neighbours gets launches of its own, so that no launch
// consists mostly of workgroups that find nothing to do (one block of 256 MiB beside seven of 4 KB in
// a Reduce_scatterv: 70 % of the HBM peak when all ran side by side, 79 % now).
template <typename F>
void plan_launches(SegParams &seg, unsigned nseg, size_t max_len, size_t tile_elems, size_t per_launch, F launch) {
  seg.mapped = 0;
  size_t most = (max_len + tile_elems - 1) / tile_elems;
  if (most == 0) most = 1;
  if (most * nseg <= per_launch) {
    launch((size_t)0, most, 0u, nseg);
    return;
  }
  size_t tiles_at[ALAMD_MAX_RANKS];
  unsigned char sorted[ALAMD_MAX_RANKS], rank_order[ALAMD_MAX_RANKS];
  for (unsigned s = 0; s < nseg; ++s) {
    const size_t len = seg.ragged ? (size_t)seg.seg_len[s] : max_len;
    tiles_at[s] = (len + tile_elems - 1) / tile_elems;
    sorted[s] = rank_order[s] = (unsigned char)s;
  }
  // Walks the positions of `order` in runs of similar length; calls visit(t0, nt, s0, n) per launch
  // and returns their number.
  auto walk = [&](const unsigned char *order, auto visit) {
    unsigned launches = 0;
    for (unsigned s0 = 0; s0 < nseg;) {
      size_t lo = tiles_at[order[s0]], hi = lo;
      unsigned n = 1;
      // four side by side, or as many as it takes to fill a launch when the segments are short
      const size_t fill = per_launch / (lo ? lo : 1);
      const unsigned most_side = fill > 4 ? (unsigned)fill : 4;
      while (s0 + n < nseg && n < most_side) {
        const size_t t = tiles_at[order[s0 + n]], nlo = t < lo ? t : lo, nhi = t > hi ? t : hi;
        if (nhi > 2 * nlo) break;
        lo = nlo;
        hi = nhi;
        ++n;
      }
      if (hi > 0) {
        const size_t cut = hi * n <= per_launch + per_launch / 2 ? hi : floor_pow2(per_launch / n);
        // a remainder of less than half a cut rides with the launch before it
        for (size_t t0 = 0; t0 < hi;) {
          const size_t nt = hi - t0 < cut + cut / 2 ? hi - t0 : cut;
          visit(t0, nt, s0, n);
          ++launches;
          t0 += nt;
        }
      }
      s0 += n;
    }
    return launches;
  };
  auto nothing = [](size_t, size_t, unsigned, unsigned) {};
  // Ragged segments may be taken longest first instead of in rank order, so that neighbours are
  // alike: worth it when that saves a quarter of the launches (64 blocks of random lengths up to
  // 4 MB: 37 % of peak in rank order, where most runs are one or two segments and each launch too
  // short to fill the device, 54 % sorted; 16 blocks up to 16 MB: 62 % and 67 %).  Eight large blocks
  // need about as many launches either way and run 1 to 2 points better in rank order.
  if (seg.ragged) {
    for (unsigned i = 1; i < nseg; ++i) {  // insertion sort, stable
      const unsigned char o = sorted[i];
      unsigned k = i;
      for (; k > 0 && tiles_at[sorted[k - 1]] < tiles_at[o]; --k) sorted[k] = sorted[k - 1];
      sorted[k] = o;
    }
    if (4 * walk(sorted, nothing) <= 3 * walk(rank_order, nothing)) {
      seg.mapped = 1;
      for (unsigned s = 0; s < nseg; ++s) seg.order[s] = sorted[s];
      walk(sorted, launch);
      return;
    }
  }
  walk(rank_order, launch);
}

// chain: null for an ordinary launch; else the scratch of a chained launch (one segment, one output,
// every tile in one launch; displ_bytes and nvec_tiles are filled in here).
struct ChainScratch { unsigned *ticket, *flags, *error; size_t max_tiles; unsigned max_polls; };
int launch_fold(const FoldParams &p, unsigned nseg, size_t max_len, int dtype, int op, bool acc_is_in,
                hipStream_t stream, const ChainScratch *chain = nullptr, size_t displ_bytes = 0);
int launch_tree(const TreeParams &p, int slots, unsigned nseg, size_t max_len, int dtype, int op,
                hipStream_t stream, const ChainScratch *chain = nullptr, size_t displ_bytes = 0);
// Clears the ticket counter, the error word and the first `tiles` flags on `stream` (a kernel, not a
// memset, so that the call may be captured into a graph).
int chain_clear(const ChainScratch &cs, size_t tiles, hipStream_t stream);
// Looks up, for the current device, the address of the scratch array that
// alamd_reduce_scatterv_noalloc uses (once per device).
int chain_static_init();

// A result that goes to several buffers is folded into one of them and then
// spread (one write stream per workgroup) when that is faster than writing
// every tile to all of them from the fold kernel: from three outputs up, once
// outputs x bytes reaches 128 MiB (the more outputs, the earlier the interleaved
// write streams of the single kernel cost more than a second launch).  us per
// call in one kernel / in two steps, on buffers that no earlier call has touched:
//   3 outputs: 16 MiB 18 / 22, 32 MiB 36 / 39, 64 MiB 72 / 72, 128 MiB 140 / 142
//   4 outputs: 16 MiB 24 / 27, 32 MiB 49 / 48, 64 MiB 95 / 91, 128 MiB 190 / 183
//   5 outputs: 16 MiB 29 / 33, 32 MiB 61 / 59, 64 MiB 120 / 112
//   8 outputs: 8 MiB 22 / 22, 16 MiB 52 / 46, 32 MiB 101 / 88, 64 MiB 196 / 170
//   16 outputs: 4 MiB 21 / 25, 8 MiB 50 / 44, 16 MiB 100 / 84
//   33 outputs: 2 MiB 30 / 32, 4 MiB 67 / 58, 8 MiB 120 / 103
// (on the same buffers again and again the single kernel holds out up to twice
// these sizes: 8 outputs 16 MiB 41 / 46, 32 MiB 84 / 88, 64 MiB 197 / 170).
// (Tunables::two_step_min_total_bytes, two_step_min_outputs)
// The two steps alternate over pieces of the result of this many bytes, so that
// the spread reads what the fold has just written from the 256 MiB memory-side
// cache instead of HBM (P = 8, 1 GiB per rank, buffers no earlier call has
// touched: 80 % of peak with pieces of 64 to 256 MiB, 75 % with the whole
// result folded first; no difference up to 256 MiB per rank, which stay one piece).
// (Tunables::two_step_piece_bytes)
// The fused ring allreduce does the same over pieces of this many bytes in all
// (32 MiB of each of eight segments: what the memory-side cache holds).  P = 8,
// bf16, untouched buffers, 256 MiB / 1 GiB per rank, default and alternatives
// taking turns in one process: 256 MiB pieces 79.6 % / 79.6 % of peak, 64 MiB
// 78.5 % / 77.8 %, 128 MiB - / 79.1 %, 512 MiB and the whole result folded
// first - / 71.5 % (at 256 MiB per rank the whole result is one piece).
// (Tunables::ring_piece_bytes)

// Copies [src, src + bytes) to each of dests[0..ndest) (none overlapping the
// source, any alignment).
int launch_spread(const char *src, char *const *dests, int ndest, size_t bytes, hipStream_t stream);
// The general form: source q = fp.in[q], fp.seg.seg_len[q] bytes, copied to byte offset
// fp.seg.seg_off[q] of every fp.out[0..fp.P) except where that is the source itself.
// from_hbm: the sources are slices no launch has just written (see launch_spread_table's definition).
int launch_spread_table(const FoldParams &fp, int nsrc, bool from_hbm, hipStream_t stream);

}  // namespace alamd
