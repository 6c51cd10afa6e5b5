// Tile access through buffer instructions.
//
// A workgroup owns one tile of THREADS*U 128-bit vectors per stream; each wave
// covers U KiB of it contiguously (lane l of wave w touches bytes
// w*U*1024 + u*1024 + l*16, u = 0..U-1).  The buffer descriptor is rebuilt per
// tile from a uniform base address, so the per-lane offset never changes and
// the address arithmetic stays in scalar registers; the descriptor's record
// count makes the hardware drop out-of-range lanes, which is the guard for a
// partial last tile.  Loads carry the non-temporal hint (every byte is read
// once), stores are written through (sc0 sc1) so that dirty lines do not
// gather in L2 and drain in bursts between the reads.
#pragma once

#include "alamd_common.h"

namespace alamd {

constexpr int kAuxLoadStream = 2;    // nt
constexpr int kAuxStoreStream = 17;  // sc0 | sc1
// Write-dominated kernels (one source to several destinations): the source is
// read again for every destination, so its loads stay cacheable; the stores
// are non-temporal and written through.
constexpr int kAuxLoadCached = 0;
constexpr int kAuxStoreNt = 19;      // sc0 | sc1 | nt
constexpr unsigned kRsrcFlags = 0x00020000u;

// Workgroups are handed to the eight XCDs round-robin and each XCD then works
// through its share at its own pace, so over a long launch the XCDs drift
// apart and the addresses in flight spread over more DRAM pages.  Very long
// inputs are therefore cut into consecutive launches on the same stream, each
// of which costs about 4.5 us of launch, ramp and drain.  The best cut shrinks
// with the number of streams.  Measured with the streaming fold on untouched
// fp32 buffers of 4.5 to 9 GiB in all, % of the HBM peak by MiB per stream and
// launch (32 / 64 / 128 / 256 / 512 / 1024 / 2048):
//   P = 2:  70 76 80 82 83 83 84    P = 4:  72 79 82 84 86 86     P = 8:  75 80 82 83 83 83
//   P = 12: 76 79 81 82 81          P = 16: 77 80 80 79 79        P = 32: 77 79 77 76
//   P = 64: 80 80 78
// The rule below picks 1024, 512, 256, 256, 128, 64 and 32 MiB for these.
constexpr size_t kLaunchBytes = (size_t)4 << 30;
// Tiles (of `tile_bytes` per stream) in one launch of a kernel that reads `nin` streams and
// writes one: the largest power of two that keeps the launch within launch_bytes.
inline size_t floor_pow2(size_t v) {
  size_t t = 1;
  while (t * 2 <= v) t *= 2;
  return t;
}
inline size_t launch_tiles(int nin, size_t tile_bytes, size_t launch_bytes = kLaunchBytes) {
  const size_t t = floor_pow2(launch_bytes / ((size_t)(nin + 1) * tile_bytes));
  return t < 8 ? 8 : t;
}

// Bytes per stream of a tile of the streaming fold and tree kernels (one wave, one vector per lane) and
// of the fold's block shape (128 threads x 8 vectors).
constexpr size_t kStreamTileBytes = 1024;
constexpr size_t kBlockTileBytes = 16384;

// Loads of 128 bits run at full rate from any 4-byte-aligned address; from an
// address that splits its dwords they lose about a fifth of the bandwidth.
// Stores want whole 64-byte lines: on buffers that no earlier launch has
// touched, a fold whose output starts 4, 16 or 32 bytes off a 64-byte boundary
// runs at 70.6 % of the HBM peak against 79 %.  The kernels therefore handle
// the leading elements one by one up to the output's next 64-byte boundary
// (at most 63 bytes' worth), if that leaves the first input's vectors on a
// dword boundary; otherwise up to the first input's next dword boundary.
__host__ __device__ inline size_t head_count(size_t elem_size, const char *out, const char *first, size_t len) {
  const uintptr_t o = reinterpret_cast<uintptr_t>(out), f = reinterpret_cast<uintptr_t>(first);
  const size_t bytes = ((o ^ f) & 3u) == 0 ? (64u - (unsigned)(o & 63u)) & 63u : (4u - (unsigned)(f & 3u)) & 3u;
  const size_t h = bytes / elem_size;
  return h < len ? h : len;
}
// The streaming kernels (one wave and 1 KiB per stream and tile) want more: a tile that starts off a
// 1 KiB boundary of its streams shares its first and last 128-byte lines with its neighbours, which run
// at the same time on other XCDs, and both fetch them.  P = 8 fold of f32, 256 MiB per rank, every
// buffer the same number of bytes off a 2 MiB boundary: 0: 85 % of the HBM peak, 1 KiB and more: 85,
// 512: 83.5, 256: 83, 128: 82, 64: 74.  From kBigHeadFromBytes per segment on, the leading elements
// therefore reach to the first input's next 1 KiB boundary (f32, every buffer 4 bytes off: 73 -> 84 %;
// output 20 bytes off the inputs: 73 -> 77 %, reads that split lines costing more than writes that do;
// such launches now do what stands below), spread over the segment's first workgroups, 64 elements each; shorter segments keep the rule above,
// since their few workgroups would spend longer on the elements than on the tiles.
constexpr size_t kBigHeadFromBytes = (size_t)64 << 10;
// Where some input sits at another distance from a 64-byte boundary than the output, one side has to
// split lines.  Then the output's tiles start on its 1 KiB boundary instead (whole lines written), and
// the launch hands runs of four consecutive tiles to one XCD (kXcdRunLog2, xcd_run_tile in
// alamd_dispatch.h), whose L2 then fetches most of the lines that neighbouring tiles share only once
// (f32, output 20 bytes off the inputs: 77 % with the inputs on their boundary, 74 % with the output on
// its boundary and the usual order of tiles, 80.5 % with runs of four; runs of two: 78, of eight: 79; on
// buffers that split no lines runs cost up to a point, so only these launches take them).
constexpr int kXcdRunLog2 = 2;
__host__ __device__ inline size_t stream_head_count(size_t elem_size, const char *out, const char *first, size_t len,
                                                    bool to_output = false) {
  if (len * elem_size < kBigHeadFromBytes) return head_count(elem_size, out, first, len);
  const uintptr_t f = reinterpret_cast<uintptr_t>(to_output ? out : first);
  return ((kStreamTileBytes - (size_t)(f & (kStreamTileBytes - 1))) & (kStreamTileBytes - 1)) / elem_size;
}
// Whether a segment's tiles go by the output (see above): some input at another distance from a 64-byte
// boundary than the output, all of them on the output's dword grid (else the loads would split dwords,
// which costs more), the segment long enough for tiles on 1 KiB boundaries.
template <typename NextInput>
inline bool tiles_by_output(size_t elem_size, const char *out, size_t len, int nin, NextInput input) {
  if (len * elem_size < kBigHeadFromBytes) return false;
  const uintptr_t o = reinterpret_cast<uintptr_t>(out);
  bool differs = false;
  for (int k = 0; k < nin; ++k) {
    const char *in = input(k);
    if (!in) continue;
    const uintptr_t d = reinterpret_cast<uintptr_t>(in) ^ o;
    if (d & 3u) return false;
    differs = differs || ((reinterpret_cast<uintptr_t>(in) - o) & 63u) != 0;
  }
  return differs;
}
template <typename T> __device__ __forceinline__ size_t head_elems(const char *out, const char *first, size_t len) {
  return head_count(sizeof(T), out, first, len);
}

// The streaming kernels are compiled for up to kStreamMaxWaves waves per SIMD; how many a launch really
// gets is set when it is launched, through the LDS it asks for: a CU has 160 KiB and a workgroup is one
// wave, so with 160 KiB / n bytes each n workgroups fit a CU (LDS is handed out by the KiB, so the
// counts that can be had are 32, 26, 22, 20, 17, 16, 14, 13, 12, ...).  The kernels never touch that memory.
// What counts is how many read requests the device keeps in flight: with one or two KiB per wave, as
// the streaming kernels have them, the memory system is at its best with 22 waves per CU for a fold
// and 16 for a tree (which has a pair of slots in flight where the fold has one stream); it loses 5 to
// 25 points with fewer and 2 to 6 with more.  Untouched fp32 buffers, % of the HBM peak by workgroups
// per CU (12 / 14 / 16 / 20 / 22 / 26 / 32):
//   fold  P = 2:  69 73 81 82 84 85 85    P = 4:  66 70 81 84 83 81 79    P = 8:  63 66 77 80 84 82 80
//         P = 16 (three streams up front): 62 65 75 80 84 81 80          P = 64 (three): 58 61 74 76 82 80 81
//   tree  P = 2:  71 75 82 83 84 85 84    P = 4:  79 82 81 80 79 80 79    P = 8:  80 83 81 81 80 80 80
//         P = 16: 79 80 82 81 79 79 79    P = 64: 84 84 83 80 80 80 81
//   (a tree of 16-bit floats or a float min / max, P = 8: 14: 75, 16: 84, 20: 83, 26: 81)
// Launches that move less than 256 MiB in all, much of which the caches hold, want more: 32 and 26
// (16 MiB per rank, P = 8, repeated on the same buffers: 23.0 us against 25.1 us with 22; of these only
// the ones below 32 MiB still stream, the others take the block shape: see above Tile).
constexpr int kStreamMaxWaves = 8;
inline unsigned stream_lds_bytes(int wgs_per_cu) {
  const int n = wgs_per_cu < 4 ? 4 : (wgs_per_cu > 4 * kStreamMaxWaves ? 4 * kStreamMaxWaves : wgs_per_cu);
  return (unsigned)((160u * 1024u / (unsigned)n) & ~127u);
}
// A launch that writes every tile to three or more buffers is better off with 16 whatever its size
// (8 MiB per rank to 8 buffers, repeated: 22.2 us against 24.1 us; 16 MiB, untouched: 51.0 against 52.8).
// Workgroups per CU of a streaming launch over `streams` inputs that moves `total_bytes` in all and
// writes every tile to `outputs` buffers.
// A launch of few rounds (`tiles` workgroups in all over `cus` CUs; 0: unknown) is a matter of whole
// rounds where a wave lives long, i.e. over many ranks: 64 ranks, 6048 tiles: 83 us with 22 per CU (two
// rounds, the second all but empty), 59 us with 26 (one); 48 ranks, 6672 tiles: 63 us with 22 or 26, 49 us
// with 32; 16 ranks, 23120 tiles: 62 / 59 / 58 us.  A fold of up to five rounds therefore takes the
// setting with the fewest rounds; from there on the rounds overlap and the rule above holds (16 ranks,
// 30832 tiles, six rounds: 79 us with 22, 83 us with 32; P = 8, 262144 tiles: 85 % with 22, 80 % with 32).  A tree, with twice the loads per wave, only goes from two
// rounds to one where 22 or 26 per CU do that (64 ranks, 4528 tiles: 59 -> 46 us); more per CU cost it
// more than the round saves.
// (no launch of more streaming tiles than this has few rounds on any device, nor lies below the size
// where the block shape ends: 384 MiB of 1 KiB tiles)
constexpr size_t kFewRoundsTiles = (size_t)384 << 10;
inline int stream_wgs_per_cu(bool tree, int streams, int outputs, size_t total_bytes, size_t tiles = 0, int cus = 0) {
  if (outputs >= 3) return 16;
  int n = tree ? 16 : 22;
  if (total_bytes < ((size_t)256 << 20)) n = tree ? 26 : 32;
  else if (streams <= 2) n = 26;
  if (tiles == 0 || cus <= 0) return n;
  auto rounds = [&](int m) { return (tiles + (size_t)m * (size_t)cus - 1) / ((size_t)m * (size_t)cus); };
  size_t best = rounds(n);
  if (tree ? best != 2 : (best < 2 || best > 5)) return n;
  const int more[3] = {22, 26, tree ? 26 : 32};
  for (int m : more)
    if (m > n && rounds(m) < best && (!tree || rounds(m) == 1)) { best = rounds(m); n = m; }
  return n;
}

// Between 32 and 384 MiB (bytes a launch reads and writes in all) the fold and tree kernels take the
// block shape instead (128 or 256 threads x 4 or 8 vectors, every load of a lane issued up front, two
// waves per SIMD): a launch of tens of microseconds, much of whose data the caches hold, gains more from
// having a sixteenth of the workgroups to hand out and from workgroups that are done after one trip to
// memory than it loses by what queues up in front of the L2.  The bare patterns (8 streams read, 1 or 8
// written, the same buffers again and again), us per launch, streaming (best setting) against block:
//   MiB per stream        4            8             16            32           64     128
//   1 written       4.8 / 4.1   10.8 / 10.3   21.6 / 20.8   43.9 / 43.0   88 / 93   178 / 187
//   8 written      10.0 / 7.5   20.9 / 19.2   40.3 / 37.8   76.2 / 78.8
// Below, a launch is over before the second round of workgroups starts, and what counts is how many
// start at once (library calls, P = 8, 64 KiB to 2 MiB per rank: 3.5 to 5.0 us streaming, 4.3 to 5.4 us
// in blocks).  The figures above are for powers of two, whose tiles deal out evenly over the CUs; which
// launches between the two sizes really take the block shape is use_block_shape's rule (alamd_dispatch.h).
// (kBlockShapeFromBytes and kBlockShapeBelowBytes, with the other sizes the planner goes by, in alamd_common.h.)

template <int U, int THREADS> struct Tile {
  static constexpr size_t BYTES = (size_t)THREADS * U * 16;
  unsigned vo;
  __device__ __forceinline__ Tile() {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    vo = wave * (U * 1024u) + lane * 16u;
  }
  // Descriptor over [base, base + nbytes); nbytes <= BYTES.
  static __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const char *base, int nbytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(base), 0, nbytes, kRsrcFlags);
  }
  __device__ __forceinline__ u32x4 load(__amdgpu_buffer_rsrc_t r, int u) const {
    return __builtin_amdgcn_raw_buffer_load_b128(r, vo + (unsigned)u * 1024u, 0, kAuxLoadStream);
  }
  __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t r, int u, u32x4 v) const {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, vo + (unsigned)u * 1024u, 0, kAuxStoreStream);
  }
  __device__ __forceinline__ u32x4 load_cached(__amdgpu_buffer_rsrc_t r, int u) const {
    return __builtin_amdgcn_raw_buffer_load_b128(r, vo + (unsigned)u * 1024u, 0, kAuxLoadCached);
  }
  __device__ __forceinline__ void store_nt(__amdgpu_buffer_rsrc_t r, int u, u32x4 v) const {
    __builtin_amdgcn_raw_buffer_store_b128(v, r, vo + (unsigned)u * 1024u, 0, kAuxStoreNt);
  }
};

// Stores one tile's result to out[j0 .. j0 + nj): the pointers are fetched four at a time, so that a
// wave that writes several buffers does not wait for one scalar load per buffer, one after the other.
template <typename TL, int U>
__device__ __forceinline__ void store_to_outputs(const TL &tl, char *const *out, int j0, int nj, size_t byte_off,
                                                 int nrec, const u32x4 (&v)[U]) {
  const int end = j0 + nj;
  for (int j = j0; j < end; j += 4) {
    char *o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = out[j + k < end ? j + k : end - 1];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (j + k < end) {
        const auto r = TL::rsrc(o[k] + byte_off, nrec);
#pragma unroll
        for (int u = 0; u < U; ++u) tl.store(r, u, v[u]);
      }
    }
  }
}

}  // namespace alamd
