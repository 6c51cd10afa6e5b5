// Halo face pack / unpack for a 3-D grid with x fastest.  A face is a list of
// rows (runs along x); rows of the y and z faces are whole interior lines,
// rows of the x faces are only `halo` elements long and one allocation line
// apart.  All selected faces are handled by one launch over a flat grid of
// workgroups (at these sizes, a few MiB per face, launch latency is a large
// part of the cost): every face owns a range of workgroups, the x faces first.
//
// Data moves in the widest power-of-two unit (up to 128 bits) that the row
// length, row pitch and base addresses allow.  A workgroup covers a tile of
// rows x units: LX = 2^k lanes side by side along a row, 256 / LX rows per
// pass, U passes, so a thread finds its place with shifts and one 32-bit
// division per access (by the number of rows in a plane).
//
// The short runs of an x face cost a whole cache line each, whatever is done
// with the rest of the line, so the x faces are bound by the number of lines
// the device can move, not by bytes.  When both x faces are selected they are
// handled as one face of twice the row length: neighbouring lanes take the -x
// and the +x run of a row, and the +x run of row y usually lies in the same
// 128-byte line as the -x run of row y+1, which a wave then fetches once
// (516^3 fp64 grid, halo 2: 1.25 lines per row instead of 2; both faces
// together 12.2 us against 14.4 us).
#include "alamd_common.h"

namespace alamd {

namespace {

constexpr int kThreads = 256;
constexpr int kPasses = 2;  // rows in flight per thread (1, 2, 4 within 5 %; 8 is 10-25 % slower)

struct HaloFace {
  char *buf;                   // contiguous face buffer (of a pair: the -x face's)
  char *buf2;                  // of a pair: the +x face's buffer
  unsigned long long goff;     // byte offset in the grid of the face's first element
  unsigned long long pitch_z;  // bytes between planes
  unsigned long long pitch_y;  // bytes between rows
  unsigned upr;                // units per row of one face buffer
  unsigned cols;               // units per row handled here: upr, or 2 * upr for a pair
  unsigned delta2;             // of a pair: bytes from the -x run of a row to its +x run
  unsigned ny;                 // rows per plane of the face
  unsigned nslots;             // rows * column tiles
  unsigned lx_log2;            // lanes side by side along a row: 1 << lx_log2
  unsigned ctiles;             // column tiles (of 1 << lx_log2 units) per row
  unsigned blk0;               // first workgroup of this face
};

struct HaloParams {
  HaloFace f[6];
  char *grid;
  int nf;
};

template <int UB> struct unit_of;
template <> struct unit_of<1> { using type = uint8_t; };
template <> struct unit_of<2> { using type = uint16_t; };
template <> struct unit_of<4> { using type = uint32_t; };
template <> struct unit_of<8> { using type = uint64_t; };
template <> struct unit_of<16> { using type = u32x4; };

// Store written through to memory (sc0 sc1).  The ghost cells of an x face are
// runs of a few bytes in lines of their own: kept in L2 as dirty partial lines
// they cost more when they are evicted later (six-face unpack of the 516^3
// fp64 grid 15.5 us with plain stores, 13.6 us written through; non-temporal
// stores of such runs take 45 us).
template <int UB> __device__ __forceinline__ void store_through(char *p, typename unit_of<UB>::type v) {
  if constexpr (UB == 16) asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
  else if constexpr (UB == 8) asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
  else if constexpr (UB == 4) asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"(p), "v"(v) : "memory");
  else if constexpr (UB == 2) asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(p), "v"((uint32_t)v) : "memory");
  else asm volatile("global_store_byte %0, %1, off sc0 sc1" ::"v"(p), "v"((uint32_t)v) : "memory");
}

// The grid loads of a pack under another cache policy (16-byte units only; Tunables::halo_load_policy, a
// measurement setting).  An x face needs 16 bytes of every 128-byte line it touches, so a policy under
// which the L2 asked memory for 32- or 64-byte sectors instead of whole lines would cut its traffic.  None
// does: under every policy below every read request that leaves the L2 is 128 bytes (329 k requests for
// both x faces, 462 k for all six, none of 32 bytes, 352 of 64), and the times are the same within 1 %
// (nt: +20 % on the six-face launch).  The plain load stays.
template <int LP> __device__ __forceinline__ u32x4 load_policy(const char *p) {
  u32x4 v;
  if constexpr (LP == 1) asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(v) : "v"(p) : "memory");
  else if constexpr (LP == 2) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  else if constexpr (LP == 3) asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
  else asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1 nt" : "=v"(v) : "v"(p) : "memory");
  return v;
}

template <int UB, bool PACK, int LP = 0>
__global__ void __launch_bounds__(kThreads) halo_kernel(const HaloParams p) {
  using Unit = typename unit_of<UB>::type;
  constexpr int U = kPasses;
  int fi = 0;
#pragma unroll
  for (int k = 1; k < 6; ++k)
    if (k < p.nf && blockIdx.x >= p.f[k].blk0) fi = k;
  const HaloFace &f = p.f[fi];
  const unsigned lx = 1u << f.lx_log2, ly = (unsigned)kThreads >> f.lx_log2;
  const unsigned tx = threadIdx.x & (lx - 1), ty = threadIdx.x >> f.lx_log2;
  // a slot is (row, column tile); consecutive slots of a row are consecutive column tiles
  const unsigned s0 = (blockIdx.x - f.blk0) * (ly * U) + ty;
  Unit v[U];
  char *g[U], *b[U];
  bool ok[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const unsigned s = s0 + (unsigned)u * ly;
    ok[u] = s < f.nslots;
    unsigned r = s, ct = 0;
    if (f.ctiles > 1) {
      r = s / f.ctiles;
      ct = s - r * f.ctiles;
    }
    const unsigned col = ct * lx + tx;
    ok[u] = ok[u] && col < f.cols;
    const bool second = col >= f.upr;  // the +x face of a pair
    const unsigned c1 = second ? col - f.upr : col;
    const unsigned z = r / f.ny, y = r - z * f.ny;
    g[u] = p.grid + f.goff + (unsigned long long)z * f.pitch_z + (unsigned long long)y * f.pitch_y +
           (unsigned long long)c1 * UB + (second ? f.delta2 : 0u);
    b[u] = (second ? f.buf2 : f.buf) + ((unsigned long long)r * f.upr + c1) * UB;
  }
  if constexpr (LP > 0 && UB == 16 && PACK) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (ok[u]) v[u] = load_policy<LP>(g[u]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the compiler does not count loads made by asm statements
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (ok[u]) v[u] = *reinterpret_cast<const Unit *>(PACK ? g[u] : b[u]);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (ok[u]) {
      if (PACK) *reinterpret_cast<Unit *>(b[u]) = v[u];
      else store_through<UB>(g[u], v[u]);
    }
  }
}

int halo_launch(void *grid, void *const bufs[6], const size_t dims[3], size_t halo, size_t es,
                unsigned face_mask, bool pack, hipStream_t stream) {
  if (!dims) return set_error(ALAMD_ERR_INVALID_ARG, "null dims");
  if (es == 0 || es > 16 || (es & (es - 1)) != 0)
    return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "element size %zu is not a power of two up to 16", es);
  if (face_mask & ~0x3fu) return set_error(ALAMD_ERR_INVALID_ARG, "face mask 0x%x names a face above 5", face_mask);
  for (int d = 0; d < 3; ++d)
    if (dims[d] == 0 || halo > dims[d])
      return set_error(ALAMD_ERR_INVALID_ARG, "halo width %zu does not fit interior extent %zu", halo, dims[d]);
  if (halo == 0 || face_mask == 0) return ALAMD_OK;
  if (!grid || !bufs) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer");
  const size_t sx = dims[0] + 2 * halo, sy = dims[1] + 2 * halo;
  if (sx * es > 0xffffffffull) return set_error(ALAMD_ERR_INVALID_ARG, "grid extent too large");
  // widest unit every selected face allows
  size_t unit = 16;
  auto shrink = [&unit](size_t v) { while (unit > 1 && v % unit != 0) unit /= 2; };
  shrink(reinterpret_cast<uintptr_t>(grid));
  shrink(sx * es);
  size_t lo[6][3], ext[6][3];
  for (int face = 0; face < 6; ++face) {
    if (!(face_mask & (1u << face))) continue;
    if (!bufs[face]) return set_error(ALAMD_ERR_INVALID_ARG, "buffer of face %d is null", face);
    const int axis = face / 2, plus = face % 2;
    for (int d = 0; d < 3; ++d) { lo[face][d] = halo; ext[face][d] = dims[d]; }
    ext[face][axis] = halo;
    // pack reads the interior boundary slab, unpack writes the ghost slab
    if (pack) lo[face][axis] = plus ? dims[axis] : halo;
    else lo[face][axis] = plus ? halo + dims[axis] : 0;
    shrink(reinterpret_cast<uintptr_t>(bufs[face]));
    shrink(ext[face][0] * es);
    shrink(lo[face][0] * es);
  }
  HaloParams hp;
  hp.grid = static_cast<char *>(grid);
  hp.nf = 0;
  unsigned long long blocks = 0;
  const bool pair = (face_mask & 3u) == 3u;
  for (int face = 0; face < 6; ++face) {
    if (!(face_mask & (1u << face)) || (pair && face == 1)) continue;
    HaloFace &f = hp.f[hp.nf++];
    f.buf = f.buf2 = static_cast<char *>(bufs[face]);
    f.goff = ((lo[face][2] * sy + lo[face][1]) * sx + lo[face][0]) * es;
    f.pitch_y = sx * es;
    f.pitch_z = sx * sy * es;
    f.upr = f.cols = (unsigned)(ext[face][0] * es / unit);
    f.delta2 = 0;
    if (pair && face == 0) {
      f.buf2 = static_cast<char *>(bufs[1]);
      f.cols = 2 * f.upr;
      f.delta2 = (unsigned)((lo[1][0] - lo[0][0]) * es);
    }
    f.ny = (unsigned)ext[face][1];
    // lanes along a row: the largest power of two that divides the row length (so that no lane
    // of a column tile is idle), at most the workgroup
    unsigned l = 0;
    while (l < 8 && f.cols % (2u << l) == 0) ++l;
    f.lx_log2 = l;
    f.ctiles = f.cols >> l;
    const unsigned long long rows = (unsigned long long)ext[face][1] * ext[face][2];
    const unsigned long long slots = rows * f.ctiles;
    if (ext[face][1] > 0xffffffffull || slots > 0xfff00000ull)
      return set_error(ALAMD_ERR_INVALID_ARG, "grid extent too large");
    f.nslots = (unsigned)slots;
    const unsigned per_block = ((unsigned)kThreads >> l) * kPasses;
    f.blk0 = (unsigned)blocks;
    blocks += (slots + per_block - 1) / per_block;
    if (blocks > 0x7fffffffull) return set_error(ALAMD_ERR_INVALID_ARG, "grid extent too large");
  }
  for (int k = hp.nf; k < 6; ++k) {
    hp.f[k] = hp.f[0];
    hp.f[k].blk0 = 0xffffffffu;
  }
  void (*kern)(const HaloParams) = nullptr;
  switch (unit) {
  case 16: {
    const size_t lp = tunables().halo_load_policy;
    kern = !pack ? halo_kernel<16, false>
           : lp == 1 ? halo_kernel<16, true, 1> : lp == 2 ? halo_kernel<16, true, 2> : lp == 3 ? halo_kernel<16, true, 3>
           : lp == 4 ? halo_kernel<16, true, 4> : halo_kernel<16, true>;
    break;
  }
  case 8: kern = pack ? halo_kernel<8, true> : halo_kernel<8, false>; break;
  case 4: kern = pack ? halo_kernel<4, true> : halo_kernel<4, false>; break;
  case 2: kern = pack ? halo_kernel<2, true> : halo_kernel<2, false>; break;
  default: kern = pack ? halo_kernel<1, true> : halo_kernel<1, false>; break;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks, 1, 1), dim3(kThreads, 1, 1), 0, stream, hp);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

}  // namespace
}  // namespace alamd

using namespace alamd;

extern "C" {

size_t alamd_halo_face_elems(const size_t dims[3], size_t halo, int face) {
  if (!dims || face < 0 || face > 5) return 0;
  size_t ext[3] = {dims[0], dims[1], dims[2]};
  ext[face / 2] = halo;
  return ext[0] * ext[1] * ext[2];
}

int alamd_halo_pack(void *const bufs[6], const void *grid, const size_t dims[3], size_t halo,
                    size_t elem_size, unsigned face_mask, void *stream) {
  return halo_launch(const_cast<void *>(grid), bufs, dims, halo, elem_size, face_mask, true, as_stream(stream));
}

int alamd_halo_unpack(void *grid, const void *const bufs[6], const size_t dims[3], size_t halo,
                      size_t elem_size, unsigned face_mask, void *stream) {
  return halo_launch(grid, const_cast<void *const *>(bufs), dims, halo, elem_size, face_mask, false,
                     as_stream(stream));
}

}  // extern "C"
