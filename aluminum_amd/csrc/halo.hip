// Halo face pack / unpack for a 3-D grid with x fastest.  A face is a list of
// rows (runs along x); rows of the y and z faces are whole interior lines,
// rows of the x faces are only `halo` elements long and one allocation line
// apart.  All selected faces are handled by one launch (blockIdx.y = face):
// at these sizes (a few MiB per face) launch latency is a large part of the
// cost.  Data moves in the widest power-of-two unit (up to 128 bits) that the
// row length, row pitch and base addresses allow, so that the contiguous side
// of every face is accessed in whole coalesced runs.
#include "alamd_common.h"

namespace alamd {

namespace {

constexpr int kThreads = 256;

struct HaloFace {
  char *buf;                      // contiguous face buffer
  unsigned long long grid_off;    // byte offset of the face's first element in the grid
  unsigned long long pitch_y;     // bytes between rows adjacent in y
  unsigned long long pitch_z;     // bytes between rows adjacent in z
  unsigned long long nunits;      // units in the face
  unsigned upr;                   // units per row
  unsigned rows_y;                // rows per z-plane of the face
};

struct HaloParams {
  HaloFace f[6];
  char *grid;
};

template <int UB> struct unit_of;
template <> struct unit_of<1> { using type = uint8_t; };
template <> struct unit_of<2> { using type = uint16_t; };
template <> struct unit_of<4> { using type = uint32_t; };
template <> struct unit_of<8> { using type = uint64_t; };
template <> struct unit_of<16> { using type = u32x4; };

// U = independent accesses per thread: the short rows of the x faces need
// several in flight, but a launch also needs a few workgroups per CU, so the
// host picks the largest U that leaves enough of them.
template <int UB, bool PACK, int U>
__global__ void __launch_bounds__(kThreads) halo_kernel(const HaloParams p) {
  using Unit = typename unit_of<UB>::type;
  const HaloFace &f = p.f[blockIdx.y];
  const unsigned long long n = f.nunits;
  const unsigned upr = f.upr, rows_y = f.rows_y;
  for (unsigned long long i0 = (unsigned long long)blockIdx.x * (kThreads * U) + threadIdx.x; i0 < n;
       i0 += (unsigned long long)gridDim.x * (kThreads * U)) {
    Unit v[U];
    char *g[U];
    char *b[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned long long i = i0 + (unsigned long long)u * kThreads;
      if (i < n) {
        // faces hold fewer than 2^32 rows
        const unsigned long long row = i / upr;
        const unsigned col = (unsigned)(i - row * upr);
        const unsigned long long z = row / rows_y;
        const unsigned y = (unsigned)(row - z * rows_y);
        g[u] = p.grid + f.grid_off + z * f.pitch_z + (unsigned long long)y * f.pitch_y + (unsigned long long)col * UB;
        b[u] = f.buf + i * UB;
        v[u] = *reinterpret_cast<const Unit *>(PACK ? g[u] : b[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const unsigned long long i = i0 + (unsigned long long)u * kThreads;
      if (i < n) *reinterpret_cast<Unit *>(PACK ? b[u] : g[u]) = v[u];
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
  HaloParams hp;
  hp.grid = static_cast<char *>(grid);
  // widest unit every selected face allows
  size_t unit = 16;
  auto shrink = [&unit](size_t v) { while (unit > 1 && v % unit != 0) unit /= 2; };
  shrink(reinterpret_cast<uintptr_t>(grid));
  shrink(sx * es);
  int nf = 0;
  unsigned long long max_units = 0;
  size_t lo[6][3], ext[6][3];
  int sel[6];
  for (int face = 0; face < 6; ++face) {
    if (!(face_mask & (1u << face))) continue;
    if (!bufs[face]) return set_error(ALAMD_ERR_INVALID_ARG, "buffer of face %d is null", face);
    const int axis = face / 2, plus = face % 2;
    for (int d = 0; d < 3; ++d) { lo[nf][d] = halo; ext[nf][d] = dims[d]; }
    ext[nf][axis] = halo;
    // pack reads the interior boundary slab, unpack writes the ghost slab
    if (pack) lo[nf][axis] = plus ? dims[axis] : halo;
    else lo[nf][axis] = plus ? halo + dims[axis] : 0;
    shrink(reinterpret_cast<uintptr_t>(bufs[face]));
    shrink(ext[nf][0] * es);
    shrink(lo[nf][0] * es);
    sel[nf] = face;
    ++nf;
  }
  for (int k = 0; k < nf; ++k) {
    HaloFace &f = hp.f[k];
    f.buf = static_cast<char *>(bufs[sel[k]]);
    f.grid_off = ((lo[k][2] * sy + lo[k][1]) * sx + lo[k][0]) * es;
    f.pitch_y = sx * es;
    f.pitch_z = sx * sy * es;
    f.upr = (unsigned)(ext[k][0] * es / unit);
    f.rows_y = (unsigned)ext[k][1];
    f.nunits = (unsigned long long)f.upr * ext[k][1] * ext[k][2];
    if (ext[k][0] * es / unit > 0xffffffffull || ext[k][1] > 0xffffffffull)
      return set_error(ALAMD_ERR_INVALID_ARG, "grid extent too large");
    if (f.nunits > max_units) max_units = f.nunits;
  }
  for (int k = nf; k < 6; ++k) hp.f[k] = hp.f[0];
  // 8 accesses per thread if that still gives two workgroups per CU over all faces, else 2
  const unsigned two_per_cu = stream_grid((size_t)-1 / 2, 1, 2);
  const bool wide = (max_units + kThreads * 8 - 1) / (kThreads * 8) * nf >= two_per_cu;
  const int acc = wide ? 8 : 2;
  unsigned per_face = (stream_grid((size_t)-1 / 2, 1, 8) + nf - 1) / nf;
  unsigned gx = stream_grid((size_t)max_units, (size_t)kThreads * acc, 8);
  if (gx > per_face) gx = per_face < 1 ? 1 : per_face;
  const dim3 grid_dim(gx, nf, 1), block(kThreads, 1, 1);
  void (*kern)(const HaloParams) = nullptr;
  auto pick = [&](auto ub) {
    constexpr int UB = decltype(ub)::value;
    if (wide) return pack ? halo_kernel<UB, true, 8> : halo_kernel<UB, false, 8>;
    return pack ? halo_kernel<UB, true, 2> : halo_kernel<UB, false, 2>;
  };
  switch (unit) {
  case 16: kern = pick(std::integral_constant<int, 16>{}); break;
  case 8: kern = pick(std::integral_constant<int, 8>{}); break;
  case 4: kern = pick(std::integral_constant<int, 4>{}); break;
  case 2: kern = pick(std::integral_constant<int, 2>{}); break;
  default: kern = pick(std::integral_constant<int, 1>{}); break;
  }
  hipLaunchKernelGGL(kern, grid_dim, block, 0, stream, hp);
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
