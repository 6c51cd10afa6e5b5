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
// apart and the addresses in flight spread over more DRAM pages.  A launch
// therefore covers at most this many tiles per stream (64 MiB at 16 KiB per
// tile); longer inputs are cut into consecutive launches on the same stream.
constexpr size_t kMaxTilesPerLaunch = 4096;

// Loads of 128 bits run at full rate from any 4-byte-aligned address; from an
// address that splits its dwords they lose about a fifth of the bandwidth
// (stores do not care).  For element types narrower than 4 bytes the kernels
// therefore handle up to three bytes' worth of leading elements one by one, so
// that the vectors of the stream at `first` start on a dword boundary.
template <typename T> __device__ __forceinline__ size_t head_elems(const char *first, size_t len) {
  if constexpr (sizeof(T) >= 4) {
    return 0;
  } else {
    const size_t h = ((4u - (unsigned)(reinterpret_cast<uintptr_t>(first) & 3u)) & 3u) / sizeof(T);
    return h < len ? h : len;
  }
}

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

}  // namespace alamd
