// Test and bench support: the counter-based input generator, the exposed
// 16-bit float conversions, and a plain streaming copy.
#include "alamd_common.h"
#include "aluminum_amd_support.h"
#include "alamd_tile.h"

namespace alamd {

namespace {

constexpr uint64_t kGamma = 0x9E3779B97F4A7C15ull;

__device__ __forceinline__ uint64_t fin64(uint64_t z) {
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27; z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}

__device__ __forceinline__ uint64_t mix64(uint64_t seed_hash, uint64_t idx) {
  return fin64(seed_hash + (idx + 1) * kGamma);
}

__device__ __forceinline__ uint32_t ih12_sum(uint64_t b0) {
  const uint64_t b1 = fin64(b0 + kGamma), b2 = fin64(b1 + kGamma);
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    s += (uint32_t)((b0 >> (16 * k)) & 0xffffu);
    s += (uint32_t)((b1 >> (16 * k)) & 0xffffu);
    s += (uint32_t)((b2 >> (16 * k)) & 0xffffu);
  }
  return s;
}

// Every operation is a single correctly rounded fp64 operation (no fused
// multiply-add), so the host formula gives the same bits.
__device__ __forceinline__ double gen_f64(uint64_t bits, int dist) {
  switch (dist) {
  case ALAMD_DIST_UNIFORM_09_11: {
    const double u = (double)(bits >> 11) * 0x1p-53;
    const double t = __dmul_rn(u, 0.2);
    return __dadd_rn(0.9, t);
  }
  case ALAMD_DIST_UNIFORM_01: return (double)(bits >> 11) * 0x1p-53;
  case ALAMD_DIST_BOOL01: return (double)(bits >> 63);
  case ALAMD_DIST_NORMAL: return (double)ih12_sum(bits) * 0x1p-16 - 6.0;
  case ALAMD_DIST_SMALLINT: return (double)((int)(bits >> 60) - 8);
  default: return (double)(int64_t)bits * 0x1p-63;
  }
}

__device__ __forceinline__ uint64_t gen_int(uint64_t bits, int dist, bool is_signed) {
  switch (dist) {
  case ALAMD_DIST_FULLRANGE: return bits;
  case ALAMD_DIST_BOOL01: return bits >> 63;
  default: return is_signed ? (uint64_t)((int64_t)(bits >> 60) - 8) : (bits >> 60);
  }
}

__global__ void __launch_bounds__(256) fill_kernel(void *dst, size_t n, int dtype, int dist,
                                                   uint64_t seed_hash, uint64_t idx0) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    const uint64_t bits = mix64(seed_hash, idx0 + i);
    switch (dtype) {
    case ALAMD_I8: ((int8_t *)dst)[i] = (int8_t)gen_int(bits, dist, true); break;
    case ALAMD_U8: ((uint8_t *)dst)[i] = (uint8_t)gen_int(bits, dist, false); break;
    case ALAMD_I16: ((int16_t *)dst)[i] = (int16_t)gen_int(bits, dist, true); break;
    case ALAMD_U16: ((uint16_t *)dst)[i] = (uint16_t)gen_int(bits, dist, false); break;
    case ALAMD_I32: ((int32_t *)dst)[i] = (int32_t)gen_int(bits, dist, true); break;
    case ALAMD_U32: ((uint32_t *)dst)[i] = (uint32_t)gen_int(bits, dist, false); break;
    case ALAMD_I64: ((int64_t *)dst)[i] = (int64_t)gen_int(bits, dist, true); break;
    case ALAMD_U64: ((uint64_t *)dst)[i] = gen_int(bits, dist, false); break;
    case ALAMD_F16: ((uint16_t *)dst)[i] = narrow<f16_t>((float)gen_f64(bits, dist)).b; break;
    case ALAMD_BF16: ((uint16_t *)dst)[i] = narrow<bf16_t>((float)gen_f64(bits, dist)).b; break;
    case ALAMD_F32: ((float *)dst)[i] = (float)gen_f64(bits, dist); break;
    default: ((double *)dst)[i] = gen_f64(bits, dist); break;
    }
  }
}

template <typename H>
__global__ void __launch_bounds__(256) narrow_kernel(uint16_t *dst, const float *src, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    dst[i] = narrow<H>(src[i]).b;
}

template <typename H>
__global__ void __launch_bounds__(256) widen_kernel(float *dst, const uint16_t *src, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    H h;
    h.b = src[i];
    dst[i] = widen(h);
  }
}

constexpr int kCopyU = 8, kCopyThreads = 128;
// Any alignment: b.head + b.tail single bytes by the first workgroup, b.vec bytes in tiles.
// Two waves per SIMD and launches of 256 MiB: measured on 8 GiB that no earlier
// launch has touched, 81.6 % of the HBM peak (one launch 76 %, 64 MiB launches
// 76 %, four or eight waves per SIMD 73 % / 70 %).
constexpr size_t kCopyTilesPerLaunch = 16384;
__global__ void __launch_bounds__(kCopyThreads) __attribute__((amdgpu_waves_per_eu(1, 2)))
copy_kernel_vec(char *dst, const char *src, ByteSplit b, size_t tile0) {
  using TL = Tile<kCopyU, kCopyThreads>;
  const TL tl;
  if (tile0 == 0 && blockIdx.x == 0 && threadIdx.x < b.head + b.tail) {
    const size_t i = threadIdx.x < b.head ? threadIdx.x : b.vec + threadIdx.x;
    dst[i] = src[i];
  }
  const size_t tb = (tile0 + blockIdx.x) * TL::BYTES;
  if (tb >= b.vec) return;
  const int nrec = b.vec - tb > TL::BYTES ? (int)TL::BYTES : (int)(b.vec - tb);
  const auto rs = TL::rsrc(src + b.head + tb, nrec);
  const auto rd = TL::rsrc(dst + b.head + tb, nrec);
  u32x4 v[kCopyU];
#pragma unroll
  for (int u = 0; u < kCopyU; ++u) v[u] = tl.load(rs, u);
#pragma unroll
  for (int u = 0; u < kCopyU; ++u) tl.store(rd, u, v[u]);
}

}  // namespace
}  // namespace alamd

using namespace alamd;

extern "C" {

int alamd_fill(void *dst, size_t count, int dtype, int dist, uint64_t seed, uint64_t idx0, void *stream) {
  if (alamd_dtype_size(dtype) == 0) return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);
  if (dist < ALAMD_DIST_UNIFORM_PM1 || dist > ALAMD_DIST_SMALLINT)
    return set_error(ALAMD_ERR_INVALID_ARG, "unknown distribution %d", dist);
  if (count == 0) return ALAMD_OK;
  if (!dst) return set_error(ALAMD_ERR_INVALID_ARG, "null destination");
  // host half of the hash: the per-stream constant
  uint64_t z = seed + 0x9E3779B97F4A7C15ull;
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27; z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  const unsigned grid = stream_grid(count, 256 * 8, 16);
  hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(256), 0, as_stream(stream), dst, count, dtype, dist, z, idx0);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

int alamd_narrow_f32(void *dst16, const float *src, size_t count, int dtype, void *stream) {
  if (dtype != ALAMD_F16 && dtype != ALAMD_BF16)
    return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "narrowing target must be fp16 or bf16");
  if (count == 0) return ALAMD_OK;
  if (!dst16 || !src) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer");
  const unsigned grid = stream_grid(count, 256 * 8, 16);
  if (dtype == ALAMD_F16)
    hipLaunchKernelGGL(narrow_kernel<f16_t>, dim3(grid), dim3(256), 0, as_stream(stream), (uint16_t *)dst16, src, count);
  else
    hipLaunchKernelGGL(narrow_kernel<bf16_t>, dim3(grid), dim3(256), 0, as_stream(stream), (uint16_t *)dst16, src, count);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

int alamd_widen_f32(float *dst, const void *src16, size_t count, int dtype, void *stream) {
  if (dtype != ALAMD_F16 && dtype != ALAMD_BF16)
    return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "widening source must be fp16 or bf16");
  if (count == 0) return ALAMD_OK;
  if (!dst || !src16) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer");
  const unsigned grid = stream_grid(count, 256 * 8, 16);
  if (dtype == ALAMD_F16)
    hipLaunchKernelGGL(widen_kernel<f16_t>, dim3(grid), dim3(256), 0, as_stream(stream), dst, (const uint16_t *)src16, count);
  else
    hipLaunchKernelGGL(widen_kernel<bf16_t>, dim3(grid), dim3(256), 0, as_stream(stream), dst, (const uint16_t *)src16, count);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

int alamd_copy(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return ALAMD_OK;
  if (!dst || !src) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer");
  const ByteSplit b = split_bytes(dst, src, bytes);
  const size_t tile = Tile<kCopyU, kCopyThreads>::BYTES;
  size_t tiles = (b.vec + tile - 1) / tile;
  if (tiles == 0) tiles = 1;
  // a remainder of less than half a launch rides with the launch before it
  for (size_t t0 = 0; t0 < tiles;) {
    const size_t nt = tiles - t0 < kCopyTilesPerLaunch + kCopyTilesPerLaunch / 2 ? tiles - t0 : kCopyTilesPerLaunch;
    hipLaunchKernelGGL(copy_kernel_vec, dim3((unsigned)nt), dim3(kCopyThreads), 0, as_stream(stream), (char *)dst,
                       (const char *)src, b, t0);
    t0 += nt;
  }
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

}  // extern "C"
