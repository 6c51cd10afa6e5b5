// What the memory system gives to the access patterns the combine is made of, with the two tile shapes
// of the library's kernels (alamd_tile.h) and nothing else: no arithmetic beyond an xor, no layout logic.
//
//   stream   the shape of an ordinary fold launch: one wave per workgroup, one 128-bit vector per lane
//            and stream (1 KiB per wave and stream), two streams requested up front and one more for
//            every stream consumed, a number of workgroups per CU set through the LDS a launch asks
//            for, the whole call in one launch
//   block    the shape of a chained launch (and of every fold launch before the streaming shape):
//            128 threads x 8 vectors per stream, every load of a lane issued up front, two waves per
//            SIMD, launches of 64 MiB per stream
//
// Every pattern walks rotating buffer sets, so that nothing a launch touches was touched by the
// launches just before it.
//
//   read8    eight streams read, nothing written
//   read1    one stream read
//   write1   one stream written
//   copy     one read, one written
//   mix8     eight read, one written (the P = 8 fold)
//   mix8ip   eight read, the result written over the stream read last
//   mix2, mix3, mix4, mix6   the folds of fewer ranks
//
// usage: bench_hbm [pattern ...] [--mib N per stream, default 256] [--sets S, default 4] [--reps R, default 12]
//                  [--wgs N workgroups per CU of the stream shape, default: the library's choice]
// Prints one JSON line per pattern and shape.  A bench / profiling aid; not part of the library.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "alamd_tile.h"

using namespace alamd;

#define CK(x)                                                                                      \
  do {                                                                                             \
    hipError_t e_ = (x);                                                                           \
    if (e_ != hipSuccess) {                                                                        \
      std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);                   \
      std::exit(2);                                                                                \
    }                                                                                              \
  } while (0)

struct Streams {
  const char *in[8];
  char *out;
  unsigned long long tile0;
};

// A read-only kernel stores only if the xor of everything it read equals a value no input produces,
// i.e. never.
__device__ __forceinline__ bool never_seen(const u32x4 &v, unsigned never) { return v[0] == never && v[1] == never; }

// NR streams read (xor-combined), one written if WRITE; block shape.
constexpr int kU = 8, kThreads = 128;
template <int NR, bool WRITE>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 2)))
block_kernel(const Streams p, unsigned never) {
  using TL = Tile<kU, kThreads>;
  const TL tl;
  const size_t tb = ((size_t)p.tile0 + blockIdx.x) * TL::BYTES;
  u32x4 acc[kU];
#pragma unroll
  for (int u = 0; u < kU; ++u) acc[u] = u32x4{0u, 0u, 0u, 0u};
  if constexpr (NR > 0) {
    u32x4 x[NR][kU];
#pragma unroll
    for (int k = 0; k < NR; ++k) {
      const auto r = TL::rsrc(p.in[k] + tb, (int)TL::BYTES);
#pragma unroll
      for (int u = 0; u < kU; ++u) x[k][u] = tl.load(r, u);
    }
#pragma unroll
    for (int k = 0; k < NR; ++k)
#pragma unroll
      for (int u = 0; u < kU; ++u) acc[u] ^= x[k][u];
  } else {
#pragma unroll
    for (int u = 0; u < kU; ++u) acc[u] = u32x4{blockIdx.x, threadIdx.x, (unsigned)u, never};
  }
  bool store = WRITE;
  if constexpr (!WRITE) {
    unsigned any = 0;
#pragma unroll
    for (int u = 0; u < kU; ++u) any |= never_seen(acc[u], never) ? 1u : 0u;
    store = any != 0;
  }
  if (store) {
    const auto r = TL::rsrc(p.out + tb, (int)TL::BYTES);
#pragma unroll
    for (int u = 0; u < kU; ++u) tl.store(r, u, acc[u]);
  }
}

// The same in the stream shape: the loop of the library's fold with an xor for the step.
template <int NR, bool WRITE>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(1, kStreamMaxWaves)))
stream_kernel(const Streams p, unsigned never) {
  using TL = Tile<1, 64>;
  const TL tl;
  const size_t tb = ((size_t)p.tile0 + blockIdx.x) * TL::BYTES;
  u32x4 acc = u32x4{blockIdx.x, threadIdx.x, 0u, never};
  if constexpr (NR > 0) {
    constexpr int FRONT = 2;
    u32x4 x[FRONT];
#pragma unroll
    for (int j = 0; j < FRONT; ++j)
      if (j < NR) x[j] = tl.load(TL::rsrc(p.in[j] + tb, (int)TL::BYTES), 0);
    __builtin_amdgcn_sched_barrier(0);
    auto load_after = [&](__amdgpu_buffer_rsrc_t rs, const u32x4 &after) {
      unsigned vo = tl.vo;
      asm volatile("" : "+v"(vo) : "v"(after));
      return __builtin_amdgcn_raw_buffer_load_b128(rs, vo, 0, kAuxLoadStream);
    };
    acc = x[0];
#pragma unroll
    for (int k = 1; k < NR; ++k) {
      acc ^= x[k % FRONT];
      if (k + FRONT - 1 < NR) x[(k + FRONT - 1) % FRONT] = load_after(TL::rsrc(p.in[k + FRONT - 1] + tb, (int)TL::BYTES), acc);
      asm volatile("" : "+v"(acc));
    }
  }
  if (WRITE || never_seen(acc, never)) tl.store(TL::rsrc(p.out + tb, (int)TL::BYTES), 0, acc);
}

__global__ void noise_kernel(unsigned *dst, size_t words, unsigned salt) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (size_t)gridDim.x * blockDim.x) {
    unsigned x = (unsigned)i * 2654435761u + salt * 40503u;
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    dst[i] = x;
  }
}

struct Pattern {
  const char *name;
  int nread, nwrite;
  bool inplace;
  void (*block)(const Streams, unsigned);
  void (*stream)(const Streams, unsigned);
};
#define PATTERN(name, nr, wr, ip) {name, nr, wr ? 1 : 0, ip, block_kernel<nr, wr>, stream_kernel<nr, wr>}

int main(int argc, char **argv) {
  size_t mib = 256;
  int sets = 4, reps = 12, wgs = 0;
  std::vector<std::string> want;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--mib" && i + 1 < argc) mib = std::strtoull(argv[++i], nullptr, 10);
    else if (a == "--sets" && i + 1 < argc) sets = std::atoi(argv[++i]);
    else if (a == "--reps" && i + 1 < argc) reps = std::atoi(argv[++i]);
    else if (a == "--wgs" && i + 1 < argc) wgs = std::atoi(argv[++i]);
    else want.push_back(a);
  }
  const Pattern all[] = {
      PATTERN("read8", 8, false, false), PATTERN("read1", 1, false, false), PATTERN("write1", 0, true, false),
      PATTERN("copy", 1, true, false),   PATTERN("mix8", 8, true, false),   PATTERN("mix8ip", 8, true, true),
      PATTERN("mix2", 2, true, false),   PATTERN("mix3", 3, true, false),   PATTERN("mix4", 4, true, false),
      PATTERN("mix6", 6, true, false),
  };
  const size_t bytes = mib << 20;
  if (bytes % Tile<kU, kThreads>::BYTES != 0 || sets < 1 || reps < 1) { std::printf("bad sizes\n"); return 2; }
  // every set: eight inputs and one output
  std::vector<std::vector<char *>> buf((size_t)sets, std::vector<char *>(9, nullptr));
  // mixed bits: the rate of a pattern depends a little on the data (all-zero buffers run several per cent
  // faster than real ones)
  unsigned salt = 1;
  for (auto &s : buf)
    for (auto &b : s) {
      CK(hipMalloc(reinterpret_cast<void **>(&b), bytes));
      hipLaunchKernelGGL(noise_kernel, dim3(4096), dim3(256), 0, 0, reinterpret_cast<unsigned *>(b), bytes / 4, salt++);
    }
  CK(hipGetLastError());
  CK(hipDeviceSynchronize());
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (const Pattern &pt : all) {
    bool run = want.empty();
    for (const auto &w : want) run = run || w == pt.name;
    if (!run) continue;
    for (int shape = 0; shape < 2; ++shape) {
      const bool stream = shape == 0;
      const size_t tile = stream ? kStreamTileBytes : Tile<kU, kThreads>::BYTES;
      const size_t tiles = bytes / tile;
      const size_t per_launch = stream ? tiles : ((size_t)64 << 20) / tile;
      const int streams = pt.nread > 0 ? pt.nread : 1;
      const int n = wgs ? wgs : stream_wgs_per_cu(false, streams, 1, (size_t)(pt.nread + pt.nwrite) * bytes);
      auto call = [&](int set) {
        Streams p;
        for (int k = 0; k < 8; ++k) p.in[k] = buf[(size_t)set][(size_t)k];
        p.out = pt.inplace ? buf[(size_t)set][7] : buf[(size_t)set][8];
        for (size_t t0 = 0; t0 < tiles; t0 += per_launch) {
          p.tile0 = t0;
          const size_t nt = tiles - t0 < per_launch ? tiles - t0 : per_launch;
          if (stream) hipLaunchKernelGGL(pt.stream, dim3((unsigned)nt), dim3(64), stream_lds_bytes(n), 0, p, 0xdeadbeefu);
          else hipLaunchKernelGGL(pt.block, dim3((unsigned)nt), dim3(kThreads), 0, 0, p, 0xdeadbeefu);
        }
      };
      for (int i = 0; i < sets; ++i) call(i);  // warm-up: one pass over every set
      CK(hipDeviceSynchronize());
      CK(hipEventRecord(e0));
      for (int i = 0; i < reps; ++i) call(i % sets);
      CK(hipEventRecord(e1));
      CK(hipEventSynchronize(e1));
      float ms = 0;
      CK(hipEventElapsedTime(&ms, e0, e1));
      const double moved = (double)(pt.nread + pt.nwrite) * (double)bytes * reps;
      std::printf("{\"pattern\": \"%s\", \"shape\": \"%s\", \"workgroups_per_cu\": %d, \"streams_read\": %d, "
                  "\"streams_written\": %d, \"mib_per_stream\": %zu, \"buffer_sets\": %d, \"calls\": %d, "
                  "\"launches_per_call\": %zu, \"ms_per_call\": %.4f, \"gbps\": %.1f, \"frac_of_8tbps\": %.4f}\n",
                  pt.name, stream ? "stream" : "block", stream ? n : 8, pt.nread, pt.nwrite, mib, sets, reps,
                  (tiles + per_launch - 1) / per_launch, ms / reps, moved / (ms * 1e-3) * 1e-9,
                  moved / (ms * 1e-3) * 1e-9 / 8000.0);
      std::fflush(stdout);
    }
  }
  return 0;
}
