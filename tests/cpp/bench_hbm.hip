// What the memory system gives to the access patterns the combine is made of,
// with the tile structure of the library's kernels (alamd_tile.h: 128 threads x
// 8 vectors of 128 bits per stream, non-temporal loads, write-through stores,
// two waves per SIMD, launches of 4096 tiles per stream) and nothing else: no
// arithmetic beyond an xor, no layout logic.  Every pattern walks rotating
// buffer sets, so that nothing a launch touches was touched by the launches
// just before it.
//
//   read8    eight streams read, nothing written
//   read1    one stream read
//   write1   one stream written
//   copy     one read, one written
//   mix8     eight read, one written (the shape of the P = 8 fold)
//   mix8ip   eight read, the result written over the stream read last
//   mix2, mix3, mix4, mix6   the folds of fewer ranks
//
// usage: bench_hbm [pattern ...] [--mib N per stream, default 256] [--sets S, default 4] [--reps R, default 12]
// Prints one JSON line per pattern.  A bench / profiling aid; not part of the library.
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

constexpr int kU = 8, kThreads = 128;
using TL = Tile<kU, kThreads>;

struct Streams {
  const char *in[8];
  char *out;
  unsigned long long tile0;
};

// NR streams read (xor-combined), one written if WRITE; a read-only kernel stores only if the xor of
// everything it read equals a value no input produces, i.e. never.
template <int NR, bool WRITE>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 2)))
probe_kernel(const Streams p, unsigned never) {
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
    for (int u = 0; u < kU; ++u) any |= (acc[u][0] == never && acc[u][1] == never) ? 1u : 0u;
    store = any != 0;
  }
  if (store) {
    const auto r = TL::rsrc(p.out + tb, (int)TL::BYTES);
#pragma unroll
    for (int u = 0; u < kU; ++u) tl.store(r, u, acc[u]);
  }
}

struct Pattern {
  const char *name;
  int nread, nwrite;
  bool inplace;
  void (*kern)(const Streams, unsigned);
};

int main(int argc, char **argv) {
  size_t mib = 256;
  int sets = 4, reps = 12;
  std::vector<std::string> want;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--mib" && i + 1 < argc) mib = std::strtoull(argv[++i], nullptr, 10);
    else if (a == "--sets" && i + 1 < argc) sets = std::atoi(argv[++i]);
    else if (a == "--reps" && i + 1 < argc) reps = std::atoi(argv[++i]);
    else want.push_back(a);
  }
  const Pattern all[] = {
      {"read8", 8, 0, false, probe_kernel<8, false>}, {"read1", 1, 0, false, probe_kernel<1, false>},
      {"write1", 0, 1, false, probe_kernel<0, true>}, {"copy", 1, 1, false, probe_kernel<1, true>},
      {"mix8", 8, 1, false, probe_kernel<8, true>},   {"mix8ip", 8, 1, true, probe_kernel<8, true>},
      {"mix2", 2, 1, false, probe_kernel<2, true>},   {"mix3", 3, 1, false, probe_kernel<3, true>},
      {"mix4", 4, 1, false, probe_kernel<4, true>},   {"mix6", 6, 1, false, probe_kernel<6, true>},
  };
  const size_t bytes = mib << 20;
  if (bytes % TL::BYTES != 0 || sets < 1 || reps < 1) { std::printf("bad sizes\n"); return 2; }
  const size_t tiles = bytes / TL::BYTES;
  // every set: eight inputs and one output
  std::vector<std::vector<char *>> buf((size_t)sets, std::vector<char *>(9, nullptr));
  for (auto &s : buf)
    for (auto &b : s) {
      CK(hipMalloc(reinterpret_cast<void **>(&b), bytes));
      CK(hipMemset(b, 0x5a, bytes));
    }
  CK(hipDeviceSynchronize());
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (const Pattern &pt : all) {
    bool run = want.empty();
    for (const auto &w : want) run = run || w == pt.name;
    if (!run) continue;
    // the library's launch cut: about 0.6 GiB over all streams of a launch
    const size_t per_launch = launch_tiles(pt.nread, TL::BYTES);
    auto call = [&](int set) {
      Streams p;
      for (int k = 0; k < 8; ++k) p.in[k] = buf[(size_t)set][(size_t)k];
      p.out = pt.inplace ? buf[(size_t)set][7] : buf[(size_t)set][8];
      for (size_t t0 = 0; t0 < tiles; t0 += per_launch) {
        p.tile0 = t0;
        const size_t nt = tiles - t0 < per_launch ? tiles - t0 : per_launch;
        hipLaunchKernelGGL(pt.kern, dim3((unsigned)nt), dim3(kThreads), 0, 0, p, 0xdeadbeefu);
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
    std::printf("{\"pattern\": \"%s\", \"streams_read\": %d, \"streams_written\": %d, \"mib_per_stream\": %zu, "
                "\"buffer_sets\": %d, \"calls\": %d, \"launches_per_call\": %zu, \"ms_per_call\": %.4f, "
                "\"gbps\": %.1f, \"frac_of_8tbps\": %.4f}\n",
                pt.name, pt.nread, pt.nwrite, mib, sets, reps, (tiles + per_launch - 1) / per_launch, ms / reps,
                moved / (ms * 1e-3) * 1e-9, moved / (ms * 1e-3) * 1e-9 / 8000.0);
    std::fflush(stdout);
  }
  return 0;
}
