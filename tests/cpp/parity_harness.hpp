// Parity harness shared by test_backend and test_ops: per-rank seeded inputs,
// the collective through the Aluminum-shaped front end on one GPU, the same
// collective by the CPU oracle, then a bit-exact comparison (the reference does
// the same against MPI with a tolerance: test/test_ops.cpp:200-225,
// test/op_runner.hpp:312-324).
#pragma once

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <thread>
#include <vector>

#include <unistd.h>

#include "aluminum_amd/Al.hpp"
#include "aluminum_amd_support.h"
#include "oracle.h"

using Backend = Al::HipCombineBackend;
using Algo = Al::amd::CombineAlgorithm;
using Op = Al::ReductionOperator;

static std::atomic<int> g_fail{0}, g_checks{0};  // one translation unit per program
static thread_local int t_fail = 0;               // the calling thread's share of g_fail
#define HIPCHK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); std::exit(2); } } while (0)
#define EXPECT(cond, ...) do { ++g_checks; if (!(cond)) { ++g_fail; ++t_fail; std::printf("FAIL line %d: ", __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); } } while (0)

template <typename T> struct DevBuf {
  T *p = nullptr;
  size_t n = 0;
  explicit DevBuf(size_t n_) : n(n_) { HIPCHK(hipMalloc(reinterpret_cast<void **>(&p), (n ? n : 1) * sizeof(T))); }
  ~DevBuf() { (void)hipFree(p); }
  void up(const std::vector<T> &h) { HIPCHK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> down() const {
    std::vector<T> h(n);
    HIPCHK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
};

template <typename T> std::vector<T> gen(size_t n, int dist, unsigned seed) {
  std::vector<T> v(n);
  alo_fill(v.data(), n, Al::amd::TypeMap<T>::value, dist, seed, 0);
  return v;
}

// The special values that tests/golden/mpich_golden.c (plant_specials_many) plants for more than two ranks:
// element i of `rank` comes from a pool of NaN, zeros of both signs, infinities, denormals and a few
// ordinary values by a fixed rule; every fourth element is a zero of one sign or the other.
template <typename T> std::vector<T> planted(size_t n, int rank) {
  static const uint32_t pool[] = {0x7fc00000u, 0xbf800000u, 0x00000000u, 0x80000000u, 0x7f800000u,
                                  0xff800000u, 0x00000001u, 0x80000001u, 0x3f800000u, 0x7f7fffffu,
                                  0x00800000u, 0x00400000u, 0x3e99999au};
  const size_t cnt = sizeof(pool) / sizeof(pool[0]);
  std::vector<T> v(n);
  for (size_t i = 0; i < n; ++i) {
    const uint64_t h = alo_mix64(77, (uint64_t)i * 64u + (uint64_t)rank);
    uint32_t u = pool[(size_t)(h % cnt)];
    if (i % 4 == 0) u = (h >> 32) % 3 == 0 ? 0x80000000u : 0u;
    float f;
    std::memcpy(&f, &u, 4);
    if constexpr (std::is_same<T, float>::value) v[i] = f;
    else if constexpr (std::is_same<T, double>::value) v[i] = (double)f;
    else if constexpr (std::is_same<T, Al::amd::bfloat16_bits>::value) v[i].bits = alo_f32_to_bf16(f);
    else if constexpr (std::is_same<T, Al::amd::half_bits>::value) v[i].bits = alo_f32_to_f16(f);
    else v[i] = T();
  }
  return v;
}

// NaN payloads are outside the parity claim; the seeded inputs hold no NaN.
template <typename T> bool same_bits(const std::vector<T> &a, const std::vector<T> &b) {
  return a.size() == b.size() && (a.empty() || std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0);
}

// The oracle's order for an algorithm of the front end.  `automatic` is stated here on its own, not
// asked of the library: what MPICH 3.3.2 does on one host (pinned by the golden vectors in tests/golden;
// test_backend's test_automatic_against_mpich checks the front end itself against that library's bits).
static int order_of(Algo a, size_t total_bytes) {
  switch (a) {
  case Algo::automatic:  // Reduce_scatter(v); Allreduce and Reduce go through rooted_order
  case Algo::automatic_mpi_blocking:
    return total_bytes < (512u << 10) ? ALO_ORDER_TREE_HALV : ALO_ORDER_PAIRWISE_DESC;
  case Algo::rank_order: return ALO_ORDER_RANK_ASC;
  case Algo::tree_doubling: return ALO_ORDER_TREE_DBL;
  case Algo::tree_halving: return ALO_ORDER_TREE_HALV;
  case Algo::tree_binomial: return ALO_ORDER_TREE_BINOMIAL;
  case Algo::tree_reduce_scatter_gather: return ALO_ORDER_TREE_RSG;
  case Algo::tree_reduce_scatter_gather_spread: return ALO_ORDER_TREE_RSG_SPREAD;
  case Algo::pairwise: return ALO_ORDER_PAIRWISE_DESC;
  default: return ALO_ORDER_RING;
  }
}

struct OrderPick { int order, start; };
// Allreduce (root = 0) and Reduce.
static OrderPick rooted_order(Algo a, int dt, size_t count, size_t elem_size, int P, int root) {
  if (a == Algo::automatic || a == Algo::automatic_mpi_blocking) {
    size_t pof2 = 1;
    while (2 * pof2 <= (size_t)P) pof2 *= 2;
    const bool user_op = dt == ALO_F16 || dt == ALO_BF16;
    if (user_op || count * elem_size <= 2048 || count < pof2) return {ALO_ORDER_TREE_BINOMIAL, root};
    return {a == Algo::automatic ? ALO_ORDER_TREE_RSG : ALO_ORDER_TREE_RSG_SPREAD, 0};
  }
  if (a == Algo::tree_binomial) return {ALO_ORDER_TREE_BINOMIAL, root};
  return {order_of(a, 0), 0};
}

template <typename T>
void test_allreduce(int P, size_t n, Op op, Algo algo, int dist, bool inplace, bool nonblocking, hipStream_t stream) {
  const int dt = Al::amd::TypeMap<T>::value;
  std::vector<std::vector<T>> in;
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  for (int r = 0; r < P; ++r) {
    in.push_back(gen<T>(n, dist, 1000u + (unsigned)r));
    send.emplace_back(new DevBuf<T>(n));
    recv.emplace_back(new DevBuf<T>(n));
    send[r]->up(in[r]);
  }
  Al::amd::World world(P, stream);
  std::vector<Backend::req_type> reqs(P);
  for (int r = 0; r < P; ++r) {
    auto &comm = world.comm(r);
    if (nonblocking) {
      if (inplace) Al::NonblockingAllreduce<Backend>(send[r]->p, n, op, comm, reqs[r], algo);
      else Al::NonblockingAllreduce<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, n, op, comm, reqs[r], algo);
      if (r + 1 < P) EXPECT(!Al::Test<Backend>(reqs[r]), "request complete before every rank called");
    } else if (inplace) {
      Al::Allreduce<Backend>(send[r]->p, n, op, comm, algo);
    } else {
      Al::Allreduce<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, n, op, comm, algo);
    }
  }
  if (nonblocking)
    for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
  HIPCHK(hipStreamSynchronize(stream));
  if (nonblocking)
    for (int r = 0; r < P; ++r) EXPECT(Al::Test<Backend>(reqs[r]), "request not complete after synchronisation");

  std::vector<T> want(n);
  if (algo == Algo::ring || algo == Algo::ring_fused) {
    std::vector<std::vector<T>> bufs = in;
    std::vector<void *> ptrs;
    for (auto &b : bufs) ptrs.push_back(b.data());
    alo_ring_allreduce(ptrs.data(), P, n, dt, (int)op, (size_t)(4u << 20) / sizeof(T));
    want = bufs[0];
  } else {
    std::vector<const void *> ptrs;
    for (auto &b : in) ptrs.push_back(b.data());
    const OrderPick pick = rooted_order(algo, dt, n, sizeof(T), P, 0);
    alo_combine(want.data(), ptrs.data(), P, n, dt, (int)op, pick.order, pick.start);
  }
  for (int r = 0; r < P; ++r) {
    auto got = inplace ? send[r]->down() : recv[r]->down();
    EXPECT(same_bits(got, want), "allreduce dt=%d P=%d n=%zu op=%d algo=%d inplace=%d nb=%d rank %d", dt, P, n,
           (int)op, (int)algo, inplace, nonblocking, r);
  }
}

template <typename T>
void test_reduce(int P, size_t n, Op op, int root, hipStream_t stream, int nonblocking = -1, bool inplace = false,
                 int dist = ALO_DIST_UNIFORM_PM1, Algo algo = Algo::automatic) {
  const int dt = Al::amd::TypeMap<T>::value;
  std::vector<std::vector<T>> in;
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  std::vector<T> marker(n);
  if (n) std::memset(marker.data(), 0x5a, n * sizeof(T));
  for (int r = 0; r < P; ++r) {
    in.push_back(gen<T>(n, dist, 1000u + (unsigned)r));
    send.emplace_back(new DevBuf<T>(n));
    recv.emplace_back(new DevBuf<T>(n));
    send[r]->up(in[r]);
    recv[r]->up(marker);
  }
  Al::amd::World world(P, stream);
  std::vector<Backend::req_type> reqs(P);
  const bool nb = nonblocking < 0 ? (n % 2) == 0 : nonblocking != 0;  // default: even sizes non-blocking
  for (int r = P - 1; r >= 0; --r) {  // any calling order
    if (inplace) {
      if (nb) Al::NonblockingReduce<Backend>(send[r]->p, n, op, root, world.comm(r), reqs[r], algo);
      else Al::Reduce<Backend>(send[r]->p, n, op, root, world.comm(r), algo);
    } else if (nb) {
      Al::NonblockingReduce<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, n, op, root, world.comm(r), reqs[r], algo);
    } else {
      Al::Reduce<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, n, op, root, world.comm(r), algo);
    }
  }
  for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
  HIPCHK(hipStreamSynchronize(stream));
  std::vector<T> want(n);
  std::vector<const void *> ptrs;
  for (auto &b : in) ptrs.push_back(b.data());
  const OrderPick pick = rooted_order(algo, dt, n, sizeof(T), P, root);
  alo_combine(want.data(), ptrs.data(), P, n, dt, (int)op, pick.order, pick.start);
  for (int r = 0; r < P; ++r) {
    // in place only the root's buffer changes; the others keep their contribution
    if (inplace) EXPECT(same_bits(send[r]->down(), r == root ? want : in[r]), "reduce in place P=%d n=%zu root=%d rank %d", P, n, root, r);
    else EXPECT(same_bits(recv[r]->down(), r == root ? want : marker), "reduce P=%d n=%zu root=%d rank %d", P, n, root, r);
  }
}

template <typename T>
void test_reduce_scatter(int P, size_t count, Op op, Algo algo, bool inplace, hipStream_t stream,
                         bool nonblocking = false, int dist = ALO_DIST_UNIFORM_PM1) {
  const int dt = Al::amd::TypeMap<T>::value;
  const size_t n = count * (size_t)P;
  std::vector<std::vector<T>> in;
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  for (int r = 0; r < P; ++r) {
    in.push_back(gen<T>(n, dist, 1000u + (unsigned)r));
    send.emplace_back(new DevBuf<T>(n));
    recv.emplace_back(new DevBuf<T>(count));
    send[r]->up(in[r]);
  }
  Al::amd::World world(P, stream);
  std::vector<Backend::req_type> reqs(P);
  for (int r = 0; r < P; ++r) {
    if (nonblocking) {
      if (inplace) Al::NonblockingReduce_scatter<Backend>(send[r]->p, count, op, world.comm(r), reqs[r], algo);
      else Al::NonblockingReduce_scatter<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, count, op, world.comm(r), reqs[r], algo);
    } else if (inplace) {
      Al::Reduce_scatter<Backend>(send[r]->p, count, op, world.comm(r), algo);
    } else {
      Al::Reduce_scatter<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, count, op, world.comm(r), algo);
    }
  }
  for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
  HIPCHK(hipStreamSynchronize(stream));
  std::vector<std::vector<T>> want(P, std::vector<T>(count));
  std::vector<const void *> sp;
  std::vector<void *> rp;
  for (int r = 0; r < P; ++r) { sp.push_back(in[r].data()); rp.push_back(want[r].data()); }
  alo_reduce_scatter(rp.data(), sp.data(), P, count, dt, (int)op,
                     algo == Algo::ring_fused ? ALO_ORDER_RING : order_of(algo, n * sizeof(T)));
  for (int r = 0; r < P; ++r) {
    auto got = inplace ? send[r]->down() : recv[r]->down();
    got.resize(count);  // in place the result is at the start of the buffer
    EXPECT(same_bits(got, want[r]), "reduce_scatter P=%d count=%zu algo=%d inplace=%d rank %d", P, count, (int)algo,
           inplace, r);
  }
}

template <typename T> void test_allgather(int P, size_t count, bool inplace, hipStream_t stream, bool nonblocking = false) {
  std::vector<std::vector<T>> in;
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  std::vector<T> want;
  for (int r = 0; r < P; ++r) {
    in.push_back(gen<T>(count, ALO_DIST_UNIFORM_PM1, 1000u + (unsigned)r));
    want.insert(want.end(), in[r].begin(), in[r].end());
    send.emplace_back(new DevBuf<T>(count));
    recv.emplace_back(new DevBuf<T>(count * (size_t)P));
    send[r]->up(in[r]);
    if (inplace) HIPCHK(hipMemcpy(recv[r]->p + (size_t)r * count, in[r].data(), count * sizeof(T), hipMemcpyHostToDevice));
  }
  Al::amd::World world(P, stream);
  std::vector<Backend::req_type> reqs(P);
  for (int r = 0; r < P; ++r) {
    if (nonblocking) {
      if (inplace) Al::NonblockingAllgather<Backend>(recv[r]->p, count, world.comm(r), reqs[r]);
      else Al::NonblockingAllgather<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, count, world.comm(r), reqs[r]);
    } else if (inplace) {
      Al::Allgather<Backend>(recv[r]->p, count, world.comm(r));
    } else {
      Al::Allgather<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, count, world.comm(r));
    }
  }
  for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
  HIPCHK(hipStreamSynchronize(stream));
  for (int r = 0; r < P; ++r)
    EXPECT(same_bits(recv[r]->down(), want), "allgather P=%d count=%zu inplace=%d rank %d", P, count, inplace, r);
}

// Per-rank counts base + unit*((3b) mod 5), rank 1 contributing nothing.
template <typename T>
void test_v_variants(int P, bool inplace, hipStream_t stream, bool nonblocking = false, size_t base = 5,
                     size_t unit = 37, Op op = Op::sum, bool do_reduce_scatterv = true, bool do_allgatherv = true,
                     int dist = ALO_DIST_UNIFORM_PM1) {
  const int dt = Al::amd::TypeMap<T>::value;
  std::vector<size_t> counts, displs_ag;
  size_t total = 0;
  for (int b = 0; b < P; ++b) { counts.push_back(b == 1 ? 0 : base + unit * (size_t)((b * 3) % 5)); total += counts.back(); }
  if (do_reduce_scatterv) {
    std::vector<std::vector<T>> in;
    std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
    for (int r = 0; r < P; ++r) {
      in.push_back(gen<T>(total, dist, 300u + (unsigned)r));
      send.emplace_back(new DevBuf<T>(total));
      recv.emplace_back(new DevBuf<T>(counts[r]));
      send[r]->up(in[r]);
    }
    Al::amd::World world(P, stream);
    std::vector<Backend::req_type> reqs(P);
    for (int r = 0; r < P; ++r) {
      if (nonblocking) {
        if (inplace) Al::NonblockingReduce_scatterv<Backend>(send[r]->p, counts, op, world.comm(r), reqs[r]);
        else Al::NonblockingReduce_scatterv<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, counts, op, world.comm(r), reqs[r]);
      } else if (inplace) {
        Al::Reduce_scatterv<Backend>(send[r]->p, counts, op, world.comm(r));
      } else {
        Al::Reduce_scatterv<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, counts, op, world.comm(r));
      }
    }
    for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
    HIPCHK(hipStreamSynchronize(stream));
    std::vector<std::vector<T>> want;
    std::vector<const void *> sp;
    std::vector<void *> rp;
    for (int r = 0; r < P; ++r) { want.emplace_back(counts[r] ? counts[r] : 1); sp.push_back(in[r].data()); }
    for (int r = 0; r < P; ++r) rp.push_back(want[r].data());
    alo_reduce_scatterv(rp.data(), sp.data(), P, counts.data(), dt, (int)op,
                        order_of(Algo::automatic, total * sizeof(T)));
    for (int r = 0; r < P; ++r) {
      auto got = inplace ? send[r]->down() : recv[r]->down();
      got.resize(counts[r]);
      want[r].resize(counts[r]);
      EXPECT(same_bits(got, want[r]), "reduce_scatterv P=%d inplace=%d rank %d", P, inplace, r);
    }
  }
  // allgatherv: slices placed back to front
  if (do_allgatherv) {
    size_t at = total;
    for (int q = 0; q < P; ++q) { at -= counts[q]; displs_ag.push_back(at); }
    std::vector<std::vector<T>> in;
    std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
    std::vector<T> want(total);
    for (int r = 0; r < P; ++r) {
      in.push_back(gen<T>(counts[r], ALO_DIST_UNIFORM_PM1, 400u + (unsigned)r));
      std::copy(in[r].begin(), in[r].end(), want.begin() + (long)displs_ag[r]);
      send.emplace_back(new DevBuf<T>(counts[r]));
      recv.emplace_back(new DevBuf<T>(total));
      send[r]->up(in[r]);
      if (inplace && counts[r])
        HIPCHK(hipMemcpy(recv[r]->p + displs_ag[r], in[r].data(), counts[r] * sizeof(T), hipMemcpyHostToDevice));
    }
    Al::amd::World world(P, stream);
    std::vector<Backend::req_type> reqs(P);
    for (int r = 0; r < P; ++r) {
      if (nonblocking) {
        if (inplace) Al::NonblockingAllgatherv<Backend>(recv[r]->p, counts, displs_ag, world.comm(r), reqs[r]);
        else Al::NonblockingAllgatherv<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, counts, displs_ag, world.comm(r), reqs[r]);
      } else if (inplace) {
        Al::Allgatherv<Backend>(recv[r]->p, counts, displs_ag, world.comm(r));
      } else {
        Al::Allgatherv<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, counts, displs_ag, world.comm(r));
      }
    }
    for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
    HIPCHK(hipStreamSynchronize(stream));
    for (int r = 0; r < P; ++r)
      EXPECT(same_bits(recv[r]->down(), want), "allgatherv P=%d inplace=%d rank %d", P, inplace, r);
  }
}
