// Parity test of the Aluminum-shaped C++ front end (include/aluminum_amd/Al.hpp)
// against the CPU oracle, in the manner of the reference's test_ops
// (test/test_ops.cpp:200-225, test/op_runner.hpp:312-324): per-rank seeded
// inputs, the collective through the backend, the same collective on the host,
// then an element-wise comparison - bit-exact here.
//
// Runs on one GPU; every logical rank of the World lives in its memory.
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "aluminum_amd/Al.hpp"
#include "oracle.h"

using Backend = Al::HipCombineBackend;
using Algo = Al::amd::CombineAlgorithm;
using Op = Al::ReductionOperator;

static int g_fail = 0, g_checks = 0;
#define HIPCHK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); std::exit(2); } } while (0)
#define EXPECT(cond, ...) do { ++g_checks; if (!(cond)) { ++g_fail; std::printf("FAIL line %d: ", __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); } } while (0)

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

// NaN payloads are outside the parity claim; the seeded inputs hold no NaN.
template <typename T> bool same_bits(const std::vector<T> &a, const std::vector<T> &b) {
  return a.size() == b.size() && (a.empty() || std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0);
}

static int order_of(Algo a, size_t bytes, bool reduce_scatter, size_t total_bytes) {
  switch (a) {
  case Algo::automatic:
    if (reduce_scatter) return total_bytes < (512u << 10) ? ALO_ORDER_TREE_HALV : ALO_ORDER_PAIRWISE_DESC;
    return bytes <= 2048 ? ALO_ORDER_TREE_BINOMIAL : ALO_ORDER_TREE_DBL;
  case Algo::rank_order: return ALO_ORDER_RANK_ASC;
  case Algo::tree_doubling: return ALO_ORDER_TREE_DBL;
  case Algo::tree_halving: return ALO_ORDER_TREE_HALV;
  case Algo::tree_binomial: return ALO_ORDER_TREE_BINOMIAL;
  case Algo::pairwise: return ALO_ORDER_PAIRWISE_DESC;
  default: return ALO_ORDER_RING;
  }
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
    alo_combine(want.data(), ptrs.data(), P, n, dt, (int)op, order_of(algo, n * sizeof(T), false, 0), 0);
  }
  for (int r = 0; r < P; ++r) {
    auto got = inplace ? send[r]->down() : recv[r]->down();
    EXPECT(same_bits(got, want), "allreduce dt=%d P=%d n=%zu op=%d algo=%d inplace=%d nb=%d rank %d", dt, P, n,
           (int)op, (int)algo, inplace, nonblocking, r);
  }
}

template <typename T> void test_reduce(int P, size_t n, Op op, int root, hipStream_t stream) {
  const int dt = Al::amd::TypeMap<T>::value;
  std::vector<std::vector<T>> in;
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  const std::vector<T> marker(n, T(7));
  for (int r = 0; r < P; ++r) {
    in.push_back(gen<T>(n, ALO_DIST_UNIFORM_PM1, 1000u + (unsigned)r));
    send.emplace_back(new DevBuf<T>(n));
    recv.emplace_back(new DevBuf<T>(n));
    send[r]->up(in[r]);
    recv[r]->up(marker);
  }
  Al::amd::World world(P, stream);
  std::vector<Backend::req_type> reqs(P);
  const bool nb = (n % 2) == 0;  // even sizes go through the non-blocking form
  for (int r = P - 1; r >= 0; --r) {  // any calling order
    if (nb) Al::NonblockingReduce<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, n, op, root, world.comm(r), reqs[r]);
    else Al::Reduce<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, n, op, root, world.comm(r));
  }
  for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
  HIPCHK(hipStreamSynchronize(stream));
  std::vector<T> want(n);
  std::vector<const void *> ptrs;
  for (auto &b : in) ptrs.push_back(b.data());
  alo_combine(want.data(), ptrs.data(), P, n, dt, (int)op, order_of(Algo::automatic, n * sizeof(T), false, 0), 0);
  for (int r = 0; r < P; ++r)
    EXPECT(same_bits(recv[r]->down(), r == root ? want : marker), "reduce P=%d n=%zu root=%d rank %d", P, n, root, r);
}

template <typename T> void test_reduce_scatter(int P, size_t count, Op op, Algo algo, bool inplace, hipStream_t stream) {
  const int dt = Al::amd::TypeMap<T>::value;
  const size_t n = count * (size_t)P;
  std::vector<std::vector<T>> in;
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  for (int r = 0; r < P; ++r) {
    in.push_back(gen<T>(n, ALO_DIST_UNIFORM_PM1, 1000u + (unsigned)r));
    send.emplace_back(new DevBuf<T>(n));
    recv.emplace_back(new DevBuf<T>(count));
    send[r]->up(in[r]);
  }
  Al::amd::World world(P, stream);
  for (int r = 0; r < P; ++r) {
    if (inplace) Al::Reduce_scatter<Backend>(send[r]->p, count, op, world.comm(r), algo);
    else Al::Reduce_scatter<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, count, op, world.comm(r), algo);
  }
  HIPCHK(hipStreamSynchronize(stream));
  std::vector<std::vector<T>> want(P, std::vector<T>(count));
  std::vector<const void *> sp;
  std::vector<void *> rp;
  for (int r = 0; r < P; ++r) { sp.push_back(in[r].data()); rp.push_back(want[r].data()); }
  alo_reduce_scatter(rp.data(), sp.data(), P, count, dt, (int)op,
                     algo == Algo::ring_fused ? ALO_ORDER_RING : order_of(algo, 0, true, n * sizeof(T)));
  for (int r = 0; r < P; ++r) {
    auto got = inplace ? send[r]->down() : recv[r]->down();
    got.resize(count);  // in place the result is at the start of the buffer
    EXPECT(same_bits(got, want[r]), "reduce_scatter P=%d count=%zu algo=%d inplace=%d rank %d", P, count, (int)algo,
           inplace, r);
  }
}

template <typename T> void test_allgather(int P, size_t count, bool inplace, hipStream_t stream) {
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
  for (int r = 0; r < P; ++r) {
    if (inplace) Al::Allgather<Backend>(recv[r]->p, count, world.comm(r));
    else Al::Allgather<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, count, world.comm(r));
  }
  HIPCHK(hipStreamSynchronize(stream));
  for (int r = 0; r < P; ++r)
    EXPECT(same_bits(recv[r]->down(), want), "allgather P=%d count=%zu inplace=%d rank %d", P, count, inplace, r);
}

template <typename T> void test_v_variants(int P, bool inplace, hipStream_t stream) {
  const int dt = Al::amd::TypeMap<T>::value;
  std::vector<size_t> counts, displs_ag;
  size_t total = 0;
  for (int b = 0; b < P; ++b) { counts.push_back(b == 1 ? 0 : 5 + 37 * (size_t)((b * 3) % 5)); total += counts.back(); }
  // reduce_scatterv
  {
    std::vector<std::vector<T>> in;
    std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
    for (int r = 0; r < P; ++r) {
      in.push_back(gen<T>(total, ALO_DIST_UNIFORM_PM1, 300u + (unsigned)r));
      send.emplace_back(new DevBuf<T>(total));
      recv.emplace_back(new DevBuf<T>(counts[r]));
      send[r]->up(in[r]);
    }
    Al::amd::World world(P, stream);
    for (int r = 0; r < P; ++r) {
      if (inplace) Al::Reduce_scatterv<Backend>(send[r]->p, counts, Op::sum, world.comm(r));
      else Al::Reduce_scatterv<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, counts, Op::sum, world.comm(r));
    }
    HIPCHK(hipStreamSynchronize(stream));
    std::vector<std::vector<T>> want;
    std::vector<const void *> sp;
    std::vector<void *> rp;
    for (int r = 0; r < P; ++r) { want.emplace_back(counts[r] ? counts[r] : 1); sp.push_back(in[r].data()); }
    for (int r = 0; r < P; ++r) rp.push_back(want[r].data());
    alo_reduce_scatterv(rp.data(), sp.data(), P, counts.data(), dt, ALO_SUM, ALO_ORDER_TREE_HALV);
    for (int r = 0; r < P; ++r) {
      auto got = inplace ? send[r]->down() : recv[r]->down();
      got.resize(counts[r]);
      want[r].resize(counts[r]);
      EXPECT(same_bits(got, want[r]), "reduce_scatterv P=%d inplace=%d rank %d", P, inplace, r);
    }
  }
  // allgatherv: slices placed back to front
  {
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
    for (int r = 0; r < P; ++r) {
      if (inplace) Al::Allgatherv<Backend>(recv[r]->p, counts, displs_ag, world.comm(r));
      else Al::Allgatherv<Backend>(static_cast<const T *>(send[r]->p), recv[r]->p, counts, displs_ag, world.comm(r));
    }
    HIPCHK(hipStreamSynchronize(stream));
    for (int r = 0; r < P; ++r)
      EXPECT(same_bits(recv[r]->down(), want), "allgatherv P=%d inplace=%d rank %d", P, inplace, r);
  }
}

static void test_errors(hipStream_t stream) {
  DevBuf<float> a(64), b(64);
  Al::amd::World world(2, stream);
  bool threw = false;
  try {
    Al::Allreduce<Backend>(a.p, 64, Op::avg, world.comm(0));
    Al::Allreduce<Backend>(b.p, 64, Op::avg, world.comm(1));
  } catch (const Al::al_exception &e) {
    threw = std::string(e.what()).find("Reduction operator not supported") != std::string::npos;
  }
  EXPECT(threw, "avg must throw 'Reduction operator not supported'");
  Al::amd::World w2(2, stream);
  threw = false;
  try {
    Al::Allreduce<Backend>(a.p, 64, Op::sum, w2.comm(0));
    Al::Allreduce<Backend>(b.p, 32, Op::sum, w2.comm(1));
  } catch (const Al::al_exception &) { threw = true; }
  EXPECT(threw, "mismatched counts must throw");
  Al::amd::World w3(2, stream);
  threw = false;
  try { Al::Reduce<Backend>(a.p, 64, Op::sum, 5, w3.comm(0)); } catch (const Al::al_exception &) { threw = true; }
  EXPECT(threw, "bad root must throw");
  threw = false;
  try { Al::amd::World w4(0, stream); } catch (const Al::al_exception &) { threw = true; }
  EXPECT(threw, "empty world must throw");
  EXPECT(Backend::Name() == "HipCombineBackend", "backend name");
  Backend::req_type none = Backend::null_req;
  EXPECT(Al::Test<Backend>(none), "null request tests complete");
  Al::Wait<Backend>(none);
}

// Several collectives in flight, posted by P threads, each rank on its own stream.
static void test_threads_and_streams() {
  const int P = 4;
  const size_t n = 10000;
  std::vector<hipStream_t> streams(P);
  for (auto &s : streams) HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  {
    Al::amd::World world(streams);
    std::vector<std::vector<float>> in;
    std::vector<std::unique_ptr<DevBuf<float>>> buf, out2;
    for (int r = 0; r < P; ++r) {
      in.push_back(gen<float>(n, ALO_DIST_UNIFORM_PM1, 50u + (unsigned)r));
      buf.emplace_back(new DevBuf<float>(n));
      out2.emplace_back(new DevBuf<float>(n));
    }
    std::vector<std::thread> th;
    for (int r = 0; r < P; ++r)
      th.emplace_back([&, r] {
        HIPCHK(hipMemcpyAsync(buf[r]->p, in[r].data(), n * sizeof(float), hipMemcpyHostToDevice, streams[r]));
        // two dependent collectives back to back on this rank's stream
        Al::Allreduce<Backend>(buf[r]->p, n, Op::sum, world.comm(r), Algo::rank_order);
        Al::Allreduce<Backend>(static_cast<const float *>(buf[r]->p), out2[r]->p, n, Op::max, world.comm(r), Algo::rank_order);
      });
    for (auto &t : th) t.join();
    for (auto &s : streams) HIPCHK(hipStreamSynchronize(s));
    std::vector<float> want(n);
    std::vector<const void *> ptrs;
    for (auto &b : in) ptrs.push_back(b.data());
    alo_combine(want.data(), ptrs.data(), P, n, ALO_F32, ALO_SUM, ALO_ORDER_RANK_ASC, 0);
    for (int r = 0; r < P; ++r) {
      EXPECT(same_bits(buf[r]->down(), want), "threaded allreduce #1 rank %d", r);
      EXPECT(same_bits(out2[r]->down(), want), "threaded allreduce #2 (max of equal values) rank %d", r);
    }
  }
  for (auto &s : streams) HIPCHK(hipStreamDestroy(s));
}

static void test_flags(hipStream_t stream) {
  Al::amd::GPUStatusFlag done;
  EXPECT(done.query(), "status flag starts complete");
  Al::amd::GPUWait gate;
  DevBuf<int> x(1);
  HIPCHK(hipMemsetAsync(x.p, 0, sizeof(int), stream));
  gate.wait(stream, 1u << 22);  // bounded: the kernel ends by itself if the test dies
  HIPCHK(hipMemsetAsync(x.p, 1, sizeof(int), stream));
  done.record(stream);
  EXPECT(!done.query(), "stream ran past an unsignalled wait");
  gate.signal();
  HIPCHK(hipStreamSynchronize(stream));
  EXPECT(done.query(), "status flag set after the stream drained");
  EXPECT(!gate.timed_out(), "wait must not have expired");
  EXPECT(x.down()[0] == 0x01010101, "work behind the wait ran");
}

int main() {
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { std::printf("no GPU\n"); return 2; }
  HIPCHK(hipSetDevice(0));
  hipStream_t stream;
  HIPCHK(hipStreamCreate(&stream));
  alo_set_num_threads(4);

  const size_t sizes[] = {1, 2, 5, 64, 513, 4096, 4097, 65536, (1u << 20) + 1};
  const Algo algos[] = {Algo::automatic, Algo::rank_order, Algo::tree_doubling, Algo::tree_halving,
                        Algo::tree_binomial, Algo::ring, Algo::ring_fused};
  for (int P : {1, 2, 4, 7, 8})
    for (size_t n : sizes) {
      for (Algo a : algos) test_allreduce<float>(P, n, Op::sum, a, ALO_DIST_UNIFORM_PM1, false, false, stream);
      test_allreduce<float>(P, n, Op::prod, Algo::automatic, ALO_DIST_UNIFORM_09_11, true, false, stream);
      test_allreduce<double>(P, n, Op::sum, Algo::automatic, ALO_DIST_UNIFORM_PM1, false, true, stream);
      test_allreduce<double>(P, n, Op::min, Algo::tree_halving, ALO_DIST_UNIFORM_PM1, true, true, stream);
      test_allreduce<Al::amd::bfloat16_bits>(P, n, Op::sum, Algo::ring, ALO_DIST_NORMAL, true, false, stream);
      test_allreduce<Al::amd::half_bits>(P, n, Op::max, Algo::rank_order, ALO_DIST_NORMAL, false, false, stream);
      test_allreduce<int>(P, n, Op::bxor, Algo::automatic, ALO_DIST_FULLRANGE, false, false, stream);
      test_allreduce<unsigned char>(P, n, Op::lxor, Algo::automatic, ALO_DIST_BOOL01, true, false, stream);
      test_allreduce<long>(P, n, Op::max, Algo::automatic, ALO_DIST_FULLRANGE, false, false, stream);
      test_allreduce<short>(P, n, Op::sum, Algo::ring_fused, ALO_DIST_FULLRANGE, false, false, stream);
    }
  for (int P : {2, 5, 8})
    for (size_t n : {size_t(1), size_t(100), size_t(70001)})
      for (int root : {0, P - 1}) test_reduce<float>(P, n, Op::sum, root, stream);
  for (int P : {1, 2, 5, 8})
    for (size_t count : {size_t(1), size_t(8), size_t(1000), size_t(20000)})
      for (Algo a : {Algo::automatic, Algo::rank_order, Algo::tree_halving, Algo::pairwise, Algo::ring_fused})
        for (bool inplace : {false, true}) {
          test_reduce_scatter<float>(P, count, Op::sum, a, inplace, stream);
          test_reduce_scatter<long long>(P, count, Op::min, a, inplace, stream);
        }
  for (int P : {1, 3, 8})
    for (size_t count : {size_t(1), size_t(33), size_t(4096), size_t(50001)})
      for (bool inplace : {false, true}) {
        test_allgather<float>(P, count, inplace, stream);
        test_allgather<unsigned char>(P, count, inplace, stream);
      }
  for (int P : {1, 2, 5, 8})
    for (bool inplace : {false, true}) {
      test_v_variants<float>(P, inplace, stream);
      test_v_variants<double>(P, inplace, stream);
    }
  test_errors(stream);
  test_threads_and_streams();
  test_flags(stream);

  HIPCHK(hipStreamDestroy(stream));
  std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks, g_fail);
  return g_fail ? 1 : 0;
}
