// Parity test of the Aluminum-shaped C++ front end (include/aluminum_amd/Al.hpp)
// against the CPU oracle, in the manner of the reference's test_ops
// (test/test_ops.cpp:200-225, test/op_runner.hpp:312-324): per-rank seeded
// inputs, the collective through the backend, the same collective on the host,
// then an element-wise comparison - bit-exact here.
//
// Runs on one GPU; every logical rank of the World lives in its memory.
#include "parity_harness.hpp"

// compile-time traits of the backend
static_assert(Al::IsOpSupported<Al::AlOperation::allreduce, Backend>::value, "allreduce");
static_assert(Al::IsOpSupported<Al::AlOperation::reduce_scatterv, Backend>::value, "reduce_scatterv");
static_assert(!Al::IsOpSupported<Al::AlOperation::alltoall, Backend>::value, "alltoall is not on the path");
static_assert(Al::IsTypeSupported<Backend, float>::value && Al::IsTypeSupported<Backend, unsigned long long>::value &&
                  Al::IsTypeSupported<Backend, Al::amd::bfloat16_bits>::value, "types");
static_assert(!Al::IsTypeSupported<Backend, long double>::value, "long double has no device type");
static_assert(Al::IsReductionOpSupported<Backend, Op::bxor>::value && Al::IsReductionOpSupported<Backend, Op::avg>::value,
              "operators");
static_assert(std::is_same<Al::OpAlgoType<Al::AlOperation::allgather, Backend>::type, Algo>::value, "algo type");

static void test_errors(hipStream_t stream) {
  DevBuf<float> a(64), b(64);
  Al::amd::World world(2, stream);
  bool threw = false;
  try {
    Al::Allreduce<Backend>(a.p, 64, Op::band, world.comm(0));
    Al::Allreduce<Backend>(b.p, 64, Op::band, world.comm(1));
  } catch (const Al::al_exception &e) {
    threw = std::string(e.what()).find("Reduction operator not supported") != std::string::npos;
  }
  EXPECT(threw, "band on float must throw 'Reduction operator not supported'");
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
  EXPECT(std::string(Al::AlBackendName<Backend>) == "hip", "backend short name");
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

// The host-transfer shape end to end: device -> pinned host copy, a host step in stream order,
// pinned host -> device copy; all enqueued before anything has run.
static void test_progress_engine(hipStream_t stream) {
  const size_t n = 1000;
  DevBuf<int> x(n);
  std::vector<int> init(n);
  for (size_t i = 0; i < n; ++i) init[i] = (int)i;
  x.up(init);
  int *pinned = nullptr;
  HIPCHK(hipHostMalloc(reinterpret_cast<void **>(&pinned), n * sizeof(int), hipHostMallocDefault));
  std::memset(pinned, 0, n * sizeof(int));
  int order_seen[2] = {0, 0}, step = 0;
  {
    Al::amd::ProgressEngine pe;
    Al::amd::GPUWait gate;
    gate.wait(stream, 1u << 24);  // nothing below may run before the host opens the gate
    HIPCHK(hipMemcpyAsync(pinned, x.p, n * sizeof(int), hipMemcpyDeviceToHost, stream));
    pe.enqueue(stream, [&] {
      order_seen[0] = ++step;
      for (size_t i = 0; i < n; ++i) pinned[i] = 2 * pinned[i] + 1;  // sees what the copy before it brought
    });
    HIPCHK(hipMemcpyAsync(x.p, pinned, n * sizeof(int), hipMemcpyHostToDevice, stream));
    pe.enqueue(stream, [&] { order_seen[1] = ++step; });
    EXPECT(pe.pending() == 2, "two host steps pending");
    EXPECT(step == 0, "no host step before the stream got there");
    gate.signal();
    HIPCHK(hipStreamSynchronize(stream));
    EXPECT(order_seen[0] == 1 && order_seen[1] == 2, "host steps ran once each, in stream order");
    for (int spin = 0; spin < 2000 && pe.pending(); ++spin) std::this_thread::sleep_for(std::chrono::milliseconds(1));
    EXPECT(pe.pending() == 0, "states retired after their end flags");
  }
  const auto got = x.down();
  bool ok = true;
  for (size_t i = 0; i < n; ++i) ok = ok && got[i] == 2 * (int)i + 1;
  EXPECT(ok, "device data went through the host step");
  HIPCHK(hipHostFree(pinned));
}

int main() {
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { std::printf("no GPU\n"); return 2; }
  HIPCHK(hipSetDevice(0));
  int argc = 0;
  char **argv = nullptr;
  EXPECT(!Al::Initialized(), "not initialised before Initialize");
  Al::Initialize(argc, argv);
  EXPECT(Al::Initialized(), "initialised after Initialize");
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
  test_progress_engine(stream);

  HIPCHK(hipStreamDestroy(stream));
  Al::Finalize();
  EXPECT(!Al::Initialized(), "not initialised after Finalize");
  std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks, g_fail);
  return g_fail ? 1 : 0;
}
