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

// `automatic` against MPICH's own results: tests/golden/mpich_front_end_cases.txt holds, for every
// fixture case whose inputs are the generator's, the checksum of what MPI_Allreduce / MPI_Reduce /
// MPI_Reduce_scatter_block / MPI_Reduce_scatter returned (2 to 16 ranks, every root tried, below and
// above each size at which that library changes algorithm, fp32 / fp64 / fp16 / bf16 and integers).
// The front end, left to choose its order, must return the same bytes.  No oracle in between.
template <typename T>
static void run_mpich_case(std::string coll, int P, Op op, size_t n, int dist, unsigned seed, int root,
                           const std::vector<size_t> &counts, const std::vector<std::string> &want, hipStream_t stream) {
  const int dt = Al::amd::TypeMap<T>::value;
  // "..._blocking": what MPI_Allreduce / MPI_Reduce returned, the others what the non-blocking calls did
  Algo algo = Algo::automatic;
  const size_t tag = coll.find("_blocking");
  if (tag != std::string::npos) { coll = coll.substr(0, tag); algo = Algo::automatic_mpi_blocking; }
  const bool scatter = coll == "reduce_scatter" || coll == "reduce_scatterv";
  size_t in_len = n;
  if (coll == "reduce_scatter") in_len = n * (size_t)P;
  if (coll == "reduce_scatterv") { in_len = 0; for (size_t c : counts) in_len += c; }
  std::vector<std::unique_ptr<DevBuf<T>>> send, recv;
  for (int r = 0; r < P; ++r) {
    send.emplace_back(new DevBuf<T>(in_len));
    recv.emplace_back(new DevBuf<T>(in_len));
    if (dist == 99) {  // planted special values
      send[r]->up(planted<T>(in_len, r));
    } else if (alamd_fill(send[r]->p, in_len, dt, dist, seed + (unsigned)r, 0, stream) != ALAMD_OK) {
      EXPECT(false, "alamd_fill: %s", alamd_last_error());
      return;
    }
  }
  Al::amd::World world(P, stream);
  for (int r = 0; r < P; ++r) {
    auto &comm = world.comm(r);
    const T *src = send[r]->p;
    if (coll == "allreduce") Al::Allreduce<Backend>(src, recv[r]->p, n, op, comm, algo);
    else if (coll == "reduce") Al::Reduce<Backend>(src, recv[r]->p, n, op, root, comm, algo);
    else if (coll == "reduce_scatter") Al::Reduce_scatter<Backend>(src, recv[r]->p, n, op, comm);
    else Al::Reduce_scatterv<Backend>(src, recv[r]->p, counts, op, comm);
  }
  HIPCHK(hipStreamSynchronize(stream));
  for (int r = 0; r < P; ++r) {
    if (!scatter && r != (coll == "reduce" ? root : r)) continue;
    const size_t len = coll == "reduce_scatterv" ? counts[(size_t)r] : n;
    auto got = recv[r]->down();
    char cs[32];
    std::snprintf(cs, sizeof(cs), "%016llx", (unsigned long long)alo_checksum(got.data(), len * sizeof(T)));
    const std::string &w = scatter ? want[(size_t)r] : want[0];
    EXPECT(w == cs, "%s%s against MPICH: P=%d dt=%d op=%d n=%zu root=%d rank %d: %s, MPICH %s", coll.c_str(),
           algo == Algo::automatic ? "" : " (blocking)", P, dt, (int)op, len, root, r, cs, w.c_str());
  }
}

static void test_automatic_against_mpich(hipStream_t stream) {
  char exe[4096];
  const ssize_t len = readlink("/proc/self/exe", exe, sizeof(exe) - 1);
  EXPECT(len > 0, "readlink /proc/self/exe");
  if (len <= 0) return;
  exe[len] = 0;
  std::string path(exe);
  path = path.substr(0, path.rfind('/')) + "/../golden/mpich_front_end_cases.txt";
  std::ifstream f(path);
  EXPECT(f.good(), "cannot open %s", path.c_str());
  static const std::map<std::string, Op> ops = {
      {"sum", Op::sum}, {"prod", Op::prod}, {"min", Op::min}, {"max", Op::max}, {"lor", Op::lor}, {"land", Op::land},
      {"lxor", Op::lxor}, {"bor", Op::bor}, {"band", Op::band}, {"bxor", Op::bxor}};
  int ran = 0, reduces = 0, halves = 0, blocking = 0, specials = 0, many = 0;
  std::string line;
  while (std::getline(f, line)) {
    if (line.empty() || line[0] == '#') continue;
    std::istringstream in(line);
    std::string coll, dtype, opname;
    int P = 0, dist = 0, root = 0;
    unsigned seed = 0;
    size_t n = 0;
    std::vector<size_t> counts;
    in >> coll >> P >> dtype >> opname;
    if (coll != "reduce_scatterv") in >> n;
    in >> dist >> seed;
    if (coll == "reduce" || coll == "reduce_blocking") in >> root;
    if (coll == "reduce_scatterv")
      for (int b = 0; b < P; ++b) { size_t c = 0; in >> c; counts.push_back(c); }
    std::vector<std::string> want;
    for (std::string w; in >> w;) want.push_back(w);
    const bool scatter = coll == "reduce_scatter" || coll == "reduce_scatterv";
    EXPECT(in.eof() && want.size() == (scatter ? (size_t)P : 1u) && ops.count(opname), "malformed line: %s", line.c_str());
    if (want.size() != (scatter ? (size_t)P : 1u) || !ops.count(opname)) continue;
    const Op op = ops.at(opname);
#define RUN(NAME, T) if (dtype == NAME) run_mpich_case<T>(coll, P, op, n, dist, seed, root, counts, want, stream); else
    RUN("i8", signed char) RUN("u8", unsigned char) RUN("i16", short) RUN("u16", unsigned short) RUN("i32", int)
    RUN("u32", unsigned int) RUN("i64", long long) RUN("u64", unsigned long long) RUN("f16", Al::amd::half_bits)
    RUN("bf16", Al::amd::bfloat16_bits) RUN("f32", float) RUN("f64", double)
    EXPECT(false, "unknown dtype in %s", line.c_str());
#undef RUN
    ++ran;
    reduces += coll == "reduce";
    halves += dtype == "f16" || dtype == "bf16";
    blocking += coll.find("_blocking") != std::string::npos;
    specials += dist == 99;
    many += P >= 32;
  }
  EXPECT(ran >= 1000 && reduces >= 250 && halves >= 150 && blocking >= 150 && specials >= 100 && many >= 50,
         "too few cases: %d in all, %d reduces, %d of 16-bit floats, %d of the blocking calls, %d with special values, "
         "%d for 32 ranks and more", ran, reduces, halves, blocking, specials, many);
}

// One rank's thread polls Test on its request while another thread makes the last call, which launches
// the operation, or fails to: the outcome reaches the polling thread through the request alone.
static void test_request_polled_while_launching() {
  const size_t n = 4096;
  for (int round = 0; round < 200; ++round) {
    const bool fail = round % 4 == 3;  // band on floats: the last call finds that the operation cannot be launched
    const Op op = fail ? Op::band : Op::sum;
    hipStream_t s0, s1;
    HIPCHK(hipStreamCreateWithFlags(&s0, hipStreamNonBlocking));
    HIPCHK(hipStreamCreateWithFlags(&s1, hipStreamNonBlocking));
    {
      DevBuf<float> a(n), b(n);
      a.up(gen<float>(n, ALO_DIST_UNIFORM_PM1, 1));
      b.up(gen<float>(n, ALO_DIST_UNIFORM_PM1, 2));
      Al::amd::World world(std::vector<hipStream_t>{s0, s1});
      Backend::req_type r0;
      Al::NonblockingAllreduce<Backend>(a.p, n, op, world.comm(0), r0);
      std::atomic<int> outcome{0};  // 1: completed, 2: threw
      std::thread poller([&] {
        try {
          while (!Al::Test<Backend>(r0)) std::this_thread::yield();
          outcome = 1;
        } catch (const Al::al_exception &) { outcome = 2; }
      });
      Backend::req_type r1;
      bool threw = false;
      try {
        Al::NonblockingAllreduce<Backend>(b.p, n, op, world.comm(1), r1);
      } catch (const Al::al_exception &) { threw = true; }
      poller.join();
      EXPECT(threw == fail, "round %d: the last call %s", round, fail ? "should have thrown" : "threw");
      EXPECT(outcome == (fail ? 2 : 1), "round %d: the polling rank saw outcome %d", round, outcome.load());
      EXPECT(r0 == Backend::null_req, "round %d: request not reset", round);
      if (!fail) Al::Wait<Backend>(r1);
      HIPCHK(hipStreamSynchronize(s0));
      HIPCHK(hipStreamSynchronize(s1));
    }
    HIPCHK(hipStreamDestroy(s0));
    HIPCHK(hipStreamDestroy(s1));
  }
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


// ---- one-sided extension and halo faces ----------------------------------------

struct HaloGrid {
  size_t dims[3], h, side[3], cells;
  std::vector<double> host;
  std::unique_ptr<DevBuf<double>> dev;
  HaloGrid(size_t nx, size_t ny, size_t nz, size_t halo, unsigned seed) : h(halo) {
    dims[0] = nx; dims[1] = ny; dims[2] = nz;
    for (int d = 0; d < 3; ++d) side[d] = dims[d] + 2 * h;
    cells = side[0] * side[1] * side[2];
    host = gen<double>(cells, ALO_DIST_UNIFORM_01, seed);
    dev.reset(new DevBuf<double>(cells));
    dev->up(host);
  }
  size_t face_elems(int f) const { return alo_halo_face_elems(dims[0], dims[1], dims[2], h, f); }
};

// pack -> ext::Put to the rank itself -> unpack, against the oracle's index maps
static void test_halo_loopback(hipStream_t stream) {
  HaloGrid g(37, 20, 9, 2, 4000u);
  Al::amd::World world(1, stream);
  auto &comm = world.comm(0);
  std::vector<std::unique_ptr<DevBuf<double>>> send, recv;
  double *sp[6], *rp[6];
  for (int f = 0; f < 6; ++f) {
    EXPECT(Al::amd::halo_face_elems(g.dims, g.h, f) == g.face_elems(f), "face %d size", f);
    send.emplace_back(new DevBuf<double>(g.face_elems(f)));
    recv.emplace_back(new DevBuf<double>(g.face_elems(f)));
    sp[f] = send[f]->p;
    // the address at which the peer's (here: the rank's own) receive buffer is reachable
    rp[f] = Al::ext::AttachRemoteBuffer<Backend>(recv[f]->p, 0, comm);
    EXPECT(rp[f] == recv[f]->p, "a rank reaches its own buffer at its own address");
  }
  Al::amd::halo_pack<double>(sp, g.dev->p, g.dims, g.h, 0x3f, comm);
  for (int f = 0; f < 6; ++f) Al::ext::Put<Backend>(static_cast<const double *>(sp[f]), 0, rp[f], g.face_elems(f), comm);
  Al::ext::Sync<Backend>(0, comm);
  const double *crp[6];
  for (int f = 0; f < 6; ++f) crp[f] = rp[f];
  Al::amd::halo_unpack<double>(g.dev->p, crp, g.dims, g.h, 0x3f, comm);
  HIPCHK(hipStreamSynchronize(stream));
  std::vector<double> want = g.host;
  for (int f = 0; f < 6; ++f) {
    std::vector<double> face(g.face_elems(f));
    alo_halo_pack(face.data(), g.host.data(), g.dims[0], g.dims[1], g.dims[2], g.h, f, sizeof(double));
    EXPECT(same_bits(send[f]->down(), face), "packed face %d", f);
    alo_halo_unpack(want.data(), face.data(), g.dims[0], g.dims[1], g.dims[2], g.h, f, sizeof(double));
  }
  EXPECT(same_bits(g.dev->down(), want), "grid after the loop-back halo exchange");
  for (int f = 0; f < 6; ++f) Al::ext::DetachRemoteBuffer<Backend>(rp[f], 0, comm);
  bool threw = false;
  try { Al::ext::Put<Backend>(static_cast<const double *>(nullptr), 0, rp[0], 4, comm); } catch (const Al::al_exception &e) {
    threw = std::string(e.what()).find("Source buffer is null") != std::string::npos;
  }
  EXPECT(threw, "Put from a null buffer must throw");
  threw = false;
  try { Al::ext::Notify<Backend>(3, comm); } catch (const Al::al_exception &) { threw = true; }
  EXPECT(threw, "a peer outside the communicator must throw");
}

// Two logical ranks on two streams exchange their x faces (rank 0's +x neighbour is rank 1 and the
// other way round), with Put / Notify / Wait; wait_first: the receivers ask before the senders notify.
static void test_halo_two_ranks(bool wait_first) {
  hipStream_t s[2];
  for (auto &x : s) HIPCHK(hipStreamCreateWithFlags(&x, hipStreamNonBlocking));
  {
    Al::amd::World world(std::vector<hipStream_t>{s[0], s[1]});
    HaloGrid g0(16, 11, 13, 3, 4100u), g1(16, 11, 13, 3, 4200u);
    HaloGrid *g[2] = {&g0, &g1};
    const int out_face[2] = {1, 0};  // rank 0 sends its +x face, rank 1 its -x face
    const int in_face[2] = {1, 0};   // ... and receives into the ghost slab of the same side
    const size_t n = g0.face_elems(0);
    DevBuf<double> send0(n), send1(n), recv0(n), recv1(n);
    double *send[2] = {send0.p, send1.p}, *recv[2] = {recv0.p, recv1.p};
    Al::amd::GPUWait gate;
    gate.wait(s[1], 1u << 24);  // rank 1's stream is late: nothing of its exchange has run when rank 0 asks
    if (wait_first)
      for (int r = 0; r < 2; ++r) Al::ext::Wait<Backend>(1 - r, world.comm(r));
    for (int r = 0; r < 2; ++r) {
      double *bufs[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
      bufs[out_face[r]] = send[r];
      Al::amd::halo_pack<double>(bufs, g[r]->dev->p, g[r]->dims, g[r]->h, 1u << out_face[r], world.comm(r));
      // all ranks share one address space: the peer's receive buffer is used as it is
      Al::ext::Put<Backend>(static_cast<const double *>(send[r]), 1 - r, recv[1 - r], n, world.comm(r));
      Al::ext::Notify<Backend>(1 - r, world.comm(r));
    }
    for (int r = 0; r < 2; ++r) {
      if (!wait_first) Al::ext::Wait<Backend>(1 - r, world.comm(r));
      const double *bufs[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
      bufs[in_face[r]] = recv[r];
      Al::amd::halo_unpack<double>(g[r]->dev->p, bufs, g[r]->dims, g[r]->h, 1u << in_face[r], world.comm(r));
    }
    gate.signal();
    for (auto &x : s) HIPCHK(hipStreamSynchronize(x));
    EXPECT(!gate.timed_out(), "gate must not have expired");
    for (int r = 0; r < 2; ++r) {
      std::vector<double> face(n), want = g[r]->host;
      alo_halo_pack(face.data(), g[1 - r]->host.data(), g0.dims[0], g0.dims[1], g0.dims[2], g0.h, out_face[1 - r], sizeof(double));
      alo_halo_unpack(want.data(), face.data(), g0.dims[0], g0.dims[1], g0.dims[2], g0.h, in_face[r], sizeof(double));
      EXPECT(same_bits(g[r]->dev->down(), want), "rank %d ghost cells after the exchange (%s)", r,
             wait_first ? "wait before notify" : "notify before wait");
    }
  }
  for (auto &x : s) HIPCHK(hipStreamDestroy(x));
}

// A token goes round the ring of logical ranks and back, one thread and one stream per rank, with
// AttachRemoteBuffer / Put / Notify / Wait as the reference's ring test drives them
// (test/test_rma_ring.cpp:38-108): rank 0 starts, every other rank waits for its left neighbour,
// puts to its right one and notifies it; then the same from the last rank leftwards.  Stricter than
// there: every buffer starts from a sentinel, so a rank holds the token only if the puts brought it.
struct ThreadBarrier {
  std::mutex m;
  std::condition_variable cv;
  int n, waiting = 0;
  unsigned long generation = 0;
  explicit ThreadBarrier(int n_) : n(n_) {}
  void arrive_and_wait() {
    std::unique_lock<std::mutex> lock(m);
    const unsigned long g = generation;
    if (++waiting == n) {
      waiting = 0;
      ++generation;
      cv.notify_all();
    } else {
      cv.wait(lock, [&] { return generation != g; });
    }
  }
};

static void test_rma_token_ring(int P) {
  std::vector<hipStream_t> streams(static_cast<size_t>(P));
  for (auto &s : streams) HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  {
    Al::amd::World world(streams);
    world.set_calls_wait_for_launch(true);
    std::vector<size_t> sizes = {0};
    for (size_t n = 1; n <= (size_t(1) << 18); n *= 4) {
      sizes.push_back(n);
      if (n > 1) sizes.push_back(n + 1);
    }
    ThreadBarrier barrier(P);
    std::vector<std::unique_ptr<DevBuf<float>>> buf(static_cast<size_t>(P));
    std::vector<std::thread> th;
    for (int rank = 0; rank < P; ++rank)
      th.emplace_back([&, rank] {
        auto &comm = world.comm(rank);
        const hipStream_t stream = streams[static_cast<size_t>(rank)];
        const int rhs = (rank + 1) % P, lhs = (rank - 1 + P) % P;
        for (size_t n : sizes) {
          const std::vector<float> token = gen<float>(n, ALO_DIST_UNIFORM_PM1, 7000u + static_cast<unsigned>(n));
          buf[static_cast<size_t>(rank)].reset(new DevBuf<float>(n));
          float *mine = buf[static_cast<size_t>(rank)]->p;
          float *rhs_buf, *lhs_buf;
          if (rank % 2) {
            rhs_buf = Al::ext::AttachRemoteBuffer<Backend>(mine, rhs, comm);
            lhs_buf = Al::ext::AttachRemoteBuffer<Backend>(mine, lhs, comm);
          } else {
            lhs_buf = Al::ext::AttachRemoteBuffer<Backend>(mine, lhs, comm);
            rhs_buf = Al::ext::AttachRemoteBuffer<Backend>(mine, rhs, comm);
          }
          barrier.arrive_and_wait();
          if (rank == 0) {
            EXPECT(lhs_buf == buf[static_cast<size_t>(lhs)]->p && rhs_buf == buf[static_cast<size_t>(rhs)]->p,
                   "rank 0 reaches its neighbours' buffers (%d ranks, %zu elements)", P, n);
          }
          for (int pass = 0; pass < 2; ++pass) {
            const int first = pass == 0 ? 0 : P - 1, to = pass == 0 ? rhs : lhs, from = pass == 0 ? lhs : rhs;
            float *to_buf = pass == 0 ? rhs_buf : lhs_buf;
            if (n) HIPCHK(hipMemsetAsync(mine, 0xff, n * sizeof(float), stream));
            HIPCHK(hipStreamSynchronize(stream));
            barrier.arrive_and_wait();  // every sentinel is in place before the first put
            if (rank != first)
              Al::ext::Wait<Backend>(from, comm);
            else if (n)
              HIPCHK(hipMemcpyAsync(mine, token.data(), n * sizeof(float), hipMemcpyHostToDevice, stream));
            Al::ext::Put<Backend>(static_cast<const float *>(mine), to, to_buf, n, comm);
            Al::ext::Notify<Backend>(to, comm);
            if (rank == first) Al::ext::Wait<Backend>(from, comm);
            HIPCHK(hipStreamSynchronize(stream));
            barrier.arrive_and_wait();
            if (rank == 0)  // one thread checks, the others stand at the next barrier
              for (int r = 0; r < P; ++r)
                EXPECT(same_bits(buf[static_cast<size_t>(r)]->down(), token),
                       "token at rank %d after the pass %s (%d ranks, %zu elements)", r,
                       pass == 0 ? "rightwards" : "leftwards", P, n);
            barrier.arrive_and_wait();
          }
          Al::ext::DetachRemoteBuffer<Backend>(rhs_buf, rhs, comm);
          Al::ext::DetachRemoteBuffer<Backend>(lhs_buf, lhs, comm);
          barrier.arrive_and_wait();  // nobody frees a buffer a neighbour still reads
        }
      });
    for (auto &t : th) t.join();
  }
  for (auto &s : streams) HIPCHK(hipStreamDestroy(s));
}

// Every rank on its own stream, each stream held back by a gate the host opens late and in
// reverse order: the collective must wait for what every stream held at its rank's call, and the
// copies enqueued after the last call must see the result.
static void test_stream_order(bool threaded) {
  const int P = 4;
  const size_t n = 30000;
  std::vector<hipStream_t> streams(P);
  for (auto &s : streams) HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  {
    Al::amd::World world(streams);
    world.set_calls_wait_for_launch(threaded);
    std::vector<std::vector<float>> in;
    std::vector<std::unique_ptr<DevBuf<float>>> buf;
    std::vector<float *> pinned_in(P), pinned_out(P);
    std::vector<std::unique_ptr<Al::amd::GPUWait>> gates;
    for (int r = 0; r < P; ++r) {
      in.push_back(gen<float>(n, ALO_DIST_UNIFORM_PM1, 90u + (unsigned)r));
      buf.emplace_back(new DevBuf<float>(n));
      HIPCHK(hipMemset(buf[r]->p, 0, n * sizeof(float)));
      HIPCHK(hipHostMalloc(reinterpret_cast<void **>(&pinned_in[r]), n * sizeof(float), hipHostMallocDefault));
      HIPCHK(hipHostMalloc(reinterpret_cast<void **>(&pinned_out[r]), n * sizeof(float), hipHostMallocDefault));
      std::memcpy(pinned_in[r], in[r].data(), n * sizeof(float));
      std::memset(pinned_out[r], 0, n * sizeof(float));
      gates.emplace_back(new Al::amd::GPUWait);
    }
    auto rank_work = [&](int r) {
      gates[r]->wait(streams[r], 1u << 24);
      HIPCHK(hipMemcpyAsync(buf[r]->p, pinned_in[r], n * sizeof(float), hipMemcpyHostToDevice, streams[r]));  // producer
      Al::Allreduce<Backend>(buf[r]->p, n, Op::sum, world.comm(r), Algo::rank_order);
    };
    auto consumer = [&](int r) {
      HIPCHK(hipMemcpyAsync(pinned_out[r], buf[r]->p, n * sizeof(float), hipMemcpyDeviceToHost, streams[r]));
    };
    if (threaded) {
      // each thread enqueues its consumer as soon as its call returns
      std::vector<std::thread> th;
      for (int r = 0; r < P; ++r) th.emplace_back([&, r] { rank_work(r); consumer(r); });
      for (auto &t : th) t.join();
    } else {
      for (int r = 0; r < P; ++r) rank_work(r);
      for (int r = 0; r < P; ++r) consumer(r);  // after the last call
    }
    for (int r = P - 1; r >= 0; --r) {
      std::this_thread::sleep_for(std::chrono::milliseconds(3));
      gates[r]->signal();
    }
    for (auto &s : streams) HIPCHK(hipStreamSynchronize(s));
    std::vector<float> want(n);
    std::vector<const void *> ptrs;
    for (auto &b : in) ptrs.push_back(b.data());
    alo_combine(want.data(), ptrs.data(), P, n, ALO_F32, ALO_SUM, ALO_ORDER_RANK_ASC, 0);
    for (int r = 0; r < P; ++r) {
      EXPECT(!gates[r]->timed_out(), "gate %d must not have expired", r);
      EXPECT(std::memcmp(pinned_out[r], want.data(), n * sizeof(float)) == 0, "%s: rank %d's consumer saw the result",
             threaded ? "threads" : "one thread", r);
      HIPCHK(hipHostFree(pinned_in[r]));
      HIPCHK(hipHostFree(pinned_out[r]));
    }
  }
  for (auto &s : streams) HIPCHK(hipStreamDestroy(s));
}

// Every rank on one stream, a non-blocking operation large enough for the internal stream, each rank's
// producer enqueued just before its call: the operation has to wait for the last producer, not the first.
static void test_stream_order_shared_stream() {
  const int P = 3;
  const size_t n = (48u << 20) / sizeof(float);  // 2 * P * n * 4 bytes moved: beyond what runs on the caller's stream
  hipStream_t s;
  HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  {
    Al::amd::World world(P, s);
    std::vector<std::vector<float>> in;
    std::vector<std::unique_ptr<DevBuf<float>>> buf;
    std::vector<float *> pinned_in(P);
    float *pinned_out = nullptr;
    HIPCHK(hipHostMalloc(reinterpret_cast<void **>(&pinned_out), n * sizeof(float), hipHostMallocDefault));
    for (int r = 0; r < P; ++r) {
      in.push_back(gen<float>(n, ALO_DIST_UNIFORM_PM1, 190u + (unsigned)r));
      buf.emplace_back(new DevBuf<float>(n));
      HIPCHK(hipMemset(buf[r]->p, 0, n * sizeof(float)));
      HIPCHK(hipHostMalloc(reinterpret_cast<void **>(&pinned_in[r]), n * sizeof(float), hipHostMallocDefault));
      std::memcpy(pinned_in[r], in[r].data(), n * sizeof(float));
    }
    Al::amd::GPUWait gate;
    gate.wait(s, 1u << 24);
    std::vector<Backend::req_type> reqs(P);
    for (int r = 0; r < P; ++r) {
      HIPCHK(hipMemcpyAsync(buf[r]->p, pinned_in[r], n * sizeof(float), hipMemcpyHostToDevice, s));  // producer
      Al::NonblockingAllreduce<Backend>(buf[r]->p, n, Op::sum, world.comm(r), reqs[r], Algo::rank_order);
    }
    std::this_thread::sleep_for(std::chrono::milliseconds(3));
    gate.signal();
    for (int r = 0; r < P; ++r) Al::Wait<Backend>(reqs[r]);
    HIPCHK(hipMemcpyAsync(pinned_out, buf[P - 1]->p, n * sizeof(float), hipMemcpyDeviceToHost, s));
    HIPCHK(hipStreamSynchronize(s));
    std::vector<float> want(n);
    std::vector<const void *> ptrs;
    for (auto &b : in) ptrs.push_back(b.data());
    alo_combine(want.data(), ptrs.data(), P, n, ALO_F32, ALO_SUM, ALO_ORDER_RANK_ASC, 0);
    EXPECT(!gate.timed_out(), "the gate must not have expired");
    EXPECT(std::memcmp(pinned_out, want.data(), n * sizeof(float)) == 0,
           "one stream for every rank: the operation waited for the last rank's producer");
    for (int r = 0; r < P; ++r) HIPCHK(hipHostFree(pinned_in[r]));
    HIPCHK(hipHostFree(pinned_out));
  }
  HIPCHK(hipStreamDestroy(s));
}

// A call that throws leaves its communicator where it was; a launch that fails is reported to the
// ranks that have already returned.
static void test_error_recovery(hipStream_t stream) {
  const size_t n = 64;
  DevBuf<float> a(n), b(n);
  const auto ha = gen<float>(n, ALO_DIST_UNIFORM_PM1, 7u), hb = gen<float>(n, ALO_DIST_UNIFORM_PM1, 8u);
  a.up(ha);
  b.up(hb);
  Al::amd::World world(2, stream);
  Al::Allreduce<Backend>(a.p, n, Op::sum, world.comm(0), Algo::rank_order);
  bool threw = false;
  try { Al::Allreduce<Backend>(b.p, n / 2, Op::sum, world.comm(1), Algo::rank_order); } catch (const Al::al_exception &) { threw = true; }
  EXPECT(threw, "mismatched count must throw");
  Al::Allreduce<Backend>(b.p, n, Op::sum, world.comm(1), Algo::rank_order);  // the same rank, now as agreed
  HIPCHK(hipStreamSynchronize(stream));
  std::vector<float> want(n);
  const void *ptrs[2] = {ha.data(), hb.data()};
  alo_combine(want.data(), ptrs, 2, n, ALO_F32, ALO_SUM, ALO_ORDER_RANK_ASC, 0);
  EXPECT(same_bits(a.down(), want) && same_bits(b.down(), want), "the collective completed after the failed call");
  // a launch that fails: rank 1's receive buffer overlaps rank 0's send buffer partially
  DevBuf<float> big(3 * n);
  Backend::req_type r0, r1;
  Al::NonblockingAllreduce<Backend>(static_cast<const float *>(big.p), big.p + 2 * n, n, Op::sum, world.comm(0), r0, Algo::rank_order);
  threw = false;
  try {
    Al::NonblockingAllreduce<Backend>(static_cast<const float *>(big.p + n), big.p + n / 2, n, Op::sum, world.comm(1), r1, Algo::rank_order);
  } catch (const Al::al_exception &) { threw = true; }
  EXPECT(threw, "overlapping buffers must throw from the call that launches");
  threw = false;
  try { (void)Al::Test<Backend>(r0); } catch (const Al::al_exception &e) {
    threw = std::string(e.what()).find("could not be launched") != std::string::npos;
  }
  EXPECT(threw, "the rank that had already returned learns of the failure from its request");
  EXPECT(r0 == Backend::null_req, "a failed request is released");
  // and the world goes on
  Al::Allreduce<Backend>(a.p, n, Op::max, world.comm(0), Algo::rank_order);
  Al::Allreduce<Backend>(b.p, n, Op::max, world.comm(1), Algo::rank_order);
  HIPCHK(hipStreamSynchronize(stream));
  EXPECT(same_bits(a.down(), want), "max of equal values after the failed launch");
}

// The early-signal policies: the stream goes on as soon as the host step has started, the step
// itself completes later (ht/base_state.hpp:124-209).
static void test_progress_engine_early_signal(hipStream_t stream) {
  using PE = Al::amd::ProgressEngine;
  EXPECT(PE::root_early(true) == PE::SignalWhen::after_start && PE::root_early(false) == PE::SignalWhen::at_end &&
             PE::non_root_early(false) == PE::SignalWhen::after_start && PE::non_root_early(true) == PE::SignalWhen::at_end,
         "who is let go early under the two rooted policies");
  DevBuf<int> x(1);
  HIPCHK(hipMemsetAsync(x.p, 0, sizeof(int), stream));
  std::atomic<bool> release{false};
  std::atomic<int> polls{0};
  PE pe;
  pe.enqueue(stream, [] {}, [&] { ++polls; return release.load(); }, PE::SignalWhen::after_start);
  HIPCHK(hipMemsetAsync(x.p, 1, sizeof(int), stream));
  HIPCHK(hipStreamSynchronize(stream));  // returns although the step has not completed
  EXPECT(x.down()[0] == 0x01010101, "the stream went on after the step had started");
  EXPECT(pe.pending() == 1, "the step itself is still in progress");
  // an at-end step behind it on the same engine makes progress while the first one is polled
  int ran = 0;
  pe.enqueue(stream, [&] { ran = 1; });
  HIPCHK(hipStreamSynchronize(stream));
  EXPECT(ran == 1, "a later step ran while the early-signalled one was still polling");
  release = true;
  for (int spin = 0; spin < 2000 && pe.pending(); ++spin) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  EXPECT(pe.pending() == 0 && polls.load() > 1, "the step was polled to its end and retired");
}

// A host step that throws must not leave its stream blocked.
static void test_progress_engine_exception(hipStream_t stream) {
  DevBuf<int> x(1);
  HIPCHK(hipMemsetAsync(x.p, 0, sizeof(int), stream));
  Al::amd::ProgressEngine pe;
  pe.enqueue(stream, [] { throw std::runtime_error("host step failed"); });
  HIPCHK(hipMemsetAsync(x.p, 1, sizeof(int), stream));
  HIPCHK(hipStreamSynchronize(stream));  // returns: the step's wait was signalled all the same
  EXPECT(x.down()[0] == 0x01010101, "work behind the failed host step ran");
  for (int spin = 0; spin < 2000 && pe.pending(); ++spin) std::this_thread::sleep_for(std::chrono::milliseconds(1));
  EXPECT(pe.pending() == 0, "the failed step was retired");
  bool threw = false;
  try { pe.check(); } catch (const std::runtime_error &e) { threw = std::string(e.what()) == "host step failed"; }
  EXPECT(threw, "check() rethrows what the host step threw");
  pe.check();  // once only
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
  for (int P : {3, 5, 8})
    for (size_t n : {size_t(7), size_t(600), size_t(70001)})
      for (int root : {0, 1, P - 1}) {
        test_reduce<double>(P, n, Op::prod, root, stream, -1, false, ALO_DIST_UNIFORM_09_11);
        test_reduce<Al::amd::bfloat16_bits>(P, n, Op::sum, root, stream, -1, true, ALO_DIST_NORMAL);
        test_reduce<float>(P, n, Op::max, root, stream, -1, false, ALO_DIST_UNIFORM_PM1, Algo::tree_binomial);
        test_reduce<float>(P, n, Op::sum, root, stream, -1, false, ALO_DIST_UNIFORM_PM1, Algo::tree_reduce_scatter_gather);
      }
  test_automatic_against_mpich(stream);
  test_errors(stream);
  test_error_recovery(stream);
  test_threads_and_streams();
  test_request_polled_while_launching();
  test_stream_order(false);
  test_stream_order(true);
  test_stream_order_shared_stream();
  test_halo_loopback(stream);
  test_halo_two_ranks(false);
  test_halo_two_ranks(true);
  for (int P : {1, 2, 3, 5, 8}) test_rma_token_ring(P);
  test_progress_engine_early_signal(stream);
  test_progress_engine_exception(stream);
  test_flags(stream);
  test_progress_engine(stream);

  HIPCHK(hipStreamDestroy(stream));
  Al::Finalize();
  EXPECT(!Al::Initialized(), "not initialised after Finalize");
  std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks.load(), g_fail.load());
  std::fflush(stdout);  // before the runtime libraries are torn down
  return g_fail ? 1 : 0;
}
