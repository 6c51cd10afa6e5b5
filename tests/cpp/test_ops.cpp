// Command-line parity sweep with the options of the reference's test_ops
// (test/test_ops.cpp:470-495): one collective, one datatype, a range of message
// sizes (powers of two from --min-size to --max-size, plus size+1 with
// --odd-sizes: test/test_utils.hpp:603-617), blocking or non-blocking, in place
// or not.  Where the reference compares with MPI to 1e-4, this compares with
// the CPU oracle bit for bit.  Logical ranks (--ranks) take the place of
// `mpiexec -n`; all of them live on one GPU.
//
// usage: test_ops --op allreduce|reduce|reduce_scatter|allgather|reduce_scatterv|allgatherv
//                 [--backend hip] [--inplace] [--nonblocking] [--reduction-op sum|prod|min|max|lor|land|lxor|bor|band|bxor]
//                 [--algorithm automatic|automatic_mpi_blocking|rank_order|tree_doubling|tree_halving|tree_binomial|
//                  tree_reduce_scatter_gather|tree_reduce_scatter_gather_spread|pairwise|ring|ring_fused]
//                 [--root R] [--size N | --min-size N --max-size N] [--odd-sizes] [--datatype float|...]
//                 [--trials N] [--ranks P] [--threads N]
#include <map>

#include "parity_harness.hpp"

struct Options {
  std::string op, backend = "hip", redop = "sum", algorithm = "automatic", datatype = "float";
  bool inplace = false, nonblocking = false, odd_sizes = false, have_size = false;
  int root = 0, ranks = 4, threads = 0;
  size_t size = 0, min_size = 1, max_size = (size_t)1 << 22, trials = 1;
};

static std::vector<size_t> get_sizes(const Options &o) {
  size_t lo = o.have_size ? o.size : o.min_size, hi = o.have_size ? o.size : o.max_size;
  std::vector<size_t> sizes;
  if (lo == 0) { sizes.push_back(0); lo = 1; }
  for (size_t s = lo; s <= hi; s *= 2) {
    sizes.push_back(s);
    if (o.odd_sizes && s > 1) sizes.push_back(s + 1);
  }
  return sizes;
}

template <typename T> constexpr bool is_float_type() {
  return std::is_same<T, float>::value || std::is_same<T, double>::value || std::is_same<T, Al::amd::half_bits>::value ||
         std::is_same<T, Al::amd::bfloat16_bits>::value;
}

// Inputs that keep every operator meaningful: products stay finite, logical
// operators see zeros and ones, sums of integers wrap like the reference's.
template <typename T> int dist_for(Op op) {
  if (is_float_type<T>()) {
    if (op == Op::prod) return ALO_DIST_UNIFORM_09_11;
    return sizeof(T) == 2 ? ALO_DIST_NORMAL : ALO_DIST_UNIFORM_PM1;
  }
  if (op == Op::lor || op == Op::land || op == Op::lxor) return ALO_DIST_BOOL01;
  return ALO_DIST_FULLRANGE;
}

template <typename T> void sweep(const Options &o, Op rop, Algo algo, int thread) {
  hipStream_t stream;
  HIPCHK(hipStreamCreate(&stream));
  const int P = o.ranks;
  const int dist = dist_for<T>(rop);
  for (size_t trial = 0; trial < o.trials; ++trial)
    for (size_t size : get_sizes(o)) {
      const int before = t_fail;
      if (o.op == "allreduce") test_allreduce<T>(P, size, rop, algo, dist, o.inplace, o.nonblocking, stream);
      else if (o.op == "reduce") test_reduce<T>(P, size, rop, o.root, stream, o.nonblocking ? 1 : 0, o.inplace, dist, algo);
      else if (o.op == "reduce_scatter") test_reduce_scatter<T>(P, size, rop, algo, o.inplace, stream, o.nonblocking, dist);
      else if (o.op == "allgather") test_allgather<T>(P, size, o.inplace, stream, o.nonblocking);
      else if (o.op == "reduce_scatterv")
        test_v_variants<T>(P, o.inplace, stream, o.nonblocking, size, size / 4 + 1, rop, true, false, dist);
      else test_v_variants<T>(P, o.inplace, stream, o.nonblocking, size, size / 4 + 1, rop, false, true, dist);
      std::printf("%s %s %s %s nonblocking=%d inplace=%d root=%d ranks=%d%s size=%zu: %s\n", o.op.c_str(),
                  o.datatype.c_str(), o.redop.c_str(), o.algorithm.c_str(), o.nonblocking, o.inplace, o.root, P,
                  thread < 0 ? "" : (" thread=" + std::to_string(thread)).c_str(), size,
                  t_fail == before ? "ok" : "MISMATCH");
    }
  HIPCHK(hipStreamDestroy(stream));
}

// --threads N: N threads run the sweep at the same time, each with communicators and a stream of
// its own (test/test_ops.cpp:267-273,373-391); without it the calling thread runs it.
template <typename T> int run(const Options &o, Op rop, Algo algo) {
  if (o.threads <= 0) {
    sweep<T>(o, rop, algo, -1);
  } else {
    std::vector<std::thread> th;
    for (int i = 0; i < o.threads; ++i)
      th.emplace_back([&, i] {
        try {
          sweep<T>(o, rop, algo, i);
        } catch (const std::exception &e) {
          std::printf("thread %d: exception: %s\n", i, e.what());
          ++g_fail;
        }
      });
    for (auto &t : th) t.join();
  }
  std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks.load(), g_fail.load());
  std::fflush(stdout);  // before the runtime libraries are torn down
  return g_fail ? 1 : 0;
}

int main(int argc, char **argv) {
  Options o;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    auto next = [&]() -> std::string {
      if (i + 1 >= argc) { std::fprintf(stderr, "missing value for %s\n", a.c_str()); std::exit(2); }
      return argv[++i];
    };
    if (a == "--op") o.op = next();
    else if (a == "--backend") o.backend = next();
    else if (a == "--inplace") o.inplace = true;
    else if (a == "--nonblocking") o.nonblocking = true;
    else if (a == "--reduction-op") o.redop = next();
    else if (a == "--algorithm") o.algorithm = next();
    else if (a == "--root") o.root = std::atoi(next().c_str());
    else if (a == "--size") { o.size = std::strtoull(next().c_str(), nullptr, 10); o.have_size = true; }
    else if (a == "--min-size") o.min_size = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--max-size") o.max_size = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--odd-sizes") o.odd_sizes = true;
    else if (a == "--datatype") o.datatype = next();
    else if (a == "--trials") o.trials = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--ranks") o.ranks = std::atoi(next().c_str());
    else if (a == "--threads") o.threads = std::atoi(next().c_str());
    else if (a == "--help") { std::printf("see the head of tests/cpp/test_ops.cpp\n"); return 0; }
    else { std::fprintf(stderr, "unknown option %s\n", a.c_str()); return 2; }
  }
  static const std::map<std::string, Op> rops = {
      {"sum", Op::sum}, {"prod", Op::prod}, {"min", Op::min}, {"max", Op::max}, {"lor", Op::lor}, {"land", Op::land},
      {"lxor", Op::lxor}, {"bor", Op::bor}, {"band", Op::band}, {"bxor", Op::bxor}, {"avg", Op::avg}};
  static const std::map<std::string, Algo> algos = {
      {"automatic", Algo::automatic}, {"", Algo::automatic}, {"automatic_mpi_blocking", Algo::automatic_mpi_blocking},
      {"rank_order", Algo::rank_order},
      {"tree_doubling", Algo::tree_doubling}, {"tree_halving", Algo::tree_halving},
      {"tree_binomial", Algo::tree_binomial}, {"tree_reduce_scatter_gather", Algo::tree_reduce_scatter_gather},
      {"tree_reduce_scatter_gather_spread", Algo::tree_reduce_scatter_gather_spread}, {"pairwise", Algo::pairwise}, {"ring", Algo::ring},
      {"ring_fused", Algo::ring_fused}};
  static const char *ops[] = {"allreduce", "reduce", "reduce_scatter", "allgather", "reduce_scatterv", "allgatherv"};
  bool op_ok = false;
  for (const char *name : ops) op_ok = op_ok || o.op == name;
  if (!op_ok) { std::fprintf(stderr, "Unsupported or missing --op '%s'\n", o.op.c_str()); return 2; }
  if (o.backend != "hip" && o.backend != "HipCombineBackend") {
    std::fprintf(stderr, "Unsupported backend %s\n", o.backend.c_str());
    return 2;
  }
  if (!rops.count(o.redop)) { std::fprintf(stderr, "Unsupported reduction operator %s\n", o.redop.c_str()); return 2; }
  if (!algos.count(o.algorithm)) { std::fprintf(stderr, "Unsupported algorithm %s\n", o.algorithm.c_str()); return 2; }
  if (o.ranks < 1 || o.ranks > ALAMD_MAX_RANKS || o.root < 0 || o.root >= o.ranks) {
    std::fprintf(stderr, "bad --ranks / --root\n");
    return 2;
  }
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) { std::printf("no GPU\n"); return 2; }
  HIPCHK(hipSetDevice(0));
  const Op rop = rops.at(o.redop);
  const Algo algo = algos.at(o.algorithm);
  try {
    // the datatype names of the reference's dispatcher (test/test_utils.hpp:372-392)
    if (o.datatype == "float") return run<float>(o, rop, algo);
    if (o.datatype == "double") return run<double>(o, rop, algo);
    if (o.datatype == "char") return run<char>(o, rop, algo);
    if (o.datatype == "schar") return run<signed char>(o, rop, algo);
    if (o.datatype == "uchar") return run<unsigned char>(o, rop, algo);
    if (o.datatype == "short") return run<short>(o, rop, algo);
    if (o.datatype == "ushort") return run<unsigned short>(o, rop, algo);
    if (o.datatype == "int") return run<int>(o, rop, algo);
    if (o.datatype == "uint") return run<unsigned int>(o, rop, algo);
    if (o.datatype == "long") return run<long>(o, rop, algo);
    if (o.datatype == "ulong") return run<unsigned long>(o, rop, algo);
    if (o.datatype == "longlong") return run<long long>(o, rop, algo);
    if (o.datatype == "ulonglong") return run<unsigned long long>(o, rop, algo);
    if (o.datatype == "half") return run<Al::amd::half_bits>(o, rop, algo);
    if (o.datatype == "bfloat16") return run<Al::amd::bfloat16_bits>(o, rop, algo);
    std::fprintf(stderr, "Backend %s does not support datatype %s\n", o.backend.c_str(), o.datatype.c_str());
    return 2;
  } catch (const Al::al_exception &e) {
    std::printf("al_exception: %s\n", e.what());
    return 3;
  }
}
