// Size sweep of one collective through the Aluminum-shaped front end, with the
// method and the output rows of the reference's benchmark_ops
// (benchmark/benchmark_ops.cpp:143-195: warm-up then timed trials per size;
// benchmark/benchmark_utils_ht.hpp:34-62: GPU events on the communicator's
// stream; benchmark/benchmark_utils.hpp:151-184: one row per trial and rank,
// "Backend Type Operation Algo NonBlocking InPlace Root CommSize Size CommRank Time",
// time in seconds).  All logical ranks share one GPU and one launch, so every
// rank of a trial reports the same time.
//
// usage: bench_ops [--op allreduce|reduce|reduce_scatter|allgather|reduce_scatterv|allgatherv] [--datatype float|double|int|...]
//                  [--reduction-op sum|prod|min|max|...] [--algorithm automatic|rank_order|tree_doubling|
//                  tree_halving|tree_binomial|tree_reduce_scatter_gather|pairwise|ring|ring_fused] [--ranks P] [--root R]
//                  [--inplace] [--nonblocking] [--min-size N] [--max-size N] [--size N] [--num-iters N]
//                  [--num-warmup N] [--summarize] [--save-to-file FILE] [--no-print-table] [--backend hip]
//                  [--stream-per-rank] [--tune name=value ...]
// (--summarize: per size "Size Mean Median Stdev Min Max" over the timed trials, benchmark_ops.cpp:211-224;
// --save-to-file / --no-print-table: where the table of rows goes, :225-230.)
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "aluminum_amd/Al.hpp"
#include "aluminum_amd_support.h"

using Backend = Al::HipCombineBackend;
using Algo = Al::amd::CombineAlgorithm;
#define HIPCHK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); std::exit(2); } } while (0)

struct Options {
  std::string op = "allreduce", datatype = "float", redop = "sum", algo = "automatic";
  int ranks = 8, root = 0;
  bool inplace = false, nonblocking = false;
  size_t min_size = 1, max_size = (size_t)1 << 22, iters = 100, warmup = 10;
  bool summarize = false, print_table = true, stream_per_rank = false;
  std::string save_to;
};

// The rows of one run: trial times in seconds by message size.
struct Results {
  std::string prefix;  // "Backend Type Operation Algo NonBlocking InPlace Root CommSize "
  int ranks = 0;
  std::map<size_t, std::vector<double>> times;
  void write(std::FILE *f) const {
    std::fprintf(f, "Backend Type Operation Algo NonBlocking InPlace Root CommSize Size CommRank Time\n");
    for (const auto &kv : times)
      for (int r = 0; r < ranks; ++r)
        for (double t : kv.second) std::fprintf(f, "%s%zu %d %.9g\n", prefix.c_str(), kv.first, r, t);
  }
  void summary(std::FILE *f) const {
    std::fprintf(f, "Size\t\tMean\t\tMedian\t\tStdev\t\tMin\t\tMax\n");
    for (const auto &kv : times) {
      std::vector<double> v = kv.second;
      if (v.empty()) continue;
      std::sort(v.begin(), v.end());
      double mean = 0, sq = 0;
      for (double t : v) mean += t;
      mean /= (double)v.size();
      for (double t : v) sq += (t - mean) * (t - mean);
      const double stdev = v.size() > 1 ? std::sqrt(sq / (double)(v.size() - 1)) : 0.0;
      std::fprintf(f, "%zu\t\t%.9g\t%.9g\t%.9g\t%.9g\t%.9g\n", kv.first, mean, v[v.size() / 2], stdev, v.front(),
                   v.back());
    }
  }
};

template <typename T> int run(const Options &o, Al::ReductionOperator rop, Algo algo, const char *tname) {
  hipStream_t stream;
  HIPCHK(hipStreamCreate(&stream));
  hipEvent_t e0, e1;
  HIPCHK(hipEventCreate(&e0));
  HIPCHK(hipEventCreate(&e1));
  const int P = o.ranks;
  const int dt = Al::amd::TypeMap<T>::value;
  Results res;
  res.ranks = P;
  res.prefix = Backend::Name() + " " + tname + " " + o.op + " " + o.algo + " " + (o.nonblocking ? "1" : "0") + " " +
               (o.inplace ? "1" : "0") + " " + std::to_string(o.root) + " " + std::to_string(P) + " ";
  for (size_t size = o.min_size; size <= o.max_size; size *= 2) {
    const size_t in_elems = o.op == "reduce_scatter" || o.op == "reduce_scatterv" ? size * (size_t)P : size;
    const size_t out_elems = o.op == "allgather" || o.op == "allgatherv" ? size * (size_t)P : size;
    const size_t buf_elems = in_elems > out_elems ? in_elems : out_elems;
    std::vector<T *> in(P), out(P);
    for (int r = 0; r < P; ++r) {
      HIPCHK(hipMalloc(reinterpret_cast<void **>(&in[r]), buf_elems * sizeof(T)));
      HIPCHK(hipMalloc(reinterpret_cast<void **>(&out[r]), buf_elems * sizeof(T)));
      if (alamd_fill(in[r], buf_elems, dt, ALAMD_DIST_SMALLINT, 1u + (unsigned)r, 0, stream) != ALAMD_OK) {
        std::fprintf(stderr, "%s\n", alamd_last_error());
        return 2;
      }
    }
    // every logical rank on one stream, or each on its own (the time is still taken on rank 0's, where
    // a blocking operation runs; the others are made to wait for it)
    std::vector<hipStream_t> streams((size_t)P, stream);
    if (o.stream_per_rank)
      for (int r = 1; r < P; ++r) HIPCHK(hipStreamCreateWithFlags(&streams[(size_t)r], hipStreamNonBlocking));
    std::vector<double> times;
    {
    Al::amd::World world(streams);
    for (size_t trial = 0; trial < o.warmup + o.iters; ++trial) {
      std::vector<Backend::req_type> reqs(P);
      HIPCHK(hipStreamSynchronize(stream));  // stands in for the barrier before each trial
      HIPCHK(hipEventRecord(e0, stream));
      for (int r = 0; r < P; ++r) {
        auto &comm = world.comm(r);
        T *buf = in[r];
        const T *send = in[r];
        T *recv = out[r];
        if (o.op == "allreduce") {
          if (o.nonblocking) { if (o.inplace) Al::NonblockingAllreduce<Backend>(buf, size, rop, comm, reqs[r], algo); else Al::NonblockingAllreduce<Backend>(send, recv, size, rop, comm, reqs[r], algo); }
          else { if (o.inplace) Al::Allreduce<Backend>(buf, size, rop, comm, algo); else Al::Allreduce<Backend>(send, recv, size, rop, comm, algo); }
        } else if (o.op == "reduce") {
          if (o.nonblocking) { if (o.inplace) Al::NonblockingReduce<Backend>(buf, size, rop, o.root, comm, reqs[r], algo); else Al::NonblockingReduce<Backend>(send, recv, size, rop, o.root, comm, reqs[r], algo); }
          else { if (o.inplace) Al::Reduce<Backend>(buf, size, rop, o.root, comm, algo); else Al::Reduce<Backend>(send, recv, size, rop, o.root, comm, algo); }
        } else if (o.op == "reduce_scatter") {
          if (o.nonblocking && o.inplace) Al::NonblockingReduce_scatter<Backend>(buf, size, rop, comm, reqs[r], algo);
          else if (o.nonblocking) Al::NonblockingReduce_scatter<Backend>(send, recv, size, rop, comm, reqs[r], algo);
          else if (o.inplace) Al::Reduce_scatter<Backend>(buf, size, rop, comm, algo);
          else Al::Reduce_scatter<Backend>(send, recv, size, rop, comm, algo);
        } else if (o.op == "reduce_scatterv") {
          // every rank contributes the same count, as in the reference's benchmark
          const std::vector<size_t> counts((size_t)P, size);
          if (o.nonblocking && o.inplace) Al::NonblockingReduce_scatterv<Backend>(buf, counts, rop, comm, reqs[r], algo);
          else if (o.nonblocking) Al::NonblockingReduce_scatterv<Backend>(send, recv, counts, rop, comm, reqs[r], algo);
          else if (o.inplace) Al::Reduce_scatterv<Backend>(buf, counts, rop, comm, algo);
          else Al::Reduce_scatterv<Backend>(send, recv, counts, rop, comm, algo);
        } else if (o.op == "allgatherv") {
          const std::vector<size_t> counts((size_t)P, size);
          std::vector<size_t> displs((size_t)P);
          for (int q = 0; q < P; ++q) displs[(size_t)q] = (size_t)q * size;
          if (o.nonblocking && o.inplace) Al::NonblockingAllgatherv<Backend>(recv, counts, displs, comm, reqs[r], algo);
          else if (o.nonblocking) Al::NonblockingAllgatherv<Backend>(send, recv, counts, displs, comm, reqs[r], algo);
          else if (o.inplace) Al::Allgatherv<Backend>(recv, counts, displs, comm, algo);
          else Al::Allgatherv<Backend>(send, recv, counts, displs, comm, algo);
        } else {
          if (o.nonblocking && o.inplace) Al::NonblockingAllgather<Backend>(recv, size, comm, reqs[r], algo);
          else if (o.nonblocking) Al::NonblockingAllgather<Backend>(send, recv, size, comm, reqs[r], algo);
          else if (o.inplace) Al::Allgather<Backend>(recv, size, comm, algo);
          else Al::Allgather<Backend>(send, recv, size, comm, algo);
        }
      }
      for (int r = 0; r < P; ++r)
        if (reqs[r] != Backend::null_req) Al::Wait<Backend>(reqs[r]);
      HIPCHK(hipEventRecord(e1, stream));
      HIPCHK(hipEventSynchronize(e1));
      float ms = 0;
      HIPCHK(hipEventElapsedTime(&ms, e0, e1));
      if (trial >= o.warmup) times.push_back(ms * 1e-3);
    }
    for (int r = 1; r < P; ++r) HIPCHK(hipStreamSynchronize(streams[(size_t)r]));
    }
    if (o.stream_per_rank)
      for (int r = 1; r < P; ++r) HIPCHK(hipStreamDestroy(streams[(size_t)r]));
    res.times[size] = times;
    for (int r = 0; r < P; ++r) { HIPCHK(hipFree(in[r])); HIPCHK(hipFree(out[r])); }
  }
  if (o.summarize) res.summary(stdout);
  if (!o.save_to.empty()) {
    std::FILE *f = std::fopen(o.save_to.c_str(), "w");
    if (!f) { std::fprintf(stderr, "Error opening %s\n", o.save_to.c_str()); return 2; }
    res.write(f);
    std::fclose(f);
  }
  if (o.print_table) res.write(stdout);
  HIPCHK(hipEventDestroy(e0));
  HIPCHK(hipEventDestroy(e1));
  HIPCHK(hipStreamDestroy(stream));
  return 0;
}

int main(int argc, char **argv) {
  Options o;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    auto next = [&]() -> std::string { if (i + 1 >= argc) { std::fprintf(stderr, "missing value for %s\n", a.c_str()); std::exit(2); } return argv[++i]; };
    if (a == "--op") o.op = next();
    else if (a == "--datatype") o.datatype = next();
    else if (a == "--reduction-op") o.redop = next();
    else if (a == "--algo" || a == "--algorithm") o.algo = next();
    else if (a == "--size") o.min_size = o.max_size = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--summarize") o.summarize = true;
    else if (a == "--save-to-file") o.save_to = next();
    else if (a == "--no-print-table") o.print_table = false;
    else if (a == "--stream-per-rank") o.stream_per_rank = true;
    else if (a == "--tune") {  // name=value: one of the launch planner's settings (alamd_tune)
      const std::string kv = next();
      const size_t eq = kv.find('=');
      if (eq == std::string::npos || alamd_tune(kv.substr(0, eq).c_str(), std::strtoull(kv.c_str() + eq + 1, nullptr, 10)) != ALAMD_OK) {
        std::fprintf(stderr, "bad --tune %s\n", kv.c_str());
        return 2;
      }
    }
    else if (a == "--backend") { if (next() != "hip") { std::fprintf(stderr, "this program benchmarks the hip backend only\n"); return 2; } }
    else if (a == "--help") { std::printf("see the usage comment at the top of tests/cpp/bench_ops.cpp\n"); return 0; }
    else if (a == "--ranks") o.ranks = std::atoi(next().c_str());
    else if (a == "--root") o.root = std::atoi(next().c_str());
    else if (a == "--inplace") o.inplace = true;
    else if (a == "--nonblocking") o.nonblocking = true;
    else if (a == "--min-size") o.min_size = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--max-size") o.max_size = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--num-iters") o.iters = std::strtoull(next().c_str(), nullptr, 10);
    else if (a == "--num-warmup") o.warmup = std::strtoull(next().c_str(), nullptr, 10);
    else { std::fprintf(stderr, "unknown option %s\n", a.c_str()); return 2; }
  }
  const std::map<std::string, Al::ReductionOperator> rops = {
      {"sum", Al::ReductionOperator::sum}, {"prod", Al::ReductionOperator::prod}, {"min", Al::ReductionOperator::min},
      {"max", Al::ReductionOperator::max}, {"lor", Al::ReductionOperator::lor}, {"land", Al::ReductionOperator::land},
      {"lxor", Al::ReductionOperator::lxor}, {"bor", Al::ReductionOperator::bor}, {"band", Al::ReductionOperator::band},
      {"bxor", Al::ReductionOperator::bxor}, {"avg", Al::ReductionOperator::avg}};
  const std::map<std::string, Algo> algos = {
      {"automatic", Algo::automatic}, {"automatic_mpi_blocking", Algo::automatic_mpi_blocking},
      {"rank_order", Algo::rank_order}, {"tree_doubling", Algo::tree_doubling},
      {"tree_halving", Algo::tree_halving}, {"tree_binomial", Algo::tree_binomial}, {"tree_reduce_scatter_gather", Algo::tree_reduce_scatter_gather},
      {"tree_reduce_scatter_gather_spread", Algo::tree_reduce_scatter_gather_spread}, {"pairwise", Algo::pairwise},
      {"ring", Algo::ring}, {"ring_fused", Algo::ring_fused}};
  if (!rops.count(o.redop) || !algos.count(o.algo) || o.min_size == 0 ||
      (o.op != "allreduce" && o.op != "reduce" && o.op != "reduce_scatter" && o.op != "allgather" &&
       o.op != "reduce_scatterv" && o.op != "allgatherv")) {
    std::fprintf(stderr, "bad --op / --reduction-op / --algo / --min-size\n");
    return 2;
  }
  HIPCHK(hipSetDevice(0));
  try {
    const auto rop = rops.at(o.redop);
    const auto algo = algos.at(o.algo);
    if (o.datatype == "float") return run<float>(o, rop, algo, "f");
    if (o.datatype == "double") return run<double>(o, rop, algo, "d");
    if (o.datatype == "int") return run<int>(o, rop, algo, "i");
    if (o.datatype == "long") return run<long>(o, rop, algo, "l");
    if (o.datatype == "uchar") return run<unsigned char>(o, rop, algo, "h");
    if (o.datatype == "half") return run<Al::amd::half_bits>(o, rop, algo, "6__half");
    if (o.datatype == "bfloat16") return run<Al::amd::bfloat16_bits>(o, rop, algo, "14__hip_bfloat16");
    std::fprintf(stderr, "unknown --datatype %s\n", o.datatype.c_str());
    return 2;
  } catch (const Al::al_exception &e) {
    std::fprintf(stderr, "%s\n", e.what());
    return 1;
  }
}
