// Latency of the stream flags, in the manner of the reference's
// benchmark/benchmark_waits.cpp:71-91 and benchmark_events.cpp:76-92:
//   enqueue   host cost of enqueueing one wait / one flag write
//   resume    host signal -> the stream gets past the wait and writes the
//             next flag -> the host sees it
//   completion  a flag written by the stream against a runtime event, as
//             benchmark_events.cpp compares them: cost of recording on an
//             idle stream, and how long until the host's query sees it
// Prints one JSON line.  usage: bench_flags [iterations]
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "aluminum_amd.h"

#define CHK(x) do { if ((x) != 0) { std::printf("error: %s\n", alamd_last_error()); return 2; } } while (0)
#define HIPCHK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("HIP error %s\n", hipGetErrorString(e_)); return 2; } } while (0)

using clk = std::chrono::steady_clock;
static double us(clk::time_point a, clk::time_point b) { return std::chrono::duration<double, std::micro>(b - a).count(); }
static double median(std::vector<double> v) { std::sort(v.begin(), v.end()); return v[v.size() / 2]; }

static int run_mode(int mode, const char *name, int iters, hipStream_t stream, bool last) {
  alamd_flag *gate, *done;
  CHK(alamd_flag_create(&gate, 0));
  CHK(alamd_flag_create(&done, 0));
  std::vector<double> enq_wait, enq_write, resume;
  const uint64_t spins = mode == ALAMD_FLAG_KERNEL ? (1ull << 22) : 0;
  for (int it = 0; it < iters + 20; ++it) {
    CHK(alamd_flag_signal(gate, 0));
    CHK(alamd_flag_signal(done, 0));
    auto t0 = clk::now();
    CHK(alamd_stream_wait_flag(stream, gate, 1, mode, spins));
    auto t1 = clk::now();
    CHK(alamd_stream_write_flag(stream, done, 1, mode));
    auto t2 = clk::now();
    // let the stream reach the wait before the signal is given
    for (volatile int k = 0; k < 20000; ++k) {}
    auto t3 = clk::now();
    CHK(alamd_flag_signal(gate, 1));
    while (alamd_flag_query(done) != 1) {
      if (us(t3, clk::now()) > 5e6) { std::printf("timeout in mode %s\n", name); return 3; }
    }
    auto t4 = clk::now();
    HIPCHK(hipStreamSynchronize(stream));
    if (it >= 20) { enq_wait.push_back(us(t0, t1)); enq_write.push_back(us(t1, t2)); resume.push_back(us(t3, t4)); }
  }
  std::printf("\"%s\": {\"enqueue_wait_us\": %.3f, \"enqueue_write_us\": %.3f, \"signal_to_resume_us\": %.3f, "
              "\"signal_to_resume_min_us\": %.3f}%s",
              name, median(enq_wait), median(enq_write), median(resume),
              *std::min_element(resume.begin(), resume.end()), last ? "" : ", ");
  CHK(alamd_flag_destroy(gate));
  CHK(alamd_flag_destroy(done));
  return 0;
}

// record on an idle stream, then poll from the host: the status flag (alamd_stream_write_flag +
// alamd_flag_query) against hipEventRecord + hipEventQuery
static int run_completion(int mode, const char *name, int iters, hipStream_t stream) {
  alamd_flag *flag;
  CHK(alamd_flag_create(&flag, 0));
  hipEvent_t ev;
  HIPCHK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  std::vector<double> rec_flag, seen_flag, rec_ev, seen_ev;
  for (int it = 0; it < iters + 20; ++it) {
    CHK(alamd_flag_signal(flag, 0));
    auto t0 = clk::now();
    CHK(alamd_stream_write_flag(stream, flag, 1, mode));
    auto t1 = clk::now();
    while (alamd_flag_query(flag) != 1) {
      if (us(t1, clk::now()) > 5e6) { std::printf("timeout in completion %s\n", name); return 3; }
    }
    auto t2 = clk::now();
    HIPCHK(hipStreamSynchronize(stream));
    auto t3 = clk::now();
    HIPCHK(hipEventRecord(ev, stream));
    auto t4 = clk::now();
    while (hipEventQuery(ev) == hipErrorNotReady) {
      if (us(t4, clk::now()) > 5e6) { std::printf("timeout in completion %s\n", name); return 3; }
    }
    auto t5 = clk::now();
    HIPCHK(hipStreamSynchronize(stream));
    if (it >= 20) {
      rec_flag.push_back(us(t0, t1)); seen_flag.push_back(us(t1, t2));
      rec_ev.push_back(us(t3, t4)); seen_ev.push_back(us(t4, t5));
    }
  }
  std::printf(", \"completion_%s\": {\"flag_record_us\": %.3f, \"flag_seen_after_us\": %.3f, "
              "\"hip_event_record_us\": %.3f, \"hip_event_seen_after_us\": %.3f}",
              name, median(rec_flag), median(seen_flag), median(rec_ev), median(seen_ev));
  HIPCHK(hipEventDestroy(ev));
  CHK(alamd_flag_destroy(flag));
  return 0;
}

int main(int argc, char **argv) {
  const int iters = argc > 1 ? std::atoi(argv[1]) : 2000;
  HIPCHK(hipSetDevice(0));
  CHK(alamd_init());
  hipStream_t stream;
  HIPCHK(hipStreamCreate(&stream));
  const bool memops = alamd_stream_memops_supported() != 0;
  std::printf("{\"iterations\": %d, \"stream_memops_supported\": %s, ", iters, memops ? "true" : "false");
  int rc = run_mode(ALAMD_FLAG_KERNEL, "kernel", iters, stream, !memops);
  if (rc) return rc;
  if (memops) {
    rc = run_mode(ALAMD_FLAG_MEMOP, "memop", iters, stream, true);
    if (rc) return rc;
  }
  rc = run_completion(ALAMD_FLAG_KERNEL, "kernel", iters, stream);
  if (rc) return rc;
  if (memops && (rc = run_completion(ALAMD_FLAG_MEMOP, "memop", iters, stream))) return rc;
  std::printf("}\n");
  HIPCHK(hipStreamDestroy(stream));
  return 0;
}
