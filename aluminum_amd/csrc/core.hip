// Library-wide host code: error text, dtype table, device probe.
#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <string>

#include "alamd_common.h"

namespace alamd {

int chain_static_init();  // combine.hip

namespace {
thread_local char g_err[512] = "";
std::mutex g_dev_mutex;
int g_dev_cus[64];
bool g_dev_known[64];
}  // namespace

int set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_err[0] = 0; }

Tunables &tunables() {
  static Tunables t;
  return t;
}

namespace {
// least: the pieces of a two-step call at least 64 KiB (smaller ones would turn one call into millions
// of launches; less than one element, into a loop that never ends)
struct TunableName { const char *name; std::atomic<size_t> Tunables::*field; size_t least; };
const TunableName kTunableNames[] = {
    {"launch_bytes", &Tunables::launch_bytes, 1},
    {"two_step_min_total_bytes", &Tunables::two_step_min_total_bytes, 1},
    {"two_step_min_outputs", &Tunables::two_step_min_outputs, 1},
    {"two_step_piece_bytes", &Tunables::two_step_piece_bytes, (size_t)64 << 10},
    {"ring_piece_bytes", &Tunables::ring_piece_bytes, (size_t)64 << 10},
    {"spread_launch_bytes", &Tunables::spread_launch_bytes, 1},
    {"spread_hbm_chunk_tiles", &Tunables::spread_hbm_chunk_tiles, 1},
    {"spread_hbm_launch_chunks", &Tunables::spread_hbm_launch_chunks, 1},
    {"spread_cache_chunk_tiles", &Tunables::spread_cache_chunk_tiles, 1},
    {"spread_cache_launch_chunks", &Tunables::spread_cache_launch_chunks, 1},
    {"block_shape_from_bytes", &Tunables::block_shape_from_bytes, 1},
    {"block_shape_below_bytes", &Tunables::block_shape_below_bytes, 1},
    {"fold_front3_ranks", &Tunables::fold_front3_ranks, 0},
    {"stream_wgs_per_cu", &Tunables::stream_wgs_per_cu, 0},
    {"halo_load_policy", &Tunables::halo_load_policy, 0},
};
}  // namespace

int device_cus() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    set_error(ALAMD_ERR_HIP, "hipGetDevice failed: no usable GPU");
    return -1;
  }
  if (dev < 0 || dev >= 64) {
    set_error(ALAMD_ERR_HIP, "device index %d out of range", dev);
    return -1;
  }
  std::lock_guard<std::mutex> lock(g_dev_mutex);
  if (!g_dev_known[dev]) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
      set_error(ALAMD_ERR_HIP, "hipGetDeviceProperties failed");
      return -1;
    }
    g_dev_cus[dev] = prop.multiProcessorCount;
    g_dev_known[dev] = true;
  }
  return g_dev_cus[dev];
}

unsigned stream_grid(size_t work_items, size_t per_block, int waves) {
  const int cus = device_cus();
  size_t need = (work_items + per_block - 1) / per_block;
  size_t cap = (size_t)(cus > 0 ? cus : 256) * (size_t)(waves > 0 ? waves : 1);
  if (need < 1) need = 1;
  return (unsigned)(need < cap ? need : cap);
}

int check_type_op(int dtype, int op) {
  if (dtype < 0 || dtype >= ALAMD_NUM_DTYPES)
    return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);
  if (op < ALAMD_SUM || op > ALAMD_AVG)
    return set_error(ALAMD_ERR_UNSUPPORTED_OP, "Reduction operator not supported");
  if (is_float_dtype(dtype) && op > ALAMD_MAX && op != ALAMD_AVG)
    return set_error(ALAMD_ERR_UNSUPPORTED_OP, "Reduction operator not supported");
  return ALAMD_OK;
}

}  // namespace alamd

extern "C" {

const char *alamd_last_error(void) { return alamd::g_err; }

int alamd_version(void) { return ALAMD_VERSION_MAJOR * 100 + ALAMD_VERSION_MINOR; }

size_t alamd_dtype_size(int dtype) {
  switch (dtype) {
  case ALAMD_I8: case ALAMD_U8: return 1;
  case ALAMD_I16: case ALAMD_U16: case ALAMD_F16: case ALAMD_BF16: return 2;
  case ALAMD_I32: case ALAMD_U32: case ALAMD_F32: return 4;
  case ALAMD_I64: case ALAMD_U64: case ALAMD_F64: return 8;
  default: return 0;
  }
}

int alamd_tune(const char *name, size_t value) {
  if (!name) return alamd::set_error(ALAMD_ERR_INVALID_ARG, "null name");
  const alamd::Tunables defaults;
  for (const auto &t : alamd::kTunableNames)
    if (std::string(name) == t.name) {
      if (value != 0 && value < t.least)
        return alamd::set_error(ALAMD_ERR_INVALID_ARG, "%s must be at least %zu (0 restores the default)", name, t.least);
      (alamd::tunables().*(t.field)).store(value ? value : (defaults.*(t.field)).load());
      return ALAMD_OK;
    }
  return alamd::set_error(ALAMD_ERR_INVALID_ARG, "no launch-planner size is called %s", name);
}

size_t alamd_tuned(const char *name) {
  if (name)
    for (const auto &t : alamd::kTunableNames)
      if (std::string(name) == t.name) return (alamd::tunables().*(t.field)).load();
  return 0;
}

int alamd_check_op(int dtype, int op) { return alamd::check_type_op(dtype, op); }

int alamd_reference_order(int collective, int P, size_t count, int dtype, int root, int *order, int *start) {
  if (!order || !start) return alamd::set_error(ALAMD_ERR_INVALID_ARG, "null result pointer");
  if (P < 1 || P > ALAMD_MAX_RANKS) return alamd::set_error(ALAMD_ERR_INVALID_ARG, "number of ranks %d outside [1, %d]", P, ALAMD_MAX_RANKS);
  const size_t es = alamd_dtype_size(dtype);
  if (es == 0) return alamd::set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);
  *start = 0;
  switch (collective) {
  case ALAMD_COLL_ALLREDUCE:
  case ALAMD_COLL_REDUCE:
  case ALAMD_COLL_ALLREDUCE_BLOCKING:
  case ALAMD_COLL_REDUCE_BLOCKING: {
    const bool rooted = collective == ALAMD_COLL_REDUCE || collective == ALAMD_COLL_REDUCE_BLOCKING;
    const bool blocking = collective == ALAMD_COLL_ALLREDUCE_BLOCKING || collective == ALAMD_COLL_REDUCE_BLOCKING;
    if (rooted && (root < 0 || root >= P))
      return alamd::set_error(ALAMD_ERR_INVALID_ARG, "root %d outside [0, %d)", root, P);
    // An allreduce among ranks of one host is a reduce to rank 0 followed by a broadcast.  The reduce
    // is a binomial tree to the root, over the ranks counted from it, for short messages, for fewer
    // elements than the largest power of two of ranks and for every operation that is not one of the
    // library's own (fp16 and bf16 are user-defined operations to it); otherwise a reduce-scatter by
    // recursive halving followed by a gather, which does not depend on the root; the blocking calls
    // cut its blocks differently from the non-blocking ones.
    size_t pof2 = 1;
    while (2 * pof2 <= (size_t)P) pof2 *= 2;
    const bool user_op = dtype == ALAMD_F16 || dtype == ALAMD_BF16;
    if (user_op || count * es <= 2048 || count < pof2) {
      *order = ALAMD_ORDER_TREE_BINOMIAL;
      *start = rooted ? root : 0;
    } else {
      *order = blocking ? ALAMD_ORDER_TREE_RSG_SPREAD : ALAMD_ORDER_TREE_RSG;
    }
    return ALAMD_OK;
  }
  case ALAMD_COLL_REDUCE_SCATTER:
    // recursive halving below 512 KiB in all, pairwise exchange from there on (commutative operations,
    // user-defined ones included)
    *order = count * es < ((size_t)512 << 10) ? ALAMD_ORDER_TREE_HALV : ALAMD_ORDER_PAIRWISE_DESC;
    return ALAMD_OK;
  default:
    return alamd::set_error(ALAMD_ERR_INVALID_ARG, "unknown collective %d", collective);
  }
}

int alamd_init(void) {
  int dev = 0;
  ALAMD_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  ALAMD_HIP(hipGetDeviceProperties(&prop, dev));
  if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0)
    return alamd::set_error(ALAMD_ERR_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only",
                            dev, prop.gcnArchName);
  if (alamd::device_cus() <= 0) return ALAMD_ERR_HIP;
  return alamd::chain_static_init();
}

}  // extern "C"
