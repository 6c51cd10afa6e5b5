// Host side of the combine entry points: argument checks, the mapping of a
// named order onto one of the two kernel families, the Reduce_scatter and
// Allgather layouts.
#include <atomic>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "alamd_dispatch.h"
#include "alamd_tile.h"
#include "aluminum_amd_support.h"

namespace alamd {

namespace {

bool ranges_overlap(const void *a, size_t abytes, const void *b, size_t bbytes) {
  const uintptr_t x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
  return x < y + bbytes && y < x + abytes;
}

int floor_pow2(int p) { int q = 1; while (2 * q <= p) q *= 2; return q; }
int ceil_pow2(int p) { int q = 1; while (q < p) q *= 2; return q; }

int bit_reverse(int v, int bits) {
  int r = 0;
  for (int b = 0; b < bits; ++b) if (v & (1 << b)) r |= 1 << (bits - 1 - b);
  return r;
}

// Orders whose `start` argument means something: the first rank of a fold, the root of the binomial
// tree, the rank a halving tree's result is for.
bool order_has_start(int order) {
  return order == ALAMD_ORDER_PAIRWISE_DESC || order == ALAMD_ORDER_RING || order == ALAMD_ORDER_TREE_BINOMIAL ||
         order == ALAMD_ORDER_TREE_HALV;
}
// ... and of those, the ones for which a Reduce_scatter passes the receiving rank (the block's index).
bool order_start_per_block(int order) {
  return order == ALAMD_ORDER_PAIRWISE_DESC || order == ALAMD_ORDER_RING || order == ALAMD_ORDER_TREE_HALV;
}
bool order_is_tree(int order) {
  return order == ALAMD_ORDER_TREE_DBL || order == ALAMD_ORDER_TREE_HALV || order == ALAMD_ORDER_TREE_BINOMIAL ||
         order == ALAMD_ORDER_TREE_RSG || order == ALAMD_ORDER_TREE_RSG_SPREAD;
}
bool order_is_rsg(int order) { return order == ALAMD_ORDER_TREE_RSG || order == ALAMD_ORDER_TREE_RSG_SPREAD; }
bool order_valid(int order) { return order >= ALAMD_ORDER_RANK_ASC && order <= ALAMD_ORDER_TREE_RSG_SPREAD; }

// Fills the slot tables of a tree order over the P inputs `ins`.  start: the root of the binomial tree.
int build_tree(TreeParams &tp, const void *const *ins, int P, int order, int start) {
  for (int j = 0; j < ALAMD_MAX_RANKS; ++j) { tp.a[j] = nullptr; tp.b[j] = nullptr; }
  tp.P = P;
  tp.role_mode = ROLE_FIXED;
  tp.role_rem = tp.role_bits = tp.role_start0 = tp.role_stride = 0;
  tp.role_base = tp.role_count = 0;
  tp.role_spread = order == ALAMD_ORDER_TREE_RSG_SPREAD;
  if (order == ALAMD_ORDER_TREE_BINOMIAL) {
    // the ranks counted from the root, with wrap
    for (int j = 0; j < P; ++j) tp.a[j] = static_cast<const char *>(ins[(j + start) % P]);
    tp.nvalid = P;
    return ceil_pow2(P);
  }
  const int pof2 = floor_pow2(P), rem = P - pof2;
  const char *la[ALAMD_MAX_RANKS], *lb[ALAMD_MAX_RANKS];
  // pre-fold of the first 2 * rem ranks: the slot holds step(in = la, inout = lb).  The odd rank
  // keeps the result, except under TREE_RSG(_SPREAD), where the even one does.
  const int keep = order_is_rsg(order) ? 0 : 1;
  for (int j = 0; j < pof2; ++j) {
    if (j < rem) { la[j] = static_cast<const char *>(ins[2 * j + 1 - keep]); lb[j] = static_cast<const char *>(ins[2 * j + keep]); }
    else { la[j] = static_cast<const char *>(ins[j + rem]); lb[j] = nullptr; }
  }
  int bits = 0;
  while ((1 << bits) < pof2) ++bits;
  tp.role_rem = rem;
  tp.role_bits = bits;
  if (order == ALAMD_ORDER_TREE_HALV) tp.role_mode = ROLE_PER_SEGMENT;
  if (order_is_rsg(order)) tp.role_mode = ROLE_PER_BLOCK;
  for (int k = 0; k < pof2; ++k) {
    // pairing at distance pof2/2, ..., 1 is the adjacent-pair tree over the
    // bit-reversed slot order
    const int src = order == ALAMD_ORDER_TREE_HALV ? bit_reverse(k, bits) : k;
    tp.a[k] = la[src];
    tp.b[k] = lb[src];
  }
  tp.nvalid = pof2;
  return pof2;
}

struct Layout {
  unsigned nseg;
  SegParams seg;
  size_t max_len;
  int start0, start_stride;  // segment s is for rank (start0 + s * start_stride) mod P (orders with a start)
  // TREE_RSG(_SPREAD), when the launch covers part of a message only: where element 0 of a segment lies in the
  // message, and the message's length (0: every segment is a message of its own)
  size_t msg_base = 0, msg_count = 0;
};

// Launches the fold or tree kernels for `order` over inputs `ins`.
// `outs` has ALAMD_MAX_RANKS entries (unused ones null).
// chain / displ_bytes: see launch_fold.
int launch_order(void *const *outs, const void *const *ins, int P, const Layout &lay, int dtype, int op,
                 int order, hipStream_t stream, const ChainScratch *chain = nullptr, size_t displ_bytes = 0) {
  if (!is_float_dtype(dtype)) order = ALAMD_ORDER_RANK_ASC;  // integer ops: every order gives the same bits
  if (P == 1 && order_is_tree(order)) order = ALAMD_ORDER_RANK_ASC;
  if (order_is_tree(order)) {
    TreeParams tp;
    const int slots = build_tree(tp, ins, P, order, order == ALAMD_ORDER_TREE_BINOMIAL ? lay.start0 % P : 0);
    for (int j = 0; j < ALAMD_MAX_RANKS; ++j) tp.out[j] = static_cast<char *>(outs[j]);
    tp.seg = lay.seg;
    tp.role_start0 = lay.start0;
    tp.role_stride = lay.start_stride;
    tp.role_base = lay.msg_base;
    tp.role_count = lay.msg_count;
    return launch_tree(tp, slots, lay.nseg, lay.max_len, dtype, op, stream, chain, displ_bytes);
  }
  FoldParams fp;
  for (int r = 0; r < ALAMD_MAX_RANKS; ++r) {
    fp.in[r] = r < P ? static_cast<const char *>(ins[r]) : nullptr;
    fp.out[r] = static_cast<char *>(outs[r]);
  }
  fp.seg = lay.seg;
  fp.P = P;
  fp.start0 = lay.start0;
  fp.start_stride = lay.start_stride;
  fp.dir = order == ALAMD_ORDER_PAIRWISE_DESC ? -1 : 1;
  return launch_fold(fp, lay.nseg, lay.max_len, dtype, op, order == ALAMD_ORDER_RING, stream, chain, displ_bytes);
}

// ---- scratch of the chained launches -----------------------------------------

__global__ void chain_clear_kernel(unsigned *ticket, unsigned *flags, unsigned long long n) {
  const unsigned long long i0 = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i0 == 0) *ticket = 0u;
  for (unsigned long long i = i0; i < n; i += (unsigned long long)gridDim.x * blockDim.x) flags[i] = 0u;
}

// Bytes in front of the flags: the ticket counter and the error word, on a line of their own.
constexpr size_t kChainHeaderBytes = 256;
// The smallest tile of any kernel that can run chained (256 threads x one 128-bit vector).
constexpr size_t kChainMinTileBytes = 4096;

// One scratch buffer per (device, stream): calls on different streams may overlap in time.  A buffer
// that turns out too small is replaced by a larger one and kept until the process ends, because work
// already enqueued may still use it.
struct ChainPool {
  std::mutex mutex;
  std::map<std::pair<int, hipStream_t>, ChainScratch> live;
  std::map<std::pair<int, hipStream_t>, std::vector<void *>> retired;
};
ChainPool &chain_pool() {
  static ChainPool *pool = new ChainPool;  // never destroyed: device memory outlives static destruction order
  return *pool;
}

// Where a wait that gave up leaves its mark: one word of pinned host memory for the whole process,
// allocated by alamd_init (or by the first chained launch that may allocate), so that the host can
// read it without touching the device.  Until it exists the mark goes to the scratch's own word.
std::mutex g_expired_mutex;
unsigned *g_expired_host = nullptr, *g_expired_dev = nullptr;
std::atomic<unsigned> g_chain_polls{kChainDefaultPolls};

int expired_word_init() {
  std::lock_guard<std::mutex> lock(g_expired_mutex);
  if (g_expired_host) return ALAMD_OK;
  void *host = nullptr, *dev = nullptr;
  ALAMD_HIP(hipHostMalloc(&host, 256, hipHostMallocMapped | hipHostMallocCoherent | hipHostMallocPortable));
  *static_cast<volatile unsigned *>(host) = 0u;
  ALAMD_HIP(hipHostGetDevicePointer(&dev, host, 0));
  g_expired_dev = static_cast<unsigned *>(dev);
  g_expired_host = static_cast<unsigned *>(host);
  return ALAMD_OK;
}

// 1 (once) if a chained launch has given up a wait since the last call.
bool take_expired() {
  std::lock_guard<std::mutex> lock(g_expired_mutex);
  if (!g_expired_host) return false;
  return __atomic_exchange_n(g_expired_host, 0u, __ATOMIC_SEQ_CST) != 0u;
}

void finish_scratch(ChainScratch &cs) {
  std::lock_guard<std::mutex> lock(g_expired_mutex);
  if (g_expired_dev) cs.error = g_expired_dev;
  cs.max_polls = g_chain_polls.load();
}

ChainScratch scratch_at(void *base, size_t bytes) {
  ChainScratch cs;
  char *b = static_cast<char *>(base);
  cs.ticket = reinterpret_cast<unsigned *>(b);
  cs.error = reinterpret_cast<unsigned *>(b + 4);
  cs.flags = reinterpret_cast<unsigned *>(b + kChainHeaderBytes);
  cs.max_tiles = (bytes - kChainHeaderBytes) / sizeof(unsigned);
  cs.max_polls = kChainDefaultPolls;
  return cs;
}

// The scratch of `stream` for `tiles` tile flags.  may_allocate: a buffer that is missing or too small is
// allocated here (hipMalloc, nothing else: every chained launch clears what it uses on its own stream
// first); otherwise its absence is an error.  A stream that is being captured never allocates.
int chain_scratch_for(hipStream_t stream, size_t tiles, bool may_allocate, ChainScratch &out) {
  int dev = 0;
  ALAMD_HIP(hipGetDevice(&dev));
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  ALAMD_HIP(hipStreamIsCapturing(stream, &capturing));
  if (capturing != hipStreamCaptureStatusNone) may_allocate = false;
  ChainPool &pool = chain_pool();
  std::lock_guard<std::mutex> lock(pool.mutex);
  auto key = std::make_pair(dev, stream);
  auto it = pool.live.find(key);
  if (it != pool.live.end() && it->second.max_tiles >= tiles) {
    out = it->second;
    finish_scratch(out);
    return ALAMD_OK;
  }
  if (!may_allocate)
    return set_error(ALAMD_ERR_INVALID_ARG,
                     "an in-place block that overlaps its own input needs %zu bytes of scratch on this stream, and a "
                     "stream that is being captured cannot allocate them: call alamd_reserve_scratch first",
                     kChainHeaderBytes + tiles * sizeof(unsigned));
  if (int rc = expired_word_init()) return rc;
  size_t cap = (size_t)1 << 16;
  while (cap < tiles) cap *= 2;
  const size_t bytes = kChainHeaderBytes + cap * sizeof(unsigned);
  void *mem = nullptr;
  ALAMD_HIP(hipMalloc(&mem, bytes));
  // work already enqueued may still use the buffer this one replaces: it is kept until the stream's
  // scratch is released
  if (it != pool.live.end()) pool.retired[key].push_back(it->second.ticket);
  out = scratch_at(mem, bytes);
  pool.live[key] = out;
  finish_scratch(out);
  return ALAMD_OK;
}

// The scratch of alamd_reduce_scatterv_noalloc: part of the code object, so every device the library
// runs on holds its own copy at its own address until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress; the address it yields for the current device is what
// kernels and the clearing launch are given.
}  // namespace
static __device__ __align__(256) unsigned char scratch[ALAMD_NOALLOC_SCRATCH_BYTES];
namespace {

std::mutex g_static_mutex;
unsigned char *g_static_ptr[64];
// Who used a device's array last: the stream, and an event recorded behind its chained launch.  A call on
// another stream that comes before that event has completed would share counter and flags with work still
// running, and is refused.  (Launches recorded into a graph are not tracked: what runs beside a replay is
// the caller's to order.)
struct StaticOwner { hipStream_t stream = nullptr; hipEvent_t event = nullptr; bool pending = false; };
StaticOwner g_static_owner[64];

// Set-up, once per device, by alamd_init: the array's address on the current device and the owner's event.
int static_scratch_setup() {
  int dev = 0;
  ALAMD_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return set_error(ALAMD_ERR_HIP, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_ptr[dev]) return ALAMD_OK;
  unsigned char *ptr = nullptr;
  ALAMD_HIP(hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)));
  if (!ptr) return set_error(ALAMD_ERR_HIP, "hipGetSymbolAddress returned a null address");
  ALAMD_HIP(hipEventCreateWithFlags(&g_static_owner[dev].event, hipEventDisableTiming));
  g_static_ptr[dev] = ptr;
  return ALAMD_OK;
}

// The fixed array as scratch for a call on `stream`.  Allocates nothing: without alamd_init on this device
// it is an error.
int static_chain_scratch(hipStream_t stream, ChainScratch &out) {
  int dev = 0;
  ALAMD_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return set_error(ALAMD_ERR_HIP, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[dev] || !g_expired_host)
    return set_error(ALAMD_ERR_INVALID_ARG, "alamd_reduce_scatterv_noalloc needs alamd_init to have run on this device "
                                            "(it looks up the fixed scratch array and allocates nothing later)");
  StaticOwner &own = g_static_owner[dev];
  if (own.pending && own.stream != stream) {
    const hipError_t e = hipEventQuery(own.event);
    if (e == hipErrorNotReady)
      return set_error(ALAMD_ERR_INVALID_ARG, "the fixed scratch array is still in use by a chained launch on another "
                                              "stream of this device: keep such calls on one stream, or order them");
    if (e != hipSuccess) return set_error(ALAMD_ERR_HIP, "hipEventQuery failed: %s", hipGetErrorString(e));
    own.pending = false;
  }
  out = scratch_at(g_static_ptr[dev], ALAMD_NOALLOC_SCRATCH_BYTES);
  finish_scratch(out);
  return ALAMD_OK;
}

// Called behind a chained launch that used the fixed array.
int static_scratch_used(hipStream_t stream) {
  int dev = 0;
  ALAMD_HIP(hipGetDevice(&dev));
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  ALAMD_HIP(hipStreamIsCapturing(stream, &capturing));
  if (capturing != hipStreamCaptureStatusNone) return ALAMD_OK;
  std::lock_guard<std::mutex> lock(g_static_mutex);
  StaticOwner &own = g_static_owner[dev];
  ALAMD_HIP(hipEventRecord(own.event, stream));
  own.stream = stream;
  own.pending = true;
  return ALAMD_OK;
}

constexpr int kGatherU = 8, kGatherThreads = 128;

// Slices to several destinations: the seg_len[q] bytes of source q go to byte
// offset seg_off[q] of every destination p.out[0..P) (a destination that is
// the source itself, the in-place form, is skipped).  One workgroup per
// (destination, source, tile).  blockIdx.y counts groups of nsrc_x sources;
// blockIdx.x runs chunk by chunk (tpc tiles of each source of the group, 8 or
// 16 MiB per source); inside a chunk everything for destination 0 comes first
// (source by source: short slices of an allgather lie side by side in a
// receive buffer, so a group of them is one longer run of writes - 32 slices
// of 2 MiB to 32 buffers 68 % -> 89 % of peak, 64 of 512 KiB 66 % -> 82 % -
// as long as the group's chunks, 8 MiB at most, stay in L2 between the
// destinations: eight 8 MiB pieces of a ring in one group ran at 67 % against
// 80 % one by one), then destination 1,
// ...: at any time the device writes one contiguous stream per chunk instead
// of P interleaved ones, and re-reads the chunk of the source from cache:
// workgroups are dealt to the eight XCDs round-robin and tpc is a multiple of
// 8, so the workgroups that copy one source tile to the different destinations
// run on the same XCD and share its L2 (88 % of peak; 79 % with tpc a multiple
// of 4 only, 49 % with an odd tpc).  Measured for 1 read + 8 writes of 32 MiB:
// 88 % of the HBM peak, against 67 % when every workgroup writes its tile to
// all destinations (69 % for those writes alone).
// A chunk's share per XCD (at most 2 MiB) has to stay in that XCD's 4 MiB L2
// between the destinations: 32 MiB chunks run at 64 to 79 % of peak.  Two
// waves per SIMD: with the default occupancy the same calls run 4 to 10 points
// lower on buffers that no earlier call has touched.  Chunk length and launch
// length depend on where the source comes from (settings compared in one
// process, alternating, on separately allocated buffers; chunk tiles / chunks
// per launch):
//  - slices read from HBM (an allgather): 16 MiB chunks, launches of two chunks
//    per source.  Untouched 128 MiB slices: 1024/1 and 1024/2 83 %, 1024/4
//    79 %, 1024/8 77 %, 512/4 79 %, whole slice in one launch 77 %; untouched
//    32 MiB slices: 1024/any 83 %, 512/any 79 %; repeated buffers: 92 to 94 %.
//  - a result that a fold has just written, still in the memory-side cache (the
//    second step of a combine into several buffers): 8 MiB chunks, launches of
//    sixteen.  Allreduce at 256 MiB / 1 GiB per rank, untouched: 512/16 82 % /
//    81.5 %, 1024/8 81.5 % / 80 %, 1024/2 79.6 % / 78.8 %, whole piece in one
//    launch 80.4 % / 80.5 %; repeated: 512/16 86 %, 1024/2 83 %.
struct SpreadShape { unsigned chunk_tiles, launch_chunks; bool group_sources; };
inline SpreadShape spread_from_hbm() {
  return {(unsigned)tunables().spread_hbm_chunk_tiles, (unsigned)tunables().spread_hbm_launch_chunks, true};
}
inline SpreadShape spread_from_cache() {
  return {(unsigned)tunables().spread_cache_chunk_tiles, (unsigned)tunables().spread_cache_launch_chunks, false};
}
// Tunables::spread_launch_bytes: two 16 MiB chunks read, eight times that written
__global__ void __launch_bounds__(kGatherThreads) __attribute__((amdgpu_waves_per_eu(1, 2)))
spread_kernel(FoldParams p, unsigned tpc, unsigned tile0, unsigned src0, unsigned src_end, unsigned nsrc_x) {
  using TL = Tile<kGatherU, kGatherThreads>;
  const TL tl;
  const unsigned ndest = (unsigned)p.P;
  const unsigned per_dest = tpc * nsrc_x, per_chunk = per_dest * ndest;
  const unsigned chunk = blockIdx.x / per_chunk, rem = blockIdx.x % per_chunk;
  const unsigned dest = rem / per_dest, within = rem % per_dest;
  const unsigned qu = src0 + blockIdx.y * nsrc_x + within / tpc;
  if (qu >= src_end) return;
  const int q = (int)qu;
  const unsigned local = within % tpc;
  const char *src = p.in[q];
  const size_t len = p.seg.seg_len[q];
  char *dst = p.out[dest] + p.seg.seg_off[q];
  if (dst == src) return;
  // The tiles start where the destination reaches a 64-byte boundary: the
  // non-temporal stores go to memory line by line, and lines written in two
  // parts cost half the bandwidth (44 % of peak against 92 %).  The loads take
  // whatever alignment that leaves them.
  size_t head = (size_t)(64 - (reinterpret_cast<uintptr_t>(dst) & 63)) & 63;
  if (head > len) head = len;
  const size_t vec = (len - head) & ~(size_t)15, tail = len - head - vec;
  // the bytes before the first and after the last whole vector, once per destination
  if (tile0 == 0 && chunk == 0 && local == 0) {
    if (threadIdx.x < head) dst[threadIdx.x] = src[threadIdx.x];
    if (threadIdx.x < tail) dst[head + vec + threadIdx.x] = src[head + vec + threadIdx.x];
  }
  const size_t tb = ((size_t)tile0 + (size_t)chunk * tpc + local) * TL::BYTES;
  if (tb >= vec) return;
  const int nrec = vec - tb > TL::BYTES ? (int)TL::BYTES : (int)(vec - tb);
  const auto rs = TL::rsrc(src + head + tb, nrec);
  const auto rd = TL::rsrc(dst + head + tb, nrec);
  u32x4 v[kGatherU];
#pragma unroll
  for (int u = 0; u < kGatherU; ++u) v[u] = tl.load_cached(rs, u);
#pragma unroll
  for (int u = 0; u < kGatherU; ++u) tl.store_nt(rd, u, v[u]);
}

int misaligned(const char *what, int index) {
  return set_error(ALAMD_ERR_INVALID_ARG, "%s %d is not aligned to its element type", what, index);
}

int check_common(int P, size_t count, int dtype) {
  if (P < 1 || P > ALAMD_MAX_RANKS)
    return set_error(ALAMD_ERR_INVALID_ARG, "number of ranks %d outside [1, %d]", P, ALAMD_MAX_RANKS);
  if (alamd_dtype_size(dtype) == 0) return set_error(ALAMD_ERR_UNSUPPORTED_TYPE, "unknown dtype %d", dtype);
  if (count > (size_t)1 << 48) return set_error(ALAMD_ERR_INVALID_ARG, "count too large");
  return ALAMD_OK;
}

}  // namespace

int chain_static_init() {
  if (int rc = expired_word_init()) return rc;
  return static_scratch_setup();
}

int chain_clear(const ChainScratch &cs, size_t tiles, hipStream_t stream) {
  if (tiles > cs.max_tiles) return set_error(ALAMD_ERR_INVALID_ARG, "chain scratch too small");
  const unsigned blocks = (unsigned)((tiles + 255) / 256 < 1 ? 1 : ((tiles + 255) / 256 > 1024 ? 1024 : (tiles + 255) / 256));
  hipLaunchKernelGGL(chain_clear_kernel, dim3(blocks, 1, 1), dim3(256, 1, 1), 0, stream, cs.ticket, cs.flags,
                     (unsigned long long)tiles);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

namespace {

int launch_spread_once(const FoldParams &fp, int nsrc, SpreadShape shape, hipStream_t stream) {
  size_t max_len = 0;
  for (int q = 0; q < nsrc; ++q)
    if (fp.seg.seg_len[q] > max_len) max_len = fp.seg.seg_len[q];
  if (max_len == 0 || fp.P <= 0) return ALAMD_OK;
  const size_t tile = Tile<kGatherU, kGatherThreads>::BYTES;
  const size_t tiles = (max_len + tile - 1) / tile;
  // a multiple of 8 (see spread_kernel; workgroups past the last tile exit at once) - except for
  // slices of fewer than 8 tiles, where the idle workgroups would cost more than the sharing of an L2
  // gains (64 slices of 4 KB to 64 buffers: 50 us with seven idle workgroups beside every busy one)
  const size_t tpc = tiles >= shape.chunk_tiles ? shape.chunk_tiles : (tiles < 8 ? tiles : (tiles + 7) & ~(size_t)7);
  // A launch moves about spread_launch_bytes: with two or three destinations more chunks per launch
  // (untouched 128 MiB slices to two buffers 69 % -> 75 % of peak, 85 MiB slices to three 71 % -> 73 %;
  // four destinations ran 2 points better with the two chunks they have), and of many short sources
  // only some side by side along blockIdx.y (32 slices of 2 MiB to 32 buffers 64 % -> 69 %, 16 slices
  // of 8 MiB 77 % -> 81 %).  Compared in one process, both libraries loaded.
  size_t launch_chunks = shape.launch_chunks;
  const size_t per_chunk = tpc * tile * (size_t)(fp.P + 1);
  if (launch_chunks * per_chunk < tunables().spread_launch_bytes / 2) launch_chunks = tunables().spread_launch_bytes / per_chunk;
  const size_t all_chunks = (tiles + tpc - 1) / tpc;
  if (launch_chunks > all_chunks) launch_chunks = all_chunks;  // whatever the settings ask for
  const size_t per_launch = tpc * launch_chunks;
  size_t side = shape.group_sources ? tunables().spread_launch_bytes / (tiles * tile * (size_t)(fp.P + 1)) : (size_t)nsrc;
  if (side < 1) side = 1;
  if (side > (size_t)nsrc) side = (size_t)nsrc;
  // sources of one group: as many as keep the group's chunk within 8 MiB
  size_t in_x = shape.group_sources ? ((size_t)8 << 20) / (tpc * tile) : 1;
  if (in_x < 1) in_x = 1;
  if (in_x > side) in_x = side;
  // a launch holds fewer than 2^32 threads in x
  if (2 * per_launch * (size_t)fp.P * in_x * kGatherThreads > 0xffffffffull || tiles > 0xffffffffull)
    return set_error(ALAMD_ERR_INVALID_ARG, "count too large for one launch");
  for (int q0 = 0; q0 < nsrc; q0 += (int)side) {
    const size_t here = (size_t)(nsrc - q0) < side ? (size_t)(nsrc - q0) : side;
    const unsigned ny = (unsigned)((here + in_x - 1) / in_x);
    // a remainder of less than half a launch rides with the launch before it
    for (size_t t0 = 0; t0 < tiles;) {
      const size_t nt = tiles - t0 < per_launch + per_launch / 2 ? tiles - t0 : per_launch;
      const size_t chunks = (nt + tpc - 1) / tpc;
      hipLaunchKernelGGL(spread_kernel, dim3((unsigned)(chunks * tpc * (size_t)fp.P * in_x), ny, 1),
                         dim3(kGatherThreads, 1, 1), 0, stream, fp, (unsigned)tpc, (unsigned)t0, (unsigned)q0,
                         (unsigned)(q0 + here), (unsigned)in_x);
      t0 += nt;
    }
  }
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

}  // namespace

// from_hbm: the sources are slices that no launch has just written (an allgather).  Slices of one
// chunk (16 MiB) and more then get launches of their own, the smaller ones share one: one launch over
// several large slices is long enough for the XCDs to drift apart (32 MiB slices: 88 % of peak one by
// one, 83 % together; 8 MiB slices: 85 us together, 98 us one by one; 1 MiB: 15 us against 43 us).
// Otherwise the sources are what a fold has just written, and all of them share the launches.
int launch_spread_table(const FoldParams &fp, int nsrc, bool from_hbm, hipStream_t stream) {
  if (!from_hbm) return launch_spread_once(fp, nsrc, spread_from_cache(), stream);
  const size_t big = (size_t)spread_from_hbm().chunk_tiles * Tile<kGatherU, kGatherThreads>::BYTES;
  FoldParams rest = fp;
  for (int q = 0; q < nsrc && nsrc > 1; ++q) {
    if (fp.seg.seg_len[q] < big) continue;
    FoldParams one = fp;
    one.in[0] = fp.in[q];
    one.seg.seg_off[0] = fp.seg.seg_off[q];
    one.seg.seg_len[0] = fp.seg.seg_len[q];
    const int rc = launch_spread_once(one, 1, spread_from_hbm(), stream);
    if (rc) return rc;
    rest.seg.seg_len[q] = 0;
  }
  // The short slices share launches.  Equal ones (an allgather) go in rank order; unequal ones
  // (an allgatherv) longest first, in runs whose lengths differ by at most a factor of two, so that
  // a launch sized for its longest slice is not mostly workgroups with nothing to copy.
  int idx[ALAMD_MAX_RANKS], m = 0;
  for (int q = 0; q < nsrc; ++q)
    if (rest.seg.seg_len[q] > 0) idx[m++] = q;
  for (int i = 1; i < m; ++i) {  // insertion sort, stable
    const int o = idx[i];
    int k = i;
    for (; k > 0 && rest.seg.seg_len[idx[k - 1]] < rest.seg.seg_len[o]; --k) idx[k] = idx[k - 1];
    idx[k] = o;
  }
  for (int i0 = 0; i0 < m;) {
    FoldParams run = fp;
    int n = 0;
    const size_t longest = rest.seg.seg_len[idx[i0]];
    while (i0 + n < m && 2 * rest.seg.seg_len[idx[i0 + n]] >= longest) {
      const int q = idx[i0 + n];
      run.in[n] = fp.in[q];
      run.seg.seg_off[n] = fp.seg.seg_off[q];
      run.seg.seg_len[n] = fp.seg.seg_len[q];
      ++n;
    }
    const int rc = launch_spread_once(run, n, spread_from_hbm(), stream);
    if (rc) return rc;
    i0 += n;
  }
  return ALAMD_OK;
}

int launch_spread(const char *src, char *const *dests, int ndest, size_t bytes, hipStream_t stream) {
  if (ndest <= 0 || bytes == 0) return ALAMD_OK;
  FoldParams fp;
  fp.seg = make_seg(0, 0, 0, OUT_ALL, 0);
  for (int r = 0; r < ALAMD_MAX_RANKS; ++r) {
    fp.in[r] = nullptr;
    fp.out[r] = r < ndest ? dests[r] : nullptr;
  }
  fp.in[0] = src;
  fp.P = ndest;
  fp.seg.seg_len[0] = bytes;
  return launch_spread_table(fp, 1, false, stream);
}

namespace {

// Copies slice q (lens[q] bytes at sends[q]) to byte offset offs[q] of every recvs[r].
int launch_gather(void *const *recvs, const void *const *sends, int P, const size_t *offs, const size_t *lens,
                  hipStream_t stream) {
  FoldParams fp;
  fp.seg = make_seg(0, 0, 0, OUT_ALL, 0);
  fp.P = P;
  for (int r = 0; r < ALAMD_MAX_RANKS; ++r) {
    fp.in[r] = r < P ? static_cast<const char *>(sends[r]) : nullptr;
    fp.out[r] = r < P ? static_cast<char *>(recvs[r]) : nullptr;
  }
  for (int q = 0; q < P; ++q) {
    fp.seg.seg_off[q] = offs[q];
    fp.seg.seg_len[q] = lens[q];
  }
  return launch_spread_table(fp, P, true, stream);
}

}  // namespace

namespace {

// The in-place part of Reduce_scatterv, in ascending block order.  Block b's result overwrites
// elements [0, counts[b]) of rank b's buffer, which block k reads (from every rank's buffer) if
// displ[k] < counts[b]; only blocks k <= b can.  Consecutive blocks among which no such pair
// exists share one launch (with equal counts: block 0, then all the others, like Reduce_scatter);
// a block that overlaps its own input - in place and 0 < displ < count: it reads its rank's
// elements displ + i while it writes element i of the same buffer - goes alone, as a chained launch
// (see ChainParams), with scratch from `fixed` if given, else from the pool of the stream.
int reduce_scatterv_in_place(void *const *recvs, const void *const *sends, int P, const size_t *counts,
                             const size_t *displ, int dtype, int op, int order, hipStream_t stream,
                             const ChainScratch *fixed) {
  const size_t es = alamd_dtype_size(dtype);
  auto overlaps_itself = [&](int k) {
    return recvs[k] == sends[k] && displ[k] != 0 && displ[k] < counts[k];
  };
  for (int b = 0; b < P;) {
    if (counts[b] == 0) { ++b; continue; }
    const bool overlapped = overlaps_itself(b);
    if (!overlapped) {
      // the blocks that can go with block b
      int members[ALAMD_MAX_RANKS], n = 0, j = b + 1;
      members[n++] = b;
      for (; j < P; ++j) {
        if (counts[j] == 0) continue;
        if (overlaps_itself(j)) break;
        bool safe = true;
        if (recvs[j] == sends[j])
          for (int m = 0; m < n; ++m) safe = safe && displ[members[m]] >= counts[j];
        if (!safe) break;
        members[n++] = j;
      }
      if (n > 1) {
        Layout lay;
        lay.nseg = (unsigned)P;
        lay.seg = make_seg(0, 0, 1, OUT_SEG, 1);
        lay.seg.ragged = 1;
        void *out_tab[ALAMD_MAX_RANKS] = {nullptr};
        size_t longest = 0;
        for (int m = 0; m < n; ++m) {
          const int k = members[m];
          lay.seg.seg_off[k] = displ[k];
          lay.seg.seg_len[k] = counts[k];
          out_tab[k] = recvs[k];
          if (counts[k] > longest) longest = counts[k];
        }
        for (int k = 0; k < P; ++k)
          if (!out_tab[k]) out_tab[k] = recvs[k] ? recvs[k] : const_cast<void *>(sends[0]);  // never written: length 0
        lay.max_len = longest;
        lay.start0 = 0;
        lay.start_stride = order_start_per_block(order) ? 1 : 0;
        const int rc = launch_order(out_tab, sends, P, lay, dtype, op, order, stream);
        if (rc) return rc;
        b = j;
        continue;
      }
    }
    // One or two runs no longer than the displacement, each launched after the one before it, never read
    // what an unfinished launch writes; beyond that one chained launch (85 to 100 % of the ordinary rate at
    // P = 8) beats a train of launches.  With the fixed scratch too small for the block, up to kMaxRuns
    // plain launches stand in.
    constexpr size_t kMaxRuns = 32;
    const size_t runs = overlapped ? (counts[b] + displ[b] - 1) / displ[b] : 1;
    bool chained = runs > 2;
    if (chained && fixed && runs <= kMaxRuns &&
        (counts[b] * es + kChainMinTileBytes - 1) / kChainMinTileBytes > fixed->max_tiles)
      chained = false;
    const size_t run = overlapped && !chained ? displ[b] : counts[b];
    int rc = ALAMD_OK;
    for (size_t done = 0; done < counts[b] && rc == ALAMD_OK; done += run) {
      const size_t n = counts[b] - done < run ? counts[b] - done : run;
      const void *ins[ALAMD_MAX_RANKS];
      void *out_tab[ALAMD_MAX_RANKS] = {nullptr};
      for (int r = 0; r < P; ++r) ins[r] = static_cast<const char *>(sends[r]) + (displ[b] + done) * es;
      out_tab[0] = static_cast<char *>(recvs[b]) + done * es;
      Layout lay;
      lay.nseg = 1;
      lay.seg = make_seg(n, 0, 0, OUT_ALL, 1);
      lay.max_len = n;
      lay.start0 = order_start_per_block(order) ? b : 0;
      lay.start_stride = 0;
      lay.msg_base = done;
      lay.msg_count = counts[b];
      if (chained) {
        ChainScratch cs;
        const size_t tiles = (n * es + kChainMinTileBytes - 1) / kChainMinTileBytes;
        if (fixed) {
          cs = *fixed;
          if (tiles > cs.max_tiles)
            return set_error(ALAMD_ERR_INVALID_ARG,
                             "in-place block %d of %zu bytes is beyond the %zu bytes the fixed scratch covers", b,
                             n * es, cs.max_tiles * kChainMinTileBytes);
        } else if ((rc = chain_scratch_for(stream, tiles, true, cs))) {
          return rc;
        }
        rc = launch_order(out_tab, ins, P, lay, dtype, op, order, stream, &cs, displ[b] * es);
        if (rc == ALAMD_OK && fixed) rc = static_scratch_used(stream);
      } else {
        rc = launch_order(out_tab, ins, P, lay, dtype, op, order, stream);
      }
    }
    if (rc) return rc;
    ++b;
  }
  return ALAMD_OK;
}

}  // namespace

}  // namespace alamd

using namespace alamd;

extern "C" {

int alamd_combine(void *const *outs, int nout, const void *const *ins, int P, size_t count, int dtype,
                  int op, int order, int start, void *stream) {
  int rc = check_common(P, count, dtype);
  if (rc) return rc;
  if ((rc = check_type_op(dtype, op))) return rc;
  if (!order_valid(order)) return set_error(ALAMD_ERR_INVALID_ALGO, "Invalid algorithm");
  if (nout < 1 || nout > ALAMD_MAX_RANKS)
    return set_error(ALAMD_ERR_INVALID_ARG, "number of outputs %d outside [1, %d]", nout, ALAMD_MAX_RANKS);
  if (start < 0 || start >= P || (start != 0 && !order_has_start(order)))
    return set_error(ALAMD_ERR_INVALID_ARG, "start rank %d invalid for this order", start);
  if (!outs || !ins) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  if (count == 0) return ALAMD_OK;
  const size_t es = alamd_dtype_size(dtype), bytes = count * es;
  for (int r = 0; r < P; ++r) {
    if (!ins[r]) return set_error(ALAMD_ERR_INVALID_ARG, "input %d is null", r);
    if (!aligned_to(ins[r], es)) return misaligned("input", r);
  }
  void *out_tab[ALAMD_MAX_RANKS] = {nullptr};
  for (int j = 0; j < nout; ++j) {
    if (!outs[j]) return set_error(ALAMD_ERR_INVALID_ARG, "output %d is null", j);
    if (!aligned_to(outs[j], es)) return misaligned("output", j);
    for (int r = 0; r < P; ++r)
      if (outs[j] != ins[r] && ranges_overlap(outs[j], bytes, ins[r], bytes))
        return set_error(ALAMD_ERR_OVERLAP, "output %d partially overlaps input %d", j, r);
    for (int k = 0; k < j; ++k)
      if (ranges_overlap(outs[j], bytes, outs[k], bytes))
        return set_error(ALAMD_ERR_OVERLAP, "outputs %d and %d overlap", k, j);
    out_tab[j] = outs[j];
  }
  Layout lay;
  lay.nseg = 1;
  lay.seg = make_seg(count, 0, 0, OUT_ALL, nout);
  lay.max_len = count;
  lay.start0 = start;
  lay.start_stride = 0;
  if ((size_t)nout < tunables().two_step_min_outputs || bytes * (size_t)nout < tunables().two_step_min_total_bytes)
    return launch_order(out_tab, ins, P, lay, dtype, op, order, as_stream(stream));
  // Several outputs of a large result: a workgroup that wrote its tile to every
  // output would interleave nout write streams (measured 69 % of peak).  Instead
  // the result goes to outs[0] and is then spread from there, piece by piece.
  // In place (outs[j] == ins[j]) this is safe: a piece of the inputs is
  // overwritten by a launch that follows the fold of that piece on the same
  // stream, and no other piece reads it.
  const size_t piece = bytes > 2 * tunables().two_step_piece_bytes ? tunables().two_step_piece_bytes / es : count;
  for (size_t e0 = 0, n; e0 < count; e0 += n) {
    n = count - e0 < piece + piece / 2 ? count - e0 : piece;  // no short last piece
    Layout pl = lay;
    pl.seg = make_seg(n, 0, 0, OUT_ALL, 1);
    pl.max_len = n;
    pl.msg_base = e0;
    pl.msg_count = count;
    void *first[ALAMD_MAX_RANKS] = {nullptr};
    first[0] = static_cast<char *>(outs[0]) + e0 * es;
    const void *pin[ALAMD_MAX_RANKS];
    for (int r = 0; r < P; ++r) pin[r] = static_cast<const char *>(ins[r]) + e0 * es;
    if ((rc = launch_order(first, pin, P, pl, dtype, op, order, as_stream(stream)))) return rc;
    char *dests[ALAMD_MAX_RANKS];
    for (int j = 1; j < nout; ++j) dests[j - 1] = static_cast<char *>(outs[j]) + e0 * es;
    if ((rc = launch_spread(static_cast<const char *>(first[0]), dests, nout - 1, n * es, as_stream(stream)))) return rc;
  }
  return ALAMD_OK;
}

int alamd_reduce_scatter(void *const *recvs, const void *const *sends, int P, size_t count, int dtype,
                         int op, int order, void *stream) {
  int rc = check_common(P, count, dtype);
  if (rc) return rc;
  if ((rc = check_type_op(dtype, op))) return rc;
  if (!order_valid(order)) return set_error(ALAMD_ERR_INVALID_ALGO, "Invalid algorithm");
  if (!recvs || !sends) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  if (count == 0) return ALAMD_OK;
  const size_t es = alamd_dtype_size(dtype), blk = count * es, total = blk * (size_t)P;
  bool inplace = false;
  void *out_tab[ALAMD_MAX_RANKS] = {nullptr};
  for (int r = 0; r < P; ++r) {
    if (!sends[r] || !recvs[r]) return set_error(ALAMD_ERR_INVALID_ARG, "buffer %d is null", r);
    if (!aligned_to(sends[r], es) || !aligned_to(recvs[r], es)) return misaligned("buffer", r);
    out_tab[r] = recvs[r];
  }
  for (int b = 0; b < P; ++b) {
    for (int r = 0; r < P; ++r) {
      if (recvs[b] == sends[r] && b == r) { inplace = true; continue; }
      if (ranges_overlap(recvs[b], blk, sends[r], total))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffer %d overlaps send buffer %d", b, r);
    }
    for (int k = 0; k < b; ++k)
      if (ranges_overlap(recvs[b], blk, recvs[k], blk))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffers %d and %d overlap", k, b);
  }
  Layout lay;
  lay.seg = make_seg(count, 0, 1, OUT_SEG, 1);
  lay.max_len = count;
  lay.start0 = 0;
  lay.start_stride = order_start_per_block(order) ? 1 : 0;
  if (!inplace || P == 1) {
    lay.nseg = (unsigned)P;
    return launch_order(out_tab, sends, P, lay, dtype, op, order, as_stream(stream));
  }
  // In place every result lands on block 0 of its own send buffer, which
  // block 0's fold still has to read: fold block 0 first (it overwrites only
  // what its own lanes have read), then the other blocks.
  lay.nseg = 1;
  rc = launch_order(out_tab, sends, P, lay, dtype, op, order, as_stream(stream));
  if (rc) return rc;
  // blocks 1..P-1: shift the tables by one block
  const void *in_shift[ALAMD_MAX_RANKS];
  void *out_shift[ALAMD_MAX_RANKS] = {nullptr};
  for (int r = 0; r < P; ++r) in_shift[r] = static_cast<const char *>(sends[r]) + blk;
  for (int b = 1; b < P; ++b) out_shift[b - 1] = recvs[b];
  lay.nseg = (unsigned)(P - 1);
  lay.start0 = order_start_per_block(order) ? 1 : 0;
  return launch_order(out_shift, in_shift, P, lay, dtype, op, order, as_stream(stream));
}

int alamd_allgather(void *const *recvs, const void *const *sends, int P, size_t count, int dtype,
                    void *stream) {
  int rc = check_common(P, count, dtype);
  if (rc) return rc;
  if (!recvs || !sends) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  if (count == 0) return ALAMD_OK;
  const size_t es = alamd_dtype_size(dtype), blk = count * es;
  for (int r = 0; r < P; ++r)
    if (!sends[r] || !recvs[r]) return set_error(ALAMD_ERR_INVALID_ARG, "buffer %d is null", r);
  for (int r = 0; r < P; ++r) {
    for (int q = 0; q < P; ++q) {
      const char *slot = static_cast<const char *>(recvs[r]) + (size_t)q * blk;
      if (r == q && sends[q] == slot) continue;  // in place
      if (ranges_overlap(recvs[r], blk * (size_t)P, sends[q], blk))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffer %d overlaps send buffer %d", r, q);
    }
    for (int k = 0; k < r; ++k)
      if (ranges_overlap(recvs[r], blk * (size_t)P, recvs[k], blk * (size_t)P))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffers %d and %d overlap", k, r);
  }
  size_t offs[ALAMD_MAX_RANKS], lens[ALAMD_MAX_RANKS];
  for (int q = 0; q < P; ++q) { offs[q] = (size_t)q * blk; lens[q] = blk; }
  return launch_gather(recvs, sends, P, offs, lens, as_stream(stream));
}

static int reduce_scatterv_impl(void *const *recvs, const void *const *sends, int P, const size_t *counts,
                               int dtype, int op, int order, void *stream, const ChainScratch *fixed) {
  if (take_expired())
    return set_error(ALAMD_ERR_TIMEOUT, "an earlier in-place Reduce_scatterv gave up waiting for a tile of its chained "
                                        "launch: its result is not valid (this call has done nothing)");
  int rc = check_common(P, 0, dtype);
  if (rc) return rc;
  if ((rc = check_type_op(dtype, op))) return rc;
  if (!order_valid(order)) return set_error(ALAMD_ERR_INVALID_ALGO, "Invalid algorithm");
  if (!recvs || !sends || !counts) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  const size_t es = alamd_dtype_size(dtype);
  size_t displ[ALAMD_MAX_RANKS + 1];
  displ[0] = 0;
  for (int b = 0; b < P; ++b) {
    if (counts[b] > (size_t)1 << 48) return set_error(ALAMD_ERR_INVALID_ARG, "count too large");
    displ[b + 1] = displ[b] + counts[b];
  }
  const size_t total = displ[P] * es;
  if (total == 0) return ALAMD_OK;
  for (int r = 0; r < P; ++r) {
    if (!sends[r]) return set_error(ALAMD_ERR_INVALID_ARG, "send buffer %d is null", r);
    if (!aligned_to(sends[r], es)) return misaligned("send buffer", r);
  }
  for (int b = 0; b < P; ++b) {
    if (counts[b] == 0) continue;
    if (!recvs[b]) return set_error(ALAMD_ERR_INVALID_ARG, "receive buffer %d is null", b);
    if (!aligned_to(recvs[b], es)) return misaligned("receive buffer", b);
    for (int r = 0; r < P; ++r) {
      if (b == r && recvs[b] == sends[r]) continue;  // in place
      if (ranges_overlap(recvs[b], counts[b] * es, sends[r], total))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffer %d overlaps send buffer %d", b, r);
    }
    for (int k = 0; k < b; ++k)
      if (counts[k] && ranges_overlap(recvs[b], counts[b] * es, recvs[k], counts[k] * es))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffers %d and %d overlap", k, b);
  }
  bool any_inplace = false;
  size_t max_count = 0;
  for (int b = 0; b < P; ++b) {
    any_inplace = any_inplace || (counts[b] && recvs[b] == sends[b]);
    if (counts[b] > max_count) max_count = counts[b];
  }
  if (!any_inplace) {
    // separate receive buffers: all blocks in one launch, one segment per block
    Layout lay;
    lay.nseg = (unsigned)P;
    lay.seg = make_seg(0, 0, 1, OUT_SEG, 1);
    lay.seg.ragged = 1;
    void *out_tab[ALAMD_MAX_RANKS] = {nullptr};
    for (int b = 0; b < P; ++b) {
      lay.seg.seg_off[b] = displ[b];
      lay.seg.seg_len[b] = counts[b];
      out_tab[b] = recvs[b];
    }
    lay.max_len = max_count;
    lay.start0 = 0;
    lay.start_stride = order_start_per_block(order) ? 1 : 0;
    return launch_order(out_tab, sends, P, lay, dtype, op, order, as_stream(stream));
  }
  return reduce_scatterv_in_place(recvs, sends, P, counts, displ, dtype, op, order, as_stream(stream), fixed);
}

int alamd_reduce_scatterv(void *const *recvs, const void *const *sends, int P, const size_t *counts, int dtype,
                          int op, int order, void *stream) {
  return reduce_scatterv_impl(recvs, sends, P, counts, dtype, op, order, stream, nullptr);
}

int alamd_reduce_scatterv_noalloc(void *const *recvs, const void *const *sends, int P, const size_t *counts,
                                  int dtype, int op, int order, void *stream) {
  ChainScratch cs;
  const int rc = static_chain_scratch(as_stream(stream), cs);
  if (rc) return rc;
  return reduce_scatterv_impl(recvs, sends, P, counts, dtype, op, order, stream, &cs);
}

int alamd_reduce_scatterv_wait_expired(void) { return take_expired() ? 1 : 0; }

int alamd_set_chain_poll_limit(unsigned polls) {
  g_chain_polls.store(polls == ALAMD_CHAIN_POLLS_NONE ? 0u : polls ? polls : kChainDefaultPolls);
  return ALAMD_OK;
}

size_t alamd_planned_launches(int P, size_t count, int dtype) {
  const size_t es = alamd_dtype_size(dtype);
  if (P < 1 || P > ALAMD_MAX_RANKS || es == 0 || count == 0) return 0;
  // the planner of the fold kernels, run without launching anything
  const size_t kTileBytes = use_block_shape(count * es * (size_t)(P + 1), P, 1, false, (count * es + kBlockTileBytes - 1) / kBlockTileBytes, 256)
                                ? kBlockTileBytes : kStreamTileBytes;  // (as on a device with 256 CUs: no device is asked here)
  SegParams seg = make_seg(count, 0, 0, OUT_ALL, 1);
  size_t launches = 0;
  plan_launches(seg, 1, count, kTileBytes / es, launch_tiles(P, kTileBytes, tunables().launch_bytes),
                [&](size_t, size_t, unsigned, unsigned) { ++launches; });
  return launches;
}

int alamd_reserve_scratch(void *stream, size_t max_block_bytes) {
  if (max_block_bytes == 0) return ALAMD_OK;
  ChainScratch cs;
  const size_t tiles = (max_block_bytes + kChainMinTileBytes - 1) / kChainMinTileBytes;
  return chain_scratch_for(as_stream(stream), tiles, true, cs);
}

int alamd_release_scratch(void *stream) {
  int dev = 0;
  ALAMD_HIP(hipGetDevice(&dev));
  ALAMD_HIP(hipStreamSynchronize(as_stream(stream)));
  ChainPool &pool = chain_pool();
  std::lock_guard<std::mutex> lock(pool.mutex);
  const auto key = std::make_pair(dev, as_stream(stream));
  auto it = pool.live.find(key);
  if (it != pool.live.end()) {
    ALAMD_HIP(hipFree(it->second.ticket));
    pool.live.erase(it);
  }
  auto old = pool.retired.find(key);
  if (old != pool.retired.end()) {
    for (void *mem : old->second) ALAMD_HIP(hipFree(mem));
    pool.retired.erase(old);
  }
  return ALAMD_OK;
}

int alamd_allgatherv(void *const *recvs, const void *const *sends, int P, const size_t *counts,
                     const size_t *displs, int dtype, void *stream) {
  int rc = check_common(P, 0, dtype);
  if (rc) return rc;
  if (!recvs || !sends || !counts || !displs) return set_error(ALAMD_ERR_INVALID_ARG, "null pointer table");
  const size_t es = alamd_dtype_size(dtype);
  size_t extent = 0;  // elements a receive buffer must hold
  for (int q = 0; q < P; ++q) {
    if (counts[q] > (size_t)1 << 48 || displs[q] > (size_t)1 << 48)
      return set_error(ALAMD_ERR_INVALID_ARG, "count or displacement too large");
    if (counts[q] && displs[q] + counts[q] > extent) extent = displs[q] + counts[q];
    for (int k = 0; k < q; ++k)
      if (counts[q] && counts[k] && displs[q] < displs[k] + counts[k] && displs[k] < displs[q] + counts[q])
        return set_error(ALAMD_ERR_OVERLAP, "slices %d and %d overlap in the receive buffer", k, q);
  }
  if (extent == 0) return ALAMD_OK;
  for (int r = 0; r < P; ++r) {
    if (!recvs[r]) return set_error(ALAMD_ERR_INVALID_ARG, "receive buffer %d is null", r);
    for (int q = 0; q < P; ++q) {
      if (counts[q] == 0) continue;
      if (!sends[q]) return set_error(ALAMD_ERR_INVALID_ARG, "send buffer %d is null", q);
      const char *slot = static_cast<const char *>(recvs[r]) + displs[q] * es;
      if (r == q && sends[q] == slot) continue;  // in place
      if (ranges_overlap(recvs[r], extent * es, sends[q], counts[q] * es))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffer %d overlaps send buffer %d", r, q);
    }
    for (int k = 0; k < r; ++k)
      if (ranges_overlap(recvs[r], extent * es, recvs[k], extent * es))
        return set_error(ALAMD_ERR_OVERLAP, "receive buffers %d and %d overlap", k, r);
  }
  size_t offs[ALAMD_MAX_RANKS], lens[ALAMD_MAX_RANKS];
  for (int q = 0; q < P; ++q) { offs[q] = displs[q] * es; lens[q] = counts[q] * es; }
  return launch_gather(recvs, sends, P, offs, lens, as_stream(stream));
}

}  // extern "C"
