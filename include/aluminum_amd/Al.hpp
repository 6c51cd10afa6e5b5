/*
 * Aluminum-shaped C++ front end of the aluminum_amd combine engine.
 *
 * Header-only.  It gives the on-device engine the interface a backend policy
 * class has in the reference, so that
 *
 *     Al::Allreduce<Al::HipCombineBackend>(buf, count, Al::ReductionOperator::sum, comm);
 *
 * compiles and behaves as `Al::Allreduce<Al::HostTransferBackend>` does
 * (reference: include/Al.hpp:118-207, 222-421, 550-633, 1866-1883;
 * include/aluminum/ht_impl.hpp:125-195, 303-343, 866-904, 1113-1138), with the
 * host round trip (D2H copy, MPI_Iallreduce on the host, H2D copy;
 * include/aluminum/ht/allreduce.hpp:41-79) replaced by one kernel launch.
 *
 * One GPU holds all P logical ranks.  A `World` owns the P communicators; a
 * collective is launched when the last of the P logical ranks has made its
 * call (calls may come from one thread in any rank order, or from P threads).
 * Every call only enqueues work and returns (docs/index.rst:33-40).  Errors
 * are thrown as Al::al_exception from the calling thread.
 *
 * Stream order.  The collective starts after everything that was enqueued on
 * rank r's stream before rank r's call (the dependency is taken at the call),
 * and everything enqueued on a rank's stream after the LAST of the P calls
 * runs after the collective.  Work enqueued on a rank's stream between that
 * rank's call and the last call is not ordered against the collective: it
 * must not write the rank's send buffer or touch its receive buffer.  With P
 * processes that window does not exist; with P logical ranks in one process
 * it does, because the combine cannot be enqueued before every contribution
 * is known, and a stream cannot be made to wait for work that is enqueued
 * later without risking a deadlock on a shared hardware queue.  Callers that
 * drive the ranks from P threads can close the window with
 * World::set_calls_wait_for_launch(true): a call then returns when the
 * collective has been launched, so whatever the thread enqueues next is
 * ordered behind it.
 *
 * Needs the HIP host API (hip/hip_runtime_api.h) and libaluminum_amd.so.
 */
#ifndef ALUMINUM_AMD_AL_HPP
#define ALUMINUM_AMD_AL_HPP

#include <hip/hip_runtime_api.h>

#include <atomic>
#include <cstddef>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <deque>
#include <exception>
#include <functional>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <thread>
#include <type_traits>
#include <vector>

#include "aluminum_amd.h"

// Two ways to use this header.  On its own it is a front end of the reference's shape: it defines
// Al::al_exception, Al::ReductionOperator, Al::AlOperation, the trait templates and the Al::Allreduce /
// Reduce / Reduce_scatter(v) / Allgather(v) / Test / Wait templates itself.  With AL_AMD_WITH_REFERENCE
// defined it is one more backend inside the reference: it is included after the reference's own
// declarations (the way include/Al.hpp:2005-2014 includes the other backends), defines none of those
// and only adds Al::HipCombineBackend, its traits and its Test / Wait specialisations.
#ifdef AL_AMD_WITH_REFERENCE
#include "aluminum/base.hpp"
#include "aluminum/traits/traits_base.hpp"
#endif

namespace Al {

#ifndef AL_AMD_WITH_REFERENCE
/** Same text layout as the reference's exception (include/aluminum/base.hpp:52-70). */
class al_exception : public std::exception {
 public:
  al_exception(const std::string m, const std::string f, const int l) : msg(m), file(f), line(l) {
    err = file + ":" + std::to_string(line) + " - " + msg;
  }
  const char *what() const noexcept override { return err.c_str(); }

 private:
  const std::string msg;
  const std::string file;
  const int line;
  std::string err;
};
#endif
#define AL_AMD_THROW(s) throw ::Al::al_exception((s), __FILE__, __LINE__)
#define AL_AMD_CHECK(call)                                                   \
  do {                                                                       \
    if ((call) != ALAMD_OK) AL_AMD_THROW(std::string(alamd_last_error()));   \
  } while (0)
#define AL_AMD_CHECK_HIP(call)                                               \
  do {                                                                       \
    hipError_t al_amd_e_ = (call);                                           \
    if (al_amd_e_ != hipSuccess)                                             \
      AL_AMD_THROW(std::string("GPU error: ") + hipGetErrorString(al_amd_e_)); \
  } while (0)

#ifndef AL_AMD_WITH_REFERENCE
/** Predefined reduction operations (include/aluminum/base.hpp:103-105). */
enum class ReductionOperator { sum, prod, min, max, lor, land, lxor, bor, band, bxor, avg };

namespace amd {
inline bool &initialized_flag() {
  static bool flag = false;
  return flag;
}
}  // namespace amd

/** Start-up as in the reference (include/Al.hpp:73-104); there is no MPI to
 *  initialise, so the arguments are unused.  Checks that the current device is a
 *  gfx950.  May be called more than once. */
inline void Initialize(int & /*argc*/, char **& /*argv*/) {
  AL_AMD_CHECK(alamd_init());
  amd::initialized_flag() = true;
}
inline void Finalize() { amd::initialized_flag() = false; }
inline bool Initialized() { return amd::initialized_flag(); }
#endif
// The C ABI numbers its operators like the reference, so the front end casts.
static_assert(static_cast<int>(ReductionOperator::sum) == ALAMD_SUM && static_cast<int>(ReductionOperator::prod) == ALAMD_PROD &&
                  static_cast<int>(ReductionOperator::min) == ALAMD_MIN && static_cast<int>(ReductionOperator::max) == ALAMD_MAX &&
                  static_cast<int>(ReductionOperator::lor) == ALAMD_LOR && static_cast<int>(ReductionOperator::land) == ALAMD_LAND &&
                  static_cast<int>(ReductionOperator::lxor) == ALAMD_LXOR && static_cast<int>(ReductionOperator::bor) == ALAMD_BOR &&
                  static_cast<int>(ReductionOperator::band) == ALAMD_BAND && static_cast<int>(ReductionOperator::bxor) == ALAMD_BXOR &&
                  static_cast<int>(ReductionOperator::avg) == ALAMD_AVG,
              "ReductionOperator and alamd_op must agree");

namespace amd {

/** 16-bit float carriers for builds without the HIP half / bfloat16 headers. */
struct half_bits { uint16_t bits; };
struct bfloat16_bits { uint16_t bits; };

/** C++ type -> library dtype (the types of mpi::TypeMap, include/aluminum/mpi/utils.hpp:43-67). */
template <typename T> struct TypeMap;
#define AL_AMD_TYPEMAP(T, D) \
  template <> struct TypeMap<T> { static constexpr int value = D; }
AL_AMD_TYPEMAP(char, (static_cast<char>(-1) < 0 ? ALAMD_I8 : ALAMD_U8));
AL_AMD_TYPEMAP(signed char, ALAMD_I8);
AL_AMD_TYPEMAP(unsigned char, ALAMD_U8);
AL_AMD_TYPEMAP(short, ALAMD_I16);
AL_AMD_TYPEMAP(unsigned short, ALAMD_U16);
AL_AMD_TYPEMAP(int, ALAMD_I32);
AL_AMD_TYPEMAP(unsigned int, ALAMD_U32);
AL_AMD_TYPEMAP(long, (sizeof(long) == 8 ? ALAMD_I64 : ALAMD_I32));
AL_AMD_TYPEMAP(unsigned long, (sizeof(long) == 8 ? ALAMD_U64 : ALAMD_U32));
AL_AMD_TYPEMAP(long long, ALAMD_I64);
AL_AMD_TYPEMAP(unsigned long long, ALAMD_U64);
AL_AMD_TYPEMAP(float, ALAMD_F32);
AL_AMD_TYPEMAP(double, ALAMD_F64);
AL_AMD_TYPEMAP(half_bits, ALAMD_F16);
AL_AMD_TYPEMAP(bfloat16_bits, ALAMD_BF16);
#if defined(__clang__)
AL_AMD_TYPEMAP(_Float16, ALAMD_F16);
AL_AMD_TYPEMAP(__bf16, ALAMD_BF16);
#endif
#if defined(HIP_INCLUDE_HIP_AMD_DETAIL_HIP_FP16_H)
AL_AMD_TYPEMAP(__half, ALAMD_F16);
#endif
#if defined(_HIP_INCLUDE_HIP_AMD_DETAIL_HIP_BF16_H_)
AL_AMD_TYPEMAP(__hip_bfloat16, ALAMD_BF16);
#endif
#undef AL_AMD_TYPEMAP

/** Combine orders and ring modes a caller can ask for by name. */
enum class CombineAlgorithm {
  automatic,      /**< what the reference's host-transfer backend (and the non-blocking calls of its
                       MPI backend) yield with MPICH 3.3.2 on one host (alamd_reference_order):
                       Allreduce and Reduce - binomial tree to the root up to 2048 bytes and for
                       fp16 / bf16, reduce-scatter + gather above; Reduce_scatter(v) -
                       distance-halving tree below 512 KiB in total, descending pairwise fold from
                       there on */
  automatic_mpi_blocking,  /**< what the blocking calls of the reference's MPI backend yield there:
                       as `automatic`, except that MPI_Allreduce and MPI_Reduce cut a long message
                       into the blocks of tree_reduce_scatter_gather_spread */
  rank_order,     /**< ((x0 . x1) . x2) ... */
  tree_doubling,
  tree_halving,
  tree_binomial,  /**< to the root of a Reduce, to rank 0 otherwise */
  tree_reduce_scatter_gather,  /**< the doubling tree with the operand roles of a reduce-scatter by
                                    recursive halving of the data followed by a gather */
  tree_reduce_scatter_gather_spread,  /**< the same, with what the count is not a multiple of spread
                                    over the first blocks instead of left to the last one */
  pairwise,       /**< x_r . x_{r-1} . x_{r-2} ... for the block of rank r */
  ring,           /**< ring reduce-scatter + allgather, one launch per ring step */
  ring_fused      /**< the same values with every segment folded in one pass */
};

/** Chunk of the ring pipeline: 4 MiB, a multiple of every element size. */
inline size_t ring_chunk_bytes(size_t /*elem_size*/) { return static_cast<size_t>(4) << 20; }

class World;

/** A logical rank's communicator: rank, size and a stream
 *  (shape of internal::MPICommAndStreamWrapper,
 *  include/aluminum/mpi_comm_and_stream_wrapper.hpp:46-129). */
class Communicator {
 public:
  Communicator(const Communicator &) = delete;
  Communicator &operator=(const Communicator &) = delete;
  Communicator(Communicator &&) = default;

  int rank() const { return rank_; }
  int size() const { return size_; }
  int local_rank() const { return rank_; }
  int local_size() const { return size_; }
  hipStream_t get_stream() const { return stream_; }
  World &world() const { return *world_; }

 private:
  friend class World;
  Communicator(World *w, int r, int p, hipStream_t s) : world_(w), rank_(r), size_(p), stream_(s) {}
  World *world_;
  int rank_, size_;
  hipStream_t stream_;
  uint64_t next_seq_ = 0;
  friend struct Poster;
};

/** Timing-less events, reused: creating one costs more than recording it. */
class EventPool {
 public:
  ~EventPool() {
    for (hipEvent_t e : free_) (void)hipEventDestroy(e);
  }
  hipEvent_t take() {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      if (!free_.empty()) {
        hipEvent_t e = free_.back();
        free_.pop_back();
        return e;
      }
    }
    hipEvent_t e = nullptr;
    AL_AMD_CHECK_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    return e;
  }
  void give(hipEvent_t e) {
    std::lock_guard<std::mutex> lock(mutex_);
    free_.push_back(e);
  }

 private:
  std::mutex mutex_;
  std::vector<hipEvent_t> free_;
};

/** Completion of one launched non-blocking operation: one event, shared by
 *  the requests of all P logical ranks. */
struct OpCompletion {
  std::shared_ptr<EventPool> pool;
  hipEvent_t event = nullptr;
  hipStream_t ran_on = nullptr;  // work later on this stream is ordered behind the operation anyway
  std::mutex mutex;
  std::vector<hipStream_t> waited;  // streams already made to wait for this operation
  ~OpCompletion() {
    if (event) pool->give(event);
  }
  /** True the first time `s` asks: later waits of the same stream add nothing. */
  bool first_wait(hipStream_t s) {
    std::lock_guard<std::mutex> lock(mutex);
    for (hipStream_t w : waited)
      if (w == s) return false;
    waited.push_back(s);
    return true;
  }
};

/** Completion handle of a non-blocking operation
 *  (internal::ht::HostTransferRequest, include/aluminum/ht_impl.hpp:882-888).
 *  `done` is empty until the last logical rank has made its call. */
struct Request {
  enum { not_launched = 0, launched = 1, failed = 2 };
  // The thread that makes the last call of a collective launches it and publishes the outcome here:
  // `done` or `error` first, then `state` with release order.  Test and Wait, which any rank's thread
  // may call meanwhile, read `state` with acquire order and only then the field it names.
  std::atomic<int> state{not_launched};
  std::shared_ptr<OpCompletion> done;
  hipStream_t orig_stream = nullptr;
  std::string error;  // the launch of the operation failed: Test and Wait rethrow it
};

enum class OpKind { allreduce, reduce, reduce_scatter, allgather, reduce_scatterv, allgatherv };

/** What one logical rank contributed to one collective. */
struct Posting {
  const void *send = nullptr;
  void *recv = nullptr;
  hipStream_t stream = nullptr;
  std::shared_ptr<Request> req;  // non-blocking: the caller's request, completed at launch
  hipEvent_t ready = nullptr;    // recorded on `stream` at the call; of the ranks of one operation that
                                 // share a stream, the one that called last holds their common event
  bool posted = false;
};

struct PendingOp {
  uint64_t seq = 0;
  OpKind kind = OpKind::allreduce;
  int dtype = 0;
  size_t count = 0;
  ReductionOperator op = ReductionOperator::sum;
  CombineAlgorithm algo = CombineAlgorithm::automatic;
  int root = 0;
  bool nonblocking = false;
  int nposted = 0;
  std::vector<size_t> counts, displs;  // the *v collectives
  std::vector<Posting> ranks;
  bool launched = false;  // set (with `failure` on error) when the last rank has called
  std::string failure;
};

/** Non-blocking operations that move up to this many bytes in all run on the caller's stream: their
 *  kernels take less time (about 40 us at this size) than the 50 to 55 us that the two dependencies
 *  between streams cost which move an operation to the internal stream and back (measured with 8 ranks
 *  and 64 MiB each: blocking 95 / 168 us for a reduce / allreduce, non-blocking 150 / 226 us). */
constexpr size_t kInlineNonblockingMovedBytes = static_cast<size_t>(256) << 20;

/** The P logical ranks that live in one GPU's memory. */
class World {
 public:
  /** P communicators on one stream. */
  World(int P, hipStream_t stream) : World(std::vector<hipStream_t>(static_cast<size_t>(P > 0 ? P : 0), stream)) {}
  /** One stream per logical rank. */
  explicit World(const std::vector<hipStream_t> &streams) {
    const int P = static_cast<int>(streams.size());
    if (P < 1 || P > ALAMD_MAX_RANKS) AL_AMD_THROW("Cannot create a world with this many ranks");
    AL_AMD_CHECK(alamd_init());
    for (int r = 0; r < P; ++r) comms_.emplace_back(new Communicator(this, r, P, streams[static_cast<size_t>(r)]));
    // default priority on purpose: the internal stream only has to be a different stream
    AL_AMD_CHECK_HIP(hipStreamCreateWithFlags(&internal_stream_, hipStreamNonBlocking));
    AL_AMD_CHECK_HIP(hipEventCreateWithFlags(&sync_event_, hipEventDisableTiming));
    events_ = std::make_shared<EventPool>();
  }
  ~World() {
    for (Mail &m : mail_)
      for (hipEvent_t e : m.notified) events_->give(e);
    (void)hipStreamSynchronize(internal_stream_);
    (void)hipEventDestroy(sync_event_);
    (void)hipStreamDestroy(internal_stream_);
  }
  World(const World &) = delete;
  World &operator=(const World &) = delete;

  int size() const { return static_cast<int>(comms_.size()); }
  Communicator &comm(int r) { return *comms_.at(static_cast<size_t>(r)); }

  /** For callers that drive the logical ranks from P threads: a collective call returns only when
   *  the collective has been launched (when all P ranks have called), so that work the thread enqueues
   *  next on its stream is ordered behind it.  Must stay off when one thread makes the calls of several
   *  ranks: the first call would wait for ever. */
  void set_calls_wait_for_launch(bool on) {
    std::lock_guard<std::mutex> lock(mutex_);
    calls_wait_ = on;
  }

  /* ---- one-sided extension between logical ranks (include/aluminum/mpi_cuda/rma_self.hpp:37-71 for
   *      a rank and itself; rma_ipc.hpp:152-328 between ranks, whose handle exchange and notification
   *      messages become a table and events here, because every rank lives in this address space) ---- */

  /** Deposits `mine` for `peer` and returns what `peer` deposited for `me`. */
  void *attach(int me, int peer, void *mine);
  /** `me`'s stream has reached this point: the next rma_wait(peer, me) is ordered behind it. */
  void rma_notify(int me, int peer);
  /** Orders `me`'s stream behind the matching rma_notify of `peer`. */
  void rma_wait(int me, int peer);

  /** Registers rank's part of its next collective; launches every collective
   *  that has all P parts, in order. */
  void post(Communicator &c, OpKind kind, int dtype, const void *send, void *recv, size_t count,
            ReductionOperator op, CombineAlgorithm algo, int root, std::shared_ptr<Request> *req,
            const std::vector<size_t> *counts = nullptr, const std::vector<size_t> *displs = nullptr);

 private:
  void launch(PendingOp &p);
  /** The stream an operation runs on: blocking operations on rank 0's stream, non-blocking ones on
   *  the internal stream between the two synchronisations of ht_impl.hpp:866-888 - unless they are
   *  small: moving to another stream and back costs 50 us and more of dependencies between streams, more
   *  than their kernels could ever overlap with, so those run on rank 0's stream as well and only leave
   *  a completion event behind. */
  hipStream_t target_of(bool nonblocking, OpKind kind, int dtype, size_t count, const std::vector<size_t> &counts) {
    if (!nonblocking) return comms_[0]->get_stream();
    // bytes read and written by the kernels of the operation
    const size_t P = comms_.size();
    size_t total = 0;
    for (size_t c : counts) total += c;
    size_t elems = 0;
    switch (kind) {
    case OpKind::allreduce: elems = 2 * P * count; break;
    case OpKind::reduce: elems = (P + 1) * count; break;
    case OpKind::reduce_scatter: elems = (P + 1) * P * count; break;
    case OpKind::allgather: elems = (P + 1) * P * count; break;
    case OpKind::reduce_scatterv: elems = (P + 1) * total; break;
    case OpKind::allgatherv: elems = (P + 1) * total; break;
    }
    const bool on_internal = elems * alamd_dtype_size(dtype) > kInlineNonblockingMovedBytes;
    return on_internal ? internal_stream_ : comms_[0]->get_stream();
  }
  hipStream_t gather_streams(PendingOp &p, hipStream_t target);
  void release_streams(PendingOp &p, hipStream_t ran_on);

  std::vector<std::unique_ptr<Communicator>> comms_;
  std::deque<std::shared_ptr<PendingOp>> pending_;
  std::mutex mutex_;
  std::condition_variable launched_cv_;
  bool calls_wait_ = false;
  struct Mail {
    std::deque<hipEvent_t> notified;  // recorded by the sender, not yet waited for
    int waiting = 0;                  // waits the receiver made before the sender notified
    std::deque<void *> attached;      // buffers the sender has deposited for the receiver
  };
  std::vector<Mail> mail_;  // [from * P + to]
  Mail &mail(int from, int to) {
    if (mail_.empty()) mail_.resize(comms_.size() * comms_.size());
    return mail_[static_cast<size_t>(from) * comms_.size() + static_cast<size_t>(to)];
  }
  void check_peer(int peer) const {
    if (peer < 0 || peer >= size()) AL_AMD_THROW("Invalid peer rank");
  }
  hipStream_t internal_stream_ = nullptr;
  hipStream_t last_target_ = nullptr;  // where the latest operation ran
  bool any_launched_ = false;
  hipEvent_t sync_event_ = nullptr;
  std::shared_ptr<EventPool> events_;
};

struct Poster {
  static uint64_t peek_seq(const Communicator &c) { return c.next_seq_; }
  static uint64_t take_seq(Communicator &c) { return c.next_seq_++; }
};

inline void World::post(Communicator &c, OpKind kind, int dtype, const void *send, void *recv, size_t count,
                        ReductionOperator op, CombineAlgorithm algo, int root, std::shared_ptr<Request> *req,
                        const std::vector<size_t> *counts, const std::vector<size_t> *displs) {
  std::unique_lock<std::mutex> lock(mutex_);
  const int P = size();
  static const std::vector<size_t> none;
  const std::vector<size_t> &cv = counts ? *counts : none, &dv = displs ? *displs : none;
  if ((counts && cv.size() != static_cast<size_t>(P)) || (displs && dv.size() != static_cast<size_t>(P)))
    AL_AMD_THROW("Vector of counts or displacements is not communicator-sized");
  // Every check comes before the rank's sequence number is taken: a call that throws leaves the
  // communicator where it was, and the operations behind it are not held up.
  const uint64_t seq = Poster::peek_seq(c);
  std::shared_ptr<PendingOp> slot;
  for (auto &p : pending_)
    if (p->seq == seq) slot = p;
  if (slot && (slot->kind != kind || slot->dtype != dtype || slot->count != count || slot->op != op ||
               slot->algo != algo || slot->root != root || slot->nonblocking != (req != nullptr) ||
               slot->counts != cv || slot->displs != dv))
    AL_AMD_THROW("Logical ranks disagree on the arguments of a collective");
  // The dependency on the rank's stream is taken now, not when the last rank calls: the collective
  // waits for what was enqueued before this call, and for nothing that is enqueued after it.
  // Ranks that share a stream share one event, recorded again at each of their calls, so that it
  // stands for the latest of them.
  hipEvent_t ready = nullptr;
  if (c.get_stream() != target_of(req != nullptr, kind, dtype, count, cv)) {
    if (slot)
      for (Posting &other : slot->ranks)
        if (other.posted && other.stream == c.get_stream() && other.ready) {
          ready = other.ready;
          other.ready = nullptr;
        }
    if (!ready) ready = events_->take();
    const hipError_t e = hipEventRecord(ready, c.get_stream());
    if (e != hipSuccess) {
      events_->give(ready);
      AL_AMD_THROW(std::string("GPU error: ") + hipGetErrorString(e));
    }
  }
  if (!slot) {
    slot = std::make_shared<PendingOp>();
    pending_.push_back(slot);
    slot->seq = seq;
    slot->kind = kind;
    slot->dtype = dtype;
    slot->count = count;
    slot->op = op;
    slot->algo = algo;
    slot->root = root;
    slot->nonblocking = req != nullptr;
    slot->counts = cv;
    slot->displs = dv;
    slot->ranks.resize(static_cast<size_t>(P));
  }
  Poster::take_seq(c);
  Posting &me = slot->ranks[static_cast<size_t>(c.rank())];
  me.send = send;
  me.recv = recv;
  me.stream = c.get_stream();
  me.ready = ready;
  if (req) {
    // handed out now, "not launched yet" until the last logical rank has called
    *req = std::make_shared<Request>();
    (*req)->orig_stream = c.get_stream();
    me.req = *req;
  }
  me.posted = true;
  slot->nposted++;
  // launch in sequence order only: an operation never overtakes an earlier one
  std::string my_failure;
  while (!pending_.empty() && pending_.front()->nposted == P) {
    std::shared_ptr<PendingOp> done = pending_.front();
    pending_.pop_front();
    try {
      launch(*done);
    } catch (const std::exception &e) {
      // the ranks that have already returned learn of it through their requests (Test / Wait), or,
      // when calls wait for the launch, through the exception their own call throws
      done->failure = e.what();
      for (Posting &r : done->ranks)
        if (r.req) {
          r.req->error = done->failure;
          r.req->state.store(Request::failed, std::memory_order_release);
        }
    }
    for (Posting &r : done->ranks)
      if (r.ready) {
        events_->give(r.ready);
        r.ready = nullptr;
      }
    done->launched = true;
    if (done == slot) my_failure = done->failure;
    else if (!done->failure.empty() && my_failure.empty() && !calls_wait_) my_failure = done->failure;
  }
  launched_cv_.notify_all();
  if (calls_wait_ && !slot->launched) {
    launched_cv_.wait(lock, [&] { return slot->launched; });
    my_failure = slot->failure;
  }
  if (!my_failure.empty()) throw al_exception(my_failure, __FILE__, __LINE__);
}

inline void *World::attach(int me, int peer, void *mine) {
  check_peer(peer);
  if (peer == me) return mine;  // ConnectionSelf::attach_remote_buffer
  std::unique_lock<std::mutex> lock(mutex_);
  mail(me, peer).attached.push_back(mine);
  Mail &in = mail(peer, me);
  if (in.attached.empty()) {
    if (!calls_wait_) {
      mail(me, peer).attached.pop_back();  // a call that throws leaves nothing behind
      AL_AMD_THROW("AttachRemoteBuffer: the peer has not attached its buffer yet. All logical ranks share one "
                   "address space, so a peer's pointer can be given to Put as it is; the exchange itself needs "
                   "one thread per rank and World::set_calls_wait_for_launch(true)");
    }
    launched_cv_.wait(lock, [&] { return !in.attached.empty(); });
  }
  void *theirs = in.attached.front();
  in.attached.pop_front();
  launched_cv_.notify_all();
  return theirs;
}

inline void World::rma_notify(int me, int peer) {
  check_peer(peer);
  const hipStream_t mine = comm(me).get_stream(), theirs = comm(peer).get_stream();
  if (mine == theirs) return;  // one stream: its own order is the notification (ConnectionSelf::notify)
  std::lock_guard<std::mutex> lock(mutex_);
  hipEvent_t ev = events_->take();
  const hipError_t e = hipEventRecord(ev, mine);
  if (e != hipSuccess) {
    events_->give(ev);
    AL_AMD_THROW(std::string("GPU error: ") + hipGetErrorString(e));
  }
  Mail &m = mail(me, peer);
  if (m.waiting > 0) {
    // the receiver has already asked: from here on its stream is behind this point
    --m.waiting;
    const hipError_t w = hipStreamWaitEvent(theirs, ev, 0);
    events_->give(ev);
    if (w != hipSuccess) AL_AMD_THROW(std::string("GPU error: ") + hipGetErrorString(w));
  } else {
    m.notified.push_back(ev);
  }
  launched_cv_.notify_all();
}

inline void World::rma_wait(int me, int peer) {
  check_peer(peer);
  const hipStream_t mine = comm(me).get_stream(), theirs = comm(peer).get_stream();
  if (mine == theirs) return;  // ConnectionSelf::wait
  std::unique_lock<std::mutex> lock(mutex_);
  Mail &m = mail(peer, me);
  if (m.notified.empty() && calls_wait_) launched_cv_.wait(lock, [&] { return !m.notified.empty(); });
  if (m.notified.empty()) {
    ++m.waiting;  // the notification orders the stream when it comes (see the note on stream order above)
    return;
  }
  hipEvent_t ev = m.notified.front();
  m.notified.pop_front();
  const hipError_t w = hipStreamWaitEvent(mine, ev, 0);
  events_->give(ev);
  if (w != hipSuccess) AL_AMD_THROW(std::string("GPU error: ") + hipGetErrorString(w));
}

/** Makes `target` wait for what each rank's stream held when that rank made its call; returns it. */
inline hipStream_t World::gather_streams(PendingOp &p, hipStream_t target) {
  for (Posting &r : p.ranks) {
    // one event per distinct stream; a rank on the target stream itself needs none (stream order)
    if (r.ready && r.stream != target) AL_AMD_CHECK_HIP(hipStreamWaitEvent(target, r.ready, 0));
  }
  return target;
}

/** Makes every rank's stream wait for what ran on `ran_on` (blocking ops), or
 *  hands out completion events (non-blocking ops). */
inline void World::release_streams(PendingOp &p, hipStream_t ran_on) {
  if (p.nonblocking) {
    auto done = std::make_shared<OpCompletion>();
    done->pool = events_;
    done->event = events_->take();
    done->ran_on = ran_on;
    AL_AMD_CHECK_HIP(hipEventRecord(done->event, ran_on));
    for (auto &r : p.ranks) {
      r.req->done = done;
      r.req->state.store(Request::launched, std::memory_order_release);
    }
    return;
  }
  bool recorded = false;
  for (size_t i = 0; i < p.ranks.size(); ++i) {
    const hipStream_t s = p.ranks[i].stream;
    bool seen = s == ran_on;
    for (size_t k = 0; k < i && !seen; ++k) seen = p.ranks[k].stream == s;
    if (seen) continue;
    if (!recorded) {
      AL_AMD_CHECK_HIP(hipEventRecord(sync_event_, ran_on));
      recorded = true;
    }
    AL_AMD_CHECK_HIP(hipStreamWaitEvent(s, sync_event_, 0));
  }
}

inline void World::launch(PendingOp &p) {
  const int P = size();
  const size_t es = alamd_dtype_size(p.dtype);
  hipStream_t target = target_of(p.nonblocking, p.kind, p.dtype, p.count, p.counts);
  // Operations are launched in sequence order; one that runs on another stream than the one before
  // it waits for that one, so that it sees its results whatever the ranks' events were taken before.
  if (last_target_ != nullptr && last_target_ != target) {
    AL_AMD_CHECK_HIP(hipEventRecord(sync_event_, last_target_));
    AL_AMD_CHECK_HIP(hipStreamWaitEvent(target, sync_event_, 0));
  }
  last_target_ = target;
  gather_streams(p, target);
  std::vector<const void *> sends(static_cast<size_t>(P));
  std::vector<void *> recvs(static_cast<size_t>(P));
  for (int r = 0; r < P; ++r) {
    sends[static_cast<size_t>(r)] = p.ranks[static_cast<size_t>(r)].send;
    recvs[static_cast<size_t>(r)] = p.ranks[static_cast<size_t>(r)].recv;
  }
  const int op = static_cast<int>(p.op);
  int rc = ALAMD_OK;
  switch (p.kind) {
  case OpKind::allreduce:
  case OpKind::reduce: {
    const bool rooted = p.kind == OpKind::reduce;
    int order = ALAMD_ORDER_RANK_ASC, start = 0;
    bool ring = false;
    switch (p.algo) {
    case CombineAlgorithm::automatic:
      if (alamd_reference_order(rooted ? ALAMD_COLL_REDUCE : ALAMD_COLL_ALLREDUCE, P, p.count, p.dtype, p.root, &order,
                                &start) != ALAMD_OK)
        AL_AMD_THROW(std::string(alamd_last_error()));
      break;
    case CombineAlgorithm::automatic_mpi_blocking:
      if (alamd_reference_order(rooted ? ALAMD_COLL_REDUCE_BLOCKING : ALAMD_COLL_ALLREDUCE_BLOCKING, P, p.count,
                                p.dtype, p.root, &order, &start) != ALAMD_OK)
        AL_AMD_THROW(std::string(alamd_last_error()));
      break;
    case CombineAlgorithm::rank_order: order = ALAMD_ORDER_RANK_ASC; break;
    case CombineAlgorithm::tree_doubling: order = ALAMD_ORDER_TREE_DBL; break;
    case CombineAlgorithm::tree_halving: order = ALAMD_ORDER_TREE_HALV; break;
    case CombineAlgorithm::tree_binomial: order = ALAMD_ORDER_TREE_BINOMIAL; start = rooted ? p.root : 0; break;
    case CombineAlgorithm::tree_reduce_scatter_gather: order = ALAMD_ORDER_TREE_RSG; break;
    case CombineAlgorithm::tree_reduce_scatter_gather_spread: order = ALAMD_ORDER_TREE_RSG_SPREAD; break;
    case CombineAlgorithm::ring:
    case CombineAlgorithm::ring_fused: ring = true; break;
    default: AL_AMD_THROW("Invalid algorithm");
    }
    if (rooted) {
      if (ring) AL_AMD_THROW("Invalid algorithm");
      void *out = recvs[static_cast<size_t>(p.root)];
      rc = alamd_combine(&out, 1, sends.data(), P, p.count, p.dtype, op, order, start, target);
    } else if (ring) {
      rc = alamd_ring_allreduce_from(recvs.data(), sends.data(), P, p.count, p.dtype, op, ring_chunk_bytes(es),
                                     p.algo == CombineAlgorithm::ring ? ALAMD_RING_STEPWISE : ALAMD_RING_FUSED,
                                     target);
    } else {
      rc = alamd_combine(recvs.data(), P, sends.data(), P, p.count, p.dtype, op, order, start, target);
    }
    break;
  }
  case OpKind::reduce_scatter: {
    int order = ALAMD_ORDER_RANK_ASC, start = 0;
    switch (p.algo) {
    case CombineAlgorithm::automatic:
    case CombineAlgorithm::automatic_mpi_blocking:
      if (alamd_reference_order(ALAMD_COLL_REDUCE_SCATTER, P, p.count * static_cast<size_t>(P), p.dtype, 0, &order,
                                &start) != ALAMD_OK)
        AL_AMD_THROW(std::string(alamd_last_error()));
      break;
    case CombineAlgorithm::rank_order: order = ALAMD_ORDER_RANK_ASC; break;
    case CombineAlgorithm::tree_doubling: order = ALAMD_ORDER_TREE_DBL; break;
    case CombineAlgorithm::tree_halving: order = ALAMD_ORDER_TREE_HALV; break;
    case CombineAlgorithm::tree_binomial: order = ALAMD_ORDER_TREE_BINOMIAL; break;
    case CombineAlgorithm::pairwise: order = ALAMD_ORDER_PAIRWISE_DESC; break;
    case CombineAlgorithm::ring_fused: order = ALAMD_ORDER_RING; break;
    default: AL_AMD_THROW("Invalid algorithm");
    }
    rc = alamd_reduce_scatter(recvs.data(), sends.data(), P, p.count, p.dtype, op, order, target);
    break;
  }
  case OpKind::allgather:
    if (p.algo != CombineAlgorithm::automatic && p.algo != CombineAlgorithm::automatic_mpi_blocking)
      AL_AMD_THROW("Invalid algorithm");
    rc = alamd_allgather(recvs.data(), sends.data(), P, p.count, p.dtype, target);
    break;
  case OpKind::reduce_scatterv: {
    size_t total = 0;
    for (size_t c : p.counts) total += c;
    int order = ALAMD_ORDER_RANK_ASC, start = 0;
    switch (p.algo) {
    case CombineAlgorithm::automatic:
    case CombineAlgorithm::automatic_mpi_blocking:
      if (alamd_reference_order(ALAMD_COLL_REDUCE_SCATTER, P, total, p.dtype, 0, &order, &start) != ALAMD_OK)
        AL_AMD_THROW(std::string(alamd_last_error()));
      break;
    case CombineAlgorithm::rank_order: order = ALAMD_ORDER_RANK_ASC; break;
    case CombineAlgorithm::tree_doubling: order = ALAMD_ORDER_TREE_DBL; break;
    case CombineAlgorithm::tree_halving: order = ALAMD_ORDER_TREE_HALV; break;
    case CombineAlgorithm::tree_binomial: order = ALAMD_ORDER_TREE_BINOMIAL; break;
    case CombineAlgorithm::pairwise: order = ALAMD_ORDER_PAIRWISE_DESC; break;
    default: AL_AMD_THROW("Invalid algorithm");
    }
    rc = alamd_reduce_scatterv(recvs.data(), sends.data(), P, p.counts.data(), p.dtype, op, order, target);
    break;
  }
  case OpKind::allgatherv:
    if (p.algo != CombineAlgorithm::automatic && p.algo != CombineAlgorithm::automatic_mpi_blocking)
      AL_AMD_THROW("Invalid algorithm");
    rc = alamd_allgatherv(recvs.data(), sends.data(), P, p.counts.data(), p.displs.data(), p.dtype, target);
    break;
  }
  if (rc != ALAMD_OK) AL_AMD_THROW(std::string(alamd_last_error()));
  release_streams(p, target);
}

}  // namespace amd

/** The backend policy class (cf. HostTransferBackend, include/aluminum/ht_impl.hpp:125-146). */
class HipCombineBackend {
 public:
  using comm_type = amd::Communicator;
  using req_type = std::shared_ptr<amd::Request>;
  static constexpr std::nullptr_t null_req = nullptr;
  using allreduce_algo_type = amd::CombineAlgorithm;
  using reduce_algo_type = amd::CombineAlgorithm;
  using reduce_scatter_algo_type = amd::CombineAlgorithm;
  using allgather_algo_type = amd::CombineAlgorithm;
  using reduce_scatterv_algo_type = amd::CombineAlgorithm;
  using allgatherv_algo_type = amd::CombineAlgorithm;

  static std::string Name() { return "HipCombineBackend"; }
  /** No registration is needed for device memory (ht_impl.hpp:844-853). */
  template <typename T> static void RegisterMemory(T *, size_t, comm_type &) {}
  template <typename T> static void UnregisterMemory(T *, comm_type &) {}

  template <typename T>
  static void Allreduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op, comm_type &comm,
                        allreduce_algo_type algo) {
    comm.world().post(comm, amd::OpKind::allreduce, amd::TypeMap<T>::value, sendbuf, recvbuf, count, op, algo, 0,
                      nullptr);
  }
  template <typename T>
  static void Allreduce(T *recvbuf, size_t count, ReductionOperator op, comm_type &comm,
                        allreduce_algo_type algo) {
    Allreduce(static_cast<const T *>(recvbuf), recvbuf, count, op, comm, algo);
  }
  template <typename T>
  static void NonblockingAllreduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op,
                                   comm_type &comm, req_type &req, allreduce_algo_type algo) {
    comm.world().post(comm, amd::OpKind::allreduce, amd::TypeMap<T>::value, sendbuf, recvbuf, count, op, algo, 0,
                      &req);
  }
  template <typename T>
  static void NonblockingAllreduce(T *recvbuf, size_t count, ReductionOperator op, comm_type &comm,
                                   req_type &req, allreduce_algo_type algo) {
    NonblockingAllreduce(static_cast<const T *>(recvbuf), recvbuf, count, op, comm, req, algo);
  }

  template <typename T>
  static void Reduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op, int root,
                     comm_type &comm, reduce_algo_type algo) {
    if (root < 0 || root >= comm.size()) AL_AMD_THROW("Invalid root");
    comm.world().post(comm, amd::OpKind::reduce, amd::TypeMap<T>::value, sendbuf, recvbuf, count, op, algo, root,
                      nullptr);
  }
  template <typename T>
  static void Reduce(T *recvbuf, size_t count, ReductionOperator op, int root, comm_type &comm,
                     reduce_algo_type algo) {
    Reduce(static_cast<const T *>(recvbuf), recvbuf, count, op, root, comm, algo);
  }
  template <typename T>
  static void NonblockingReduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op, int root,
                                comm_type &comm, req_type &req, reduce_algo_type algo) {
    if (root < 0 || root >= comm.size()) AL_AMD_THROW("Invalid root");
    comm.world().post(comm, amd::OpKind::reduce, amd::TypeMap<T>::value, sendbuf, recvbuf, count, op, algo, root,
                      &req);
  }
  template <typename T>
  static void NonblockingReduce(T *recvbuf, size_t count, ReductionOperator op, int root, comm_type &comm,
                                req_type &req, reduce_algo_type algo) {
    NonblockingReduce(static_cast<const T *>(recvbuf), recvbuf, count, op, root, comm, req, algo);
  }

  /** sendbuf holds size()*count elements, recvbuf receives count
   *  (include/aluminum/ht/reduce_scatter.hpp:45-74). */
  template <typename T>
  static void Reduce_scatter(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op, comm_type &comm,
                             reduce_scatter_algo_type algo) {
    comm.world().post(comm, amd::OpKind::reduce_scatter, amd::TypeMap<T>::value, sendbuf, recvbuf, count, op,
                      algo, 0, nullptr);
  }
  template <typename T>
  static void Reduce_scatter(T *recvbuf, size_t count, ReductionOperator op, comm_type &comm,
                             reduce_scatter_algo_type algo) {
    Reduce_scatter(static_cast<const T *>(recvbuf), recvbuf, count, op, comm, algo);
  }
  template <typename T>
  static void NonblockingReduce_scatter(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op,
                                        comm_type &comm, req_type &req, reduce_scatter_algo_type algo) {
    comm.world().post(comm, amd::OpKind::reduce_scatter, amd::TypeMap<T>::value, sendbuf, recvbuf, count, op,
                      algo, 0, &req);
  }
  template <typename T>
  static void NonblockingReduce_scatter(T *recvbuf, size_t count, ReductionOperator op, comm_type &comm,
                                        req_type &req, reduce_scatter_algo_type algo) {
    NonblockingReduce_scatter(static_cast<const T *>(recvbuf), recvbuf, count, op, comm, req, algo);
  }

  /** sendbuf holds sum(counts) elements, recvbuf receives counts[rank]
   *  (include/aluminum/ht/reduce_scatterv.hpp:40-87). */
  template <typename T>
  static void Reduce_scatterv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts, ReductionOperator op,
                              comm_type &comm, reduce_scatterv_algo_type algo) {
    comm.world().post(comm, amd::OpKind::reduce_scatterv, amd::TypeMap<T>::value, sendbuf, recvbuf, 0, op, algo, 0,
                      nullptr, &counts);
  }
  template <typename T>
  static void Reduce_scatterv(T *recvbuf, std::vector<size_t> counts, ReductionOperator op, comm_type &comm,
                              reduce_scatterv_algo_type algo) {
    Reduce_scatterv(static_cast<const T *>(recvbuf), recvbuf, std::move(counts), op, comm, algo);
  }
  template <typename T>
  static void NonblockingReduce_scatterv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts,
                                         ReductionOperator op, comm_type &comm, req_type &req,
                                         reduce_scatterv_algo_type algo) {
    comm.world().post(comm, amd::OpKind::reduce_scatterv, amd::TypeMap<T>::value, sendbuf, recvbuf, 0, op, algo, 0,
                      &req, &counts);
  }
  template <typename T>
  static void NonblockingReduce_scatterv(T *recvbuf, std::vector<size_t> counts, ReductionOperator op,
                                         comm_type &comm, req_type &req, reduce_scatterv_algo_type algo) {
    NonblockingReduce_scatterv(static_cast<const T *>(recvbuf), recvbuf, std::move(counts), op, comm, req, algo);
  }

  /** sendbuf holds counts[rank] elements; recvbuf receives every rank's slice at displs[rank]
   *  (include/aluminum/ht/allgatherv.hpp:38-100). */
  template <typename T>
  static void Allgatherv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts, std::vector<size_t> displs,
                         comm_type &comm, allgatherv_algo_type algo) {
    comm.world().post(comm, amd::OpKind::allgatherv, amd::TypeMap<T>::value, sendbuf, recvbuf, 0,
                      ReductionOperator::sum, algo, 0, nullptr, &counts, &displs);
  }
  template <typename T>
  static void Allgatherv(T *recvbuf, std::vector<size_t> counts, std::vector<size_t> displs, comm_type &comm,
                         allgatherv_algo_type algo) {
    if (displs.size() != static_cast<size_t>(comm.size()))
      AL_AMD_THROW("Vector of counts or displacements is not communicator-sized");
    const T *mine = recvbuf + displs[static_cast<size_t>(comm.rank())];
    Allgatherv(mine, recvbuf, std::move(counts), std::move(displs), comm, algo);
  }
  template <typename T>
  static void NonblockingAllgatherv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts,
                                    std::vector<size_t> displs, comm_type &comm, req_type &req,
                                    allgatherv_algo_type algo) {
    comm.world().post(comm, amd::OpKind::allgatherv, amd::TypeMap<T>::value, sendbuf, recvbuf, 0,
                      ReductionOperator::sum, algo, 0, &req, &counts, &displs);
  }
  template <typename T>
  static void NonblockingAllgatherv(T *recvbuf, std::vector<size_t> counts, std::vector<size_t> displs,
                                    comm_type &comm, req_type &req, allgatherv_algo_type algo) {
    if (displs.size() != static_cast<size_t>(comm.size()))
      AL_AMD_THROW("Vector of counts or displacements is not communicator-sized");
    const T *mine = recvbuf + displs[static_cast<size_t>(comm.rank())];
    NonblockingAllgatherv(mine, recvbuf, std::move(counts), std::move(displs), comm, req, algo);
  }

  /* ---- one-sided extension (MPICUDABackend, include/aluminum/mpi_cuda_impl.hpp:70-104) ---- */

  /** Returns the address at which `peer`'s buffer is reachable: the buffer that `peer` passes to
   *  its own matching call.  For peer == comm.rank() that is local_buf itself
   *  (rma_self.hpp:44-46). */
  template <typename T> static T *AttachRemoteBuffer(T *local_buf, int peer, comm_type &comm) {
    return static_cast<T *>(comm.world().attach(comm.rank(), peer, local_buf));
  }
  /** Nothing is mapped, so nothing is unmapped (rma_self.hpp:47). */
  template <typename T> static void DetachRemoteBuffer(T *, int, comm_type &) {}
  static void Notify(int peer, comm_type &comm) { comm.world().rma_notify(comm.rank(), peer); }
  static void Wait(int peer, comm_type &comm) { comm.world().rma_wait(comm.rank(), peer); }
  /** An exchange of notifications (rma_ipc.hpp:254-262). */
  static void Sync(int peer, comm_type &comm) {
    Notify(peer, comm);
    Wait(peer, comm);
  }
  static void Sync(const int *peers, int num_peers, comm_type &comm) {
    for (int i = 0; i < num_peers; ++i) Notify(peers[i], comm);
    for (int i = 0; i < num_peers; ++i) Wait(peers[i], comm);
  }
  /** count elements from srcbuf to destbuf (a buffer of rank `dest`), on the communicator's stream
   *  (rma_self.hpp:57-70: an asynchronous copy; errors as there). */
  template <typename T>
  static void Put(const T *srcbuf, int dest, T *destbuf, size_t count, comm_type &comm) {
    if (dest < 0 || dest >= comm.size()) AL_AMD_THROW("Invalid peer rank");
    if (count == 0) return;
    if (srcbuf == nullptr) AL_AMD_THROW("Source buffer is null");
    if (destbuf == nullptr) AL_AMD_THROW("Destination buffer is null");
    AL_AMD_CHECK(alamd_copy(destbuf, srcbuf, count * sizeof(T), comm.get_stream()));
  }

  /** sendbuf holds count elements, recvbuf receives size()*count; in place the
   *  caller's slice is already at recvbuf + rank*count
   *  (include/aluminum/ht/allgather.hpp:48-81). */
  template <typename T>
  static void Allgather(const T *sendbuf, T *recvbuf, size_t count, comm_type &comm, allgather_algo_type algo) {
    comm.world().post(comm, amd::OpKind::allgather, amd::TypeMap<T>::value, sendbuf, recvbuf, count,
                      ReductionOperator::sum, algo, 0, nullptr);
  }
  template <typename T>
  static void Allgather(T *recvbuf, size_t count, comm_type &comm, allgather_algo_type algo) {
    Allgather(static_cast<const T *>(recvbuf + static_cast<size_t>(comm.rank()) * count), recvbuf, count, comm,
              algo);
  }
  template <typename T>
  static void NonblockingAllgather(const T *sendbuf, T *recvbuf, size_t count, comm_type &comm, req_type &req,
                                   allgather_algo_type algo) {
    comm.world().post(comm, amd::OpKind::allgather, amd::TypeMap<T>::value, sendbuf, recvbuf, count,
                      ReductionOperator::sum, algo, 0, &req);
  }
  template <typename T>
  static void NonblockingAllgather(T *recvbuf, size_t count, comm_type &comm, req_type &req,
                                   allgather_algo_type algo) {
    NonblockingAllgather(static_cast<const T *>(recvbuf + static_cast<size_t>(comm.rank()) * count), recvbuf, count,
                         comm, req, algo);
  }
};

/* ---- compile-time traits (include/aluminum/traits/traits_base.hpp:43-62, 86-92, 155-184;
 *      the host-transfer backend's answers: traits/ht_traits.hpp:41-105) ------ */

#ifndef AL_AMD_WITH_REFERENCE
enum class AlOperation {
  allgather, allgatherv, allreduce, alltoall, alltoallv, barrier, bcast, gather, gatherv, reduce,
  reduce_scatter, reduce_scatterv, scatter, scatterv, send, recv, sendrecv, multisendrecv
};

template <typename Backend> constexpr char AlBackendName[] = "unknown";
#endif
template <> inline constexpr char AlBackendName<HipCombineBackend>[] = "hip";

namespace amd {
/** The collectives this engine implements: the ones that combine or lay out rank contributions. */
constexpr bool implements(AlOperation op) {
  return op == AlOperation::allreduce || op == AlOperation::reduce || op == AlOperation::reduce_scatter ||
         op == AlOperation::reduce_scatterv || op == AlOperation::allgather || op == AlOperation::allgatherv;
}
template <typename T, typename = void> struct HasTypeMap : std::false_type {};
template <typename T> struct HasTypeMap<T, decltype(void(TypeMap<T>::value))> : std::true_type {};
}  // namespace amd

#ifndef AL_AMD_WITH_REFERENCE
template <AlOperation Op, typename Backend> struct IsOpSupported : std::false_type {};
template <typename Backend, typename T> struct IsTypeSupported : std::false_type {};
template <typename Backend, ReductionOperator op> struct IsReductionOpSupported : std::false_type {};
template <AlOperation Op, typename Backend> struct OpAlgoType {};
#endif
template <AlOperation Op>
struct IsOpSupported<Op, HipCombineBackend> : std::integral_constant<bool, amd::implements(Op)> {};

template <typename T> struct IsTypeSupported<HipCombineBackend, T> : amd::HasTypeMap<T> {};

/** Every operator, avg included: the sum in the collective's order followed by one division by
 *  comm.size() in the element type's arithmetic (the reference has avg on its NCCL backend only,
 *  include/aluminum/nccl_impl.hpp:176; its MPI and host-transfer backends throw, mpi/utils.hpp:192-194). */
template <ReductionOperator op> struct IsReductionOpSupported<HipCombineBackend, op> : std::true_type {};

// one specialisation per collective of the engine (the shape of AL_ADD_OP_ALGO_TYPE, traits_base.hpp:180-183)
#define AL_AMD_ALGO_TYPE(op) \
  template <> struct OpAlgoType<AlOperation::op, HipCombineBackend> { using type = amd::CombineAlgorithm; }
AL_AMD_ALGO_TYPE(allreduce);
AL_AMD_ALGO_TYPE(reduce);
AL_AMD_ALGO_TYPE(reduce_scatter);
AL_AMD_ALGO_TYPE(reduce_scatterv);
AL_AMD_ALGO_TYPE(allgather);
AL_AMD_ALGO_TYPE(allgatherv);
#undef AL_AMD_ALGO_TYPE

#ifndef AL_AMD_WITH_REFERENCE

/* ---- the public API templates (include/Al.hpp) ---------------------------- */

template <typename Backend, typename T>
void Allreduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op,
               typename Backend::comm_type &comm,
               typename Backend::allreduce_algo_type algo = Backend::allreduce_algo_type::automatic) {
  Backend::template Allreduce<T>(sendbuf, recvbuf, count, op, comm, algo);
}
template <typename Backend, typename T>
void Allreduce(T *buffer, size_t count, ReductionOperator op, typename Backend::comm_type &comm,
               typename Backend::allreduce_algo_type algo = Backend::allreduce_algo_type::automatic) {
  Backend::template Allreduce<T>(buffer, count, op, comm, algo);
}
template <typename Backend, typename T>
void NonblockingAllreduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op,
                          typename Backend::comm_type &comm, typename Backend::req_type &req,
                          typename Backend::allreduce_algo_type algo = Backend::allreduce_algo_type::automatic) {
  Backend::template NonblockingAllreduce<T>(sendbuf, recvbuf, count, op, comm, req, algo);
}
template <typename Backend, typename T>
void NonblockingAllreduce(T *buffer, size_t count, ReductionOperator op, typename Backend::comm_type &comm,
                          typename Backend::req_type &req,
                          typename Backend::allreduce_algo_type algo = Backend::allreduce_algo_type::automatic) {
  Backend::template NonblockingAllreduce<T>(buffer, count, op, comm, req, algo);
}
template <typename Backend, typename T>
void Reduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op, int root,
            typename Backend::comm_type &comm,
            typename Backend::reduce_algo_type algo = Backend::reduce_algo_type::automatic) {
  Backend::template Reduce<T>(sendbuf, recvbuf, count, op, root, comm, algo);
}
template <typename Backend, typename T>
void Reduce(T *buffer, size_t count, ReductionOperator op, int root, typename Backend::comm_type &comm,
            typename Backend::reduce_algo_type algo = Backend::reduce_algo_type::automatic) {
  Backend::template Reduce<T>(buffer, count, op, root, comm, algo);
}
template <typename Backend, typename T>
void NonblockingReduce(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op, int root,
                       typename Backend::comm_type &comm, typename Backend::req_type &req,
                       typename Backend::reduce_algo_type algo = Backend::reduce_algo_type::automatic) {
  Backend::template NonblockingReduce<T>(sendbuf, recvbuf, count, op, root, comm, req, algo);
}
template <typename Backend, typename T>
void NonblockingReduce(T *buffer, size_t count, ReductionOperator op, int root,
                       typename Backend::comm_type &comm, typename Backend::req_type &req,
                       typename Backend::reduce_algo_type algo = Backend::reduce_algo_type::automatic) {
  Backend::template NonblockingReduce<T>(buffer, count, op, root, comm, req, algo);
}
template <typename Backend, typename T>
void Reduce_scatter(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op,
                    typename Backend::comm_type &comm,
                    typename Backend::reduce_scatter_algo_type algo = Backend::reduce_scatter_algo_type::automatic) {
  Backend::template Reduce_scatter<T>(sendbuf, recvbuf, count, op, comm, algo);
}
template <typename Backend, typename T>
void Reduce_scatter(T *buffer, size_t count, ReductionOperator op, typename Backend::comm_type &comm,
                    typename Backend::reduce_scatter_algo_type algo = Backend::reduce_scatter_algo_type::automatic) {
  Backend::template Reduce_scatter<T>(buffer, count, op, comm, algo);
}
template <typename Backend, typename T>
void NonblockingReduce_scatter(const T *sendbuf, T *recvbuf, size_t count, ReductionOperator op,
                               typename Backend::comm_type &comm, typename Backend::req_type &req,
                               typename Backend::reduce_scatter_algo_type algo =
                                   Backend::reduce_scatter_algo_type::automatic) {
  Backend::template NonblockingReduce_scatter<T>(sendbuf, recvbuf, count, op, comm, req, algo);
}
template <typename Backend, typename T>
void NonblockingReduce_scatter(T *buffer, size_t count, ReductionOperator op, typename Backend::comm_type &comm,
                               typename Backend::req_type &req,
                               typename Backend::reduce_scatter_algo_type algo =
                                   Backend::reduce_scatter_algo_type::automatic) {
  Backend::template NonblockingReduce_scatter<T>(buffer, count, op, comm, req, algo);
}
template <typename Backend, typename T>
void Allgather(const T *sendbuf, T *recvbuf, size_t count, typename Backend::comm_type &comm,
               typename Backend::allgather_algo_type algo = Backend::allgather_algo_type::automatic) {
  Backend::template Allgather<T>(sendbuf, recvbuf, count, comm, algo);
}
template <typename Backend, typename T>
void Allgather(T *buffer, size_t count, typename Backend::comm_type &comm,
               typename Backend::allgather_algo_type algo = Backend::allgather_algo_type::automatic) {
  Backend::template Allgather<T>(buffer, count, comm, algo);
}
template <typename Backend, typename T>
void NonblockingAllgather(const T *sendbuf, T *recvbuf, size_t count, typename Backend::comm_type &comm,
                          typename Backend::req_type &req,
                          typename Backend::allgather_algo_type algo = Backend::allgather_algo_type::automatic) {
  Backend::template NonblockingAllgather<T>(sendbuf, recvbuf, count, comm, req, algo);
}
template <typename Backend, typename T>
void NonblockingAllgather(T *buffer, size_t count, typename Backend::comm_type &comm,
                          typename Backend::req_type &req,
                          typename Backend::allgather_algo_type algo = Backend::allgather_algo_type::automatic) {
  Backend::template NonblockingAllgather<T>(buffer, count, comm, req, algo);
}

template <typename Backend, typename T>
void Reduce_scatterv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts, ReductionOperator op,
                     typename Backend::comm_type &comm,
                     typename Backend::reduce_scatterv_algo_type algo =
                         Backend::reduce_scatterv_algo_type::automatic) {
  Backend::template Reduce_scatterv<T>(sendbuf, recvbuf, std::move(counts), op, comm, algo);
}
template <typename Backend, typename T>
void Reduce_scatterv(T *buffer, std::vector<size_t> counts, ReductionOperator op,
                     typename Backend::comm_type &comm,
                     typename Backend::reduce_scatterv_algo_type algo =
                         Backend::reduce_scatterv_algo_type::automatic) {
  Backend::template Reduce_scatterv<T>(buffer, std::move(counts), op, comm, algo);
}
template <typename Backend, typename T>
void NonblockingReduce_scatterv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts, ReductionOperator op,
                                typename Backend::comm_type &comm, typename Backend::req_type &req,
                                typename Backend::reduce_scatterv_algo_type algo =
                                    Backend::reduce_scatterv_algo_type::automatic) {
  Backend::template NonblockingReduce_scatterv<T>(sendbuf, recvbuf, std::move(counts), op, comm, req, algo);
}
template <typename Backend, typename T>
void NonblockingReduce_scatterv(T *buffer, std::vector<size_t> counts, ReductionOperator op,
                                typename Backend::comm_type &comm, typename Backend::req_type &req,
                                typename Backend::reduce_scatterv_algo_type algo =
                                    Backend::reduce_scatterv_algo_type::automatic) {
  Backend::template NonblockingReduce_scatterv<T>(buffer, std::move(counts), op, comm, req, algo);
}
template <typename Backend, typename T>
void Allgatherv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts, std::vector<size_t> displs,
                typename Backend::comm_type &comm,
                typename Backend::allgatherv_algo_type algo = Backend::allgatherv_algo_type::automatic) {
  Backend::template Allgatherv<T>(sendbuf, recvbuf, std::move(counts), std::move(displs), comm, algo);
}
template <typename Backend, typename T>
void Allgatherv(T *buffer, std::vector<size_t> counts, std::vector<size_t> displs,
                typename Backend::comm_type &comm,
                typename Backend::allgatherv_algo_type algo = Backend::allgatherv_algo_type::automatic) {
  Backend::template Allgatherv<T>(buffer, std::move(counts), std::move(displs), comm, algo);
}
template <typename Backend, typename T>
void NonblockingAllgatherv(const T *sendbuf, T *recvbuf, std::vector<size_t> counts, std::vector<size_t> displs,
                           typename Backend::comm_type &comm, typename Backend::req_type &req,
                           typename Backend::allgatherv_algo_type algo = Backend::allgatherv_algo_type::automatic) {
  Backend::template NonblockingAllgatherv<T>(sendbuf, recvbuf, std::move(counts), std::move(displs), comm, req, algo);
}
template <typename Backend, typename T>
void NonblockingAllgatherv(T *buffer, std::vector<size_t> counts, std::vector<size_t> displs,
                           typename Backend::comm_type &comm, typename Backend::req_type &req,
                           typename Backend::allgatherv_algo_type algo = Backend::allgatherv_algo_type::automatic) {
  Backend::template NonblockingAllgatherv<T>(buffer, std::move(counts), std::move(displs), comm, req, algo);
}

/* ---- one-sided extension (include/Al.hpp:1916-2001) ------------------------ */
namespace ext {
template <typename Backend, typename T>
T *AttachRemoteBuffer(T *local_buf, int peer, typename Backend::comm_type &comm) {
  return Backend::template AttachRemoteBuffer<T>(local_buf, peer, comm);
}
template <typename Backend, typename T>
void DetachRemoteBuffer(T *remote_buf, int peer, typename Backend::comm_type &comm) {
  Backend::template DetachRemoteBuffer<T>(remote_buf, peer, comm);
}
template <typename Backend> void Notify(int peer, typename Backend::comm_type &comm) { Backend::Notify(peer, comm); }
template <typename Backend> void Wait(int peer, typename Backend::comm_type &comm) { Backend::Wait(peer, comm); }
template <typename Backend> void Sync(int peer, typename Backend::comm_type &comm) { Backend::Sync(peer, comm); }
template <typename Backend> void Sync(const int *peers, int num_peers, typename Backend::comm_type &comm) {
  Backend::Sync(peers, num_peers, comm);
}
template <typename Backend, typename T>
void Put(const T *srcbuf, int dest, T *destbuf, size_t count, typename Backend::comm_type &comm) {
  Backend::template Put<T>(srcbuf, dest, destbuf, count, comm);
}
}  // namespace ext
#endif  // AL_AMD_WITH_REFERENCE

namespace amd {
/** Halo faces of a 3-D grid, x fastest (interior dims, `halo` cells on every side): the contiguous
 *  buffers that ext::Put moves in a halo exchange (test/test_rma_halo_exchange.cpp:171-197 puts
 *  buffers that are already contiguous; the strided faces are this engine's addition).  Faces:
 *  0 -x, 1 +x, 2 -y, 3 +y, 4 -z, 5 +z; bit f of face_mask selects face f.  pack fills bufs[f] from
 *  the interior boundary slab, unpack writes bufs[f] into the ghost slab; both run on the
 *  communicator's stream. */
template <typename T>
void halo_pack(T *const bufs[6], const T *grid, const size_t dims[3], size_t halo, unsigned face_mask,
               Communicator &comm) {
  void *tab[6];
  for (int f = 0; f < 6; ++f) tab[f] = bufs[f];
  AL_AMD_CHECK(alamd_halo_pack(tab, grid, dims, halo, sizeof(T), face_mask, comm.get_stream()));
}
template <typename T>
void halo_unpack(T *grid, const T *const bufs[6], const size_t dims[3], size_t halo, unsigned face_mask,
                 Communicator &comm) {
  const void *tab[6];
  for (int f = 0; f < 6; ++f) tab[f] = bufs[f];
  AL_AMD_CHECK(alamd_halo_unpack(grid, tab, dims, halo, sizeof(T), face_mask, comm.get_stream()));
}
inline size_t halo_face_elems(const size_t dims[3], size_t halo, int face) {
  return alamd_halo_face_elems(dims, halo, face);
}
}  // namespace amd

/** Host-only completion test; resets the request when complete
 *  (include/aluminum/ht_impl.hpp:1113-1126). */
template <typename Backend> bool Test(typename Backend::req_type &req);
template <> inline bool Test<HipCombineBackend>(HipCombineBackend::req_type &req) {
  if (req == HipCombineBackend::null_req) return true;
  const int state = req->state.load(std::memory_order_acquire);
  if (state == amd::Request::failed) {
    const std::string why = req->error;
    req = HipCombineBackend::null_req;
    throw al_exception("The operation could not be launched: " + why, __FILE__, __LINE__);
  }
  if (state == amd::Request::not_launched) return false;  // some logical rank has not made its call
  const hipError_t e = hipEventQuery(req->done->event);
  if (e == hipSuccess) {
    req = HipCombineBackend::null_req;
    return true;
  }
  if (e != hipErrorNotReady) AL_AMD_THROW(std::string("GPU error: ") + hipGetErrorString(e));
  return false;
}

/** Makes the communicator's stream wait for the operation; does not block the
 *  host (include/aluminum/ht_impl.hpp:1128-1138). */
template <typename Backend> void Wait(typename Backend::req_type &req);
template <> inline void Wait<HipCombineBackend>(HipCombineBackend::req_type &req) {
  if (req == HipCombineBackend::null_req) return;
  const int state = req->state.load(std::memory_order_acquire);
  if (state == amd::Request::failed) {
    const std::string why = req->error;
    req = HipCombineBackend::null_req;
    throw al_exception("The operation could not be launched: " + why, __FILE__, __LINE__);
  }
  if (state == amd::Request::not_launched) AL_AMD_THROW("Wait on an operation that not every logical rank has started");
  if (req->orig_stream != req->done->ran_on && req->done->first_wait(req->orig_stream))
    AL_AMD_CHECK_HIP(hipStreamWaitEvent(req->orig_stream, req->done->event, 0));
  req = HipCombineBackend::null_req;
}

/* ---- stream flags (include/aluminum/cuda/gpu_wait.hpp, gpu_status_flag.hpp) -- */

namespace amd {

/** Blocks a stream until the host signals (cuda::GPUWait, src/cuda/gpu_wait.cpp:38-74). */
class GPUWait {
 public:
  GPUWait() { AL_AMD_CHECK(alamd_flag_create(&flag_, 0)); }
  ~GPUWait() { (void)alamd_flag_destroy(flag_); }
  GPUWait(const GPUWait &) = delete;
  GPUWait &operator=(const GPUWait &) = delete;
  /** Enqueue the wait.  max_spins = 0 waits for ever, like the reference. */
  void wait(hipStream_t stream, uint64_t max_spins = 0) {
    AL_AMD_CHECK(alamd_stream_wait_flag(stream, flag_, 1, max_spins ? ALAMD_FLAG_KERNEL : ALAMD_FLAG_AUTO, max_spins));
  }
  void signal() { AL_AMD_CHECK(alamd_flag_signal(flag_, 1)); }
  bool timed_out() { return alamd_flag_timed_out(flag_) != 0; }

 private:
  alamd_flag *flag_ = nullptr;
};

/** A host-pollable event (cuda::GPUStatusFlag, src/cuda/gpu_status_flag.cpp:38-98):
 *  created complete; record() stores 0 from the host and has the stream store 1. */
class GPUStatusFlag {
 public:
  GPUStatusFlag() { AL_AMD_CHECK(alamd_flag_create(&flag_, 1)); }
  ~GPUStatusFlag() { (void)alamd_flag_destroy(flag_); }
  GPUStatusFlag(const GPUStatusFlag &) = delete;
  GPUStatusFlag &operator=(const GPUStatusFlag &) = delete;
  void record(hipStream_t stream) {
    AL_AMD_CHECK(alamd_flag_signal(flag_, 0));
    AL_AMD_CHECK(alamd_stream_write_flag(stream, flag_, 1, ALAMD_FLAG_AUTO));
  }
  bool query() { return alamd_flag_query(flag_) != 0; }

 private:
  alamd_flag *flag_ = nullptr;
};


/** Host steps in stream order, on one background thread: the four phases of the
 *  reference's host-transfer state machine
 *  (HostTransferCollectiveSignalAtEndState::step, include/aluminum/ht/base_state.hpp:86-117;
 *  the thread itself: src/progress.cpp) built from the two flag types above.
 *  enqueue(stream, fn) returns at once; then
 *    1. the stream, when it gets there, sets a start flag           (GPUStatusFlag::record)
 *    2. the thread sees it and runs fn() - the reference's MPI call; here whatever
 *       the caller needs between two pieces of GPU work, e.g. an exchange with another host
 *    3. the thread lets the stream go on                            (GPUWait::signal)
 *    4. the stream sets an end flag, after which the state is freed (GPUStatusFlag::record)
 *  fn must not make a HIP call that waits for `stream` (it is blocked until fn returns).
 *  The combine itself never takes this path: it runs on the GPU. */
class ProgressEngine {
 public:
  ProgressEngine() : thread_([this] { run(); }) {}
  /** Waits until every enqueued step has been retired, i.e. until every stream given to enqueue()
   *  has passed its step: destroy the engine only when those streams can make progress. */
  ~ProgressEngine() {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      stop_ = true;
    }
    wake_.notify_all();
    thread_.join();
  }
  ProgressEngine(const ProgressEngine &) = delete;
  ProgressEngine &operator=(const ProgressEngine &) = delete;

  /** When the stream is let go on: once the host step has completed
   *  (HostTransferCollectiveSignalAtEndState, ht/base_state.hpp:86-117), or as soon as it has been
   *  started, for a rank whose device data the step no longer needs (the root under
   *  HostTransferCollectiveSignalRootEarlyState, :124-163; the other ranks under
   *  HostTransferCollectiveSignalNonRootEarlyState, :170-209). */
  enum class SignalWhen { at_end, after_start };
  static SignalWhen root_early(bool is_root) { return is_root ? SignalWhen::after_start : SignalWhen::at_end; }
  static SignalWhen non_root_early(bool is_root) { return is_root ? SignalWhen::at_end : SignalWhen::after_start; }

  /** A host step that runs to its end in one call. */
  void enqueue(hipStream_t stream, std::function<void()> fn) {
    enqueue(stream, std::move(fn), [] { return true; }, SignalWhen::at_end);
  }
  /** A host step in two parts, like the reference's start_mpi_op() / poll_mpi(): `start` begins it and
   *  returns, `poll` is called until it returns true (other steps make progress in between). */
  void enqueue(hipStream_t stream, std::function<void()> start, std::function<bool()> poll, SignalWhen when) {
    auto st = std::make_unique<State>();
    st->fn = std::move(start);
    st->poll = std::move(poll);
    st->when = when;
    st->start.record(stream);
    st->go.wait(stream);
    st->end.record(stream);
    {
      std::lock_guard<std::mutex> lock(mutex_);
      states_.push_back(std::move(st));
    }
    wake_.notify_all();
  }
  /** Host steps enqueued and not yet retired. */
  size_t pending() {
    std::lock_guard<std::mutex> lock(mutex_);
    return states_.size();
  }
  /** Rethrows, once, the first exception a host step has thrown since the last call.  The stream of
   *  a step that threw is released all the same, so nothing hangs behind it. */
  void check() {
    std::exception_ptr e;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      e = failed_;
      failed_ = nullptr;
    }
    if (e) std::rethrow_exception(e);
  }

 private:
  struct State {
    GPUStatusFlag start, end;
    GPUWait go;
    std::function<void()> fn;
    std::function<bool()> poll;
    SignalWhen when = SignalWhen::at_end;
    bool started = false, signalled = false, ran = false;
  };
  void run() {
    std::unique_lock<std::mutex> lock(mutex_);
    for (;;) {
      wake_.wait(lock, [this] { return stop_ || !states_.empty(); });
      if (states_.empty()) return;  // stop requested and nothing left to retire
      bool progressed = false;
      for (size_t i = 0; i < states_.size();) {
        State *st = states_[i].get();
        if (!st->ran && (st->started || st->start.query())) {
          lock.unlock();
          std::exception_ptr failed;
          bool done = false;
          try {
            if (!st->started) st->fn();  // phase 2, outside the lock: enqueue() may be called meanwhile
            st->started = true;
            done = st->poll();
          } catch (...) {
            failed = std::current_exception();
            done = true;  // a step that throws is over
          }
          if (!st->signalled && (done || st->when == SignalWhen::after_start)) {
            try {
              st->go.signal();  // phase 3, whatever the step did: the stream must not stay blocked
            } catch (...) {
              if (!failed) failed = std::current_exception();
            }
            st->signalled = true;
          }
          lock.lock();
          if (failed && !failed_) failed_ = failed;
          st->started = true;
          st->ran = done;
          progressed = progressed || done;
        }
        if (st->ran && st->end.query()) {  // phase 4: the wait has been consumed
          states_.erase(states_.begin() + static_cast<long>(i));
          progressed = true;
        } else {
          ++i;
        }
      }
      if (!progressed) {
        lock.unlock();
        std::this_thread::sleep_for(std::chrono::microseconds(5));
        lock.lock();
      }
    }
  }
  std::mutex mutex_;
  std::condition_variable wake_;
  std::deque<std::unique_ptr<State>> states_;
  std::exception_ptr failed_;
  bool stop_ = false;
  std::thread thread_;  // last: started when everything above exists
};

}  // namespace amd

}  // namespace Al

#endif
