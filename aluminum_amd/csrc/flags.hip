// Stream flags: one int32 word in pinned, device-visible host memory that a
// stream can wait on or write to, and that the host can signal or poll.
// These are what a progress thread and a stream synchronise through
// (reference: src/cuda/gpu_wait.cpp, src/cuda/gpu_status_flag.cpp,
// src/cuda/helper_kernels.cu, include/aluminum/cuda/sync_memory.hpp).
#include <mutex>
#include <new>

#include "alamd_common.h"

struct alamd_flag {
  // Two 128-byte lines: the word itself and the "a bounded wait gave up" mark.
  char *block;
  int32_t *word;       // host address == device address (pinned, mapped)
  int32_t *timed_out;
  alamd_flag *next_free;
};

namespace alamd {
namespace {

// One lane polls the word with system-scope loads; the stream stays blocked
// behind this kernel until the host (or another agent) stores `value`.
__global__ void __launch_bounds__(64) wait_flag_kernel(const int32_t *word, int32_t value,
                                                       unsigned long long max_spins, int32_t *timed_out) {
  if (threadIdx.x != 0) return;
  unsigned long long spins = 0;
  for (;;) {
    const int32_t v = __hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
    if (v == value) break;
    if (max_spins != 0 && ++spins >= max_spins) {
      __hip_atomic_store(timed_out, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      break;
    }
    __builtin_amdgcn_s_sleep(32);
  }
}

__global__ void __launch_bounds__(64) write_flag_kernel(int32_t *word, int32_t value) {
  if (threadIdx.x == 0) __hip_atomic_store(word, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Flags come from a pool of pinned slabs: pinning host memory costs far more
// than a collective, and a host-transfer style operation uses three flags
// (reference: sync_pool with 1024 preallocated words,
// include/aluminum/cuda/sync_memory.hpp:46-63, src/cuda/cuda.cpp:70-74).
// Slabs stay pinned until the process ends.
constexpr size_t kFlagBytes = 256, kFlagsPerSlab = 128;
std::mutex g_pool_mutex;
alamd_flag *g_free_list = nullptr;

int pool_get(alamd_flag **out) {
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  if (!g_free_list) {
    void *slab = nullptr;
    // Pinned memory must be allocated, not registered after the fact.
    ALAMD_HIP(hipHostMalloc(&slab, kFlagBytes * kFlagsPerSlab, hipHostMallocMapped | hipHostMallocCoherent));
    alamd_flag *nodes = new (std::nothrow) alamd_flag[kFlagsPerSlab];
    if (!nodes) { (void)hipHostFree(slab); return set_error(ALAMD_ERR_INVALID_ARG, "out of host memory"); }
    for (size_t k = 0; k < kFlagsPerSlab; ++k) {
      nodes[k].block = static_cast<char *>(slab) + k * kFlagBytes;
      nodes[k].word = reinterpret_cast<int32_t *>(nodes[k].block);
      nodes[k].timed_out = reinterpret_cast<int32_t *>(nodes[k].block + 128);
      nodes[k].next_free = g_free_list;
      g_free_list = &nodes[k];
    }
  }
  *out = g_free_list;
  g_free_list = g_free_list->next_free;
  (*out)->next_free = nullptr;
  return ALAMD_OK;
}

void pool_put(alamd_flag *f) {
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  f->next_free = g_free_list;
  g_free_list = f;
}

int memops_supported() {
  int dev = 0, can = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&can, hipDeviceAttributeCanUseStreamWaitValue, dev) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return can ? 1 : 0;
}

int resolve_mode(int mode, bool &memop) {
  if (mode == ALAMD_FLAG_AUTO) { memop = memops_supported() != 0; return ALAMD_OK; }
  if (mode == ALAMD_FLAG_KERNEL) { memop = false; return ALAMD_OK; }
  if (mode == ALAMD_FLAG_MEMOP) {
    if (!memops_supported())
      return set_error(ALAMD_ERR_UNSUPPORTED, "stream memory operations are not supported on this device");
    memop = true;
    return ALAMD_OK;
  }
  return set_error(ALAMD_ERR_INVALID_ARG, "unknown flag mode %d", mode);
}

}  // namespace
}  // namespace alamd

using namespace alamd;

extern "C" {

int alamd_stream_memops_supported(void) { return memops_supported(); }

int alamd_flag_create(alamd_flag **flag, int32_t initial) {
  if (!flag) return set_error(ALAMD_ERR_INVALID_ARG, "null flag pointer");
  alamd_flag *f = nullptr;
  int rc = pool_get(&f);
  if (rc) return rc;
  __atomic_store_n(f->word, initial, __ATOMIC_SEQ_CST);
  __atomic_store_n(f->timed_out, 0, __ATOMIC_SEQ_CST);
  *flag = f;
  return ALAMD_OK;
}

/* The caller must not destroy a flag that a stream may still wait on or write to. */
int alamd_flag_destroy(alamd_flag *flag) {
  if (flag) pool_put(flag);
  return ALAMD_OK;
}

volatile int32_t *alamd_flag_host_ptr(alamd_flag *flag) { return flag ? flag->word : nullptr; }

int alamd_stream_wait_flag(void *stream, alamd_flag *flag, int32_t value, int mode, uint64_t max_spins) {
  if (!flag) return set_error(ALAMD_ERR_INVALID_ARG, "null flag");
  bool memop = false;
  int rc = resolve_mode(mode, memop);
  if (rc) return rc;
  if (memop && max_spins != 0 && mode == ALAMD_FLAG_AUTO) memop = false;  // only the kernel can give up
  if (memop) {
    if (max_spins != 0)
      return set_error(ALAMD_ERR_INVALID_ARG, "a stream memory operation wait cannot be bounded");
    ALAMD_HIP(hipStreamWaitValue32(as_stream(stream), flag->word, (uint32_t)value, hipStreamWaitValueEq, 0xffffffffu));
    return ALAMD_OK;
  }
  hipLaunchKernelGGL(wait_flag_kernel, dim3(1), dim3(64), 0, as_stream(stream), flag->word, value,
                     (unsigned long long)max_spins, flag->timed_out);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

int alamd_stream_write_flag(void *stream, alamd_flag *flag, int32_t value, int mode) {
  if (!flag) return set_error(ALAMD_ERR_INVALID_ARG, "null flag");
  bool memop = false;
  int rc = resolve_mode(mode, memop);
  if (rc) return rc;
  if (memop) {
    ALAMD_HIP(hipStreamWriteValue32(as_stream(stream), flag->word, (uint32_t)value, 0));
    return ALAMD_OK;
  }
  hipLaunchKernelGGL(write_flag_kernel, dim3(1), dim3(64), 0, as_stream(stream), flag->word, value);
  ALAMD_HIP(hipGetLastError());
  return ALAMD_OK;
}

int alamd_flag_signal(alamd_flag *flag, int32_t value) {
  if (!flag) return set_error(ALAMD_ERR_INVALID_ARG, "null flag");
  __atomic_store_n(flag->word, value, __ATOMIC_SEQ_CST);
  return ALAMD_OK;
}

int32_t alamd_flag_query(alamd_flag *flag) {
  return flag ? __atomic_load_n(flag->word, __ATOMIC_SEQ_CST) : 0;
}

int alamd_flag_timed_out(alamd_flag *flag) {
  return flag ? (__atomic_load_n(flag->timed_out, __ATOMIC_SEQ_CST) != 0) : 0;
}

}  // extern "C"
