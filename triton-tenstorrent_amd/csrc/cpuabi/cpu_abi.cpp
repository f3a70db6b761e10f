// libttamd_cpuabi.so: the native side of the host launcher for kernels with the reference's cpu/
// calling convention (include/ttamd_cpu_abi.h).  No GPU code and no dependency on the GPU runtime.
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <new>
#include <sched.h>

#include "ttamd_cpu_abi.h"

namespace {

// count and phase on their own cache lines: arrivals hammer one, waiters poll the other
struct alignas(64) Barrier {
  std::atomic<int32_t> count{0};
  alignas(64) std::atomic<int32_t> phase{0};
  int32_t workers = 1;
};

} // namespace

extern "C" {

__attribute__((visibility("default"))) void _cpu_barrier(void *barrier) {
  auto *b = static_cast<Barrier *>(barrier);
  if (!b || b->workers <= 1) return;
  const int32_t phase = b->phase.load(std::memory_order_acquire);
  if (b->count.fetch_add(1, std::memory_order_acq_rel) == b->workers - 1) {
    b->count.store(0, std::memory_order_relaxed);          // before the release below: the next round sees zero
    b->phase.store(phase + 1, std::memory_order_release);
    return;
  }
  // the other threads of the block may share this core: spin briefly, then give the core away
  for (int spins = 0; b->phase.load(std::memory_order_acquire) == phase; ++spins)
    if (spins > 256) sched_yield();
}

__attribute__((visibility("default"))) void *ttamd_cpu_barrier_create(int32_t workers) {
  if (workers < 1) return nullptr;
  void *mem = nullptr;
  if (posix_memalign(&mem, alignof(Barrier), sizeof(Barrier)) != 0) return nullptr;
  auto *b = new (mem) Barrier();
  b->workers = workers;
  return b;
}

__attribute__((visibility("default"))) void ttamd_cpu_barrier_destroy(void *barrier) {
  if (!barrier) return;
  static_cast<Barrier *>(barrier)->~Barrier();
  free(barrier);
}

__attribute__((visibility("default"))) void *ttamd_cpu_smem_alloc(uint64_t bytes) {
  void *mem = nullptr;
  const size_t n = bytes ? (size_t)((bytes + 63) / 64 * 64) : 64;
  if (posix_memalign(&mem, 64, n) != 0) return nullptr;
  memset(mem, 0, n);
  return mem;
}

__attribute__((visibility("default"))) void ttamd_cpu_smem_free(void *smem) { free(smem); }

__attribute__((visibility("default"))) void ttamd_cpu_block_range(int32_t blocks, int32_t workers, int32_t worker,
                                                                  int32_t *start, int32_t *end) {
  if (blocks < 0) blocks = 0;
  if (workers < 1) workers = 1;
  const int32_t base = blocks / workers, extra = blocks % workers;
  const int32_t s = worker * base + (worker < extra ? worker : extra);
  *start = s;
  *end = s + base + (worker < extra ? 1 : 0);
}

} // extern "C"
