// Host runtime behind include/ttamd_rt.h: HIP module loading, launches, events
// and the per-kernel entry points that validate a launch and bind it to one of
// the gfx950 code objects embedded in this library.
#include "ttamd_rt.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "tt_internal.h"

// ---------------------------------------------------------------------------
// embedded code objects (built by build.py with hipcc --genco, one per source)
// ---------------------------------------------------------------------------
#ifndef TTAMD_CO_DIR
#error "TTAMD_CO_DIR must name the directory holding the *.hsaco files"
#endif
#define TTAMD_EMBED(sym, file)                                                        \
  __asm__(".section .rodata\n"                                                        \
          ".balign 4096\n"                                                            \
          ".global " #sym "_begin\n" #sym "_begin:\n"                                 \
          ".incbin \"" TTAMD_CO_DIR "/" file "\"\n"                                   \
          ".global " #sym "_end\n" #sym "_end:\n"                                     \
          ".byte 0\n"                                                                 \
          ".previous\n");                                                             \
  extern "C" const char sym##_begin[];                                                \
  extern "C" const char sym##_end[];

TTAMD_EMBED(ttamd_co_elementwise, "elementwise.hsaco")
TTAMD_EMBED(ttamd_co_gemm, "gemm.hsaco")
TTAMD_EMBED(ttamd_co_attention, "attention.hsaco")
TTAMD_EMBED(ttamd_co_reduce, "reduce.hsaco")

struct rt_module_s {
  hipModule_t mod = nullptr;
  bool builtin = false;
  std::map<std::string, rt_kernel_s *> kernels;
};
struct rt_kernel_s {
  hipFunction_t fn = nullptr;
  std::string name;
};
struct rt_event_s {
  hipEvent_t ev = nullptr;
};

namespace ttamd {

thread_local std::string g_last_error;
thread_local std::string g_last_kernel;

int fail(int code, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int hip_fail(hipError_t e, const char *what) {
  return fail(RT_ERR_HIP, "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
}

#define RT_HIP(call)                                                   \
  do {                                                                 \
    hipError_t e__ = (call);                                           \
    if (e__ != hipSuccess) return ttamd::hip_fail(e__, #call);         \
  } while (0)

struct State {
  std::mutex mu;
  bool inited = false;
  int device = -1;
  rt_props props{};
  std::map<std::string, rt_module_s *> builtin;
};
State &state() {
  static State s;
  return s;
}

const rt_props *props() { return state().inited ? &state().props : nullptr; }

int builtin_kernel(const char *module, const char *name, rt_kernel *out) {
  rt_module m = nullptr;
  int rc = rt_builtin_module(module, &m);
  if (rc) return rc;
  return rt_get_kernel(m, name, out);
}

int launch(const char *module, const char *name, dim3 grid, dim3 block, uint32_t shmem,
           void *stream, void **args, size_t nargs) {
  rt_kernel k = nullptr;
  int rc = builtin_kernel(module, name, &k);
  if (rc) return rc;
  const uint32_t g[3] = {grid.x, grid.y, grid.z}, b[3] = {block.x, block.y, block.z};
  rc = rt_launch(k, g, b, shmem, stream, args, nargs);
  if (rc == 0) g_last_kernel = name;
  return rc;
}

} // namespace ttamd

using ttamd::fail;
using ttamd::state;

extern "C" {

const char *rt_last_error(void) { return ttamd::g_last_error.c_str(); }
const char *tt_last_kernel_name(void) { return ttamd::g_last_kernel.c_str(); }

int rt_device_count(int *count) {
  if (!count) return fail(RT_ERR_INVALID, "rt_device_count: null out pointer");
  RT_HIP(hipGetDeviceCount(count));
  return RT_OK;
}

int rt_init(int device) {
  auto &s = state();
  std::lock_guard<std::mutex> lk(s.mu);
  if (s.inited && s.device == device) {
    RT_HIP(hipSetDevice(device));
    return RT_OK;
  }
  if (s.inited) return fail(RT_ERR_UNSUPPORTED, "rt_init: already bound to device %d", s.device);
  int n = 0;
  RT_HIP(hipGetDeviceCount(&n));
  if (device < 0 || device >= n) return fail(RT_ERR_INVALID, "rt_init: device %d of %d", device, n);
  RT_HIP(hipSetDevice(device));
  hipDeviceProp_t p;
  RT_HIP(hipGetDeviceProperties(&p, device));
  rt_props &o = s.props;
  memset(&o, 0, sizeof(o));
  o.device = device;
  o.multiprocessor_count = p.multiProcessorCount;
  o.warp_size = p.warpSize;
  o.max_shared_mem = (int32_t)p.sharedMemPerBlock;
  o.max_num_regs = p.regsPerBlock;
  o.clock_khz = p.clockRate;
  o.mem_clock_khz = p.memoryClockRate;
  o.mem_bus_bits = p.memoryBusWidth;
  o.l2_bytes = p.l2CacheSize;
  o.total_mem = p.totalGlobalMem;
  snprintf(o.name, sizeof(o.name), "%s", p.name);
  snprintf(o.arch, sizeof(o.arch), "%s", p.gcnArchName);
  if (strncmp(o.arch, "gfx950", 6) != 0)
    return fail(RT_ERR_UNSUPPORTED, "rt_init: device arch %s, this library holds gfx950 code only",
                o.arch);
  struct Img { const char *name; const char *b; const char *e; };
  const Img imgs[] = {{"elementwise", ttamd_co_elementwise_begin, ttamd_co_elementwise_end},
                      {"gemm", ttamd_co_gemm_begin, ttamd_co_gemm_end},
                      {"attention", ttamd_co_attention_begin, ttamd_co_attention_end},
                      {"reduce", ttamd_co_reduce_begin, ttamd_co_reduce_end}};
  for (const Img &im : imgs) {
    auto *m = new rt_module_s();
    hipError_t e = hipModuleLoadData(&m->mod, im.b);
    if (e != hipSuccess) {
      delete m;
      return ttamd::hip_fail(e, (std::string("hipModuleLoadData(") + im.name + ")").c_str());
    }
    m->builtin = true;
    s.builtin[im.name] = m;
  }
  // every kernel the reductions can launch is resolved now, so that a later call, which may sit inside a graph
  // capture, neither loads code nor allocates
  static const char *const reduce_kernels[] = {"reduce1d_i8", "reduce1d_i16", "reduce1d_i32", "reduce1d_i64",
                                               "reduce1d_u8", "reduce1d_u16", "reduce1d_u32", "reduce1d_u64",
                                               "reduce1d_f32", "reduce1d_bf16", "reduce1d_f16", "reduce1d_f64",
                                               "reduce1d_clear_counter"};
  for (const char *name : reduce_kernels) {
    rt_module_s *m = s.builtin["reduce"];
    hipFunction_t fn = nullptr;
    hipError_t e = hipModuleGetFunction(&fn, m->mod, name);
    if (e != hipSuccess) return ttamd::hip_fail(e, (std::string("hipModuleGetFunction(") + name + ")").c_str());
    auto *k = new rt_kernel_s();
    k->fn = fn;
    k->name = name;
    m->kernels[name] = k;
  }
  int rc = ttamd::static_scratch_setup(device);
  if (rc) return rc;
  s.device = device;
  s.inited = true;
  return RT_OK;
}

int rt_device_props(rt_props *out) {
  if (!out) return fail(RT_ERR_INVALID, "rt_device_props: null out pointer");
  if (!state().inited) return fail(RT_ERR_NOT_INIT, "rt_device_props: call rt_init first");
  *out = state().props;
  return RT_OK;
}

int rt_malloc(void **ptr, size_t bytes) {
  if (!ptr) return fail(RT_ERR_INVALID, "rt_malloc: null out pointer");
  RT_HIP(hipMalloc(ptr, bytes));
  return RT_OK;
}
int rt_free(void *ptr) {
  RT_HIP(hipFree(ptr));
  return RT_OK;
}
int rt_memcpy(void *dst, const void *src, size_t bytes, int kind) {
  static const hipMemcpyKind kinds[] = {hipMemcpyHostToHost, hipMemcpyHostToDevice,
                                        hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice};
  if (kind < 0 || kind > 3) return fail(RT_ERR_INVALID, "rt_memcpy: kind %d", kind);
  if (bytes && (!dst || !src)) return fail(RT_ERR_INVALID, "rt_memcpy: null pointer");
  RT_HIP(hipMemcpy(dst, src, bytes, kinds[kind]));
  return RT_OK;
}
int rt_memset(void *dst, int value, size_t bytes, void *stream) {
  if (bytes && !dst) return fail(RT_ERR_INVALID, "rt_memset: null pointer");
  RT_HIP(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream));
  return RT_OK;
}

int rt_module_load(const void *image, size_t bytes, rt_module *out) {
  if (!image || !bytes || !out) return fail(RT_ERR_INVALID, "rt_module_load: null argument");
  if (!state().inited) return fail(RT_ERR_NOT_INIT, "rt_module_load: call rt_init first");
  auto *m = new rt_module_s();
  hipError_t e = hipModuleLoadData(&m->mod, image);
  if (e != hipSuccess) {
    delete m;
    return ttamd::hip_fail(e, "hipModuleLoadData");
  }
  *out = m;
  return RT_OK;
}

int rt_module_unload(rt_module m) {
  if (!m) return fail(RT_ERR_INVALID, "rt_module_unload: null module");
  if (m->builtin) return fail(RT_ERR_INVALID, "rt_module_unload: built-in modules stay loaded");
  RT_HIP(hipModuleUnload(m->mod));
  for (auto &kv : m->kernels) delete kv.second;
  delete m;
  return RT_OK;
}

int rt_builtin_module(const char *which, rt_module *out) {
  if (!which || !out) return fail(RT_ERR_INVALID, "rt_builtin_module: null argument");
  auto &s = state();
  if (!s.inited) return fail(RT_ERR_NOT_INIT, "rt_builtin_module: call rt_init first");
  auto it = s.builtin.find(which);
  if (it == s.builtin.end()) return fail(RT_ERR_NOT_FOUND, "no built-in module '%s'", which);
  *out = it->second;
  return RT_OK;
}

int rt_get_kernel(rt_module m, const char *name, rt_kernel *out) {
  if (!m || !name || !out) return fail(RT_ERR_INVALID, "rt_get_kernel: null argument");
  std::lock_guard<std::mutex> lk(state().mu);
  auto it = m->kernels.find(name);
  if (it != m->kernels.end()) {
    *out = it->second;
    return RT_OK;
  }
  hipFunction_t fn = nullptr;
  hipError_t e = hipModuleGetFunction(&fn, m->mod, name);
  if (e == hipErrorNotFound) return fail(RT_ERR_NOT_FOUND, "no kernel '%s' in module", name);
  if (e != hipSuccess) return ttamd::hip_fail(e, "hipModuleGetFunction");
  auto *k = new rt_kernel_s();
  k->fn = fn;
  k->name = name;
  m->kernels[name] = k;
  *out = k;
  return RT_OK;
}

int rt_launch(rt_kernel k, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
              void *stream, void **args, size_t nargs) {
  if (!k || !grid || !block) return fail(RT_ERR_INVALID, "rt_launch: null argument");
  if (nargs && !args) return fail(RT_ERR_INVALID, "rt_launch: null args with nargs=%zu", nargs);
  for (int i = 0; i < 3; ++i)
    if (grid[i] == 0 || block[i] == 0)
      return fail(RT_ERR_INVALID, "rt_launch(%s): zero grid/block dimension", k->name.c_str());
  if ((uint64_t)block[0] * block[1] * block[2] > 1024)
    return fail(RT_ERR_INVALID, "rt_launch(%s): more than 1024 threads per workgroup",
                k->name.c_str());
  RT_HIP(hipModuleLaunchKernel(k->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                               shared_bytes, (hipStream_t)stream, args, nullptr));
  return RT_OK;
}

int rt_sync(void *stream) {
  RT_HIP(hipStreamSynchronize((hipStream_t)stream));
  return RT_OK;
}

int rt_event_create(rt_event *out) {
  if (!out) return fail(RT_ERR_INVALID, "rt_event_create: null out pointer");
  auto *e = new rt_event_s();
  hipError_t rc = hipEventCreate(&e->ev);
  if (rc != hipSuccess) {
    delete e;
    return ttamd::hip_fail(rc, "hipEventCreate");
  }
  *out = e;
  return RT_OK;
}
int rt_event_record(rt_event e, void *stream) {
  if (!e) return fail(RT_ERR_INVALID, "rt_event_record: null event");
  RT_HIP(hipEventRecord(e->ev, (hipStream_t)stream));
  return RT_OK;
}
int rt_event_sync(rt_event e) {
  if (!e) return fail(RT_ERR_INVALID, "rt_event_sync: null event");
  RT_HIP(hipEventSynchronize(e->ev));
  return RT_OK;
}
int rt_event_elapsed_ms(rt_event start, rt_event stop, float *ms) {
  if (!start || !stop || !ms) return fail(RT_ERR_INVALID, "rt_event_elapsed_ms: null argument");
  RT_HIP(hipEventElapsedTime(ms, start->ev, stop->ev));
  return RT_OK;
}
int rt_event_destroy(rt_event e) {
  if (!e) return fail(RT_ERR_INVALID, "rt_event_destroy: null event");
  RT_HIP(hipEventDestroy(e->ev));
  delete e;
  return RT_OK;
}

} // extern "C"
