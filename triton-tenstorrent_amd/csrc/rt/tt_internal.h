// Shared between the translation units of libttamd_rt.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ttamd_rt.h"

namespace ttamd {

// Records the calling thread's error message and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);
// Properties of the initialised device, or nullptr before rt_init.
const rt_props *props();
// Looks up `name` in the built-in module `module` and launches it.
int launch(const char *module, const char *name, dim3 grid, dim3 block, uint32_t shmem,
           void *stream, void **args, size_t nargs);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t dtype_size(int dt) {
  switch (dt) {
  case TT_F32: case TT_I32: case TT_U32: return 4;
  case TT_BF16: case TT_F16: case TT_I16: case TT_U16: return 2;
  case TT_FP8E4M3: case TT_I8: case TT_U8: return 1;
  case TT_I64: case TT_U64: case TT_F64: return 8;
  default: return 0;
  }
}
// The buffer of partial results of a reduction shared between workgroups: 256 slots of 16 bytes, then the arrival
// counter.
constexpr int kReduceMaxGroups = 256;
constexpr size_t kReduceCounterAt = kReduceMaxGroups * 16, kReduceScratchBytes = kReduceCounterAt + 256;
int reduce1d_launch(int32_t op, const void *x, void *z, int32_t BLOCK, int32_t in_dtype, int32_t acc_dtype,
                    int32_t out_dtype, int32_t propagate_nan, const uint32_t grid[3], void *stream,
                    void *fixed_scratch);
// Takes the workspace that K-sliced matmul launches on (device, stream) share out of the library's table and returns
// it (null: none); the caller frees it once the stream has drained.
void *gemm_take_workspace(int device, void *stream);
// Resolves the address of the static scratch array on the current device; called by rt_init.
int static_scratch_setup(int device);
// Integer environment knob read once per name (tuning sweeps only).
int env_int(const char *name, int dflt);

} // namespace ttamd
