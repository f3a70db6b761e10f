// tt_reduce1d_kernel_noalloc: the single-block reductions for callers that cannot allocate device memory
// (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The partial results of a
// reduction shared between workgroups live in a file-scope device array instead of a buffer from hipMalloc.
#include <hip/hip_runtime.h>

#include "tt_internal.h"

using namespace ttamd;

namespace {

// 256 slots of 16 bytes and the arrival counter: 4352 bytes on every GPU this library runs on, held until the
// process ends.  In host code this name is a stand-in for the symbol, not a device address: the address on a
// given device comes from hipGetSymbolAddress and is what kernels and copies are handed.
static __device__ __align__(256) unsigned char scratch[kReduceScratchBytes];

constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices]; // per device: every GPU holds its own copy of the array at its own address

} // namespace

// Once per device, with that device current (rt_init calls it after hipSetDevice).
int ttamd::static_scratch_setup(int device) {
  if (device < 0 || device >= kMaxDevices) return fail(RT_ERR_INVALID, "static scratch: device %d", device);
  void *ptr = nullptr;
  hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
  if (!ptr) return fail(RT_ERR_HIP, "hipGetSymbolAddress(scratch) gave a null address");
  g_scratch_ptr[device] = ptr;
  return RT_OK;
}

extern "C" int tt_reduce1d_kernel_noalloc(int32_t op, const void *x, void *z, int32_t BLOCK, int32_t in_dtype,
                                          int32_t acc_dtype, int32_t out_dtype, int32_t propagate_nan,
                                          const uint32_t grid[3], void *stream) {
  const rt_props *p = props();
  if (!p) return fail(RT_ERR_NOT_INIT, "reduce1d_noalloc: call rt_init first");
  // the array holds the partial results of at most 256 workgroups of 16 KiB each; Triton's largest block
  // (1048576 elements of at most 8 bytes) needs no more, and anything beyond it is refused
  if (BLOCK > 1048576)
    return fail(RT_ERR_INVALID, "reduce1d_noalloc: BLOCK %d is beyond the 1048576 elements the static scratch covers", BLOCK);
  void *ptr = (p->device >= 0 && p->device < kMaxDevices) ? g_scratch_ptr[p->device] : nullptr;
  if (!ptr) return fail(RT_ERR_NOT_INIT, "reduce1d_noalloc: no static scratch on device %d", p->device);
  return reduce1d_launch(op, x, z, BLOCK, in_dtype, acc_dtype, out_dtype, propagate_nan, grid, stream, ptr);
}
