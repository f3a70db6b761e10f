// tt_reduce1d_kernel: launch validation and kernel selection for the single-block reductions.
#include <algorithm>
#include <map>
#include <mutex>
#include <utility>

#include <hip/hip_runtime.h>

#include "tt_internal.h"

using namespace ttamd;

namespace {
// A large block is reduced by several workgroups that leave partial results in a small device buffer (256 slots
// of 16 bytes and an arrival counter).  Launches on one stream run in order and share one buffer; every
// (device, stream) pair gets its own, allocated on first use and kept until rt_release_stream or the end of the
// process.  A launch that is being recorded into a graph never takes this path (the graph could be replayed on
// any stream, beside eager launches on the one it was recorded on, and the buffer's address would be baked in):
// it runs as one workgroup, which needs no buffer.
using ttamd::kReduceMaxGroups;
using ttamd::kReduceCounterAt;
std::mutex g_mu;
std::map<std::pair<int, void *>, void *> g_bufs;
void *partials_for(void *stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing((hipStream_t)stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_bufs.find({dev, stream});
  if (it != g_bufs.end()) return it->second;
  void *p = nullptr;
  if (hipMalloc(&p, ttamd::kReduceScratchBytes) != hipSuccess) return nullptr;
  // Cleared in the stream that will use it: hipMemset runs in the null stream, which a non-blocking stream does not
  // wait for, so the first launch's workgroups could take their tickets before the counter was put to zero under
  // them (no workgroup then sees the last ticket, nothing is stored, and the counter stays off for the launches after).
  if (hipMemsetAsync(p, 0, ttamd::kReduceScratchBytes, (hipStream_t)stream) != hipSuccess) {
    (void)hipFree(p);
    return nullptr;
  }
  g_bufs[{dev, stream}] = p;
  return p;
}

struct TypeInfo { const char *kernel; int bytes; bool is_float; };
bool type_info(int dt, TypeInfo *t) {
  switch (dt) {
  case TT_I8: *t = {"reduce1d_i8", 1, false}; return true;
  case TT_I16: *t = {"reduce1d_i16", 2, false}; return true;
  case TT_I32: *t = {"reduce1d_i32", 4, false}; return true;
  case TT_I64: *t = {"reduce1d_i64", 8, false}; return true;
  case TT_U8: *t = {"reduce1d_u8", 1, false}; return true;
  case TT_U16: *t = {"reduce1d_u16", 2, false}; return true;
  case TT_U32: *t = {"reduce1d_u32", 4, false}; return true;
  case TT_U64: *t = {"reduce1d_u64", 8, false}; return true;
  case TT_F32: *t = {"reduce1d_f32", 4, true}; return true;
  case TT_BF16: *t = {"reduce1d_bf16", 2, true}; return true;
  case TT_F16: *t = {"reduce1d_f16", 2, true}; return true;
  case TT_F64: *t = {"reduce1d_f64", 8, true}; return true;
  default: return false;
  }
}
} // namespace

// Validation and launch shared by the two entry points.  `fixed_scratch`: null = the per-stream buffer (allocated on
// first use, never while recording); otherwise the buffer to use, whose counter is put back to zero first.
int ttamd::reduce1d_launch(int32_t op, const void *x, void *z, int32_t BLOCK, int32_t in_dtype, int32_t acc_dtype,
                           int32_t out_dtype, int32_t propagate_nan, const uint32_t grid[3], void *stream,
                           void *fixed_scratch) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "reduce1d: call rt_init first");
  if (!grid) return fail(RT_ERR_INVALID, "reduce1d: null grid");
  if (!x || !z) return fail(RT_ERR_INVALID, "reduce1d: null pointer");
  if (op < TT_REDUCE_SUM || op > TT_REDUCE_XOR_SUM) return fail(RT_ERR_INVALID, "reduce1d: op %d", op);
  // TRITON_MAX_TENSOR_NUMEL
  if (BLOCK <= 0 || BLOCK > 1048576) return fail(RT_ERR_INVALID, "reduce1d: BLOCK %d (1..1048576)", BLOCK);
  if (grid[0] == 0 || grid[1] == 0 || grid[2] == 0) return fail(RT_ERR_INVALID, "reduce1d: empty grid");
  TypeInfo in, acc, out;
  if (!type_info(in_dtype, &in) || !type_info(acc_dtype, &acc) || !type_info(out_dtype, &out))
    return fail(RT_ERR_UNSUPPORTED, "reduce1d: dtypes in %d, accumulate %d, out %d", in_dtype, acc_dtype, out_dtype);
  if (reinterpret_cast<uintptr_t>(x) % in.bytes || reinterpret_cast<uintptr_t>(z) % out.bytes)
    return fail(RT_ERR_INVALID, "reduce1d: pointer not aligned to its element size");
  const bool arg = op == TT_REDUCE_ARGMIN || op == TT_REDUCE_ARGMAX;
  if (in.is_float != acc.is_float || acc.bytes < in.bytes)
    return fail(RT_ERR_UNSUPPORTED, "reduce1d: accumulate dtype %d for input dtype %d", acc_dtype, in_dtype);
  if (op == TT_REDUCE_XOR_SUM && in.is_float) return fail(RT_ERR_INVALID, "reduce1d: xor_sum of a float tensor");
  if (propagate_nan && (!in.is_float || (op != TT_REDUCE_MIN && op != TT_REDUCE_MAX)))
    return fail(RT_ERR_INVALID, "reduce1d: propagate_nan applies to float min / max only");
  int out_kind = 0;
  if (arg) {
    if (out_dtype != TT_I32 && out_dtype != TT_I64)
      return fail(RT_ERR_UNSUPPORTED, "reduce1d: the index result is i32 or i64, got dtype %d", out_dtype);
  } else if (in.is_float) {
    // the value leaves in the accumulator's type or narrower (arith.truncf), never widened
    if (!out.is_float || out.bytes > acc.bytes || (in_dtype == TT_F64) != (acc_dtype == TT_F64))
      return fail(RT_ERR_UNSUPPORTED, "reduce1d: float accumulate %d -> out %d", acc_dtype, out_dtype);
    out_kind = out_dtype == TT_F64 ? 4 : out_dtype == TT_F32 ? 1 : out_dtype == TT_BF16 ? 2 : 3;
  } else {
    if (out.is_float || out.bytes > acc.bytes)
      return fail(RT_ERR_UNSUPPORTED, "reduce1d: integer accumulate %d -> out %d (widening after the reduction "
                  "is not offered)", acc_dtype, out_dtype);
  }
  int32_t n = BLOCK, op_ = op, nan_ = propagate_nan ? 1 : 0, ob = out.bytes;
  // Every program of the logical grid computes and stores the same value; it is computed once: by one workgroup,
  // or, from 128 KiB of 16-byte aligned input on, by one workgroup per 16 KiB (256 at most) whose last finisher
  // folds their partial results.
  const int64_t bytes = (int64_t)BLOCK * in.bytes;
  uint32_t groups = 1;
  void *scratch = nullptr, *counter = nullptr;
  if (bytes >= (128 << 10) && aligned16(x) && !env_int("TTAMD_REDUCE_ONE_GROUP", 0)) {
    scratch = fixed_scratch ? fixed_scratch : partials_for(stream);
    if (scratch) {
      groups = (uint32_t)std::min<int64_t>(kReduceMaxGroups, bytes >> 14);
      counter = (char *)scratch + kReduceCounterAt;
    }
  }
  if (fixed_scratch && groups > 1) {
    // the buffer outlives the call and is shared by every call on this device: start from a counter of zero
    void *cargs[] = {&counter};
    int rc = launch("reduce", "reduce1d_clear_counter", dim3(1), dim3(64), 0, stream, cargs, 1);
    if (rc) return rc;
  }
  void *args[] = {(void *)&x, (void *)&z, &n, &op_, &nan_, &ob, &out_kind, &scratch, &counter};
  return launch("reduce", in.kernel, dim3(groups), dim3(1024), 0, stream, args, 9);
}

extern "C" int tt_reduce1d_kernel(int32_t op, const void *x, void *z, int32_t BLOCK, int32_t in_dtype,
                                  int32_t acc_dtype, int32_t out_dtype, int32_t propagate_nan,
                                  const uint32_t grid[3], void *stream) {
  return ttamd::reduce1d_launch(op, x, z, BLOCK, in_dtype, acc_dtype, out_dtype, propagate_nan, grid, stream, nullptr);
}

extern "C" int rt_release_stream(void *stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(RT_ERR_HIP, "rt_release_stream: no current device");
  void *p = nullptr;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_bufs.find({dev, stream});
    if (it != g_bufs.end()) {
      p = it->second;
      g_bufs.erase(it);
    }
  }
  void *w = ttamd::gemm_take_workspace(dev, stream);
  if (!p && !w) return RT_OK;
  hipError_t e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "rt_release_stream: hipStreamSynchronize");
  for (void *q : {p, w}) {
    if (q && (e = hipFree(q)) != hipSuccess) return hip_fail(e, "rt_release_stream: hipFree");
  }
  return RT_OK;
}
