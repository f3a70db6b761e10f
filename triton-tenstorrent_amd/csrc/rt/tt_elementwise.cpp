// tt_add_kernel / tt_add_kernel_loop / tt_muladd_kernel / tt_sin_kernel:
// launch validation and binding to the streaming kernels of elementwise.hip.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>

#include "tt_internal.h"
#include "../kernels/elementwise_geom.h"

namespace ttamd {

int env_int(const char *name, int dflt) {
  static std::mutex mu;
  static std::map<std::string, int> cache;
  std::lock_guard<std::mutex> lk(mu);
  auto it = cache.find(name);
  if (it != cache.end()) return it->second;
  const char *v = getenv(name);
  int r = (v && *v) ? atoi(v) : dflt;
  cache[name] = r;
  return r;
}

namespace {

using ewgeom::kThreads;
constexpr int kUnroll = ewgeom::kVec;

// Elements the logical grid covers: programs 0..grid-1 own `per_program`
// consecutive elements each, clipped by the n_elements mask.
int check_1d(const char *who, int32_t n, int64_t per_program, const uint32_t grid[3],
             uint32_t *n_eff) {
  if (!grid) return fail(RT_ERR_INVALID, "%s: null grid", who);
  if (n < 0) return fail(RT_ERR_INVALID, "%s: n_elements %d < 0", who, n);
  if (per_program <= 0) return fail(RT_ERR_INVALID, "%s: BLOCK_SIZE must be positive", who);
  if (grid[1] != 1 || grid[2] != 1)
    return fail(RT_ERR_INVALID, "%s: 1-D grid expected, got (%u,%u,%u)", who, grid[0], grid[1],
                grid[2]);
  int64_t covered = (int64_t)grid[0] * per_program;
  *n_eff = (uint32_t)std::min<int64_t>(n, covered);
  return RT_OK;
}

// One workgroup per run of kThreads*kUnroll vectors (plus one for a ragged end / scalar
// tail); the unaligned kernels use a grid-stride loop over a grid sized to the CU count.
uint32_t streaming_grid(uint32_t n_eff, bool aligned, int vec_per_lane = kUnroll) {
  if (aligned) {
    const uint32_t nvec = n_eff >> 2, per_wg = kThreads * vec_per_lane;
    uint32_t wgs = nvec / per_wg;
    if (wgs * per_wg < nvec || (n_eff & 3u) || wgs == 0) ++wgs; // ragged end or scalar tail
    return wgs;
  }
  const rt_props *p = props();
  int64_t cap = (int64_t)p->multiprocessor_count * env_int("TTAMD_EW_WG_PER_CU", 32);
  return (uint32_t)std::max<int64_t>(1, std::min(cap, cdiv64((int64_t)n_eff, kThreads)));
}

} // namespace
} // namespace ttamd

using namespace ttamd;

extern "C" {

static int add_common(const char *who, const void *x, const void *y, void *out, int32_t n,
                      int64_t per_program, int32_t dtype, const uint32_t grid[3], void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "%s: call rt_init first", who);
  if (dtype != TT_F32 && dtype != TT_I32)
    return fail(RT_ERR_UNSUPPORTED, "%s: dtype %d (fp32 and int32 are supported)", who, dtype);
  uint32_t n_eff = 0;
  int rc = check_1d(who, n, per_program, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK; // nothing to do, nothing to touch
  if (!x || !y || !out) return fail(RT_ERR_INVALID, "%s: null tensor pointer", who);
  bool al = aligned16(x) && aligned16(y) && aligned16(out);
  const char *name = dtype == TT_F32 ? (al ? "ew_add_f32" : "ew_add_f32_unaligned")
                                     : (al ? "ew_add_i32" : "ew_add_i32_unaligned");
  void *args[] = {&x, &y, &out, &n_eff};
  return launch("elementwise", name, dim3(streaming_grid(n_eff, al)), dim3(kThreads), 0, stream, args, 4);
}

int tt_add_kernel(const void *x, const void *y, void *out, int32_t n_elements, int32_t BLOCK_SIZE,
                  int32_t dtype, const uint32_t grid[3], void *stream) {
  return add_common("add_kernel", x, y, out, n_elements, BLOCK_SIZE, dtype, grid, stream);
}

int tt_add_kernel_loop(const void *x, const void *y, void *out, int32_t n_elements,
                       int32_t row_count, int32_t BLOCK_SIZE, int32_t dtype, const uint32_t grid[3],
                       void *stream) {
  if (row_count < 0) return fail(RT_ERR_INVALID, "add_kernel: row_count %d < 0", row_count);
  if (row_count == 0) return RT_OK; // every program's range is empty
  if (BLOCK_SIZE <= 0) return fail(RT_ERR_INVALID, "add_kernel: BLOCK_SIZE must be positive");
  return add_common("add_kernel", x, y, out, n_elements, (int64_t)BLOCK_SIZE * row_count, dtype,
                    grid, stream);
}

int tt_muladd_kernel(const void *x, const void *y, const void *z, void *out, int32_t n_elements,
                     int32_t BLOCK_SIZE, const uint32_t grid[3], void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "muladd_kernel: call rt_init first");
  uint32_t n_eff = 0;
  int rc = check_1d("muladd_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !y || !z || !out) return fail(RT_ERR_INVALID, "muladd_kernel: null tensor pointer");
  uint32_t al = aligned16(x) && aligned16(y) && aligned16(z) && aligned16(out);
  void *args[] = {&x, &y, &z, &out, &n_eff, &al};
  return launch("elementwise", "ew_muladd_f32", dim3(streaming_grid(n_eff, al != 0)), dim3(kThreads), 0,
                stream, args, 6);
}

int tt_sin_kernel(const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE,
                  const uint32_t grid[3], void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "sin_kernel: call rt_init first");
  uint32_t n_eff = 0;
  int rc = check_1d("sin_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !out) return fail(RT_ERR_INVALID, "sin_kernel: null tensor pointer");
  bool al = aligned16(x) && aligned16(out);
  void *args[] = {&x, &out, &n_eff};
  return launch("elementwise", al ? "ew_sin_f32" : "ew_sin_f32_unaligned",
                dim3(streaming_grid(n_eff, al, ewgeom::kVecTrig)), dim3(kThreads), 0, stream, args, 3);
}

int tt_unary_kernel(int32_t op, const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE,
                    const uint32_t grid[3], void *stream) {
  static const char *const names[] = {"abs", "ceil", "cos", "exp", "exp2", "floor", "log", "log2", "rsqrt", "sin", "sqrt"};
  if (!props()) return fail(RT_ERR_NOT_INIT, "unary_kernel: call rt_init first");
  if (op < 0 || op >= (int)(sizeof(names) / sizeof(names[0])))
    return fail(RT_ERR_UNSUPPORTED, "unary_kernel: op %d (tt_unary_op has 0..10)", op);
  uint32_t n_eff = 0;
  int rc = check_1d("unary_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !out) return fail(RT_ERR_INVALID, "unary_kernel: null tensor pointer");
  bool al = aligned16(x) && aligned16(out);
  char name[48];
  snprintf(name, sizeof(name), "ew_%s_f32%s", names[op], al ? "" : "_unaligned");
  void *args[] = {&x, &out, &n_eff};
  const int vec = (op == TT_OP_SIN || op == TT_OP_COS) ? ewgeom::kVecTrig : kUnroll;
  return launch("elementwise", name, dim3(streaming_grid(n_eff, al, vec)), dim3(kThreads), 0, stream, args, 3);
}

int tt_binary_kernel(int32_t op, const void *x, const void *y, void *out, int32_t n_elements,
                     int32_t BLOCK_SIZE, const uint32_t grid[3], void *stream) {
  static const char *const names[] = {"add", "sub", "mul", "div", "max", "min"};
  if (!props()) return fail(RT_ERR_NOT_INIT, "binary_kernel: call rt_init first");
  if (op < 0 || op >= (int)(sizeof(names) / sizeof(names[0])))
    return fail(RT_ERR_UNSUPPORTED, "binary_kernel: op %d (tt_binary_op has 0..5)", op);
  uint32_t n_eff = 0;
  int rc = check_1d("binary_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !y || !out) return fail(RT_ERR_INVALID, "binary_kernel: null tensor pointer");
  bool al = aligned16(x) && aligned16(y) && aligned16(out);
  char name[48];
  snprintf(name, sizeof(name), "ew_%s_f32%s", names[op], al ? "" : "_unaligned");
  void *args[] = {&x, &y, &out, &n_eff};
  return launch("elementwise", name, dim3(streaming_grid(n_eff, al, kUnroll)), dim3(kThreads), 0,
                stream, args, 4);
}

int tt_binary_const_kernel(int32_t op, const void *x, float c, int32_t flip, void *out, int32_t n_elements,
                           int32_t BLOCK_SIZE, const uint32_t grid[3], void *stream) {
  static const char *const names[] = {"add", "sub", "mul", "div", "max", "min"};
  if (!props()) return fail(RT_ERR_NOT_INIT, "binary_const_kernel: call rt_init first");
  if (op < 0 || op >= (int)(sizeof(names) / sizeof(names[0])))
    return fail(RT_ERR_UNSUPPORTED, "binary_const_kernel: op %d (tt_binary_op has 0..5)", op);
  uint32_t n_eff = 0;
  int rc = check_1d("binary_const_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !out) return fail(RT_ERR_INVALID, "binary_const_kernel: null tensor pointer");
  bool al = aligned16(x) && aligned16(out);
  char name[48];
  snprintf(name, sizeof(name), "ew_%sc_f32%s", names[op], al ? "" : "_unaligned");
  int32_t fl = flip ? 1 : 0;
  void *args[] = {&x, &c, &fl, &out, &n_eff};
  return launch("elementwise", name, dim3(streaming_grid(n_eff, al)), dim3(kThreads), 0, stream, args, 5);
}

int tt_cast_kernel(const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE, int32_t in_dtype,
                   int32_t out_dtype, const uint32_t grid[3], void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "cast_kernel: call rt_init first");
  const char *stem = nullptr;
  if (in_dtype == TT_F32 && out_dtype == TT_BF16) stem = "ew_cast_f32_bf16";
  else if (in_dtype == TT_F32 && out_dtype == TT_F16) stem = "ew_cast_f32_f16";
  else if (in_dtype == TT_I32 && out_dtype == TT_I16) stem = "ew_cast_i32_i16";
  else if (in_dtype == TT_I32 && out_dtype == TT_I8) stem = "ew_cast_i32_i8";
  else
    return fail(RT_ERR_UNSUPPORTED, "cast_kernel: dtype %d -> %d (fp32 -> bf16/fp16 and int32 -> int16/int8 exist)",
                in_dtype, out_dtype);
  uint32_t n_eff = 0;
  int rc = check_1d("cast_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !out) return fail(RT_ERR_INVALID, "cast_kernel: null tensor pointer");
  if (reinterpret_cast<uintptr_t>(x) & 3) return fail(RT_ERR_INVALID, "cast_kernel: x must be 4-byte aligned");
  void *args[] = {&x, &out, &n_eff};
  if (aligned16(x) && aligned16(out)) {
    // one workgroup per run of kThreads * kUnroll 16-byte stores, plus the ragged end
    const uint32_t per_wg = kThreads * kUnroll * 4;   // four inputs per lane and vector
    return launch("elementwise", stem, dim3((uint32_t)cdiv64(n_eff, per_wg)), dim3(kThreads), 0, stream, args, 3);
  }
  char name[48];
  snprintf(name, sizeof(name), "%s_unaligned", stem);
  return launch("elementwise", name, dim3(streaming_grid(n_eff, false)), dim3(kThreads), 0, stream, args, 3);
}

int tt_copy_kernel(const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE, int32_t dtype,
                   const uint32_t grid[3], void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "copy_kernel: call rt_init first");
  const int64_t width = dtype_size(dtype);
  if (width <= 0) return fail(RT_ERR_UNSUPPORTED, "copy_kernel: dtype %d", dtype);
  uint32_t n_eff = 0;
  int rc = check_1d("copy_kernel", n_elements, BLOCK_SIZE, grid, &n_eff);
  if (rc) return rc;
  if (n_eff == 0) return RT_OK;
  if (!x || !out) return fail(RT_ERR_INVALID, "copy_kernel: null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & (uintptr_t)(width - 1))
    return fail(RT_ERR_INVALID, "copy_kernel: pointers must be aligned to the %lld-byte element", (long long)width);
  if (aligned16(x) && aligned16(out)) {
    uint64_t nbytes = (uint64_t)n_eff * (uint64_t)width;
    // one workgroup per run of kThreads * kUnroll 16-byte vectors; the one after the last whole run takes the
    // ragged end of the vectors and the bytes past the last vector
    const uint64_t nvec = nbytes >> 4, per_wg = kThreads * kUnroll;
    uint64_t wgs = nvec / per_wg;
    if (wgs * per_wg < nvec || (nbytes & 15u)) ++wgs;
    void *args[] = {&x, &out, &nbytes};
    return launch("elementwise", "ew_copy_b128", dim3((uint32_t)wgs), dim3(kThreads), 0, stream, args, 3);
  }
  char name[48];
  snprintf(name, sizeof(name), "ew_copy_b%d_unaligned", (int)width * 8);
  void *args[] = {&x, &out, &n_eff};
  return launch("elementwise", name, dim3(streaming_grid(n_eff, false)), dim3(kThreads), 0, stream, args, 3);
}

} // extern "C"
