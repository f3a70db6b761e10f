/*
 * CPU oracle: a plain-C restatement of what the reference's example kernels
 * compute when they are lowered through its cpu/ (Triton-CPU) path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels
 * are compared against and the "port" CPU baseline that the benchmark times;
 * nothing in the shipped package links, imports or calls it.
 *
 * Every function cites the reference file:line it restates.  The execution
 * model is the reference's persistent one: the logical grid of
 * gridX*gridY*gridZ programs is cut into one contiguous [block_start,
 * block_end) range per worker and each worker loops over its range calling the
 * kernel body with pid = block index
 * (cpu/lib/Dialect/TritonCPU/Transforms/MakePersistentKernel.cpp:144-198,
 *  cpu/lib/TritonCPUToLLVM/GPUOpToLLVM.cpp:16-22).  Workers are OpenMP threads.
 *
 * Pinning status (what independent check fixes each function) is listed in
 * oracle/README.md and exercised by tests/test_oracle_*.py:
 *   orc_block_range, orc_pid_decode, orc_tile_of_pid, orc_tile_of_pid_pointer :
 *       brute-force coverage / bijection properties, a literal transcription of
 *       both sources' decode on a grid with a short last group
 *   orc_add_*      : closed form (numpy), bit-exact
 *   orc_sin_f32    : float64 libm sin rounded once to fp32
 *   orc_unary/binary_f32: numpy's float32 operations bit for bit where the operation is
 *       exact, numpy float64 rounded once elsewhere; hand-written tables for NaN and
 *       signed zero in maximum/minimum
 *   orc_matmul_*   : textbook sum_k a*b vs numpy float64 on exactly
 *       representable inputs, B = I, tile-order independence
 *   orc_matmul_tiled: its tile-major index maps against a brute-force python
 *       loop; bit-equal to orc_matmul on the re-tiled operands, ragged shapes
 *       included; the reference's own 32x64 @ 64x32 fp16 self-check (atol 1e-2)
 *   orc_attn_fwd   : textbook softmax attention in float64, row-0 closed form,
 *       uniform-K running mean, base-2 log-sum-exp identity
 *   GELU epilogue, fp8 scaled GEMM: NOT in the reference; "parity unpinned" by
 *       it (pinned only against torch/numpy closed forms).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* element type codes shared with the python wrapper */
enum { ORC_F32 = 0, ORC_I32 = 1, ORC_BF16 = 2, ORC_F16 = 3, ORC_FP8E4M3 = 4 };
/* epilogue codes for orc_matmul */
enum {
  ORC_EPI_NONE = 0,         /* C = cast(acc)                       09-persistent-matmul.py:141 */
  ORC_EPI_BIAS_FULL = 1,    /* C = cast(acc) + bias[M,N] in half   09-matmul-fused.py:139-146  */
  ORC_EPI_BIAS_ROW_GELU = 2,/* C = cast(gelu(acc + bias[n])) fp32  (not in the reference)      */
  ORC_EPI_LEAKY_RELU = 3,   /* C = cast(leaky_relu(acc)) fp32      03-matrix-multiplication.py:370-374 */
  ORC_EPI_BIAS_ROW = 4      /* C = cast(acc + bias[n]) fp32        (row bias without activation) */
};

/* ------------------------------------------------------------------ */
/* scalar conversions                                                  */
/* ------------------------------------------------------------------ */
static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return u32_as_f32((uint32_t)h << 16); }

/* round-to-nearest-even fp32 -> bf16 (what `acc.to(bf16)` does) */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_as_u32(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return u32_as_f32(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-08f;
    return sign ? -v : v;
  }
  if (exp == 31) return u32_as_f32(sign | 0x7f800000u | (man << 13));
  return u32_as_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even fp32 -> fp16 */
static inline uint16_t f32_to_f16(float f) {
  uint32_t u = f32_as_u32(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);           /* NaN */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* >= 65520 -> inf */
  if (a < 0x38800000u) {                                            /* subnormal half / zero */
    /* result = rne(|f| * 2^24) as an integer in [0, 1024] */
    float scaled = u32_as_f32(a) * 16777216.0f;
    float r = nearbyintf(scaled); /* default rounding mode = RNE */
    return (uint16_t)(sign | (uint32_t)r);
  }
  uint32_t m = a + 0xc8000000u;   /* rebias exponent by -112 */
  m += 0xfffu + ((m >> 13) & 1u); /* RNE on the 13 dropped bits */
  return (uint16_t)(sign | (m >> 13));
}

/* OCP fp8 e4m3fn: 1-4-3, bias 7, no inf, NaN = S.1111.111, max finite 448 */
static inline float fp8e4m3_to_f32(uint8_t b) {
  uint32_t sign = (uint32_t)(b & 0x80u) << 24;
  uint32_t exp = (b >> 3) & 0xfu;
  uint32_t man = b & 7u;
  if (exp == 15 && man == 7) return u32_as_f32(sign | 0x7fc00000u);
  if (exp == 0) {
    float v = (float)man * 0.001953125f; /* man * 2^-9 */
    return sign ? -v : v;
  }
  return u32_as_f32(sign | ((exp + 120u) << 23) | (man << 20));
}

/* saturating RNE fp32 -> e4m3fn (the host-side quantiser of the fp8 config) */
static inline uint8_t f32_to_fp8e4m3(float f) {
  uint32_t u = f32_as_u32(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  float a = fabsf(f);
  if (a != a) return (uint8_t)(sign | 0x7f);
  if (a >= 448.0f) return (uint8_t)(sign | 0x7e); /* saturate to 448 */
  if (a < 0.015625f) {                            /* below 2^-6: subnormal grid 2^-9 */
    float r = nearbyintf(a * 512.0f);
    return (uint8_t)(sign | (uint8_t)r);          /* r == 8 lands on exp=1,man=0 */
  }
  uint32_t au = f32_as_u32(a);
  au += 0x7ffffu + ((au >> 20) & 1u);             /* RNE on the 20 dropped bits */
  uint32_t exp = (au >> 23) - 120u;
  uint32_t man = (au >> 20) & 7u;
  uint32_t code = (exp << 3) | man;
  if (code > 0x7e) code = 0x7e;
  return (uint8_t)(sign | code);
}

static inline float load_elem(const void *p, int64_t i, int dt) {
  switch (dt) {
  case ORC_BF16: return bf16_to_f32(((const uint16_t *)p)[i]);
  case ORC_F16: return f16_to_f32(((const uint16_t *)p)[i]);
  case ORC_FP8E4M3: return fp8e4m3_to_f32(((const uint8_t *)p)[i]);
  default: return ((const float *)p)[i];
  }
}

static inline float round_to(float v, int dt) {
  switch (dt) {
  case ORC_BF16: return bf16_to_f32(f32_to_bf16(v));
  case ORC_F16: return f16_to_f32(f32_to_f16(v));
  case ORC_FP8E4M3: return fp8e4m3_to_f32(f32_to_fp8e4m3(v));
  default: return v;
  }
}

static inline void store_elem(void *p, int64_t i, int dt, float v) {
  switch (dt) {
  case ORC_BF16: ((uint16_t *)p)[i] = f32_to_bf16(v); break;
  case ORC_F16: ((uint16_t *)p)[i] = f32_to_f16(v); break;
  case ORC_FP8E4M3: ((uint8_t *)p)[i] = f32_to_fp8e4m3(v); break;
  default: ((float *)p)[i] = v; break;
  }
}

ORC_API void orc_convert(const void *src, int src_dt, void *dst, int dst_dt, int64_t n) {
  for (int64_t i = 0; i < n; ++i) store_elem(dst, i, dst_dt, load_elem(src, i, src_dt));
}

/* ------------------------------------------------------------------ */
/* SPMD plumbing                                                       */
/* ------------------------------------------------------------------ */

/* Contiguous balanced split of num_blocks logical programs over num_workers:
 * base = nb / nw, rem = nb % nw, start(w) = w*base + min(w, rem),
 * end = start + base + (w < rem)
 * (npu/lib/TritonNPUToTenstorrent/D2M/SPMDOpToD2M.cpp:38-112; the host mirror
 *  is examples/matmul_tensor_descriptor/matmul_multi_core_tma.cpp:139-158). */
ORC_API void orc_block_range(int64_t num_blocks, int num_workers, int worker,
                             int64_t *start, int64_t *end) {
  int64_t base = num_blocks / num_workers;
  int64_t rem = num_blocks % num_workers;
  int64_t w = worker;
  int64_t s = w * base + (w < rem ? w : rem);
  *start = s;
  *end = s + base + (w < rem ? 1 : 0);
}

/* Linear block index -> 3-D program id: x = b % gX, y = (b % (gX*gY)) / gX,
 * z = b / (gX*gY)   (cpu/lib/TritonCPUToLLVM/GPUOpToLLVM.cpp:73-101). */
ORC_API void orc_pid_decode(int64_t b, int gx, int gy, int *x, int *y, int *z) {
  int64_t gxy = (int64_t)gx * gy;
  *x = (int)(b % gx);
  *y = (int)((b % gxy) / gx);
  *z = (int)(b / gxy);
}

/* GROUP_SIZE_M swizzle of the descriptor matmuls
 * (examples/matmul_tensor_descriptor/09-persistent-matmul.py:118-126). */
ORC_API void orc_tile_of_pid(int pid, int num_pid_m, int num_pid_n, int group_m,
                             int *pid_m, int *pid_n) {
  int num_pid_in_group = group_m * num_pid_n;
  int group_id = pid / num_pid_in_group;
  int first_pid_m = group_id * group_m;
  int group_size_m = num_pid_m - first_pid_m;
  if (group_size_m > group_m) group_size_m = group_m;
  *pid_m = first_pid_m + (pid % group_size_m);
  *pid_n = (pid % num_pid_in_group) / group_size_m;
}

/* The pointer-based matmul_kernel decodes its program id differently
 * (examples/matmul/03-matrix-multiplication.py:273-282): the row inside a group
 * is taken from the position inside the group, not from the program id itself:
 *   pid_m = first_pid_m + ((pid % num_pid_in_group) % group_size_m).
 * The two forms agree whenever group_id * num_pid_in_group is a multiple of
 * group_size_m, i.e. always except in a last, shorter group. */
ORC_API void orc_tile_of_pid_pointer(int pid, int num_pid_m, int num_pid_n, int group_m,
                                     int *pid_m, int *pid_n) {
  int num_pid_in_group = group_m * num_pid_n;
  int group_id = pid / num_pid_in_group;
  int first_pid_m = group_id * group_m;
  int group_size_m = num_pid_m - first_pid_m;
  if (group_size_m > group_m) group_size_m = group_m;
  *pid_m = first_pid_m + ((pid % num_pid_in_group) % group_size_m);
  *pid_n = (pid % num_pid_in_group) / group_size_m;
}

static int pick_threads(int nthreads) {
#ifdef _OPENMP
  if (nthreads <= 0) nthreads = omp_get_max_threads();
#else
  nthreads = 1;
#endif
  return nthreads;
}

/* ------------------------------------------------------------------ */
/* Elementwise                                                         */
/* ------------------------------------------------------------------ */

/* add_kernel (python/tutorials/01-vector-add.py:29-54): program pid owns
 * offsets pid*BLOCK + [0, BLOCK); lanes with offset >= n are masked: loads
 * yield 0 and stores are dropped
 * (cpu/lib/TritonCPUToLLVM/LoadStoreOpToLLVM.cpp:248-253,349-366).
 * Only `grid` programs run: elements past grid*BLOCK stay untouched. */
ORC_API void orc_add_f32(const float *x, const float *y, float *out, int32_t n,
                         int32_t block, int32_t grid, int nthreads) {
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      for (int64_t i = lo; i < hi; ++i) out[i] = x[i] + y[i];
    }
  }
}

/* int32 variant: arith.addi, two's-complement wraparound. */
ORC_API void orc_add_i32(const int32_t *x, const int32_t *y, int32_t *out, int32_t n,
                         int32_t block, int32_t grid, int nthreads) {
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      for (int64_t i = lo; i < hi; ++i)
        out[i] = (int32_t)((uint32_t)x[i] + (uint32_t)y[i]);
    }
  }
}

/* muladd_kernel (python/tutorials/01-vector-mul-add.py:30-57): x*y + z with
 * enable_fp_fusion on by default (backend/compiler.py:29) => contraction to one
 * fused multiply-add is what the cpu/ path emits; `fused`=0 gives the unfused
 * two-rounding form. */
ORC_API void orc_muladd_f32(const float *x, const float *y, const float *z, float *out,
                            int32_t n, int32_t block, int32_t grid, int fused,
                            int nthreads) {
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      if (fused) {
        for (int64_t i = lo; i < hi; ++i) out[i] = fmaf(x[i], y[i], z[i]);
      } else {
        for (int64_t i = lo; i < hi; ++i) {
          volatile float p = x[i] * y[i];
          out[i] = p + z[i];
        }
      }
    }
  }
}

/* sin_kernel (examples/01-sin-kernel.py:17-29).  The cpu/ path calls an LLVM
 * sin intrinsic resolved by libm or SLEEF; neither is bit-specified, so the
 * oracle is the correctly rounded value: float64 sin rounded once to fp32. */
ORC_API void orc_sin_f32(const float *x, float *out, int32_t n, int32_t block,
                         int32_t grid, int nthreads) {
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      for (int64_t i = lo; i < hi; ++i) out[i] = (float)sin((double)x[i]);
    }
  }
}

/* Faster fp32 libm variant used only as the timed CPU baseline of the sin
 * config (what a libm-backed cpu/ build would execute). */
ORC_API void orc_sinf_f32(const float *x, float *out, int32_t n, int32_t block,
                          int32_t grid, int nthreads) {
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      for (int64_t i = lo; i < hi; ++i) out[i] = sinf(x[i]);
    }
  }
}

/*
 * The unary and binary operations the reference's compute lowering accepts
 * (npu/lib/Dialect/TritonTenstorrent/Transforms/ConvertComputeOps.cpp:162-182), in the
 * masked-block form of sin_kernel / add_kernel.  Exact operations are done in fp32
 * (IEEE: correctly rounded); transcendental ones in float64 libm, rounded once to fp32.
 * arith.maximumf / minimumf: NaN if either operand is NaN, -0 ordered below +0.
 * Operation codes are tt_unary_op / tt_binary_op of the C ABI header.
 */
static inline float orc_unary_apply(int op, float x) {
  switch (op) {
  case 0: return fabsf(x);
  case 1: return ceilf(x);
  case 2: return (float)cos((double)x);
  case 3: return (float)exp((double)x);
  case 4: return (float)exp2((double)x);
  case 5: return floorf(x);
  case 6: return (float)log((double)x);
  case 7: return (float)log2((double)x);
  case 8: return (float)(1.0 / sqrt((double)x));
  case 9: return (float)sin((double)x);
  default: return sqrtf(x);
  }
}
static inline float orc_binary_apply(int op, float a, float b) {
  switch (op) {
  case 0: return a + b;
  case 1: return a - b;
  case 2: return a * b;
  case 3: return a / b;
  case 4:
    if (a != a) return a;
    if (b != b) return b;
    if (a == b) return signbit(a) ? b : a;
    return a > b ? a : b;
  default:
    if (a != a) return a;
    if (b != b) return b;
    if (a == b) return signbit(a) ? a : b;
    return a < b ? a : b;
  }
}
ORC_API int orc_unary_f32(int op, const float *x, float *out, int32_t n, int32_t block, int32_t grid,
                          int nthreads) {
  if (op < 0 || op > 10) return -1;
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      for (int64_t i = lo; i < hi; ++i) out[i] = orc_unary_apply(op, x[i]);
    }
  }
  return 0;
}
ORC_API int orc_binary_f32(int op, const float *x, const float *y, float *out, int32_t n, int32_t block,
                           int32_t grid, int nthreads) {
  if (op < 0 || op > 5) return -1;
  nthreads = pick_threads(nthreads);
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
  for (int w = 0; w < nthreads; ++w) {
    int64_t bs, be;
    orc_block_range(grid, nthreads, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int64_t lo = pid * (int64_t)block, hi = lo + block;
      if (hi > n) hi = n;
      for (int64_t i = lo; i < hi; ++i) out[i] = orc_binary_apply(op, x[i], y[i]);
    }
  }
  return 0;
}
/* one operand a constant of the kernel: out[i] = x[i] OP c, or c OP x[i] when flip is set; x and out may be
 * the same buffer (the one-element-per-program form of test_core.py::test_load_store_same_ptr has block = 1) */
ORC_API int orc_binary_const_f32(int op, const float *x, float c, int flip, float *out, int32_t n, int32_t block,
                                 int32_t grid) {
  if (op < 0 || op > 5) return -1;
  for (int64_t pid = 0; pid < grid; ++pid) {
    int64_t lo = pid * (int64_t)block, hi = lo + block;
    if (hi > n) hi = n;
    for (int64_t i = lo; i < hi; ++i) out[i] = flip ? orc_binary_apply(op, c, x[i]) : orc_binary_apply(op, x[i], c);
  }
  return 0;
}
/* arith.trunci: the low bits are kept */
ORC_API void orc_trunci(const int32_t *x, void *out, int bits, int32_t n, int32_t block, int32_t grid) {
  for (int64_t pid = 0; pid < grid; ++pid) {
    int64_t lo = pid * (int64_t)block, hi = lo + block;
    if (hi > n) hi = n;
    for (int64_t i = lo; i < hi; ++i) {
      if (bits == 16) ((int16_t *)out)[i] = (int16_t)(uint16_t)((uint32_t)x[i] & 0xffffu);
      else ((int8_t *)out)[i] = (int8_t)(uint8_t)((uint32_t)x[i] & 0xffu);
    }
  }
}

/* ------------------------------------------------------------------ */
/* Single-block reductions                                             */
/* ------------------------------------------------------------------ */
/*
 * kernel(X, Z, BLOCK): tl.store(Z, tl.<op>(tl.load(X + arange(BLOCK)), axis=0)) -- the form the
 * reference's CI runs on its cpu/ path (.github/workflows/integration-tests-cpu.yml:105,
 * test_core.py::test_reduce1d).  What is restated is the tt.reduce of the IR, folded from the left:
 *   sum      arith.addi / arith.addf in the accumulate type (i8 / i16 sums run in i32; a bf16 or f16
 *            sum rounds to that type after every addition, as arith.addf on that type does)
 *   min/max  arith.minsi|minui|maxsi|maxui, arith.minnumf|maxnumf (NaN dropped) or, with
 *            propagate_nan, arith.minimumf|maximumf
 *   argmin / argmax and min/max with indices: the combine region of triton/language/standard.py
 *            (_argmin_combine / _argmax_combine):  tie = v1 == v2 and i1 < i2 (tie_break_left only);
 *            first = v1 < v2 (resp. >) or tie;  select(first, (v1,i1), (v2,i2))
 *   xor_sum  arith.xori
 * dtype codes: 0 f32, 1 i32, 2 bf16, 3 f16, 5 i16, 6 i8, 7 i64, 8 f64, 9 u8, 10 u16, 11 u32, 12 u64.
 * Returns 0, or -1 for a combination the IR cannot hold.
 */
static int red_bytes(int dt) {
  switch (dt) {
  case 6: case 9: return 1;
  case 2: case 3: case 5: case 10: return 2;
  case 0: case 1: case 11: return 4;
  case 7: case 8: case 12: return 8;
  default: return 0;
  }
}
static int red_is_float(int dt) { return dt == 0 || dt == 2 || dt == 3 || dt == 8; }
static int red_is_unsigned(int dt) { return dt >= 9 && dt <= 12; }

static double red_load_f(const void *x, int64_t i, int dt) {
  switch (dt) {
  case 0: return ((const float *)x)[i];
  case 2: return bf16_to_f32(((const uint16_t *)x)[i]);
  case 3: return f16_to_f32(((const uint16_t *)x)[i]);
  default: return ((const double *)x)[i];
  }
}
/* the integer element, sign- or zero-extended to 64 bits and held as the bit pattern */
static uint64_t red_load_i(const void *x, int64_t i, int dt) {
  switch (dt) {
  case 6: return (uint64_t)(int64_t)((const int8_t *)x)[i];
  case 5: return (uint64_t)(int64_t)((const int16_t *)x)[i];
  case 1: return (uint64_t)(int64_t)((const int32_t *)x)[i];
  case 7: return (uint64_t)((const int64_t *)x)[i];
  case 9: return ((const uint8_t *)x)[i];
  case 10: return ((const uint16_t *)x)[i];
  case 11: return ((const uint32_t *)x)[i];
  default: return ((const uint64_t *)x)[i];
  }
}
/* wrap a 64-bit pattern to the accumulate width and extend it again with the input's sign rule */
static uint64_t red_wrap(uint64_t v, int acc_bytes, int is_unsigned) {
  if (acc_bytes == 8) return v;
  const int sh = 64 - 8 * acc_bytes;
  return is_unsigned ? (v << sh) >> sh : (uint64_t)(((int64_t)(v << sh)) >> sh);
}
static double red_round_f(double v, int dt) {
  switch (dt) {
  case 0: return (float)v;
  case 2: return bf16_to_f32(f32_to_bf16((float)v));
  case 3: return f16_to_f32(f32_to_f16((float)v));
  default: return v;
  }
}
static int red_less_i(uint64_t a, uint64_t b, int is_unsigned) {
  return is_unsigned ? a < b : (int64_t)a < (int64_t)b;
}

ORC_API int orc_reduce1d(int op, const void *x, int32_t n, int in_dt, int acc_dt, int out_dt,
                         int tie_break_left, int propagate_nan, void *z) {
  const int ib = red_bytes(in_dt), ab = red_bytes(acc_dt), ob = red_bytes(out_dt);
  if (op < 0 || op > 5 || n <= 0 || !ib || !ab || !ob) return -1;
  const int isf = red_is_float(in_dt), uns = red_is_unsigned(in_dt);
  if (isf != red_is_float(acc_dt) || ab < ib) return -1;
  if (op == 5 && isf) return -1;
  const int arg = op == 3 || op == 4;
  if (arg ? (out_dt != 1 && out_dt != 7) : (red_is_float(out_dt) != isf || ob > ab)) return -1;
  int64_t idx = 0;
  if (isf) {
    /* f32 arithmetic on f16 / bf16 / f32 operands held in a double is exact before the rounding
     * step below, except that an f32 sum is rounded twice (double, then float): innocuous, a double
     * sum of two floats is exact unless their exponents differ by more than 29. */
    double acc = red_round_f(red_load_f(x, 0, in_dt), acc_dt);
    for (int64_t i = 1; i < n; ++i) {
      const double v = red_round_f(red_load_f(x, i, in_dt), acc_dt);
      switch (op) {
      case 0: acc = red_round_f(acc + v, acc_dt); break;
      case 1:
        if (propagate_nan) acc = (acc != acc || v != v) ? NAN : (v < acc ? v : acc);
        else acc = fmin(acc, v);
        break;
      case 2:
        if (propagate_nan) acc = (acc != acc || v != v) ? NAN : (v > acc ? v : acc);
        else acc = fmax(acc, v);
        break;
      default: {
        const int tie = tie_break_left && acc == v && idx < i;
        const int first = (op == 3 ? acc < v : acc > v) || tie;
        if (!first) { acc = v; idx = i; }
      }
      }
    }
    if (!arg) {
      switch (out_dt) {
      case 0: *(float *)z = (float)acc; break;
      case 2: *(uint16_t *)z = f32_to_bf16((float)acc); break;
      case 3: *(uint16_t *)z = f32_to_f16((float)acc); break;
      default: *(double *)z = acc;
      }
    }
  } else {
    uint64_t acc = red_wrap(red_load_i(x, 0, in_dt), ab, uns);
    for (int64_t i = 1; i < n; ++i) {
      const uint64_t v = red_wrap(red_load_i(x, i, in_dt), ab, uns);
      switch (op) {
      case 0: acc = red_wrap(acc + v, ab, uns); break;
      case 5: acc = red_wrap(acc ^ v, ab, uns); break;
      case 1: if (red_less_i(v, acc, uns)) acc = v; break;
      case 2: if (red_less_i(acc, v, uns)) acc = v; break;
      default: {
        const int tie = tie_break_left && acc == v && idx < i;
        const int first = (op == 3 ? red_less_i(acc, v, uns) : red_less_i(v, acc, uns)) || tie;
        if (!first) { acc = v; idx = i; }
      }
      }
    }
    if (!arg) {
      switch (ob) {
      case 1: *(uint8_t *)z = (uint8_t)acc; break;
      case 2: *(uint16_t *)z = (uint16_t)acc; break;
      case 4: *(uint32_t *)z = (uint32_t)acc; break;
      default: *(uint64_t *)z = acc;
      }
    }
  }
  if (arg) {
    if (out_dt == 7) *(int64_t *)z = idx;
    else *(int32_t *)z = (int32_t)idx;
  }
  return 0;
}

/* ------------------------------------------------------------------ */
/* Tile matmul family                                                  */
/* ------------------------------------------------------------------ */

static inline float gelu_erf(float x) {
  /* exact-erf GELU in fp32: 0.5*x*(1+erf(x/sqrt(2))) */
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}

/*
 * matmul_kernel_tma / matmul_kernel_fused, one logical program per
 * BM x BN output tile
 * (examples/matmul_tensor_descriptor/09-persistent-matmul.py:102-145,
 *  python/tutorials/09-matmul-fused.py:100-148).
 *   - pid -> (pid_m, pid_n) through the GROUP_SIZE_M swizzle (:118-126)
 *   - fp32 accumulator, K walked in BK steps (:131-139); A is [M,K] row-major
 *     with leading stride lda, B is [K,N] row-major (NOT transposed) with ldb
 *   - descriptor loads beyond the tensor are zero-padded, stores are clipped
 *     (triton/tools/tensor_descriptor.py padding="zero")
 *   - one RNE rounding fp32 -> out dtype (:141), then the epilogue selected by
 *     `epi` (see the enum above for the reference line each follows)
 * acc64 != 0 accumulates in double instead (used to state tolerances against a
 * rounding-free sum, never as the parity target).
 * scale multiplies the accumulator before the cast (fp8 per-tensor scales;
 * pass 1.0f otherwise).
 */
ORC_API int orc_matmul(const void *a, int64_t lda, const void *b, int64_t ldb, void *c,
                       int64_t ldc, const void *bias, int64_t ldbias, int32_t M,
                       int32_t N, int32_t K, int32_t BM, int32_t BN, int32_t BK,
                       int32_t group_m, int32_t grid, int in_dt, int out_dt, int epi,
                       float scale, int acc64, int nthreads) {
  if (BM <= 0 || BN <= 0 || BK <= 0 || group_m <= 0) return -1;
  int num_pid_m = (M + BM - 1) / BM, num_pid_n = (N + BN - 1) / BN;
  if (grid > num_pid_m * num_pid_n) return -2; /* pid outside the tile grid */
  nthreads = pick_threads(nthreads);
  int k_tiles = (K + BK - 1) / BK;
#pragma omp parallel num_threads(nthreads)
  {
#ifdef _OPENMP
    int w = omp_get_thread_num(), nw = omp_get_num_threads();
#else
    int w = 0, nw = 1;
#endif
    float *accf = (float *)malloc(sizeof(float) * (size_t)BM * BN);
    double *accd = acc64 ? (double *)malloc(sizeof(double) * (size_t)BM * BN) : NULL;
    float *at = (float *)malloc(sizeof(float) * (size_t)BM * BK);
    float *bt = (float *)malloc(sizeof(float) * (size_t)BK * BN);
    int64_t bs, be;
    orc_block_range(grid, nw, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int pid_m, pid_n;
      orc_tile_of_pid((int)pid, num_pid_m, num_pid_n, group_m, &pid_m, &pid_n);
      int64_t om = (int64_t)pid_m * BM, on = (int64_t)pid_n * BN;
      for (int i = 0; i < BM * BN; ++i) accf[i] = 0.0f;
      if (acc64) for (int i = 0; i < BM * BN; ++i) accd[i] = 0.0;
      for (int kt = 0; kt < k_tiles; ++kt) {
        int64_t ok = (int64_t)kt * BK;
        /* descriptor loads with zero padding */
        for (int i = 0; i < BM; ++i)
          for (int k = 0; k < BK; ++k)
            at[i * BK + k] = (om + i < M && ok + k < K)
                                 ? load_elem(a, (om + i) * lda + ok + k, in_dt) : 0.0f;
        for (int k = 0; k < BK; ++k)
          for (int j = 0; j < BN; ++j)
            bt[k * BN + j] = (ok + k < K && on + j < N)
                                 ? load_elem(b, (ok + k) * ldb + on + j, in_dt) : 0.0f;
        /* acc = dot(a, b, acc) */
        if (!acc64) {
          for (int i = 0; i < BM; ++i) {
            float *arow = accf + (size_t)i * BN;
            for (int k = 0; k < BK; ++k) {
              float av = at[i * BK + k];
              const float *brow = bt + (size_t)k * BN;
              for (int j = 0; j < BN; ++j) arow[j] += av * brow[j];
            }
          }
        } else {
          for (int i = 0; i < BM; ++i) {
            double *arow = accd + (size_t)i * BN;
            for (int k = 0; k < BK; ++k) {
              double av = at[i * BK + k];
              const float *brow = bt + (size_t)k * BN;
              for (int j = 0; j < BN; ++j) arow[j] += av * (double)brow[j];
            }
          }
        }
      }
      /* epilogue + clipped store */
      for (int i = 0; i < BM; ++i) {
        if (om + i >= M) break;
        for (int j = 0; j < BN; ++j) {
          if (on + j >= N) break;
          float acc = acc64 ? (float)(accd[(size_t)i * BN + j] * (double)scale)
                            : (scale == 1.0f ? accf[(size_t)i * BN + j]
                                             : accf[(size_t)i * BN + j] * scale);
          float v;
          switch (epi) {
          case ORC_EPI_BIAS_FULL: {
            /* c = acc.to(dtype); c = c + bias  -- the add is done in the
             * half-precision type: exact fp32 sum of two half values rounded
             * once to the half type is the IEEE half add. */
            float cv = round_to(acc, out_dt);
            float bv = load_elem(bias, (om + i) * ldbias + on + j, out_dt);
            v = cv + bv;
            break;
          }
          case ORC_EPI_BIAS_ROW_GELU:
            v = gelu_erf(acc + load_elem(bias, on + j, ORC_F32));
            break;
          case ORC_EPI_BIAS_ROW:
            v = acc + load_elem(bias, on + j, ORC_F32);
            break;
          case ORC_EPI_LEAKY_RELU:
            v = acc >= 0.0f ? acc : 0.01f * acc;
            break;
          default:
            v = acc;
          }
          store_elem(c, (om + i) * ldc + on + j, out_dt, v);
        }
      }
    }
    free(accf); free(accd); free(at); free(bt);
  }
  return 0;
}

/*
 * matmul_kernel, the pointer-based kernel on tile-major operands
 * (examples/matmul/03-matrix-multiplication.py:242-391; leaky_relu :396-397).
 * TILE_M/N/K are the BLOCK sizes (:262-264).  Element (m,k) of A lives at
 *   ((m / TILE_M) * num_tiles_k + k / TILE_K) * TILE_M*TILE_K + (m % TILE_M) * TILE_K + k % TILE_K   (:326-337)
 * element (k,n) of B at
 *   ((k / TILE_K) * num_tiles_n + n / TILE_N) * TILE_K*TILE_N + (k % TILE_K) * TILE_N + n % TILE_N   (:349-357)
 * and element (m,n) of C at the same form with (TILE_M, TILE_N, num_tiles_n)                        (:377-385).
 * Row and column indices are wrapped (offs_m % M, offs_n % N, :308-309), loads are
 * masked on k < K only (:340-342, 359-361), the store on m < M and n < N (:387-388).
 * acc is fp32 (:320), the activation acts on it before the cast (:370-374), and the
 * result is always cast to fp16 (:374).  The strides in the signature are not used
 * by the kernel (:251-253) and are not taken here.  Programs are split over workers
 * as in orc_matmul; the program id is decoded by orc_tile_of_pid_pointer (:273-282).
 */
ORC_API int orc_matmul_tiled(const void *a, const void *b, void *c, int32_t M, int32_t N, int32_t K,
                             int32_t BM, int32_t BN, int32_t BK, int32_t group_m, int32_t grid,
                             int in_dt, int leaky_relu, int acc64, int nthreads) {
  if (BM <= 0 || BN <= 0 || BK <= 0 || group_m <= 0 || M <= 0 || N <= 0) return -1;
  int num_pid_m = (M + BM - 1) / BM, num_pid_n = (N + BN - 1) / BN;
  if (grid > num_pid_m * num_pid_n) return -2;
  nthreads = pick_threads(nthreads);
  const int64_t ntk = (K + BK - 1) / BK, ntn = num_pid_n;
#pragma omp parallel num_threads(nthreads)
  {
#ifdef _OPENMP
    int w = omp_get_thread_num(), nw = omp_get_num_threads();
#else
    int w = 0, nw = 1;
#endif
    float *accf = (float *)malloc(sizeof(float) * (size_t)BM * BN);
    double *accd = acc64 ? (double *)malloc(sizeof(double) * (size_t)BM * BN) : NULL;
    float *at = (float *)malloc(sizeof(float) * (size_t)BM * BK);
    float *bt = (float *)malloc(sizeof(float) * (size_t)BK * BN);
    int64_t bs, be;
    orc_block_range(grid, nw, w, &bs, &be);
    for (int64_t pid = bs; pid < be; ++pid) {
      int pid_m, pid_n;
      orc_tile_of_pid_pointer((int)pid, num_pid_m, num_pid_n, group_m, &pid_m, &pid_n);
      int64_t om = (int64_t)pid_m * BM, on = (int64_t)pid_n * BN;
      for (int i = 0; i < BM * BN; ++i) accf[i] = 0.0f;
      if (acc64) for (int i = 0; i < BM * BN; ++i) accd[i] = 0.0;
      for (int64_t kt = 0; kt < ntk; ++kt) {
        for (int i = 0; i < BM; ++i) {
          int64_t m = (om + i) % M;
          for (int k = 0; k < BK; ++k) {
            int64_t kk = kt * BK + k;
            int64_t off = ((m / BM) * ntk + kk / BK) * ((int64_t)BM * BK) + (m % BM) * BK + kk % BK;
            at[i * BK + k] = kk < K ? load_elem(a, off, in_dt) : 0.0f;
          }
        }
        for (int k = 0; k < BK; ++k) {
          int64_t kk = kt * BK + k;
          for (int j = 0; j < BN; ++j) {
            int64_t n = (on + j) % N;
            int64_t off = ((kk / BK) * ntn + n / BN) * ((int64_t)BK * BN) + (kk % BK) * BN + n % BN;
            bt[k * BN + j] = kk < K ? load_elem(b, off, in_dt) : 0.0f;
          }
        }
        for (int i = 0; i < BM; ++i)
          for (int k = 0; k < BK; ++k) {
            float av = at[i * BK + k];
            const float *brow = bt + (size_t)k * BN;
            if (!acc64) {
              float *arow = accf + (size_t)i * BN;
              for (int j = 0; j < BN; ++j) arow[j] += av * brow[j];
            } else {
              double *arow = accd + (size_t)i * BN;
              for (int j = 0; j < BN; ++j) arow[j] += (double)av * (double)brow[j];
            }
          }
      }
      for (int i = 0; i < BM; ++i) {
        if (om + i >= M) break;
        for (int j = 0; j < BN; ++j) {
          if (on + j >= N) break;
          float acc = acc64 ? (float)accd[(size_t)i * BN + j] : accf[(size_t)i * BN + j];
          if (leaky_relu) acc = acc >= 0.0f ? acc : 0.01f * acc;
          int64_t m = om + i, n = on + j;
          int64_t off = ((m / BM) * ntn + n / BN) * ((int64_t)BM * BN) + (m % BM) * BN + n % BN;
          store_elem(c, off, ORC_F16, acc);
        }
      }
    }
    free(accf); free(accd); free(at); free(bt);
  }
  return 0;
}

/* ------------------------------------------------------------------ */
/* Fused attention forward                                             */
/* ------------------------------------------------------------------ */

/*
 * _attn_fwd + _attn_fwd_inner (examples/fused-attn/06-fused-attention.py:143-215,
 * 33-90).  q,k,v,o are bf16 viewed as 2-D [Z*H*N_CTX, D] with strides [D,1]
 * (:243-246); Mout is fp32 [Z*H*N_CTX].  grid = (cdiv(N_CTX,BLOCK_M), Z*H, 1)
 * (:253-254); linear block index b decodes to start_m = b % gridX,
 * off_hz = b / gridX.  stage = 3 causal, 1 non-causal (:235).
 * Recipe restated line by line:
 *   qk_scale = sm_scale * 1.44269504                       (:188-189)
 *   m_i = -inf, l_i = 1.0, acc = 0                          (:184-186)
 *   off-band blocks:  m_ij = max(m_i, rowmax(qk)*qk_scale);
 *                     qk = qk*qk_scale - m_ij               (:63-64)
 *   on-band block:    qk = qk*qk_scale + (m >= n ? 0 : -1.0e6);
 *                     m_ij = max(m_i, rowmax(qk)); qk -= m_ij (:57-61)
 *   p = exp2(qk); alpha = exp2(m_i - m_ij); l_ij = rowsum(p) in fp32 (:65-68)
 *   acc = acc*alpha + dot(bf16(p), v)                       (:79-83)
 *   l_i = l_i*alpha + l_ij; m_i = m_ij                      (:86-87)
 *   epilogue: m_i += log2(l_i); acc /= l_i; store M, bf16(acc) (:211-215)
 */
static void attn_block(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                       uint16_t *o, float *Mout, float sm_scale, int H, int N_CTX, int D,
                       int BLOCK_M, int BLOCK_N, int stage, int start_m, int off_hz,
                       float *qf, float *acc, float *qk, float *m_i, float *l_i) {
  (void)H;
  int64_t offset_y = (int64_t)off_hz * N_CTX; /* off_z*(N_CTX*H) + off_h*N_CTX */
  int64_t qo = offset_y + (int64_t)start_m * BLOCK_M;
  float qk_scale = sm_scale * 1.44269504f;
  int rows = BLOCK_M;
  if ((int64_t)start_m * BLOCK_M + rows > N_CTX) rows = N_CTX - start_m * BLOCK_M;
  for (int i = 0; i < rows; ++i) {
    m_i[i] = -INFINITY;
    l_i[i] = 1.0f;
    for (int d = 0; d < D; ++d) {
      acc[(size_t)i * D + d] = 0.0f;
      qf[(size_t)i * D + d] = bf16_to_f32(q[(qo + i) * D + d]);
    }
  }
  for (int pass = 0; pass < 2; ++pass) {
    int inner; /* STAGE seen by _attn_fwd_inner */
    if (pass == 0) { if (!(stage & 1)) continue; inner = 4 - stage; }
    else { if (!(stage & 2)) continue; inner = 2; }
    int lo, hi;
    if (inner == 1) { lo = 0; hi = start_m * BLOCK_M; }
    else if (inner == 2) { lo = start_m * BLOCK_M; hi = (start_m + 1) * BLOCK_M; }
    else { lo = 0; hi = N_CTX; }
    for (int start_n = lo; start_n < hi; start_n += BLOCK_N) {
      int cols = BLOCK_N;
      for (int i = 0; i < rows; ++i) {
        int om = start_m * BLOCK_M + i;
        float rmax = -INFINITY;
        for (int j = 0; j < cols; ++j) {
          int64_t kn = start_n + j;
          float s = 0.0f;
          if (kn < N_CTX) { /* rows past the tensor read as zero */
            const uint16_t *kr = k + (offset_y + kn) * D;
            const float *qr = qf + (size_t)i * D;
            for (int d = 0; d < D; ++d) s += qr[d] * bf16_to_f32(kr[d]);
          }
          if (inner == 2) s = s * qk_scale + (om >= start_n + j ? 0.0f : -1.0e6f);
          qk[j] = s;
          if (s > rmax) rmax = s;
        }
        float m_ij;
        if (inner == 2) {
          m_ij = fmaxf(m_i[i], rmax);
          for (int j = 0; j < cols; ++j) qk[j] -= m_ij;
        } else {
          m_ij = fmaxf(m_i[i], rmax * qk_scale);
          for (int j = 0; j < cols; ++j) qk[j] = qk[j] * qk_scale - m_ij;
        }
        float l_ij = 0.0f;
        for (int j = 0; j < cols; ++j) { qk[j] = exp2f(qk[j]); l_ij += qk[j]; }
        float alpha = exp2f(m_i[i] - m_ij);
        float *ar = acc + (size_t)i * D;
        for (int d = 0; d < D; ++d) ar[d] *= alpha;
        for (int j = 0; j < cols; ++j) {
          int64_t kn = start_n + j;
          if (kn >= N_CTX) continue;
          float p = bf16_to_f32(f32_to_bf16(qk[j]));
          const uint16_t *vr = v + (offset_y + kn) * D;
          for (int d = 0; d < D; ++d) ar[d] += p * bf16_to_f32(vr[d]);
        }
        l_i[i] = l_i[i] * alpha + l_ij;
        m_i[i] = m_ij;
      }
    }
  }
  for (int i = 0; i < rows; ++i) {
    Mout[qo + i] = m_i[i] + log2f(l_i[i]);
    float *ar = acc + (size_t)i * D;
    for (int d = 0; d < D; ++d) o[(qo + i) * D + d] = f32_to_bf16(ar[d] / l_i[i]);
  }
}

ORC_API int orc_attn_fwd(float sm_scale, float *Mout, int32_t Z, int32_t H,
                         const uint16_t *q, const uint16_t *k, const uint16_t *v,
                         uint16_t *o, int32_t N_CTX, int32_t D, int32_t BLOCK_M,
                         int32_t BLOCK_N, int32_t stage, int32_t grid_x, int32_t grid_y,
                         int nthreads) {
  if (BLOCK_N > D) return -1;               /* static_assert(BLOCK_N <= HEAD_DIM) (:158) */
  if (stage != 1 && stage != 3) return -2;
  if (grid_y > Z * H) return -3;
  if ((int64_t)grid_x * BLOCK_M > N_CTX + BLOCK_M - 1) return -4;
  nthreads = pick_threads(nthreads);
  int64_t nblocks = (int64_t)grid_x * grid_y;
#pragma omp parallel num_threads(nthreads)
  {
#ifdef _OPENMP
    int w = omp_get_thread_num(), nw = omp_get_num_threads();
#else
    int w = 0, nw = 1;
#endif
    float *qf = (float *)malloc(sizeof(float) * (size_t)BLOCK_M * D);
    float *acc = (float *)malloc(sizeof(float) * (size_t)BLOCK_M * D);
    float *qk = (float *)malloc(sizeof(float) * (size_t)BLOCK_N);
    float *m_i = (float *)malloc(sizeof(float) * (size_t)BLOCK_M);
    float *l_i = (float *)malloc(sizeof(float) * (size_t)BLOCK_M);
    int64_t bs, be;
    orc_block_range(nblocks, nw, w, &bs, &be);
    for (int64_t b = bs; b < be; ++b) {
      int px, py, pz;
      orc_pid_decode(b, grid_x, grid_y, &px, &py, &pz);
      attn_block(q, k, v, o, Mout, sm_scale, H, N_CTX, D, BLOCK_M, BLOCK_N, stage, px, py,
                 qf, acc, qk, m_i, l_i);
    }
    free(qf); free(acc); free(qk); free(m_i); free(l_i);
  }
  return 0;
}

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
