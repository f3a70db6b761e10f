// Shared device-side pieces of the tile-matmul kernels: argument block, type
// conversions, the GROUP_SIZE_M tile order and the epilogues.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// element type codes (same values as tt_dtype in the C ABI header)
#define DT_F32 0
#define DT_I32 1
#define DT_BF16 2
#define DT_F16 3
#define DT_FP8 4

// epilogue codes (same values as tt_epilogue)
#define EPI_NONE 0
#define EPI_BIAS_FULL 1
#define EPI_BIAS_ROW_GELU 2
#define EPI_LEAKY_RELU 3
#define EPI_BIAS_ROW 4

#include "gemm_args.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }
// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
  r = ((u & 0x7fffffffu) > 0x7f800000u) ? (u | 0x00400000u) : r;
  return (uint16_t)(r >> 16);
}
// two fp32 -> packed bf16 pair (lo in bits 0-15) with one v_cvt_pk_bf16_f32: round to nearest even
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f); // v_cvt_f16_f32: RNE
}
// OCP e4m3fn -> fp32, exact
__device__ __forceinline__ float fp8_to_f32(uint8_t b) {
  uint32_t sign = (uint32_t)(b & 0x80u) << 24;
  uint32_t exp = (b >> 3) & 0xfu, man = b & 7u;
  float sub = (float)man * 0.001953125f;
  uint32_t nrm = ((exp + 120u) << 23) | (man << 20);
  uint32_t mag = exp == 0 ? f32_bits(sub) : nrm;
  mag = (exp == 15 && man == 7) ? 0x7fc00000u : mag;
  return bits_f32(sign | mag);
}
// fp32 -> e4m3fn, round-to-nearest-even, saturating at +-448
__device__ __forceinline__ uint8_t f32_to_fp8(float f) {
  uint32_t u = f32_bits(f);
  uint32_t sign = (u >> 24) & 0x80u;
  float a = __builtin_fabsf(f);
  uint32_t code;
  if (a != a) code = 0x7f;
  else if (a >= 448.0f) code = 0x7e;
  else if (a < 0.015625f) code = (uint32_t)__builtin_rintf(a * 512.0f);
  else {
    uint32_t au = f32_bits(a);
    au += 0x7ffffu + ((au >> 20) & 1u);
    code = (((au >> 23) - 120u) << 3) | ((au >> 20) & 7u);
    code = code > 0x7eu ? 0x7eu : code;
  }
  return (uint8_t)(sign | code);
}

template <int DT> __device__ __forceinline__ float load_as_f32(const void *p, int64_t i) {
  if constexpr (DT == DT_BF16) return bf16_to_f32(((const uint16_t *)p)[i]);
  else if constexpr (DT == DT_F16) return f16_to_f32(((const uint16_t *)p)[i]);
  else if constexpr (DT == DT_FP8) return fp8_to_f32(((const uint8_t *)p)[i]);
  else return ((const float *)p)[i];
}
template <int DT> __device__ __forceinline__ float round_through(float v) {
  if constexpr (DT == DT_BF16) return bf16_to_f32(f32_to_bf16(v));
  else if constexpr (DT == DT_F16) return f16_to_f32(f32_to_f16(v));
  else if constexpr (DT == DT_FP8) return fp8_to_f32(f32_to_fp8(v));
  else return v;
}
template <int DT> __device__ __forceinline__ void store_from_f32(void *p, int64_t i, float v) {
  if constexpr (DT == DT_BF16) ((uint16_t *)p)[i] = f32_to_bf16(v);
  else if constexpr (DT == DT_F16) ((uint16_t *)p)[i] = f32_to_f16(v);
  else if constexpr (DT == DT_FP8) ((uint8_t *)p)[i] = f32_to_fp8(v);
  else ((float *)p)[i] = v;
}

// pid -> (pid_m, pid_n), the GROUP_SIZE_M order of
// examples/matmul_tensor_descriptor/09-persistent-matmul.py:118-126
__device__ __forceinline__ void tile_of_pid(int pid, int num_pid_m, int num_pid_n, int group_m,
                                            int &pid_m, int &pid_n) {
  int num_pid_in_group = group_m * num_pid_n;
  int group_id = pid / num_pid_in_group;
  int first_pid_m = group_id * group_m;
  int group_size_m = min(num_pid_m - first_pid_m, group_m);
  pid_m = first_pid_m + (pid % group_size_m);
  pid_n = (pid % num_pid_in_group) / group_size_m;
}

// The pointer-based matmul_kernel takes the row from the position inside the group
// (examples/matmul/03-matrix-multiplication.py:281); the two decodes differ only in a last, shorter group.
__device__ __forceinline__ void tile_of_pid_pointer(int pid, int num_pid_m, int num_pid_n, int group_m,
                                                    int &pid_m, int &pid_n) {
  int num_pid_in_group = group_m * num_pid_n;
  int group_id = pid / num_pid_in_group;
  int first_pid_m = group_id * group_m;
  int group_size_m = min(num_pid_m - first_pid_m, group_m);
  int in_group = pid % num_pid_in_group;
  pid_m = first_pid_m + (in_group % group_size_m);
  pid_n = in_group / group_size_m;
}

// erf-form GELU, 0.5*x*(1+erf(x/sqrt(2))).  erf by Abramowitz & Stegun 7.1.26,
// erf(z) = 1 - (a1 t + ... + a5 t^5) exp(-z^2) for z >= 0 with t = 1/(1 + p z): absolute error <= 1.5e-7,
// branch-free, one rcp and one exp2 instead of the library routine's ~40 operations (the epilogue runs on
// 256 accumulators per lane with the matrix pipe idle).  Written out in x itself, with z = |x|/sqrt(2),
//   gelu(x) = 0.5 (x + |x| erf(z)) = max(x, 0) - |x| * (0.5 (a1 t + ... + a5 t^5)) * exp2(-x^2 * 0.5 log2(e))
// so the scaling by 1/sqrt(2), the sign and the halving cost nothing: 11 VALU operations, rcp and exp2.
__device__ __forceinline__ float gelu_erf(float x) {
  const float ax = __builtin_fabsf(x);
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f * 0.70710678118654752440f, ax, 1.0f));
  float p = __builtin_fmaf(0.5f * 1.061405429f, t, 0.5f * -1.453152027f);
  p = __builtin_fmaf(p, t, 0.5f * 1.421413741f);
  p = __builtin_fmaf(p, t, 0.5f * -0.284496736f);
  p = __builtin_fmaf(p, t, 0.5f * 0.254829592f);
  p = p * t;
  const float e = __builtin_amdgcn_exp2f((x * -0.72134752044448170368f) * x);
  return __builtin_fmaf(-ax, p * e, __builtin_fmaxf(x, 0.0f));
}

// Epilogue on one fp32 accumulator value destined for C[m,n]; returns the fp32
// value that is then rounded once to the output type.
template <int OUT_DT>
__device__ __forceinline__ float apply_epilogue(const GemmArgs &g, float acc, int64_t m, int64_t n) {
  switch (g.epi) {
  case EPI_BIAS_FULL: {
    // c = acc.to(half); c = c + bias  (the add rounds once more, in the store)
    float cv = round_through<OUT_DT>(acc);
    return cv + load_as_f32<OUT_DT>(g.bias, m * g.ldbias + n);
  }
  case EPI_BIAS_ROW_GELU: return gelu_erf(acc + ((const float *)g.bias)[n]);
  case EPI_BIAS_ROW: return acc + ((const float *)g.bias)[n];
  case EPI_LEAKY_RELU: return acc >= 0.0f ? acc : 0.01f * acc;
  default: return acc;
  }
}

// Same, with the epilogue fixed at compile time (one kernel per epilogue keeps
// the unrolled fast-path epilogue free of per-element switches).
template <int OUT_DT, int EPI>
__device__ __forceinline__ float apply_epilogue_ct(const GemmArgs &g, float acc, int64_t m, int64_t n) {
  if constexpr (EPI == EPI_BIAS_FULL) {
    float cv = round_through<OUT_DT>(acc);
    return cv + load_as_f32<OUT_DT>(g.bias, m * g.ldbias + n);
  } else if constexpr (EPI == EPI_BIAS_ROW_GELU) {
    return gelu_erf(acc + ((const float *)g.bias)[n]);
  } else if constexpr (EPI == EPI_BIAS_ROW) {
    return acc + ((const float *)g.bias)[n];
  } else if constexpr (EPI == EPI_LEAKY_RELU) {
    return acc >= 0.0f ? acc : 0.01f * acc;
  } else {
    return acc;
  }
}
