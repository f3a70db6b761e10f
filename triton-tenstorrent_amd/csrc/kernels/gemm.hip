// Tile-matmul kernels for gfx950: matmul_kernel_tma, matmul_kernel_fused, the
// fp8-scaled sibling and the pointer-based matmul_kernel on tile-major buffers
// (examples/matmul_tensor_descriptor/09-persistent-matmul.py:102-145,
//  python/tutorials/09-matmul-fused.py:100-148,
//  examples/matmul/03-matrix-multiplication.py:242-391).
//
// gemm_any_*   : every shape, stride, tile size (multiples of 32), partial
//                logical grid, ragged edges with descriptor zero-padding and
//                clipped stores.  One wavefront owns one 32x32 piece of a
//                logical tile and walks K with v_mfma_f32_32x32x16, operands
//                straight from global memory.  Correctness path, not a fast one.
#include <type_traits>

#include "gemm_common.h"

namespace {

// Operand fragment of v_mfma_f32_32x32x16_{bf16,f16}: lane l holds row (A) or
// column (B) l%32 and the 8 consecutive k of group l/32.
template <int IN_DT> struct Frag;
template <> struct Frag<DT_BF16> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ uint16_t enc(const void *p, int64_t i) { return ((const uint16_t *)p)[i]; }
  static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Frag<DT_F16> {
  typedef f16x8 vec;
  static __device__ __forceinline__ uint16_t enc(const void *p, int64_t i) { return ((const uint16_t *)p)[i]; }
  static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
// e4m3 values are exactly representable in bf16 (3 mantissa bits, narrower
// exponent range), so the any-shape path widens them and reuses the bf16 MFMA.
template <> struct Frag<DT_FP8> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ uint16_t enc(const void *p, int64_t i) {
    return (uint16_t)(f32_bits(fp8_to_f32(((const uint8_t *)p)[i])) >> 16);
  }
  static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// Element offset of (r, c) in a tile-major buffer: tiles of TR x TC, row-major inside a tile,
// ntc tiles per tile row (03-matrix-multiplication.py:326-337).
__device__ __forceinline__ int64_t tiled_off(int64_t r, int64_t c, int TR, int TC, int64_t ntc) {
  return ((r / TR) * ntc + c / TC) * ((int64_t)TR * TC) + (r % TR) * TC + c % TC;
}

template <int IN_DT, int OUT_DT, bool TILED = false>
__device__ __forceinline__ void gemm_any_body(const GemmArgs &g) {
  using F = Frag<IN_DT>;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  const int sub_n = g.BN >> 5;
  const int spt = (g.BM >> 5) * sub_n; // 32x32 pieces per logical tile
  const int64_t items = (int64_t)g.grid * spt;
  const int64_t stride = (int64_t)gridDim.x * waves_per_block;
  const int r32 = lane & 31, kg = lane >> 5;
  const int64_t ntk = (g.K + g.BK - 1) / g.BK, ntn = g.num_pid_n; // tile-major only
  for (int64_t it = (int64_t)blockIdx.x * waves_per_block + wave; it < items; it += stride) {
    const int pid = (int)(it / spt), sub = (int)(it % spt);
    int pid_m, pid_n;
    if constexpr (TILED) tile_of_pid_pointer(pid, g.num_pid_m, g.num_pid_n, g.group_m, pid_m, pid_n);
    else tile_of_pid(pid, g.num_pid_m, g.num_pid_n, g.group_m, pid_m, pid_n);
    const int64_t m0 = (int64_t)pid_m * g.BM + (sub / sub_n) * 32;
    const int64_t n0 = (int64_t)pid_n * g.BN + (sub % sub_n) * 32;
    if (m0 >= g.M || n0 >= g.N) continue; // piece lies wholly in the padding (wave-uniform)
    const int64_t am = m0 + r32, bn = n0 + r32;
    const bool am_ok = am < g.M, bn_ok = bn < g.N;
    f32x16 acc = {0};
    // a descriptor with NaN padding pads the last BLOCK_SIZE_K step, so the walk then runs to the end of that step
    const int k_end = (!TILED && (g.pad_a | g.pad_b)) ? (g.K + g.BK - 1) / g.BK * g.BK : g.K;
    for (int k0 = 0; k0 < k_end; k0 += 16) {
      union { typename F::vec v; uint16_t s[8]; } a, b;
      const int kb = k0 + kg * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = kb + j;
        const bool k_ok = k < g.K;
        if constexpr (TILED) {
          a.s[j] = (am_ok && k_ok) ? F::enc(g.a, tiled_off(am, k, g.BM, g.BK, ntk)) : (uint16_t)0;
          b.s[j] = (bn_ok && k_ok) ? F::enc(g.b, tiled_off(k, bn, g.BK, g.BN, ntn)) : (uint16_t)0;
        } else {
          a.s[j] = (am_ok && k_ok) ? F::enc(g.a, am * g.lda + k) : (k < k_end ? g.pad_a : (uint16_t)0);
          b.s[j] = (bn_ok && k_ok) ? F::enc(g.b, (int64_t)k * g.ldb + bn) : (k < k_end ? g.pad_b : (uint16_t)0);
        }
      }
      acc = F::mfma(a.v, b.v, acc);
    }
    // accumulator register r of lane l is C[(r/4)*8 + (l/32)*4 + r%4][l%32]
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int64_t m = m0 + (r >> 2) * 8 + kg * 4 + (r & 3);
      const int64_t n = n0 + r32;
      if (m < g.M && n < g.N) {
        float v = apply_epilogue<OUT_DT>(g, acc[r] * g.scale, m, n);
        store_from_f32<OUT_DT>(g.c, TILED ? tiled_off(m, n, g.BM, g.BN, ntn) : m * g.ldc + n, v);
      }
    }
  }
}

} // namespace

extern "C" {

#define GEMM_ANY(name, IN, OUT)                                                        \
  __global__ __launch_bounds__(256) void name(GemmArgs g) { gemm_any_body<IN, OUT>(g); }

GEMM_ANY(gemm_any_bf16_bf16, DT_BF16, DT_BF16)
GEMM_ANY(gemm_any_f16_f16, DT_F16, DT_F16)
GEMM_ANY(gemm_any_fp8_bf16, DT_FP8, DT_BF16)
GEMM_ANY(gemm_any_fp8_f16, DT_FP8, DT_F16)
GEMM_ANY(gemm_any_fp8_fp8, DT_FP8, DT_FP8)

// matmul_kernel: tile-major operands, fp16 result whatever the input type
// (03-matrix-multiplication.py:374)
__global__ __launch_bounds__(256) void gemm_anytiled_f16_f16(GemmArgs g) { gemm_any_body<DT_F16, DT_F16, true>(g); }
__global__ __launch_bounds__(256) void gemm_anytiled_bf16_f16(GemmArgs g) { gemm_any_body<DT_BF16, DT_F16, true>(g); }

} // extern "C"

// Second half of a launch whose K was cut into slices (gemm_splitk_* in gemm_tile.h): g.a is the workspace of
// g.ksplit slabs of M x N fp32 sums.  A thread adds the slabs of eight neighbouring columns in slice order (so the
// result does not depend on which workgroup finished when), applies scale and epilogue as the one-pass kernels do
// and stores sixteen bytes of C.  Row-major C: N is a multiple of 8.  Tile-major C (g.tiled: 32x32 tiles, any N):
// eight neighbouring columns lie inside one tile; a group that reaches past N goes by element, and the padding of the
// buffer is never written.
template <int OUT_DT> __device__ __forceinline__ void splitk_reduce_body(const GemmArgs &g) {
  const int64_t n8 = g.ldws / 8, groups = (int64_t)g.M * n8, slab = (int64_t)g.M * g.ldws;
  const float *ws = (const float *)g.a;
  for (int64_t it = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; it < groups; it += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = it / n8, n = (it - m * n8) * 8;
    const float *p = ws + m * g.ldws + n;
    f32x4 lo, hi;
    // the slabs' loads all in flight before the first addition (a loop of dependent loads took one memory round trip
    // per slab); the additions stay in slice order
    auto sum_of = [&](auto s_) __attribute__((always_inline)) {
      constexpr int S = decltype(s_)::value;
      f32x4 l[S], h[S];
#pragma unroll
      for (int sl = 0; sl < S; ++sl) {
        l[sl] = *(const f32x4 *)(p + sl * slab);
        h[sl] = *(const f32x4 *)(p + sl * slab + 4);
      }
      lo = l[0];
      hi = h[0];
#pragma unroll
      for (int sl = 1; sl < S; ++sl) {
        lo += l[sl];
        hi += h[sl];
      }
    };
    switch (g.ksplit) {
    case 2: sum_of(std::integral_constant<int, 2>{}); break;
    case 4: sum_of(std::integral_constant<int, 4>{}); break;
    case 8: sum_of(std::integral_constant<int, 8>{}); break;
    case 16: sum_of(std::integral_constant<int, 16>{}); break;
    default:
      lo = *(const f32x4 *)p;
      hi = *(const f32x4 *)(p + 4);
      for (int sl = 1; sl < g.ksplit; ++sl) {
        lo += *(const f32x4 *)(p + sl * slab);
        hi += *(const f32x4 *)(p + sl * slab + 4);
      }
    }
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = apply_epilogue<OUT_DT>(g, (e < 4 ? lo[e] : hi[e - 4]) * g.scale, m, n + e);
    u32x4 pk;
#pragma unroll
    for (int w = 0; w < 4; ++w)    // rounded as the one-pass kernels round
      pk[w] = OUT_DT == DT_BF16 ? pack_bf16x2(v[2 * w], v[2 * w + 1])
                                : (uint32_t)f32_to_f16(v[2 * w]) | ((uint32_t)f32_to_f16(v[2 * w + 1]) << 16);
    if (g.tiled) {
      const int64_t ntn = (g.N + 31) / 32;
      uint16_t *dst = (uint16_t *)g.c + (((m >> 5) * ntn + (n >> 5)) << 10) + (m & 31) * 32 + (n & 31);
      if (n + 8 <= g.N) {
        *(u32x4 *)dst = pk;
      } else {
        for (int e = 0; n + e < g.N; ++e) dst[e] = (uint16_t)(e & 1 ? pk[e >> 1] >> 16 : pk[e >> 1] & 0xffffu);
      }
    } else {
      *(u32x4 *)((uint16_t *)g.c + m * g.ldc + n) = pk;
    }
  }
}
extern "C" {
__global__ __launch_bounds__(256) void gemm_splitk_reduce_bf16(GemmArgs g) { splitk_reduce_body<DT_BF16>(g); }
__global__ __launch_bounds__(256) void gemm_splitk_reduce_f16(GemmArgs g) { splitk_reduce_body<DT_F16>(g); }

} // extern "C"

#include "gemm_tile.h"
#include "gemm_tile_fp8.h"
