// Fused attention forward for gfx950: _attn_fwd
// (examples/fused-attn/06-fused-attention.py:143-215, inner loop :33-90).
//
// Work layout: one wavefront owns 32 query rows of one (batch, head).  Both
// products are computed transposed so that every per-query quantity (running
// max m_i, running sum l_i, rescale alpha) lives in the lane that owns the
// query and never has to cross lanes:
//   S^T[key, q]  = K[key, :] . Q[q, :]      A = K rows,  B = Q rows
//   O^T[d,  q]  += V[key, d]^T . P^T[key,q]  A = V^T,     B = P^T
// v_mfma_f32_32x32x16_bf16 result register r of lane l is element
// [(r/4)*8 + (l/32)*4 + r%4][l%32], i.e. column l%32 = the query.
//
// Numerics follow the kernel source: qk_scale = sm_scale*1.44269504, exp2-based
// softmax, l_ij summed in fp32 before P is rounded to bf16, additive -1.0e6 on
// masked entries of the diagonal block, M = m_i + log2(l_i).
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));

#include "attention_args.h"

namespace {

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __builtin_bit_cast(float, (uint32_t)h << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
  r = ((u & 0x7fffffffu) > 0x7f800000u) ? (u | 0x00400000u) : r;
  return (uint16_t)(r >> 16);
}
__device__ __forceinline__ float xor32_max(float v) {
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float xor32_sum(float v) { return v + __shfl_xor(v, 32, 64); }

// Any HEAD_DIM in {16,32,64,128,256}; operands straight from global memory.
template <int D> __device__ __forceinline__ void attn_any_body(const AttnArgs &a) {
  constexpr int DK = D / 16;            // k-steps of the S^T product
  constexpr int DT = (D + 31) / 32;     // 32-row tiles of O^T
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c32 = lane & 31, g = lane >> 5;
  const int head = blockIdx.y;
  // heavy (late) query blocks first: under the causal mask they do the most work
  const int qblk = (int)gridDim.x - 1 - (int)blockIdx.x;
  const int q0 = qblk * 128 + wave * 32;
  if (q0 >= a.rows) return; // wave-uniform
  const int64_t base = (int64_t)head * a.n_ctx;
  const float qk_scale = a.sm_scale * 1.44269504f;

  union Frag { bf16x8 v; u16x8 u; uint16_t s[8]; };
  Frag qf[DK];
  {
    const uint16_t *qrow = a.q + (base + q0 + c32) * a.ldq;
#pragma unroll
    for (int s = 0; s < DK; ++s)
#pragma unroll
      for (int j = 0; j < 8; ++j) qf[s].s[j] = qrow[s * 16 + g * 8 + j];
  }
  f32x16 acc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc[t] = (f32x16){0};
  float m_i = -__builtin_inff(), l_i = 1.0f;
  const int my_q = q0 + c32;
  const int n_end = a.causal ? q0 + 32 : a.n_ctx;
  for (int n0 = 0; n0 < n_end; n0 += 32) {
    // S^T tile: 32 keys x 32 queries
    f32x16 st = {0};
    {
      const uint16_t *krow = a.k + (base + n0 + c32) * a.ldk;
#pragma unroll
      for (int s = 0; s < DK; ++s) {
        Frag kf;
#pragma unroll
        for (int j = 0; j < 8; ++j) kf.s[j] = krow[s * 16 + g * 8 + j];
        st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf.v, qf[s].v, st, 0, 0, 0);
      }
    }
    const bool on_band = a.causal && (n0 + 32 > q0); // the block that straddles the diagonal
    float rmax = -__builtin_inff();
    float m_ij;
    if (on_band) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = n0 + (r >> 2) * 8 + g * 4 + (r & 3);
        st[r] = st[r] * qk_scale + (my_q >= key ? 0.0f : -1.0e6f);
        rmax = fmaxf(rmax, st[r]);
      }
      rmax = xor32_max(rmax);
      m_ij = fmaxf(m_i, rmax);
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] -= m_ij;
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) rmax = fmaxf(rmax, st[r]);
      rmax = xor32_max(rmax);
      m_ij = fmaxf(m_i, rmax * qk_scale);
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] = st[r] * qk_scale - m_ij;
    }
    float l_ij = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      st[r] = __builtin_amdgcn_exp2f(st[r]);
      l_ij += st[r];
    }
    l_ij = xor32_sum(l_ij);
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_ij);
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] *= alpha;
    // P^T fragments: k-step s uses result registers 8s..8s+7
    Frag pf[2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int j = 0; j < 8; ++j) pf[s].s[j] = f32_to_bf16(st[s * 8 + j]);
    // O^T += V^T . P^T
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      const int d = t * 32 + c32;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        Frag vf;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = n0 + s * 16 + (j >> 2) * 8 + g * 4 + (j & 3);
          vf.s[j] = (d < D) ? a.v[(base + key) * a.ldv + d] : (uint16_t)0;
        }
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[s].v, acc[t], 0, 0, 0);
      }
    }
    l_i = l_i * alpha + l_ij;
    m_i = m_ij;
  }
  // epilogue
  if (g == 0) a.m[base + my_q] = m_i + __builtin_log2f(l_i);
  uint16_t *orow = a.o + (base + my_q) * a.ldo;
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int d = t * 32 + r4 * 8 + g * 4;
      if (d < D) {
#pragma unroll
        for (int j = 0; j < 4; ++j) orow[d + j] = f32_to_bf16(acc[t][r4 * 4 + j] / l_i);
      }
    }
}

} // namespace

extern "C" {

#define ATTN_ANY(D)                                                                    \
  __global__ __launch_bounds__(256) void attn_any_d##D(AttnArgs a) { attn_any_body<D>(a); }
ATTN_ANY(16)
ATTN_ANY(32)
ATTN_ANY(64)
ATTN_ANY(128)
ATTN_ANY(256)

} // extern "C"
