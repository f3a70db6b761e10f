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
// masked entries of the diagonal block, M = m_i + log2(l_i).  The causal mask is
// evaluated as the source does at BLOCK_M = 32, whatever BLOCK_M the launch names:
// -1.0e6 inside the 32x32 tile on the diagonal, keys past it not visited.  At a
// larger BLOCK_M the source adds -1.0e6 to those keys as well, which differs only
// where a masked score exceeds the unmasked ones by more than 1e6.
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
// two fp32 -> packed bf16 pair (lo in bits 0-15) with one v_cvt_pk_bf16_f32: round to nearest even
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// Reductions across the two wavefront halves.  v_permlane32_swap exchanges the high half of
// its first register with the low half of its second: fed v twice it leaves the low half's
// value in every lane of the first and the high half's in every lane of the second.  Written
// as asm because the compiler's builtin folds the second result into the first; the s_nop
// covers the two wait states the instruction needs after a VALU write of its operands.
struct Halves { float lo, hi; };
__device__ __forceinline__ Halves halves_of(float v) {
  Halves r = {v, v};
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(r.lo), "+v"(r.hi));
  return r;
}
__device__ __forceinline__ float xor32_max(float v) {
  const Halves r = halves_of(v);
  return fmaxf(r.lo, r.hi);
}
__device__ __forceinline__ float xor32_sum(float v) {
  const Halves r = halves_of(v);
  return r.lo + r.hi;
}

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

// ===========================================================================
// attn_tile_d{64,128}: the fast path (N_CTX a multiple of 256, 16-byte aligned
// contiguous rows, full grid).
//
// One workgroup = 8 wavefronts = 256 query rows of one (batch, head); K and V are
// streamed through LDS in blocks of 64 keys, double buffered, shared by all eight
// wavefronts; two wavefronts per SIMD, so one's softmax (VALU, exp2) overlaps the
// other's MFMAs.  The per-wavefront math is the transposed scheme described at the
// top of this file, with K fragments read row-wise (ds_read_b128) and V^T fragments
// read through the transposing ds_read_b64_tr_b16.
//
// LDS tiles are [key][d] with 16-byte chunks XOR-swizzled:
//   K: logical chunk c of row r sits at c ^ ((r / rows_per_256B) & (chunks-1))
//   V: logical chunk c of row r sits at c ^ (vswz(r) << 2)   (4-row x 64-byte reads)
// Global -> LDS copies are direct (global_load_lds_dwordx4), issued by wavefronts 4-7: thread
// t writes byte 16*(t-256) of each 4 KiB slab, the swizzle is applied to the global address.
//
// Workgroup order: a 1-D grid; ids are dealt round-robin to the 8 XCDs by the
// dispatcher, so id -> (xcd, slot) -> head = xcd*heads_per_xcd + slot/qblocks keeps
// every head's K/V inside one XCD's L2; within a head the late (heavy under the
// causal mask) query blocks go first.
// ===========================================================================
namespace fastattn {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;

constexpr int BN = 64;

// RAGGED: N_CTX a multiple of 32 but not of 256.  A wavefront is then either wholly inside the sequence or
// wholly outside it (it computes and stores nothing, but keeps up with the barriers and its share of the copies);
// the last key block may hold 32 keys only: its copies fetch the rows past N_CTX from the last row instead, the
// second 32-key tile is left out of both products and its scores count as -inf.
//
// WAVES = 4: 128 queries per workgroup, one wavefront per SIMD with the whole register file, all four wavefronts
// sharing the copies (how head dim 256 ran before attention_pipe256.h; no kernel instantiates it now).
// Issue priority of a wavefront over a block: 3 through the two MFMA phases, 1 through the softmax, 2 at the end of
// the block, never the default 0.  Measured A/B in one process (causal / not causal TFLOP/s): head dim 256 (one
// wavefront per SIMD) 575 -> 667 / 658 -> 766, and a constant priority of 3 does the same there, so what counts is
// leaving priority 0; head dim 32 495 -> 513 / 650 -> 665; head dim 128 on ragged lengths 827 -> 838 / 1017 -> 1024;
// head dim 64 is 0.5-1 % slower with any scheme tried and keeps the default.  The GEMM kernels do not react at all.
template <int D> __device__ __forceinline__ void attn_phase_prio(int phase) {
  if constexpr (D != 64) {
    switch (phase) {
    case 1: __builtin_amdgcn_s_setprio(1); break;
    case 3: __builtin_amdgcn_s_setprio(2); break;
    default: __builtin_amdgcn_s_setprio(3); break;
    }
  }
}
#define ATTN_SETPRIO(phase) attn_phase_prio<D>(phase)
template <int D, bool RAGGED = false, int WAVES = 8>
__device__ __forceinline__ void body(const AttnArgs &a, uint8_t *lds0, uint8_t *lds1) {
  constexpr int BM = WAVES * 32;
  constexpr int DK = D / 16;            // k-steps of S^T
  constexpr int DT = D / 32;            // 32-row tiles of O^T
  constexpr int ROW = D * 2;            // bytes per K/V row
  constexpr int CH = D / 8;             // 16-byte chunks per row
  constexpr int RPB = ROW >= 256 ? 1 : 256 / ROW;   // rows per 256 bytes (1 for D >= 128, 2 for D=64, 4 for D=32)
  constexpr int TILE = BN * ROW;        // bytes of one K (or V) tile
  constexpr int SLAB = 256 * 16;        // bytes one pass of the four copying wavefronts moves
  constexpr int NSLAB = TILE / SLAB;    // 4 for D=128, 2 for D=64
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, hi = lane >> 5;

  // ---- which (head, query block) ----
  const int qblocks = RAGGED ? (a.rows + BM - 1) / BM : a.rows / BM;
  const int total = qblocks * a.heads;
  int id = blockIdx.x;
  if (total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const int head = id / qblocks;
  const int qblk = qblocks - 1 - (id % qblocks);
  const int q0 = qblk * BM;
  const int qw = q0 + wave * 32;        // this wavefront's first query
  const int my_q = qw + c32;
  const int64_t base = (int64_t)head * a.n_ctx;
  const float qk_scale = a.sm_scale * 1.44269504f;
  const int n_end = a.causal ? (RAGGED ? min(q0 + BM, a.n_ctx) : q0 + BM) : a.n_ctx;
  const int nblk = RAGGED ? (n_end + BN - 1) / BN : n_end / BN;
  const bool live = !RAGGED || qw < a.n_ctx;   // wave-uniform

  // ---- global -> LDS copy constants ----
  // Only wavefronts 4-7 copy, thread t - 256 owning byte 16*(t - 256) of each slab: a copy instruction
  // holds up the issuing wavefront, and these are the ones that lose issue arbitration on their SIMD
  // anyway (the older wavefront wins), so the first four run on undisturbed (+2-3 % measured).
  // slab i covers rows i*(SLAB/ROW) ..; row = i*(SLAB/ROW) + t/CH, position t%CH
  const int ctid = tid & 255;
  const int crow = ctid / CH, cpos = ctid % CH;
  // the K swizzle follows the row's index in the tile; with 512-byte rows (D = 256) a slab holds 8 rows only, so
  // the chunk a thread fetches differs between slabs: NV variants, slab i uses variant i % NV
  constexpr int RPS = SLAB / ROW;                               // rows per slab
  constexpr int NV = (CH * RPB > RPS) ? (CH * RPB) / RPS : 1;   // 4 for D=256, else 1
  const int v_swz = (D >= 128) ? (crow & 3) : (D == 64) ? ((crow >> 1) & 1) : 0;   // D = 32: a row is the whole window
  const int v_chunk = cpos ^ (v_swz << 2);
  int k_chunks[NV];
  uint32_t k_voffs[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    k_chunks[j] = cpos ^ (((j * RPS + crow) / RPB) & (CH - 1));
    k_voffs[j] = (uint32_t)(((int64_t)crow * a.ldk + k_chunks[j] * 8) * 2);
  }
  const uint32_t v_voff = (uint32_t)(((int64_t)crow * a.ldv + v_chunk * 8) * 2);
  const int lds_wave = (wave & 3) * 1024;
  const uint8_t *kg = (const uint8_t *)(a.k + base * a.ldk);
  const uint8_t *vg = (const uint8_t *)(a.v + base * a.ldv);
  auto dma_one = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst) {
    const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(dst + lds_wave);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(src_uniform)
                 : "memory", "m0");
  };
  auto dma_block = [&](int blk, uint8_t *stage) { // K tile then V tile of key block blk
    if (WAVES == 8 && wave < 4) return;
    const int64_t row0 = (int64_t)blk * BN;
    if (RAGGED && row0 + BN > a.n_ctx) {
      // the half block at the end of the sequence: rows past it are fetched from its last row
      const int last = a.n_ctx - 1 - (int)row0;
#pragma unroll
      for (int i = 0; i < NSLAB; ++i) {
        const int r = min(i * (SLAB / ROW) + crow, last);
        dma_one(kg + row0 * a.ldk * 2, (uint32_t)(((int64_t)r * a.ldk + k_chunks[i % NV] * 8) * 2), stage + i * SLAB);
      }
#pragma unroll
      for (int i = 0; i < NSLAB; ++i) {
        const int r = min(i * (SLAB / ROW) + crow, last);
        dma_one(vg + row0 * a.ldv * 2, (uint32_t)(((int64_t)r * a.ldv + v_chunk * 8) * 2), stage + TILE + i * SLAB);
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < NSLAB; ++i)
      dma_one(kg + (row0 + i * (SLAB / ROW)) * a.ldk * 2, k_voffs[i % NV], stage + i * SLAB);
#pragma unroll
    for (int i = 0; i < NSLAB; ++i)
      dma_one(vg + (row0 + i * (SLAB / ROW)) * a.ldv * 2, v_voff, stage + TILE + i * SLAB);
  };

  // ---- fragment read constants ----
  // K (A operand of S^T): lane = key row c32 of a 32-key tile, chunk 2s+hi of its row
  const int k_rowoff = c32 * ROW;
  const int k_x = (c32 / RPB) & (CH - 1);
  // V^T (A operand of O^T) through transposing reads: see the B operand of the GEMM
  const int G4 = lane >> 4, i16 = lane & 15, qd = i16 >> 2;
  // key row within a 16-key step: h2*8 + hi*4 + qd ; d chunk (4 elems): dt*32 + (G4&1)*16 + (i16&3)*4
  const int v_key = hi * 4 + qd; // + h2*8 + step*16
  const int v_cc = (G4 & 1) * 2 + ((i16 >> 1) & 1); // 16-byte chunk within the 64-byte d-tile window
  const int v_half = (i16 & 1) << 3;

  // ---- Q fragments (B operand of S^T), straight from global ----
  union Frag { bf16x8 v; u16x8 u; s16x4 h[2]; uint32_t w[4]; };
  Frag qf[DK];
  if (live) {
    const uint16_t *qrow = a.q + (base + my_q) * a.ldq;
#pragma unroll
    for (int s = 0; s < DK; ++s) qf[s].u = *(const u16x8 *)(qrow + s * 16 + hi * 8);
    // Make the loads land here.  Otherwise the compiler defers its s_waitcnt vmcnt(n) for them into
    // the key loop, where n is wrong by the copies issued from assembly, which it cannot count: the
    // wait then sits behind every block's freshly issued copies and serialises their whole latency.
#pragma unroll
    for (int s = 0; s < DK; ++s) asm volatile("" : "+v"(qf[s].v));
  }
  f32x16 acc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc[t] = (f32x16){0};
  float m_i = -__builtin_inff(), l_i = 1.0f;

  dma_block(0, lds0);
  for (int b = 0; b < nblk; ++b) {
    uint8_t *cur = (b & 1) ? lds1 : lds0;
    uint8_t *nxt = (b & 1) ? lds0 : lds1;
    // block b has landed; every wave is done with the other stage
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (b + 1 < nblk) dma_block(b + 1, nxt);
    const int n0 = b * BN;
    if (!live || (a.causal && n0 > qw + 31)) continue; // outside the sequence, or wholly above this wavefront's diagonal
    ATTN_SETPRIO(0);
    const bool both = !RAGGED || n0 + 32 < n_end;      // the block's second 32-key tile exists (wave-uniform)

    // ---- S^T = K . Q^T : two 32-key tiles ----
    f32x16 st[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      st[kt] = (f32x16){0};
      if (RAGGED && kt == 1 && !both) {
#pragma unroll
        for (int r = 0; r < 16; ++r) st[1][r] = -__builtin_inff();
        break;
      }
      const uint8_t *kb = cur + kt * 32 * ROW + k_rowoff;
#pragma unroll
      for (int s = 0; s < DK; ++s) {
        Frag kf;
        kf.v = *(const bf16x8 *)(kb + (((2 * s + hi) ^ k_x) << 4));
        st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf.v, qf[s].v, st[kt], 0, 0, 0);
      }
    }
    // Order for the scheduler: fragment reads run four MFMAs ahead of their use (left to itself it puts a
    // read right in front of the MFMA that needs it, and half of the MFMAs then wait out the LDS latency).
    constexpr int AHEAD = 4;
    __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
    for (int i = 0; i < 2 * DK - AHEAD; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
    ATTN_SETPRIO(1);
    // ---- online softmax (per lane = per query; keys run over registers and the hi half) ----
    const bool on_band = a.causal && (n0 + BN - 1 > qw);
    float rmax = -__builtin_inff();
    float m_ij;
    if (on_band) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = n0 + kt * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          // additive -1.0e6 inside this wavefront's 32x32 tile on the diagonal, as the source does at BLOCK_M = 32;
          // the block's keys past that tile are not part of the product at all
          st[kt][r] = st[kt][r] * qk_scale + (my_q >= key ? 0.0f : (key > qw + 31 ? -__builtin_inff() : -1.0e6f));
          rmax = fmaxf(rmax, st[kt][r]);
        }
      rmax = xor32_max(rmax);
      m_ij = fmaxf(m_i, rmax);
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) st[kt][r] -= m_ij;
    } else {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) rmax = fmaxf(rmax, st[kt][r]);
      rmax = xor32_max(rmax);
      m_ij = fmaxf(m_i, rmax * qk_scale);
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) st[kt][r] = st[kt][r] * qk_scale - m_ij;
    }
    float l_ij = 0.0f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        st[kt][r] = __builtin_amdgcn_exp2f(st[kt][r]);
        l_ij += st[kt][r];
      }
    l_ij = xor32_sum(l_ij);
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_ij);
    // alpha == 1 for every query of the wavefront once the running maxima have settled:
    // multiplying by 1.0f is the identity, so the rescale can be skipped exactly
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] *= alpha;
    }
    l_i = l_i * alpha + l_ij;
    m_i = m_ij;
    ATTN_SETPRIO(2);
    // ---- P^T fragments: 16-key step k4 uses registers 8*(k4&1).. of st[k4>>1] ----
    Frag pf[4];
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        pf[k4].w[j] = pack_bf16x2(st[k4 >> 1][(k4 & 1) * 8 + 2 * j], st[k4 >> 1][(k4 & 1) * 8 + 2 * j + 1]);
    // ---- O^T += V^T . P^T ----
    const uint8_t *vb = cur + TILE;
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4) {
      if (RAGGED && k4 == 2 && !both) break;           // P is zero there; leave the clamped V rows out altogether
#pragma unroll
      for (int t = 0; t < DT; ++t) {
        Frag vf;
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const int key = k4 * 16 + h2 * 8 + v_key; // row in the tile
          const int swz = (D >= 128) ? (key & 3) : (D == 64) ? ((key >> 1) & 1) : 0;
          const int chunk = (t * 4 + v_cc) ^ (swz << 2);
          vf.h[h2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(vb + key * ROW + (chunk << 4) + v_half));
        }
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[k4].v, acc[t], 0, 0, 0);
      }
    }
    // the same for P.V: two transposing reads per fragment
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 1);
#pragma unroll
    for (int i = 0; i < 4 * DT - AHEAD; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 1);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 1);
    ATTN_SETPRIO(3);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (!live) return;
  // ---- epilogue ----
  if (hi == 0) a.m[base + my_q] = m_i + __builtin_log2f(l_i);
  uint16_t *orow = a.o + (base + my_q) * a.ldo;
  const float inv_l = 1.0f / l_i;
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int d = t * 32 + r4 * 8 + hi * 4;
      typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
      // one division per query, then multiplications: within one fp32 unit in the last place of acc / l_i, far
      // below the bf16 rounding that follows (a full division is ten instructions, and there are 4*D of them)
      u32x2_t pk = {pack_bf16x2(acc[t][r4 * 4 + 0] * inv_l, acc[t][r4 * 4 + 1] * inv_l),
                    pack_bf16x2(acc[t][r4 * 4 + 2] * inv_l, acc[t][r4 * 4 + 3] * inv_l)};
      *(u32x2_t *)(orow + d) = pk;
    }
}

} // namespace fastattn

extern "C" {

#define ATTN_TILE(D)                                                                       \
  __global__ __launch_bounds__(512) void attn_tile_d##D(AttnArgs a) {                      \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[2 * 64 * D * 2];                \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[2 * 64 * D * 2];                \
    fastattn::body<D>(a, lds0, lds1);                                                      \
  }
ATTN_TILE(32)
// head dim 128 on whole 256-query blocks: attention_pipe.h

#define ATTN_RAGGED(D)                                                                     \
  __global__ __launch_bounds__(512) void attn_ragged_d##D(AttnArgs a) {                    \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[2 * 64 * D * 2];                \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[2 * 64 * D * 2];                \
    fastattn::body<D, true>(a, lds0, lds1);                                                \
  }
ATTN_RAGGED(32)
// (head dim 64: attn_ragged_d64 in attention_pipe.h)

// (head dim 256: attn_tile_d256 and attn_ragged_d256 in attention_pipe256.h)

} // extern "C"

#include "attention_pipe.h"
#include "attention_pipe256.h"
