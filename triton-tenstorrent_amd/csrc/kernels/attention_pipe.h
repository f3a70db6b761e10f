// attn_tile_d128, attn_ragged_d128, attn_tile_d64: _attn_fwd (examples/fused-attn/06-fused-attention.py:33-90,
// 143-215) at head dim 128 (whole 256-query blocks, the configuration the fused-attention benchmark is quoted on, and
// any length that is a whole number of 32-query tiles) and at head dim 64 (whole blocks).
//
// Same work layout and numerics as the kernels in attention.hip (one wavefront = 32 queries, both products
// transposed, K/V blocks of 64 keys in LDS), with the block loop written as a software pipeline:
//
//   block period j of a wavefront
//     phase 1   MFMA: S^T(j+1) = K(j+1) . Q^T          VALU: row maxima of S^T(j), alpha, rescale, first exps
//     -------   s_waitcnt vmcnt(0) + s_barrier  (block j+2 has landed; block j-1's stage is free)
//     phase 2   MFMA: O^T += V(j)^T . P^T(j)           VALU: the remaining exps, row sums
//                                                      copies: block j+3 into the freed stage, one per four MFMAs
//
// so that every MFMA has softmax work of another block to issue in its shadow, in one instruction stream.  What
// that needs: a ring of four 32 KiB stages (blocks j .. j+3), two sets of score registers that swap roles every
// block (the main loop is unrolled by four: stage offsets become instruction immediates, and no register is
// copied), and the first fragment reads of each phase issued during the phase before (K(j+2) is visible from the
// barrier of period j on, V(j) long before).  Fragment reads run one group of two MFMAs ahead.
//
// Measured on this kernel, one change at a time (4x32x4096x128, TFLOP/s causal / full mask, same box):
//   phases in sequence, two stages (attention.hip's body)           863 / 1024
//   + software pipeline, four stages, unrolled by four              867 / 1022
//   + barrier between the phases, cross-phase fragment prefetch     889 / 1046
//   + reference maximum raised only when outgrown by 2^8 (below)    936 / 1117
//   + query blocks i and n-1-i in one workgroup                    1015 / 1112
// and, measured against that kernel in one process on another box (996 / 1121 there):
//   + K tiles of all stages below 64 KiB of LDS, V tiles above: every fragment address is register + immediate (the
//     stage offsets no longer fit the instruction's 16-bit field otherwise: 18 VALU additions per block)
//   + falling issue priority over a phase (below)
//   + a workgroup's items back to back: each one's trailing copies fetch the first key blocks of the next, Q is
//     loaded behind the first copies, one workgroup per CU walks its share of the items      1027 / 1149
//
// Two stated differences from a literal evaluation of the source, both inside the tolerance of the parity tests:
//  * The exponent reference m_i of a row is the running maximum of the source, except that a new block maximum
//    replaces it only when some row of the wavefront exceeds its reference by more than 8 (log2 units).  Until
//    then p = exp2(s - m_i) may reach 2^8 instead of 1, l_i and the accumulator carry the same factor, and
//    O = acc / l_i and M = m_i + log2(l_i) are what they would be with the true maximum, up to rounding: every
//    quantity is floating point with the same relative precision at either scale.  What it saves is the
//    multiplication of the 64 accumulator registers by alpha, which with an exact running maximum is needed in
//    four of five blocks (some row out of 32 sees a new maximum).
//  * Keys are blocked by 64 whatever BLOCK_N says (fp32 summation order only), and the causal mask is evaluated as
//    the source does at BLOCK_M = 32: additive -1.0e6 inside the 32x32 tile on the diagonal, keys past it not
//    visited (at a larger BLOCK_M the source adds -1.0e6 to those too, which shows only in scores above 1e6).
#pragma once
#include <type_traits>

namespace pipeattn {

union Frag { bf16x8 v; u16x8 u; fastattn::s16x4 h[2]; uint32_t w[4]; };   // one MFMA operand: 8 bf16 of a lane

using fastattn::lds_s16x4;
using fastattn::lds_void;
using fastattn::s16x4;

#define PIPE_FENCE() __builtin_amdgcn_sched_barrier(0)

constexpr int BN = 64;        // keys per block
constexpr int NST = 4;        // LDS stages
constexpr int GK = 2, GV = 2; // fragments per read group
constexpr float LAZY_T = 8.0f;
// A wavefront's issue priority falls from 3 to 1 over each phase, a step every PRIO_STEP MFMAs: of the two
// wavefronts of a SIMD the one that is behind then wins arbitration.  Left alone the older wavefront always wins: it
// ran its phases in 1190 + 1020 cycles and waited 800 at the barrier for the other one's 1380 + 1560.
constexpr int PRIO_STEP = 4, PRIO_TOP = 3;
#define PIPE_PRIO_OF(step, steps) (PRIO_TOP - (step) * 2 / ((steps) - 1))   // 3, 3, 2, 1: never the default 0
__device__ __forceinline__ void set_prio(int p) {   // s_setprio takes an immediate
  switch (p) {
  case 0: __builtin_amdgcn_s_setprio(0); break;
  case 1: __builtin_amdgcn_s_setprio(1); break;
  case 2: __builtin_amdgcn_s_setprio(2); break;
  default: __builtin_amdgcn_s_setprio(3); break;
  }
}

// PREFETCHED: blocks 0, 1, 2 of this item are already in stages 0, 1, 2 (the item before it fetched them with its
// trailing copies).  next_head: the head of the item that follows in this workgroup (this item's own head when none
// does): this item's trailing copies fetch that head's first key blocks.  next_qblk: that item's query block, -1 when
// there is none.  Whole blocks: a wavefront's Q fragments (qf, the caller's) are dead once its last block's scores are
// done, so it loads the next item's Q into them before it normalises and stores this item's results, and a chained
// item starts with its Q on the way or there (the wavefronts that finish an item early have it long before): +1 % causal.
// (Loading it a phase earlier, behind the last P.V MFMAs, spills in the masked period: 20 % slower.)
//
// RAGGED: N_CTX is a whole number of 32-query wavefront tiles but not of 256-query blocks.  A wavefront whose tile lies
// past the end computes and stores nothing but keeps up with the barriers and its share of the copies; copies of rows
// past the end fetch the last 32 rows instead; keys past the end get a score of -inf (under the causal mask the
// diagonal block does that anyway); and the item's stream of blocks is padded to a multiple of four periods, so that
// the next item's first blocks land in stages 0, 1, 2 as they do for whole blocks.
template <int D, bool PREFETCHED, bool RAGGED = false>
__device__ __forceinline__ void body(const AttnArgs &a, uint8_t *lds, const int head, const int qblk, const int next_head,
                                     const int next_qblk, Frag (&qf)[D / 16]) {
  constexpr int BM = 256;
  constexpr int DK = D / 16, DT = D / 32, ROW = D * 2, CH = D / 8;
  constexpr int TILE = BN * ROW, STG = TILE, VBASE = NST * TILE;   // stage s: K at s*TILE, V at VBASE + s*TILE
  constexpr int RPB = 256 / ROW;               // rows per 256 bytes of LDS: the K swizzle advances every RPB rows
  constexpr int RPP = 8192 / ROW;              // rows that one copy instruction of the workgroup covers (512 x 16 B)
  constexpr int PPT = BN / RPP;                // such pieces per K or V tile
  constexpr int SLOTS = D / 8;                 // MFMAs per phase: 2*DK = 4*DT
  constexpr int SPS = 16 / SLOTS;              // softmax work items per MFMA slot
  static_assert(D == 128 || D == 64, "LDS swizzles exist for 256- and 128-byte rows");
  static_assert((NST & (NST - 1)) == 0, "the stage ring wraps with a mask");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, hi = lane >> 5;

  const int q0 = qblk * BM;
  // wavefronts s and s+4 share a SIMD: they take the 32-query sub-blocks s and 7-s, so that under the causal mask
  // every SIMD has the same number of key blocks to work through
  const int sub = wave < 4 ? wave : 11 - wave;
  const int qw = q0 + sub * 32;
  const int my_q = qw + c32;
  const int64_t base = (int64_t)head * a.n_ctx;
  const float qk_scale = a.sm_scale * 1.44269504f;
  const bool live = !RAGGED || qw < a.n_ctx;                      // wave-uniform
  const int kend = RAGGED ? (a.causal ? min(q0 + BM, a.n_ctx) : a.n_ctx) : 0;
  const int nblk = RAGGED ? (kend + BN - 1) / BN : (a.causal ? (q0 + BM) / BN : a.n_ctx / BN);   // key blocks of this item
  const int nstream = RAGGED ? (nblk + 3) & ~3 : nblk;            // periods the workgroup goes through (a multiple of 4)
  const int L = a.causal ? (qw + 31) / BN : nblk - 1;             // this wavefront's last block (the masked one when causal)
  const int last_rows = a.n_ctx - 32;                             // RAGGED: first row of the last 32 that exist

  // ---- copies: 512 threads x 16 B = 8 KiB per instruction round, two rounds per K or V tile ----
  const int crow = tid / CH, cpos = tid % CH;       // row within a round of RPP rows, chunk position
  const int k_chunk = cpos ^ ((crow / RPB) & (CH - 1));                       // K: logical chunk c of row r sits at c ^ ((r / RPB) & (CH-1))
  const int v_chunk = cpos ^ ((D == 128 ? (crow & 3) : ((crow >> 1) & 1)) << 2);   // V: at c ^ ((r & 3) << 2), 128-byte rows: c ^ (((r >> 1) & 1) << 2)
  const uint32_t k_voff = (uint32_t)(((int64_t)crow * a.ldk + k_chunk * 8) * 2);
  const uint32_t v_voff = (uint32_t)(((int64_t)crow * a.ldv + v_chunk * 8) * 2);
  // (RAGGED at 128-byte rows: the same with rows 32-63 of a tile fetched from rows 0-31, for a half block at the end)
  const uint32_t k_voff_half = (uint32_t)(((int64_t)(crow & 31) * a.ldk + k_chunk * 8) * 2);
  const uint32_t v_voff_half = (uint32_t)(((int64_t)(crow & 31) * a.ldv + v_chunk * 8) * 2);
  const uint8_t *kg = (const uint8_t *)(a.k + base * a.ldk);
  const uint8_t *vg = (const uint8_t *)(a.v + base * a.ldv);
  const uint8_t *kg_next = (const uint8_t *)(a.k + (int64_t)next_head * a.n_ctx * a.ldk);
  const uint8_t *vg_next = (const uint8_t *)(a.v + (int64_t)next_head * a.n_ctx * a.ldv);
  const int lds_wave = wave * 1024;
  auto dma_one = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst) {
    const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(dst + lds_wave);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(src_uniform)
                 : "memory", "m0");
  };
  // piece r (0, 1: the two halves of K; 2, 3: of V) of block blk into the stage at byte offset stage_o.  A block past
  // the last one is fetched from the last one again (a harmless refetch into a stage nobody reads any more), so
  // that every wavefront issues four copies per block period and the vmcnt waits are the same everywhere.
  auto dma_piece = [&](int blk, int stage_o, int r) {
    const bool own = blk < nstream;
    // (RAGGED: periods nblk .. nstream-1 are padding and refetch the last block; any 32 rows that do not exist are
    // fetched from the last 32 that do)
    int64_t row0 = (int64_t)(own ? (RAGGED ? min(blk, nblk - 1) : blk) : blk - nstream) * BN + (r % PPT) * RPP;
    uint32_t kvo = k_voff, vvo = v_voff;
    if constexpr (RAGGED && RPP == 64) {
      // (128-byte rows: one copy instruction is a whole 64-row tile.  A block at or past the end is fetched from the
      // last one that starts inside the sequence, and where that one is a half block its threads of rows 32-63
      // fetch rows 0-31 again)
      row0 = min(row0, (int64_t)((a.n_ctx - 1) / 64) * 64);
      if (row0 + 64 > a.n_ctx) {
        kvo = k_voff_half;
        vvo = v_voff_half;
      }
    } else if (RAGGED) {
      row0 = min(row0, (int64_t)last_rows);
    }
    if (r < PPT) dma_one((own ? kg : kg_next) + row0 * a.ldk * 2, kvo, lds + stage_o + (r % PPT) * 8192);
    else dma_one((own ? vg : vg_next) + row0 * a.ldv * 2, vvo, lds + VBASE + stage_o + (r % PPT) * 8192);
  };
  // The same for whole blocks only, from two running pointers (K and V rows of the block that is fetched next) instead
  // of a 64-bit product per piece: the pieces of a block are issued in order and the pointers step after the last one,
  // into the next item's keys when this item's run out.
  const int64_t kstep = (int64_t)BN * a.ldk * 2, vstep = (int64_t)BN * a.ldv * 2;
  const int64_t kpiece = (int64_t)RPP * a.ldk * 2, vpiece = (int64_t)RPP * a.ldv * 2;
  const uint8_t *kp = kg + 3 * kstep, *vp = vg + 3 * vstep;   // block 3: blocks 0..2 are the prologue's (or the item before's)
  auto dma_run = [&](int blk, int stage_o, int r) {
    if constexpr (RAGGED) {
      dma_piece(blk, stage_o, r);
    } else {
      if (r < PPT) dma_one(kp + (r % PPT) * kpiece, k_voff, lds + stage_o + (r % PPT) * 8192);
      else dma_one(vp + (r % PPT) * vpiece, v_voff, lds + VBASE + stage_o + (r % PPT) * 8192);
      if (r == 2 * PPT - 1) {
        const bool wrap = blk + 1 == nstream;
        kp = wrap ? kg_next : kp + kstep;
        vp = wrap ? vg_next : vp + vstep;
      }
    }
  };
  auto dma_block = [&](int blk, int stage_o) {
#pragma unroll
    for (int r = 0; r < 2 * PPT; ++r) dma_piece(blk, stage_o, r);
  };
  auto dma_block_run = [&](int blk, int stage_o) {
#pragma unroll
    for (int r = 0; r < 2 * PPT; ++r) dma_run(blk, stage_o, r);
  };

  // ---- fragment addresses ----
  int k_off[DK];                 // K (A operand of S^T): lane = key row c32 of a 32-key tile, chunk 2s+hi of its row
#pragma unroll
  for (int s = 0; s < DK; ++s) k_off[s] = c32 * ROW + (((2 * s + hi) ^ ((c32 / RPB) & (CH - 1))) << 4);
  const int G4 = lane >> 4, i16 = lane & 15, qd = i16 >> 2;
  const int v_cc = (G4 & 1) * 2 + ((i16 >> 1) & 1);
  int v_off[DT];                 // V^T (A operand of O^T) through transposing reads: key row hi*4+qd (+ k4*16 + h2*8)
#pragma unroll
  for (int t = 0; t < DT; ++t)
    v_off[t] = VBASE + (hi * 4 + qd) * ROW + (((t * 4 + v_cc) ^ ((D == 128 ? qd : ((qd >> 1) & 1)) << 2)) << 4) + ((i16 & 1) << 3);

  f32x16 acc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc[t] = (f32x16){0};
  float m_i = -__builtin_inff(), l_i = 1.0f;

  auto rdK = [&](const uint8_t *stage, int i) -> bf16x8 {   // fragment i: 32-key tile i&1, k-step i>>1
    return *(const bf16x8 *)(stage + (i & 1) * 32 * ROW + k_off[i >> 1]);
  };
  auto rdV = [&](const uint8_t *stage, int i) -> bf16x8 {   // fragment i: 16-key step i>>2, d-tile i&3
    Frag f;
    const int k4 = i / DT, t = i % DT;
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
      f.h[h2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(stage + v_off[t] + (k4 * 16 + h2 * 8) * ROW));
    return f.v;
  };

  // ---- prologue: blocks 0, 1, 2 in flight; S^T(0); the first K fragments of block 1 ----
  if constexpr (!PREFETCHED) {
    dma_block(0, 0);
    dma_block(1, STG);
    dma_block(2, 2 * STG);
  }
  // Q after the copies, so that the two round trips to memory overlap; the wait the compiler puts in front of the
  // first use of Q is for everything older as well, the copies included
  {
    if constexpr (!PREFETCHED || RAGGED) {   // (otherwise the item before this one loaded them)
      // (RAGGED: a wavefront past the end loads the last row that exists and never uses it)
      const uint16_t *qrow = a.q + (base + (RAGGED ? min(my_q, a.n_ctx - 1) : my_q)) * a.ldq;
#pragma unroll
      for (int s = 0; s < DK; ++s) qf[s].u = *(const u16x8 *)(qrow + s * 16 + hi * 8);
    }
    // the loads land here: the compiler's own vmcnt bookkeeping does not see the copies issued from assembly
#pragma unroll
    for (int s = 0; s < DK; ++s) asm volatile("" : "+v"(qf[s].v));
  }
  f32x16 s0[2], s1[2];   // scores of the current block and of the next, alternating roles
  if constexpr (!PREFETCHED) asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");   // every wavefront's copies have landed
  s0[0] = s0[1] = (f32x16){0};
#pragma unroll
  for (int i = 0; i < 2 * DK; ++i) s0[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rdK(lds, i), qf[i >> 1].v, s0[i & 1], 0, 0, 0);
  bf16x8 kpre[GK], vpre[GV];   // first fragment group of the coming phase, requested during the phase before
#pragma unroll
  for (int i = 0; i < GK; ++i) kpre[i] = rdK(lds + STG, i);

  // One block period of this wavefront.  LAST: no next block to start on; MASKED: the block on the diagonal.
  // cur_o, nxt_o, nn_o: byte offsets of the stages of blocks j, j+1, j+2; free_o: of the stage block j+3 goes into.
  // sc holds S^T(j) on entry, sn receives S^T(j+1).
  auto period = [&](int j, int cur_o, int nxt_o, int nn_o, int free_o, f32x16 (&sc)[2], f32x16 (&sn)[2], auto last_,
                    auto masked_) {
    constexpr bool LAST = decltype(last_)::value, MASKED = decltype(masked_)::value;
    const uint8_t *cur = lds + cur_o, *nxt = lds + nxt_o;
    bf16x8 kf[2 * GK], vf[2 * GV];
    float rmax0 = -__builtin_inff(), rmax1 = -__builtin_inff(), m_ij, alpha, l_ij = 0.0f;
    uint32_t pw[16];   // P^T as packed bf16 pairs: pw[k4*4 + jj]
    auto max_part = [&](int part) {   // part 0..3: 8 elements each
      const int kt = part >> 1, r0 = (part & 1) * 8;
      float &rm = kt ? rmax1 : rmax0;
#pragma unroll
      for (int r = 0; r < 8; r += 2) rm = fmaxf(fmaxf(rm, sc[kt][r0 + r]), sc[kt][r0 + r + 1]);
    };
    auto stats = [&]() {
      const float rmax = xor32_max(fmaxf(rmax0, rmax1));
      m_ij = MASKED ? fmaxf(m_i, rmax) : fmaxf(m_i, rmax * qk_scale);
      // the reference moves only when some row of the wavefront outgrew it by more than LAZY_T (then every row
      // takes its true running maximum); otherwise it stays, alpha is 1 and nothing is rescaled
      if (__builtin_amdgcn_ballot_w64(m_ij > m_i + LAZY_T) == 0) m_ij = m_i;
      alpha = __builtin_amdgcn_exp2f(m_i - m_ij);
    };
    auto rescale = [&]() {
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[t][r] *= alpha;
      }
    };
    auto exp_part = [&](int e) {     // e = 0..15: two elements -> one packed pair.  k4 = e>>2 uses sc[k4>>1][(k4&1)*8 ..]
      const int k4 = e >> 2, jj = e & 3;
      const int kt = k4 >> 1, r = (k4 & 1) * 8 + 2 * jj;
      float p0, p1;
      if (MASKED) {
        p0 = __builtin_amdgcn_exp2f(sc[kt][r] - m_ij);
        p1 = __builtin_amdgcn_exp2f(sc[kt][r + 1] - m_ij);
      } else {
        p0 = __builtin_amdgcn_exp2f(sc[kt][r] * qk_scale - m_ij);
        p1 = __builtin_amdgcn_exp2f(sc[kt][r + 1] * qk_scale - m_ij);
      }
      l_ij += p0;          // fp32 sum before the cast (06-fused-attention.py:67)
      l_ij += p1;
      pw[e] = pack_bf16x2(p0, p1);
    };
    auto pfrag = [&](int k4) -> bf16x8 {
      Frag f;
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) f.w[jj] = pw[k4 * 4 + jj];
      return f.v;
    };
    if constexpr (MASKED) {
      // the block on the diagonal: qk * qk_scale + where(mask, 0, -1.0e6) inside this wavefront's 32x32 tile
      // (06-fused-attention.py:58-59 at BLOCK_M = 32); keys past that tile are not part of the product
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = j * BN + kt * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          // (RAGGED, no causal mask: the block that ends past N_CTX; its keys past the end are not part of the product)
          const float add = (RAGGED && !a.causal) ? (key >= a.n_ctx ? -__builtin_inff() : 0.0f)
                                                  : (my_q >= key ? 0.0f : (key > qw + 31 ? -__builtin_inff() : -1.0e6f));
          sc[kt][r] = sc[kt][r] * qk_scale + add;
        }
    }
    if constexpr (!LAST) {
      // ---------- phase 1: S^T(j+1) MFMAs, softmax(j) VALU ----------
      sn[0] = sn[1] = (f32x16){0};
#pragma unroll
      for (int i = 0; i < GK; ++i) kf[i] = kpre[i];
#pragma unroll
      for (int i = 0; i < 2 * DK; ++i) {
        if (i % PRIO_STEP == 0) set_prio(PIPE_PRIO_OF(i / PRIO_STEP, 2 * DK / PRIO_STEP));
        if (i % GK == 0 && i + GK < 2 * DK) {
#pragma unroll
          for (int g = GK - 1; g >= 0; --g) kf[(i + GK + g) % (2 * GK)] = rdK(nxt, i + GK + g);
        }
        sn[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i % (2 * GK)], qf[i >> 1].v, sn[i & 1], 0, 0, 0);
        if (i == 2 * DK - 4) {
#pragma unroll
          for (int g = GV - 1; g >= 0; --g) vpre[g] = rdV(cur, g);
        }
        // the softmax of block j in 16 work items, SPS of them per MFMA: four partial maxima, the statistics (and
        // the rescale, when there is one), a gap, then 10 of the 16 pairs of exponentials
        bool with_stats = false;
#pragma unroll
        for (int w = i * SPS; w < (i + 1) * SPS; ++w) {
          if (w < 4) max_part(w);
          if (w == 4) {
            stats();
            with_stats = true;
          }
          if (w >= 6) exp_part(w - 6);
        }
        PIPE_FENCE();
        if (with_stats) {
          rescale();
          PIPE_FENCE();
        }
      }
    } else {
#pragma unroll
      for (int g = 0; g < GV; ++g) vpre[g] = rdV(cur, g);
#pragma unroll
      for (int i = 0; i < 4; ++i) max_part(i);
      stats();
      rescale();
#pragma unroll
      for (int e = 0; e < 10; ++e) exp_part(e);
      PIPE_FENCE();
    }
    // every wavefront is done with block j-1 (its stage is overwritten during phase 2) and block j+2, whose copies
    // were issued one block period ago, has landed
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    // ---------- phase 2: P.V(j) MFMAs, the rest of softmax(j), the copies of block j+3 ----------
#pragma unroll
    for (int i = 0; i < GV; ++i) vf[i] = vpre[i];
#pragma unroll
    for (int i = 0; i < 4 * DT; ++i) {
      const int k4 = i / DT, t = i % DT;
      if (i % PRIO_STEP == 0) set_prio(PIPE_PRIO_OF(i / PRIO_STEP, 4 * DT / PRIO_STEP));
      if (i % GV == 0 && i + GV < 4 * DT) {
#pragma unroll
        for (int g = GV - 1; g >= 0; --g) vf[(i + GV + g) % (2 * GV)] = rdV(cur, i + GV + g);
      }
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i % (2 * GV)], pfrag(k4), acc[t], 0, 0, 0);
      if (i % (SLOTS / (2 * PPT)) == 1) dma_run(j + 3, free_o, i / (SLOTS / (2 * PPT)));
      if (!LAST && i == 4 * DT - 4) {
#pragma unroll
        for (int g = GK - 1; g >= 0; --g) kpre[g] = rdK(lds + nn_o, g);
      }
#pragma unroll
      for (int w = i * SPS; w < (i + 1) * SPS; ++w) {
        if (w < 6) exp_part(10 + w);          // pairs 10..15 are needed from the second half of the phase on
        if (w == 6) {
          l_ij = xor32_sum(l_ij);
          l_i = l_i * alpha + l_ij;
          m_i = m_ij;
        }
      }
      PIPE_FENCE();
    }
  };

  const std::false_type F{};
  const std::true_type T{};
  int j = 0, cur_o = 0;
  auto nx = [&](int o) { return (o + STG) & (NST * STG - 1); };
  if (live) {
    for (; j + 4 <= L; j += 4) {       // stage offsets known at compile time, score registers alternating
      period(j, 0, STG, 2 * STG, 3 * STG, s0, s1, F, F);
      period(j + 1, STG, 2 * STG, 3 * STG, 0, s1, s0, F, F);
      period(j + 2, 2 * STG, 3 * STG, 0, STG, s0, s1, F, F);
      period(j + 3, 3 * STG, 0, STG, 2 * STG, s1, s0, F, F);
    }
    // what is left (at most three blocks and the last one) runs with the stage offsets in registers
    const int rest = L - j;
    if (rest & 1) {
      period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, F, F);
      s0[0] = s1[0];
      s0[1] = s1[1];
      cur_o = nx(cur_o);
      ++j;
    }
    if (rest & 2) {
      period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, F, F);
      cur_o = nx(cur_o);
      ++j;
      period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s1, s0, F, F);
      cur_o = nx(cur_o);
      ++j;
    }
    if (a.causal || (RAGGED && (a.n_ctx & (BN - 1)))) period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, T, T);
    else period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, T, F);
    cur_o = nx(cur_o);
    ++j;
  }
  // done (or, RAGGED, never started): keep up with the others' barriers and this wavefront's share of the copies;
  // cur_o is the stage of block j
  for (; j < nstream; ++j) {
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    dma_block_run(j + 3, nx(nx(nx(cur_o))));
    cur_o = nx(cur_o);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the trailing copies land before the stages are reused or released
  if constexpr (!RAGGED) {
    if (next_qblk >= 0) {   // the next item's Q, on its way while this item's results are stored
      const uint16_t *qrow = a.q + ((int64_t)next_head * a.n_ctx + next_qblk * BM + sub * 32 + c32) * a.ldq;
#pragma unroll
      for (int s = 0; s < DK; ++s) qf[s].u = *(const u16x8 *)(qrow + s * 16 + hi * 8);
    } else {
#pragma unroll
      for (int s = 0; s < DK; ++s) qf[s].u = (u16x8){0, 0, 0, 0, 0, 0, 0, 0};   // (no next item.  Written all the same: left
                                                                                 // alone, the old fragments count as live through
                                                                                 // the last periods on this path, and those spill)
    }
  }
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
      u32x2_t pk = {pack_bf16x2(acc[t][r4 * 4 + 0] * inv_l, acc[t][r4 * 4 + 1] * inv_l),
                    pack_bf16x2(acc[t][r4 * 4 + 2] * inv_l, acc[t][r4 * 4 + 3] * inv_l)};
      *(u32x2_t *)(orow + d) = pk;
    }
}

} // namespace pipeattn

// Persistent: gridDim.x workgroups (one per CU when there is that much work) walk the (head, pair of query blocks)
// items in the order the dispatcher would have dealt one-item workgroups: item n of workgroup g is g + n * gridDim.x,
// re-dealt so that an XCD's workgroups hold neighbouring items of the same heads.  A workgroup's items run back to
// back: each one's trailing copies fetch the first key blocks of the next.
template <int D, bool RAGGED>
__device__ __forceinline__ void attn_pipe(const AttnArgs &a, uint8_t *lds) {
  const int qblocks = RAGGED ? (a.rows + 255) / 256 : a.rows / 256;
  const int per_head = (qblocks + 1) / 2, total = per_head * a.heads;
  auto decode = [&](int n, int &head, int &p) {
    int id = n;
    if (total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
    head = id / per_head;
    p = id % per_head;
  };
  // the items of this workgroup in order: (n, which), which = 0: query block qblocks-1-p, 1: query block p
  auto advance = [&](int &n, int &head, int &p, int &which) -> bool {
    if (which == 0 && p != qblocks - 1 - p) {
      which = 1;
      return true;
    }
    n += (int)gridDim.x;
    if (n >= total) return false;
    decode(n, head, p);
    which = 0;
    return true;
  };
  int n = blockIdx.x, head, p, which = 0;
  if (n >= total) return;
  decode(n, head, p);
  int n2 = n, head2 = head, p2 = p, which2 = which;
  bool more = advance(n2, head2, p2, which2);
  pipeattn::Frag qf[D / 16];   // Q fragments of the running item; its last period refills them for the next
  pipeattn::body<D, false, RAGGED>(a, lds, head, which ? p : qblocks - 1 - p, more ? head2 : head,
                                   more ? (which2 ? p2 : qblocks - 1 - p2) : -1, qf);
  asm volatile("s_barrier" ::: "memory");   // nobody reads this item's stages any more; the next item's first blocks have landed
  while (more) {
    n = n2; head = head2; p = p2; which = which2;
    more = advance(n2, head2, p2, which2);
    pipeattn::body<D, true, RAGGED>(a, lds, head, which ? p : qblocks - 1 - p, more ? head2 : head,
                                    more ? (which2 ? p2 : qblocks - 1 - p2) : -1, qf);
    asm volatile("s_barrier" ::: "memory");
  }
}

extern "C" {

__global__ __launch_bounds__(512) void attn_tile_d128(AttnArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[pipeattn::NST * 2 * 64 * 128 * 2];
  attn_pipe<128, false>(a, lds);
}

// the same for sequence lengths that are whole 32-query tiles but not whole 256-query blocks
__global__ __launch_bounds__(512) void attn_ragged_d128(AttnArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[pipeattn::NST * 2 * 64 * 128 * 2];
  attn_pipe<128, true>(a, lds);
}

// head dim 64 on whole 256-query blocks: the same pipeline with 128-byte rows (8 + 8 MFMAs per block period)
__global__ __launch_bounds__(512) void attn_tile_d64(AttnArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[pipeattn::NST * 2 * 64 * 64 * 2];
  attn_pipe<64, false>(a, lds);
}

// and for lengths that are whole 32-query tiles but not whole 256-query blocks
__global__ __launch_bounds__(512) void attn_ragged_d64(AttnArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[pipeattn::NST * 2 * 64 * 64 * 2];
  attn_pipe<64, true>(a, lds);
}

} // extern "C"
