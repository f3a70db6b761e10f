// attn_tile_d256, attn_ragged_d256: _attn_fwd (examples/fused-attn/06-fused-attention.py:33-90, 143-215) at head dim
// 256 on whole 128-query blocks and on any length that is a whole number of 32-query tiles, as the software pipeline
// of attention_pipe.h re-cut for one wavefront per SIMD.
//
// At this head dim a wavefront's O^T is 128 registers and its Q 64, so a workgroup is four wavefronts of 32 queries,
// one per SIMD, each with the whole register file: O^T and Q live in AGPRs, scores and fragments in VGPRs, and every
// MFMA is written in assembly so that these classes are what the instruction gets (given the builtin at this
// occupancy, the compiler puts every MFMA result into AGPRs and each score then costs a copy).  K/V blocks are 32
// keys (a K or V tile of 32 rows x 512 bytes is 16 KiB), four stages of K + V = 128 KiB of LDS, K tiles below 64 KiB
// and V tiles above so that stage offsets fit the 16-bit offset field of an LDS read.
//
//   block period j of a wavefront (16 + 16 MFMAs of 32x32x16)
//     phase 1   MFMA: S^T(j+1) = K(j+1) . Q^T          VALU: row maxima of S^T(j), alpha, rescale, 12 of 16 exps
//     -------   s_waitcnt vmcnt(0) + s_barrier  (block j+2 has landed; block j-1's stage is free)
//     phase 2   MFMA: O^T += V(j)^T . P^T(j)           VALU: the last exps, row sums
//                                                      copies: block j+3 into the freed stage, one per two MFMAs
//
// Numerics, the lazy exponent reference and the evaluation of the causal mask at BLOCK_M = 32 are those of
// attention_pipe.h (its header states both differences from a literal evaluation of the source).  With 32-key blocks
// the masked block of a wavefront is exactly its own 32x32 tile on the diagonal.
//
// A block's scores are one 32x32 tile, i.e. sixteen MFMAs that accumulate into the same registers.  An MFMA whose
// addend is the result of the MFMA right before it needs idle states between the two that the hardware does not
// insert by itself (eight passes occupy the pipe for eight issue slots, the result can be read as an addend after
// ten or eleven), so the even and the odd k-steps accumulate in two register sets of their own, every MFMA depends
// on the one before the last, and the softmax adds the two sets before it reads them (sixteen additions per block).
//
// What the compiler cannot know about MFMAs written in assembly is that their results arrive late: a score
// register is read by the softmax a whole phase after the MFMA that wrote it, and the places where that distance
// is not there by construction (after the prologue's S^T(0), in front of the period that has no phase 1, in front of
// the epilogue) carry explicit idle states.
#pragma once
#include <type_traits>

namespace pipe256 {

using pipeattn::Frag;
using fastattn::lds_s16x4;
using fastattn::lds_void;

constexpr int D = 256, BM = 128, BN = 32, NST = 4;
constexpr int DK = D / 16, DT = D / 32, ROW = D * 2, CH = D / 8;
constexpr int TILE = BN * ROW, STG = TILE, VBASE = NST * TILE;   // stage s: K at s*TILE, V at VBASE + s*TILE
constexpr int GK = 2, GV = 2;                                    // fragments per read group
constexpr float LAZY_T = 8.0f;
#define P256_FENCE() __builtin_amdgcn_sched_barrier(0)
// 24 idle states, after which an 8-pass MFMA has written back; the registers it wrote are named, so that no read of
// them is scheduled in front
#define P256_IDLE_V(x) asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" : "+v"(x))
// (the accumulators are not named as operands: that made the compiler keep a second copy of half of them; a
// scheduling fence on either side keeps their reads behind the idle states instead)
#define P256_IDLE_ACC(o)                                    \
  do {                                                      \
    P256_FENCE();                                           \
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory"); \
    P256_FENCE();                                           \
  } while (0)

// Two idle states in front of every MFMA.  The compiler treats these statements as opaque: when it has moved an
// operand between the register files (a Q fragment it keeps in VGPRs copied into an AGPR, a K fragment it parked in
// AGPRs read back), the v_accvgpr_write / v_accvgpr_read sits right in front of the statement, and an MFMA that
// issues directly behind such a copy reads the register before the copy has landed (measured: scores off by a few
// per cent, exact with one idle state in between; which operands the allocator moves changes from build to build).
// Costs 2 % of the kernel's time.
#define P256_PAD "s_nop 1\n\t"
// S^T (+)= K . Q^T: scores in VGPRs, Q in AGPRs.  ZERO: the first k-step of a block takes 0 as its addend.
template <bool ZERO> __device__ __forceinline__ void mfma_s(f32x16 &s, bf16x8 k, bf16x8 q) {
  // (the first k-step of each of the two chains; its Q fragment is a VGPR operand, see QV below)
  if constexpr (ZERO)
    asm volatile(P256_PAD "v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "+v"(s) : "v"(k), "v"(q));
  else
    asm volatile(P256_PAD "v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(k), "a"(q));
}
// Idle states behind an MFMA, inside its statement, for the places where the compiler may put code of its own that
// reads the result right behind the statement: it does not know that the statement holds an MFMA and leaves none of
// the wait states that a read of an MFMA's result needs (eleven for this MFMA).  Two kinds of such places exist.  In
// the periods outside the main loop (the up to three left over and the last one of an item) the register allocator
// may move each 16-register accumulator tile to VGPRs directly behind the MFMA that writes it last, as it did in the
// ragged kernel.  And where control flow joins behind a period, it copies accumulator registers between the
// register sets the paths use.  Without the idle states such copies hold what the tile held before the MFMA: wrong
// output values in some d-tiles of some rows, with the right M.
#define P256_TAIL "\n\ts_nop 7\n\ts_nop 7"
// O^T += V^T . P^T: accumulators in AGPRs
template <bool TAIL> __device__ __forceinline__ void mfma_o(f32x16 &o, bf16x8 v, bf16x8 p) {
  if constexpr (TAIL)
    asm volatile(P256_PAD "v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" P256_TAIL : "+a"(o) : "v"(v), "v"(p));
  else
    asm volatile(P256_PAD "v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(o) : "v"(v), "v"(p));
}

// the same with one direct-to-LDS copy behind it (m0, its LDS destination, is written by the compiler in front of
// the statement: the MFMA is the wait state that the copy needs after a write to m0)
template <bool TAIL>
__device__ __forceinline__ void mfma_o_copy(f32x16 &o, bf16x8 v, bf16x8 p, uint32_t m0v, uint32_t voff, const uint8_t *src) {
  if constexpr (TAIL)
    asm volatile(P256_PAD "v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5" P256_TAIL
                 : "+a"(o)
                 : "v"(v), "v"(p), "{m0}"(m0v), "v"(voff), "s"(src)
                 : "memory");
  else
    asm volatile(P256_PAD "v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5"
                 : "+a"(o)
                 : "v"(v), "v"(p), "{m0}"(m0v), "v"(voff), "s"(src)
                 : "memory");
}

// PREFETCHED, next_head, next_qblk: as in pipeattn::body (blocks 0, 1, 2 of this item are already in stages 0, 1, 2;
// this item's trailing copies fetch the first key blocks of the next item; its Q is loaded before this item's
// results are stored).
//
// RAGGED: N_CTX is a whole number of 32-query tiles but not of 128-query blocks.  Key blocks are 32 keys, so every
// block of the sequence is whole and no key needs masking for the length's sake.  A wavefront whose tile lies past
// the end computes and stores nothing but keeps up with the barriers and its share of the copies; an item's stream
// of blocks is padded to a multiple of four periods (the padding refetches the item's last block into a stage that
// nobody reads), so that the next item's first blocks land in stages 0, 1, 2 as they do for whole blocks; and an
// item with fewer than three blocks has the others of its first three fetched from its last one.  Q is loaded when
// the item starts.
template <bool PREFETCHED, bool RAGGED = false>
__device__ __forceinline__ void body(const AttnArgs &a, uint8_t *lds, const int head, const int qblk, const int next_head,
                                     const int next_qblk, Frag (&qf)[DK]) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, hi = lane >> 5;

  const int q0 = qblk * BM;
  const int qw = q0 + wave * 32;
  const int my_q = qw + c32;
  const int64_t base = (int64_t)head * a.n_ctx;
  const float qk_scale = a.sm_scale * 1.44269504f;
  const bool live = !RAGGED || qw < a.n_ctx;                     // wave-uniform
  const int nreal = (a.causal ? (RAGGED ? min(q0 + BM, a.n_ctx) : q0 + BM) : a.n_ctx) / BN;   // key blocks of this item
  const int nblk = RAGGED ? (nreal + 3) & ~3 : nreal;            // periods the workgroup goes through (a multiple of 4)
  const int L = a.causal ? qw / BN : nreal - 1;                  // this wavefront's last block (the masked one when causal)
  // RAGGED: the real blocks of the item that follows (this item's own when none does)
  const int next_q0 = (next_qblk >= 0 ? next_qblk : qblk) * BM;
  const int next_nreal = RAGGED ? (a.causal ? min(next_q0 + BM, a.n_ctx) : a.n_ctx) / BN : 3;

  // ---- copies: 256 threads x 16 B = 4 KiB = 8 rows per instruction round, four rounds per K or V tile ----
  const int crow = tid / CH, cpos = tid % CH;
  // K: logical chunk c of row r sits at c ^ (r & 31); V: at c ^ ((r & 3) << 2)
  // (the offset of a round inside its tile is part of the thread's offset, so that a tile's four copies share one base)
  uint32_t k_voff[4], v_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    k_voff[i] = (uint32_t)(((int64_t)(i * 8 + crow) * a.ldk + (cpos ^ ((i * 8 + crow) & 31)) * 8) * 2);
    v_voff[i] = (uint32_t)(((int64_t)(i * 8 + crow) * a.ldv + (cpos ^ ((crow & 3) << 2)) * 8) * 2);
  }
  const uint8_t *kg = (const uint8_t *)(a.k + base * a.ldk);
  const uint8_t *vg = (const uint8_t *)(a.v + base * a.ldv);
  const uint8_t *kg_next = (const uint8_t *)(a.k + (int64_t)next_head * a.n_ctx * a.ldk);
  const uint8_t *vg_next = (const uint8_t *)(a.v + (int64_t)next_head * a.n_ctx * a.ldv);
  const int lds_wave = wave * 1024;
  auto dma_one = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst) __attribute__((always_inline)) {
    const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(dst + lds_wave);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(voff), "s"(src_uniform)
                 : "memory", "m0");
  };
  const int64_t kstep = (int64_t)BN * a.ldk * 2, vstep = (int64_t)BN * a.ldv * 2;
  // where period blk of this item's stream fetches from: its own block blk (RAGGED: the last real one for the padding
  // periods and for an item of fewer than three blocks), past the stream the next item's first blocks (RAGGED: as
  // many as that item has)
  auto block_src = [&](int blk, const uint8_t *&kb, const uint8_t *&vb) __attribute__((always_inline)) {
    const bool own = blk < nblk;
    const int64_t b = own ? (RAGGED ? min(blk, nreal - 1) : blk) : (RAGGED ? min(blk - nblk, next_nreal - 1) : blk - nblk);
    kb = (own ? kg : kg_next) + b * kstep;
    vb = (own ? vg : vg_next) + b * vstep;
  };
  // piece r (0-3: the four 8-row rounds of K; 4-7: of V) of block blk into the stage at byte offset stage_o
  auto dma_piece = [&](int blk, int stage_o, int r) __attribute__((always_inline)) {
    const uint8_t *kb, *vb;
    block_src(blk, kb, vb);
    if (r < 4) dma_one(kb, k_voff[r], lds + stage_o + r * 4096);
    else dma_one(vb, v_voff[r - 4], lds + VBASE + stage_o + (r - 4) * 4096);
  };
  // the same from two running pointers (K and V rows of the block that is fetched next), stepped after the last piece
  // of a block and switched to the next item's keys when this item's run out
  const uint8_t *kp, *vp;   // block 3 at first: blocks 0..2 are the prologue's (or the item before's)
  block_src(3, kp, vp);
  auto dma_step = [&](int blk) __attribute__((always_inline)) {
    if constexpr (RAGGED) {
      block_src(blk + 1, kp, vp);
    } else {
      const bool wrap = blk + 1 == nblk;
      kp = wrap ? kg_next : kp + kstep;
      vp = wrap ? vg_next : vp + vstep;
    }
  };
  auto dma_run = [&](int blk, int stage_o, int r) __attribute__((always_inline)) {
    if (r < 4) dma_one(kp, k_voff[r], lds + stage_o + r * 4096);
    else dma_one(vp, v_voff[r - 4], lds + VBASE + stage_o + (r - 4) * 4096);
    if (r == 7) dma_step(blk);
  };

  // ---- fragment addresses ----
  int k_off[DK];                 // K (A operand of S^T): lane = key row c32, chunk 2s+hi of its row
#pragma unroll
  for (int s = 0; s < DK; ++s) k_off[s] = c32 * ROW + (((2 * s + hi) ^ c32) << 4);
  const int G4 = lane >> 4, i16 = lane & 15, qd = i16 >> 2;
  const int v_cc = (G4 & 1) * 2 + ((i16 >> 1) & 1);
  int v_off[DT];                 // V^T (A operand of O^T) through transposing reads: key row hi*4+qd (+ k4*16 + h2*8)
#pragma unroll
  for (int t = 0; t < DT; ++t)
    v_off[t] = VBASE + (hi * 4 + qd) * ROW + (((t * 4 + v_cc) ^ (qd << 2)) << 4) + ((i16 & 1) << 3);

  f32x16 acc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) {
    acc[t] = (f32x16){0};
    asm volatile("" : "+a"(acc[t]));
  }
  float m_i = -__builtin_inff(), l_i = 1.0f;

  auto rdK = [&](const uint8_t *stage, int i) __attribute__((always_inline)) -> bf16x8 {   // k-step i
    return *(const bf16x8 *)(stage + k_off[i]);
  };
  auto rdV = [&](const uint8_t *stage, int i) __attribute__((always_inline)) -> bf16x8 {   // 16-key step i / DT, d-tile i % DT
    Frag f;
    const int k4 = i / DT, t = i % DT;
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
      f.h[h2] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(stage + v_off[t] + (k4 * 16 + h2 * 8) * ROW));
    return f.v;
  };

  // ---- prologue: blocks 0, 1, 2 in flight; S^T(0); the first K fragments of block 1 ----
  if constexpr (!PREFETCHED) {
#pragma unroll
    for (int b = 0; b < 3; ++b)
#pragma unroll
      for (int r = 0; r < 8; ++r) dma_piece(b, b * STG, r);
  }
  if constexpr (!PREFETCHED || RAGGED) {   // (otherwise the item before this one loaded them)
    // (RAGGED: a wavefront past the end loads the last row that exists and never uses it)
    const uint16_t *qrow = a.q + (base + (RAGGED ? min(my_q, a.n_ctx - 1) : my_q)) * a.ldq;
#pragma unroll
    for (int s = 0; s < DK; ++s) qf[s].u = *(const u16x8 *)(qrow + s * 16 + hi * 8);
  }
  // the loads land here: the compiler's own vmcnt bookkeeping does not see the copies issued from assembly
  // QV: of the sixteen Q fragments the first two stay in VGPRs and the other fourteen in AGPRs, which is what the
  // register allocator arrives at by itself; named so in the constraints, it has no reason to copy them around
#pragma unroll
  for (int s = 0; s < DK; ++s) {
    if (s < 2) asm volatile("" : "+v"(qf[s].v));
    else asm volatile("" : "+a"(qf[s].v));
  }
  if constexpr (!PREFETCHED) asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");   // every wavefront's copies have landed
  // Scores: the even k-steps of a block accumulate in s0 or s1 (alternating from block to block: the softmax of a
  // block reads its set while the next block's MFMAs write the other), the odd k-steps of every block in sb.
  f32x16 s0, s1, sb;
  asm volatile("" : "=v"(s0));
  asm volatile("" : "=v"(s1));
  asm volatile("" : "=v"(sb));
  bf16x8 kpre[GK], vpre[GV];   // first fragment group of the coming phase, requested during the phase before
  if (live) {
#pragma unroll
    for (int i = 0; i < DK; ++i) {
      f32x16 &dst = (i & 1) ? sb : s0;
      if (i < 2) mfma_s<true>(dst, rdK(lds, i), qf[i].v);
      else mfma_s<false>(dst, rdK(lds, i), qf[i].v);
    }
#pragma unroll
    for (int i = 0; i < GK; ++i) kpre[i] = rdK(lds + STG, i);
    P256_IDLE_V(sb);             // S^T(0) is read at once
  }

  // One block period of this wavefront.  LAST: no next block to start on; MASKED: the block on the diagonal.
  // cur_o, nxt_o, nn_o: byte offsets of the stages of blocks j, j+1, j+2; free_o: of the stage block j+3 goes into.
  // sc holds S^T(j) on entry, sn receives S^T(j+1).
  // tail_: 0 in the main loop; 1: the period may be followed by something else than the next period (its last MFMA
  // leaves idle states); 2: a period outside the main loop (every P.V MFMA leaves them): see P256_TAIL
  auto period = [&](int j, int cur_o, int nxt_o, int nn_o, int free_o, f32x16 &sc, f32x16 &sn, auto last_,
                    auto masked_, auto tail_) __attribute__((always_inline)) {
    constexpr bool LAST = decltype(last_)::value, MASKED = decltype(masked_)::value;
    constexpr int TAIL = decltype(tail_)::value;
    static_assert(!LAST || TAIL == 2, "");
    const uint8_t *cur = lds + cur_o, *nxt = lds + nxt_o;
    bf16x8 kf[2 * GK], vf[2 * GV];
    float rmax0 = -__builtin_inff(), rmax1 = -__builtin_inff(), m_ij, alpha, l_ij = 0.0f;
    Frag pf[2];        // P^T of the two 16-key steps as packed bf16 pairs
    auto max_part = [&](int part) __attribute__((always_inline)) {   // part 0, 1: 8 elements each
      float &rm = part ? rmax1 : rmax0;
#pragma unroll
      for (int r = 0; r < 8; r += 2) rm = fmaxf(fmaxf(rm, sc[part * 8 + r]), sc[part * 8 + r + 1]);
    };
    auto stats = [&]() __attribute__((always_inline)) {
      const float rmax = xor32_max(fmaxf(rmax0, rmax1));
      m_ij = MASKED ? fmaxf(m_i, rmax) : fmaxf(m_i, rmax * qk_scale);
      // the reference moves only when some row of the wavefront outgrew it by more than LAZY_T (then every row
      // takes its true running maximum); otherwise it stays, alpha is 1 and nothing is rescaled
      if (__builtin_amdgcn_ballot_w64(m_ij > m_i + LAZY_T) == 0) m_ij = m_i;
      alpha = __builtin_amdgcn_exp2f(m_i - m_ij);
    };
    auto rescale = [&]() __attribute__((always_inline)) {
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
        // one 32-row tile at a time, so that no more than sixteen accumulator registers are out of the AGPRs at once
#pragma unroll
        for (int t = 0; t < DT; ++t) {
          f32x16 x = acc[t];
#pragma unroll
          for (int r = 0; r < 16; ++r) x[r] *= alpha;
          acc[t] = x;
          asm volatile("" : "+a"(acc[t]));
          P256_FENCE();
        }
      }
    };
    auto exp_part = [&](int e) __attribute__((always_inline)) {     // e = 0..7: two elements -> one packed pair of 16-key step e >> 2
      const int k4 = e >> 2, jj = e & 3, r = k4 * 8 + 2 * jj;
      float p0, p1;
      if (MASKED) {
        p0 = __builtin_amdgcn_exp2f(sc[r] - m_ij);
        p1 = __builtin_amdgcn_exp2f(sc[r + 1] - m_ij);
      } else {
        p0 = __builtin_amdgcn_exp2f(sc[r] * qk_scale - m_ij);
        p1 = __builtin_amdgcn_exp2f(sc[r + 1] * qk_scale - m_ij);
      }
      l_ij += p0;          // fp32 sum before the cast (06-fused-attention.py:67)
      l_ij += p1;
      pf[k4].w[jj] = pack_bf16x2(p0, p1);
    };
    if constexpr (LAST) P256_IDLE_ACC(acc);   // (no phase 1 between the P.V MFMAs before and a rescale below)
    // the two halves of S^T(j); sb is written again by the second MFMA of phase 1
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] += sb[r];
    if constexpr (MASKED) {
      // the block on the diagonal: qk * qk_scale + where(mask, 0, -1.0e6) inside this wavefront's 32x32 tile
      // (06-fused-attention.py:58-59 at BLOCK_M = 32), which with 32-key blocks is the whole block
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        // (without the mask this is the last block of the row: the same form with nothing added, so that one form of
        // the last period serves both)
        const int key = j * BN + (r >> 2) * 8 + hi * 4 + (r & 3);
        sc[r] = sc[r] * qk_scale + ((!a.causal || my_q >= key) ? 0.0f : -1.0e6f);
      }
    }
    if constexpr (!LAST) {
      // ---------- phase 1: S^T(j+1) MFMAs, softmax(j) VALU ----------
      asm volatile("" : "=v"(sn));
#pragma unroll
      for (int i = 0; i < GK; ++i) kf[i] = kpre[i];
#pragma unroll
      for (int i = 0; i < DK; ++i) {
        if (i % GK == 0 && i + GK < DK) {
#pragma unroll
          for (int g = GK - 1; g >= 0; --g) kf[(i + GK + g) % (2 * GK)] = rdK(nxt, i + GK + g);
        }
        if (i == 0) {
          P256_FENCE();       // (the additions above have read sb before its chain starts again)
          mfma_s<true>(sn, kf[0], qf[0].v);
        } else if (i == 1) {
          mfma_s<true>(sb, kf[1], qf[1].v);
        } else {
          mfma_s<false>((i & 1) ? sb : sn, kf[i % (2 * GK)], qf[i].v);
        }
        if (i == DK - 4) {
#pragma unroll
          for (int g = GV - 1; g >= 0; --g) vpre[g] = rdV(cur, g);
        }
        // the softmax of block j: the two partial maxima, the statistics (and the rescale, when there is one), a
        // gap, then 6 of the 8 pairs of exponentials, one per two MFMAs
        if (i < 2) max_part(i);
        if (i == 2) stats();
        if (i >= 4 && i % 2 == 0) exp_part((i - 4) / 2);
        P256_FENCE();
        if (i == 2) {
          rescale();
          P256_FENCE();
        }
      }
    } else {
#pragma unroll
      for (int g = 0; g < GV; ++g) vpre[g] = rdV(cur, g);
      max_part(0);
      max_part(1);
      stats();
      rescale();
#pragma unroll
      for (int e = 0; e < 6; ++e) exp_part(e);
      P256_FENCE();
    }
    // every wavefront is done with block j-1 (its stage is overwritten during phase 2) and block j+2, whose copies
    // were issued one block period ago, has landed
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    // ---------- phase 2: P.V(j) MFMAs, the rest of softmax(j), the copies of block j+3 ----------
#pragma unroll
    for (int i = 0; i < GV; ++i) vf[i] = vpre[i];
#pragma unroll
    for (int i = 0; i < 2 * DT; ++i) {
      const int k4 = i / DT, t = i % DT;
      if (i % GV == 0 && i + GV < 2 * DT) {
#pragma unroll
        for (int g = GV - 1; g >= 0; --g) vf[(i + GV + g) % (2 * GV)] = rdV(cur, i + GV + g);
      }
      if (i % 2 == 1) {
        const int r = i / 2;
        const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(lds + (r < 4 ? 0 : VBASE) + free_o + (r & 3) * 4096 + lds_wave);
        if (TAIL == 2 || (TAIL == 1 && i == 2 * DT - 1))
          mfma_o_copy<true>(acc[t], vf[i % (2 * GV)], pf[k4].v, m0v, r < 4 ? k_voff[r] : v_voff[r - 4], r < 4 ? kp : vp);
        else
          mfma_o_copy<false>(acc[t], vf[i % (2 * GV)], pf[k4].v, m0v, r < 4 ? k_voff[r] : v_voff[r - 4], r < 4 ? kp : vp);
        if (r == 7) dma_step(j + 3);
      } else {
        mfma_o<TAIL == 2>(acc[t], vf[i % (2 * GV)], pf[k4].v);
      }
      if (!LAST && i == 2 * DT - 4) {
#pragma unroll
        for (int g = GK - 1; g >= 0; --g) kpre[g] = rdK(lds + nn_o, g);
      }
      if (i < 2) exp_part(6 + i);             // pairs 4..7 are needed from the second half of the phase on
      if (i == 2) {
        l_ij = xor32_sum(l_ij);
        l_i = l_i * alpha + l_ij;
        m_i = m_ij;
      }
      P256_FENCE();
    }
  };

  const std::false_type F{};
  const std::true_type T{};
  const std::integral_constant<int, 0> T0{};
  const std::integral_constant<int, 1> T1{};
  const std::integral_constant<int, 2> T2{};
  int j = 0, cur_o = 0;
  auto nx = [&](int o) { return (o + STG) & (NST * STG - 1); };
  __builtin_amdgcn_s_setprio(3);
  if (live) {
    for (; j + 4 <= L; j += 4) {       // stage offsets known at compile time, score registers alternating
      period(j, 0, STG, 2 * STG, 3 * STG, s0, s1, F, F, T0);
      period(j + 1, STG, 2 * STG, 3 * STG, 0, s1, s0, F, F, T0);
      period(j + 2, 2 * STG, 3 * STG, 0, STG, s0, s1, F, F, T0);
      period(j + 3, 3 * STG, 0, STG, 2 * STG, s1, s0, F, F, T1);
    }
    // what is left (at most three blocks and the last one) runs with the stage offsets in registers
    const int rest = L - j;
    if (rest & 1) {
      period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, F, F, T2);
      s0 = s1;
      cur_o = nx(cur_o);
      ++j;
    }
    if (rest & 2) {
      period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, F, F, T2);
      cur_o = nx(cur_o);
      ++j;
      period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s1, s0, F, F, T2);
      cur_o = nx(cur_o);
      ++j;
    }
    period(j, cur_o, nx(cur_o), nx(nx(cur_o)), nx(nx(nx(cur_o))), s0, s1, T, T, T2);
    cur_o = nx(cur_o);
    ++j;
  }
  // done (or, RAGGED, never started): keep up with the others' barriers and this wavefront's share of the copies;
  // cur_o is the stage of block j
  for (; j < nblk; ++j) {
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int r = 0; r < 8; ++r) dma_run(j + 3, nx(nx(nx(cur_o))), r);
    cur_o = nx(cur_o);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the trailing copies land before the stages are reused or released
  P256_IDLE_ACC(acc);                                // the last P.V MFMAs have written back before the accumulators are read
  if constexpr (!RAGGED) {
    if (next_qblk >= 0) {   // the next item's Q, on its way while this item's results are stored
      const uint16_t *qrow = a.q + ((int64_t)next_head * a.n_ctx + next_qblk * BM + wave * 32 + c32) * a.ldq;
#pragma unroll
      for (int s = 0; s < DK; ++s) qf[s].u = *(const u16x8 *)(qrow + s * 16 + hi * 8);
    }
  }
  if (!live) return;
  // ---- epilogue ----
  if (hi == 0) a.m[base + my_q] = m_i + __builtin_log2f(l_i);
  uint16_t *orow = a.o + (base + my_q) * a.ldo;
  const float inv_l = 1.0f / l_i;
#pragma unroll
  for (int t = 0; t < DT; ++t) {
    // (one tile at a time: with all 128 accumulator registers copied out at once, the next item's Q fragments,
    // loaded above, do not stay in AGPRs)
    P256_FENCE();
    const f32x16 x = acc[t];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int d = t * 32 + r4 * 8 + hi * 4;
      typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
      u32x2_t pk = {pack_bf16x2(x[r4 * 4 + 0] * inv_l, x[r4 * 4 + 1] * inv_l),
                    pack_bf16x2(x[r4 * 4 + 2] * inv_l, x[r4 * 4 + 3] * inv_l)};
      *(u32x2_t *)(orow + d) = pk;
    }
  }
}

} // namespace pipe256

// Persistent, as attn_pipe: gridDim.x workgroups walk the (head, pair of query blocks) items in the order the
// dispatcher would have dealt one-item workgroups, a workgroup's items back to back.
template <bool RAGGED> __device__ __forceinline__ void attn_pipe256(const AttnArgs &a, uint8_t *lds) {
  const int qblocks = RAGGED ? (a.rows + pipe256::BM - 1) / pipe256::BM : a.rows / pipe256::BM;
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
  pipeattn::Frag qf[pipe256::DK];   // Q fragments of the running item; its end refills them for the next
  pipe256::body<false, RAGGED>(a, lds, head, which ? p : qblocks - 1 - p, more ? head2 : head,
                       more ? (which2 ? p2 : qblocks - 1 - p2) : -1, qf);
  asm volatile("s_barrier" ::: "memory");   // nobody reads this item's stages any more; the next item's first blocks have landed
  while (more) {
    n = n2; head = head2; p = p2; which = which2;
    more = advance(n2, head2, p2, which2);
    pipe256::body<true, RAGGED>(a, lds, head, which ? p : qblocks - 1 - p, more ? head2 : head,
                        more ? (which2 ? p2 : qblocks - 1 - p2) : -1, qf);
    asm volatile("s_barrier" ::: "memory");
  }
}

extern "C" {

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_tile_d256(AttnArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[pipe256::NST * 2 * pipe256::TILE];
  attn_pipe256<false>(a, lds);
}

// the same for sequence lengths that are whole 32-query tiles but not whole 128-query blocks
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_ragged_d256(AttnArgs a) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[pipe256::NST * 2 * pipe256::TILE];
  attn_pipe256<true>(a, lds);
}

} // extern "C"
