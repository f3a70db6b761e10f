// gemm_tile_fp8_*: fast path of the fp8 (OCP e4m3) tile matmul with per-tensor scales,
// C = half(acc * scale_a * scale_b).
//
// Same organisation as the bf16 fast path (gemm_tile.h): 256x256 macro tile per workgroup
// of 4 wavefronts, 128x128 per wavefront, a ring of four 32 KiB LDS stages filled by
// direct-to-LDS copies three steps ahead, persistent XCD-aware grid, transposed product so
// that the epilogue stores 4 consecutive n per lane.  What differs:
//   * one step is K = 64 (64 one-byte elements per A row = the same 64 bytes as 32 bf16),
//     consumed by ONE v_mfma_f32_32x32x64_f8f6f4 per accumulator (no block scales, i.e. 1.0;
//     the per-tensor scales are applied in the epilogue);
//   * a lane's operand is 32 bytes: k = 32*(lane/32) .. +31.  A rows are k-contiguous: two
//     ds_read_b128.  B is [K,N] with n contiguous: ds_read_b64_tr_b8 transposes an 8x16
//     block of bytes across 16 lanes (result lane i, byte j = source lane 2j + i/8, byte
//     i%8), four of them per fragment;
//   * LDS layout: A rows of 64 B, logical chunk c at c ^ ((m>>2)&3); B rows of 256 B,
//     logical chunk c at c ^ ((k&7)<<1) (8 k-rows x 2 chunks land on 16 distinct bank
//     groups).
// Requirements: M, N multiples of 256, K a multiple of 256, 16-byte aligned rows, full grid.
#pragma once
#include <type_traits>

#include "gemm_tile.h"

namespace fast8 {

constexpr int BM = 256, BN = 256, BK = 64, R = 4;
constexpr int A_BYTES = BM * BK;       // 16 KiB
constexpr int B_BYTES = BK * BN;       // 16 KiB
constexpr int STAGE = A_BYTES + B_BYTES;

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef __attribute__((address_space(3))) void lds_void;

// RAGGED (M any, N a multiple of 16, K a multiple of 64): as in the 16-bit kernel, fetches past the edges are
// clamped into the matrix, K is padded to whole turns of the ring with steps copied from a page of zeros, and
// the stores are clipped.
// MB = 2: the half-tile pass over the tail of the persistent loop, as in the 16-bit kernel: a workgroup computes a
// 128x256 half of a macro tile, each wavefront 64x128 (2x4 accumulators), two A slabs and six copies per step.
// STREAM: the stores of a 16-bit C go past the caches: the host's choice for an output that the 256 MiB memory-side
// cache does not hold (a plain store leaves its line there and in the L2, and a C beyond that size only evicts
// operands on its way through: 16384 x 16384 x 1024 runs 28 % faster with streaming stores and x 4096 8.6 %, x 8192
// the same; 8192^3, whose C fits, slower).  The variants are kernels of their own: the two forms of the epilogue
// inside one kernel cost the benchmark shapes 1-2 %.
// SPLITK (the clamping half-tile pass alone): K in g.ksplit equal slices, work item = (slice, tile, live half), the
// slice's fp32 sums into slab `slice` of the workspace at g.c; gemm_splitk_reduce_* adds the slabs, scales and rounds
// (see the 16-bit kernel).
template <int OUT_DT, bool RAGGED = false, int MB = 4, bool STREAM = false, bool SPLITK = false>
__device__ __forceinline__ void body(const GemmArgs &g, const fast::Ring &ring) {
  static_assert(!SPLITK || (RAGGED && MB == 2 && !STREAM), "slices of K: the clamping half-tile pass");
  const int gK = SPLITK ? g.K / g.ksplit : g.K;      // the K of one work item
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = RAGGED ? (g.M + BM - 1) / BM : g.M / BM, tiles_n = RAGGED ? (g.N + BN - 1) / BN : g.N / BN;
  const int tiles_mv = SPLITK ? tiles_m * g.ksplit : tiles_m;   // SPLITK: row tm + tiles_m * s of the item grid is slice s of tile row tm
  const fast::PassItems items =
      fast::pass_items<MB, true, false, SPLITK>(tiles_mv * tiles_n, (SPLITK && tiles_m == 1) ? g.M : fast::BM);
  const int total = items.total;
  const int nk_real = gK / BK;                                   // steps that carry data
  const int nk = RAGGED ? (nk_real + R - 1) / R * R : nk_real;    // steps per tile, a multiple of R

  // ---- global -> LDS: thread t writes byte 16*t of each 4 KiB slab ----
  // A slab i (64 rows of 64 B): row = i*64 + (t>>2), position t&3 holds chunk (t&3)^((row>>2)&3)
  const int a_row = tid >> 2;
  const int a_chunk = (tid & 3) ^ ((a_row >> 2) & 3);
  // B slab i (16 k-rows of 256 B): k = i*16 + (t>>4), position t&15 holds chunk (t&15)^((k&7)<<1)
  const int b_k = tid >> 4;
  const int b_chunk = (tid & 15) ^ ((b_k & 7) << 1);
  const uint32_t a_voff = (uint32_t)((int64_t)a_row * g.lda + a_chunk * 16);
  const uint32_t b_voff = (uint32_t)((int64_t)b_k * g.ldb + b_chunk * 16);
  const int64_t a_slab = 64 * g.lda, b_slab = 16 * g.ldb;
  // (SPLITK: slice s takes steps s, s + ksplit, ..., as in the 16-bit kernel)
  const int64_t a_kstep = SPLITK ? (int64_t)BK * g.ksplit : BK;
  const int64_t b_kstep = (int64_t)BK * g.ldb * (SPLITK ? g.ksplit : 1);
  const int lds_wave = wave * 1024;

  // ---- LDS -> fragments ----
  const int l32 = lane & 31, hi = lane >> 5;
  const int a_base = (wm * (32 * MB) + l32) * 64;
  const int a_x = (l32 >> 2) & 3;
  int a_pos[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) a_pos[h] = a_base + (((2 * hi + h) ^ a_x) << 4);
  // APAIR (the macro-tile pass), as in the 16-bit kernel: A is copied in 128-byte row segments, two K
  // steps at a time, so that every request to the L2 is a whole cache line.  The A regions of stages 2P and 2P+1
  // hold rows 0-127 and 128-255 of the macro tile for steps 4n + 2P and 4n + 2P + 1, 128 bytes per row, step s in
  // logical chunks 4s .. 4s+3, chunk c at c ^ ((row >> 1) & 7): the sixteen lanes of a pass of a 16-byte read
  // (rows {0-3, 12-15, 20-23, 24-27} or {4-7, 8-11, 16-19, 28-31} of a fragment, two rows to a line of banks) then
  // meet sixteen different positions.
  constexpr bool APAIR = MB == 4;
  int a_pp[2][2];      // [step of the pair][half of the lane's 32 bytes]: region base (stage 2P) + a_pp + i * 4096
#pragma unroll
  for (int st = 0; st < 2; ++st)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      a_pp[st][h] = wm * STAGE + l32 * 128 + (((4 * st + 2 * hi + h) ^ ((l32 >> 1) & 7)) << 4);
  // copies of a pair: slab i (0..7) = rows 32i .. 32i+31; thread t: row t>>3, position t&7
  const uint32_t a_voff_pair = (uint32_t)((int64_t)(tid >> 3) * g.lda + (((tid & 7) ^ ((tid >> 4) & 7)) << 4));
  const int64_t a_slab32 = 32 * g.lda;
  const int pair_r8 = tid >> 3, pair_c = (tid & 7) ^ ((tid >> 4) & 7);   // row in the slab, logical chunk
  const int G4 = lane >> 4, i16 = lane & 15, rj = i16 >> 1;
  int b_pos[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    b_pos[j] = A_BYTES + (hi * 32 + rj) * 256 + ((((wn * 8 + j * 2) ^ (rj << 1)) | (G4 & 1)) << 4) + ((i16 & 1) << 3);

  const uint8_t *A = (const uint8_t *)g.a;
  const uint8_t *B = (const uint8_t *)g.b;

  struct Frags {
    union { i32x4 q[2]; i32x8 v; } a[MB];
    union { i32x2 d[4]; i32x8 v; } b[4];
  };
  Frags f0, f1;
  f32x16 acc[MB][4];

  // the 24 LDS reads of one step in the order the MFMAs want them (MB == 2: the first 20):
  // b0 (4 reads) a0 (2) b1 (4) b2 (4) b3 (4) a1 (2) a2 (2) a3 (2)
  // (J: ring index of the stage, a constant wherever this is called)
  auto rd = [&](Frags &f, const uint8_t *stage, int J, int r) {
    auto rb = [&](int j, int q) {
      f.b[j].d[q] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2 *)(stage + b_pos[j] + q * 2048));
    };
    auto ra = [&](int i, int h) {
      if constexpr (APAIR) f.a[i].q[h] = *(const i32x4 *)(ring.s[J & 2] + a_pp[J & 1][h] + i * 4096);
      else f.a[i].q[h] = *(const i32x4 *)(stage + a_pos[h] + i * 2048);
    };
    if (r < 4) rb(0, r);
    else if (r < 6) ra(0, r - 4);
    else if (r < 18) rb(1 + (r - 6) / 4, (r - 6) % 4);
    else ra(1 + (r - 18) / 2, (r - 18) % 2);
  };
  auto mm = [&](Frags &f, int n) {
    const int i = n >> 2, j = n & 3;
    // both scale operands the constant 0: the compiler then emits the instruction without its scale-loading half
    // (v_mfma_f32_32x32x64_f8f6f4, block scales 1.0), half the code bytes and one operand read less per MFMA
    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.b[j].v, f.a[i].v, acc[i][j], 0, 0, 0, 0, 0, 0);
  };
  auto dma_one = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst_slab) {
    const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(dst_slab + lds_wave);
    // (m0 written by the compiler, as in the 16-bit kernel)
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "{m0}"(m0v), "v"(voff), "s"(src_uniform)
                 : "memory");
  };
  const uint8_t *a_cur, *b_cur, *a_nxt, *b_nxt;
  struct Voffs { uint32_t a[4]; uint32_t b; int last_row; };   // RAGGED: a tile's per-thread offsets, clamped into the matrix
  Voffs vo_cur, vo_nxt;
  const uint32_t z_voff = (uint32_t)tid * 16;
  // (whole tiles: the offsets are the same for every tile, so only the first call works them out)
  auto tile_bases = [&](int t, const uint8_t *&ap, const uint8_t *&bp, Voffs &vo, bool offsets = RAGGED) {
    int tm, tn, half;
    fast::item_tile<MB>(items, min(t, total - 1), tiles_mv, tiles_n, tm, tn, half);
    int slice = 0;
    if constexpr (SPLITK) {
      slice = tm / tiles_m;
      tm -= slice * tiles_m;
    }
    int64_t row0 = (int64_t)tm * BM + half * 128;
    // RAGGED: a lower half that starts past the last row is pointed at the upper half's rows; its stores all
    // fall to the clipping
    if (RAGGED && MB == 2 && row0 >= g.M) row0 = (int64_t)tm * BM;
    ap = A + row0 * g.lda + (int64_t)slice * BK;
    bp = B + (int64_t)tn * BN + (int64_t)slice * BK * g.ldb;
    if (RAGGED || offsets) {
      const int last_row = RAGGED ? g.M - 1 - (int)row0 : BM;
      vo.last_row = last_row;
      const int last_chunk = RAGGED ? (g.N - tn * BN) / 16 - 1 : 16;        // N is a multiple of 16
#pragma unroll
      for (int i = 0; i < MB; ++i) vo.a[i] = (uint32_t)((int64_t)min(i * 64 + a_row, last_row) * g.lda + a_chunk * 16);
      vo.b = (uint32_t)((int64_t)b_k * g.ldb + min(b_chunk, last_chunk) * 16);
    }
  };
  // `inner`: step kk belongs to this tile and carries data (see the 16-bit kernel)
  auto dma_single = [&](int kk, uint8_t *stage, int i, auto inner_) {
    constexpr bool inner = decltype(inner_)::value;
    const bool over = !inner && kk >= nk;
    const int k = over ? kk - nk : kk;
    if constexpr (inner) {
      if (i < MB)
        dma_one(a_cur + (int64_t)k * a_kstep, vo_cur.a[i], stage + i * 4096);
      else
        dma_one(b_cur + (int64_t)k * b_kstep + (i - MB) * b_slab, vo_cur.b, stage + A_BYTES + (i - MB) * 4096);
    } else if constexpr (RAGGED) {
      const bool zero = k >= nk_real;
      const Voffs &vo = over ? vo_nxt : vo_cur;
      if (i < MB) {
        const uint8_t *ap = zero ? fast::zero_page : (over ? a_nxt : a_cur) + (int64_t)k * a_kstep;
        dma_one(ap, zero ? z_voff : vo.a[i], stage + i * 4096);
      } else {
        const uint8_t *bp = zero ? fast::zero_page : (over ? b_nxt : b_cur) + (int64_t)k * b_kstep + (i - MB) * b_slab;
        dma_one(bp, zero ? z_voff : vo.b, stage + A_BYTES + (i - MB) * 4096);
      }
    } else if (i < MB) {
      const uint8_t *ap = (over ? a_nxt : a_cur) + (int64_t)k * a_kstep;
      dma_one(ap + i * a_slab, a_voff, stage + i * 4096);
    } else {
      const uint8_t *bp = (over ? b_nxt : b_cur) + (int64_t)k * b_kstep;
      dma_one(bp + (i - MB) * b_slab, b_voff, stage + A_BYTES + (i - MB) * 4096);
    }
  };

  auto use_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" ::"a"(acc[i][j]));
  };
  // APAIR: copy number i (0..7) of the pair of steps (kk, kk+1), kk even, into pair buffer P
  auto dma_pair = [&](int kk, int P, int i, auto inner_) {
    constexpr bool inner = decltype(inner_)::value;
    const bool over = !inner && kk >= nk;
    const int k = over ? kk - nk : kk;
    uint8_t *dst = ring.s[2 * P + (i >> 2)] + (i & 3) * 4096;
    if constexpr (RAGGED) {
      // as in the 16-bit kernel: rows past M come from the last row; K is a whole number of steps here, so a pair
      // holds 128, 64 (its second step is padding: fetched from the pair's first chunk, cleared by clear_pair) or 0
      // bytes (the page of zeros) of each row; the turns of a tile whose 256 rows all exist take the form without
      // any of this (value 2), because the VALU operations below, once per copy, would cost more than the whole
      // lines gain
      if constexpr (decltype(inner_)::value == 2) {
        dma_one(a_cur + (int64_t)(k >> 1) * 128 + i * a_slab32, a_voff_pair, dst);
      } else {
        const int valid = inner ? 128 : min(max(g.K - 64 * k, 0), 128);
        int r8 = pair_r8, c = pair_c;
        asm volatile("" : "+v"(r8), "+v"(c));
        const int row = min(i * 32 + r8, (over ? vo_nxt : vo_cur).last_row);
        if (!inner && 16 * c + 16 > valid) c = 0;
        const uint32_t voff = (uint32_t)row * (uint32_t)g.lda + (uint32_t)c * 16;
        const uint8_t *ap = valid == 0 ? fast::zero_page : (over ? a_nxt : a_cur) + (int64_t)(k >> 1) * 128;
        dma_one(ap, valid == 0 ? z_voff : voff, dst);
      }
    } else {
      const uint8_t *ap = (over ? a_nxt : a_cur) + (int64_t)(k >> 1) * 128 + i * a_slab32;
      dma_one(ap, a_voff_pair, dst);
    }
  };
  // RAGGED: this thread's sixteen bytes of each slab of pair buffer P, when they belong to the pair's second step
  // and that step is padding
  auto clear_pair = [&](int P) {
    typedef __attribute__((address_space(3))) i32x4 lds_i32x4;
    if (pair_c >= 4) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *(lds_i32x4 *)(lds_void *)(ring.s[2 * P + (i >> 2)] + (i & 3) * 4096 + lds_wave + lane * 16) = (i32x4){0, 0, 0, 0};
    }
  };
  // One step (K += 64) on ring stage I: 16 MFMAs on `c` (read from stage I during the previous
  // step), the next stage's fragments into `p`, and the refill of stage I itself with step k+R.
  auto step = [&](auto I_, int k, Frags &c, Frags &p, auto inner_) {
    constexpr int I = decltype(I_)::value;
    uint8_t *cur = ring.s[I], *nxt = ring.s[(I + 1) % R];
    mm(c, 0);
    FENCE();
    // every wave's reads of stage I have returned (they fed `c`), and this wave's share of the
    // copy into stage I+1 has landed (the 16 younger copies may still be in flight); after the
    // barrier that holds for all waves: I+1 may be read, I may be overwritten
    if constexpr (MB == 4) {
      // APAIR: an odd step issues the 8 copies of the A pair whose buffer its barrier has freed (steps k+3, k+4) and
      // then its 4 B copies, an even step only its 4 B copies; a barrier needs B of the next step and the A pair
      // that step lies in, which on an even step leaves 4 + 8 + 4 younger copies in flight and on an odd one 4 + 4.
      if constexpr (RAGGED && APAIR && (I & 1) && !decltype(inner_)::value) {
        // the pair about to open (its first step is the next one) has a padding step for its second: clear it
        const int kn = k + 1 == nk ? 0 : k + 1;
        if (g.K - 64 * kn == 64) {
          asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
          clear_pair(((I + 1) % R) >> 1);
        }
      }
      if constexpr (APAIR && (I & 1))
        asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else
        asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      FENCE();
#pragma unroll
      for (int n = 1; n < 16; ++n) {
        if (n <= 12) {
          rd(p, nxt, (I + 1) % R, 2 * (n - 1));
          rd(p, nxt, (I + 1) % R, 2 * (n - 1) + 1);
        }
        if constexpr (APAIR) {
          if constexpr (I & 1) {
            if (n >= 3 && n <= 14) {          // twelve copies, one per MFMA (64 cycles)
              if (n - 3 < 8) dma_pair(k + 3, (I - 1) >> 1, n - 3, inner_);
              else dma_single(k + R, cur, MB + n - 11, inner_);
            }
          } else {
            if (n >= 5 && n <= 14 && (n - 5) % 3 == 0) dma_single(k + R, cur, MB + (n - 5) / 3, inner_);
          }
        } else {
          if (n & 1) dma_single(k + R, cur, n >> 1, inner_); // one copy per two MFMAs: thin enough not to stall issue
        }
        mm(c, n);
        FENCE();
      }
    } else {
      // half tiles: 8 MFMAs, 20 fragment reads (three per MFMA) and 6 copies per step; the two youngest
      // steps' copies (12) may still be in flight at the barrier
      asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      FENCE();
#pragma unroll
      for (int n = 1; n < 8; ++n) {
#pragma unroll
        for (int r = 3 * (n - 1); r < 3 * n && r < 20; ++r) rd(p, nxt, (I + 1) % R, r);
        if (n <= 6) dma_single(k + R, cur, n - 1, inner_);
        mm(c, n);
        FENCE();
      }
    }
    // Outside the peeled turns nothing reads the accumulators before the epilogue, and an MFMA is a pure function
    // to the compiler: it sinks all 64 of a turn past the turn's barriers, down to the epilogue, keeps four steps
    // of fragments alive for that and spills them (each reload is a memory operation whose wait drains the copies
    // in flight: such a turn then takes four times its time).  A use of every accumulator here keeps the MFMAs
    // in the step they belong to.
    if constexpr (!decltype(inner_)::value) use_acc();
  };

  int t = blockIdx.x;
  if (t >= total) return;
  tile_bases(t, a_cur, b_cur, vo_cur, true);
  // no copy of the fill looks at the next tile.  RAGGED: where it lies is worked out before the last turns of each
  // tile, so that its offsets are not held through the turns before; whole tiles: one tile ahead, at the end of a tile
  a_nxt = a_cur;
  b_nxt = b_cur;
  vo_nxt = vo_cur;
  if constexpr (!RAGGED) tile_bases(t + (int)gridDim.x < total ? t + (int)gridDim.x : t, a_nxt, b_nxt, vo_nxt);
  // fill the ring with steps 0..R-1
  if constexpr (APAIR) {
    // in the order the steps of a turn issue them: pair (0,1), B 0, B 1, B 2, pair (2,3), B 3
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_pair(0, 0, i, std::false_type{});
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) dma_single(s, ring.s[s], MB + i, std::false_type{});
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_pair(2, 1, i, std::false_type{});
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_single(3, ring.s[3], MB + i, std::false_type{});
  } else {
#pragma unroll
    for (int s = 0; s < R; ++s)
#pragma unroll
      for (int i = 0; i < MB + 4; ++i) dma_single(s, ring.s[s], i, std::false_type{});
  }
  if constexpr (RAGGED && APAIR) {
    if (g.K < 256 && (g.K & 127)) {          // one of the first tile's two pairs ends in a padding step
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      clear_pair(g.K < 128 ? 0 : 1);
    }
  }
  // step 0 has landed when only the (R - 1) * (MB + 4) younger copies are left in flight (APAIR: B 1, B 2, the
  // second pair and B 3)
  if constexpr (APAIR)
    asm volatile("s_waitcnt vmcnt(20) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  else if constexpr (MB == 4)
    asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  else
    asm volatile("s_waitcnt vmcnt(18) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
  for (int r = 0; r < 16 + 2 * MB; ++r) rd(f0, ring.s[0], 0, r);

  for (; t < total; t += gridDim.x) {
    int tm, tn, half;
    fast::item_tile<MB>(items, t, tiles_mv, tiles_n, tm, tn, half);
    int slice = 0;
    if constexpr (SPLITK) {
      slice = tm / tiles_m;
      tm -= slice * tiles_m;
    }
    const int64_t m0 = (int64_t)tm * BM + half * 128, n0 = (int64_t)tn * BN;
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = (f32x16){0};
    int k = 0;
    // turns of the ring whose copies (up to step k + 2R - 1) all carry this tile's data
    if (RAGGED && APAIR && __builtin_amdgcn_readfirstlane(vo_cur.last_row) >= BM - 1) {
      // (a tile whose 256 rows all exist: the copies of A need no clamping)
      for (; k + 2 * R <= nk_real; k += R) {
        step(std::integral_constant<int, 0>{}, k, f0, f1, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 1>{}, k + 1, f1, f0, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 2>{}, k + 2, f0, f1, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{}, k + 3, f1, f0, std::integral_constant<int, 2>{});
      }
    }
    for (; k + 2 * R <= nk_real; k += R) {
      step(std::integral_constant<int, 0>{}, k, f0, f1, std::true_type{});
      step(std::integral_constant<int, 1>{}, k + 1, f1, f0, std::true_type{});
      step(std::integral_constant<int, 2>{}, k + 2, f0, f1, std::true_type{});
      step(std::integral_constant<int, 3>{}, k + 3, f1, f0, std::true_type{});
    }
    // the remaining turns copy the next tile's first steps (this tile's again when there is none: a harmless
    // refetch); RAGGED: where that tile lies is worked out only now
    if constexpr (RAGGED) tile_bases(t + (int)gridDim.x < total ? t + (int)gridDim.x : t, a_nxt, b_nxt, vo_nxt);
    for (; k < nk; k += R) {
      step(std::integral_constant<int, 0>{}, k, f0, f1, std::false_type{});
      step(std::integral_constant<int, 1>{}, k + 1, f1, f0, std::false_type{});
      step(std::integral_constant<int, 2>{}, k + 2, f0, f1, std::false_type{});
      step(std::integral_constant<int, 3>{}, k + 3, f1, f0, std::false_type{});
    }
    a_cur = a_nxt;
    b_cur = b_nxt;
    if constexpr (RAGGED) {
      vo_cur = vo_nxt;
    } else {
      // whole tiles: only the two addresses change from tile to tile; the tile after the next
      const int t2 = t + 2 * (int)gridDim.x;
      tile_bases(t2 < total ? t2 : (t + (int)gridDim.x < total ? t + (int)gridDim.x : t), a_nxt, b_nxt, vo_nxt);
    }
    // ---- epilogue: acc[i][j] register r of lane l is C[m][n] with
    //      m = i*32 + l%32,  n = j*32 + (r/4)*8 + (l/32)*4 + r%4
    const int64_t m = m0 + wm * (32 * MB) + l32;
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const int64_t mi = m + i * 32;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (SPLITK) {
          // the slice's sums as they are: four columns of a row are sixteen contiguous bytes of the slab
          float *slab = (float *)g.c + (int64_t)slice * g.M * g.ldws;
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const int64_t n = n0 + wn * 128 + j * 32 + r4 * 8 + hi * 4;
            if (mi >= g.M || n >= g.N) continue;
            *(f32x4 *)(slab + mi * g.ldws + n) =
                (f32x4){acc[i][j][r4 * 4], acc[i][j][r4 * 4 + 1], acc[i][j][r4 * 4 + 2], acc[i][j][r4 * 4 + 3]};
          }
        } else if constexpr (OUT_DT == DT_FP8) {
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const int64_t n = n0 + wn * 128 + j * 32 + r4 * 8 + hi * 4;
            if (RAGGED && (mi >= g.M || n >= g.N)) continue;
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][r4 * 4 + e] * g.scale;
            // FP8_OUTPUT (09-persistent-matmul.py:116,173): four e4m3 codes, one 4-byte store
            const uint32_t q = (uint32_t)f32_to_fp8(v[0]) | ((uint32_t)f32_to_fp8(v[1]) << 8) |
                               ((uint32_t)f32_to_fp8(v[2]) << 16) | ((uint32_t)f32_to_fp8(v[3]) << 24);
            *(uint32_t *)((uint8_t *)g.c + mi * g.ldc + n) = q;
          }
        } else {
          // 16-byte stores, four lanes to a row's 64 contiguous bytes.  A lane holds columns 8g + 4hi .. +3 (g = 0..3) of
          // row l % 32 of the 32x32 block.  First the lane pair (l, l+32) exchanges its middle column groups
          // (v_permlane32_swap): the lower lane then holds columns 0-7 and 16-23, the upper one 8-15 and 24-31.  Then
          // sixteen-lane rows 0 / 1 and 2 / 3 of the wavefront exchange (v_permlane16_swap: odd rows of its first
          // operand <-> even rows of its second) the second piece of the lanes that hold block row r < 16 with the first
          // piece of the lanes that hold block row r + 16: afterwards every lane's first piece belongs to block row
          // l % 16 and its second to block row l % 16 + 16, at columns {0, 16, 8, 24}[l / 16] .. +7, so that one store
          // instruction writes sixteen rows in segments of 64 bytes (32-byte segments before: the writes that reached
          // memory were 1.15 times the bytes of C).
          u32x4 pc[2];      // after the swaps: [0] block row l % 16, [1] block row l % 16 + 16
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            u32x2 p[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              float v[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) v[e] = acc[i][j][(2 * q + h) * 4 + e] * g.scale;
              if constexpr (OUT_DT == DT_BF16)
                p[h] = (u32x2){pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
              else
                p[h] = (u32x2){(uint32_t)f32_to_f16(v[0]) | ((uint32_t)f32_to_f16(v[1]) << 16),
                               (uint32_t)f32_to_f16(v[2]) | ((uint32_t)f32_to_f16(v[3]) << 16)};
            }
            asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(p[0].x), "+v"(p[1].x));
            asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(p[0].y), "+v"(p[1].y));
            pc[q] = (u32x4){p[0].x, p[0].y, p[1].x, p[1].y};   // columns q*16 + hi*8 .. +7 of block row l % 32
          }
          asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(pc[0].x), "+v"(pc[1].x));
          asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(pc[0].y), "+v"(pc[1].y));
          asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(pc[0].z), "+v"(pc[1].z));
          asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(pc[0].w), "+v"(pc[1].w));
          const int64_t n = n0 + wn * 128 + j * 32 + ((lane >> 4) & 1) * 16 + hi * 8;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int64_t mr = m0 + wm * (32 * MB) + i * 32 + half * 16 + (lane & 15);
            if (RAGGED && (mr >= g.M || n >= g.N)) continue;     // N is a multiple of 16
            if constexpr (STREAM)
              __builtin_nontemporal_store(pc[half], (u32x4 *)((uint16_t *)g.c + mr * g.ldc + n));
            else
              *(u32x4 *)((uint16_t *)g.c + mr * g.ldc + n) = pc[half];
          }
        }
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

} // namespace fast8

extern "C" {

#define GEMM_TILE_FP8(name, OUT, STREAM)                                                            \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast8::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast8::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast8::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast8::STAGE];                            \
    fast::Ring ring = {{lds0, lds1, lds2, lds3}};                                                    \
    fast8::body<OUT, false, 4, STREAM>(g, ring);                                                     \
    fast8::body<OUT, false, 2, STREAM>(g, ring);                                                     \
  }

GEMM_TILE_FP8(gemm_tile_fp8_bf16, DT_BF16, false)
GEMM_TILE_FP8(gemm_tile_fp8_f16, DT_F16, false)
GEMM_TILE_FP8(gemm_tile_fp8_fp8, DT_FP8, false)
GEMM_TILE_FP8(gemm_tile_fp8_bf16_stream, DT_BF16, true)
GEMM_TILE_FP8(gemm_tile_fp8_f16_stream, DT_F16, true)

#define GEMM_RAGGED_FP8(name, OUT, STREAM)                                                          \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast8::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast8::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast8::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast8::STAGE];                            \
    fast::Ring ring = {{lds0, lds1, lds2, lds3}};                                                    \
    fast8::body<OUT, true, 4, STREAM>(g, ring);                                                      \
    fast8::body<OUT, true, 2, STREAM>(g, ring);                                                      \
  }
GEMM_RAGGED_FP8(gemm_ragged_fp8_bf16, DT_BF16, false)
GEMM_RAGGED_FP8(gemm_ragged_fp8_f16, DT_F16, false)
GEMM_RAGGED_FP8(gemm_ragged_fp8_fp8, DT_FP8, false)
GEMM_RAGGED_FP8(gemm_ragged_fp8_bf16_stream, DT_BF16, true)
GEMM_RAGGED_FP8(gemm_ragged_fp8_f16_stream, DT_F16, true)

// few tiles under a long K: slices of K as work items (see SPLITK in body), fp32 sums into the workspace
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_splitk_fp8(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast8::STAGE];
  __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast8::STAGE];
  __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast8::STAGE];
  __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast8::STAGE];
  fast::Ring ring = {{lds0, lds1, lds2, lds3}};
  fast8::body<DT_BF16, true, 2, false, true>(g, ring);
}

} // extern "C"
