// gemm_tile_*: the fast tile-matmul path for gfx950.
//
// Requirements (checked by the host): M and N multiples of 256, K a multiple of
// 128, 16-byte aligned bases and leading strides, and a logical grid that covers
// every tile -- then which physical tile computes which part of C does not show
// in the result (up to fp32 summation order).
//
// One workgroup (4 wavefronts, 2x2) computes a 256x256 macro tile.  Each
// wavefront owns 128x128 of it: 8x8 v_mfma_f32_16x16x32 accumulators (256
// registers), hence one wavefront per SIMD.  The grid is persistent, one
// workgroup per CU, striding over the macro tiles in an XCD-aware order.
//
// Why the 16x16x32 shape and not 32x32x16: the part is power-limited under this kernel, and per flop the
// smaller tile with the deeper dot product costs less energy (an accumulator is read and written once per 32
// multiply-adds instead of once per 16).  A loop of nothing but MFMAs on random operands sustains 1990 TFLOP/s
// with it against 1735 with 32x32x16 (2440 with all-zero operands, either shape); this kernel went from 1343
// to 1470 on 8192^3 in one process.  Fragment bytes read from LDS per step are the same for both shapes.
//
// K is walked in steps of 32 through a ring of four LDS stages (A 256x32 +
// B 32x256 = 32 KiB per stage).  Data goes global -> LDS directly
// (global_load_lds_dwordx4, no register staging) three steps ahead of its use,
// and the ring runs on across tile boundaries, so the first steps of the next
// tile are already in flight while the current tile's epilogue stores C.  LDS ->
// registers runs one step ahead of the MFMAs that consume it (two full sets of
// fragments).  A single wavefront thus keeps its matrix pipe fed without a second
// one to hide behind: every stall that matters (HBM/L2 latency, LDS latency) is
// covered by distance in the software pipeline.
//
// LDS layout per stage (16-byte chunks, XOR-swizzled so that the row-wise A
// reads and the transposing B reads are both bank-conflict free):
//   A: row m = 64 B = 4 chunks;   logical chunk c sits at c ^ a_swz((m>>2)&3)
//   B: row k = 512 B = 32 chunks; logical chunk c sits at c ^ (((k&3)<<2) | (((k>>3)&1)<<1));
//      the k rows are dealt to the four 4 KiB slabs as {0-3, 8-11}, {4-7, 12-15}, {16-19, 24-27}, {20-23, 28-31}
// (The macro-tile pass of the plain row-major kernel keeps A differently: 128-byte rows holding two K steps, copied
// as whole cache lines, see APAIR in body.)
// A direct-to-LDS load writes lane l's 16 bytes at (wave-uniform base) + 16*l,
// so thread t owns byte 16*t of every 4 KiB slab and the swizzle is applied to
// the global address it fetches.
//
// The product is formed transposed, acc = mfma(Bfrag, Afrag): a result lane then
// holds 4 consecutive n of one m, so epilogue stores and bias loads are 8 bytes
// wide (16 after an exchange between neighbouring lane groups).  B fragments need
// k along the lane's registers while memory has n contiguous: ds_read_b64_tr_b16
// transposes a 4x16 block of 16-bit values across each group of 16 lanes on the
// way out of LDS.
//
// RAGGED variant (M any, N and K multiples of 8): same kernel, three differences.  Rows of A
// beyond M and 16-byte column chunks of B beyond N are fetched from the last valid row / chunk instead (their
// products land in parts of the macro tile that are never stored); K is padded to whole turns of the ring
// with steps whose A and B slabs are copied from a page of zeros (exact: 0 * 0 accumulates nothing, whatever
// the real operands hold; a last step that ends past K is cleared from K on once it has landed); and the stores
// are clipped at M and N.  The MFMA stream has no branch in it.
#pragma once
#include <type_traits>

#include "gemm_common.h"

namespace fast {

// source of the zero steps of the RAGGED variant: 256 lanes x 16 bytes
__device__ __attribute__((aligned(4096))) const uint8_t zero_page[4096] = {0};

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int R = 4;                        // ring depth
constexpr int A_BYTES = BM * BK * 2;        // 16 KiB
constexpr int B_BYTES = BK * BN * 2;        // 16 KiB
constexpr int STAGE = A_BYTES + B_BYTES;    // 32 KiB
constexpr int DMA_PER_STEP = 8;             // direct-to-LDS loads per thread and step

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void global_void;

template <int IN_DT> struct MFMA;
// Written as assembly with the accumulator tied to an AGPR: given the builtin, the compiler moves some of the 64
// four-register accumulators of a wavefront through VGPRs around every MFMA (copies and the wait states they need
// inside the K loop).  Each accumulator is touched once per step, far from any hazard distance; the epilogue waits
// out the last MFMAs before it reads (see there).
template <> struct MFMA<DT_BF16> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ void run(vec a, vec b, f32x4 &c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  // The MFMA and, behind it, one direct-to-LDS copy (m0: its LDS destination, written by the compiler in front of
  // the statement): the MFMA is the wait state that the copy needs after a write to m0.
  static __device__ __forceinline__ void run_copy(vec a, vec b, f32x4 &c, uint32_t m0v, uint32_t voff, const uint8_t *src) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5"
                 : "+a"(c)
                 : "v"(a), "v"(b), "{m0}"(m0v), "v"(voff), "s"(src)
                 : "memory");
  }
};
template <> struct MFMA<DT_F16> {
  typedef f16x8 vec;
  static __device__ __forceinline__ void run(vec a, vec b, f32x4 &c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  // The MFMA and, behind it, one direct-to-LDS copy (m0: its LDS destination, written by the compiler in front of
  // the statement): the MFMA is the wait state that the copy needs after a write to m0.
  static __device__ __forceinline__ void run_copy(vec a, vec b, f32x4 &c, uint32_t m0v, uint32_t voff, const uint8_t *src) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5"
                 : "+a"(c)
                 : "v"(a), "v"(b), "{m0}"(m0v), "v"(voff), "s"(src)
                 : "memory");
  }
};

// Macro-tile order: the dispatcher deals consecutive workgroup ids round-robin
// to the 8 XCDs, so give each XCD a contiguous run of tile ids (its L2 then sees
// neighbouring tiles) and walk the ids in 8-row column-major bands.
__device__ __forceinline__ void tile_of(int t, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int total = tiles_m * tiles_n;
  constexpr int XCD = 8, G = 8;
  int id = t;
  if (total % XCD == 0) id = (t % XCD) * (total / XCD) + t / XCD;
  const int in_group = G * tiles_n;
  const int group = id / in_group;
  const int first_m = group * G;
  const int gsz = min(tiles_m - first_m, G);
  tm = first_m + (id % in_group) % gsz;
  tn = (id % in_group) / gsz;
}

// Work items of one pass of a kernel that finishes a short last round as parts of tiles: the macro-tile pass
// (MB == 4) takes the whole rounds of the grid, or every tile when the tail is not worth splitting; the
// half-tile pass (MB == 2) takes the two 128-row halves of each tail tile when those keep at most the whole grid
// busy, and (QUARTERS) the quarter-tile pass (MB == 1) the four 64-row quarters when even they do.
// `live_rows`: rows of a macro tile that exist, where that is the same for every tile (256 for whole tiles; M for a
// clamping kernel whose matrix is a single row of tiles).  Halves and quarters that lie wholly past them are not
// work items: a 64-row matrix is finished as one quarter per tile, not as four of which three store nothing.
struct PassItems {
  int total;       // items of this pass
  int first_tile;  // MB < 4: id of the first tail tile
  int tail_tiles;
  int parts;       // MB < 4: live parts of a tile (halves: 1..2, quarters: 1..4)
};
// ALLQ: every tile is finished as its live quarters, or halves (the kernels of the K slices, whose launches have no
// whole round).
template <int MB, bool SPLIT_TAIL, bool QUARTERS = false, bool ALLQ = false>
__device__ __forceinline__ PassItems pass_items(int total_tiles, int live_rows) {
  PassItems p = {total_tiles, 0, 0, 1};
  if constexpr (ALLQ) {      // (the fp8 kernels' smallest part is the half)
    p.parts = MB == 2 ? (live_rows + 127) >> 7 : (live_rows + 63) >> 6;
    p.total = p.parts * total_tiles;
    p.tail_tiles = total_tiles;
  } else if constexpr (SPLIT_TAIL) {
    const int whole = total_tiles / (int)gridDim.x * (int)gridDim.x;
    p.tail_tiles = total_tiles - whole;
    const int q_live = (live_rows + 63) >> 6, h_live = (live_rows + 127) >> 7;
    const bool quarters = QUARTERS && p.tail_tiles > 0 && q_live * p.tail_tiles <= (int)gridDim.x;
    const bool halves = !quarters && p.tail_tiles > 0 && h_live * p.tail_tiles <= (int)gridDim.x;
    if (MB == 4) {
      p.total = (quarters || halves) ? whole : total_tiles;
    } else {
      p.parts = MB == 2 ? h_live : q_live;
      p.total = MB == 2 ? (halves ? h_live * p.tail_tiles : 0) : (quarters ? q_live * p.tail_tiles : 0);
      p.first_tile = whole;
    }
  }
  return p;
}
// item -> macro tile and which part of it (0 .. 4/MB - 1).  Workgroup ids go round-robin over the 8 XCDs and
// tile_of gives tile t to XCD t % 8's run of ids, so parts are dealt in groups of 8 tiles: all parts of a tile
// then stay on the XCD that tile's neighbours ran on.
template <int MB>
__device__ __forceinline__ void item_tile(const PassItems &p, int item, int tiles_m, int tiles_n, int &tm, int &tn,
                                          int &part) {
  if constexpr (MB == 4) {
    part = 0;
    tile_of(item, tiles_m, tiles_n, tm, tn);
  } else {
    // (p.parts is the constant 4 / MB in the kernels for whole tiles: shifts and masks there)
    int j;
    if (p.tail_tiles % 8 == 0) {
      j = (item >> 3) / p.parts * 8 + (item & 7);
      part = (item >> 3) % p.parts;
    } else {
      j = item / p.parts;
      part = item % p.parts;
    }
    tile_of(p.first_tile + j, tiles_m, tiles_n, tm, tn);
  }
}

#define FENCE() __builtin_amdgcn_sched_barrier(0)

// Swizzle of A's 16-byte chunks within a 64-byte row, by the row's group of four (0..3) -> 0, 2, 3, 1.
// A 16-byte LDS read of a wavefront is served in four passes of sixteen lanes, and not of neighbouring lanes:
// lanes {0-3, 12-15, 20-23, 24-27} go together, then {4-7, 8-11, 16-19, 28-31}, and the same with 32 added.  With
// the fragment layout of the 16x16x32 MFMA (lane l: row l%16, chunk l/16) a pass therefore holds two groups of four
// rows with chunk g and two with chunk g^1, and each group of four rows spans all 256 bytes of the banks at one
// chunk position: the four positions of a pass must differ.  c ^ (row group) does not do that (measured: every A
// read took twice its cycles, SQ_LDS_BANK_CONFLICT = a third of SQ_LDS_IDX_ACTIVE); this permutation does.
__device__ __forceinline__ int a_swz(int row_group) { return (((row_group ^ (row_group >> 1)) & 1) << 1) | (row_group >> 1); }
// The same for A rows of 128 bytes (8 chunks: two K steps side by side, the layout of the plain kernel's macro-tile
// pass): two rows share a line of banks, so the eight even (odd) rows of a pass need eight different positions.
__device__ __forceinline__ int a_swz_pair(int row) { return (row & 2) | ((row & 8) >> 1); }

struct Ring {
  uint8_t *s[R];
};

// TILED: operands are the tile-major buffers of the pointer-based matmul_kernel with 32x32x32
// tiles (examples/matmul/03-matrix-multiplication.py:326-385).  A 32x32 tile is 2 KiB
// contiguous, i.e. exactly 32 of this kernel's 64-byte LDS rows, so only the global addresses
// of the copies and of the result change: a thread's offset inside a slab, the distance
// between slabs and between K steps.  LDS layout, fragments and MFMA schedule are the same.
//
// MB: 32-row blocks of C per wavefront.  4 is the 256x256 macro tile described above.  With 2 a workgroup
// computes a 128x256 HALF of a macro tile (each wavefront 64x128: 4x8 accumulators, two A slabs and six
// copies per step, 32 MFMAs per step), used for the tail of the persistent loop: when the macro
// tiles left over after the last whole round of the grid would keep at most half of the workgroups busy,
// the kernel runs body<MB=4> over the whole rounds and then body<MB=2> over the halves of the tail tiles,
// two workgroups per tile, instead of leaving half of the chip idle for a whole tile's time.  (RAGGED: a
// half tile that lies wholly past the last row computes the other half's rows again and stores nothing.)
//
// With MB == 1 (QUARTERS) a workgroup computes a 64x256 quarter (each wavefront 32x128: 2x8 accumulators, one A slab
// and five copies per step, 16 MFMAs per step): a problem of at most CUs/4 macro tiles, or such a tail, then fills
// the chip four workgroups to a tile.  A quarter's step moves 20 KiB for a quarter of the flops and its fragment
// reads (18 per wavefront and 16 MFMAs) keep the LDS busier than the matrix pipe, so it runs at about two thirds of
// the macro tile's rate: worth it only where the alternative is idle CUs.
//
// STREAM: the stores of C go past the caches.  A plain store leaves its line in the L2 and in the 256 MiB
// memory-side cache, which drain it while the next tile multiplies; that is right while C fits there.  A larger C
// only evicts operands on its way through, which shows where K is short and operands are re-read soon:
// 16384 x 16384 x 1024 runs 8.5 % faster with streaming stores and x 2048 3.7 %, x 4096 0.6 % slower, 8192^3 0.5 %
// slower and 8192 x 8192 x 1024 (a C of 128 MiB) 15 % slower.  The host picks the streaming kernels for a C beyond
// 256 MiB at K <= 2048.  They are kernels of their own (plain epilogue only): with both forms of the stores inside
// one kernel, several instantiations spilled copy offsets whose reloads the compiler then waits for inside the K
// loop, with every copy in flight counted in (tile-major 8192^3: 1585 -> 1482 TFLOP/s).
//
// SPLITK: K is dealt to g.ksplit slices of equal size, a step at a time, and a work item is one slice of one macro tile;
// slice s of tile (tm, tn) leaves its fp32 sums, nothing applied, in slab s of a workspace of ksplit x M x N floats
// that g.c points at, and gemm_splitk_reduce adds the slabs in slice order and does the rest.  For a C of few macro
// tiles under a long K: 128 x 8192 x 8192 has 32 tiles for 256 CUs, each streaming all of K on its own.
template <int IN_DT, int OUT_DT, int EPI, bool TILED = false, bool RAGGED = false, int MB = 4, bool SPLIT_TAIL = false,
          bool QUARTERS = false, bool STREAM = false, bool SPLITK = false, bool ALLQ = false>
__device__ __forceinline__ void body(const GemmArgs &g, const Ring &ring) {
  static_assert(!ALLQ || (MB == 1 && SPLITK), "quarters only: the K-slice kernels");
  // where B's slabs start in a stage.  ALLQ: right behind the one A slab a quarter has, so that a stage is 20 KiB,
  // the ring 80 KiB and two workgroups share a CU
  constexpr int B_OFF = ALLQ ? 4096 : A_BYTES;
  static_assert(MB == 4 || ((MB == 2 || (MB == 1 && QUARTERS)) && SPLIT_TAIL), "part tiles exist for the tail passes only");
  static_assert(!SPLITK || (RAGGED && EPI == EPI_NONE && !STREAM), "slices of K: the clamping kernels");
  const int gK = SPLITK ? g.K / g.ksplit : g.K;      // the K of one work item
  // TILED && RAGGED: the buffers are padded to whole 32x32 tiles (zeros), so "the matrix" the fetches are clamped
  // into is the padded one and K needs no more than whole turns of the ring; the stores are clipped at the
  // real M and N (the padding of C is never written, as under the reference's store mask).
  const int Mf = TILED ? (g.M + 31) / 32 * 32 : g.M, Nf = TILED ? (g.N + 31) / 32 * 32 : g.N;   // fetchable extent
  const int Kf = (TILED || RAGGED) ? (gK + 31) / 32 * 32 : gK;   // K in whole steps (row-major RAGGED: the last step may end past K)
  using X = MFMA<IN_DT>;
  using vec = typename X::vec;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = RAGGED ? (g.M + BM - 1) / BM : g.M / BM, tiles_n = RAGGED ? (g.N + BN - 1) / BN : g.N / BN;
  const int tiles_mv = SPLITK ? tiles_m * g.ksplit : tiles_m;   // SPLITK: row tm + tiles_m * s of the item grid is slice s of tile row tm
  const int total_tiles = tiles_mv * tiles_n;
  const PassItems items = pass_items<MB, SPLIT_TAIL, QUARTERS, ALLQ>(total_tiles, (RAGGED && tiles_m == 1) ? g.M : BM);
  const int total = items.total;
  const int nk_real = Kf / BK;                                    // steps that carry data
  const int nk = RAGGED ? (nk_real + R - 1) / R * R : nk_real;    // steps per tile, a multiple of R

  // ---- global -> LDS: thread t writes byte 16*t of each 4 KiB slab ----
  // A slab i (64 rows): row = i*64 + (t>>2), chunk position t&3 holds logical chunk (t&3) ^ a_swz((row>>2)&3)
  const int a_row = tid >> 2;
  const int a_chunk = (tid & 3) ^ a_swz((a_row >> 2) & 3);
  // B slab i (8 rows of 512 B): row t>>5 of the slab holds k = b_row0(i) + b_kk, b_row0(i) = 4*(i&1) + 16*(i>>1),
  // b_kk = (t>>5 & 3) + 8*(t>>7); position t&31 holds logical chunk (t&31) ^ (((k&3)<<2) | (((k>>3)&1)<<1)).  The
  // swizzle depends on bits 0, 1 and 3 of k, and the rows are dealt to the slabs so that these are the three bits of
  // t>>5: one offset register then serves all four slabs.
  const int b_r = tid >> 5;
  const int b_kk = (b_r & 3) + 8 * (b_r >> 2);
  const int b_chunk = (tid & 31) ^ ((b_r & 3) << 2) ^ ((b_r >> 2) << 1);
  auto b_row0 = [](int i) { return 4 * (i & 1) + 16 * (i >> 1); };
  // row-major:  A(m,k) at m*lda + k,  B(k,n) at k*ldb + n
  // tile-major: A(m,k) at ((m/32)*ntk + k/32)*1024 + (m%32)*32 + k%32,
  //             B(k,n) at ((k/32)*ntn + n/32)*1024 + (k%32)*32 + n%32          (elements)
  const int64_t ntk = (SPLITK ? (g.K + 31) / 32 : Kf / 32), ntn = Nf / 32;   // (tiles per tile row of the buffers: of all of K)
  const uint32_t a_voff = TILED ? (uint32_t)((((int64_t)(a_row >> 5) * ntk << 10) + (a_row & 31) * 32 + a_chunk * 8) * 2)
                                : (uint32_t)(((int64_t)a_row * g.lda + a_chunk * 8) * 2); // bytes, per thread
  const uint32_t b_voff = TILED ? (uint32_t)((((b_chunk >> 2) << 10) + b_kk * 32 + (b_chunk & 3) * 8) * 2)
                                : (uint32_t)(((int64_t)b_kk * g.ldb + b_chunk * 8) * 2);
  const int64_t a_slab = TILED ? 2 * ntk * 2048 : 64 * g.lda * 2;                  // bytes, uniform
  const int64_t b_rows4 = TILED ? 4 * 32 * 2 : 4 * g.ldb * 2;                       // four k rows of B
  auto b_slab_off = [&](int i) { return ((i & 1) + 4 * (i >> 1)) * b_rows4; };      // slab i's first row, b_row0(i)
  // (SPLITK: the slices are dealt step by step, slice s takes steps s, s + ksplit, ...: all slices then walk
  // through neighbouring rows of B at any one time instead of through ksplit fronts K / ksplit rows apart)
  const int64_t a_kstep1 = TILED ? 2048 : BK * 2;
  const int64_t b_kstep1 = TILED ? ntn * 2048 : (int64_t)BK * g.ldb * 2;
  const int64_t a_kstep = SPLITK ? a_kstep1 * g.ksplit : a_kstep1, b_kstep = SPLITK ? b_kstep1 * g.ksplit : b_kstep1;
  const int lds_wave = wave * 1024;

  // ---- LDS -> fragments ----
  // v_mfma_f32_16x16x32: lane l supplies row (column) l%16 of its operand, k = 8*(l/16) .. +7.
  // A fragment i (16 rows): one 16-byte read, row 16i + l%16, logical chunk l/16.
  // B fragment j (16 columns): two transposing reads, k = 8*(l/16) + 4h + q, q = (l%16)/4, h = 0, 1: the sixteen lanes
  // of a group read a 4 x 16 block (row q, 8 bytes at column 4*(l%4)) and lane i receives column i's four k.
  const int G4 = lane >> 4, i16 = lane & 15, q = i16 >> 2;
  constexpr int NA = 2 * MB;                 // A fragments of a wavefront's 32*MB rows; it has 8 B fragments
  const int a_pos = (wm * (32 * MB) + i16) * 64 + ((G4 ^ a_swz(q)) << 4);   // fragment i: + i * 1024
  // APAIR (the macro-tile pass on row-major operands): A is copied in 128-byte row segments, two K steps at a
  // time, so that every request to the L2 is a whole cache line (64-byte segments are one request each too: 67 M
  // of the 101 M read requests of an 8192^3 launch; with whole lines the kernel measured 4.3 % faster, timing-only
  // variant).  The A regions of stages 2P and 2P+1 together hold the pair of steps (4n + 2P, 4n + 2P + 1): rows
  // 0-127 of the macro tile in the first, rows 128-255 in the second, 128 bytes per row, step h in logical chunks
  // 4h .. 4h+3.  A wavefront's rows all lie in region wm.
  constexpr bool APAIR = !TILED && MB == 4;
  int a_pp[2];      // fragment i of step-half h: region base (stage 2P) + a_pp[h] + i * 2048
#pragma unroll
  for (int h = 0; h < 2; ++h) a_pp[h] = wm * STAGE + i16 * 128 + (((4 * h + G4) ^ a_swz_pair(i16)) << 4);
  // copies of a pair: slab i (0..7) = rows 32i .. 32i+31; thread t: row t>>3, position t&7
  const uint32_t a_voff_pair = (uint32_t)(((int64_t)(tid >> 3) * g.lda) * 2 + (((tid & 7) ^ a_swz_pair(tid >> 3)) << 4));
  const int64_t a_slab32 = 32 * g.lda * 2;
  const int pair_r8 = tid >> 3, pair_c = (tid & 7) ^ a_swz_pair(tid >> 3);   // row in the slab, logical chunk
  // APAIR on whole tiles: a slab's distance from the first one rides in the thread's offset register, one register
  // per slab, so that the copies of a step share one scalar address: two scalar additions less per copy, and with
  // one wavefront per SIMD every instruction between two MFMAs counts (two more scalar instructions per copy cost
  // 2.6 %).  The clamping kernel has no registers to spare for it (it measured 1.5 % slower with them).
  uint32_t a_vp[8], b_vs[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a_vp[i] = a_voff_pair + (uint32_t)(i * a_slab32);
#pragma unroll
  for (int i = 0; i < 4; ++i) b_vs[i] = b_voff + (uint32_t)b_slab_off(i);
  // k = 8*G4 + 4h + q lies in slab h + 2*(G4>>1), row q + 4*(G4&1) of it; its swizzle is (q<<2) | ((G4&1)<<1)
  const int b_base = B_OFF + ((16 * (G4 >> 1) + 4 * (G4 & 1) + q) * 512) + ((wn * 16 + ((i16 >> 1) & 1)) << 4) +
                     ((i16 & 1) << 3);
  int b_pos[8];                                                             // half h: + h * 4096
#pragma unroll
  for (int j = 0; j < 8; ++j) b_pos[j] = b_base + ((j ^ ((q << 1) | (G4 & 1))) << 5);

  const uint8_t *A = (const uint8_t *)g.a;
  const uint8_t *B = (const uint8_t *)g.b;
  const long long probe_c0 = g.probe ? clock64() : 0, probe_w0 = g.probe ? wall_clock64() : 0;

  // Fragment registers: two sets (the step being multiplied and the next one).  B fragments are kept as
  // their two transposed halves (k 0-3 and k 4-7 of the lane's group).
  struct Frags {
    vec a[NA];
    union { s16x4 h[2]; vec v; } b[8];
  };
  Frags f0, f1;
  f32x4 acc[NA][8]; // [16-row block][16-column block]
  constexpr int NR = 16 + NA;   // LDS reads per step
  constexpr int NM = 8 * NA;    // MFMAs per step

  // The LDS reads of one step, in the order the MFMAs will want them:
  // b0.lo b0.hi a0 b1.lo b1.hi ... b7.lo b7.hi a1 ... a(NA-1)
  // (J: ring index of the stage, a constant wherever this is called)
  auto rd = [&](Frags &f, const uint8_t *stage, int J, int r) {
    if constexpr (APAIR) {
      if (r == 2 || r >= 17) {
        const int i = r == 2 ? 0 : r - 16;
        f.a[i] = *(const vec *)(ring.s[J & 2] + a_pp[J & 1] + i * 2048);
        return;
      }
    }
    if (r == 2) {
      f.a[0] = *(const vec *)(stage + a_pos);
    } else if (r < 17) {
      const int rr = r < 2 ? r : r - 1; // 0..15 over the b reads
      const int j = rr >> 1, h = rr & 1;
      f.b[j].h[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(stage + b_pos[j] + h * 4096));
    } else {
      f.a[r - 16] = *(const vec *)(stage + a_pos + (r - 16) * 1024);
    }
  };
  // MFMA number n (0..NM-1) of a step, row-block major: needs a[n/8] and each b once per row block
  auto mm = [&](Frags &f, int n) {
    // (odd row blocks walk the columns backwards: every MFMA then shares one operand with the one before it)
    const int i = n >> 3, j = (i & 1) ? 7 - (n & 7) : (n & 7);
    X::run(f.b[j].v, f.a[i], acc[i][j]);
  };
  // One direct-to-LDS copy: lane l's 16 bytes land at dst_slab + wave*1024 + 16*l.
  // Written as assembly on purpose: the compiler's own bookkeeping of such copies is
  // conservative (it drains every outstanding one before an LDS read it cannot prove
  // unrelated), which would flatten the multi-step prefetch.  Completion is tracked by
  // hand instead: copies retire in issue order, and each step's barrier waits with
  // s_waitcnt vmcnt(n) for exactly the copies that the following reads depend on.
  auto dma_plain = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst_slab) {
    const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(dst_slab + lds_wave);
    // (m0 is the compiler's to write: it then sees a scalar instruction between the MFMA before and this statement
    // and does not pad with a wait state of its own; the one M0 needs before the copy reads it stays in here)
    asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "{m0}"(m0v), "v"(voff), "s"(src_uniform)
                 : "memory");
  };
  // MFMA number n of a step and a copy in one statement (inside the K loop every copy rides behind an MFMA)
  auto mm_copy = [&](Frags &f, int n, const uint8_t *src_uniform, uint32_t voff, uint8_t *dst_slab) {
    const int i = n >> 3, j = (i & 1) ? 7 - (n & 7) : (n & 7);
    const uint32_t m0v = (uint32_t)(uintptr_t)(lds_void *)(dst_slab + lds_wave);
    X::run_copy(f.b[j].v, f.a[i], acc[i][j], m0v, voff, src_uniform);
  };

  // RAGGED with K not a multiple of 32: the last step of every tile holds columns (A) and rows (B) past K:
  // whatever a tile-major buffer holds there, or what the redirected copies of row-major operands brought in
  // (dma_single).  The source masks them to zero
  // (03-matrix-multiplication.py:340-342, 359-361), so a thread clears, in the stage that received the last data
  // step, the part of its OWN sixteen bytes of each slab that lies past K, once its copies have landed and before
  // the barrier that opens the stage for reading.
  const int k_tail = RAGGED ? gK & 31 : 0;                       // valid k of the last data step, 0 = all 32 (row-major: a multiple of 8)
  auto clear_past_k = [&](uint8_t *stage) {
    if constexpr (RAGGED) {
      typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
      // A: this thread's chunk holds k = 8*a_chunk .. 8*a_chunk + 7 of one row, two per 32-bit word
      // (APAIR keeps A in pairs of steps and clears them by the pair, clear_pair)
      if constexpr (!APAIR) {
        const int ka = a_chunk * 8;
        u32x4 keep;
#pragma unroll
        for (int w = 0; w < 4; ++w)
          keep[w] = (ka + 2 * w + 1 < k_tail) ? 0xffffffffu : (ka + 2 * w < k_tail) ? 0x0000ffffu : 0u;
#pragma unroll
        for (int i = 0; i < MB; ++i) {
          lds_u32x4 *p = (lds_u32x4 *)(lds_void *)(stage + i * 4096 + lds_wave + lane * 16);
          *p = *p & keep;
        }
      }
      // B: this thread's sixteen bytes of slab i lie in k row b_row0(i) + b_kk
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lds_u32x4 *p = (lds_u32x4 *)(lds_void *)(stage + B_OFF + i * 4096 + lds_wave + lane * 16);
        if (b_row0(i) + b_kk >= k_tail) *p = (u32x4){0, 0, 0, 0};
      }
    }
  };

  // The stream of steps this workgroup executes: tile after tile, nk steps each.
  // a_cur/b_cur point at the current tile's A rows / B columns, a_nxt/b_nxt at the next
  // tile's (or the current one again when there is none: a harmless refetch).
  const uint8_t *a_cur, *b_cur, *a_nxt, *b_nxt;
  // RAGGED: per-thread byte offsets of a tile's copies, rows and column chunks clamped into the matrix.
  // The A offsets then carry the whole row offset from the tile's first row (a clamp can point backwards
  // from a slab's own first row, and the instruction's register offset is unsigned).
  struct Voffs { uint32_t a[4]; uint32_t b; int last_row; };
  Voffs vo_cur, vo_nxt;
  const uint32_t z_voff = (uint32_t)tid * 16;
  // (whole tiles: the offsets are the same for every tile, so only the first call works them out)
  auto tile_bases = [&](int t, const uint8_t *&ap, const uint8_t *&bp, Voffs &vo, bool offsets = RAGGED) {
    int tm, tn, part;
    item_tile<MB>(items, min(t, total - 1), tiles_mv, tiles_n, tm, tn, part);
    int slice = 0;
    if constexpr (SPLITK) {
      slice = tm / tiles_m;
      tm -= slice * tiles_m;
    }
    int64_t row0 = (int64_t)tm * BM + part * (64 * MB);
    // RAGGED: a lower half that starts past the last row has nothing to fetch or store; it is pointed at the
    // upper half's rows (which exist) and its stores all fall to the clipping
    if (RAGGED && MB < 4 && row0 >= Mf) row0 = (int64_t)tm * BM;
    ap = A + (TILED ? (row0 / 32) * ntk * 2048 : row0 * g.lda * 2);
    bp = B + (TILED ? (int64_t)tn * (BN / 32) * 2048 : (int64_t)tn * BN * 2);
    if constexpr (SPLITK) {      // the slice's first step
      ap += (int64_t)slice * a_kstep1;
      bp += (int64_t)slice * b_kstep1;
    }
    if (RAGGED || offsets) {
      // per-thread offsets of the tile's copies from ap / bp, one per A slab (RAGGED: rows and column chunks
      // clamped into the matrix)
      const int last_row = RAGGED ? Mf - 1 - (int)row0 : BM;  // >= 0
      vo.last_row = last_row;
      const int last_chunk = RAGGED ? (Nf - tn * BN) / 8 - 1 : 32;   // >= 0: the fetchable N is a multiple of 8
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const int r = min(i * 64 + a_row, last_row);
        vo.a[i] = TILED ? (uint32_t)((((int64_t)(r >> 5) * ntk << 10) + (r & 31) * 32 + a_chunk * 8) * 2)
                        : (uint32_t)(((int64_t)r * g.lda + a_chunk * 8) * 2);
      }
      const int cc = min(b_chunk, last_chunk);
      vo.b = TILED ? (uint32_t)((((cc >> 2) << 10) + b_kk * 32 + (cc & 3) * 8) * 2)
                   : (uint32_t)(((int64_t)b_kk * g.ldb + cc * 8) * 2);
    }
  };
  // copy number i (0..MB-1: A slabs, MB..MB+3: B slabs) of step kk into `stage`; kk may run past
  // nk into the next tile
  // `inner`: the caller knows that step kk belongs to this tile and carries data, so the choices between this
  // tile and the next and (RAGGED) between data and the page of zeros are not made at run time, and a copy's
  // source is one scalar address per operand and step plus the thread's offset for that slab
  // (f, n: the MFMA that the copy is issued behind, n < 0: none)
  auto dma_single = [&](int kk, uint8_t *stage, int i, auto inner_, Frags &f, int n) {
    constexpr bool inner = decltype(inner_)::value;
    const bool over = !inner && kk >= nk;
    const int k = over ? kk - nk : kk;
    auto dma_one = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst_slab) {
      if (n >= 0) mm_copy(f, n, src_uniform, voff, dst_slab);
      else dma_plain(src_uniform, voff, dst_slab);
    };
    if constexpr (inner) {
      if (i < MB)
        dma_one(a_cur + (int64_t)k * a_kstep, vo_cur.a[i], stage + i * 4096);
      else if constexpr (APAIR && !RAGGED)
        dma_one(b_cur + (int64_t)k * b_kstep, b_vs[i - MB], stage + B_OFF + (i - MB) * 4096);
      else
        dma_one(b_cur + (int64_t)k * b_kstep + b_slab_off(i - MB), vo_cur.b, stage + B_OFF + (i - MB) * 4096);
    } else if constexpr (RAGGED) {
      const bool zero = k >= nk_real;                         // a padding step: both operands are zeros
      // row-major operands, last data step of a K that is not a whole number of steps: the 16-byte chunks of A past
      // K belong to the next row (past the buffer, for the last row) and the rows of B past K do not exist.  They
      // are fetched from the step's first chunk / first eight rows instead, which exist (K is a multiple of 8), and
      // cleared once they have landed (clear_past_k).  A wavefront's rows of a B slab all lie in one group of eight
      // (b_row0(i)/8 + wave/2), so the choice is the wavefront's and the copy's base address stays scalar.
      // Tile-major buffers are padded to whole tiles and need no redirection.
      const bool tail = !TILED && k_tail != 0 && k == nk_real - 1;
      const Voffs &vo = over ? vo_nxt : vo_cur;
      if (i < MB) {
        const uint8_t *ap = zero ? zero_page : (over ? a_nxt : a_cur) + (int64_t)k * a_kstep;
        const uint32_t av = (tail && a_chunk * 8 >= k_tail) ? vo.a[i] - (uint32_t)a_chunk * 16 : vo.a[i];
        dma_one(ap, zero ? z_voff : av, stage + i * 4096);
      } else {
        const int ib = i - MB;
        const bool redirect = tail && ((b_row0(ib) >> 3) + (wave >> 1)) * 8 >= k_tail;   // to row & 7
        const uint8_t *bp = zero ? zero_page
                                 : (over ? b_nxt : b_cur) + (int64_t)k * b_kstep + (redirect ? (ib & 1) * b_rows4 : b_slab_off(ib));
        const uint32_t bv = redirect ? vo.b - (uint32_t)((wave >> 1) * 2 * b_rows4) : vo.b;
        dma_one(bp, zero ? z_voff : bv, stage + B_OFF + (i - MB) * 4096);
      }
    } else if (i < MB) {
      const uint8_t *ap = (over ? a_nxt : a_cur) + (int64_t)k * a_kstep;
      dma_one(ap + i * a_slab, a_voff, stage + i * 4096);
    } else {
      const uint8_t *bp = (over ? b_nxt : b_cur) + (int64_t)k * b_kstep;
      if constexpr (APAIR) dma_one(bp, b_vs[i - MB], stage + B_OFF + (i - MB) * 4096);
      else dma_one(bp + b_slab_off(i - MB), b_voff, stage + B_OFF + (i - MB) * 4096);
    }
  };

  // APAIR: copy number i (0..7) of the pair of steps (kk, kk+1), kk even, into pair buffer P
  auto dma_pair = [&](int kk, int P, int i, auto inner_, Frags &f, int n) {
    constexpr bool inner = decltype(inner_)::value;
    const bool over = !inner && kk >= nk;
    const int k = over ? kk - nk : kk;
    auto dma_one = [&](const uint8_t *src_uniform, uint32_t voff, uint8_t *dst_slab) {
      if (n >= 0) mm_copy(f, n, src_uniform, voff, dst_slab);
      else dma_plain(src_uniform, voff, dst_slab);
    };
    uint8_t *dst = ring.s[2 * P + (i >> 2)] + (i & 3) * 4096;
    if constexpr (RAGGED) {
      // rows past M are fetched from the last row; a pair that ends past K (K is a multiple of 8) fetches the
      // chunks past K from the pair's first chunk, which exists, and clear_pair zeroes them once they have landed;
      // a pair that starts at or past K comes from the page of zeros
      const int valid = inner ? 64 : min(max(gK - 32 * k, 0), 64);
      const int last_row = (over ? vo_nxt : vo_cur).last_row;
      if constexpr (decltype(inner_)::value == 2) {
        // a whole pair of a tile that lies inside the matrix (all but the last row of tiles; the caller knows):
        // nothing depends on the lane but the constant offset.  It matters: between two 16-cycle MFMAs a lone
        // wavefront has room for three other instructions, and the half dozen VALU operations of the path below,
        // once per copy, cost the kernel 8 % (a branch per copy instead cost more).
        dma_one(a_cur + (int64_t)(k >> 1) * 128 + i * a_slab32, a_voff_pair, dst);
      } else {
        // (worked out here, from one register each: left free, the compiler keeps the eight slabs' rows in
        // registers from the start of the kernel, spills them, and a reload in a step drains the copies in flight)
        int r8 = pair_r8, c = pair_c;
        asm volatile("" : "+v"(r8), "+v"(c));
        const int row = min(i * 32 + r8, last_row);
        if (!inner && 8 * c + 8 > valid) c = 0;
        const uint32_t voff = (uint32_t)row * (uint32_t)(g.lda * 2) + (uint32_t)c * 16;
        const uint8_t *ap = valid == 0 ? zero_page : (over ? a_nxt : a_cur) + (int64_t)(k >> 1) * 128;
        dma_one(ap, valid == 0 ? z_voff : voff, dst);
      }
    } else {
      const uint8_t *ap = (over ? a_nxt : a_cur) + (int64_t)(k >> 1) * 128;
      dma_one(ap, a_vp[i], dst);
    }
  };
  // RAGGED APAIR: this thread's sixteen bytes of each slab of pair buffer P, when they hold k at or past `valid`
  auto clear_pair = [&](int P, int valid) {
    typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
    if (8 * pair_c + 8 > valid) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *(lds_u32x4 *)(lds_void *)(ring.s[2 * P + (i >> 2)] + (i & 3) * 4096 + lds_wave + lane * 16) = (u32x4){0, 0, 0, 0};
    }
  };

  // One step (K += 32) on ring stage I: the NM MFMAs on `c` (read from stage I during the previous step), the next
  // stage's fragments into `p`, and the refill of stage I itself with step k+R.
  //   The first MFMA goes out before the barrier, so that the matrix pipe has work while the wavefronts meet.
  //   The fragment reads ride one per MFMA behind the barrier; the MB + 4 copies that refill the stage follow
  //   them, one per five MFMAs (80 cycles): a wavefront that issues copies back to back stalls behind the memory
  //   pipeline's input queue, and its MFMAs stall with it.  (Placement matters little here: two MFMAs or four
  //   before the barrier, reads on every second MFMA, copies every third to seventh MFMA from the 7th to the 30th
  //   on all measured within 1 % of each other, 1477-1497 TFLOP/s on 8192^3; two reads per MFMA cost 1.5 %.)
  auto step = [&](auto I_, int k, Frags &c, Frags &p, auto inner_) {
    constexpr int I = decltype(I_)::value;
    uint8_t *cur = ring.s[I], *nxt = ring.s[(I + 1) % R];
    mm(c, 0);
    FENCE();
    if constexpr (RAGGED && !decltype(inner_)::value) {
      if constexpr (APAIR && (I & 1)) {
        // the pair about to open (its first step is the next one) ends past K: clear what lies past
        const int valid = min(max(gK - 32 * (k + 1 == nk ? 0 : k + 1), 0), 64);
        if (valid > 0 && valid < 64) {
          asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
          clear_pair(((I + 1) % R) >> 1, valid);
        }
      }
      if (k_tail && (k + 1 == nk ? 0 : k + 1) == nk_real - 1) {   // the stage about to open holds a tile's last data step
        if constexpr (APAIR && (I & 1))
          asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if constexpr (MB == 4)
          asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if constexpr (MB == 2)
          asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        else
          asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
        clear_past_k(nxt);
      }
    }
    // Every wave's reads of stage I have returned (they fed `c`), and this wave's share of the copy into stage
    // I+1 has landed (the copies of the two younger steps may still be in flight); after the barrier that holds for
    // all waves: I+1 may be read, I may be overwritten.
    // (the copies of the two younger steps, 2 * (MB + 4) of them, may still be in flight)
    // APAIR: an odd step issues the 8 copies of the A pair whose buffer its barrier has freed (steps k+3, k+4) and
    // then its 4 B copies, an even step only its 4 B copies; a barrier needs B of the next step and the A pair that
    // step lies in, which on an even step leaves 4 + 8 + 4 younger copies in flight and on an odd one 4 + 4.
    if constexpr (APAIR && (I & 1))
      asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else if constexpr (MB == 4)
      asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else if constexpr (MB == 2)
      asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    FENCE();
#pragma unroll
    for (int n = 1; n < NM; ++n) {
      bool with_copy = false;
      if constexpr (MB == 1) {
        // quarter tiles: 18 reads and 5 copies beside 15 MFMAs: two reads per MFMA, a copy with every third
        if (2 * (n - 1) < NR) rd(p, nxt, (I + 1) % R, 2 * (n - 1));
        if (2 * (n - 1) + 1 < NR) rd(p, nxt, (I + 1) % R, 2 * (n - 1) + 1);
        if (n % 3 == 0) {
          dma_single(k + R, cur, n / 3 - 1, inner_, c, n);
          with_copy = true;
        }
      } else {
        if (n <= NR) rd(p, nxt, (I + 1) % R, n - 1);
        if constexpr (APAIR) {
          if constexpr (I & 1) {
            if (n >= 26 && n <= 59 && (n - 26) % 3 == 0) {
              const int c12 = (n - 26) / 3;
              if (c12 < 8) dma_pair(k + 3, (I - 1) >> 1, c12, inner_, c, n);
              else dma_single(k + R, cur, MB + c12 - 8, inner_, c, n);
              with_copy = true;
            }
          } else {
            if (n >= 30 && n <= 54 && (n - 30) % 8 == 0) {
              dma_single(k + R, cur, MB + (n - 30) / 8, inner_, c, n);
              with_copy = true;
            }
          }
        } else if constexpr (MB == 4) {
          if (n >= 25 && n <= 60 && n % 5 == 0) {
            dma_single(k + R, cur, n / 5 - 5, inner_, c, n);
            with_copy = true;
          }
        } else {
          if (n % 5 == 0 && n <= 30) {
            dma_single(k + R, cur, n / 5 - 1, inner_, c, n);
            with_copy = true;
          }
        }
      }
      if (!with_copy) mm(c, n);   // (a copy took MFMA n with it)
      FENCE();
    }
  };

  // ---- fill the ring: steps 0..R-1 of the first tile ----
  int t = blockIdx.x;
  if (t >= total) return;
  tile_bases(t, a_cur, b_cur, vo_cur, true);
  // no copy of the fill looks at the next tile.  RAGGED: where it lies is worked out before the last turns of each
  // tile, so that its offsets are not held through the turns before; whole tiles: one tile ahead, at the end of a tile
  a_nxt = a_cur;
  b_nxt = b_cur;
  vo_nxt = vo_cur;
  if constexpr (!RAGGED) tile_bases(t + (int)gridDim.x < total ? t + (int)gridDim.x : t, a_nxt, b_nxt, vo_nxt);
  if constexpr (APAIR) {
    // in the order the steps of a turn issue them: pair (0,1), B 0, B 1, B 2, pair (2,3), B 3
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_pair(0, 0, i, std::false_type{}, f0, -1);
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) dma_single(s, ring.s[s], MB + i, std::false_type{}, f0, -1);
#pragma unroll
    for (int i = 0; i < 8; ++i) dma_pair(2, 1, i, std::false_type{}, f0, -1);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma_single(3, ring.s[3], MB + i, std::false_type{}, f0, -1);
  } else {
#pragma unroll
    for (int s = 0; s < R; ++s)
#pragma unroll
      for (int i = 0; i < MB + 4; ++i) dma_single(s, ring.s[s], i, std::false_type{}, f0, -1);
  }
  static_assert(DMA_PER_STEP == 8 && R == 4, "the hand-written vmcnt waits assume MB + 4 copies per step and 4 stages");
  if (RAGGED && k_tail && nk_real == 1) {   // a single data step: it is the one that ends past K
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    clear_past_k(ring.s[0]);
  }
  if constexpr (RAGGED && APAIR) {
    if (gK < 128 && (gK & 63)) {          // one of the first tile's two pairs ends past K
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (gK < 64) clear_pair(0, gK);
      else clear_pair(1, gK - 64);
    }
  }
  // step 0 has landed when only the (R - 1) * (MB + 4) younger copies are left in flight
  if constexpr (APAIR)
    asm volatile("s_waitcnt vmcnt(20) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // pair (0,1) and B 0 have landed
  else if constexpr (MB == 4)
    asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  else if constexpr (MB == 2)
    asm volatile("s_waitcnt vmcnt(18) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  else
    asm volatile("s_waitcnt vmcnt(15) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
  for (int r = 0; r < NR; ++r) rd(f0, ring.s[0], 0, r);

  for (; t < total; t += gridDim.x) {
    int tm, tn, part;
    item_tile<MB>(items, t, tiles_mv, tiles_n, tm, tn, part);
    int slice = 0;
    if constexpr (SPLITK) {
      slice = tm / tiles_m;
      tm -= slice * tiles_m;
    }
    const int64_t m0 = (int64_t)tm * BM + part * (64 * MB), n0 = (int64_t)tn * BN;
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = (f32x4){0, 0, 0, 0};

    int k = 0;
    // turns of the ring whose copies (up to step k + 2R - 1) all carry this tile's data
    // (row-major operands whose last step ends past K: that step's copies need the redirection above, so it stays
    // out of these turns)
    const int nk_inner = nk_real - ((!TILED && k_tail) ? 1 : 0);
    if (RAGGED && APAIR && __builtin_amdgcn_readfirstlane(vo_cur.last_row) >= BM - 1) {
      // (a tile whose 256 rows all exist: the copies of A need no clamping)
      for (; k + 2 * R <= nk_inner; k += R) {
        step(std::integral_constant<int, 0>{}, k, f0, f1, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 1>{}, k + 1, f1, f0, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 2>{}, k + 2, f0, f1, std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{}, k + 3, f1, f0, std::integral_constant<int, 2>{});
      }
    }
    for (; k + 2 * R <= nk_inner; k += R) {
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
    // the ring already holds the next tile's first steps; move the tile window on
    a_cur = a_nxt;
    b_cur = b_nxt;
    if constexpr (RAGGED) {
      vo_cur = vo_nxt;
    } else {
      // whole tiles: only the two addresses change from tile to tile; the tile after the next
      const int t2 = t + 2 * (int)gridDim.x;
      tile_bases(t2 < total ? t2 : (t + (int)gridDim.x < total ? t + (int)gridDim.x : t), a_nxt, b_nxt, vo_nxt);
    }

    // ---- epilogue: acc[i][j] register e of lane l is C[m][n] with
    //      m = i*16 + l%16,  n = j*16 + (l/16)*4 + e
    // The MFMAs are assembly to the compiler, which therefore does not know to wait for the last of them before it
    // reads an accumulator: sixteen idle cycles cover the four passes of a 16x16x32.
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
    const int64_t m = m0 + wm * (32 * MB) + i16;
    if constexpr (SPLITK) {
      // the slice's sums as they are: a lane's four columns of a row are sixteen contiguous bytes of the slab
      float *slab = (float *)g.c + (int64_t)slice * g.M * g.ldws;
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        const int64_t mi = m + i * 16;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int64_t n = n0 + wn * 128 + j * 16 + G4 * 4;
          if (mi < g.M && n < g.N) *(f32x4 *)(slab + mi * g.ldws + n) = acc[i][j];   // (ldws is a multiple of 8)
        }
      }
      continue;
    }
    // A row bias depends on n only: its 32 values for this lane are fetched once, all loads in flight
    // together, instead of one dependent load per use in the loop below.
    constexpr bool ROW_BIAS = EPI == EPI_BIAS_ROW || EPI == EPI_BIAS_ROW_GELU;
    f32x4 brow[ROW_BIAS ? 8 : 1];
    if constexpr (ROW_BIAS) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        brow[j] = *(const f32x4 *)((const float *)g.bias + (RAGGED ? min(n0 + wn * 128 + j * 16 + G4 * 4, (int64_t)g.N - 4)
                                                                   : n0 + wn * 128 + j * 16 + G4 * 4));
    }
    // the four columns n .. n+3 of row mi that this lane holds for (i, j), after scale, epilogue and rounding
    auto packed = [&](int i, int j, int64_t mi, int64_t n) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x = acc[i][j][e] * g.scale;
        if constexpr (EPI == EPI_BIAS_ROW_GELU)
          v[e] = gelu_erf(x + brow[j][e]);
        else if constexpr (EPI == EPI_BIAS_ROW)
          v[e] = x + brow[j][e];
        else
          v[e] = apply_epilogue_ct<OUT_DT, EPI>(g, x, mi, n + e);
      }
      if constexpr (OUT_DT == DT_BF16)
        return (u32x2){pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
      else
        return (u32x2){(uint32_t)f32_to_f16(v[0]) | ((uint32_t)f32_to_f16(v[1]) << 16),
                       (uint32_t)f32_to_f16(v[2]) | ((uint32_t)f32_to_f16(v[3]) << 16)};
    };
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int64_t mi = m + i * 16;
#pragma unroll
      for (int jp = 0; jp < 4; ++jp) {
        if constexpr (!(RAGGED && TILED)) {
          // Of the 32 columns of the block pair (2jp, 2jp+1), lane group G4 = l/16 holds 4*G4 .. +3 and 16 + 4*G4 .. +3
          // of one row.  Swapping the odd groups' first piece with the even groups' second (v_permlane16_swap: odd
          // rows of sixteen lanes of its first operand <-> even rows of its second) leaves groups 0, 1, 2, 3 with
          // columns 0-7, 16-23, 8-15, 24-31: each lane stores 16 contiguous bytes, four lanes a row's 64 (8 columns
          // never straddle a 32x32 tile of a tile-major C, nor the edge of a clipped one, whose N is a multiple of
          // 8).  Every lane takes part in the swap; clipped lanes only skip the store, and read a full bias, if
          // there is one, at a clamped position.
          const int64_t nb = n0 + wn * 128 + jp * 32;
          const int64_t mb = RAGGED ? min(mi, (int64_t)g.M - 1) : mi;
          const int64_t nl = nb + G4 * 4, nh = nb + 16 + G4 * 4;
          u32x2 p0 = packed(i, 2 * jp, mb, RAGGED ? min(nl, (int64_t)g.N - 4) : nl);
          u32x2 p1 = packed(i, 2 * jp + 1, mb, RAGGED ? min(nh, (int64_t)g.N - 4) : nh);
          asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(p0.x), "+v"(p1.x));
          asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(p0.y), "+v"(p1.y));
          const int64_t n = nb + (G4 & 1) * 16 + (G4 >> 1) * 8;
          if (RAGGED && (mi >= g.M || n >= g.N)) continue;
          const int64_t coff = TILED ? (((mi >> 5) * ntn + (n >> 5)) << 10) + (mi & 31) * 32 + (n & 31) : mi * g.ldc + n;
          if constexpr (STREAM)
            __builtin_nontemporal_store((u32x4){p0.x, p0.y, p1.x, p1.y}, (u32x4 *)((uint16_t *)g.c + coff));
          else
            *(u32x4 *)((uint16_t *)g.c + coff) = (u32x4){p0.x, p0.y, p1.x, p1.y};
        } else {
#pragma unroll
          for (int j = 2 * jp; j < 2 * jp + 2; ++j) {
            const int64_t n = n0 + wn * 128 + j * 16 + G4 * 4;
            if (mi >= g.M || n >= g.N) continue;
            const u32x2 pk = packed(i, j, mi, n);
            const int64_t coff = (((mi >> 5) * ntn + (n >> 5)) << 10) + (mi & 31) * 32 + (n & 31);
            if (n + 3 >= g.N) {               // N is anything here: the last group goes by element
              for (int e = 0; e < 4 && n + e < g.N; ++e)
                ((uint16_t *)g.c)[coff + e] = (uint16_t)(e & 1 ? pk[e >> 1] >> 16 : pk[e >> 1] & 0xffffu);
              continue;
            }
            *(u32x2 *)((uint16_t *)g.c + coff) = pk;
          }
        }
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the trailing refetches must land before the LDS is released
  if (MB == 4 && g.probe && blockIdx.x == 0 && tid == 0) {
    g.probe[0] = (unsigned long long)(clock64() - probe_c0);
    g.probe[1] = (unsigned long long)(wall_clock64() - probe_w0);
  }
}

} // namespace fast

extern "C" {

#define GEMM_TILE(name, IN, OUT, EPI, STREAM)                                                      \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast::STAGE];                            \
    fast::Ring ring = {{lds0, lds1, lds2, lds3}};                                                   \
    fast::body<IN, OUT, EPI, false, false, 4, true, true, STREAM>(g, ring);                         \
    fast::body<IN, OUT, EPI, false, false, 2, true, true, STREAM>(g, ring);                         \
    fast::body<IN, OUT, EPI, false, false, 1, true, true, STREAM>(g, ring);                         \
  }
#define GEMM_TILE_ALL_EPI(prefix, IN, OUT)                    \
  GEMM_TILE(prefix##_epi0, IN, OUT, EPI_NONE, false)           \
  GEMM_TILE(prefix##_epi1, IN, OUT, EPI_BIAS_FULL, false)      \
  GEMM_TILE(prefix##_epi2, IN, OUT, EPI_BIAS_ROW_GELU, false)  \
  GEMM_TILE(prefix##_epi3, IN, OUT, EPI_LEAKY_RELU, false)     \
  GEMM_TILE(prefix##_epi4, IN, OUT, EPI_BIAS_ROW, false)       \
  GEMM_TILE(prefix##_epi0_stream, IN, OUT, EPI_NONE, true)

GEMM_TILE_ALL_EPI(gemm_tile_bf16, DT_BF16, DT_BF16)
GEMM_TILE_ALL_EPI(gemm_tile_f16, DT_F16, DT_F16)

// the same kernels for M any, N % 8 == 0, K % 8 == 0 (a last 32-deep step that ends past K is cleared in LDS)
#define GEMM_TILE_RAGGED(name, IN, OUT, EPI, STREAM)                                               \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast::STAGE];                            \
    fast::Ring ring = {{lds0, lds1, lds2, lds3}};                                                   \
    fast::body<IN, OUT, EPI, false, true, 4, true, true, STREAM>(g, ring);                          \
    fast::body<IN, OUT, EPI, false, true, 2, true, true, STREAM>(g, ring);                          \
    fast::body<IN, OUT, EPI, false, true, 1, true, true, STREAM>(g, ring);                          \
  }
#define GEMM_TILE_RAGGED_ALL_EPI(prefix, IN, OUT)                    \
  GEMM_TILE_RAGGED(prefix##_epi0, IN, OUT, EPI_NONE, false)           \
  GEMM_TILE_RAGGED(prefix##_epi1, IN, OUT, EPI_BIAS_FULL, false)      \
  GEMM_TILE_RAGGED(prefix##_epi2, IN, OUT, EPI_BIAS_ROW_GELU, false)  \
  GEMM_TILE_RAGGED(prefix##_epi3, IN, OUT, EPI_LEAKY_RELU, false)     \
  GEMM_TILE_RAGGED(prefix##_epi4, IN, OUT, EPI_BIAS_ROW, false)       \
  GEMM_TILE_RAGGED(prefix##_epi0_stream, IN, OUT, EPI_NONE, true)
GEMM_TILE_RAGGED_ALL_EPI(gemm_ragged_bf16, DT_BF16, DT_BF16)
GEMM_TILE_RAGGED_ALL_EPI(gemm_ragged_f16, DT_F16, DT_F16)

// Slices of K as work items (see SPLITK in body), fp32 sums into the workspace.  Such a launch has at most one round
// of quarter tiles, so the kernel is the quarter-tile body alone: 16 + 48 accumulator and fragment registers instead
// of 256 + 128 and a ring of 4 x 20 KiB, i.e. two workgroups per CU.  That is what these launches want: the small
// ones among them stream B once from memory, and twice the copies in flight per CU is 30 % more bandwidth there.
#define GEMM_SPLITK(name, IN)                                                                      \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds[4][20480];                                \
    fast::Ring ring = {{lds[0], lds[1], lds[2], lds[3]}};                                           \
    fast::body<IN, IN, EPI_NONE, false, true, 1, true, true, false, true, true>(g, ring);           \
  }
GEMM_SPLITK(gemm_splitk_bf16, DT_BF16)
GEMM_SPLITK(gemm_splitk_f16, DT_F16)
// the same on the tile-major buffers of matmul_kernel (the workspace is row-major all the same)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_splitk_tiled_f16(GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[4][20480];
  fast::Ring ring = {{lds[0], lds[1], lds[2], lds[3]}};
  fast::body<DT_F16, DT_F16, EPI_NONE, true, true, 1, true, true, false, true, true>(g, ring);
}

// matmul_kernel on tile-major fp16 buffers, plain and with leaky_relu
#define GEMM_TILED(name, EPI)                                                                      \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast::STAGE];                            \
    fast::Ring ring = {{lds0, lds1, lds2, lds3}};                                                   \
    fast::body<DT_F16, DT_F16, EPI, true, false, 4, true>(g, ring);                                 \
    fast::body<DT_F16, DT_F16, EPI, true, false, 2, true>(g, ring);                                 \
  }
GEMM_TILED(gemm_tiled_f16_epi0, EPI_NONE)
GEMM_TILED(gemm_tiled_f16_epi3, EPI_LEAKY_RELU)

// the same for any M, N, K (buffers padded to whole 32x32 tiles)
#define GEMM_TILED_RAGGED(name, EPI)                                                               \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds2[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds3[fast::STAGE];                            \
    fast::Ring ring = {{lds0, lds1, lds2, lds3}};                                                   \
    fast::body<DT_F16, DT_F16, EPI, true, true, 4, true>(g, ring);                                  \
    fast::body<DT_F16, DT_F16, EPI, true, true, 2, true>(g, ring);                                  \
  }
GEMM_TILED_RAGGED(gemm_tiledragged_f16_epi0, EPI_NONE)
GEMM_TILED_RAGGED(gemm_tiledragged_f16_epi3, EPI_LEAKY_RELU)

// Diagnostic, launched by bench.py only: what the part sustains for this kernel's MFMAs alone.  One wavefront per SIMD
// holds eight A and eight B fragments taken from `src` (so that the operand statistics are the benchmark's: MFMAs on
// zeros draw far less power and run at the full clock) and issues the 64 MFMAs of a K step, in the kernel's order and
// on AGPR accumulators, `iters` times: no LDS, no copies, no barrier.  The kernels above are bounded by power, so this
// figure, at the clock the box grants under it, is the ceiling they can be laid against (2^20 flops per wavefront and
// iteration; 64 x 16 x 256 fragments of 16 bytes are read from `src`).
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_mfma_ceiling_bf16(int iters, const bf16x8 *src,
                                                                                                      float *sink,
                                                                                                      unsigned long long *probe) {
  // probe: workgroup 0 leaves {core-clock cycles, 100 MHz ticks} of its run there (the clock granted under this loop)
  const long long probe_c0 = clock64(), probe_w0 = wall_clock64();
  bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = src[((blockIdx.x & 63) * 16 + i) * 256 + threadIdx.x];
    b[i] = src[((blockIdx.x & 63) * 16 + 8 + i) * 256 + threadIdx.x];
  }
  f32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 64; ++n) {
      const int i = n >> 3, j = (i & 1) ? 7 - (n & 7) : (n & 7);   // odd row blocks walk backwards, as in the K step
      fast::MFMA<DT_BF16>::run(b[j], a[i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) t += acc[i][j][e];
  if (t == 12345.678f) sink[0] = t;   // (keeps the accumulators alive; never true in practice)
  if (probe && blockIdx.x == 0 && threadIdx.x == 0) {
    probe[0] = (unsigned long long)(clock64() - probe_c0);
    probe[1] = (unsigned long long)(wall_clock64() - probe_w0);
  }
}

} // extern "C"
