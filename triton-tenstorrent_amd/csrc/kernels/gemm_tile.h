// gemm_tile_*: the fast tile-matmul path for gfx950.
//
// Requirements (checked by the host): M and N multiples of 256, K a multiple of
// 64, 16-byte aligned bases and leading strides, and a logical grid that covers
// every tile -- then which physical tile computes which part of C does not show
// in the result (up to fp32 summation order).
//
// One workgroup (4 wavefronts, 2x2) computes a 256x256 macro tile, walking K in
// steps of 64 through two LDS stages (A 256x64 + B 64x256 = 64 KiB per stage).
// Each wavefront owns 128x128: 4x4 v_mfma_f32_32x32x16 accumulators (256
// registers), so one wavefront per SIMD.  The grid is persistent, one workgroup
// per CU, striding over the macro tiles in an XCD-aware order.
//
// Data path: global -> LDS directly (global_load_lds_dwordx4, no register
// staging), issued one whole K-step ahead; LDS -> registers one 16-deep
// sub-step ahead of the MFMAs that consume them, so a single wavefront keeps
// its matrix pipe busy without help from a second one.
//
// LDS layout (16-byte chunks, XOR-swizzled so that the row-wise A reads and the
// transposing B reads are both bank-conflict free):
//   A: row m = 128 B = 8 chunks;  logical chunk c sits at c ^ ((m>>1)&7)
//   B: row k = 512 B = 32 chunks; logical chunk c sits at c ^ ((k&3)<<2)
// A direct-to-LDS load writes lane l's 16 bytes at (wave-uniform base) + 16*l,
// so thread t owns byte 16*t of every 4 KiB slab and the swizzle is applied to
// the global address it fetches.
//
// The product is formed transposed, acc = mfma(Bfrag, Afrag): a result lane then
// holds 4 consecutive n of one m, so epilogue stores and bias loads are 8 bytes
// wide.  B fragments need k along the lane's registers while memory has n
// contiguous: ds_read_b64_tr_b16 transposes a 4x16 block of 16-bit values
// across each group of 16 lanes on the way out of LDS.
#pragma once
#include "gemm_common.h"

namespace fast {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int A_BYTES = BM * BK * 2;        // 32 KiB
constexpr int B_BYTES = BK * BN * 2;        // 32 KiB
constexpr int STAGE = A_BYTES + B_BYTES;    // 64 KiB

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void global_void;

template <int IN_DT> struct MFMA;
template <> struct MFMA<DT_BF16> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x16 run(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct MFMA<DT_F16> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x16 run(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
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

// scheduling hints: one group of `n` instructions of a class, in program order
#define SCHED_MFMA(n) __builtin_amdgcn_sched_group_barrier(0x008, n, 0)
#define SCHED_DSRD(n) __builtin_amdgcn_sched_group_barrier(0x100, n, 0)
#define SCHED_VMEM(n) __builtin_amdgcn_sched_group_barrier(0x010, n, 0)

template <int IN_DT, int OUT_DT, int EPI>
__device__ __forceinline__ void body(const GemmArgs &g, uint8_t *lds0, uint8_t *lds1) {
  using X = MFMA<IN_DT>;
  using vec = typename X::vec;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = g.M / BM, tiles_n = g.N / BN;
  const int total = tiles_m * tiles_n;
  const int nk = g.K / BK;

  // ---- global -> LDS: thread t writes byte 16*t of each 4 KiB slab ----
  // A slab i (32 rows): row = i*32 + (t>>3), chunk position t&7 holds logical chunk (t&7)^((row>>1)&7)
  const int a_row = tid >> 3;
  const int a_chunk = (tid & 7) ^ ((a_row >> 1) & 7);
  // B slab i (8 k-rows): k = i*8 + (t>>5), chunk position t&31 holds logical chunk (t&31)^((k&3)<<2)
  const int b_k = tid >> 5;
  const int b_chunk = (tid & 31) ^ ((b_k & 3) << 2);
  const uint32_t a_voff = (uint32_t)(((int64_t)a_row * g.lda + a_chunk * 8) * 2); // bytes, per thread
  const uint32_t b_voff = (uint32_t)(((int64_t)b_k * g.ldb + b_chunk * 8) * 2);
  const int64_t a_slab = 32 * g.lda * 2, b_slab = 8 * g.ldb * 2;                   // bytes, uniform
  const int lds_wave = wave * 1024;

  // ---- LDS -> fragments ----
  const int l32 = lane & 31, hi = lane >> 5;
  const int a_base = (wm * 128 + l32) * 128;
  const int a_x = (lane >> 1) & 7;
  int a_pos[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) a_pos[s] = a_base + (((s * 2 + hi) ^ a_x) << 4);
  const int G4 = lane >> 4, i16 = lane & 15, q = i16 >> 2;
  const int b_base = A_BYTES + (((G4 >> 1) * 8 + q) * 512) + ((wn * 16 + (G4 & 1) * 2 + ((i16 >> 1) & 1)) << 4) +
                     ((i16 & 1) << 3);
  int b_pos[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) b_pos[j] = b_base + ((j ^ q) << 6);

  const uint8_t *A = (const uint8_t *)g.a;
  const uint8_t *B = (const uint8_t *)g.b;

  for (int t = blockIdx.x; t < total; t += gridDim.x) {
    int tm, tn;
    tile_of(t, tiles_m, tiles_n, tm, tn);
    const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
    const uint8_t *a_tile = A + m0 * g.lda * 2; // + kt*128 per K-step
    const uint8_t *b_tile = B + n0 * 2;         // + kt*64*ldb*2 per K-step
    const int64_t b_kstep = (int64_t)BK * g.ldb * 2;

    // direct-to-LDS copy of K-step kt (clamped: past the end it refetches the last one
    // into a stage nobody reads again, which keeps the loop body branch-free)
    auto dma = [&](int kt, uint8_t *stage) {
      kt = min(kt, nk - 1);
      const uint8_t *ap = a_tile + (int64_t)kt * (BK * 2);
      const uint8_t *bp = b_tile + (int64_t)kt * b_kstep;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_global_load_lds((global_void *)(ap + i * a_slab + a_voff),
                                         (lds_void *)(stage + i * 4096 + lds_wave), 16, 0, 0);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_global_load_lds((global_void *)(bp + i * b_slab + b_voff),
                                         (lds_void *)(stage + A_BYTES + i * 4096 + lds_wave), 16, 0, 0);
    };
    auto read_a = [&](const uint8_t *stage, int s, vec (&f)[4]) {
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = *(const vec *)(stage + a_pos[s] + i * 4096);
    };
    auto read_b = [&](const uint8_t *stage, int s, vec (&f)[4]) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t *p = stage + b_pos[j] + s * 8192;
        union { s16x4 h[2]; vec v; } u;
        u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p));
        u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 2048));
        f[j] = u.v;
      }
    };

    f32x16 acc[4][4]; // [m-tile][n-tile]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = (f32x16){0};
    auto mma = [&](vec (&fa)[4], vec (&fb)[4], int i0, int i1) {
#pragma unroll
      for (int i = i0; i < i1; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = X::run(fb[j], fa[i], acc[i][j]);
    };

    vec fa0[4], fb0[4], fa1[4], fb1[4];

    // One K-step on stage `cur`; `nxt` is being filled with K-step kt+1 meanwhile.
    // Entry: fa0/fb0 hold sub-step 0 of `cur`.  Exit: fa0/fb0 hold sub-step 0 of `nxt`.
    auto kstep = [&](int kt, uint8_t *cur, uint8_t *nxt) {
      read_a(cur, 1, fa1); read_b(cur, 1, fb1);
      mma(fa0, fb0, 0, 4);
      for (int r = 0; r < 12; ++r) { SCHED_MFMA(1); SCHED_DSRD(1); }
      SCHED_MFMA(4);

      read_a(cur, 2, fa0); read_b(cur, 2, fb0);
      mma(fa1, fb1, 0, 4);
      for (int r = 0; r < 12; ++r) { SCHED_MFMA(1); SCHED_DSRD(1); }
      SCHED_MFMA(4);

      read_a(cur, 3, fa1); read_b(cur, 3, fb1);
      mma(fa0, fb0, 0, 3);
      for (int r = 0; r < 12; ++r) { SCHED_MFMA(1); SCHED_DSRD(1); }
      // every wave has its last fragments of `cur` and the copy into `nxt` has landed:
      // after the barrier `nxt` may be read and `cur` may be overwritten
      __syncthreads();
      dma(kt + 2, cur);
      mma(fa0, fb0, 3, 4);

      read_a(nxt, 0, fa0); read_b(nxt, 0, fb0);
      mma(fa1, fb1, 0, 4);
      // the 16 copies go out first (they have the longest way to go), two per MFMA
      for (int r = 0; r < 4; ++r) { SCHED_MFMA(1); SCHED_VMEM(2); }
      for (int r = 0; r < 4; ++r) { SCHED_MFMA(1); SCHED_VMEM(2); SCHED_DSRD(1); }
      for (int r = 0; r < 8; ++r) { SCHED_MFMA(1); SCHED_DSRD(1); }
      SCHED_MFMA(4);
    };

    __syncthreads(); // the previous tile's fragment reads are done before the stages are refilled
    dma(0, lds0);
    dma(1, lds1);
    __builtin_amdgcn_s_waitcnt(0x4F70); // vmcnt(16): K-step 0 has landed, K-step 1 still in flight
    __builtin_amdgcn_s_barrier();
    read_a(lds0, 0, fa0); read_b(lds0, 0, fb0);

    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
      kstep(kt, lds0, lds1);
      kstep(kt + 1, lds1, lds0);
    }
    if (kt < nk) kstep(kt, lds0, lds1);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): drain the clamped refetches before the stages are reused

    // ---- epilogue: acc[i][j] register r of lane l is C[m][n] with
    //      m = i*32 + l%32,  n = j*32 + (r/4)*8 + (l/32)*4 + r%4
    const int64_t m = m0 + wm * 128 + l32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t mi = m + i * 32;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int64_t n = n0 + wn * 128 + j * 32 + r4 * 8 + hi * 4;
          uint16_t o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float v = apply_epilogue_ct<OUT_DT, EPI>(g, acc[i][j][r4 * 4 + e] * g.scale, mi, n + e);
            if constexpr (OUT_DT == DT_BF16) o[e] = f32_to_bf16(v);
            else o[e] = f32_to_f16(v);
          }
          u32x2 pk = {(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
          *(u32x2 *)((uint16_t *)g.c + mi * g.ldc + n) = pk;
        }
      }
    }
  }
}

} // namespace fast

extern "C" {

#define GEMM_TILE(name, IN, OUT, EPI)                                                              \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds0[fast::STAGE];                            \
    __shared__ __attribute__((aligned(1024))) uint8_t lds1[fast::STAGE];                            \
    fast::body<IN, OUT, EPI>(g, lds0, lds1);                                                        \
  }
#define GEMM_TILE_ALL_EPI(prefix, IN, OUT)             \
  GEMM_TILE(prefix##_epi0, IN, OUT, EPI_NONE)           \
  GEMM_TILE(prefix##_epi1, IN, OUT, EPI_BIAS_FULL)      \
  GEMM_TILE(prefix##_epi2, IN, OUT, EPI_BIAS_ROW_GELU)  \
  GEMM_TILE(prefix##_epi3, IN, OUT, EPI_LEAKY_RELU)     \
  GEMM_TILE(prefix##_epi4, IN, OUT, EPI_BIAS_ROW)

GEMM_TILE_ALL_EPI(gemm_tile_bf16, DT_BF16, DT_BF16)
GEMM_TILE_ALL_EPI(gemm_tile_f16, DT_F16, DT_F16)

} // extern "C"
