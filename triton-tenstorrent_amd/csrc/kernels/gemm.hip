// Tile-matmul kernels for gfx950: matmul_kernel_tma, matmul_kernel_fused and the
// fp8-scaled sibling
// (examples/matmul_tensor_descriptor/09-persistent-matmul.py:102-145,
//  python/tutorials/09-matmul-fused.py:100-148).
//
// gemm_any_*   : every shape, stride, tile size (multiples of 32), partial
//                logical grid, ragged edges with descriptor zero-padding and
//                clipped stores.  One wavefront owns one 32x32 piece of a
//                logical tile and walks K with v_mfma_f32_32x32x16, operands
//                straight from global memory.  Correctness path, not a fast one.
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

template <int IN_DT, int OUT_DT> __device__ __forceinline__ void gemm_any_body(const GemmArgs &g) {
  using F = Frag<IN_DT>;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  const int sub_n = g.BN >> 5;
  const int spt = (g.BM >> 5) * sub_n; // 32x32 pieces per logical tile
  const int64_t items = (int64_t)g.grid * spt;
  const int64_t stride = (int64_t)gridDim.x * waves_per_block;
  const int r32 = lane & 31, kg = lane >> 5;
  for (int64_t it = (int64_t)blockIdx.x * waves_per_block + wave; it < items; it += stride) {
    const int pid = (int)(it / spt), sub = (int)(it % spt);
    int pid_m, pid_n;
    tile_of_pid(pid, g.num_pid_m, g.num_pid_n, g.group_m, pid_m, pid_n);
    const int64_t m0 = (int64_t)pid_m * g.BM + (sub / sub_n) * 32;
    const int64_t n0 = (int64_t)pid_n * g.BN + (sub % sub_n) * 32;
    if (m0 >= g.M || n0 >= g.N) continue; // piece lies wholly in the padding (wave-uniform)
    const int64_t am = m0 + r32, bn = n0 + r32;
    const bool am_ok = am < g.M, bn_ok = bn < g.N;
    f32x16 acc = {0};
    for (int k0 = 0; k0 < g.K; k0 += 16) {
      union { typename F::vec v; uint16_t s[8]; } a, b;
      const int kb = k0 + kg * 8;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = kb + j;
        const bool k_ok = k < g.K;
        a.s[j] = (am_ok && k_ok) ? F::enc(g.a, am * g.lda + k) : (uint16_t)0;
        b.s[j] = (bn_ok && k_ok) ? F::enc(g.b, (int64_t)k * g.ldb + bn) : (uint16_t)0;
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
        store_from_f32<OUT_DT>(g.c, m * g.ldc + n, v);
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

} // extern "C"

// ===========================================================================
// gemm_tile_*  : the fast path.  Requirements (checked by the host): M, N
//                multiples of 256, K a multiple of 64, 16-byte aligned bases and
//                leading strides, and a logical grid that covers every tile --
//                then which physical tile computes which part of C is free, and
//                C is bit-for-bit independent of it up to fp32 summation order.
//
// One workgroup (4 wavefronts, 2x2) computes a 256x256 macro tile, walking K in
// steps of 64 through two LDS stages (A 256x64 and B 64x256 per stage, 64 KiB).
// Each wavefront owns 128x128 of it: 4x4 v_mfma_f32_32x32x16 accumulators.
// The grid is persistent (one workgroup per CU) and strides over the macro
// tiles in an XCD-aware, L2-friendly order.
//
// LDS layout (16-byte chunks, XOR-swizzled so that both the row-wise A reads and
// the transposing B reads are bank-conflict free):
//   A stage: row m (128 B = 8 chunks); logical chunk c sits at c ^ ((m>>1)&7)
//   B stage: row k (512 B = 32 chunks); logical chunk c sits at c ^ ((k&3)<<2)
// Global->LDS copies are laid out so that thread t writes byte t*16 of each
// 4 KiB slab: the swizzle is applied on the global address instead.
//
// The product is formed transposed, acc = mfma(Bfrag, Afrag): the result lane
// then holds 4 consecutive n for one m, which makes the epilogue's stores and
// bias loads 8 bytes wide.  B fragments (k along the lane's registers, but n
// contiguous in memory) come from ds_read_b64_tr_b16, which transposes a 4x16
// block of 16-bit values across each group of 16 lanes.
// ===========================================================================
namespace {

constexpr int FT_BM = 256, FT_BN = 256, FT_BK = 64;
constexpr int FT_A_BYTES = FT_BM * FT_BK * 2;            // 32 KiB
constexpr int FT_B_BYTES = FT_BK * FT_BN * 2;            // 32 KiB
constexpr int FT_STAGE = FT_A_BYTES + FT_B_BYTES;        // 64 KiB

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

template <int IN_DT> struct FastFrag;
template <> struct FastFrag<DT_BF16> {
  typedef bf16x8 vec;
  static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct FastFrag<DT_F16> {
  typedef f16x8 vec;
  static __device__ __forceinline__ f32x16 mfma(vec a, vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// Macro-tile order: consecutive ids are dealt round-robin to the 8 XCDs by the
// hardware dispatcher, so give each XCD a contiguous run of ids (its L2 then
// sees neighbouring tiles), and walk the ids in GROUP-wide column-major bands.
__device__ __forceinline__ void fast_tile_of(int t, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int total = tiles_m * tiles_n;
  constexpr int XCD = 8;
  int id = t;
  if (total % XCD == 0) id = (t % XCD) * (total / XCD) + t / XCD;
  constexpr int G = 8;
  const int in_group = G * tiles_n;
  const int group = id / in_group;
  const int first_m = group * G;
  const int gsz = min(tiles_m - first_m, G);
  tm = first_m + (id % in_group) % gsz;
  tn = (id % in_group) / gsz;
}

template <int IN_DT, int OUT_DT, int EPI>
__device__ __forceinline__ void gemm_tile_body(const GemmArgs &g, uint8_t *lds) {
  using F = FastFrag<IN_DT>;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = g.M / FT_BM, tiles_n = g.N / FT_BN;
  const int total = tiles_m * tiles_n;
  const int nk = g.K / FT_BK;

  // ---- per-thread constants of the global->LDS copy ----
  // A: slab i (32 rows): row = i*32 + (tid>>3), LDS chunk position tid&7
  const int a_row = tid >> 3;
  const int a_chunk = (tid & 7) ^ ((a_row >> 1) & 7);
  // B: slab i (8 k-rows): k = i*8 + (tid>>5), LDS chunk position tid&31
  const int b_k = tid >> 5;
  const int b_chunk = (tid & 31) ^ ((b_k & 3) << 2);
  const int st_off = tid * 16;

  // ---- per-lane constants of the fragment reads ----
  const int l32 = lane & 31, hi = lane >> 5;
  const int a_base = (wm * 128 + l32) * 128;
  const int a_x = (lane >> 1) & 7;
  int a_pos[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) a_pos[s] = (((s * 2 + hi) ^ a_x) << 4);
  const int G4 = lane >> 4, i16 = lane & 15, q = i16 >> 2;
  const int b_base = FT_A_BYTES + (((G4 >> 1) * 8 + q) * 512) + ((wn * 16 + (G4 & 1) * 2 + ((i16 >> 1) & 1)) << 4) +
                     ((i16 & 1) << 3);
  int b_j[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) b_j[j] = ((j ^ q) << 6);

  const uint16_t *A = (const uint16_t *)g.a;
  const uint16_t *B = (const uint16_t *)g.b;

  for (int t = blockIdx.x; t < total; t += gridDim.x) {
    int tm, tn;
    fast_tile_of(t, tiles_m, tiles_n, tm, tn);
    const int64_t m0 = (int64_t)tm * FT_BM, n0 = (int64_t)tn * FT_BN;
    const uint16_t *ag = A + (m0 + a_row) * g.lda + a_chunk * 8;
    const uint16_t *bg = B + (int64_t)b_k * g.ldb + n0 + b_chunk * 8;
    const int64_t a_slab = 32 * g.lda, b_slab = 8 * g.ldb;

    u32x4 ra[8], rb[8];
    auto load_global = [&](int kt) {
      const uint16_t *ap = ag + (int64_t)kt * FT_BK;
      const uint16_t *bp = bg + (int64_t)kt * FT_BK * g.ldb;
#pragma unroll
      for (int i = 0; i < 8; ++i) ra[i] = *(const u32x4 *)(ap + i * a_slab);
#pragma unroll
      for (int i = 0; i < 8; ++i) rb[i] = *(const u32x4 *)(bp + i * b_slab);
    };
    auto store_lds = [&](int stage) {
      uint8_t *sa = lds + stage * FT_STAGE + st_off;
#pragma unroll
      for (int i = 0; i < 8; ++i) *(u32x4 *)(sa + i * 4096) = ra[i];
#pragma unroll
      for (int i = 0; i < 8; ++i) *(u32x4 *)(sa + FT_A_BYTES + i * 4096) = rb[i];
    };

    f32x16 acc[4][4]; // [m-tile][n-tile]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = (f32x16){0};

    __syncthreads(); // the previous tile's last reads are done before the stages are refilled
    load_global(0);
    store_lds(0);
    __syncthreads();
    if (nk > 1) load_global(1);

    for (int kt = 0; kt < nk; ++kt) {
      const uint8_t *sb = lds + (kt & 1) * FT_STAGE;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        typename F::vec af[4], bf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          af[i] = *(const typename F::vec *)(sb + a_base + i * 4096 + a_pos[s]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint8_t *p = sb + b_base + s * 8192 + b_j[j];
          union { s16x4 h[2]; typename F::vec v; } u;
          u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p));
          u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 2048));
          bf[j] = u.v;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = F::mfma(bf[j], af[i], acc[i][j]);
      }
      if (kt + 1 < nk) store_lds((kt + 1) & 1);
      __syncthreads();
      if (kt + 2 < nk) load_global(kt + 2);
    }

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

} // namespace

extern "C" {

#define GEMM_TILE(name, IN, OUT, EPI)                                                              \
  __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(GemmArgs g) { \
    __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * FT_STAGE];                            \
    gemm_tile_body<IN, OUT, EPI>(g, lds);                                                           \
  }
#define GEMM_TILE_ALL_EPI(prefix, IN, OUT)        \
  GEMM_TILE(prefix##_epi0, IN, OUT, EPI_NONE)      \
  GEMM_TILE(prefix##_epi1, IN, OUT, EPI_BIAS_FULL) \
  GEMM_TILE(prefix##_epi2, IN, OUT, EPI_BIAS_ROW_GELU) \
  GEMM_TILE(prefix##_epi3, IN, OUT, EPI_LEAKY_RELU) \
  GEMM_TILE(prefix##_epi4, IN, OUT, EPI_BIAS_ROW)

GEMM_TILE_ALL_EPI(gemm_tile_bf16, DT_BF16, DT_BF16)
GEMM_TILE_ALL_EPI(gemm_tile_f16, DT_F16, DT_F16)

} // extern "C"
