// tt_matmul_kernel_tma / tt_matmul_kernel_fused / tt_matmul_kernel_tma_fp8_scaled / tt_matmul_kernel:
// launch validation and kernel selection for the tile-matmul family.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>

#include "tt_internal.h"
#include "../kernels/gemm_args.h"

using namespace ttamd;

namespace {

// rt_gemm_clock_probe: armed for one launch; the last reading {core-clock cycles, 100 MHz ticks} of workgroup 0
std::atomic<int> g_probe_armed{0};
std::atomic<unsigned long long> g_probe_last[2];

// Workgroups of the persistent macro-tile kernels: one per CU, or one per tile when there are fewer tiles.
// The plain kernels (`splits`) finish a tail of at most grid/2 macro tiles as half tiles on twice the
// workgroups, so a problem of at most CUs/2 tiles is launched with two workgroups per tile; those that also have
// the quarter-tile pass (`quarters`) get four workgroups per tile for a problem of at most CUs/4 tiles.
// `live_rows`: rows of a tile that exist when the matrix is a single row of tiles (else 256): halves and quarters
// wholly past them are not work items, so a 64-row matrix gets one workgroup per tile in the quarter pass.
int64_t live_parts(int64_t live_rows, int64_t rows_per_part) { return cdiv64(std::min<int64_t>(live_rows, 256), rows_per_part); }
uint32_t persistent_grid(int64_t tiles, bool splits, bool quarters = false, int64_t live_rows = 256) {
  const int64_t cus = props()->multiprocessor_count;
  if (tiles >= cus) return (uint32_t)cus;
  const bool no_split = env_int("TTAMD_GEMM_NO_SPLIT", 0) != 0;
  if (quarters && live_parts(live_rows, 64) * tiles <= cus && !no_split) return (uint32_t)(live_parts(live_rows, 64) * tiles);
  if (splits && live_parts(live_rows, 128) * tiles <= cus && !no_split) return (uint32_t)(live_parts(live_rows, 128) * tiles);
  return (uint32_t)tiles;
}

// K in slices (gemm_splitk_*): the slices' fp32 sums pass through a workspace of ksplit x M x N floats.  Launches on
// one stream run in order and share one workspace; every (device, stream) pair gets its own on first use, grown when
// a launch needs more (the stream is drained first) and kept until rt_release_stream or the end of the process.  A
// launch that is being recorded into a graph does not take this path: the graph could be replayed on any stream,
// beside eager launches on the one it was recorded on, with the workspace's address baked in.
constexpr int64_t kSplitKMaxBytes = 64ll << 20;
std::mutex g_ws_mu;
struct Workspace { void *p; int64_t bytes; };
std::map<std::pair<int, void *>, Workspace> g_ws;
void *splitk_workspace(void *stream, int64_t bytes) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing((hipStream_t)stream, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lk(g_ws_mu);
  Workspace &w = g_ws[{dev, stream}];
  if (w.bytes >= bytes) return w.p;
  if (w.p) {
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess || hipFree(w.p) != hipSuccess) return nullptr;
    w = {nullptr, 0};
  }
  void *p = nullptr;
  if (hipMalloc(&p, (size_t)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  w = {p, bytes};
  return p;
}

// Slices of K for a launch of `tiles` macro tiles, or 1.  A problem of few tiles is finished as quarter tiles (64
// rows by 256 columns, `parts` live ones per tile); where even those leave CUs idle and K is long, slices of K make
// more of them: the largest power of two up to 16 that gives at most one quarter tile per CU (the kernel fits two
// on a CU, but past one per CU the growing workspace costs more than the slices save: 128 x 8192 x 8192 37, 44 and
// 53 us with 4, 8 and 16 slices), keeps every slice at sixteen steps or more and the workspace within bounds.  What it costs is one more launch and a pass over ksplit x M x N floats in
// each direction (taken at 6 us, the adding kernel alone runs 4-5, and 4 TB/s); what it saves is (1 - 1/ksplit) of K/32 quarter-tile steps of about
// 0.235 us.
// (`bk`: K of a step, 32 for the 16-bit kernels and 64 for fp8, whose part is the half tile; `step_us`: what a
// step of such a part takes)
int pick_ksplit(int64_t tiles, int64_t parts, int64_t M, int64_t N, int64_t K, int64_t bk = 32, double step_us = 0.235) {
  const int64_t cus = props()->multiprocessor_count;
  if (env_int("TTAMD_GEMM_NO_SPLITK", 0) || 2 * parts * tiles > cus) return 1;
  int s = 1;
  while (s < 16 && 2 * s * parts * tiles <= cus && K % (2 * s * 4 * bk) == 0 && K / (2 * s) >= 16 * bk &&
         2 * s * M * N * 4 <= kSplitKMaxBytes)
    s *= 2;
  // The steps a slice saves go as 1/s, the pass over the workspace grows as s: with a = K/bk steps of step_us and
  // b = the microseconds one more slab costs, a/s + b*s is least at s = sqrt(a/b); the power of two below 1.4 times
  // that (fp8 128 x 8192 x 8192: 28.7 us at 4 slices, 32.2 at the 8 that fit; 512 x 2048 x 8192: 26.4 against 29.8).
  const double a_us = (double)(K / bk) * step_us, b_us = (double)M * N * 8 / 4.0e6;
  while (s > 2 && s > 1.4 * std::sqrt(a_us / b_us)) s /= 2;
  if (const int forced = env_int("TTAMD_GEMM_KSPLIT", 0)) s = (K % (forced * 4 * bk) == 0 && (int64_t)forced * M * N * 4 <= kSplitKMaxBytes) ? forced : 1;
  if (s == 1) return 1;
  const double saved_us = (double)(K / bk) * (1.0 - 1.0 / s) * step_us;
  const double cost_us = 6.0 + (double)s * M * N * 8 / 4.0e6;
  return (saved_us > cost_us || env_int("TTAMD_GEMM_KSPLIT", 0)) ? s : 1;
}

// The pair of launches of a matmul computed in slices of K, or kNoWorkspace when the stream is recording or the
// workspace cannot be had (the caller then launches in one pass).
constexpr int kNoWorkspace = -12345;
int launch_in_slices(const GemmArgs &g, int ksplit, int64_t tiles, int64_t live_rows, const char *slices_kernel,
                     const char *sum_kernel, void *stream, int64_t rows_per_part = 64) {
  // From the lookup of the workspace to the second launch nothing of another thread's comes between: two threads
  // that feed one stream would otherwise interleave their pairs (the second's slices landing under the first's
  // sums), or one would grow the workspace, which frees the old one, between the other's lookup and launches.
  static std::mutex pair_mu;
  std::lock_guard<std::mutex> pair(pair_mu);
  const int64_t ldws = cdiv64(g.N, 8) * 8;
  void *ws = splitk_workspace(stream, (int64_t)ksplit * g.M * ldws * 4);
  if (!ws) return kNoWorkspace;
  GemmArgs part = g, sum = g;
  part.c = ws;
  part.ksplit = sum.ksplit = ksplit;
  part.ldws = sum.ldws = ldws;
  part.epi = TT_EPI_NONE;
  void *pargs[] = {&part};
  // every tile as its live quarters (fp8: halves); the 16-bit kernels fit two workgroups on a CU
  const uint32_t pwgs = (uint32_t)std::min<int64_t>(live_parts(live_rows, rows_per_part) * tiles * ksplit,
                                                    (rows_per_part == 64 ? 2 : 1) * (int64_t)props()->multiprocessor_count);
  const int lrc = launch("gemm", slices_kernel, dim3(pwgs), dim3(256), 0, stream, pargs, 1);
  if (lrc) return lrc;
  sum.a = ws;
  void *sargs[] = {&sum};
  const int64_t groups = (int64_t)g.M * (ldws / 8);
  const uint32_t swgs = (uint32_t)std::min<int64_t>(cdiv64(groups, 256), (int64_t)props()->multiprocessor_count * 8);
  return launch("gemm", sum_kernel, dim3(swgs), dim3(256), 0, stream, sargs, 1);
}

int check_desc(const char *who, const char *what, const tt_desc2d *d, int64_t rows, int64_t cols) {
  if (!d) return fail(RT_ERR_INVALID, "%s: null %s descriptor", who, what);
  if (!d->base) return fail(RT_ERR_INVALID, "%s: %s descriptor has a null base", who, what);
  if (d->dtype != TT_F32 && d->dtype != TT_BF16 && d->dtype != TT_F16 && d->dtype != TT_FP8E4M3)
    return fail(RT_ERR_UNSUPPORTED, "%s: %s dtype %d", who, what, d->dtype);
  if (d->strides[1] != 1)
    return fail(RT_ERR_INVALID, "%s: %s descriptor's last stride is %lld, must be 1", who, what,
                (long long)d->strides[1]);
  if (d->shape[0] != rows || d->shape[1] != cols)
    return fail(RT_ERR_INVALID, "%s: %s descriptor is [%d,%d], the launch says [%lld,%lld]", who, what,
                d->shape[0], d->shape[1], (long long)rows, (long long)cols);
  if (d->strides[0] < cols)
    return fail(RT_ERR_INVALID, "%s: %s leading stride %lld < row length %lld", who, what,
                (long long)d->strides[0], (long long)cols);
  if (reinterpret_cast<uintptr_t>(d->base) % dtype_size(d->dtype))
    return fail(RT_ERR_INVALID, "%s: %s base is not aligned to its element size", who, what);
  return RT_OK;
}

int run_matmul(const char *who, const tt_desc2d *a, const tt_desc2d *b, const tt_desc2d *c,
               const tt_desc2d *bias, int32_t M, int32_t N, int32_t K, int32_t BM, int32_t BN,
               int32_t BK, int32_t group_m, int32_t epi, float scale, const uint32_t grid[3],
               void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "%s: call rt_init first", who);
  if (!grid) return fail(RT_ERR_INVALID, "%s: null grid", who);
  if (M <= 0 || N <= 0 || K < 0) return fail(RT_ERR_INVALID, "%s: M,N,K = %d,%d,%d", who, M, N, K);
  if (BM <= 0 || BN <= 0 || BK <= 0 || group_m <= 0)
    return fail(RT_ERR_INVALID, "%s: BLOCK sizes and GROUP_SIZE_M must be positive", who);
  if (BM % 32 || BN % 32)
    return fail(RT_ERR_UNSUPPORTED, "%s: BLOCK_SIZE_M/N = %d/%d, multiples of 32 are supported", who,
                BM, BN);
  int rc;
  if ((rc = check_desc(who, "a", a, M, K))) return rc;
  if ((rc = check_desc(who, "b", b, K, N))) return rc;
  if ((rc = check_desc(who, "c", c, M, N))) return rc;
  if (a->dtype != b->dtype) return fail(RT_ERR_INVALID, "%s: a and b dtypes differ", who);
  if (grid[1] != 1 || grid[2] != 1)
    return fail(RT_ERR_INVALID, "%s: 1-D grid expected, got (%u,%u,%u)", who, grid[0], grid[1], grid[2]);
  const int64_t num_pid_m = cdiv64(M, BM), num_pid_n = cdiv64(N, BN);
  if ((int64_t)grid[0] > num_pid_m * num_pid_n)
    return fail(RT_ERR_INVALID, "%s: grid %u exceeds the %lld tiles of the problem", who, grid[0],
                (long long)(num_pid_m * num_pid_n));
  if (grid[0] == 0) return fail(RT_ERR_INVALID, "%s: empty grid", who);

  GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a->base; g.b = b->base; g.c = c->base;
  g.lda = a->strides[0]; g.ldb = b->strides[0]; g.ldc = c->strides[0];
  g.M = M; g.N = N; g.K = K; g.BM = BM; g.BN = BN; g.BK = BK;
  g.group_m = group_m; g.grid = (int32_t)grid[0];
  g.num_pid_m = (int32_t)num_pid_m; g.num_pid_n = (int32_t)num_pid_n;
  g.epi = epi; g.scale = scale;
  switch (epi) {
  case TT_EPI_NONE: case TT_EPI_LEAKY_RELU: break;
  case TT_EPI_BIAS_FULL:
    if ((rc = check_desc(who, "bias", bias, M, N))) return rc;
    if (bias->dtype != c->dtype)
      return fail(RT_ERR_INVALID, "%s: the full bias must have the output dtype", who);
    g.bias = bias->base; g.ldbias = bias->strides[0];
    break;
  case TT_EPI_BIAS_ROW: case TT_EPI_BIAS_ROW_GELU:
    if (!bias || !bias->base) return fail(RT_ERR_INVALID, "%s: null bias descriptor", who);
    if (bias->dtype != TT_F32) return fail(RT_ERR_UNSUPPORTED, "%s: the row bias must be fp32", who);
    if (!((bias->shape[0] == 1 && bias->shape[1] == N) || (bias->shape[0] == N && bias->shape[1] == 1)))
      return fail(RT_ERR_INVALID, "%s: row bias must have N = %d elements, got [%d,%d]", who, N,
                  bias->shape[0], bias->shape[1]);
    if (bias->shape[1] == 1 && bias->shape[0] != 1 && bias->strides[0] != 1)
      return fail(RT_ERR_INVALID, "%s: row bias must be contiguous", who);
    g.bias = bias->base;
    break;
  default: return fail(RT_ERR_INVALID, "%s: unknown epilogue %d", who, epi);
  }

  // padding == "nan" (backend/driver.py:322-329): elements of a and b outside the matrix read as NaN instead
  // of zero.  Rows past M and columns past N only feed results that are never stored, so the option shows
  // only when K is not a whole number of BLOCK_SIZE_K steps: then every product picks up NaN * x.  Those
  // launches take the any-shape kernel, which reads out-of-range elements as pad_a / pad_b; for all others
  // the result is the zero-padded one.  On the output (and on a full bias, whose out-of-range elements are
  // added to results that are not stored) the option has no meaning and is ignored.
  const int in = a->dtype, out = c->dtype;
  const uint16_t nan16 = in == TT_F16 ? 0x7e00 : 0x7fc0;   // e4m3 operands are widened to bf16 in that kernel
  g.pad_a = a->padding_nan ? nan16 : 0;
  g.pad_b = b->padding_nan ? nan16 : 0;
  const bool nan_shows = (a->padding_nan || b->padding_nan) && K % BK != 0;
  const char *name = nullptr;
  if (in == TT_BF16 && out == TT_BF16) name = "gemm_any_bf16_bf16";
  else if (in == TT_F16 && out == TT_F16) name = "gemm_any_f16_f16";
  else if (in == TT_FP8E4M3 && out == TT_BF16) name = "gemm_any_fp8_bf16";
  else if (in == TT_FP8E4M3 && out == TT_F16) name = "gemm_any_fp8_f16";
  else if (in == TT_FP8E4M3 && out == TT_FP8E4M3) name = "gemm_any_fp8_fp8";
  else return fail(RT_ERR_UNSUPPORTED, "%s: no kernel for input dtype %d -> output dtype %d", who, in, out);

  // Fast path: whole 256x256x64 macro tiles, 16-byte aligned rows, and a grid that covers
  // the problem (then the assignment of output to programs does not show in the result).
  const bool full_grid = (int64_t)grid[0] == num_pid_m * num_pid_n;
  const bool half_io = (in == TT_BF16 && out == TT_BF16) || (in == TT_F16 && out == TT_F16);
  // (leading strides below 2^23 elements: a thread's offset from its tile's first row is a 32-bit byte count)
  const bool fast_shape = M % 256 == 0 && N % 256 == 0 && K % 128 == 0 && K >= 128 && g.lda < (1 << 23) && g.ldb < (1 << 23);
  const bool fast_align = aligned16(g.a) && aligned16(g.b) && aligned16(g.c) && g.lda % 8 == 0 &&
                          g.ldb % 8 == 0 && g.ldc % 8 == 0;
  // The same kernel with clamped fetches, zero-padded K steps and clipped stores takes every other shape
  // whose rows can be fetched in 16-byte pieces (N and K multiples of 8; a last K step that ends past K has its
  // copies redirected into the matrix and the surplus cleared in shared memory).
  const bool ragged_shape = !fast_shape && N % 8 == 0 && K % 8 == 0 && g.lda < (1 << 23) && g.ldb < (1 << 23);
  if (full_grid && half_io && (fast_shape || ragged_shape) && fast_align && !nan_shows && !env_int("TTAMD_GEMM_FORCE_ANY", 0)) {
    char fast_name[64];
    // a C that the 256 MiB memory-side cache does not hold is stored past the caches while K is short (plain epilogue)
    const bool past_caches = epi == TT_EPI_NONE && (int64_t)M * N * 2 > (256ll << 20) && K <= 2048;
    snprintf(fast_name, sizeof(fast_name), "gemm_%s_%s_epi%d%s", fast_shape ? "tile" : "ragged", in == TT_BF16 ? "bf16" : "f16",
             epi, past_caches ? "_stream" : "");
    const int64_t tiles = cdiv64(M, 256) * cdiv64(N, 256);
    const int64_t live_rows = M <= 256 ? M : 256;      // of a tile, where the matrix is a single row of tiles
    const int ksplit = pick_ksplit(tiles, live_parts(live_rows, 64), M, N, K);
    if (ksplit > 1) {
      const int lrc = launch_in_slices(g, ksplit, tiles, live_rows, in == TT_BF16 ? "gemm_splitk_bf16" : "gemm_splitk_f16",
                                       out == TT_BF16 ? "gemm_splitk_reduce_bf16" : "gemm_splitk_reduce_f16", stream);
      if (lrc != kNoWorkspace) return lrc;
    }
    const uint32_t wgs = persistent_grid(tiles, true, true, fast_shape ? 256 : live_rows);
    // Diagnostic (TTAMD_GEMM_CLOCK_PROBE=1): workgroup 0 reports its core-clock cycles and
    // 100 MHz ticks; the launch is then synchronous and prints the effective clock.
    static unsigned long long *probe_buf = nullptr;
    const bool armed = g_probe_armed.exchange(0) != 0;     // rt_gemm_clock_probe(1, ...): this launch only
    const bool probe = armed || env_int("TTAMD_GEMM_CLOCK_PROBE", 0) != 0;
    if (probe && !probe_buf && hipMalloc((void **)&probe_buf, 16) != hipSuccess) probe_buf = nullptr;
    g.probe = probe ? probe_buf : nullptr;
    void *fargs[] = {&g};
    int lrc = launch("gemm", fast_name, dim3(wgs), dim3(256), 0, stream, fargs, 1);
    if (lrc == 0 && g.probe) {
      unsigned long long h[2] = {0, 0};
      if (hipStreamSynchronize((hipStream_t)stream) == hipSuccess &&
          hipMemcpy(h, probe_buf, 16, hipMemcpyDeviceToHost) == hipSuccess && h[1]) {
        g_probe_last[0] = h[0];
        g_probe_last[1] = h[1];
      }
      if (h[1] && !armed)
        fprintf(stderr, "[ttamd] %s: workgroup 0 ran %llu core cycles in %.1f us -> %.3f GHz\n", fast_name, h[0],
                h[1] / 100.0, h[0] / (h[1] * 10.0));
    }
    return lrc;
  }

  // fp8 fast path: e4m3 in, bf16/fp16 out, scale in the epilogue, K in steps of 64 through a 4-stage ring
  const bool fp8_io = in == TT_FP8E4M3 && (out == TT_BF16 || out == TT_F16 || out == TT_FP8E4M3) && epi == TT_EPI_NONE;
  const bool fp8_shape = M % 256 == 0 && N % 256 == 0 && K % 256 == 0 && K >= 256 && g.lda < (1 << 24) && g.ldb < (1 << 24);
  // 16-bit results leave in 16-byte stores (8 elements), e4m3 results in 4-byte ones
  const bool fp8_align = aligned16(g.a) && aligned16(g.b) && aligned16(g.c) && g.lda % 16 == 0 && g.ldb % 16 == 0 &&
                         g.ldc % (out == TT_FP8E4M3 ? 4 : 8) == 0;
  const bool fp8_ragged = !fp8_shape && N % 16 == 0 && K % 64 == 0 && g.lda < (1 << 24) && g.ldb < (1 << 24);
  if (full_grid && fp8_io && (fp8_shape || fp8_ragged) && fp8_align && !nan_shows && !env_int("TTAMD_GEMM_FORCE_ANY", 0)) {
    const int64_t tiles = cdiv64(M, 256) * cdiv64(N, 256);
    // few tiles under a long K: in slices of K, as for the 16-bit kernels; the part is the half tile here, whose step
    // of K = 64 takes 8 MFMAs of 64 cycles
    const int64_t live_rows8 = M <= 256 ? M : 256;
    const int ksplit8 = out == TT_FP8E4M3 ? 1 : pick_ksplit(tiles, live_parts(live_rows8, 128), M, N, K, 64, 0.3);
    if (ksplit8 > 1) {
      const int lrc = launch_in_slices(g, ksplit8, tiles, live_rows8, "gemm_splitk_fp8",
                                       out == TT_BF16 ? "gemm_splitk_reduce_bf16" : "gemm_splitk_reduce_f16", stream, 128);
      if (lrc != kNoWorkspace) return lrc;
    }
    const uint32_t wgs = persistent_grid(tiles, true);
    void *fargs[] = {&g};
    char fp8_name[64];
    // a 16-bit C that the 256 MiB memory-side cache does not hold is stored past the caches while K is short
    const bool past_caches = out != TT_FP8E4M3 && (int64_t)M * N * 2 > (256ll << 20) && K <= 4096;
    snprintf(fp8_name, sizeof(fp8_name), "gemm_%s_fp8_%s%s", fp8_shape ? "tile" : "ragged",
             out == TT_BF16 ? "bf16" : out == TT_F16 ? "f16" : "fp8", past_caches ? "_stream" : "");
    return launch("gemm", fp8_name, dim3(wgs), dim3(256), 0, stream, fargs, 1);
  }

  const int64_t items = (int64_t)grid[0] * (BM / 32) * (BN / 32);
  const int64_t cap = (int64_t)props()->multiprocessor_count * 8;
  const uint32_t blocks = (uint32_t)std::max<int64_t>(1, std::min(cap, cdiv64(items, 4)));
  void *args[] = {&g};
  return launch("gemm", name, dim3(blocks), dim3(256), 0, stream, args, 1);
}

} // namespace

void *ttamd::gemm_take_workspace(int device, void *stream) {
  std::lock_guard<std::mutex> lk(g_ws_mu);
  auto it = g_ws.find({device, stream});
  if (it == g_ws.end()) return nullptr;
  void *p = it->second.p;
  g_ws.erase(it);
  return p;
}

extern "C" {

int rt_gemm_clock_probe(int32_t arm, uint64_t reading[2]) {
  if (arm) g_probe_armed.store(1);
  if (reading) {
    reading[0] = g_probe_last[0].load();
    reading[1] = g_probe_last[1].load();
  }
  return RT_OK;
}

int tt_matmul_kernel_tma(const tt_desc2d *a, const tt_desc2d *b, const tt_desc2d *c, int32_t M,
                         int32_t N, int32_t K, int32_t BLOCK_SIZE_M, int32_t BLOCK_SIZE_N,
                         int32_t BLOCK_SIZE_K, int32_t GROUP_SIZE_M, const uint32_t grid[3],
                         void *stream) {
  return run_matmul("matmul_kernel_tma", a, b, c, nullptr, M, N, K, BLOCK_SIZE_M, BLOCK_SIZE_N,
                    BLOCK_SIZE_K, GROUP_SIZE_M, TT_EPI_NONE, 1.0f, grid, stream);
}

int tt_matmul_kernel_fused(const tt_desc2d *a, const tt_desc2d *b, const tt_desc2d *c,
                           const tt_desc2d *bias, int32_t M, int32_t N, int32_t K,
                           int32_t BLOCK_SIZE_M, int32_t BLOCK_SIZE_N, int32_t BLOCK_SIZE_K,
                           int32_t GROUP_SIZE_M, int32_t epilogue, const uint32_t grid[3],
                           void *stream) {
  return run_matmul("matmul_kernel_fused", a, b, c, bias, M, N, K, BLOCK_SIZE_M, BLOCK_SIZE_N,
                    BLOCK_SIZE_K, GROUP_SIZE_M, epilogue, 1.0f, grid, stream);
}

int tt_matmul_kernel_tma_fp8_scaled(const tt_desc2d *a, const tt_desc2d *b, const tt_desc2d *c,
                                    int32_t M, int32_t N, int32_t K, float scale_a, float scale_b,
                                    int32_t BLOCK_SIZE_M, int32_t BLOCK_SIZE_N, int32_t BLOCK_SIZE_K,
                                    int32_t GROUP_SIZE_M, const uint32_t grid[3], void *stream) {
  if (a && a->dtype != TT_FP8E4M3)
    return fail(RT_ERR_INVALID, "matmul_kernel_tma_fp8_scaled: a and b must be fp8 e4m3");
  return run_matmul("matmul_kernel_tma_fp8_scaled", a, b, c, nullptr, M, N, K, BLOCK_SIZE_M,
                    BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M, TT_EPI_NONE, scale_a * scale_b, grid,
                    stream);
}

int tt_matmul_kernel(const void *a_ptr, const void *b_ptr, void *c_ptr, int32_t M, int32_t N, int32_t K,
                     int64_t stride_am, int64_t stride_ak, int64_t stride_bk, int64_t stride_bn,
                     int64_t stride_cm, int64_t stride_cn, int32_t BLOCK_SIZE_M, int32_t BLOCK_SIZE_N,
                     int32_t BLOCK_SIZE_K, int32_t GROUP_SIZE_M, int32_t leaky_relu, int32_t in_dtype,
                     const uint32_t grid[3], void *stream) {
  const char *who = "matmul_kernel";
  if (!props()) return fail(RT_ERR_NOT_INIT, "%s: call rt_init first", who);
  if (!grid) return fail(RT_ERR_INVALID, "%s: null grid", who);
  if (!a_ptr || !b_ptr || !c_ptr) return fail(RT_ERR_INVALID, "%s: null operand", who);
  if (M <= 0 || N <= 0 || K < 0) return fail(RT_ERR_INVALID, "%s: M,N,K = %d,%d,%d", who, M, N, K);
  const int32_t BM = BLOCK_SIZE_M, BN = BLOCK_SIZE_N, BK = BLOCK_SIZE_K;
  if (BM <= 0 || BN <= 0 || BK <= 0 || GROUP_SIZE_M <= 0)
    return fail(RT_ERR_INVALID, "%s: BLOCK sizes and GROUP_SIZE_M must be positive", who);
  if (BM % 32 || BN % 32)
    return fail(RT_ERR_UNSUPPORTED, "%s: BLOCK_SIZE_M/N = %d/%d, multiples of 32 are supported", who, BM, BN);
  // the kernel asserts positive strides (tl.assume, :292-297) and then does not use them
  if (stride_am <= 0 || stride_ak <= 0 || stride_bk <= 0 || stride_bn <= 0 || stride_cm <= 0 || stride_cn <= 0)
    return fail(RT_ERR_INVALID, "%s: strides must be positive", who);
  if (in_dtype != TT_F16 && in_dtype != TT_BF16)
    return fail(RT_ERR_UNSUPPORTED, "%s: input dtype %d; fp16 and bf16 are supported", who, in_dtype);
  if ((reinterpret_cast<uintptr_t>(a_ptr) | reinterpret_cast<uintptr_t>(b_ptr) | reinterpret_cast<uintptr_t>(c_ptr)) & 1)
    return fail(RT_ERR_INVALID, "%s: operands must be 2-byte aligned", who);
  if (grid[1] != 1 || grid[2] != 1)
    return fail(RT_ERR_INVALID, "%s: 1-D grid expected, got (%u,%u,%u)", who, grid[0], grid[1], grid[2]);
  const int64_t num_pid_m = cdiv64(M, BM), num_pid_n = cdiv64(N, BN);
  if (grid[0] == 0) return fail(RT_ERR_INVALID, "%s: empty grid", who);
  if ((int64_t)grid[0] > num_pid_m * num_pid_n)
    return fail(RT_ERR_INVALID, "%s: grid %u exceeds the %lld tiles of the problem", who, grid[0],
                (long long)(num_pid_m * num_pid_n));

  GemmArgs g;
  memset(&g, 0, sizeof(g));
  g.a = a_ptr; g.b = b_ptr; g.c = c_ptr;
  g.M = M; g.N = N; g.K = K; g.BM = BM; g.BN = BN; g.BK = BK;
  g.group_m = GROUP_SIZE_M; g.grid = (int32_t)grid[0];
  g.num_pid_m = (int32_t)num_pid_m; g.num_pid_n = (int32_t)num_pid_n;
  g.epi = leaky_relu ? TT_EPI_LEAKY_RELU : TT_EPI_NONE;
  g.scale = 1.0f;
  g.tiled = 1;
  void *args[] = {&g};

  // Fast path: 32x32x32 tiles (the reference's configuration), fp16, 16-byte aligned buffers, a grid that
  // covers the problem.  Whole 256x256x128 macro tiles take the plain kernel, everything else its clamping
  // instantiation (the buffers are padded to whole 32x32 tiles, which is all it needs).
  const bool full_grid = (int64_t)grid[0] == num_pid_m * num_pid_n;
  // the fast kernel keeps a thread's byte offset inside an A slab in 32 bits: 7 tile rows of ntk tiles of 2 KiB
  const bool offsets_fit = cdiv64(K, 32) * 14336 + 4096 < (int64_t)1 << 32;
  if (full_grid && offsets_fit && in_dtype == TT_F16 && BM == 32 && BN == 32 && BK == 32 && aligned16(a_ptr) &&
      aligned16(b_ptr) && aligned16(c_ptr) && !env_int("TTAMD_GEMM_FORCE_ANY", 0)) {
    const bool whole = M % 256 == 0 && N % 256 == 0 && K % 128 == 0 && K >= 128;
    const int64_t tiles = cdiv64(M, 256) * cdiv64(N, 256);
    // few tiles under a long K: in slices of K, as for the row-major kernels
    const int64_t live_rows = M <= 256 ? M : 256;
    const int ksplit = pick_ksplit(tiles, live_parts(live_rows, 64), M, cdiv64(N, 8) * 8, K);
    if (ksplit > 1) {
      const int lrc = launch_in_slices(g, ksplit, tiles, live_rows, "gemm_splitk_tiled_f16", "gemm_splitk_reduce_f16", stream);
      if (lrc != kNoWorkspace) return lrc;
    }
    const uint32_t wgs = persistent_grid(tiles, true, false, whole ? 256 : live_rows);
    char name[48];
    snprintf(name, sizeof(name), "gemm_tiled%s_f16_epi%d", whole ? "" : "ragged", leaky_relu ? 3 : 0);
    return launch("gemm", name, dim3(wgs), dim3(256), 0, stream, args, 1);
  }
  const int64_t items = (int64_t)grid[0] * (BM / 32) * (BN / 32);
  const int64_t cap = (int64_t)props()->multiprocessor_count * 8;
  const uint32_t blocks = (uint32_t)std::max<int64_t>(1, std::min(cap, cdiv64(items, 4)));
  return launch("gemm", in_dtype == TT_F16 ? "gemm_anytiled_f16_f16" : "gemm_anytiled_bf16_f16", dim3(blocks), dim3(256),
                0, stream, args, 1);
}

} // extern "C"
