// tt_attn_fwd: launch validation and kernel selection for fused attention.
#include <algorithm>
#include <cstdio>
#include <cstring>

#include "tt_internal.h"
#include "../kernels/attention_args.h"

using namespace ttamd;

namespace {
int check_qkvo(const char *what, const tt_desc2d *d, int64_t rows, int32_t head_dim) {
  if (!d || !d->base) return fail(RT_ERR_INVALID, "_attn_fwd: null %s descriptor", what);
  if (d->dtype != TT_BF16)
    return fail(RT_ERR_UNSUPPORTED, "_attn_fwd: %s dtype %d, the kernel computes in bf16", what, d->dtype);
  if (d->padding_nan) return fail(RT_ERR_UNSUPPORTED, "_attn_fwd: NaN padding is not supported");
  if (d->shape[0] != rows || d->shape[1] != head_dim)
    return fail(RT_ERR_INVALID, "_attn_fwd: %s descriptor is [%d,%d], expected [%lld,%d]", what,
                d->shape[0], d->shape[1], (long long)rows, head_dim);
  if (d->strides[1] != 1 || d->strides[0] < head_dim)
    return fail(RT_ERR_INVALID, "_attn_fwd: %s strides [%lld,%lld]", what, (long long)d->strides[0],
                (long long)d->strides[1]);
  if (reinterpret_cast<uintptr_t>(d->base) % 2)
    return fail(RT_ERR_INVALID, "_attn_fwd: %s base is not 2-byte aligned", what);
  return RT_OK;
}
} // namespace

extern "C" int tt_attn_fwd(float sm_scale, float *M, int32_t Z, int32_t H, const tt_desc2d *desc_q,
                           const tt_desc2d *desc_k, const tt_desc2d *desc_v, const tt_desc2d *desc_o,
                           int32_t N_CTX, int32_t HEAD_DIM, int32_t BLOCK_M, int32_t BLOCK_N,
                           int32_t STAGE, const uint32_t grid[3], void *stream) {
  if (!props()) return fail(RT_ERR_NOT_INIT, "_attn_fwd: call rt_init first");
  if (!grid || !M) return fail(RT_ERR_INVALID, "_attn_fwd: null grid or M pointer");
  if (Z <= 0 || H <= 0 || N_CTX <= 0) return fail(RT_ERR_INVALID, "_attn_fwd: Z,H,N_CTX = %d,%d,%d", Z, H, N_CTX);
  if (STAGE != 1 && STAGE != 3) return fail(RT_ERR_INVALID, "_attn_fwd: STAGE %d (1 = full, 3 = causal)", STAGE);
  if (BLOCK_M <= 0 || BLOCK_N <= 0) return fail(RT_ERR_INVALID, "_attn_fwd: BLOCK sizes must be positive");
  if (BLOCK_N > HEAD_DIM) // tl.static_assert(BLOCK_N <= HEAD_DIM)
    return fail(RT_ERR_INVALID, "_attn_fwd: BLOCK_N %d > HEAD_DIM %d", BLOCK_N, HEAD_DIM);
  if (BLOCK_M % 32 || N_CTX % BLOCK_M || N_CTX % BLOCK_N || BLOCK_M % BLOCK_N)
    return fail(RT_ERR_UNSUPPORTED,
                "_attn_fwd: need BLOCK_M %% 32 == 0, N_CTX %% BLOCK_M == 0, N_CTX %% BLOCK_N == 0 and "
                "BLOCK_M %% BLOCK_N == 0 (got N_CTX %d, BLOCK_M %d, BLOCK_N %d)", N_CTX, BLOCK_M, BLOCK_N);
  const int64_t y_dim = (int64_t)Z * H * N_CTX;
  if (y_dim > INT32_MAX) return fail(RT_ERR_UNSUPPORTED, "_attn_fwd: Z*H*N_CTX exceeds int32");
  int rc;
  if ((rc = check_qkvo("q", desc_q, y_dim, HEAD_DIM))) return rc;
  if ((rc = check_qkvo("k", desc_k, y_dim, HEAD_DIM))) return rc;
  if ((rc = check_qkvo("v", desc_v, y_dim, HEAD_DIM))) return rc;
  if ((rc = check_qkvo("o", desc_o, y_dim, HEAD_DIM))) return rc;
  if (grid[2] != 1) return fail(RT_ERR_INVALID, "_attn_fwd: gridZ must be 1");
  if (grid[0] == 0 || grid[1] == 0) return fail(RT_ERR_INVALID, "_attn_fwd: empty grid");
  if ((int64_t)grid[0] * BLOCK_M > N_CTX || (int64_t)grid[1] > (int64_t)Z * H)
    return fail(RT_ERR_INVALID, "_attn_fwd: grid (%u,%u) exceeds (N_CTX/BLOCK_M, Z*H) = (%d,%d)", grid[0],
                grid[1], N_CTX / BLOCK_M, Z * H);
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = (const uint16_t *)desc_q->base; a.k = (const uint16_t *)desc_k->base;
  a.v = (const uint16_t *)desc_v->base; a.o = (uint16_t *)desc_o->base; a.m = M;
  a.ldq = desc_q->strides[0]; a.ldk = desc_k->strides[0]; a.ldv = desc_v->strides[0];
  a.ldo = desc_o->strides[0];
  a.n_ctx = N_CTX; a.rows = (int32_t)(grid[0] * (int64_t)BLOCK_M); a.heads = (int32_t)grid[1];
  a.causal = STAGE == 3; a.sm_scale = sm_scale;
  // Fast path: every query of every head, 16-byte aligned rows, N_CTX in whole wavefronts of 32 queries.
  // Whole 256-query blocks take the plain kernel, other lengths its instantiation with a clipped tail.
  const bool full = (int64_t)grid[0] * BLOCK_M == N_CTX && (int64_t)grid[1] == (int64_t)Z * H;
  const bool al = aligned16(a.q) && aligned16(a.k) && aligned16(a.v) && aligned16(a.o) && a.ldq % 8 == 0 &&
                  a.ldk % 8 == 0 && a.ldv % 8 == 0 && a.ldo % 4 == 0;
  if (full && al && N_CTX % 32 == 0 && (HEAD_DIM == 32 || HEAD_DIM == 64 || HEAD_DIM == 128 || HEAD_DIM == 256) &&
      !env_int("TTAMD_ATTN_FORCE_ANY", 0)) {
    void *fargs[] = {&a};
    const int queries = HEAD_DIM == 256 ? 128 : 256;   // per workgroup: 4 or 8 wavefronts of 32
    uint32_t wgs = (uint32_t)(cdiv64(N_CTX, queries) * (int64_t)Z * H);
    // head dims 64, 128 and 256: an item is the pair of query blocks i and n-1-i of a head, and
    // the grid is persistent: one workgroup per CU walks its share of the items back to back (fewer workgroups when
    // there are fewer items)
    if (HEAD_DIM != 32) {
      const int64_t items = cdiv64(cdiv64(N_CTX, queries), 2) * (int64_t)Z * H;
      wgs = (uint32_t)std::min<int64_t>(items, props()->multiprocessor_count);
    }
    char name[32];
    snprintf(name, sizeof(name), "attn_%s_d%d", N_CTX % queries == 0 ? "tile" : "ragged", HEAD_DIM);
    return launch("attention", name, dim3(wgs), dim3(2 * queries), 0, stream, fargs, 1);
  }
  const char *name = nullptr;
  switch (HEAD_DIM) {
  case 16: name = "attn_any_d16"; break;
  case 32: name = "attn_any_d32"; break;
  case 64: name = "attn_any_d64"; break;
  case 128: name = "attn_any_d128"; break;
  case 256: name = "attn_any_d256"; break;
  default: return fail(RT_ERR_UNSUPPORTED, "_attn_fwd: HEAD_DIM %d (16,32,64,128,256 are supported)", HEAD_DIM);
  }
  void *args[] = {&a};
  return launch("attention", name, dim3((uint32_t)cdiv64(a.rows, 128), (uint32_t)a.heads), dim3(256), 0,
                stream, args, 1);
}
