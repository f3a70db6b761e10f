/* A caller of libttamd_rt.so written in plain C: what a cgo / JNI / ctypes-free embedder of the C ABI looks like.
 * tests/test_c_abi.py compiles it with gcc against include/ttamd_rt.h (which shows that the header is valid C and
 * that every symbol used resolves) and, on a GPU box, runs it: an fp32 vector add with a masked tail, an int32
 * reduction and a bf16 tile matmul on small integers, each compared with values computed here on the host.
 * Exit status 0 = all equal; anything else prints what differed. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ttamd_rt.h"

#define CHECK(call)                                                                     \
  do {                                                                                  \
    int rc_ = (call);                                                                   \
    if (rc_ != RT_OK) {                                                                 \
      fprintf(stderr, "%s -> %d: %s\n", #call, rc_, rt_last_error());                   \
      return 2;                                                                         \
    }                                                                                   \
  } while (0)

static uint16_t to_bf16(float f) { /* exact for the small integers used here */
  uint32_t u;
  memcpy(&u, &f, 4);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

int main(void) {
  CHECK(rt_init(0));
  rt_props props;
  CHECK(rt_device_props(&props));
  printf("device %s (%s), %d CUs\n", props.name, props.arch, props.multiprocessor_count);

  /* ---- add_kernel: n = 5000, BLOCK_SIZE = 1024, grid = 5; the sentinel past n must survive ---- */
  enum { N = 5000, PAD = 24 };
  float *hx = malloc(sizeof(float) * N), *hy = malloc(sizeof(float) * N), *ho = malloc(sizeof(float) * (N + PAD));
  for (int i = 0; i < N; ++i) { hx[i] = 0.25f * (float)i; hy[i] = 1.0f / (float)(i + 1); }
  void *dx, *dy, *dout;
  CHECK(rt_malloc(&dx, sizeof(float) * N));
  CHECK(rt_malloc(&dy, sizeof(float) * N));
  CHECK(rt_malloc(&dout, sizeof(float) * (N + PAD)));
  for (int i = 0; i < N + PAD; ++i) ho[i] = 7.5f;
  CHECK(rt_memcpy(dx, hx, sizeof(float) * N, 1));
  CHECK(rt_memcpy(dy, hy, sizeof(float) * N, 1));
  CHECK(rt_memcpy(dout, ho, sizeof(float) * (N + PAD), 1));
  const uint32_t grid_add[3] = {5, 1, 1};
  CHECK(tt_add_kernel(dx, dy, dout, N, 1024, TT_F32, grid_add, NULL));
  CHECK(rt_sync(NULL));
  CHECK(rt_memcpy(ho, dout, sizeof(float) * (N + PAD), 2));
  for (int i = 0; i < N; ++i)
    if (ho[i] != hx[i] + hy[i]) { fprintf(stderr, "add: element %d is %g, expected %g\n", i, ho[i], hx[i] + hy[i]); return 1; }
  for (int i = N; i < N + PAD; ++i)
    if (ho[i] != 7.5f) { fprintf(stderr, "add: wrote past n at %d\n", i); return 1; }
  printf("add_kernel ok via %s\n", tt_last_kernel_name());

  /* ---- reduce1d: sum and argmax of 512 int32 ---- */
  int32_t hv[512], hz[2] = {0, 0};
  int64_t want_sum = 0;
  int want_arg = 0;
  for (int i = 0; i < 512; ++i) {
    hv[i] = (int32_t)((i * 2654435761u) >> 8) - (1 << 23);
    want_sum += hv[i];
    if (hv[i] > hv[want_arg]) want_arg = i;
  }
  void *dv, *dz;
  CHECK(rt_malloc(&dv, sizeof(hv)));
  CHECK(rt_malloc(&dz, sizeof(hz)));
  CHECK(rt_memcpy(dv, hv, sizeof(hv), 1));
  const uint32_t grid_one[3] = {1, 1, 1};
  CHECK(tt_reduce1d_kernel(TT_REDUCE_SUM, dv, dz, 512, TT_I32, TT_I32, TT_I32, 0, grid_one, NULL));
  CHECK(tt_reduce1d_kernel(TT_REDUCE_ARGMAX, dv, (int32_t *)dz + 1, 512, TT_I32, TT_I32, TT_I32, 0, grid_one, NULL));
  CHECK(rt_sync(NULL));
  CHECK(rt_memcpy(hz, dz, sizeof(hz), 2));
  if (hz[0] != (int32_t)want_sum || hz[1] != want_arg) {
    fprintf(stderr, "reduce1d: sum %d (expected %d), argmax %d (expected %d)\n", hz[0], (int32_t)want_sum, hz[1], want_arg);
    return 1;
  }
  printf("reduce1d ok via %s\n", tt_last_kernel_name());

  /* ---- matmul_kernel_tma: 64x96 = (64x32) . (32x96), bf16, small integers => exact ---- */
  enum { M = 64, NN = 96, K = 32 };
  uint16_t *ha = malloc(2 * M * K), *hb = malloc(2 * K * NN), *hc = malloc(2 * M * NN);
  for (int i = 0; i < M * K; ++i) ha[i] = to_bf16((float)((i * 7) % 5 - 2));
  for (int i = 0; i < K * NN; ++i) hb[i] = to_bf16((float)((i * 3) % 7 - 3));
  void *da, *db, *dc;
  CHECK(rt_malloc(&da, 2 * M * K));
  CHECK(rt_malloc(&db, 2 * K * NN));
  CHECK(rt_malloc(&dc, 2 * M * NN));
  CHECK(rt_memcpy(da, ha, 2 * M * K, 1));
  CHECK(rt_memcpy(db, hb, 2 * K * NN, 1));
  tt_desc2d a_desc = {da, {M, K}, {K, 1}, {32, 32}, 0, TT_BF16};
  tt_desc2d b_desc = {db, {K, NN}, {NN, 1}, {32, 32}, 0, TT_BF16};
  tt_desc2d c_desc = {dc, {M, NN}, {NN, 1}, {32, 32}, 0, TT_BF16};
  const uint32_t grid_mm[3] = {(M / 32) * (NN / 32), 1, 1};
  CHECK(tt_matmul_kernel_tma(&a_desc, &b_desc, &c_desc, M, NN, K, 32, 32, 32, 1, grid_mm, NULL));
  CHECK(rt_sync(NULL));
  CHECK(rt_memcpy(hc, dc, 2 * M * NN, 2));
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < NN; ++n) {
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) acc += from_bf16(ha[m * K + k]) * from_bf16(hb[k * NN + n]);
      if (from_bf16(hc[m * NN + n]) != acc) {
        fprintf(stderr, "matmul: C[%d][%d] = %g, expected %g\n", m, n, from_bf16(hc[m * NN + n]), acc);
        return 1;
      }
    }
  printf("matmul_kernel_tma ok via %s\n", tt_last_kernel_name());

  /* an error path: a status code and a message, never an abort */
  if (tt_add_kernel(dx, dy, dout, -1, 1024, TT_F32, grid_add, NULL) != RT_ERR_INVALID || !strstr(rt_last_error(), "n_elements")) {
    fprintf(stderr, "negative n was not refused as expected: %s\n", rt_last_error());
    return 1;
  }
  CHECK(rt_free(dx)); CHECK(rt_free(dy)); CHECK(rt_free(dout)); CHECK(rt_free(dv)); CHECK(rt_free(dz));
  CHECK(rt_free(da)); CHECK(rt_free(db)); CHECK(rt_free(dc));
  free(hx); free(hy); free(ho); free(ha); free(hb); free(hc);
  printf("C ABI ok\n");
  return 0;
}
