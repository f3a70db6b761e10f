// Argument block shared by the attention kernels and their host launcher.
#pragma once
#include <stdint.h>

struct AttnArgs {
  const uint16_t *q, *k, *v; // bf16 [Z*H*N_CTX, D], row stride ld* (elements)
  uint16_t *o;
  float *m;                  // [Z*H*N_CTX]
  int64_t ldq, ldk, ldv, ldo;
  int32_t n_ctx;
  int32_t rows;              // query rows to produce per head: min(N_CTX, gridX*BLOCK_M)
  int32_t heads;             // (batch, head) pairs to produce: gridY
  int32_t causal;            // STAGE == 3
  float sm_scale;
};
