// Argument block shared by the tile-matmul kernels and their host launcher.
#pragma once
#include <stdint.h>

// One argument block for every tile-matmul kernel (passed by value).
struct GemmArgs {
  const void *a;    // [M,K] row-major, leading stride lda (elements)
  const void *b;    // [K,N] row-major, leading stride ldb
  void *c;          // [M,N] row-major, leading stride ldc
  const void *bias; // [M,N] of the output type (EPI_BIAS_FULL) or fp32 [N] (row forms)
  int64_t lda, ldb, ldc, ldbias;
  int32_t M, N, K;
  int32_t BM, BN, BK;       // logical tile of one program
  int32_t group_m;          // GROUP_SIZE_M
  int32_t grid;             // number of logical programs
  int32_t num_pid_m, num_pid_n;
  int32_t epi;
  float scale;              // multiplies the accumulator before the cast
  uint16_t pad_a, pad_b;    // any-shape kernels: what an element of a / b outside the matrix reads as (16-bit operand bits):
                            // 0, or a NaN for descriptors with padding == "nan" (backend/driver.py:322-329)
  int32_t tiled;            // operands are tile-major buffers with tiles BM x BK, BK x BN, BM x BN (ld* unused)
  int32_t ksplit;           // gemm_splitk_*: slices of K (K is a multiple of 128 * ksplit); c is then the workspace of
                            // ksplit x M x ldws fp32 sums.  gemm_splitk_reduce_*: slabs to add; a is then the workspace
  int64_t ldws;             // leading stride of a slab of that workspace in floats: N rounded up to a multiple of 8
  unsigned long long *probe; // diagnostic: workgroup 0 stores {core-clock cycles, 100 MHz ticks} of its run, or null
};
