/*
 * libttamd_rt.so -- C ABI of the MI355X (gfx950) host runtime.
 *
 * Two layers:
 *   rt_*  a thin loader/launcher over the HIP module API (hipModuleLoadData /
 *         hipModuleGetFunction / hipModuleLaunchKernel, hipMalloc'd buffers,
 *         hipEvents).  It takes the place of the device handle that the
 *         reference launcher drives through knexus:
 *         device.load_library / lib.get_kernel   backend/driver.py:68-74
 *         create_schedule / create_command / set_arg / finalize / run
 *                                                backend/driver.py:114-170
 *   tt_*  one entry point per kernel NAME of the reference examples, taking the
 *         same launch-time arguments (pointers, i32 sizes, tensor descriptors,
 *         the constexpr BLOCK sizes and the logical grid) and binding them to a
 *         hand-written gfx950 kernel.  The logical grid keeps the reference's
 *         meaning: program `pid` of gridX*gridY*gridZ does exactly the work the
 *         example kernel source gives it; the runtime is free to execute those
 *         programs on a persistent physical grid sized to the CU count
 *         (cpu/lib/Dialect/TritonCPU/Transforms/MakePersistentKernel.cpp:144-198).
 *
 * Conventions: every function returns 0 on success and a negative rt_status on
 * failure, never aborts and never throws; rt_last_error() gives the message of
 * the calling thread's last failure.  The caller owns every buffer and keeps it
 * alive until the stream has run the launch.  `stream` is a hipStream_t (NULL =
 * the default stream); launches are asynchronous on it.  Pointers handed to
 * tt_* are device pointers.  Distinct streams may be driven from distinct
 * threads; kernels are immutable after rt_init.
 */
#ifndef TTAMD_RT_H
#define TTAMD_RT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTAMD_API __attribute__((visibility("default")))

typedef enum rt_status {
  RT_OK = 0,
  RT_ERR_INVALID = -1,     /* bad argument (null pointer, negative size, bad grid) */
  RT_ERR_HIP = -2,         /* a HIP call failed; rt_last_error() has its string    */
  RT_ERR_NOT_FOUND = -3,   /* unknown kernel / symbol name                         */
  RT_ERR_UNSUPPORTED = -4, /* valid request this build has no kernel for           */
  RT_ERR_NOT_INIT = -5     /* rt_init has not succeeded on this device             */
} rt_status;

/* element types of tensors and descriptors (Triton type strings in comments) */
typedef enum tt_dtype {
  TT_F32 = 0,     /* *fp32    */
  TT_I32 = 1,     /* *i32     */
  TT_BF16 = 2,    /* *bf16    */
  TT_F16 = 3,     /* *fp16    */
  TT_FP8E4M3 = 4, /* *fp8e4nv (OCP e4m3fn) */
  TT_I16 = 5,     /* *i16 (result of a narrowing cast; reductions) */
  TT_I8 = 6,      /* *i8  (result of a narrowing cast; reductions) */
  TT_I64 = 7,     /* the rest: reductions only */
  TT_F64 = 8,
  TT_U8 = 9,      /* unsigned: Triton's IR is signless, the sign is that of the extension / compare ops */
  TT_U16 = 10,
  TT_U32 = 11,
  TT_U64 = 12
} tt_dtype;

/* ----------------------------------------------------------------------- */
/* rt_*: device, memory, modules, launches, events                          */
/* ----------------------------------------------------------------------- */

/* What TTUtils.get_device_properties reports (backend/driver.py:76-82), read
 * from hipGetDeviceProperties. */
typedef struct rt_props {
  int32_t device;
  int32_t multiprocessor_count; /* CUs */
  int32_t warp_size;            /* 64 */
  int32_t max_shared_mem;       /* LDS bytes per workgroup */
  int32_t max_num_regs;         /* 32-bit registers per workgroup */
  int32_t clock_khz;            /* max engine clock */
  int32_t mem_clock_khz;
  int32_t mem_bus_bits;
  int32_t l2_bytes;
  int32_t reserved;
  uint64_t total_mem;           /* HBM bytes */
  char name[128];
  char arch[64];                /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
} rt_props;

typedef struct rt_module_s *rt_module;
typedef struct rt_kernel_s *rt_kernel;
typedef struct rt_event_s *rt_event;

/* Selects `device`, creates its context and loads the built-in code objects.
 * Idempotent.  Replaces torch.nexus.get_device / set_runtime
 * (backend/driver.py:462-468). */
TTAMD_API int rt_init(int device);
TTAMD_API int rt_device_count(int *count);
TTAMD_API int rt_device_props(rt_props *out);

/* Raw device memory for callers without torch (C++ benches, tests).
 * kind: 0 host->host, 1 host->device, 2 device->host, 3 device->device. */
TTAMD_API int rt_malloc(void **ptr, size_t bytes);
TTAMD_API int rt_free(void *ptr);
TTAMD_API int rt_memcpy(void *dst, const void *src, size_t bytes, int kind);
TTAMD_API int rt_memset(void *dst, int value, size_t bytes, void *stream);

/* Code objects.  rt_module_load takes a gfx950 code object image in memory
 * (device.load_library, backend/driver.py:72); rt_builtin_module returns one of
 * the images embedded in this library ("elementwise", "gemm", "attention", "reduce"). */
TTAMD_API int rt_module_load(const void *image, size_t bytes, rt_module *out);
TTAMD_API int rt_module_unload(rt_module m);
TTAMD_API int rt_builtin_module(const char *which, rt_module *out);
/* lib.get_kernel(name) (backend/driver.py:73): a device symbol of module m. */
TTAMD_API int rt_get_kernel(rt_module m, const char *name, rt_kernel *out);
/* command.set_arg... + finalize(grid, block, shared) + schedule.run()
 * (backend/driver.py:117-168), asynchronous on `stream`.  args[i] points at
 * the i-th kernel parameter value. */
TTAMD_API int rt_launch(rt_kernel k, const uint32_t grid[3], const uint32_t block[3],
              uint32_t shared_bytes, void *stream, void **args, size_t nargs);
TTAMD_API int rt_sync(void *stream);

/* hipEvent timing: the device-side counterpart of TTDeviceInterface.Event
 * (backend/driver.py:390-442). */
TTAMD_API int rt_event_create(rt_event *out);
TTAMD_API int rt_event_record(rt_event e, void *stream);
TTAMD_API int rt_event_sync(rt_event e);
TTAMD_API int rt_event_elapsed_ms(rt_event start, rt_event stop, float *ms);
TTAMD_API int rt_event_destroy(rt_event e);

TTAMD_API const char *rt_last_error(void);

/* ----------------------------------------------------------------------- */
/* tt_*: the example kernels                                                */
/* ----------------------------------------------------------------------- */

/* A rank-2 host tensor descriptor as the launcher flattens it:
 * base, shape..., strides..., padding flag (backend/driver.py:141-159, 322-329;
 * device-side type list test/Tenstorrent/dot_op_to_ttkernel.mlir:412).
 * Strides are in elements; the last stride must be 1. */
typedef struct tt_desc2d {
  void *base;
  int32_t shape[2];
  int64_t strides[2];
  int32_t block_shape[2];
  int32_t padding_nan; /* 1 if padding == "nan" (driver.py:326): elements outside the matrix read as NaN (matmul
                          operands; meaningless on outputs; refused by tt_attn_fwd) */
  int32_t dtype;       /* tt_dtype */
} tt_desc2d;

/* Epilogues of the fused tile matmul. */
typedef enum tt_epilogue {
  TT_EPI_NONE = 0,
  /* c = acc.to(half) + bias[M,N], added in the half type
   * (python/tutorials/09-matmul-fused.py:139-146) */
  TT_EPI_BIAS_FULL = 1,
  /* c = (gelu_erf(acc + bias[n])).to(half), epilogue in fp32 on the accumulator
   * (no counterpart in the reference; placement follows the leaky_relu
   * precedent examples/matmul/03-matrix-multiplication.py:370-374) */
  TT_EPI_BIAS_ROW_GELU = 2,
  /* c = leaky_relu(acc).to(half) (03-matrix-multiplication.py:370-374,393-395) */
  TT_EPI_LEAKY_RELU = 3,
  /* c = (acc + bias[n]).to(half) */
  TT_EPI_BIAS_ROW = 4
} tt_epilogue;

/* add_kernel(x_ptr, y_ptr, output_ptr, n_elements, BLOCK_SIZE)
 * python/tutorials/01-vector-add.py:29-54.  dtype TT_F32 or TT_I32.
 * Programs 0..grid[0]-1 each own BLOCK_SIZE consecutive elements; lanes at or
 * past n_elements are masked, elements past grid[0]*BLOCK_SIZE are untouched. */
TTAMD_API int tt_add_kernel(const void *x, const void *y, void *out, int32_t n_elements,
                  int32_t BLOCK_SIZE, int32_t dtype, const uint32_t grid[3], void *stream);

/* add_kernel(x_ptr, y_ptr, output_ptr, n_elements, row_count, BLOCK_SIZE)
 * python/tutorials/01-vector-add.loop.py:30-62: program pid owns
 * [pid*BLOCK_SIZE*row_count, min(.. + BLOCK_SIZE*row_count, n_elements)). */
TTAMD_API int tt_add_kernel_loop(const void *x, const void *y, void *out, int32_t n_elements,
                       int32_t row_count, int32_t BLOCK_SIZE, int32_t dtype,
                       const uint32_t grid[3], void *stream);

/* muladd_kernel(x_ptr, y_ptr, z_ptr, output_ptr, n_elements, BLOCK_SIZE)
 * python/tutorials/01-vector-mul-add.py:30-57; fp32, x*y+z contracted to one
 * fused multiply-add (enable_fp_fusion default, backend/compiler.py:29). */
TTAMD_API int tt_muladd_kernel(const void *x, const void *y, const void *z, void *out,
                     int32_t n_elements, int32_t BLOCK_SIZE, const uint32_t grid[3],
                     void *stream);

/* sin_kernel(x_ptr, output_ptr, n_elements, BLOCK_SIZE)
 * examples/01-sin-kernel.py:17-29; fp32. */
TTAMD_API int tt_sin_kernel(const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE,
                  const uint32_t grid[3], void *stream);

/* The elementwise operations the reference's compute lowering accepts
 * (npu/lib/Dialect/TritonTenstorrent/Transforms/ConvertComputeOps.cpp:162-182), each as
 * a kernel of the same masked-block form as sin_kernel / add_kernel: program pid owns
 * BLOCK_SIZE consecutive fp32 elements, lanes at or past n_elements are masked.
 *   unary (math.absf ceil cos exp exp2 floor log log2 rsqrt sin sqrt):  out[i] = op(x[i])
 *   binary (arith.addf subf mulf divf maximumf minimumf):              out[i] = x[i] op y[i]
 *   narrowing (arith.truncf fp32 -> bf16 / fp16, round to nearest even;
 *              arith.trunci int32 -> int16 / int8, low bits kept)
 * abs, ceil, floor, sqrt, the four arithmetic operations and the casts are exact
 * (correctly rounded); maximum / minimum return NaN if either operand is NaN and
 * order -0 below +0; the transcendental ones are within 2 ulp of the exact result. */
typedef enum tt_unary_op {
  TT_OP_ABS = 0, TT_OP_CEIL = 1, TT_OP_COS = 2, TT_OP_EXP = 3, TT_OP_EXP2 = 4, TT_OP_FLOOR = 5,
  TT_OP_LOG = 6, TT_OP_LOG2 = 7, TT_OP_RSQRT = 8, TT_OP_SIN = 9, TT_OP_SQRT = 10
} tt_unary_op;
typedef enum tt_binary_op {
  TT_OP_ADD = 0, TT_OP_SUB = 1, TT_OP_MUL = 2, TT_OP_DIV = 3, TT_OP_MAXIMUM = 4, TT_OP_MINIMUM = 5
} tt_binary_op;
TTAMD_API int tt_unary_kernel(int32_t op, const void *x, void *out, int32_t n_elements,
                    int32_t BLOCK_SIZE, const uint32_t grid[3], void *stream);
TTAMD_API int tt_binary_kernel(int32_t op, const void *x, const void *y, void *out, int32_t n_elements,
                     int32_t BLOCK_SIZE, const uint32_t grid[3], void *stream);
/* The same with one operand a compile-time constant of the kernel: out[i] = x[i] OP c, or c OP x[i] when flip
 * is set.  x and out may be the same buffer.  With BLOCK_SIZE = 1 and n_elements = grid[0] this is the
 * one-element-per-program form of test_core.py::test_load_store_same_ptr (x = load(p + pid); store(p + pid, x * 2)),
 * which the reference's CI runs beside test_reduce1d (.github/workflows/integration-tests-cpu.yml:105). */
TTAMD_API int tt_binary_const_kernel(int32_t op, const void *x, float c, int32_t flip, void *out, int32_t n_elements,
                           int32_t BLOCK_SIZE, const uint32_t grid[3], void *stream);
TTAMD_API int tt_cast_kernel(const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE,
                   int32_t in_dtype, int32_t out_dtype, const uint32_t grid[3], void *stream);
/* out[i] = x[i] for i < n_elements: the masked block loaded and stored back unchanged, the kernel that
 * test_launch.py::test_memory_leak launches in the reference's CI (.github/workflows/integration-tests-cpu.yml:106;
 * masked load and store: cpu/lib/TritonCPUToLLVM/MaskedOpsToLLVM.cpp:33-114).  dtype is any tt_dtype; the copy is
 * by bytes.  x and out must be aligned to the element and must not overlap unless they are equal. */
TTAMD_API int tt_copy_kernel(const void *x, void *out, int32_t n_elements, int32_t BLOCK_SIZE, int32_t dtype,
                   const uint32_t grid[3], void *stream);

/* kernel(X, Z, BLOCK): x = tl.load(X + tl.arange(0, BLOCK)); tl.store(Z, tl.<op>(x, axis=0))
 * The single-block reductions the reference's CI runs on its cpu/ path
 * (.github/workflows/integration-tests-cpu.yml:105, test_core.py::test_reduce1d; cross-lane lowering
 * cpu/lib/TritonCPUToLLVM/TargetInfo.cpp:95-225): sum, min, max, argmin, argmax, xor_sum over BLOCK
 * elements of in_dtype (any of tt_dtype but fp8), 1 <= BLOCK <= 1048576.
 * acc_dtype is the element type the tt.reduce of the IR runs in (i8 sums in i32, bf16 max in fp32 ...):
 * integer sum / xor_sum wrap at that width and min / max are exact; float sums are carried in fp32
 * (fp64 for f64) in tree order, so they agree with any other order only to rounding.
 * out_dtype is Z's element type: acc_dtype or narrower (truncation / one RNE rounding); i32 or i64
 * for the index of argmin / argmax, which is the smallest index attaining the extremum
 * (tie_break_left; without it any such index is a legal result).  Float min / max drop NaN operands
 * (arith.minnumf / maxnumf) unless propagate_nan (arith.minimumf / maximumf); the index reductions
 * on NaN input return an index that depends on the fold order, as the reference's do.
 * Every program of the grid would store the same value; it is computed once.  Blocks of 128 KiB and more
 * (16-byte aligned) are folded by several workgroups through a small device buffer that the library keeps
 * per (device, stream): the first such call on a stream allocates it (hipMalloc, 4352 bytes), calls on
 * different streams do not share it, and rt_release_stream frees it.  A call on a stream that is recording a
 * graph never uses that buffer, whether it exists or not: it runs as one workgroup, so a recorded graph holds
 * no address of the library's and may be replayed on any stream beside eager calls. */
typedef enum tt_reduce_op {
  TT_REDUCE_SUM = 0, TT_REDUCE_MIN = 1, TT_REDUCE_MAX = 2, TT_REDUCE_ARGMIN = 3, TT_REDUCE_ARGMAX = 4,
  TT_REDUCE_XOR_SUM = 5
} tt_reduce_op;
TTAMD_API int tt_reduce1d_kernel(int32_t op, const void *x, void *z, int32_t BLOCK, int32_t in_dtype,
                       int32_t acc_dtype, int32_t out_dtype, int32_t propagate_nan,
                       const uint32_t grid[3], void *stream);
/* Frees what the library allocated for `stream` on the current device (the buffer above and the workspace of
 * tt_matmul_kernel_tma / _fused, below), after waiting for the stream; call it before destroying a stream that ran
 * large reductions or matmuls of few tiles.  No counterpart in the reference. */
TTAMD_API int rt_release_stream(void *stream);
/* The same reductions, same arguments and results, for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  It calls no hipMalloc / hipFree at any time: the partial results of a block folded by several
 * workgroups live in a 4352-byte device array that is part of the library's own image (one copy on every GPU the
 * library runs on, for the life of the process), and its kernels are resolved by rt_init.  BLOCK beyond 1048576
 * elements is refused (RT_ERR_INVALID).  Every call on a GPU shares that GPU's array: calls that may run at the
 * same time on one GPU (two streams, or two graphs replayed side by side) race and must be ordered by the
 * caller; calls on one stream, eager or replayed, are ordered already.  Recorded into a graph it keeps the
 * several-workgroup form (tt_reduce1d_kernel records one workgroup). */
TTAMD_API int tt_reduce1d_kernel_noalloc(int32_t op, const void *x, void *z, int32_t BLOCK, int32_t in_dtype,
                               int32_t acc_dtype, int32_t out_dtype, int32_t propagate_nan,
                               const uint32_t grid[3], void *stream);

/* matmul_kernel_tma(a_desc, b_desc, c_desc, M, N, K, BLOCK_SIZE_M, BLOCK_SIZE_N,
 *                   BLOCK_SIZE_K, GROUP_SIZE_M, FP8_OUTPUT, WARP_SPECIALIZE)
 * examples/matmul_tensor_descriptor/09-persistent-matmul.py:102-145.
 * A [M,K] and B [K,N] (not transposed) row-major, fp32 accumulate, one
 * round-to-nearest-even cast to c->dtype.  grid[0] logical programs, one per
 * BLOCK_SIZE_M x BLOCK_SIZE_N tile in GROUP_SIZE_M-swizzled order.
 * A launch with a 16-bit result (this entry point, _fused, _fp8_scaled and tt_matmul_kernel) whose C has few 256x256 tiles under a long K (at most half the CUs
 * busy even with 64-row pieces of tiles, K a multiple of 256, of 512 for fp8) is computed in slices of K: the slices' fp32 sums pass
 * through a workspace of at most 64 MiB that the library keeps per (device, stream), allocated by the first such
 * call on the stream (hipMalloc), grown by a call that needs more (the stream is drained first) and freed by
 * rt_release_stream; the sums are added in slice order, so results do not change from launch to launch, and the
 * epilogue is applied to the whole sum.  A call on a stream that is recording a graph never takes that route. */
TTAMD_API int tt_matmul_kernel_tma(const tt_desc2d *a, const tt_desc2d *b, const tt_desc2d *c,
                         int32_t M, int32_t N, int32_t K, int32_t BLOCK_SIZE_M,
                         int32_t BLOCK_SIZE_N, int32_t BLOCK_SIZE_K, int32_t GROUP_SIZE_M,
                         const uint32_t grid[3], void *stream);

/* matmul_kernel_fused(a_desc, b_desc, c_desc, bias_desc, M, N, K, ...)
 * python/tutorials/09-matmul-fused.py:100-148.  `epilogue` is a tt_epilogue;
 * TT_EPI_BIAS_FULL is the reference kernel, the row-bias forms take a bias
 * descriptor of shape [1,N] (or [N,1] viewed as such) holding fp32. */
TTAMD_API int tt_matmul_kernel_fused(const tt_desc2d *a, const tt_desc2d *b, const tt_desc2d *c,
                           const tt_desc2d *bias, int32_t M, int32_t N, int32_t K,
                           int32_t BLOCK_SIZE_M, int32_t BLOCK_SIZE_N, int32_t BLOCK_SIZE_K,
                           int32_t GROUP_SIZE_M, int32_t epilogue, const uint32_t grid[3],
                           void *stream);

/* matmul_kernel_tma with fp8 e4m3 descriptors and two per-tensor fp32 scales:
 * c = (acc * scale_a * scale_b).to(c->dtype).  The reference has fp8 inputs
 * (09-persistent-matmul.py:116,173) but no scales; this sibling name is new. */
TTAMD_API int tt_matmul_kernel_tma_fp8_scaled(const tt_desc2d *a, const tt_desc2d *b,
                                    const tt_desc2d *c, int32_t M, int32_t N, int32_t K,
                                    float scale_a, float scale_b, int32_t BLOCK_SIZE_M,
                                    int32_t BLOCK_SIZE_N, int32_t BLOCK_SIZE_K,
                                    int32_t GROUP_SIZE_M, const uint32_t grid[3],
                                    void *stream);

/* matmul_kernel(a_ptr, b_ptr, c_ptr, M, N, K, stride_am, stride_ak, stride_bk,
 *               stride_bn, stride_cm, stride_cn, BLOCK_SIZE_M, BLOCK_SIZE_N,
 *               BLOCK_SIZE_K, GROUP_SIZE_M, ACTIVATION)
 * examples/matmul/03-matrix-multiplication.py:242-391 (wrapper :403-421): the
 * pointer-based kernel.  a, b and c are TILE-MAJOR buffers with tiles of
 * BLOCK_M x BLOCK_K, BLOCK_K x BLOCK_N and BLOCK_M x BLOCK_N elements, row-major
 * inside a tile, tiles in row-major order (:326-337, 349-357, 377-385); ragged
 * edges need the buffers padded to whole tiles; what the padding holds does not
 * matter (elements past K are masked to zero as in the kernel, :340-342, 359-361;
 * rows past M and columns past N only feed results that are never stored, and
 * the padding of c is never written).  The strides are checked to be
 * positive, as the kernel asserts, and otherwise unused, as in the kernel.
 * in_dtype is TT_F16 or TT_BF16; c is always fp16 (:374).  leaky_relu != 0
 * applies ACTIVATION == "leaky_relu" to the fp32 accumulator (:370-373, 396-397). */
TTAMD_API int tt_matmul_kernel(const void *a_ptr, const void *b_ptr, void *c_ptr, int32_t M, int32_t N,
                     int32_t K, int64_t stride_am, int64_t stride_ak, int64_t stride_bk,
                     int64_t stride_bn, int64_t stride_cm, int64_t stride_cn, int32_t BLOCK_SIZE_M,
                     int32_t BLOCK_SIZE_N, int32_t BLOCK_SIZE_K, int32_t GROUP_SIZE_M,
                     int32_t leaky_relu, int32_t in_dtype, const uint32_t grid[3], void *stream);

/* _attn_fwd(sm_scale, M, Z, H, desc_q, desc_k, desc_v, desc_o, N_CTX, HEAD_DIM,
 *           BLOCK_M, BLOCK_N, FP8_OUTPUT, STAGE, warp_specialize, IS_HOPPER)
 * examples/fused-attn/06-fused-attention.py:143-215.  bf16 descriptors of shape
 * [Z*H*N_CTX, HEAD_DIM]; M receives m_i + log2(l_i); STAGE 3 = causal, 1 = full;
 * grid = (cdiv(N_CTX, BLOCK_M), Z*H, 1).
 * Numerics are the source's (qk_scale = sm_scale * 1.44269504, exp2, l_ij summed
 * in fp32 before P is rounded to bf16, fp32 accumulation), with two stated
 * differences from a literal evaluation, both inside the tolerance the parity
 * tests state (O within 2e-2, M within 1e-3 of the source's values):
 *  - the exponent reference m_i of a row follows the running maximum lazily: a
 *    new block maximum replaces it only when some row of its 32-query tile
 *    exceeds it by more than 8 (log2 units).  Until then p = exp2(s - m_i) may
 *    reach 2^8 instead of 1; l_i and the accumulator carry the same factor, so
 *    O = acc / l_i and M = m_i + log2(l_i) are those of the true maximum up to
 *    fp32 rounding;
 *  - keys are taken in blocks of 64 whatever BLOCK_N says (fp32 summation order
 *    only), and the causal mask is evaluated as the source does at BLOCK_M = 32:
 *    -1.0e6 is added to masked scores inside the 32x32 tile on the diagonal and
 *    keys past it are not visited.  At a larger BLOCK_M the source adds -1.0e6
 *    to those as well; exp2 of that is exactly 0 unless a score exceeds 1e6, so
 *    the results differ only for such scores. */
TTAMD_API int tt_attn_fwd(float sm_scale, float *M, int32_t Z, int32_t H, const tt_desc2d *desc_q,
                const tt_desc2d *desc_k, const tt_desc2d *desc_v, const tt_desc2d *desc_o,
                int32_t N_CTX, int32_t HEAD_DIM, int32_t BLOCK_M, int32_t BLOCK_N,
                int32_t STAGE, const uint32_t grid[3], void *stream);

/* Diagnostic, no counterpart in the reference: what core clock does the part grant under the 16-bit macro-tile GEMM?
 * arm != 0 makes the NEXT launch of that kernel (tt_matmul_kernel_tma / _fused on a shape of whole 256x256x128 macro
 * tiles) synchronous and records workgroup 0's core-clock cycles and the 100 MHz wall ticks of its run; reading
 * (may be null) receives the last record, {0, 0} when there is none: clock in GHz = reading[0] / reading[1] / 10.
 * The kernels are bounded by power, so their rate follows this clock, which differs from box to box. */
TTAMD_API int rt_gemm_clock_probe(int32_t arm, uint64_t reading[2]);

/* Name of the device kernel the last tt_* call on this thread launched (for
 * profiles and tests that assert which path ran). */
TTAMD_API const char *tt_last_kernel_name(void);

#ifdef __cplusplus
}
#endif
#endif /* TTAMD_RT_H */
