// Single-block reductions over a 1-D tensor: the kernel form
//   x = tl.load(X + tl.arange(0, BLOCK)); tl.store(Z, tl.<op>(x, axis=0))
// that the reference's CI runs on its cpu/ path (.github/workflows/integration-tests-cpu.yml:105,
// test_core.py::test_reduce1d; lowering of the cross-lane steps: cpu/lib/TritonCPUToLLVM/TargetInfo.cpp:95-225).
//
// One workgroup of 1024 lanes (up to 256 of them for blocks of 128 KiB and more, see reduce_body): each lane folds a strided share of the elements, 64 lanes fold with
// __shfl_xor, the sixteen wavefronts fold through LDS, lane 0 stores.  Integers are carried in 64 bits
// (sum and xor wrap, so truncating the 64-bit result to the accumulator width of the IR gives that
// width's wraparound result; min/max compare exactly); f16/bf16/f32 are carried in fp32, f64 in fp64.
// The arg-reductions and the value of min/max with indices order (value, index) pairs by value, then
// by the smaller index, which is the tie_break_left combine of triton/language/standard.py and one
// of the legal results without it.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace {

enum Op : int { SUM = 0, MIN = 1, MAX = 2, ARGMIN = 3, ARGMAX = 4, XOR = 5 };
constexpr int kLanes = 1024;
constexpr int kAhead = 8;    // loads a lane issues before it folds them

struct bf16_t { uint16_t bits; };
struct f16_t { __half h; };

template <typename T> struct Carry;   // type a lane folds in
template <> struct Carry<int8_t> { using type = int64_t; };
template <> struct Carry<int16_t> { using type = int64_t; };
template <> struct Carry<int32_t> { using type = int64_t; };
template <> struct Carry<int64_t> { using type = int64_t; };
template <> struct Carry<uint8_t> { using type = uint64_t; };
template <> struct Carry<uint16_t> { using type = uint64_t; };
template <> struct Carry<uint32_t> { using type = uint64_t; };
template <> struct Carry<uint64_t> { using type = uint64_t; };
template <> struct Carry<float> { using type = float; };
template <> struct Carry<bf16_t> { using type = float; };
template <> struct Carry<f16_t> { using type = float; };
template <> struct Carry<double> { using type = double; };

template <typename T> __device__ __forceinline__ typename Carry<T>::type widen(T v) { return (typename Carry<T>::type)v; }
template <> __device__ __forceinline__ float widen<bf16_t>(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }
template <> __device__ __forceinline__ float widen<f16_t>(f16_t v) { return __half2float(v.h); }

template <typename C> struct Pair { C v; int32_t i; };   // i < 0: empty

template <typename C> __device__ __forceinline__ C num_max(C a, C b) { return a > b ? a : b; }
template <typename C> __device__ __forceinline__ C num_min(C a, C b) { return a < b ? a : b; }
// arith.maxnumf / minnumf: a NaN operand is dropped.  nan_mode != 0 selects arith.maximumf / minimumf.
template <> __device__ __forceinline__ float num_max<float>(float a, float b) { return fmaxf(a, b); }
template <> __device__ __forceinline__ float num_min<float>(float a, float b) { return fminf(a, b); }
template <> __device__ __forceinline__ double num_max<double>(double a, double b) { return fmax(a, b); }
template <> __device__ __forceinline__ double num_min<double>(double a, double b) { return fmin(a, b); }

template <typename C> __device__ __forceinline__ bool is_nan(C) { return false; }
template <> __device__ __forceinline__ bool is_nan<float>(float v) { return v != v; }
template <> __device__ __forceinline__ bool is_nan<double>(double v) { return v != v; }

template <int op, typename C> __device__ __forceinline__ C fold_value(bool nan_mode, C a, C b) {
  switch (op) {
  case SUM:
    if constexpr (__is_floating_point(C)) return a + b;
    else return (C)((uint64_t)a + (uint64_t)b);   // wraps; no signed overflow
  case XOR:
    if constexpr (sizeof(C) == 8 && !__is_floating_point(C)) return a ^ b;
    else return a;
  case MIN:
    if (nan_mode && (is_nan(a) || is_nan(b))) return is_nan(a) ? a : b;
    return num_min(a, b);
  default:
    if (nan_mode && (is_nan(a) || is_nan(b))) return is_nan(a) ? a : b;
    return num_max(a, b);
  }
}

template <int op, typename C> __device__ __forceinline__ Pair<C> fold(bool nan_mode, Pair<C> a, Pair<C> b) {
  if (b.i < 0) return a;
  if (a.i < 0) return b;
  if (op == ARGMIN || op == ARGMAX) {
    const bool first = (op == ARGMIN ? a.v < b.v : a.v > b.v) || (a.v == b.v && a.i < b.i);
    return first ? a : b;
  }
  return Pair<C>{fold_value<op>(nan_mode, a.v, b.v), 0};
}

template <typename C> __device__ __forceinline__ Pair<C> shuffle_xor(Pair<C> p, int m) {
  Pair<C> r;
  if constexpr (sizeof(C) == 8) {
    union { C c; int32_t w[2]; } u, o;
    u.c = p.v;
    o.w[0] = __shfl_xor(u.w[0], m, 64);
    o.w[1] = __shfl_xor(u.w[1], m, 64);
    r.v = o.c;
  } else {
    r.v = __shfl_xor(p.v, m, 64);
  }
  r.i = __shfl_xor(p.i, m, 64);
  return r;
}

template <typename C> __device__ __forceinline__ void store_value(void *z, int out_bytes, int out_kind, C v) {
  // out_kind: 0 integer of out_bytes, 1 f32, 2 bf16 (RNE), 3 f16 (RNE), 4 f64
  if constexpr (__is_floating_point(C)) {
    if (out_kind == 4) *(double *)z = (double)v;
    else if (out_kind == 1) *(float *)z = (float)v;
    else if (out_kind == 3) *(__half *)z = __float2half_rn((float)v);
    else {
      const float f = (float)v;
      uint32_t u = __float_as_uint(f);
      if (f != f) u = 0x7fc00000u;
      else u += 0x7fffu + ((u >> 16) & 1u);
      *(uint16_t *)z = (uint16_t)(u >> 16);
    }
  } else {
    const uint64_t u = (uint64_t)v;
    if (out_bytes == 1) *(uint8_t *)z = (uint8_t)u;
    else if (out_bytes == 2) *(uint16_t *)z = (uint16_t)u;
    else if (out_bytes == 4) *(uint32_t *)z = (uint32_t)u;
    else *(uint64_t *)z = u;
  }
}

// out_bytes is never wider than the integer accumulator of the IR (the host checks), so storing the
// low out_bytes of the 64-bit result is that accumulator's wraparound result, truncated as the IR does.
template <typename T, int op>
__device__ __forceinline__ void reduce_body(const T *__restrict__ x, void *__restrict__ z, int n, int nan_mode,
                                            int out_bytes, int out_kind, void *scratch, unsigned *counter) {
  using C = typename Carry<T>::type;
  __shared__ Pair<C> part[kLanes / 64];
  const int tid = threadIdx.x;
  const int G = (int)gridDim.x, b = (int)blockIdx.x;
  Pair<C> p{C(0), -1};
  // 16-byte loads when X is 16-byte aligned: kAhead of them per lane are issued before the first fold
  // waits on one; the ragged end (and an unaligned X) goes element by element.
  // With more than one workgroup (large blocks on an aligned X) the vectors are dealt in contiguous runs, the
  // ragged end goes to the last workgroup, every workgroup leaves its partial result in `scratch`, and the one
  // that finishes last folds the partials in workgroup order and stores.
  constexpr int kPer = 16 / (int)sizeof(T);
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
  int lo = 0, hi = n;
  if (G > 1) {
    const int nvec = n / kPer, per = (nvec + G - 1) / G;
    lo = min(b * per, nvec) * kPer;
    hi = b == G - 1 ? n : min((b + 1) * per, nvec) * kPer;
  }
  int done = lo;
  if (vec) {
    const uint4 *xv = reinterpret_cast<const uint4 *>(x);
    const int vend = hi / kPer;
    int j = lo / kPer + tid;
    for (; j + (kAhead - 1) * kLanes < vend; j += kAhead * kLanes) {
      union { uint4 q; T e[kPer]; } v[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) v[u].q = xv[j + u * kLanes];
#pragma unroll
      for (int u = 0; u < kAhead; ++u)
#pragma unroll
        for (int e = 0; e < kPer; ++e)
          p = fold<op>(nan_mode != 0, p, Pair<C>{widen<T>(v[u].e[e]), (j + u * kLanes) * kPer + e});
    }
    if (j < vend) {   // fewer than kAhead vectors left for this lane: again all loads first
      union { uint4 q; T e[kPer]; } v[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead - 1; ++u)
        if (j + u * kLanes < vend) v[u].q = xv[j + u * kLanes];
#pragma unroll
      for (int u = 0; u < kAhead - 1; ++u)
        if (j + u * kLanes < vend) {
#pragma unroll
          for (int e = 0; e < kPer; ++e)
            p = fold<op>(nan_mode != 0, p, Pair<C>{widen<T>(v[u].e[e]), (j + u * kLanes) * kPer + e});
        }
    }
    done = vend * kPer;
  }
  for (int i = done + tid; i < hi; i += kLanes) p = fold<op>(nan_mode != 0, p, Pair<C>{widen<T>(x[i]), i});
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) p = fold<op>(nan_mode != 0, p, shuffle_xor(p, m));
  if ((tid & 63) == 0) part[tid >> 6] = p;
  __syncthreads();
  if (tid == 0)
    for (int w = 1; w < kLanes / 64; ++w) p = fold<op>(nan_mode != 0, p, part[w]);
  if (G > 1) {
    // the workgroup's result goes to its slot; the workgroup that takes the last ticket folds all the slots,
    // one per lane, the same way
    __shared__ int last;
    volatile Pair<C> *slots = (volatile Pair<C> *)scratch;
    if (tid == 0) {
      slots[b].v = p.v;
      slots[b].i = p.i;
      __threadfence();                                   // the partial is visible before the ticket is taken
      // the counter wraps to zero by itself with the G-th ticket, so it is ready for the next launch that uses it
      last = atomicInc(counter, (unsigned)(G - 1)) == (unsigned)(G - 1);
    }
    __syncthreads();
    if (!last) return;
    __threadfence();
    p = Pair<C>{C(0), -1};
    if (tid < G) {
      p.v = slots[tid].v;
      p.i = slots[tid].i;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) p = fold<op>(nan_mode != 0, p, shuffle_xor(p, m));
    if ((tid & 63) == 0) part[tid >> 6] = p;
    __syncthreads();
    if (tid == 0)
      for (int w = 1; w < kLanes / 64; ++w) p = fold<op>(nan_mode != 0, p, part[w]);
  }
  if (tid == 0) {
    if (op == ARGMIN || op == ARGMAX) {
      if (out_bytes == 8) *(int64_t *)z = p.i;
      else *(int32_t *)z = p.i;
    } else {
      store_value<C>(z, out_bytes, out_kind, p.v);
    }
  }
}

} // namespace

#define REDUCE_KERNEL(name, T)                                                                                        \
  extern "C" __global__ __launch_bounds__(kLanes) void name(const void *x, void *z, int n, int op, int nan_mode,     \
                                                             int out_bytes, int out_kind, void *scratch,        \
                                                             unsigned *counter) {                                    \
    switch (op) {                                                                                                     \
    case SUM: reduce_body<T, SUM>((const T *)x, z, n, nan_mode, out_bytes, out_kind, scratch, counter); break; \
    case MIN: reduce_body<T, MIN>((const T *)x, z, n, nan_mode, out_bytes, out_kind, scratch, counter); break; \
    case MAX: reduce_body<T, MAX>((const T *)x, z, n, nan_mode, out_bytes, out_kind, scratch, counter); break; \
    case ARGMIN: reduce_body<T, ARGMIN>((const T *)x, z, n, nan_mode, out_bytes, out_kind, scratch, counter); break; \
    case ARGMAX: reduce_body<T, ARGMAX>((const T *)x, z, n, nan_mode, out_bytes, out_kind, scratch, counter); break; \
    default: reduce_body<T, XOR>((const T *)x, z, n, nan_mode, out_bytes, out_kind, scratch, counter); break; \
    }                                                                                                                 \
  }

// Puts the arrival counter of a buffer of partial results back to zero (a kernel rather than a memset, so that it
// can be recorded into a graph).
extern "C" __global__ __launch_bounds__(64) void reduce1d_clear_counter(unsigned *counter) {
  if (threadIdx.x == 0) *counter = 0u;
}

REDUCE_KERNEL(reduce1d_i8, int8_t)
REDUCE_KERNEL(reduce1d_i16, int16_t)
REDUCE_KERNEL(reduce1d_i32, int32_t)
REDUCE_KERNEL(reduce1d_i64, int64_t)
REDUCE_KERNEL(reduce1d_u8, uint8_t)
REDUCE_KERNEL(reduce1d_u16, uint16_t)
REDUCE_KERNEL(reduce1d_u32, uint32_t)
REDUCE_KERNEL(reduce1d_u64, uint64_t)
REDUCE_KERNEL(reduce1d_f32, float)
REDUCE_KERNEL(reduce1d_bf16, bf16_t)
REDUCE_KERNEL(reduce1d_f16, f16_t)
REDUCE_KERNEL(reduce1d_f64, double)
