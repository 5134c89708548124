// Shared device/host helpers for the gfx950 kernels (wave64, CDNA4).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <limits>
#include <type_traits>

#include "../../include/fast_rnnt_amd.h"

namespace frnnt {

constexpr int kWave = 64;

// ---- host side: thread-local error text --------------------------------------
char *error_buffer();
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);
// Makes `bytes` of dynamic LDS available to `kernel` on the current device (needed
// above 64 KB); remembers what it has granted, so the runtime is asked once.
bool allow_lds(const void *kernel, size_t bytes);

// ---- device side -----------------------------------------------------------------
template <typename R>
struct Num;

template <>
struct Num<float> {
  static __device__ __forceinline__ float neg_inf() { return -__builtin_huge_valf(); }
  // v_exp_f32 / v_log_f32 based; absolute error of log1p(exp(d)) stays below
  // 1e-7 for d <= 0, far under one ulp of lattice scores of magnitude >= 1.
  static __device__ __forceinline__ float exp_(float x) { return __expf(x); }
  static __device__ __forceinline__ float log1p_(float x) { return __logf(1.0f + x); }
};

template <>
struct Num<double> {
  static __device__ __forceinline__ double neg_inf() { return -__builtin_huge_val(); }
  static __device__ __forceinline__ double exp_(double x) { return exp(x); }
  static __device__ __forceinline__ double log1p_(double x) { return log1p(x); }
};

// ---- 2-byte floating-point storage (float16, bfloat16): memory holds the 16-bit
// patterns, arithmetic is float32; stores round to nearest even.
struct HalfIO {
  static __device__ __forceinline__ float load(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
  }
  static __device__ __forceinline__ uint16_t store(float f) {
    const _Float16 v = (_Float16)f;  // round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
  }
};
struct Bf16IO {
  static __device__ __forceinline__ float load(uint16_t h) {
    return __uint_as_float((unsigned)h << 16);
  }
  static __device__ __forceinline__ uint16_t store(float f) {
    const unsigned u = __float_as_uint(f);
    if (f != f) return (uint16_t)((u >> 16) | 0x0040u);        // stays a NaN
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);  // round to nearest even
  }
};

// A 2-byte element as a value type, for templates written over the element type: converts
// to and from float, the arithmetic happens in AccOf<...>::type.
template <typename IO>
struct Narrow {
  uint16_t bits;
  Narrow() = default;
  __device__ __forceinline__ Narrow(float f) : bits(IO::store(f)) {}
  __device__ __forceinline__ operator float() const { return IO::load(bits); }
};
using f16_t = Narrow<HalfIO>;
using bf16_t = Narrow<Bf16IO>;
template <typename R>
struct AccOf {
  typedef R type;
};
template <typename IO>
struct AccOf<Narrow<IO>> {
  typedef float type;
};

// log(exp(a) + exp(b)) with the reference's handling of non-finite operands
// (fast_rnnt/csrc/mutual_information.h:36-65): the larger operand is returned
// untouched when the difference is not a finite number.
template <typename R>
__device__ __forceinline__ R log_add(R a, R b) {
  const bool lt = a < b;
  const R hi = lt ? b : a;
  const R gap = lt ? (a - b) : (b - a);
  if (gap - gap != 0) return hi;
  return hi + Num<R>::log1p_(Num<R>::exp_(gap));
}

// Whole-wave shift right by one (DPP wave_shr:1, a full-rate VALU modifier on
// gfx9-family parts, no LDS trip): lane L receives the value held by lane L-1.
// With lane 0 receiving 0 the compiler can fold the
// shift into the consuming VALU instruction.
__device__ __forceinline__ float from_lane_below_zero(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x138, 0xf, 0xf, true));
}
__device__ __forceinline__ double from_lane_below_zero(double v) {
  const long long vi = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_update_dpp(0, (int)(vi & 0xffffffffLL), 0x138, 0xf, 0xf, true);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(vi >> 32), 0x138, 0xf, 0xf, true);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// Shift right by one in which lane 0 keeps the value it holds in `first` (a DPP move
// leaves lanes without a source lane at their old contents).
__device__ __forceinline__ float from_lane_below_or(float v, float first) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(first), __float_as_int(v),
                                                    0x138, 0xf, 0xf, false));
}
__device__ __forceinline__ double from_lane_below_or(double v, double first) {
  const long long vi = __double_as_longlong(v), fi = __double_as_longlong(first);
  const int lo = __builtin_amdgcn_update_dpp((int)(fi & 0xffffffffLL), (int)(vi & 0xffffffffLL),
                                             0x138, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp((int)(fi >> 32), (int)(vi >> 32), 0x138, 0xf, 0xf,
                                             false);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// The value one lane holds, for all lanes (the lane index is wave-uniform).
__device__ __forceinline__ float read_lane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ double read_lane(double v, int lane) {
  const long long vi = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_readlane((int)(vi & 0xffffffffLL), lane);
  const int hi = __builtin_amdgcn_readlane((int)(vi >> 32), lane);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// Value held by lane+1 (whole-wave shift left by one, DPP wave_shl:1); lane 63 receives 0.
__device__ __forceinline__ float from_lane_above(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x130, 0xf, 0xf, true));
}
__device__ __forceinline__ double from_lane_above(double v) {
  const long long vi = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_update_dpp(0, (int)(vi & 0xffffffffLL), 0x130, 0xf, 0xf, true);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(vi >> 32), 0x130, 0xf, 0xf, true);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// loss = -scores, -mean(scores) or -sum(scores) (rnnt_loss.py:330-340) by ONE wave: every
// lane sums a contiguous slice, then a fixed butterfly over the lanes.
template <typename R>
__device__ __forceinline__ void reduce_scores(const R *__restrict__ scores, R *__restrict__ loss,
                                              int B, int reduction, int lane) {
  if (reduction == 0) {
    for (int b = lane; b < B; b += kWave) loss[b] = -scores[b];
    return;
  }
  const int per = (B + kWave - 1) / kWave;
  R acc = 0;
  for (int k = 0; k < per; ++k) {
    const int b = lane * per + k;
    if (b < B) acc += scores[b];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (lane == 0) loss[0] = reduction == 1 ? -(acc / (R)B) : -acc;
}

// The recursion's backward with a gradient of ones which, on its way, also reduces the
// forward's scores to the loss (a staging wave of the first workgroup does it once its
// tiles are done): saves the launch of a reduction kernel.  Host side, mi_recursion.hip.
int mi_backward_and_loss(const float *px, const int64_t *boundary, const float *p, float *px_grad,
                         float *py_grad, const float *scores, float *loss, int B, int S, int T,
                         int modified, int reduction, void *stream);
int mi_backward_and_loss(const double *px, const int64_t *boundary, const double *p,
                         double *px_grad, double *py_grad, const double *scores, double *loss,
                         int B, int S, int T, int modified, int reduction, void *stream);

}  // namespace frnnt
