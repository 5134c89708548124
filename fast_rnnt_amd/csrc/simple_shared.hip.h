// What the kernels of the simple (additive-joiner) loss share between their two source
// files: simple_normalizer.hip (the forward's normalizer product, compiled with a scheduling
// strategy of its own) and simple_logprobs.hip (everything else).
#pragma once
#include "xcd_grid.hip.h"

namespace frnnt {
namespace {

enum { kRegular = 0, kModified = 1, kConstrained = 2 };

// What the lattice recursion uses of utterance b: rows [s_begin, s_end] and frames
// [t_begin, t_end) of py, rows [s_begin, s_end) of px.  A caller that goes on to the
// recursion with the same boundary passes it as `window`: the kernels then leave px / py /
// the normalizers outside it undefined, and take the gradients to vanish there (the
// recursion writes exact zeros).  Without a window everything counts.
struct Limits {
  int s_begin, t_begin, s_end, t_end;
};
__device__ __forceinline__ Limits limits_of(const int64_t *window, int b, int S, int T) {
  Limits w{0, 0, S, T};
  if (window) {
    // clamped: a boundary row outside the lattice must not widen any loop
    w.s_begin = (int)max((int64_t)0, min(window[4 * b + 0], (int64_t)S));
    w.t_begin = (int)max((int64_t)0, min(window[4 * b + 1], (int64_t)T));
    w.s_end = (int)max((int64_t)0, min(window[4 * b + 2], (int64_t)S));
    w.t_end = (int)max((int64_t)0, min(window[4 * b + 3], (int64_t)T));
  }
  return w;
}

// The normalizer kernel is the first of its call (no ranks yet): utterance b stays on XCD
// b % 8, and a batch of fewer than eight is cut into parts along the frames until it reaches
// every XCD (the parts of an utterance share its lm rows, the small operand).
inline int frame_part_shift_for(int B, int t_tiles) {
  int shift = 0;
  while ((B << shift) < dgemm::kXcds && (2 << shift) <= t_tiles) ++shift;
  return shift;
}
__device__ __forceinline__ bool place_frames(int id, int t_tiles, int s_tiles, int part_shift, int B,
                                             int &b, int &s_idx, int &t_idx) {
  using dgemm::kXcds;
  const int t_per = (t_tiles + (1 << part_shift) - 1) >> part_shift;
  const int unit_tiles = t_per * s_tiles;
  const int xcd = id % kXcds, slot = id / kXcds, round = slot / unit_tiles;
  const int within = slot - round * unit_tiles;
  const int unit = round * kXcds + xcd;
  b = unit >> part_shift;
  s_idx = within / t_per;
  t_idx = (unit & ((1 << part_shift) - 1)) * t_per + (within - s_idx * t_per);
  return b < B && t_idx < t_tiles;
}
typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));

// exp(x - m) as one fused multiply-add and one v_exp_f32: 2^(x log2(e) - m log2(e)),
// with shift2 = -m log2(e) prepared per row; x = -inf gives 0.
constexpr float kLog2e = 1.44269504088896341f;
// The largest of three, as the one instruction it is.  fmaxf() costs a canonicalising
// v_max_f32 per operand on top (the compiler quiets signalling NaNs first), which tripled the
// instruction count of the row maxima in the GEMM loops; v_max3_f32 itself ignores quiet NaNs
// like fmaxf and quiets signalling ones.
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float exp_shifted(float x, float shift2) {
  return __builtin_amdgcn_exp2f(__builtin_fmaf(x, kLog2e, shift2));
}

}  // namespace

// The float32 normalizer product with px / py in its epilogue (simple_normalizer.hip): the
// 96- or 128-row form, whichever pads S + 1 less.
void launch_normalizer_f32(const float *lm, const float *am, const int64_t *symbols,
                           const int64_t *boundary, float *lm_max, float *am_max, float *px,
                           float *py, float *norm_raw, const int64_t *window, int B, int S, int T,
                           int C, int term, int rnnt_type, hipStream_t stream);

}  // namespace frnnt
