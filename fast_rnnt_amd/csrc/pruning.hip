// Pruning bounds and the pruning gather of the pruned RNN-T loss.
//
// prune_ranges (fast_rnnt/python/fast_rnnt/rnnt_loss.py:638-777, helpers
// :550-632): for every frame pick the window start s that maximises
//   sum_{j<R} py_grad[b,s+j,t] - px_grad[b,s-1,t]        (0 for s = 0)
// with the window sum formed strictly left to right in the input precision and
// ties resolved to the first maximum, replace the starts of frames at or beyond
// T_b - 1 by max(S_b - R + 1, 0), then make the starts non-decreasing, starting
// at 0, with steps smaller than r (r = R for the regular lattice, 2 otherwise)
// by two suffix-minimum passes.  One wave per utterance; the per-frame starts
// live in LDS and the suffix minima are a chunked wave scan.
//
// prune_gather (rnnt_loss.py:780-818): lm_pruned[b,t,j,:] = lm[b, ranges[b,t,j], :]
// and its adjoint, a deterministic segmented sum (one block per lm row).
#include <climits>

#include "common.hip.h"

namespace frnnt {
namespace {

// suffix minimum of v[0..n) in place; v in LDS, one wave
__device__ __forceinline__ void suffix_min_inplace(int *v, int n, int lane) {
  const int per = (n + kWave - 1) / kWave;
  const int lo = lane * per, hi = min(n, lo + per);
  int local = INT_MAX;
  for (int k = hi - 1; k >= lo; --k) local = min(local, v[k]);
  // minimum over all chunks to the right of this lane's chunk
  int right = INT_MAX;
  {
    int acc = local;  // inclusive suffix scan over lanes
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const int o = __shfl_down(acc, off, kWave);
      if (lane + off < kWave) acc = min(acc, o);
    }
    const int next = __shfl_down(acc, 1, kWave);
    right = (lane + 1 < kWave) ? next : INT_MAX;
  }
  __syncthreads();
  int run = right;
  for (int k = hi - 1; k >= lo; --k) {
    run = min(run, v[k]);
    v[k] = run;
  }
  __syncthreads();
}

template <typename R>
__global__ void __launch_bounds__(kWave)
    prune_ranges_kernel(const R *__restrict__ px_grad, const R *__restrict__ py_grad,
                        const int64_t *__restrict__ boundary, int64_t *__restrict__ ranges, int S,
                        int T, int T1, int Rr) {
  extern __shared__ int start[];  // [T]
  const int b = blockIdx.x, lane = threadIdx.x;
  const R *gx = px_grad + (long)b * S * T1;
  const R *gy = py_grad + (long)b * (S + 1) * T;
  const int n = S + 2 - Rr;  // candidate window starts
  const int64_t Sb = boundary[4 * b + 2], Tb = boundary[4 * b + 3];
  int64_t tail = Sb - Rr + 1;
  if (tail < 0) tail = 0;
  for (int t = lane; t < T; t += kWave) {
    int best = 0;
    R best_score = 0;
    for (int s = 0; s < n; ++s) {
      R sum = gy[(long)s * T + t];
      for (int j = 1; j < Rr; ++j) sum = sum + gy[(long)(s + j) * T + t];
      const R below = s >= 1 ? gx[(long)(s - 1) * T1 + t] : (R)0;
      const R score = sum - below;
      // first maximum wins; a NaN score counts as the maximum, like torch.argmax
      if (s == 0 || score > best_score || (score != score && best_score == best_score)) {
        best = s;
        best_score = score;
      }
    }
    start[t] = ((int64_t)t < Tb - 1) ? best : (int)tail;
  }
  __syncthreads();
  const int r = (T1 != T) ? Rr : 2;
  suffix_min_inplace(start, T, lane);
  for (int t = lane; t < T; t += kWave) start[t] = (r - 1) * t - start[t];
  __syncthreads();
  suffix_min_inplace(start, T, lane);
  for (int t = lane; t < T; t += kWave) {
    const int y = max(start[t], 0);
    const int64_t s0 = (int64_t)(r - 1) * t - y;
    int64_t *out = ranges + ((long)b * T + t) * Rr;
    for (int j = 0; j < Rr; ++j) out[j] = s0 + j;
  }
}

// one wave per output row (b, t, j)
template <typename R>
__global__ void __launch_bounds__(256)
    prune_gather_kernel(const R *__restrict__ lm, const int64_t *__restrict__ ranges,
                        R *__restrict__ out, long rows, int TR, int S1, int C) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const long b = row / TR;
  int64_t s = ranges[row];
  R *dst = out + row * C;
  if (s < 0 || s >= S1) {
    for (int c = lane; c < C; c += kWave) dst[c] = std::numeric_limits<R>::quiet_NaN();
    return;
  }
  const R *src = lm + (b * S1 + s) * C;
  for (int c = lane; c < C; c += kWave) dst[c] = src[c];
}

// adjoint: one block per lm row (b, s); frames are visited in order, so the sum
// is deterministic
template <typename R>
__global__ void __launch_bounds__(256)
    prune_scatter_kernel(const R *__restrict__ grad, const int64_t *__restrict__ ranges,
                         R *__restrict__ lm_grad, int TR, int S1, int C) {
  const int b = blockIdx.x / S1, s = blockIdx.x % S1;
  const int64_t *rb = ranges + (long)b * TR;
  const R *gb = grad + (long)b * TR * C;
  for (int c0 = 0; c0 < C; c0 += 256) {
    const int c = c0 + threadIdx.x;
    R acc = 0;
    for (int k = 0; k < TR; ++k)
      if (rb[k] == s && c < C) acc += gb[(long)k * C + c];
    if (c < C) lm_grad[((long)b * S1 + s) * C + c] = acc;
  }
}

template <typename R>
int ranges_impl(const R *px_grad, const R *py_grad, const int64_t *boundary, int64_t *ranges, int B,
                int S, int T, int modified, int s_range, void *stream) {
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "prune_ranges: negative size");
  if (s_range < 1 || s_range > S + 1)
    return fail(FRNNT_EINVAL, "prune_ranges: s_range must lie in [1, S + 1]");
  if (B == 0 || T == 0) return FRNNT_OK;
  if (!px_grad || !py_grad || !boundary || !ranges)
    return fail(FRNNT_EINVAL, "prune_ranges: null pointer");
  const size_t lds = (size_t)T * sizeof(int);
  if (lds > 150 * 1024) return fail(FRNNT_ELIMIT, "prune_ranges: T=%d exceeds the LDS table", T);
  auto kernel = prune_ranges_kernel<R>;
  if (!allow_lds(reinterpret_cast<const void *>(kernel), lds))
    return check_launch("prune_ranges: hipFuncSetAttribute");
  hipLaunchKernelGGL(kernel, dim3(B), dim3(kWave), lds, static_cast<hipStream_t>(stream), px_grad,
                     py_grad, boundary, ranges, S, T, modified ? T : T + 1, s_range);
  return check_launch("prune_ranges");
}

template <typename R>
int gather_impl(const R *lm, const int64_t *ranges, R *out, int B, int S, int T, int Rr, int C,
                void *stream) {
  if (B < 0 || S < 0 || T < 0 || Rr < 0 || C < 0)
    return fail(FRNNT_EINVAL, "prune_gather: negative size");
  const long rows = (long)B * T * Rr;
  if (rows == 0 || C == 0) return FRNNT_OK;
  if (!lm || !ranges || !out) return fail(FRNNT_EINVAL, "prune_gather: null pointer");
  hipLaunchKernelGGL(prune_gather_kernel<R>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), lm, ranges, out, rows, T * Rr, S + 1, C);
  return check_launch("prune_gather");
}

template <typename R>
int scatter_impl(const R *grad, const int64_t *ranges, R *lm_grad, int B, int S, int T, int Rr,
                 int C, void *stream) {
  if (B < 0 || S < 0 || T < 0 || Rr < 0 || C < 0)
    return fail(FRNNT_EINVAL, "prune_gather_bwd: negative size");
  if (B == 0 || C == 0) return FRNNT_OK;
  if (!lm_grad || ((long)T * Rr > 0 && (!grad || !ranges)))
    return fail(FRNNT_EINVAL, "prune_gather_bwd: null pointer");
  hipLaunchKernelGGL(prune_scatter_kernel<R>, dim3((unsigned)(B * (S + 1))), dim3(256), 0,
                     static_cast<hipStream_t>(stream), grad, ranges, lm_grad, T * Rr, S + 1, C);
  return check_launch("prune_gather_bwd");
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_prune_ranges_f32(const float *px_grad, const float *py_grad, const int64_t *boundary,
                           int64_t *ranges, int B, int S, int T, int modified, int s_range,
                           void *stream) {
  return frnnt::ranges_impl<float>(px_grad, py_grad, boundary, ranges, B, S, T, modified, s_range,
                                   stream);
}
int frnnt_prune_ranges_f64(const double *px_grad, const double *py_grad, const int64_t *boundary,
                           int64_t *ranges, int B, int S, int T, int modified, int s_range,
                           void *stream) {
  return frnnt::ranges_impl<double>(px_grad, py_grad, boundary, ranges, B, S, T, modified, s_range,
                                    stream);
}
int frnnt_prune_gather_f32(const float *lm, const int64_t *ranges, float *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream) {
  return frnnt::gather_impl<float>(lm, ranges, lm_pruned, B, S, T, R, C, stream);
}
int frnnt_prune_gather_f64(const double *lm, const int64_t *ranges, double *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream) {
  return frnnt::gather_impl<double>(lm, ranges, lm_pruned, B, S, T, R, C, stream);
}
int frnnt_prune_gather_bwd_f32(const float *grad, const int64_t *ranges, float *lm_grad, int B,
                               int S, int T, int R, int C, void *stream) {
  return frnnt::scatter_impl<float>(grad, ranges, lm_grad, B, S, T, R, C, stream);
}
int frnnt_prune_gather_bwd_f64(const double *grad, const int64_t *ranges, double *lm_grad, int B,
                               int S, int T, int R, int C, void *stream) {
  return frnnt::scatter_impl<double>(grad, ranges, lm_grad, B, S, T, R, C, stream);
}

}  // extern "C"
