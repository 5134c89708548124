// px / py of the "simple" RNN-T loss (additive joiner) and their backward.
//
// Forward (fast_rnnt/python/fast_rnnt/rnnt_loss.py:66-227):
//   lm_max[b,s] = max_c lm[b,s,c]           am_max[b,t] = max_c am[b,t,c]
//   P[b,s,t]    = sum_c exp(lm - lm_max) * exp(am - am_max)      <- MFMA GEMM,
//                                                    exp fused into the tile loads
//   norm        = log(P + tiny) + lm_max + am_max
//   px[b,s,t]   = am[b,t,sym[b,s]] + lm[b,s,sym[b,s]] - norm[b,s,t]   (t < T)
//   py[b,s,t]   = am[b,t,term]     + lm[b,s,term]     - norm[b,s,t]
//   regular:     px[b,s,T] = -inf and, with a boundary, px[b,s,T_b] = -inf
//   constrained: px[b,s,t] += py[b,s+1,t]
// The epilogue of the GEMM writes px, py and log(P + tiny) straight from the
// accumulators; the normalizers never make a round trip through HBM.
//
// Backward: with gx = dL/dpx (masked like px), gy = dL/dpy (+ gx one row up for
// constrained), W = -(gx + gy) and D = W / (P + tiny):
//   dL/dlm[b,s,c] = exp(lm - lm_max) * sum_t D[s,t] exp(am[t,c] - am_max[t])
//                   + [c = sym[b,s]] sum_t gx[s,t] + [c = term] sum_t gy[s,t]
//   dL/dam[b,t,c] = exp(am - am_max) * sum_s D[s,t] exp(lm[s,c] - lm_max[s])
//                   + sum_s [c = sym[b,s]] gx[s,t] + [c = term] sum_s gy[s,t]
// i.e. two more GEMMs with the same fused-exp loaders (what autograd derives for
// rnnt_loss.py:174-220; the derivatives through the two max() cancel).
#include "tile_gemm.hip.h"

namespace frnnt {
namespace {

enum { kRegular = 0, kModified = 1, kConstrained = 2 };

template <typename R>
__device__ __forceinline__ R wave_max(R v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const R o = __shfl_xor(v, off, 64);
    v = o > v ? o : v;
  }
  return v;
}
template <typename R>
__device__ __forceinline__ R wave_sum(R v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// One wave per row of lm (first n_lm rows) or am (the rest): max over C.
template <typename R>
__global__ void __launch_bounds__(256)
    row_max_kernel(const R *__restrict__ lm, const R *__restrict__ am, R *__restrict__ lm_max,
                   R *__restrict__ am_max, long n_lm, long n_am, int C) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= n_lm + n_am) return;
  const R *src = row < n_lm ? lm + row * C : am + (row - n_lm) * C;
  R m = Num<R>::neg_inf();
  for (int c = lane; c < C; c += kWave) {
    const R v = src[c];
    m = (v > m || v != v) ? v : m;  // NaN propagates, like torch.max
  }
  {
    // reduce, keeping NaN if any lane saw one
    R r = m;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const R o = __shfl_xor(r, off, 64);
      r = (o > r || o != o) ? o : r;
    }
    m = r;
  }
  if (lane == 0) {
    if (row < n_lm)
      lm_max[row] = m;
    else
      am_max[row - n_lm] = m;
  }
}

template <typename R>
__device__ __forceinline__ R tiny_of();
template <>
__device__ __forceinline__ float tiny_of<float>() {
  return 1.17549435e-38f;
}
template <>
__device__ __forceinline__ double tiny_of<double>() {
  return 2.2250738585072014e-308;
}
template <typename R>
__device__ __forceinline__ R accurate_log(R x);
template <>
__device__ __forceinline__ float accurate_log<float>(float x) {
  return logf(x);
}
template <>
__device__ __forceinline__ double accurate_log<double>(double x) {
  return log(x);
}

// grid = (ceil(T/64), ceil((S+1)/64), B)
template <typename R>
__global__ void __launch_bounds__(kGemmThreads)
    simple_fwd_kernel(const R *__restrict__ lm, const R *__restrict__ am,
                      const int64_t *__restrict__ symbols, const int64_t *__restrict__ boundary,
                      const R *__restrict__ lm_max, const R *__restrict__ am_max,
                      R *__restrict__ px, R *__restrict__ py, R *__restrict__ norm_raw, int S,
                      int T, int C, int term, int rnnt_type) {
  __shared__ R lds[4 * TileK<R>::value * kPitch];
  const int b = blockIdx.z;
  const int s_tile = blockIdx.y * kTileM, t_tile = blockIdx.x * kTileN;
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const R *lmb = lm + (long)b * S1 * C;
  const R *amb = am + (long)b * T * C;
  const R *lmx = lm_max + (long)b * S1;
  const R *amx = am_max + (long)b * T;

  WaveAcc<R> acc;
  tile_matmul<R, LoaderKFast<R, true>, LoaderKFast<R, true>>(acc, lds, lmb, C, lmx, s_tile, S1,
                                                             amb, C, amx, t_tile, T, C);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t t_mask = (rnnt_type == kRegular && boundary) ? boundary[4 * b + 3] : -1;
  const int64_t *symb = symbols + (long)b * S;
  R *pxb = px + (long)b * S * T1;
  R *pyb = py + (long)b * S1 * T;
  R *nrb = norm_raw ? norm_raw + (long)b * S1 * T : nullptr;
  acc.for_each((wave >> 1) * 32, (wave & 1) * 32, lane, [&](int m, int n, R sum) {
    const int s = s_tile + m, t = t_tile + n;
    if (s >= S1 || t >= T) return;
    const R raw = accurate_log<R>(sum + tiny_of<R>());
    if (nrb) nrb[(long)s * T + t] = raw;
    const R norm = raw + lmx[s] + amx[t];
    pyb[(long)s * T + t] = (amb[(long)t * C + term] + lmb[(long)s * C + term]) - norm;
    if (s < S) {
      const int64_t sym = symb[s];
      R v;
      if (sym < 0 || sym >= C)
        v = std::numeric_limits<R>::quiet_NaN();  // out-of-vocabulary symbol
      else
        v = (amb[(long)t * C + sym] + lmb[(long)s * C + sym]) - norm;
      if (t == t_mask) v = Num<R>::neg_inf();
      pxb[(long)s * T1 + t] = v;
    }
  });
  // the extra column of the regular lattice: nothing can be emitted after the last frame
  if (rnnt_type == kRegular && blockIdx.x == 0) {
    for (int m = threadIdx.x; m < kTileM; m += kGemmThreads)
      if (s_tile + m < S) pxb[(long)(s_tile + m) * T1 + T] = Num<R>::neg_inf();
  }
}

// constrained lattice: px[b,s,t] += py[b,s+1,t]   (rnnt_loss.py:224-225)
template <typename R>
__global__ void __launch_bounds__(256)
    add_next_row_kernel(R *__restrict__ px, const R *__restrict__ py, long total, int S, int T) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const long b = idx / ((long)S * T);
  const long rem = idx - b * (long)S * T;
  const int s = (int)(rem / T), t = (int)(rem - (long)s * T);
  px[idx] += py[(b * (S + 1) + s + 1) * T + t];
}

// ---- backward ------------------------------------------------------------------------
// The first B*(S+1) blocks each take one lattice row (b, s): D[b,s,:] and the two
// row sums; the remaining blocks take 64 frames each and form the column sums.
template <typename R>
__global__ void __launch_bounds__(64)
    simple_bwd_prep_kernel(const R *__restrict__ gpx, const R *__restrict__ gpy,
                           const R *__restrict__ norm_raw, const int64_t *__restrict__ boundary,
                           R *__restrict__ dmat, R *__restrict__ row_x, R *__restrict__ row_y,
                           R *__restrict__ col_y, int B, int S, int T, int rnnt_type) {
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int lane = threadIdx.x;
  const long n_rows = (long)B * S1;
  auto gx_at = [&](int b, int s, int t, int64_t t_mask) -> R {
    if (s < 0 || s >= S || t == t_mask) return (R)0;
    return gpx[((long)b * S + s) * T1 + t];
  };
  if (blockIdx.x < n_rows) {
    const int b = blockIdx.x / S1, s = blockIdx.x % S1;
    const int64_t t_mask = (rnnt_type == kRegular && boundary) ? boundary[4 * b + 3] : -1;
    R sx = 0, sy = 0;
    for (int t = lane; t < T; t += kWave) {
      const R gx = gx_at(b, s, t, t_mask);
      R gy = gpy[((long)b * S1 + s) * T + t];
      if (rnnt_type == kConstrained) gy += gx_at(b, s - 1, t, t_mask);
      const long at = ((long)b * S1 + s) * T + t;
      dmat[at] = -(gx + gy) * fast_exp<R>(-norm_raw[at]);
      sx += gx;
      sy += gy;
    }
    sx = wave_sum(sx);
    sy = wave_sum(sy);
    if (lane == 0) {
      row_x[(long)b * S1 + s] = sx;
      row_y[(long)b * S1 + s] = sy;
    }
  } else {
    const int tiles = (T + kWave - 1) / kWave;
    const long cb = blockIdx.x - n_rows;
    const int b = (int)(cb / tiles), t = (int)(cb % tiles) * kWave + lane;
    if (t >= T) return;
    const int64_t t_mask = (rnnt_type == kRegular && boundary) ? boundary[4 * b + 3] : -1;
    R acc = 0;
    for (int s = 0; s < S1; ++s) {
      R gy = gpy[((long)b * S1 + s) * T + t];
      if (rnnt_type == kConstrained) gy += gx_at(b, s - 1, t, t_mask);
      acc += gy;
    }
    col_y[(long)b * T + t] = acc;
  }
}

// lm gradient: grid = (ceil(C/64), ceil((S+1)/64), B); K runs over frames.
template <typename R>
__global__ void __launch_bounds__(kGemmThreads)
    simple_bwd_lm_kernel(const R *__restrict__ lm, const R *__restrict__ am,
                         const int64_t *__restrict__ symbols, const R *__restrict__ lm_max,
                         const R *__restrict__ am_max, const R *__restrict__ dmat,
                         const R *__restrict__ row_x, const R *__restrict__ row_y,
                         R *__restrict__ lm_grad, int S, int T, int C, int term) {
  __shared__ R lds[4 * TileK<R>::value * kPitch];
  const int b = blockIdx.z;
  const int s_tile = blockIdx.y * kTileM, c_tile = blockIdx.x * kTileN;
  const int S1 = S + 1;
  const R *lmb = lm + (long)b * S1 * C;
  const R *amb = am + (long)b * T * C;
  const R *lmx = lm_max + (long)b * S1;
  const R *amx = am_max + (long)b * T;
  const R *db = dmat + (long)b * S1 * T;

  WaveAcc<R> acc;
  tile_matmul<R, LoaderKFast<R, false>, LoaderRowFast<R, true>>(acc, lds, db, T, nullptr, s_tile,
                                                                S1, amb, C, amx, c_tile, C, T);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  acc.for_each((wave >> 1) * 32, (wave & 1) * 32, lane, [&](int m, int n, R sum) {
    const int s = s_tile + m, c = c_tile + n;
    if (s >= S1 || c >= C) return;
    R g = fast_exp<R>(lmb[(long)s * C + c] - lmx[s]) * sum;
    if (s < S && symbols[(long)b * S + s] == c) g += row_x[(long)b * S1 + s];
    if (c == term) g += row_y[(long)b * S1 + s];
    lm_grad[((long)b * S1 + s) * C + c] = g;
  });
}

// am gradient: grid = (ceil(C/64), ceil(T/64), B); K runs over lattice rows.
template <typename R>
__global__ void __launch_bounds__(kGemmThreads)
    simple_bwd_am_kernel(const R *__restrict__ lm, const R *__restrict__ am,
                         const R *__restrict__ lm_max, const R *__restrict__ am_max,
                         const R *__restrict__ dmat, const R *__restrict__ col_y,
                         R *__restrict__ am_grad, int S, int T, int C, int term) {
  __shared__ R lds[4 * TileK<R>::value * kPitch];
  const int b = blockIdx.z;
  const int t_tile = blockIdx.y * kTileM, c_tile = blockIdx.x * kTileN;
  const int S1 = S + 1;
  const R *lmb = lm + (long)b * S1 * C;
  const R *amb = am + (long)b * T * C;
  const R *lmx = lm_max + (long)b * S1;
  const R *amx = am_max + (long)b * T;
  const R *db = dmat + (long)b * S1 * T;

  WaveAcc<R> acc;
  tile_matmul<R, LoaderRowFast<R, false>, LoaderRowFast<R, true>>(acc, lds, db, T, nullptr, t_tile,
                                                                  T, lmb, C, lmx, c_tile, C, S1);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  acc.for_each((wave >> 1) * 32, (wave & 1) * 32, lane, [&](int m, int n, R sum) {
    const int t = t_tile + m, c = c_tile + n;
    if (t >= T || c >= C) return;
    R g = fast_exp<R>(amb[(long)t * C + c] - amx[t]) * sum;
    if (c == term) g += col_y[(long)b * T + t];
    am_grad[((long)b * T + t) * C + c] = g;
  });
}

// am_grad[b,t,sym[b,s]] += gx[b,s,t]: one thread per (b,t), rows visited in
// order, so repeated symbols accumulate deterministically.
template <typename R>
__global__ void __launch_bounds__(256)
    simple_bwd_symbols_kernel(const R *__restrict__ gpx, const int64_t *__restrict__ symbols,
                              const int64_t *__restrict__ boundary, R *__restrict__ am_grad,
                              int B, int S, int T, int C, int rnnt_type) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)B * T) return;
  const int b = (int)(idx / T), t = (int)(idx % T);
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  if (rnnt_type == kRegular && boundary && boundary[4 * b + 3] == t) return;
  R *row = am_grad + idx * C;
  for (int s = 0; s < S; ++s) {
    const int64_t sym = symbols[(long)b * S + s];
    if (sym >= 0 && sym < C) row[sym] += gpx[((long)b * S + s) * T1 + t];
  }
}

template <typename R>
int fwd_impl(const R *lm, const R *am, const int64_t *symbols, const int64_t *boundary, R *px,
             R *py, R *lm_max, R *am_max, R *norm_raw, int B, int S, int T, int C, int term,
             int rnnt_type, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "simple_logprobs_fwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2)
    return fail(FRNNT_EINVAL, "simple_logprobs_fwd: rnnt_type must be 0, 1 or 2");
  if (term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "simple_logprobs_fwd: termination symbol outside [0, C)");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !px || !py || !lm_max || !am_max)
    return fail(FRNNT_EINVAL, "simple_logprobs_fwd: null pointer");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long n_lm = (long)B * (S + 1), n_am = (long)B * T;
  const long rows = n_lm + n_am;
  hipLaunchKernelGGL(row_max_kernel<R>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, lm,
                     am, lm_max, am_max, n_lm, n_am, C);
  {
    // at least one column of tiles, so that the -inf column of an empty-frame
    // regular lattice is still written
    const int t_tiles = T > 0 ? (T + kTileN - 1) / kTileN : 1;
    const dim3 grid(t_tiles, (S + 1 + kTileM - 1) / kTileM, B);
    hipLaunchKernelGGL(simple_fwd_kernel<R>, grid, dim3(kGemmThreads), 0, stream, lm, am, symbols,
                       boundary, lm_max, am_max, px, py, norm_raw, S, T, C, term, rnnt_type);
    if (rnnt_type == kConstrained && S > 0 && T > 0) {
      const long total = (long)B * S * T;
      hipLaunchKernelGGL(add_next_row_kernel<R>, dim3((unsigned)((total + 255) / 256)), dim3(256),
                         0, stream, px, py, total, S, T);
    }
  }
  return check_launch("simple_logprobs_fwd");
}

template <typename R>
int bwd_impl(const R *lm, const R *am, const int64_t *symbols, const int64_t *boundary,
             const R *lm_max, const R *am_max, const R *norm_raw, const R *px_grad,
             const R *py_grad, R *dmat, R *row_x, R *row_y, R *col_y, R *lm_grad, R *am_grad,
             int B, int S, int T, int C, int term, int rnnt_type, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "simple_logprobs_bwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "simple_logprobs_bwd: bad rnnt_type or termination symbol");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !lm_max || !am_max || !norm_raw || !px_grad ||
      !py_grad || !dmat || !row_x || !row_y || !col_y)
    return fail(FRNNT_EINVAL, "simple_logprobs_bwd: null pointer");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long prep_blocks = (long)B * (S + 1) + (long)B * ((T + kWave - 1) / kWave);
  hipLaunchKernelGGL(simple_bwd_prep_kernel<R>, dim3((unsigned)prep_blocks), dim3(64), 0, stream,
                     px_grad, py_grad, norm_raw, boundary, dmat, row_x, row_y, col_y, B, S, T,
                     rnnt_type);
  const int c_tiles = (C + kTileN - 1) / kTileN;
  if (lm_grad) {
    const dim3 grid(c_tiles, (S + 1 + kTileM - 1) / kTileM, B);
    hipLaunchKernelGGL(simple_bwd_lm_kernel<R>, grid, dim3(kGemmThreads), 0, stream, lm, am,
                       symbols, lm_max, am_max, dmat, row_x, row_y, lm_grad, S, T, C, term);
  }
  if (am_grad && T > 0) {
    const dim3 grid(c_tiles, (T + kTileM - 1) / kTileM, B);
    hipLaunchKernelGGL(simple_bwd_am_kernel<R>, grid, dim3(kGemmThreads), 0, stream, lm, am, lm_max,
                       am_max, dmat, col_y, am_grad, S, T, C, term);
    if (S > 0) {
      const long n = (long)B * T;
      hipLaunchKernelGGL(simple_bwd_symbols_kernel<R>, dim3((unsigned)((n + 255) / 256)),
                         dim3(256), 0, stream, px_grad, symbols, boundary, am_grad, B, S, T, C,
                         rnnt_type);
    }
  }
  return check_launch("simple_logprobs_bwd");
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_simple_logprobs_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                  const int64_t *boundary, float *px, float *py, float *lm_max,
                                  float *am_max, float *norm_raw, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, void *stream) {
  return frnnt::fwd_impl<float>(lm, am, symbols, boundary, px, py, lm_max, am_max, norm_raw, B, S,
                                T, C, termination_symbol, rnnt_type, stream);
}
int frnnt_simple_logprobs_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, double *px, double *py, double *lm_max,
                                  double *am_max, double *norm_raw, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, void *stream) {
  return frnnt::fwd_impl<double>(lm, am, symbols, boundary, px, py, lm_max, am_max, norm_raw, B, S,
                                 T, C, termination_symbol, rnnt_type, stream);
}
int frnnt_simple_logprobs_bwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                  const int64_t *boundary, const float *lm_max,
                                  const float *am_max, const float *norm_raw, const float *px_grad,
                                  const float *py_grad, float *dmat, float *row_x, float *row_y,
                                  float *col_y, float *lm_grad, float *am_grad, int B, int S,
                                  int T, int C, int termination_symbol, int rnnt_type,
                                  void *stream) {
  return frnnt::bwd_impl<float>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, px_grad,
                                py_grad, dmat, row_x, row_y, col_y, lm_grad, am_grad, B, S, T, C,
                                termination_symbol, rnnt_type, stream);
}
int frnnt_simple_logprobs_bwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, const double *lm_max,
                                  const double *am_max, const double *norm_raw,
                                  const double *px_grad, const double *py_grad, double *dmat,
                                  double *row_x, double *row_y, double *col_y, double *lm_grad,
                                  double *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, void *stream) {
  return frnnt::bwd_impl<double>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, px_grad,
                                 py_grad, dmat, row_x, row_y, col_y, lm_grad, am_grad, B, S, T, C,
                                 termination_symbol, rnnt_type, stream);
}

}  // extern "C"
