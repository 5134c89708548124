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
#include "direct_gemm.hip.h"
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
// 256-thread workgroups.  The first ceil(B*(S+1)/4) of them give each wave one
// lattice row (b, s): D[b,s,:] and the two row sums.  The remaining ones take 64
// frames of one utterance each and form the column sums, the four waves splitting
// the lattice rows.  Loads are issued in batches of four before anything is
// stored, so a row costs one memory round trip, not one per 64 frames.
template <typename R>
__global__ void __launch_bounds__(256)
    simple_bwd_prep_kernel(const R *__restrict__ gpx, const R *__restrict__ gpy,
                           const R *__restrict__ norm_raw, const int64_t *__restrict__ boundary,
                           R *__restrict__ dmat, R *__restrict__ row_x, R *__restrict__ row_y,
                           R *__restrict__ col_y, int B, int S, int T, int ldd, int rnnt_type) {
  __shared__ R partial[4][kWave];
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long n_rows = (long)B * S1;
  const long row_blocks = (n_rows + 3) / 4;
  const bool constrained = rnnt_type == kConstrained;
  if (blockIdx.x < row_blocks) {
    const long row = (long)blockIdx.x * 4 + wave;
    if (row >= n_rows) return;
    const int b = (int)(row / S1), s = (int)(row % S1);
    const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;
    const R *gx_row = s < S ? gpx + ((long)b * S + s) * T1 : nullptr;
    const R *gx_prev = (constrained && s >= 1) ? gpx + ((long)b * S + s - 1) * T1 : nullptr;
    const R *gy_row = gpy + row * T;
    const R *nr_row = norm_raw + row * T;
    R *d_row = dmat + row * ldd;
    R sx = 0, sy = 0;
    for (int t0 = 0; t0 < T; t0 += 4 * kWave) {
      R gx[4], gy[4], nr[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * kWave + lane;
        const bool ok = t < T;
        gx[u] = (ok && gx_row && t != t_mask) ? gx_row[t] : (R)0;
        gy[u] = ok ? gy_row[t] : (R)0;
        if (ok && gx_prev && t != t_mask) gy[u] += gx_prev[t];
        nr[u] = ok ? nr_row[t] : (R)0;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int t = t0 + u * kWave + lane;
        if (t < T) d_row[t] = -(gx[u] + gy[u]) * fast_exp<R>(-nr[u]);
        sx += gx[u];
        sy += gy[u];
      }
    }
    sx = wave_sum(sx);
    sy = wave_sum(sy);
    if (lane == 0) {
      row_x[row] = sx;
      row_y[row] = sy;
    }
  } else {
    const int tiles = (T + kWave - 1) / kWave;
    const long cb = blockIdx.x - row_blocks;
    const int b = (int)(cb / tiles), t = (int)(cb % tiles) * kWave + lane;
    const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;
    const bool ok = t < T;
    R acc = 0;
    for (int s0 = wave; s0 < S1; s0 += 16) {
      R v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int s = s0 + 4 * u;
        v[u] = (ok && s < S1) ? gpy[((long)b * S1 + s) * T + t] : (R)0;
        if (constrained && ok && s >= 1 && s < S1 && t != t_mask)
          v[u] += gpx[((long)b * S + s - 1) * T1 + t];
      }
      acc += (v[0] + v[1]) + (v[2] + v[3]);
    }
    partial[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && ok)
      col_y[(long)b * T + t] = (partial[0][lane] + partial[1][lane]) + (partial[2][lane] + partial[3][lane]);
  }
}

// px_grad[b,:,:] *= score_grad[b], py_grad[b,:,:] *= score_grad[b], in place.
template <typename R>
__global__ void __launch_bounds__(256)
    scale_by_batch_kernel(R *__restrict__ gpx, R *__restrict__ gpy,
                          const R *__restrict__ score_grad, long per_x, long per_y, int B) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long nx = per_x * B, ny = per_y * B;
  if (idx < nx)
    gpx[idx] *= score_grad[idx / per_x];
  else if (idx < nx + ny)
    gpy[idx - nx] *= score_grad[(idx - nx) / per_y];
}

// lm gradient: grid = (ceil(C/64), ceil((S+1)/64), B); K runs over frames.
template <typename R>
__global__ void __launch_bounds__(kGemmThreads)
    simple_bwd_lm_kernel(const R *__restrict__ lm, const R *__restrict__ am,
                         const int64_t *__restrict__ symbols, const R *__restrict__ lm_max,
                         const R *__restrict__ am_max, const R *__restrict__ dmat,
                         const R *__restrict__ row_x, const R *__restrict__ row_y,
                         R *__restrict__ lm_grad, int S, int T, int C, int ldd, int term) {
  __shared__ R lds[4 * TileK<R>::value * kPitch];
  const int b = blockIdx.z;
  const int s_tile = blockIdx.y * kTileM, c_tile = blockIdx.x * kTileN;
  const int S1 = S + 1;
  const R *lmb = lm + (long)b * S1 * C;
  const R *amb = am + (long)b * T * C;
  const R *lmx = lm_max + (long)b * S1;
  const R *amx = am_max + (long)b * T;
  const R *db = dmat + (long)b * S1 * ldd;

  WaveAcc<R> acc;
  tile_matmul<R, LoaderKFast<R, false>, LoaderRowFast<R, true>>(acc, lds, db, ldd, nullptr, s_tile,
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
                         R *__restrict__ am_grad, int S, int T, int C, int ldd, int term) {
  __shared__ R lds[4 * TileK<R>::value * kPitch];
  const int b = blockIdx.z;
  const int t_tile = blockIdx.y * kTileM, c_tile = blockIdx.x * kTileN;
  const int S1 = S + 1;
  const R *lmb = lm + (long)b * S1 * C;
  const R *amb = am + (long)b * T * C;
  const R *lmx = lm_max + (long)b * S1;
  const R *amx = am_max + (long)b * T;
  const R *db = dmat + (long)b * S1 * ldd;

  WaveAcc<R> acc;
  tile_matmul<R, LoaderRowFast<R, false>, LoaderRowFast<R, true>>(acc, lds, db, ldd, nullptr, t_tile,
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


// ---- fp32: register-direct MFMA kernels (direct_gemm.hip.h) ------------------------
constexpr int kFwdWaves = 4;  // K split of the forward normalizer GEMM
constexpr int kLmWaves = 4;   // K split of the lm-gradient GEMM

// 1-D XCD-aware grid over (b, s-tile, t-tile); 8 waves split C between them.
template <bool kVec>
__global__ void __launch_bounds__(kFwdWaves *kWave)
    simple_fwd_direct_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                             const int64_t *__restrict__ symbols,
                             const int64_t *__restrict__ boundary,
                             const float *__restrict__ lm_max, const float *__restrict__ am_max,
                             float *__restrict__ px, float *__restrict__ py,
                             float *__restrict__ norm_raw, int B, int S, int T, int C, int term,
                             int rnnt_type) {
  using namespace dgemm;
  __shared__ float lds[kFwdWaves * kBM * kBN];
  __shared__ float row_term[kBM], row_sym[kBM], row_max[kBM];  // lm[s,term], lm[s,sym[s]], lm_max[s]
  __shared__ int row_symbol[kBM];
  __shared__ float col_term[kBN], col_max[kBN];                // am[t,term], am_max[t]
  const int S1 = S + 1;
  const int t_tiles = T > 0 ? (T + kBN - 1) / kBN : 1, s_tiles = (S1 + kBM - 1) / kBM;
  int b, tile;
  if (!decode_block(t_tiles * s_tiles, B, b, tile)) return;
  const int s_tile = (tile / t_tiles) * kBM, t_tile = (tile % t_tiles) * kBN;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const float *lmb = lm + (long)b * S1 * C;
  const float *amb = am + (long)b * T * C;
  const float *lmx = lm_max + (long)b * S1;
  const float *amx = am_max + (long)b * T;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, r32 = lane & 31;
  const float ninf = -__builtin_huge_valf();

  const int s_row = s_tile + r32, t_row0 = t_tile + r32, t_row1 = t_tile + 32 + r32;
  const bool a_ok = s_row < S1, b_ok0 = t_row0 < T, b_ok1 = t_row1 < T;

  Acc acc;
  acc.clear();
  Frag a, b0, b1, an, b0n, b1n;
  auto fetch = [&](Frag &fa, Frag &f0, Frag &f1, int kb) {
    const int k0 = kb + 16 * half;
    load_kfast<kVec>(fa, lmb, s_row * C, a_ok, k0, C, ninf);
    load_kfast<kVec>(f0, amb, t_row0 * C, b_ok0, k0, C, ninf);
    load_kfast<kVec>(f1, amb, t_row1 * C, b_ok1, k0, C, ninf);
  };
  int kb = wave * kBK;
  if (kb < C) fetch(an, b0n, b1n, kb);

  // Everything the epilogue needs from global memory is requested now, behind the
  // first operand fetch, so that its latency hides under the GEMM loop:
  // am[b, t, sym[b, s]] for this thread's output elements ...
  constexpr int kPer = kBM * kBN / (kFwdWaves * kWave);
  float am_sym[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int e = j * (kFwdWaves * kWave) + tid;
    const int s = s_tile + e / kBN, t = t_tile + e % kBN;
    am_sym[j] = 0.f;
    if (s < S && t < T) {
      const int64_t y = symbols[(long)b * S + s];
      if (y >= 0 && y < C) am_sym[j] = amb[(long)t * C + y];
    }
  }
  // ... and the per-row / per-column terms, shared through LDS
  if (tid < kBM) {
    const int s = s_tile + tid;
    float vt = 0.f, vs = 0.f, vm = 0.f;
    int sym = -1;
    if (s < S1) {
      vt = lmb[(long)s * C + term];
      vm = lmx[s];
      if (s < S) {
        const int64_t y = symbols[(long)b * S + s];
        sym = (y >= 0 && y < C) ? (int)y : -1;
        if (sym >= 0) vs = lmb[(long)s * C + sym];
      }
    }
    row_term[tid] = vt;
    row_sym[tid] = vs;
    row_max[tid] = vm;
    row_symbol[tid] = sym;
  } else if (tid >= 64 && tid < 64 + kBN) {
    const int t = t_tile + tid - 64;
    col_term[tid - 64] = t < T ? amb[(long)t * C + term] : 0.f;
    col_max[tid - 64] = t < T ? amx[t] : 0.f;
  }
  const float a_shift = a_ok ? lmx[s_row] : 0.f;
  const float b_shift0 = b_ok0 ? amx[t_row0] : 0.f;
  const float b_shift1 = b_ok1 ? amx[t_row1] : 0.f;

  for (; kb < C; kb += kFwdWaves * kBK) {
    a = an;
    b0 = b0n;
    b1 = b1n;
    if (kb + kFwdWaves * kBK < C) fetch(an, b0n, b1n, kb + kFwdWaves * kBK);
    exp_shift_scalar(a, a_shift);
    exp_shift_scalar(b0, b_shift0);
    exp_shift_scalar(b1, b_shift1);
    acc.mma(a, b0, b1);
  }

  const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;
  float *pxb = px + (long)b * S * T1;
  float *pyb = py + (long)b * S1 * T;
  float *nrb = norm_raw ? norm_raw + (long)b * S1 * T : nullptr;
  // (the barrier inside reduce_and_emit also publishes row_* / col_* to all waves)
  int slot = 0;
  reduce_and_emit<kFwdWaves>(
      acc, lds, [&](int, int) -> float { return am_sym[slot++]; },
      [&](int m, int n, float sum, float am_at_sym) {
        const int s = s_tile + m, t = t_tile + n;
        if (s >= S1 || t >= T) return;
        const float raw = logf(sum + 1.17549435e-38f);
        if (nrb) nrb[(long)s * T + t] = raw;
        const float norm = raw + row_max[m] + col_max[n];
        pyb[(long)s * T + t] = (col_term[n] + row_term[m]) - norm;
        if (s < S) {
          float v = std::numeric_limits<float>::quiet_NaN();  // out-of-vocabulary symbol
          if (row_symbol[m] >= 0) v = (am_at_sym + row_sym[m]) - norm;
          if (t == t_mask) v = ninf;
          pxb[(long)s * T1 + t] = v;
        }
      });
  // the extra column of the regular lattice: nothing can be emitted after the last frame
  if (rnnt_type == kRegular && t_tile == 0 && tid < kBM && s_tile + tid < S)
    pxb[(long)(s_tile + tid) * T1 + T] = ninf;
}

// lm gradient: grid = (ceil(C/64), ceil((S+1)/32), B); k runs over frames.
template <bool kVec>
__global__ void __launch_bounds__(kLmWaves *kWave)
    simple_bwd_lm_direct_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                                const int64_t *__restrict__ symbols,
                                const float *__restrict__ lm_max,
                                const float *__restrict__ am_max, const float *__restrict__ dmat,
                                const float *__restrict__ row_x, const float *__restrict__ row_y,
                                float *__restrict__ lm_grad, int B, int S, int T, int C,
                                int ldd, int term) {
  using namespace dgemm;
  __shared__ float lds[kLmWaves * kBM * kBN];
  const int S1 = S + 1;
  const int c_tiles = (C + kBN - 1) / kBN, s_tiles = (S1 + kBM - 1) / kBM;
  int b, tile;
  if (!decode_block(c_tiles * s_tiles, B, b, tile)) return;
  const int s_tile = (tile / c_tiles) * kBM, c_tile = (tile % c_tiles) * kBN;
  const float *lmb = lm + (long)b * S1 * C;
  const float *amb = am + (long)b * T * C;
  const float *lmx = lm_max + (long)b * S1;
  const float *amx = am_max + (long)b * T;
  const float *db = dmat + (long)b * S1 * ldd;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = lane >> 5, r32 = lane & 31;
  const float ninf = -__builtin_huge_valf();

  const int s_row = s_tile + r32, c0 = c_tile + r32, c1 = c_tile + 32 + r32;
  const bool a_ok = s_row < S1, b_ok0 = c0 < C, b_ok1 = c1 < C;

  // this thread's lm[b, s, c] for the epilogue, requested ahead of the GEMM loop
  constexpr int kPer = kBM * kBN / (kLmWaves * kWave);
  float lm_sc[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int e = j * (kLmWaves * kWave) + (int)threadIdx.x;
    const int s = s_tile + e / kBN, c = c_tile + e % kBN;
    lm_sc[j] = (s < S1 && c < C) ? lmb[(long)s * C + c] : 0.f;
  }
  Acc acc;
  acc.clear();
  for (int kb = wave * kBK; kb < T; kb += kLmWaves * kBK) {
    const int k0 = kb + 16 * half;
    Frag a, b0, b1, mx;
    load_kfast<kVec>(a, db, s_row * ldd, a_ok, k0, T, 0.f);
    load_rowfast(b0, amb, C, c0, b_ok0, k0, T, ninf);
    load_rowfast(b1, amb, C, c1, b_ok1, k0, T, ninf);
    load_kfast<false>(mx, amx, 0, true, k0, T, 0.f);
    exp_shift_each(b0, mx);
    exp_shift_each(b1, mx);
    acc.mma(a, b0, b1);
  }
  int slot = 0;
  reduce_and_emit<kLmWaves>(
      acc, lds, [&](int, int) -> float { return lm_sc[slot++]; },
      [&](int m, int n, float sum, float lm_at) {
        const int s = s_tile + m, c = c_tile + n;
        if (s >= S1 || c >= C) return;
        float g = __expf(lm_at - lmx[s]) * sum;
        if (s < S && symbols[(long)b * S + s] == c) g += row_x[(long)b * S1 + s];
        if (c == term) g += row_y[(long)b * S1 + s];
        lm_grad[((long)b * S1 + s) * C + c] = g;
      });
}

// am gradient: k runs over the S+1 lattice rows -- too short to split, so each of
// the four waves of a workgroup owns its own 32 (frames) x 32 (vocabulary) tile;
// small tiles keep the register count low enough for four waves per SIMD, which
// is what hides the memory latency of this streaming kernel.
// The per-symbol term  sum_s [c = sym[b,s]] gx[b,s,t]  is a second product on the
// matrix core, gx^T times a one-hot matrix made in registers from the symbols: it is
// exact (products by 0 or 1) and has a fixed summation order.
__global__ void __launch_bounds__(256)
    simple_bwd_am_direct_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                                const int64_t *__restrict__ symbols,
                                const int64_t *__restrict__ boundary,
                                const float *__restrict__ lm_max,
                                const float *__restrict__ am_max, const float *__restrict__ dmat,
                                const float *__restrict__ gpx, const float *__restrict__ col_y,
                                float *__restrict__ am_grad, int B, int S, int T, int C, int ldd,
                                int term, int rnnt_type) {
  using namespace dgemm;
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int c_tiles = (C + 31) / 32, t_groups = (T + 4 * kBM - 1) / (4 * kBM);
  int b, tile;
  if (!decode_block(c_tiles * t_groups, B, b, tile)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t_tile = ((tile / c_tiles) * 4 + wave) * kBM, c_tile = (tile % c_tiles) * 32;
  if (t_tile >= T) return;
  const float *lmb = lm + (long)b * S1 * C;
  const float *amb = am + (long)b * T * C;
  const float *lmx = lm_max + (long)b * S1;
  const float *amx = am_max + (long)b * T;
  const float *db = dmat + (long)b * S1 * ldd;
  const float *gxb = gpx + (long)b * S * T1;
  const int64_t *symb = symbols + (long)b * S;
  const int half = lane >> 5, r32 = lane & 31;
  const float ninf = -__builtin_huge_valf();
  const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;

  const int t_row = t_tile + r32, c0 = c_tile + r32;
  const bool a_ok = t_row < T, g_ok = t_row < T && t_row != t_mask, b_ok = c0 < C;

  // epilogue inputs first: am[b, t, c] of this lane's 16 output elements
  float am_tc[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int t = t_tile + 8 * (v / 4) + 4 * half + (v % 4);
    am_tc[v] = (t < T && c0 < C) ? amb[(long)t * C + c0] : 0.f;
  }

  floatx16 acc, hot;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = hot[v] = 0.f;
  // symbols are < C < 2^31: their low words (little endian) are enough to compare
  const int *sym_lo = reinterpret_cast<const int *>(symb);
#pragma unroll 1
  for (int kb = 0; kb < S1; kb += kBK) {
    const int k0 = kb + 16 * half;
    Frag a, g, b0, mx;
    load_rowfast(a, db, ldd, t_row, a_ok, k0, S1, 0.f);
    load_rowfast(g, gxb, T1, t_row, g_ok, k0, S, 0.f);
    load_rowfast(b0, lmb, C, c0, b_ok, k0, S1, ninf);
    load_kfast<false>(mx, lmx, 0, true, k0, S1, 0.f);
    exp_shift_each(b0, mx);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int y = (k0 + i < S) ? sym_lo[2 * (k0 + i)] : -1;
      const float h = (y == c0) ? 1.f : 0.f;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b0.v[i], acc, 0, 0, 0);
      hot = __builtin_amdgcn_mfma_f32_32x32x2f32(g.v[i], h, hot, 0, 0, 0);
    }
  }
  if (c0 >= C) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int t = t_tile + 8 * (v / 4) + 4 * half + (v % 4);
    if (t >= T) continue;
    float gsum = __expf(am_tc[v] - amx[t]) * acc[v] + hot[v];
    if (c0 == term) gsum += col_y[(long)b * T + t];
    am_grad[((long)b * T + t) * C + c0] = gsum;
  }
}

// launchers: float goes to the register-direct kernels, double to the LDS-tiled ones
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

void launch_fwd_gemm(const float *lm, const float *am, const int64_t *symbols,
                     const int64_t *boundary, const float *lm_max, const float *am_max, float *px,
                     float *py, float *norm_raw, int B, int S, int T, int C, int term,
                     int rnnt_type, hipStream_t stream) {
  const int t_tiles = T > 0 ? (T + dgemm::kBN - 1) / dgemm::kBN : 1;
  const int s_tiles = (S + 1 + dgemm::kBM - 1) / dgemm::kBM;
  const bool vec = (C % 4 == 0) && aligned16(lm) && aligned16(am);
  auto kernel = vec ? simple_fwd_direct_kernel<true> : simple_fwd_direct_kernel<false>;
  hipLaunchKernelGGL(kernel, dim3(dgemm::xcd_grid(t_tiles * s_tiles, B)),
                     dim3(kFwdWaves * kWave), 0, stream, lm, am, symbols, boundary, lm_max, am_max,
                     px, py, norm_raw, B, S, T, C, term, rnnt_type);
}
void launch_fwd_gemm(const double *lm, const double *am, const int64_t *symbols,
                     const int64_t *boundary, const double *lm_max, const double *am_max,
                     double *px, double *py, double *norm_raw, int B, int S, int T, int C,
                     int term, int rnnt_type, hipStream_t stream) {
  const int t_tiles = T > 0 ? (T + kTileN - 1) / kTileN : 1;
  const dim3 grid(t_tiles, (S + 1 + kTileM - 1) / kTileM, B);
  hipLaunchKernelGGL(simple_fwd_kernel<double>, grid, dim3(kGemmThreads), 0, stream, lm, am,
                     symbols, boundary, lm_max, am_max, px, py, norm_raw, S, T, C, term,
                     rnnt_type);
}
void launch_bwd_lm(const float *lm, const float *am, const int64_t *symbols, const float *lm_max,
                   const float *am_max, const float *dmat, const float *row_x, const float *row_y,
                   float *lm_grad, int B, int S, int T, int C, int ldd, int term,
                   hipStream_t stream) {
  const int tiles = ((C + dgemm::kBN - 1) / dgemm::kBN) * ((S + 1 + dgemm::kBM - 1) / dgemm::kBM);
  const bool vec = (ldd % 4 == 0) && aligned16(dmat);
  auto kernel = vec ? simple_bwd_lm_direct_kernel<true> : simple_bwd_lm_direct_kernel<false>;
  hipLaunchKernelGGL(kernel, dim3(dgemm::xcd_grid(tiles, B)), dim3(kLmWaves * kWave), 0, stream,
                     lm, am, symbols, lm_max, am_max, dmat, row_x, row_y, lm_grad, B, S, T, C, ldd,
                     term);
}
void launch_bwd_lm(const double *lm, const double *am, const int64_t *symbols,
                   const double *lm_max, const double *am_max, const double *dmat,
                   const double *row_x, const double *row_y, double *lm_grad, int B, int S, int T,
                   int C, int ldd, int term, hipStream_t stream) {
  const dim3 grid((C + kTileN - 1) / kTileN, (S + 1 + kTileM - 1) / kTileM, B);
  hipLaunchKernelGGL(simple_bwd_lm_kernel<double>, grid, dim3(kGemmThreads), 0, stream, lm, am,
                     symbols, lm_max, am_max, dmat, row_x, row_y, lm_grad, S, T, C, ldd, term);
}
void launch_bwd_am(const float *lm, const float *am, const int64_t *symbols,
                   const int64_t *boundary, const float *lm_max, const float *am_max,
                   const float *dmat, const float *gpx, const float *col_y, float *am_grad, int B,
                   int S, int T, int C, int ldd, int term, int rnnt_type, hipStream_t stream) {
  const int tiles = ((C + 31) / 32) * ((T + 4 * dgemm::kBM - 1) / (4 * dgemm::kBM));
  hipLaunchKernelGGL(simple_bwd_am_direct_kernel, dim3(dgemm::xcd_grid(tiles, B)), dim3(256), 0,
                     stream, lm, am, symbols, boundary, lm_max, am_max, dmat, gpx, col_y, am_grad,
                     B, S, T, C, ldd, term, rnnt_type);
}
void launch_bwd_am(const double *lm, const double *am, const int64_t *symbols,
                   const int64_t *boundary, const double *lm_max, const double *am_max,
                   const double *dmat, const double *gpx, const double *col_y, double *am_grad,
                   int B, int S, int T, int C, int ldd, int term, int rnnt_type,
                   hipStream_t stream) {
  const dim3 grid((C + kTileN - 1) / kTileN, (T + kTileM - 1) / kTileM, B);
  hipLaunchKernelGGL(simple_bwd_am_kernel<double>, grid, dim3(kGemmThreads), 0, stream, lm, am,
                     lm_max, am_max, dmat, col_y, am_grad, S, T, C, ldd, term);
  if (S > 0) {  // the double path keeps the separate per-symbol scatter
    const long n = (long)B * T;
    hipLaunchKernelGGL(simple_bwd_symbols_kernel<double>, dim3((unsigned)((n + 255) / 256)),
                       dim3(256), 0, stream, gpx, symbols, boundary, am_grad, B, S, T, C,
                       rnnt_type);
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
    // (the grid always has at least one column of tiles, so that the -inf column of
    // an empty-frame regular lattice is still written)
    launch_fwd_gemm(lm, am, symbols, boundary, lm_max, am_max, px, py, norm_raw, B, S, T, C, term,
                    rnnt_type, stream);
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
             const R *lm_max, const R *am_max, const R *norm_raw, const R *score_grad, R *px_grad,
             R *py_grad, R *dmat, R *row_x, R *row_y, R *col_y, R *lm_grad, R *am_grad, int B,
             int S, int T, int C, int term, int rnnt_type, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "simple_logprobs_bwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "simple_logprobs_bwd: bad rnnt_type or termination symbol");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !lm_max || !am_max || !norm_raw || !px_grad ||
      !py_grad || !dmat || !row_x || !row_y || !col_y)
    return fail(FRNNT_EINVAL, "simple_logprobs_bwd: null pointer");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (score_grad) {
    const int T1 = rnnt_type == kRegular ? T + 1 : T;
    const long per_x = (long)S * T1, per_y = (long)(S + 1) * T;
    const long total = (per_x + per_y) * B;
    if (total > 0)
      hipLaunchKernelGGL(scale_by_batch_kernel<R>, dim3((unsigned)((total + 255) / 256)),
                         dim3(256), 0, stream, px_grad, py_grad, score_grad, per_x, per_y, B);
  }
  const int ldd = (T + 3) & ~3;  // leading dimension of dmat: 16-byte rows
  const long prep_blocks = ((long)B * (S + 1) + 3) / 4 + (long)B * ((T + kWave - 1) / kWave);
  hipLaunchKernelGGL(simple_bwd_prep_kernel<R>, dim3((unsigned)prep_blocks), dim3(256), 0, stream,
                     px_grad, py_grad, norm_raw, boundary, dmat, row_x, row_y, col_y, B, S, T, ldd,
                     rnnt_type);
  if (lm_grad)
    launch_bwd_lm(lm, am, symbols, lm_max, am_max, dmat, row_x, row_y, lm_grad, B, S, T, C, ldd,
                  term, stream);
  if (am_grad && T > 0)
    launch_bwd_am(lm, am, symbols, boundary, lm_max, am_max, dmat, px_grad, col_y, am_grad, B, S,
                  T, C, ldd, term, rnnt_type, stream);
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
                                  const float *am_max, const float *norm_raw,
                                  const float *score_grad, float *px_grad, float *py_grad,
                                  float *dmat, float *row_x, float *row_y, float *col_y,
                                  float *lm_grad, float *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, void *stream) {
  return frnnt::bwd_impl<float>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, score_grad,
                                px_grad, py_grad, dmat, row_x, row_y, col_y, lm_grad, am_grad, B,
                                S, T, C, termination_symbol, rnnt_type, stream);
}
int frnnt_simple_logprobs_bwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, const double *lm_max,
                                  const double *am_max, const double *norm_raw,
                                  const double *score_grad, double *px_grad, double *py_grad,
                                  double *dmat, double *row_x, double *row_y, double *col_y,
                                  double *lm_grad, double *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, void *stream) {
  return frnnt::bwd_impl<double>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, score_grad,
                                 px_grad, py_grad, dmat, row_x, row_y, col_y, lm_grad, am_grad, B,
                                 S, T, C, termination_symbol, rnnt_type, stream);
}

}  // extern "C"
