// The lm-only / am-only smoothing of get_rnnt_logprobs_smoothed
// (fast_rnnt/python/fast_rnnt/rnnt_loss.py:1135-1369) and its backward.
//
// With pj / qj the joint px / py (from frnnt_simple_logprobs_fwd) and
//   sigma[b,s,c] = softmax_c lm[b,s,:]            Ln[b,s]  = logsumexp_c lm[b,s,:]
//   U[c]         = mean_{b,s} sigma[b,s,c] + tiny                      ("unigram lm")
//   An[b,t]      = log sum_c exp(am[b,t,c]) U[c]
// the reference forms, left to right,
//   px = pj * k + (lm[b,s,sym] - Ln[b,s]) * l + ((am[b,t,sym] + log U[sym]) - An[b,t]) * a
//   py = qj * k + (lm[b,s,term] - Ln[b,s]) * l + ((am[b,t,term] + log U[term]) - An[b,t]) * a
// (k = 1 - l - a; for the regular lattice the am-only part of column T is -inf).
//
// Everything here is row-wise streaming work (one wave per lm or am row) plus two
// reductions over the whole batch -- U over the lm rows, and in the backward pass the
// gradient of U over the am rows -- which run in two deterministic stages (per-block
// partial sums, then a sum over blocks).  The gradients follow from the formulas above:
//   d/d lm[b,s,c] = l ([c=sym] rx + [c=term] ry) - l (rx + ry) sigma
//                   + sigma (gU[c] - sum_c' sigma[c'] gU[c']) / N
//   d/d am[b,t,c] = a (sum_s [c=sym_s] gx[b,s,t] + [c=term] cy[b,t]) - a G[b,t] q[b,t,c]
//   gU[c] = a (sum_{(b,s): sym=c} rx[b,s] + [c=term] sum_{b,s} ry[b,s]) / U[c]
//           - a sum_{b,t} G[b,t] exp(am[b,t,c] - max) / Z[b,t]
// with rx / ry the row sums of the incoming px / py gradients, cy / G the column sums of
// gy / gx + gy, q = exp(am - max) U / Z the am-only posterior and Z = exp(An - max).
#include "common.hip.h"

namespace frnnt {
namespace {

constexpr int kRowsPerBlock = 16;  // rows summed by one block of the batch reductions

template <typename R>
__device__ __forceinline__ R wave_max_nan(R v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const R o = __shfl_xor(v, off, 64);
    v = (o > v || o != o) ? o : v;
  }
  return v;
}
template <typename R>
__device__ __forceinline__ R wave_total(R v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
template <typename R>
__device__ __forceinline__ R tiny_value();
template <>
__device__ __forceinline__ float tiny_value<float>() {
  return 1.17549435e-38f;
}
template <>
__device__ __forceinline__ double tiny_value<double>() {
  return 2.2250738585072014e-308;
}

// ---- forward ------------------------------------------------------------------------

// one wave per lm row: maximum and sum of exp(x - max)
template <typename R>
__global__ void __launch_bounds__(256)
    lm_row_stats_kernel(const R *__restrict__ lm, R *__restrict__ row_max, R *__restrict__ row_sum,
                        long rows, int C) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const R *x = lm + row * C;
  R m = Num<R>::neg_inf();
  for (int c = lane; c < C; c += kWave) {
    const R v = x[c];
    m = (v > m || v != v) ? v : m;
  }
  m = wave_max_nan(m);
  R sum = 0;
  for (int c = lane; c < C; c += kWave) sum += Num<R>::exp_(x[c] - m);
  sum = wave_total(sum);
  if (lane == 0) {
    row_max[row] = m;
    row_sum[row] = sum;
  }
}

// partial[block][c] = sum over the block's rows of weight[row] * exp(x[row][c] - max[row]) * scale[row]
// (scale = 1 / row_sum for the unigram, weight absent; for the backward reduction over am
// rows weight[row] / z[row]).  Threads walk c, rows are visited in order.
template <typename R>
__global__ void __launch_bounds__(256)
    weighted_column_partial_kernel(const R *__restrict__ x, const R *__restrict__ row_max,
                                   const R *__restrict__ numer, const R *__restrict__ denom,
                                   R *__restrict__ partial, long rows, int C) {
  const long row0 = (long)blockIdx.x * kRowsPerBlock;
  // per-row weight and maximum (the same for every thread); rows past the end weigh nothing
  R w[kRowsPerBlock], m[kRowsPerBlock];
  long at[kRowsPerBlock];
#pragma unroll
  for (int k = 0; k < kRowsPerBlock; ++k) {
    const bool ok = row0 + k < rows;
    const long row = ok ? row0 + k : row0;
    w[k] = ok ? (numer ? numer[row] : (R)1) / denom[row] : (R)0;
    m[k] = row_max[row];
    at[k] = row * C;
  }
  for (int c = threadIdx.x; c < C; c += 256) {
    R v[kRowsPerBlock];
#pragma unroll
    for (int k = 0; k < kRowsPerBlock; ++k) v[k] = x[at[k] + c];  // all in flight
    R acc = 0;
#pragma unroll
    for (int k = 0; k < kRowsPerBlock; ++k)
      if (row0 + k < rows) acc += Num<R>::exp_(v[k] - m[k]) * w[k];
    partial[(long)blockIdx.x * C + c] = acc;
  }
}

// The reductions over all rows of the batch end in a sum per vocabulary entry.  A block
// of 1024 threads takes 16 entries: 64 groups of 16 threads, every group walks its share
// of the rows (64-byte reads, eight in flight: with some hundred rows a single request
// round), and the groups' sums meet in LDS in a fixed order, so the result does not
// depend on timing.
constexpr int kColsPerBlock = 16;
constexpr int kRowGroups = 64;
constexpr int kUnigramThreads = kColsPerBlock * kRowGroups;

template <typename R>
__device__ __forceinline__ R sum_of_groups(R mine, R (*meet)[kColsPerBlock], int col, int grp) {
  meet[grp][col] = mine;
  __syncthreads();
  R total = 0;
  if (grp == 0)
#pragma unroll
    for (int k = 0; k < kRowGroups; ++k) total += meet[k][col];
  return total;  // meaningful in group 0
}

// sum over this group's share of the partial rows, eight loads in flight, added in order
template <typename R>
__device__ __forceinline__ R sum_partials(const R *__restrict__ partial, int blocks, int C, int c,
                                          int grp) {
  R acc = 0;
  int k = grp;
  for (; k < blocks; k += 8 * kRowGroups) {
    R v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      v[u] = k + u * kRowGroups < blocks ? partial[(long)(k + u * kRowGroups) * C + c] : (R)0;
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  return acc;
}

// unigram[c] = (sum of the partials) / N + tiny
template <typename R>
__global__ void __launch_bounds__(kUnigramThreads)
    unigram_final_kernel(const R *__restrict__ partial, R *__restrict__ unigram, int blocks, long N,
                         int C) {
  __shared__ R meet[kRowGroups][kColsPerBlock];
  const int col = threadIdx.x % kColsPerBlock, grp = threadIdx.x / kColsPerBlock;
  const int c = blockIdx.x * kColsPerBlock + col;
  R acc = c < C ? sum_partials(partial, blocks, C, c, grp) : (R)0;
  acc = sum_of_groups(acc, meet, col, grp);
  if (grp == 0 && c < C) unigram[c] = acc / (R)N + tiny_value<R>();
}

// one wave per am row: maximum and z = sum_c exp(x - max) unigram[c]
template <typename R>
__global__ void __launch_bounds__(256)
    am_row_stats_kernel(const R *__restrict__ am, const R *__restrict__ unigram,
                        R *__restrict__ row_max, R *__restrict__ row_z, long rows, int C) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const R *x = am + row * C;
  R m = Num<R>::neg_inf();
  for (int c = lane; c < C; c += kWave) {
    const R v = x[c];
    m = (v > m || v != v) ? v : m;
  }
  m = wave_max_nan(m);
  R z = 0;
  for (int c = lane; c < C; c += kWave) z += Num<R>::exp_(x[c] - m) * unigram[c];
  z = wave_total(z);
  if (lane == 0) {
    row_max[row] = m;
    row_z[row] = z;
  }
}

// one thread per px / py element, t fastest
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_combine_kernel(const R *__restrict__ lm, const R *__restrict__ am,
                            const int64_t *__restrict__ symbols,
                            const int64_t *__restrict__ boundary, const R *__restrict__ pxj,
                            const R *__restrict__ pyj, const R *__restrict__ lm_max,
                            const R *__restrict__ lm_sum, const R *__restrict__ am_max,
                            const R *__restrict__ am_z, const R *__restrict__ unigram,
                            R *__restrict__ px, R *__restrict__ py, int B, int S, int T, int C,
                            int term, int regular, R k_joint, R k_lm, R k_am) {
  const int T1 = regular ? T + 1 : T;
  const int S1 = S + 1;
  const long n_px = (long)B * S * T1, n_py = (long)B * S1 * T;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx < n_px) {
    const int t = (int)(idx % T1);
    const long bs = idx / T1;
    const int s = (int)(bs % S), b = (int)(bs / S);
    const long lrow = (long)b * S1 + s;
    const int64_t sym = symbols[(long)b * S + s];
    const bool in = sym >= 0 && sym < C;
    const R nan = std::numeric_limits<R>::quiet_NaN();
    const R ln = log(lm_sum[lrow]) + lm_max[lrow];
    const R lm_only = (in ? lm[lrow * C + sym] : nan) - ln;
    R am_only = Num<R>::neg_inf();
    if (t < T) {
      const long arow = (long)b * T + t;
      const R an = log(am_z[arow]) + am_max[arow];
      am_only = ((in ? am[arow * C + sym] : nan) + (in ? log(unigram[sym]) : nan)) - an;
    }
    R v = pxj[idx] * k_joint + lm_only * k_lm + am_only * k_am;
    // nothing can be emitted after an utterance's last frame (fix_for_boundary,
    // rnnt_loss.py:45-63, applied by the reference after the interpolation)
    if (boundary && regular && boundary[4 * b + 3] == t) v = Num<R>::neg_inf();
    px[idx] = v;
  } else if (idx < n_px + n_py) {
    const long j = idx - n_px;
    const int t = (int)(j % T);
    const long lrow = j / T;
    const int b = (int)(lrow / S1);
    const long arow = (long)b * T + t;
    const R ln = log(lm_sum[lrow]) + lm_max[lrow];
    const R an = log(am_z[arow]) + am_max[arow];
    const R lm_only = lm[lrow * C + term] - ln;
    const R am_only = (am[arow * C + term] + log(unigram[term])) - an;
    py[j] = pyj[j] * k_joint + lm_only * k_lm + am_only * k_am;
  }
}

// The same interpolation, a workgroup per (utterance, 8 frames).  The elementwise form above
// reads am[b, t, sym[b, s]] with t along the lanes: a different 4 C-byte row -- a whole cache
// line -- for every cell (B = 32, S = 80, T = 250, C = 500: 77 MB fetched for 5 MB written).
// Here the tile's am values are gathered once with s along the lanes (the lanes of a frame
// share its row's lines) into LDS, the per-row terms of lm and the per-frame normalizers are
// staged beside them, and px / py leave with t along the lanes.  Same operations in the same
// order as the elementwise form: bit-identical results.
constexpr int kCombineFrames = 8;
template <typename R>
size_t combine_tile_lds_bytes(int S) {
  const int S1 = S + 1, pitch = S1 | 1;
  return ((size_t)kCombineFrames * pitch + 3 * (size_t)S1 + kCombineFrames) * sizeof(R);
}
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_combine_tile_kernel(const R *__restrict__ lm, const R *__restrict__ am,
                                 const int64_t *__restrict__ symbols,
                                 const int64_t *__restrict__ boundary, const R *__restrict__ pxj,
                                 const R *__restrict__ pyj, const R *__restrict__ lm_max,
                                 const R *__restrict__ lm_sum, const R *__restrict__ am_max,
                                 const R *__restrict__ am_z, const R *__restrict__ unigram,
                                 R *__restrict__ px, R *__restrict__ py, int S, int T, int C,
                                 int term, int regular, R k_joint, R k_lm, R k_am) {
  extern __shared__ __align__(16) unsigned char combine_lds[];
  const int S1 = S + 1, T1 = regular ? T + 1 : T, pitch = S1 | 1;
  R *am_s = reinterpret_cast<R *>(combine_lds);  // [32][pitch]: am[t][sym[s]], column S: am[t][term]
  R *lm_x = am_s + kCombineFrames * pitch;        // [S1] lm[s][sym[s]] - log-normalizer of row s
  R *lm_y = lm_x + S1;                            // [S1] lm[s][term] - log-normalizer of row s
  R *lu_s = lm_y + S1;                            // [S1] log(unigram[sym[s]]), entry S: log(unigram[term])
  R *an_s = lu_s + S1;                            // [32] log-normalizer of the am-only model per frame
  const int b = blockIdx.y, t0 = blockIdx.x * kCombineFrames;
  const int tid = threadIdx.x;
  const R nan = std::numeric_limits<R>::quiet_NaN();
  const R ninf = Num<R>::neg_inf();
  for (int s = tid; s < S1; s += 256) {
    const long lrow = (long)b * S1 + s;
    const R ln = log(lm_sum[lrow]) + lm_max[lrow];
    lm_y[s] = lm[lrow * C + term] - ln;
    if (s < S) {
      const int64_t sym = symbols[(long)b * S + s];
      const bool in = sym >= 0 && sym < C;
      lm_x[s] = (in ? lm[lrow * C + sym] : nan) - ln;
      lu_s[s] = in ? log(unigram[sym]) : nan;
    } else {
      lu_s[s] = log(unigram[term]);
    }
  }
  if (tid < kCombineFrames) {
    const int t = t0 + tid;
    if (t < T) {
      const long arow = (long)b * T + t;
      an_s[tid] = log(am_z[arow]) + am_max[arow];
    }
  }
  for (int i = tid; i < kCombineFrames * S1; i += 256) {
    const int tl = i / S1, s = i - tl * S1, t = t0 + tl;
    if (t >= T) continue;
    int64_t col = term;
    if (s < S) col = symbols[(long)b * S + s];
    am_s[tl * pitch + s] = (col >= 0 && col < C) ? am[((long)b * T + t) * C + col] : nan;
  }
  __syncthreads();
  const int t_mask = (boundary && regular) ? (int)boundary[4 * b + 3] : -1;
  const R *pxjb = pxj + (long)b * S * T1;
  R *pxb = px + (long)b * S * T1;
  for (int i = tid; i < kCombineFrames * S; i += 256) {
    const int s = i / kCombineFrames, tl = i % kCombineFrames, t = t0 + tl;
    if (t >= T1) continue;
    R am_only = ninf;
    if (t < T) am_only = (am_s[tl * pitch + s] + lu_s[s]) - an_s[tl];
    R v = pxjb[(long)s * T1 + t] * k_joint + lm_x[s] * k_lm + am_only * k_am;
    // nothing can be emitted after an utterance's last frame (fix_for_boundary,
    // rnnt_loss.py:45-63, applied by the reference after the interpolation)
    if (t == t_mask) v = ninf;
    pxb[(long)s * T1 + t] = v;
  }
  const R *pyjb = pyj + (long)b * S1 * T;
  R *pyb = py + (long)b * S1 * T;
  for (int i = tid; i < kCombineFrames * S1; i += 256) {
    const int s = i / kCombineFrames, tl = i % kCombineFrames, t = t0 + tl;
    if (t >= T) continue;
    const R am_only = (am_s[tl * pitch + S] + lu_s[S]) - an_s[tl];
    pyb[(long)s * T + t] = pyjb[(long)s * T + t] * k_joint + lm_y[s] * k_lm + am_only * k_am;
  }
}

// ---- backward -----------------------------------------------------------------------

// Row sums rx, ry (one wave per lattice row; rx over all T1 columns) and column sums
// cy = sum_s gy, G = sum_s (gx + gy) over the frames (64 frames per block, waves split
// the rows); also the gradients of the joint inputs, k * (gx, gy).
// t_masks (optional): per utterance the frame whose px the forward kernel set to -inf for
// the regular lattice; like the reference's scatter_ there (rnnt_loss.py:45-63) that cuts
// the gradient, whatever the recursion left in px_grad at those cells (1 when no path
// exists at all, 0 otherwise).
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_bwd_sums_kernel(const R *__restrict__ gpx, const R *__restrict__ gpy,
                             const int64_t *__restrict__ boundary,
                             R *__restrict__ gxj, R *__restrict__ gyj, R *__restrict__ row_x,
                             R *__restrict__ row_y, R *__restrict__ col_y, R *__restrict__ col_g,
                             int B, int S, int T, int T1, R k_joint) {
  __shared__ R part[2][4][kWave];
  const int S1 = S + 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long n_rows = (long)B * S1;
  const long row_blocks = (n_rows + 3) / 4;
  if (blockIdx.x < row_blocks) {
    const long row = (long)blockIdx.x * 4 + wave;
    if (row >= n_rows) return;
    const int b = (int)(row / S1), s = (int)(row % S1);
    const int t_mask = boundary ? (int)boundary[4 * b + 3] : -1;
    R sx = 0, sy = 0;
    if (s < S) {
      const long o = ((long)b * S + s) * T1;
      for (int t = lane; t < T1; t += kWave) {
        const R v = t == t_mask ? (R)0 : gpx[o + t];
        gxj[o + t] = v * k_joint;
        sx += v;
      }
    }
    const long o = row * T;
    for (int t = lane; t < T; t += kWave) {
      const R v = gpy[o + t];
      gyj[o + t] = v * k_joint;
      sy += v;
    }
    sx = wave_total(sx);
    sy = wave_total(sy);
    if (lane == 0) {
      row_x[row] = sx;
      row_y[row] = sy;
    }
  } else {
    const int tiles = (T + kWave - 1) / kWave;
    const long cb = blockIdx.x - row_blocks;
    const int b = (int)(cb / tiles), t = (int)(cb % tiles) * kWave + lane;
    const bool ok = t < T;
    const bool masked = boundary && boundary[4 * b + 3] == t;
    R ax = 0, ay = 0;
    for (int s = wave; s < S1; s += 4) {
      if (ok) {
        ay += gpy[((long)b * S1 + s) * T + t];
        if (s < S && !masked) ax += gpx[((long)b * S + s) * T1 + t];
      }
    }
    part[0][wave][lane] = ax;
    part[1][wave][lane] = ay;
    __syncthreads();
    if (wave == 0 && ok) {
      const R x = (part[0][0][lane] + part[0][1][lane]) + (part[0][2][lane] + part[0][3][lane]);
      const R y = (part[1][0][lane] + part[1][1][lane]) + (part[1][2][lane] + part[1][3][lane]);
      col_y[(long)b * T + t] = y;
      col_g[(long)b * T + t] = x + y;
    }
  }
}

// gU[c] = a (sum_{(b,s): sym=c} rx + [c=term] sum ry) / U[c] - a sum of the partials,
// the partials being sum_rows G[row] exp(am - max) / z[row].  Same layout as
// unigram_final_kernel.  The (b, s) pairs pass through LDS in chunks -- symbol and
// row_x, fetched once by the whole block -- and every group scans a contiguous share
// of each chunk.
constexpr int kPairChunk = 2048;

template <typename R>
__global__ void __launch_bounds__(kUnigramThreads)
    unigram_grad_kernel(const R *__restrict__ partial, const int64_t *__restrict__ symbols,
                        const R *__restrict__ row_x, const R *__restrict__ row_y,
                        const R *__restrict__ unigram, R *__restrict__ g_unigram, int blocks,
                        int B, int S, int C, int term, R k_am) {
  __shared__ R meet[kRowGroups][kColsPerBlock];
  __shared__ int pair_sym[kPairChunk];
  __shared__ R pair_x[kPairChunk];
  const int col = threadIdx.x % kColsPerBlock, grp = threadIdx.x / kColsPerBlock;
  const int c = blockIdx.x * kColsPerBlock + col;
  const int S1 = S + 1, n = B * S1;
  R acc = c < C ? sum_partials(partial, blocks, C, c, grp) : (R)0, direct = 0;
  for (int row0 = 0; row0 < n; row0 += kPairChunk) {
    const int count = min(kPairChunk, n - row0);
    __syncthreads();
    for (int i = threadIdx.x; i < count; i += kUnigramThreads) {
      const int row = row0 + i, b = row / S1, s = row - b * S1;
      const int64_t y = s < S ? symbols[(long)b * S + s] : -1;
      pair_sym[i] = (y >= 0 && y < C) ? (int)y : -1;
      pair_x[i] = row_x[row];
    }
    __syncthreads();
    const int share = (count + kRowGroups - 1) / kRowGroups;
    const int first = grp * share, last = min(first + share, count);
    for (int i = first; i < last; ++i)
      if (pair_sym[i] == c) direct += pair_x[i];
  }
  // the termination symbol's column also takes the sum of row_y over all rows: the whole
  // block adds it up (every thread a strided share, eight loads in flight, then a fixed
  // tree), not the sixteen threads of that column alone
  if (term / kColsPerBlock == (int)blockIdx.x) {  // (uniform)
    R part = 0;
    for (int row0 = threadIdx.x; row0 < n; row0 += 8 * kUnigramThreads) {
      R v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[u] = row0 + u * kUnigramThreads < n ? row_y[row0 + u * kUnigramThreads] : (R)0;
#pragma unroll
      for (int u = 0; u < 8; ++u) part += v[u];
    }
    __syncthreads();  // pair_x is free now
    pair_x[threadIdx.x] = part;
    __syncthreads();
    for (int off = kUnigramThreads / 2; off > 0; off >>= 1) {
      if ((int)threadIdx.x < off) pair_x[threadIdx.x] += pair_x[threadIdx.x + off];
      __syncthreads();
    }
    if (c == term && grp == 0) direct += pair_x[0];
  }
  acc = sum_of_groups(acc, meet, col, grp);
  __syncthreads();
  direct = sum_of_groups(direct, meet, col, grp);
  if (grp == 0 && c < C) g_unigram[c] = k_am * direct / unigram[c] - k_am * acc;
}

// one wave per lm row
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_bwd_lm_kernel(const R *__restrict__ lm, const int64_t *__restrict__ symbols,
                           const R *__restrict__ lm_max, const R *__restrict__ lm_sum,
                           const R *__restrict__ row_x, const R *__restrict__ row_y,
                           const R *__restrict__ g_unigram, R *__restrict__ lm_grad, long rows,
                           int S, int C, int term, R k_lm, R inv_n) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const int S1 = S + 1;
  const int b = (int)(row / S1), s = (int)(row % S1);
  const R *x = lm + row * C;
  const R m = lm_max[row], inv = (R)1 / lm_sum[row];
  R dot = 0;
  for (int c = lane; c < C; c += kWave) dot += Num<R>::exp_(x[c] - m) * inv * g_unigram[c];
  dot = wave_total(dot);
  const R rx = row_x[row], ry = row_y[row];
  const int64_t sym = s < S ? symbols[(long)b * S + s] : -1;
  R *g = lm_grad + row * C;
  for (int c = lane; c < C; c += kWave) {
    const R sigma = Num<R>::exp_(x[c] - m) * inv;
    R v = sigma * ((g_unigram[c] - dot) * inv_n - k_lm * (rx + ry));
    if (c == sym) v += k_lm * rx;
    if (c == term) v += k_lm * ry;
    g[c] = v;
  }
}

// one wave per am row: everything but the per-symbol terms
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_bwd_am_kernel(const R *__restrict__ am, const R *__restrict__ am_max,
                           const R *__restrict__ am_z, const R *__restrict__ unigram,
                           const R *__restrict__ col_y, const R *__restrict__ col_g,
                           R *__restrict__ am_grad, long rows, int C, int term, R k_am) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const R *x = am + row * C;
  const R m = am_max[row];
  const R w = -k_am * col_g[row] / am_z[row];
  const R cy = k_am * col_y[row];
  R *g = am_grad + row * C;
  for (int c = lane; c < C; c += kWave) {
    R v = w * Num<R>::exp_(x[c] - m) * unigram[c];
    if (c == term) v += cy;
    g[c] = v;
  }
}

// am_grad[b,t,sym] += a * sum over the rows s' >= s with the same symbol of gx[b,s',t]:
// one block per (b, s); only the first row of each symbol works, so a column of
// am_grad[b] has one owner and the rows are added in order.
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_bwd_symbols_kernel(const R *__restrict__ gpx, const int64_t *__restrict__ symbols,
                                const int64_t *__restrict__ boundary, R *__restrict__ am_grad,
                                int S, int T, int T1, int C, R k_am) {
  const int b = blockIdx.x / S, s = blockIdx.x % S;
  const int t_mask = boundary ? (int)boundary[4 * b + 3] : -1;
  const int64_t *sym_b = symbols + (long)b * S;
  const int64_t sym = sym_b[s];
  if (sym < 0 || sym >= C) return;
  for (int k = 0; k < s; ++k)
    if (sym_b[k] == sym) return;  // an earlier row owns this symbol
  for (int t = threadIdx.x; t < T; t += 256) {
    R acc = 0;
    for (int k = s; k < S; ++k)
      if (sym_b[k] == sym && t != t_mask) acc += gpx[((long)b * S + k) * T1 + t];
    am_grad[((long)b * T + t) * C + sym] += k_am * acc;
  }
}

// The am row kernel with the per-symbol terms folded in:
// am_grad[b,t,sym[b,s]] += a * gx[b,s,t] for every s.  A wave keeps a row of C sums in
// LDS.  Lane l holds the symbols and the frame's gx of rows l, l + 64, ... (one strided
// load per 64 rows).  An integer LDS minimum per symbol names the first row that carries
// it; those rows write their gx side by side (one writer per column), and the few rows
// whose symbol occurred before add theirs afterwards one at a time, in the order of s --
// LDS carries out a wave's instructions in order, so the sum is always formed the same
// way.  That replaces a second pass that had to read, modify and write one cache line of
// am_grad per (b, s, t).
constexpr int kSymRowsPerLane = 4;  // up to 256 symbols per utterance
template <typename R>
__global__ void __launch_bounds__(256)
    smoothed_bwd_am_sym_kernel(const R *__restrict__ am, const R *__restrict__ am_max,
                               const R *__restrict__ am_z, const R *__restrict__ unigram,
                               const R *__restrict__ col_y, const R *__restrict__ col_g,
                               const R *__restrict__ gpx, const int64_t *__restrict__ symbols,
                               const int64_t *__restrict__ boundary, R *__restrict__ am_grad,
                               long rows, int S, int T, int T1, int C, int term, R k_am) {
  extern __shared__ __align__(16) unsigned char sym_lds[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register
  const long row = (long)blockIdx.x * 4 + wave;
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  R *extra = reinterpret_cast<R *>(sym_lds) + (size_t)wave * C;
  int *first = reinterpret_cast<int *>(sym_lds + (size_t)4 * C * sizeof(R)) + (size_t)wave * C;
  const int b = (int)(row / T), t = (int)(row % T);
  const bool masked = boundary && boundary[4 * b + 3] == t;  // (wave-uniform)
  int sym[kSymRowsPerLane];
  R gx[kSymRowsPerLane];
#pragma unroll
  for (int q = 0; q < kSymRowsPerLane; ++q) {
    const int s = q * kWave + lane;
    const int64_t y = s < S ? symbols[(long)b * S + s] : -1;
    sym[q] = (y >= 0 && y < C) ? (int)y : -1;
    gx[q] = (s < S && !masked) ? gpx[((long)b * S + s) * T1 + t] : (R)0;
  }
  for (int c = lane; c < C; c += kWave) {
    extra[c] = 0;
    first[c] = 0x7fffffff;
  }
#pragma unroll
  for (int q = 0; q < kSymRowsPerLane; ++q)
    if (q * kWave < S && sym[q] >= 0) atomicMin(&first[sym[q]], q * kWave + lane);
  bool later[kSymRowsPerLane];
#pragma unroll
  for (int q = 0; q < kSymRowsPerLane; ++q) {
    later[q] = false;
    if (q * kWave < S && sym[q] >= 0) {
      later[q] = first[sym[q]] != q * kWave + lane;
      if (!later[q]) extra[sym[q]] = gx[q];
    }
  }
#pragma unroll
  for (int q = 0; q < kSymRowsPerLane; ++q) {
    if (q * kWave >= S) break;
    unsigned long long todo = __ballot(later[q]);
    while (todo) {
      const int i = __ffsll((long long)todo) - 1;
      if (lane == i) extra[sym[q]] += gx[q];
      todo &= todo - 1;
    }
  }
  const R *x = am + row * C;
  const R m = am_max[row];
  const R w = -k_am * col_g[row] / am_z[row];
  const R cy = k_am * col_y[row];
  R *g = am_grad + row * C;
  for (int c = lane; c < C; c += kWave) {
    R v = w * Num<R>::exp_(x[c] - m) * unigram[c];
    if (c == term) v += cy;
    g[c] = v + k_am * extra[c];
  }
}

template <typename R>
int fwd_impl(const R *lm, const R *am, const int64_t *symbols, const int64_t *boundary,
             const R *pxj, const R *pyj, R *px,
             R *py, R *lm_max, R *lm_sum, R *am_max, R *am_z, R *unigram, R *partial, int B, int S,
             int T, int C, int term, int regular, double lm_only_scale, double am_only_scale,
             void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "smoothed_logprobs_fwd: bad size");
  if (term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "smoothed_logprobs_fwd: termination symbol outside [0, C)");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !pxj || !pyj || !px || !py || !lm_max || !lm_sum ||
      !am_max || !am_z || !unigram || !partial)
    return fail(FRNNT_EINVAL, "smoothed_logprobs_fwd: null pointer");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long n_lm = (long)B * (S + 1), n_am = (long)B * T;
  const int blocks = (int)((n_lm + kRowsPerBlock - 1) / kRowsPerBlock);
  hipLaunchKernelGGL(lm_row_stats_kernel<R>, dim3((unsigned)((n_lm + 3) / 4)), dim3(256), 0, stream,
                     lm, lm_max, lm_sum, n_lm, C);
  hipLaunchKernelGGL(weighted_column_partial_kernel<R>, dim3(blocks), dim3(256), 0, stream, lm,
                     lm_max, (const R *)nullptr, lm_sum, partial, n_lm, C);
  hipLaunchKernelGGL(unigram_final_kernel<R>, dim3((C + kColsPerBlock - 1) / kColsPerBlock), dim3(kUnigramThreads), 0, stream, partial,
                     unigram, blocks, n_lm, C);
  if (n_am > 0)
    hipLaunchKernelGGL(am_row_stats_kernel<R>, dim3((unsigned)((n_am + 3) / 4)), dim3(256), 0,
                       stream, am, unigram, am_max, am_z, n_am, C);
  const int T1 = regular ? T + 1 : T;
  const long total = (long)B * S * T1 + (long)B * (S + 1) * T;
  const R k_lm = (R)lm_only_scale, k_am = (R)am_only_scale;
  const R k_joint = (R)(1.0 - lm_only_scale - am_only_scale);
  // (the tile form needs 8 x (S + 1) values in LDS; lattices too tall for that keep the
  // elementwise form)
  const size_t tile_lds = combine_tile_lds_bytes<R>(S);
  if (total > 0 && tile_lds <= (size_t)96 * 1024 &&
      allow_lds(reinterpret_cast<const void *>(smoothed_combine_tile_kernel<R>), tile_lds))
    hipLaunchKernelGGL(smoothed_combine_tile_kernel<R>,
                       dim3((unsigned)((T1 + kCombineFrames - 1) / kCombineFrames), (unsigned)B),
                       dim3(256), tile_lds, stream, lm, am, symbols, boundary, pxj, pyj, lm_max,
                       lm_sum, am_max, am_z, unigram, px, py, S, T, C, term, regular, k_joint, k_lm,
                       k_am);
  else if (total > 0)
    hipLaunchKernelGGL(smoothed_combine_kernel<R>, dim3((unsigned)((total + 255) / 256)),
                       dim3(256), 0, stream, lm, am, symbols, boundary, pxj, pyj, lm_max, lm_sum, am_max,
                       am_z, unigram, px, py, B, S, T, C, term, regular, k_joint, k_lm, k_am);
  return check_launch("smoothed_logprobs_fwd");
}

template <typename R>
int bwd_impl(const R *lm, const R *am, const int64_t *symbols, const int64_t *boundary,
             const R *lm_max, const R *lm_sum,
             const R *am_max, const R *am_z, const R *unigram, const R *px_grad, const R *py_grad,
             R *pxj_grad, R *pyj_grad, R *lm_grad, R *am_grad, R *row_x, R *row_y, R *col_y,
             R *col_g, R *g_unigram, R *partial, int B, int S, int T, int C, int term, int regular,
             double lm_only_scale, double am_only_scale, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "smoothed_logprobs_bwd: bad size");
  if (term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "smoothed_logprobs_bwd: termination symbol outside [0, C)");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !lm_max || !lm_sum || !am_max || !am_z || !unigram ||
      !px_grad || !py_grad || !pxj_grad || !pyj_grad || !lm_grad || !am_grad || !row_x ||
      !row_y || !col_y || !col_g || !g_unigram || !partial)
    return fail(FRNNT_EINVAL, "smoothed_logprobs_bwd: null pointer");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const int T1 = regular ? T + 1 : T;
  const long n_lm = (long)B * (S + 1), n_am = (long)B * T;
  const R k_lm = (R)lm_only_scale, k_am = (R)am_only_scale;
  const R k_joint = (R)(1.0 - lm_only_scale - am_only_scale);
  const int64_t *t_masks = regular ? boundary : nullptr;
  const long sums_blocks = (n_lm + 3) / 4 + (long)B * ((T + kWave - 1) / kWave);
  hipLaunchKernelGGL(smoothed_bwd_sums_kernel<R>, dim3((unsigned)sums_blocks), dim3(256), 0, stream,
                     px_grad, py_grad, t_masks, pxj_grad, pyj_grad, row_x, row_y, col_y, col_g, B, S,
                     T, T1, k_joint);
  const int blocks = (int)((n_am + kRowsPerBlock - 1) / kRowsPerBlock);
  if (n_am > 0)
    hipLaunchKernelGGL(weighted_column_partial_kernel<R>, dim3(blocks), dim3(256), 0, stream, am,
                       am_max, col_g, am_z, partial, n_am, C);
  hipLaunchKernelGGL(unigram_grad_kernel<R>, dim3((C + kColsPerBlock - 1) / kColsPerBlock), dim3(kUnigramThreads), 0, stream, partial,
                     symbols, row_x, row_y, unigram, g_unigram, n_am > 0 ? blocks : 0, B, S, C, term,
                     k_am);
  hipLaunchKernelGGL(smoothed_bwd_lm_kernel<R>, dim3((unsigned)((n_lm + 3) / 4)), dim3(256), 0,
                     stream, lm, symbols, lm_max, lm_sum, row_x, row_y, g_unigram, lm_grad, n_lm, S, C,
                     term, k_lm, (R)(1.0 / (double)n_lm));
  if (n_am > 0) {
    // one row of sums and one of row numbers per wave in LDS, when that fits
    const size_t sym_lds = (size_t)4 * C * (sizeof(R) + sizeof(int));
    if (S > 0 && S <= kSymRowsPerLane * kWave && sym_lds <= 64 * 1024 &&
        allow_lds(reinterpret_cast<const void *>(smoothed_bwd_am_sym_kernel<R>), sym_lds)) {
      hipLaunchKernelGGL(smoothed_bwd_am_sym_kernel<R>, dim3((unsigned)((n_am + 3) / 4)), dim3(256),
                         sym_lds, stream, am, am_max, am_z, unigram, col_y, col_g, px_grad, symbols,
                         t_masks, am_grad, n_am, S, T, T1, C, term, k_am);
    } else {
      hipLaunchKernelGGL(smoothed_bwd_am_kernel<R>, dim3((unsigned)((n_am + 3) / 4)), dim3(256), 0,
                         stream, am, am_max, am_z, unigram, col_y, col_g, am_grad, n_am, C, term,
                         k_am);
      if (S > 0)
        hipLaunchKernelGGL(smoothed_bwd_symbols_kernel<R>, dim3((unsigned)(B * S)), dim3(256), 0,
                           stream, px_grad, symbols, t_masks, am_grad, S, T, T1, C, k_am);
    }
  }
  return check_launch("smoothed_logprobs_bwd");
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_smoothed_logprobs_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                    const int64_t *boundary,
                                    const float *px_joint, const float *py_joint, float *px,
                                    float *py, float *lm_max, float *lm_sum, float *am_max,
                                    float *am_z, float *unigram, float *partial, int B, int S,
                                    int T, int C, int termination_symbol, int regular,
                                    double lm_only_scale, double am_only_scale, void *stream) {
  return frnnt::fwd_impl<float>(lm, am, symbols, boundary, px_joint, py_joint, px, py, lm_max, lm_sum, am_max,
                                am_z, unigram, partial, B, S, T, C, termination_symbol, regular,
                                lm_only_scale, am_only_scale, stream);
}
int frnnt_smoothed_logprobs_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                    const int64_t *boundary,
                                    const double *px_joint, const double *py_joint, double *px,
                                    double *py, double *lm_max, double *lm_sum, double *am_max,
                                    double *am_z, double *unigram, double *partial, int B, int S,
                                    int T, int C, int termination_symbol, int regular,
                                    double lm_only_scale, double am_only_scale, void *stream) {
  return frnnt::fwd_impl<double>(lm, am, symbols, boundary, px_joint, py_joint, px, py, lm_max, lm_sum,
                                 am_max, am_z, unigram, partial, B, S, T, C, termination_symbol,
                                 regular, lm_only_scale, am_only_scale, stream);
}
int frnnt_smoothed_logprobs_bwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                    const int64_t *boundary, const float *lm_max, const float *lm_sum, const float *am_max,
                                    const float *am_z, const float *unigram, const float *px_grad,
                                    const float *py_grad, float *px_joint_grad,
                                    float *py_joint_grad, float *lm_grad, float *am_grad,
                                    float *row_x, float *row_y, float *col_y, float *col_g,
                                    float *g_unigram, float *partial, int B, int S, int T, int C,
                                    int termination_symbol, int regular, double lm_only_scale,
                                    double am_only_scale, void *stream) {
  return frnnt::bwd_impl<float>(lm, am, symbols, boundary, lm_max, lm_sum, am_max, am_z, unigram, px_grad,
                                py_grad, px_joint_grad, py_joint_grad, lm_grad, am_grad, row_x,
                                row_y, col_y, col_g, g_unigram, partial, B, S, T, C,
                                termination_symbol, regular, lm_only_scale, am_only_scale, stream);
}
int frnnt_smoothed_logprobs_bwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                    const int64_t *boundary, const double *lm_max, const double *lm_sum,
                                    const double *am_max, const double *am_z,
                                    const double *unigram, const double *px_grad,
                                    const double *py_grad, double *px_joint_grad,
                                    double *py_joint_grad, double *lm_grad, double *am_grad,
                                    double *row_x, double *row_y, double *col_y, double *col_g,
                                    double *g_unigram, double *partial, int B, int S, int T, int C,
                                    int termination_symbol, int regular, double lm_only_scale,
                                    double am_only_scale, void *stream) {
  return frnnt::bwd_impl<double>(lm, am, symbols, boundary, lm_max, lm_sum, am_max, am_z, unigram, px_grad,
                                 py_grad, px_joint_grad, py_joint_grad, lm_grad, am_grad, row_x,
                                 row_y, col_y, col_g, g_unigram, partial, B, S, T, C,
                                 termination_symbol, regular, lm_only_scale, am_only_scale, stream);
}

}  // extern "C"
