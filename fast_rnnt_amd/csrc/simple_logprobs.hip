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
#include <mutex>

#include "simple_shared.hip.h"
#include "tile_gemm.hip.h"

namespace frnnt {
namespace {


// Which XCD works on which utterance in the gradient products.  Workgroup i runs on XCD
// i % 8 and all tiles of an utterance stay on one XCD (one L2 holds its operands), so a launch of
// many tiles lasts as long as its fullest XCD; with utterance b on XCD b % 8 that is left to
// the order of the batch (ragged batches of 16 and 32 utterances: the fullest XCD 32 % and
// 19 % above the average).  The prep kernel therefore ranks the utterances by the cells of
// their windows (rank 0 = most) and the products deal them out by rank: rank r goes to XCD
// r % 8 in even rounds of eight and to 7 - r % 8 in odd ones, so that every XCD takes its
// larger utterances first (the same batches: 10 % and 1 % above the average; both products of
// the larger one 223 -> 210 us).  The utterance of rank r is kept, as an int, in
// row_x[r][S] -- the row sums of px_grad have no row S, nobody reads that entry as a number
// -- so a workgroup finds its utterance with one scalar load.  Batches of more than 64 and
// calls without a window rank by index.
template <typename R>
__device__ __forceinline__ int *rank_slot(R *row_x, int r, int S) {
  return reinterpret_cast<int *>(row_x + (long)r * (S + 1) + S);
}
// one wave: ranks the batch and leaves the utterance of every rank in its slot
template <typename R>
__device__ __forceinline__ void rank_utterances(R *row_x, const int64_t *window, int B, int S, int T,
                                                int lane) {
  if (!window || B > kWave) {
    for (int i = lane; i < B; i += kWave) *rank_slot(row_x, i, S) = i;
    return;
  }
  unsigned key = 0;  // lanes without an utterance rank behind every utterance
  if (lane < B) {
    const Limits w = limits_of(window, lane, S, T);
    const long cells = (long)max(w.s_end - w.s_begin + 1, 0) * max(w.t_end - w.t_begin, 0);
    // (distinct keys: equal sizes rank by index)
    key = ((unsigned)min(cells, 1L << 24) << 6 | (unsigned)(kWave - 1 - lane)) + 1u;
  }
  int rank = 0;
  for (int j = 0; j < B; ++j) rank += (unsigned)__builtin_amdgcn_readlane((int)key, j) > key ? 1 : 0;
  if (lane < B) *rank_slot(row_x, rank, S) = lane;
}
// With fewer than 32 utterances a unit of placement is a PART of an utterance: its tiles
// of every 2^part_shift-th stretch of the vocabulary (such tiles share D but nothing of lm or
// am), enough parts for eight units per XCD while a part keeps four tiles along the
// vocabulary.  A batch of two then reaches all eight XCDs instead of two (B = 2, S = 100,
// T = 400, C = 5000: both products 117 -> 36 us), and a batch of sixteen is dealt out in 64
// units (fullest XCD 2 % above the average instead of 10 %: 212 -> 201 us).
inline int part_shift_for(int B, int c_tiles) {
  if (B >= 32) return 0;
  int shift = 0;
  while ((B << shift) < 64 && (8 << shift) <= c_tiles) ++shift;
  return shift;
}
inline unsigned placed_grid(int c_tiles, int other_tiles, int B, int part_shift) {
  const long units = (long)B << part_shift;
  const int c_per = (c_tiles + (1 << part_shift) - 1) >> part_shift;
  return (unsigned)(dgemm::kXcds * ((units + dgemm::kXcds - 1) / dgemm::kXcds) * c_per * other_tiles);
}
// (utterance, tile, window) of workgroup `id` of a grid of placed_grid() workgroups; a tile is
// other * c_tiles + (its index along the vocabulary)
__device__ __forceinline__ bool place_block(int id, int c_tiles, int other_tiles, int part_shift,
                                            int B, const float *row_x, const int64_t *window, int S,
                                            int T, int &b, int &tile, Limits &lim) {
  using dgemm::kXcds;
  const int c_per = (c_tiles + (1 << part_shift) - 1) >> part_shift;
  const int unit_tiles = c_per * other_tiles;
  const int xcd = id % kXcds, slot = id / kXcds, round = slot / unit_tiles;
  const int within = slot - round * unit_tiles;
  const int unit = round * kXcds + ((round & 1) ? kXcds - 1 - xcd : xcd);
  const int rank = unit >> part_shift, part = unit & ((1 << part_shift) - 1);
  const int other = within / c_per, c_idx = part * c_per + (within - other * c_per);
  if (rank >= B || c_idx >= c_tiles) return false;
  tile = other * c_tiles + c_idx;
  b = *reinterpret_cast<const int *>(row_x + (long)rank * (S + 1) + S);
  lim = limits_of(window, b, S, T);
  return true;
}

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
// stored, so a row costs one memory round trip, not one per 64 frames.  The last
// workgroup ranks the utterances for the gradient products (rank_utterances).
template <typename R>
__global__ void __launch_bounds__(256)
    simple_bwd_prep_kernel(const R *__restrict__ gpx, const R *__restrict__ gpy,
                           const R *__restrict__ norm_raw, const int64_t *__restrict__ boundary,
                           const int64_t *__restrict__ window, R *__restrict__ dmat,
                           R *__restrict__ row_x, R *__restrict__ row_y, R *__restrict__ col_y,
                           int B, int S, int T, int ldd, int rnnt_type) {
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
    // outside the window nothing is read (the normalizers there may be undefined): D = 0
    const Limits lim = limits_of(window, b, S, T);
    const bool row_in = s >= lim.s_begin && s <= lim.s_end;
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
        const bool ok = t < T && row_in && t >= lim.t_begin && t < lim.t_end;
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
      if (s < S) row_x[row] = sx;  // (entry S of a row belongs to rank_utterances)
      row_y[row] = sy;
    }
  } else if (blockIdx.x == gridDim.x - 1) {
    if (wave == 0) rank_utterances(row_x, window, B, S, T, lane);
  } else {
    const int tiles = (T + kWave - 1) / kWave;
    const long cb = blockIdx.x - row_blocks;
    const int b = (int)(cb / tiles), t = (int)(cb % tiles) * kWave + lane;
    const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;
    const Limits lim = limits_of(window, b, S, T);
    const bool ok = t < T && t >= lim.t_begin && t < lim.t_end;
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
    if (wave == 0 && t < T)
      col_y[(long)b * T + t] = (partial[0][lane] + partial[1][lane]) + (partial[2][lane] + partial[3][lane]);
  }
}

// px_grad[b,:,:] *= g_b, py_grad[b,:,:] *= g_b in place, with
// g_b = scale * score_grad[b * stride].  blockIdx.y is the utterance; a workgroup
// takes 1024 consecutive elements of its px_grad part or of its py_grad part.
template <typename R>
__global__ void __launch_bounds__(256)
    scale_by_batch_kernel(R *__restrict__ gpx, R *__restrict__ gpy,
                          const R *__restrict__ score_grad, int stride, R scale, int per_x,
                          int per_y, int x_blocks) {
  const int b = blockIdx.y;
  const R g = scale * score_grad[(long)b * stride];
  const bool is_x = (int)blockIdx.x < x_blocks;
  R *base = is_x ? gpx + (long)b * per_x : gpy + (long)b * per_y;
  const int n = is_x ? per_x : per_y;
  const int first = (is_x ? blockIdx.x : blockIdx.x - x_blocks) * 1024 + threadIdx.x;
  R v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) v[u] = (first + 256 * u < n) ? base[first + 256 * u] : (R)0;
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (first + 256 * u < n) base[first + 256 * u] = v[u] * g;
}

// loss = -scores, -mean(scores) or -sum(scores); one wave
template <typename R>
__global__ void __launch_bounds__(kWave)
    loss_reduce_kernel(const R *__restrict__ scores, R *__restrict__ loss, int B, int reduction) {
  reduce_scores(scores, loss, B, reduction, (int)threadIdx.x);
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


// four consecutive floats at any element-aligned address (global memory takes
// unaligned 16-byte accesses); `valid` (0..4) leading elements are read, the rest is 0
__device__ __forceinline__ dgemm::floatx4 load4_guarded(const float *base, int off, int valid,
                                                        float fill = 0.f) {
  dgemm::floatx4 r = {fill, fill, fill, fill};
  if (valid >= 4) {
    const floatx4u t = *reinterpret_cast<const floatx4u *>(base + off);
    r[0] = t[0], r[1] = t[1], r[2] = t[2], r[3] = t[3];
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < valid) r[i] = base[off + i];
  }
  return r;
}

// ---- fp32: MFMA kernels with LDS slabs / panels (xcd_grid.hip.h) --------------------

// lm gradient:  lm.grad[s,c] = exp(lm[s,c] - max[s]) * sum_t D[s,t] exp(am[t,c] - max[t])
// + [c = sym[s]] row_x[s] + [c = term] row_y[s].  Same scheme as the normalizer GEMM:
// k runs over frames and is split between the waves of a workgroup; a wave turns its
// 32-frame slabs -- D[96 rows][32 k], fetched as coalesced 16-byte pieces and
// transposed through its own LDS region, and exp(am[32 k][32 c] - max) -- into MFMA
// operands without waiting for any other wave; the partial sums meet once at the end.
// A workgroup covers kS lattice rows x 32 vocabulary entries and takes the frames in slabs
// of kK: 96 rows with 32 frames, or 128 rows with 16 (the form that pads S+1 less, as in
// the normalizer kernel).
constexpr int kLmC = 32;
constexpr int kLmWaves = 4;
constexpr int kLmThreads = kLmWaves * kWave;
constexpr int kLmOutPitch = kLmC + 1;  // pitch of a wave's partial sums in LDS
template <int kS, int kK>
struct LmShape {
  // (row pitch of the D slab: 16-byte aligned rows, as in PanelShape)
  static constexpr int kPitch = kK + 4;
  static constexpr int kSlab = kS * kPitch + kK * kLmC;  // floats per wave: D slab, then am slab
  static constexpr int kSums = kS * kLmOutPitch;         // floats of a wave's partial sums
  static constexpr size_t kLdsBytes =
      (size_t)kLmWaves * (kSlab > kSums ? kSlab : kSums) * sizeof(float);
  static constexpr int kItems = kS * kLmC / 4 / kLmThreads;  // 16-byte outputs per thread
  static constexpr int kRowLanes = kK / 4;                   // lanes that share a row of the D slab
  static constexpr int kRowsPerLoad = kWave / kRowLanes;
  static_assert(kS % kRowsPerLoad == 0 && kK % 8 == 0 && kS % 32 == 0, "shape");
};

template <int kS, int kK>
__device__ __forceinline__ void simple_bwd_lm_slab_body(
    int block_id, const float *__restrict__ lm, const float *__restrict__ am,
    const int64_t *__restrict__ symbols, const float *__restrict__ lm_max,
    const float *__restrict__ am_max, const float *__restrict__ dmat,
    const float *__restrict__ row_x, const float *__restrict__ row_y,
    float *__restrict__ lm_grad, const int64_t *__restrict__ window, int B, int S, int T, int C,
    int ldd, int term, int part_shift) {
  using Shape = LmShape<kS, kK>;
  constexpr int kLmS = kS, kLmK = kK, kLmPitch = Shape::kPitch, kLmSlab = Shape::kSlab;
  constexpr int kLmItems = Shape::kItems;
  using namespace dgemm;
  extern __shared__ __align__(16) float lm_lds[];
  const int S1 = S + 1;
  const int c_tiles = (C + kLmC - 1) / kLmC, s_tiles = (S1 + kLmS - 1) / kLmS;
  int b, tile;
  Limits lim;
  if (!place_block(block_id, c_tiles, s_tiles, part_shift, B, row_x, window, S, T, b, tile, lim))
    return;
  const int s_tile = (tile / c_tiles) * kLmS, c_tile = (tile % c_tiles) * kLmC;
  const float *lmb = lm + (long)b * S1 * C;
  const float *amb = am + (long)b * T * C;
  const float *lmx = lm_max + (long)b * S1;
  const float *amx = am_max + (long)b * T;
  const float *db = dmat + (long)b * S1 * ldd;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, r32 = lane & 31;
  // With a window, D vanishes at frames >= t_end and on rows > s_end: the sum over frames
  // stops at t_end (the row maxima of later frames may not even be defined) and 32-row
  // tiles past s_end are left at 0.
  const int t_lim = __builtin_amdgcn_readfirstlane(lim.t_end);
  const int s_lim = __builtin_amdgcn_readfirstlane(min(S1, lim.s_end + 1));

  // what this lane fetches of every slab: D rows sub_a + kRowsA j at k-offset kq_a; am
  // rows (frames) sub + 8 j at vocabulary offset kq
  constexpr int kRowsA = Shape::kRowsPerLoad;
  constexpr int kLoadsA = kLmS / kRowsA, kLoadsB = kLmK / 8;
  const int sub = lane >> 3, kq = 4 * (lane & 7);
  const int sub_a = lane / Shape::kRowLanes, kq_a = 4 * (lane % Shape::kRowLanes);
  floatx4 sa[kLoadsA], sb[kLoadsB];
  float shift2[kLoadsB];  // -(the frame's maximum) * log2(e)
  // The loads go through buffer resources that cover D[b] and am[b]: one instruction
  // each, no branch; a row past the last one lies past the resource and reads as 0.
  // Frames at and past T (the last slab) must give products of 0: there D is replaced
  // by 0 (the pad of a D row is not defined; am reads as 0 or holds the next utterance's
  // frames, exp of which is finite).  Vocabulary columns at and past C belong to the next
  // row: they only feed output columns that are never written.
  typedef int intx4 __attribute__((ext_vector_type(4)));
  const __amdgpu_buffer_rsrc_t d_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(db), 0, S1 * ldd * 4, 0x00020000);
  const __amdgpu_buffer_rsrc_t am_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(amb), 0, T * C * 4, 0x00020000);
  const int d_off = ((s_tile + sub_a) * ldd + kq_a) * 4, am_off = (sub * C + c_tile + kq) * 4;  // bytes
  auto as_floats = [](intx4 raw) {
    return floatx4{__int_as_float(raw[0]), __int_as_float(raw[1]), __int_as_float(raw[2]),
                   __int_as_float(raw[3])};
  };
  auto fetch = [&](int k0) {
#pragma unroll
    for (int j = 0; j < kLoadsA; ++j)
      sa[j] = as_floats(__builtin_amdgcn_raw_buffer_load_b128(
          d_rs, d_off, (kRowsA * j * ldd + k0) * 4, 0));  // (uniform part: scalar register)
    if (k0 + kLmK > t_lim) {  // (wave-uniform) the slab that holds the last frame
#pragma unroll
      for (int j = 0; j < kLoadsA; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (k0 + kq_a + i >= t_lim) sa[j][i] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < kLoadsB; ++j) {
      const int tr = k0 + sub + 8 * j;
      sb[j] = as_floats(__builtin_amdgcn_raw_buffer_load_b128(
          am_rs, am_off, (k0 + 8 * j) * C * 4, 0));
      shift2[j] = tr < t_lim ? -amx[tr] * kLog2e : 0.f;
      // a frame past the last one meets D = 0; its factor only has to be finite
      if (tr >= t_lim) sb[j] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
  };
  const int chunks = (t_lim + kLmK - 1) / kLmK;
  int chunk = wave;
  if (chunk < chunks) fetch(chunk * kLmK);

  // epilogue inputs behind the first slab: this thread's pieces of lm (row item / 8,
  // vocabulary entries 4 (item % 8) ..)
  floatx4 lm_in[kLmItems];
#pragma unroll
  for (int j = 0; j < kLmItems; ++j) {
    const int item = tid + kLmThreads * j;
    const int sr = s_tile + item / 8, c = c_tile + 4 * (item % 8);
    lm_in[j] = load4_guarded(lmb, sr * C + c, sr < S1 ? min(4, max(C - c, 0)) : 0);
  }
  // ... and its rows' maximum, symbol and row sums
  float row_mx[kLmItems], row_rx[kLmItems], row_ry[kLmItems];
  int row_sym[kLmItems];
#pragma unroll
  for (int j = 0; j < kLmItems; ++j) {
    const int sr = s_tile + (tid + kLmThreads * j) / 8;
    const bool ok = sr < S1;
    row_mx[j] = ok ? lmx[sr] : 0.f;
    row_sym[j] = sr < S ? (int)symbols[(long)b * S + sr] : -1;
    row_rx[j] = ok ? row_x[(long)b * S1 + sr] : 0.f;
    row_ry[j] = ok ? row_y[(long)b * S1 + sr] : 0.f;
  }

  const int live_tiles = min(kLmS / 32, (s_lim - s_tile + 31) / 32);  // 32-row tiles with rows that count
  float *as = lm_lds + wave * kLmSlab;
  float *bs = as + kLmS * kLmPitch;
  floatx16 acc[kLmS / 32];
#pragma unroll
  for (int j = 0; j < kLmS / 32; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
  for (; chunk < chunks; chunk += kLmWaves) {
#pragma unroll
    for (int j = 0; j < kLoadsA; ++j)
      *reinterpret_cast<floatx4 *>(as + (sub_a + kRowsA * j) * kLmPitch + kq_a) = sa[j];
#pragma unroll
    for (int j = 0; j < kLoadsB; ++j) {
      floatx4 e;
#pragma unroll
      for (int i = 0; i < 4; ++i) e[i] = exp_shifted(sb[j][i], shift2[j]);
      *reinterpret_cast<floatx4 *>(bs + (sub + 8 * j) * kLmC + kq) = e;
    }
    if (chunk + kLmWaves < chunks) fetch((chunk + kLmWaves) * kLmK);
    // MFMA i of the slab multiplies frames i (lanes 0..31) and i + kK / 2 (lanes 32..63) -- the
    // order in which a slab's frames are summed is free -- so that a lane takes its D row's
    // share of the slab with 16-byte reads
    constexpr int kHalfK = kLmK / 2;
    const float *ap = as + r32 * kLmPitch + kHalfK * half;
    const float *bp = bs + kHalfK * half * kLmC + r32;
    float bv[kHalfK];
#pragma unroll
    for (int i = 0; i < kHalfK; ++i) bv[i] = bp[i * kLmC];
#pragma unroll
    for (int j = 0; j < kLmS / 32; ++j)
      if (j < live_tiles) {
#pragma unroll
        for (int i4 = 0; i4 < kHalfK / 4; ++i4) {
          const floatx4 a = *reinterpret_cast<const floatx4 *>(ap + j * 32 * kLmPitch + 4 * i4);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], bv[4 * i4 + i], acc[j], 0, 0, 0);
        }
      }
  }

  // the partial sums meet: [wave][kS][33] in the slab space
  __syncthreads();
  float *part = lm_lds + wave * Shape::kSums;
#pragma unroll
  for (int j = 0; j < kLmS / 32; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      part[(32 * j + 8 * (v / 4) + 4 * half + (v % 4)) * kLmOutPitch + r32] = acc[j][v];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kLmItems; ++j) {
    const int item = tid + kLmThreads * j;
    const int m = item / 8, n = 4 * (item % 8), sr = s_tile + m, c = c_tile + n;
    if (sr >= S1 || c >= C) continue;
    const float mx = row_mx[j], rx = row_rx[j], ry = row_ry[j];
    const int sym = row_sym[j];
    float g[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kLmWaves; ++w)
        sum += lm_lds[w * Shape::kSums + m * kLmOutPitch + n + i];
      g[i] = __expf(lm_in[j][i] - mx) * sum;
      if (c + i == sym) g[i] += rx;
      if (c + i == term) g[i] += ry;
    }
    float *dst = lm_grad + ((long)b * S1 + sr) * C + c;
    if (c + 4 <= C) {
      *reinterpret_cast<floatx4u *>(dst) = floatx4u{g[0], g[1], g[2], g[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (c + i < C) dst[i] = g[i];
    }
  }
}

// am gradient, LDS-panel form.  k runs over the S+1 lattice rows, which is short, so
// a workgroup brings ALL of k (up to 128 rows per pass) for its 64 (frames) x 64
// (vocabulary) tile into LDS: D[k][t] and exp(lm[k][c] - max[k]) are both contiguous
// along the output dimension, so the panels arrive as coalesced 16-byte loads, and the
// matrix cores read the dense product's operands from LDS only.  What bounds this kernel is the number of
// vector-memory INSTRUCTIONS a compute unit can retire (an instruction costs about
// the same whether it moves 4 or 16 bytes per lane), so every global access here is
// 16 bytes wide and row-contiguous: the am tile comes in that way too, and the
// result leaves through an LDS transpose as whole 256-byte row segments.
// Every global load is in flight before the first one is consumed: a workgroup pays
// one memory round trip.
// The per-symbol term  sum_s [c = sym[b,s]] gx[b,s,t]  is a second product on the
// matrix core, gx^T times a one-hot matrix made in registers from the symbols: it is
// exact (products by 0 or 1) and has a fixed summation order; k-pairs none of whose
// symbols falls into the wave's 32 vocabulary columns are skipped (wave-uniform).  With
// a large vocabulary almost every pair is skipped, so gx has no panel: a wave reads the
// few 128-byte row pieces it needs straight from memory, the first eight of them
// requested before the dense product so that they arrive under it.
constexpr int kAmT = 64;       // frames per workgroup
constexpr int kAmC = 64;       // vocabulary entries per workgroup
constexpr int kAmHotAhead = 8; // per-symbol pairs whose gx values are requested ahead
constexpr int kAmOutPitch = 68;  // row pitch of the result tiles staged in LDS
constexpr int kAmQ = kAmT / 4;   // 16-byte pieces per panel row (kAmT == kAmC)

constexpr int kAmCap = 64;     // most lattice rows per pass
// rows of k per pass: passes of equal (even) size, none above kAmCap
int am_rows_per_pass(int S) {
  const int passes = (S + 1 + kAmCap - 1) / kAmCap;
  return std::min(kAmCap, ((S + 1 + passes - 1) / passes + 1) & ~1);
}
size_t am_panel_lds_bytes(int rows_cap) {
  const size_t panels = (size_t)rows_cap * (kAmT + kAmC) * sizeof(float);
  const size_t staging = (size_t)2 * kAmT * kAmOutPitch * sizeof(float);
  return std::max(panels, staging) + (size_t)(2 * rows_cap + 2 * kAmT) * sizeof(float);
}

// kCap: most lattice rows a pass may hold (the launch's rows_cap is at most that); it sets
// how many panel pieces a thread keeps in registers.
template <int kCap>
__device__ __forceinline__ void simple_bwd_am_panel_body(
    int block_id, const float *__restrict__ lm, const float *__restrict__ am,
    const int64_t *__restrict__ symbols, const int64_t *__restrict__ boundary,
    const float *__restrict__ lm_max, const float *__restrict__ am_max,
    const float *__restrict__ dmat, const float *__restrict__ gpx,
    const float *__restrict__ row_x, const float *__restrict__ col_y,
    float *__restrict__ am_grad, const int64_t *__restrict__ window, int B, int S, int T, int C,
    int ldd, int term, int rnnt_type, int rows_cap, int part_shift) {
  using namespace dgemm;
  extern __shared__ __align__(16) float am_lds[];
  int *sym_s = reinterpret_cast<int *>(am_lds);   // [rows_cap] symbols of the pass (-1: none)
  float *lmx_s = am_lds + rows_cap;               // [rows_cap] lm_max of the pass
  float *shift_s = lmx_s + rows_cap;              // [kAmT] am_max of the tile's frames
  float *extra_s = shift_s + kAmT;                // [kAmT] col_y of the tile's frames
  float *As = extra_s + kAmT;                     // [rows_cap][kAmT]   D[k][t]
  float *Bs = As + rows_cap * kAmT;               // [rows_cap][kAmC]   exp(lm[k][c] - max[k])
  float *out_acc = As;                            // result tiles, after the last pass
  float *out_hot = As + kAmT * kAmOutPitch;
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int c_tiles = (C + kAmC - 1) / kAmC, t_tiles = (T + kAmT - 1) / kAmT;
  int b, tile;
  Limits lim;
  if (!place_block(block_id, c_tiles, t_tiles, part_shift, B, row_x, window, S, T, b, tile, lim))
    return;
  const int t_tile = (tile / c_tiles) * kAmT, c_tile = (tile % c_tiles) * kAmC;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, r32 = lane & 31;
  const int wt = (wave >> 1) * 32, wc = (wave & 1) * 32;  // this wave's 32 x 32 sub-tile
  const float *lmb = lm + (long)b * S1 * C;
  const float *amb = am + (long)b * T * C;
  const float *db = dmat + (long)b * S1 * ldd;
  const float *gxb = gpx + (long)b * S * T1;
  // symbols are < C < 2^31: their low words (little endian) are enough to compare
  const int *sym_lo = reinterpret_cast<const int *>(symbols + (long)b * S);
  const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;
  const int c_lo = c_tile + wc;  // first vocabulary column of this wave
  // a thread's 16-byte piece of a 64-wide row: row q_row + 16 * step, columns 4 * q_col ..
  const int q_row = tid / kAmQ, q_col = 4 * (tid % kAmQ);
  // With a window, D vanishes on rows > s_end and at frames >= t_end, where the frames'
  // maxima may not even be defined: such frames get exact zeros, the sum over the lattice
  // rows stops at s_end, and a tile without a frame below t_end only stores zeros.
  const int t_lim = lim.t_end, k_lim = min(S1, lim.s_end + 1);
  if (t_tile >= t_lim) {
#pragma unroll
    for (int j = 0; j < kAmT / 16; ++j) {
      const int t = t_tile + q_row + 16 * j, c = c_tile + q_col;
      if (t >= T || c >= C) continue;
      float *dst = am_grad + ((long)b * T + t) * C + c;
      if (c + 4 <= C) {
        *reinterpret_cast<floatx4u *>(dst) = floatx4u{0.f, 0.f, 0.f, 0.f};
      } else {
        for (int i = 0; i < 4; ++i)
          if (c + i < C) dst[i] = 0.f;
      }
    }
    return;
  }

  // epilogue inputs: per-frame terms through LDS (visible after the barriers of the
  // first pass), and this thread's pieces of the am tile, rows q_row + 16 * j
  if (tid < kAmT) {
    const int t = t_tile + tid;
    shift_s[tid] = t < t_lim ? am_max[(long)b * T + t] : 0.f;
    extra_s[tid] = t < t_lim ? col_y[(long)b * T + t] : 0.f;
  }
  // The panel and tile loads go through buffer resources that cover D[b], lm[b] and
  // am[b]: one instruction each, no branch, any alignment.  A row past the last one lies
  // past the resource and reads as 0; a column past the end of a row belongs to the next
  // row, and only feeds frames >= T or vocabulary entries >= C, which are never written.
  typedef int intx4 __attribute__((ext_vector_type(4)));
  // (rows that do not count lie past the resources: they read as 0 and move no data)
  const __amdgpu_buffer_rsrc_t d_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(db), 0, k_lim * ldd * 4, 0x00020000);
  const __amdgpu_buffer_rsrc_t lm_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(lmb), 0, k_lim * C * 4, 0x00020000);
  const __amdgpu_buffer_rsrc_t am_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(amb), 0, T * C * 4, 0x00020000);
  auto get4 = [](__amdgpu_buffer_rsrc_t rs, int byte_offset) {
    const intx4 raw = __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset, 0, 0);
    return floatx4{__int_as_float(raw[0]), __int_as_float(raw[1]), __int_as_float(raw[2]),
                   __int_as_float(raw[3])};
  };
  floatx4 am_in[kAmT / 16];
#pragma unroll
  for (int j = 0; j < kAmT / 16; ++j)
    am_in[j] = get4(am_rs, ((t_tile + q_row + 16 * j) * C + c_tile + q_col) * 4);

  floatx16 acc, hot;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = hot[v] = 0.f;
  constexpr int kSteps = kCap / 16;
  constexpr int kNowhere = (int)0x80000000;  // an offset outside every resource: reads 0, moves nothing
  floatx4 ra[kSteps], rb[kSteps];
  // a pass's pieces of the two panels: rows k0 + q_row + 16 j of D and of lm, while they
  // belong to the pass
  auto request = [&](int k0) {
    const int end = min(k0 + rows_cap, k_lim);
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const int k = k0 + q_row + 16 * j;
      ra[j] = get4(d_rs, k < end ? (k * ldd + t_tile + q_col) * 4 : kNowhere);
      rb[j] = get4(lm_rs, k < end ? (k * C + c_tile + q_col) * 4 : kNowhere);
    }
  };
  request(0);
  for (int k0 = 0; k0 < k_lim; k0 += rows_cap) {
    const int rows = min(rows_cap, k_lim - k0);
    const int pairs = (rows + 1) / 2;
    if (k0 > 0) __syncthreads();  // the previous pass's readers are done with the panels
    for (int k = tid; k < 2 * pairs; k += 256) {
      sym_s[k] = (k0 + k < S) ? sym_lo[2 * (k0 + k)] : -1;
      lmx_s[k] = (k < rows) ? lm_max[(long)b * S1 + k0 + k] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const int k = q_row + 16 * j;
      if (k >= 2 * pairs) continue;
      *reinterpret_cast<floatx4 *>(As + k * kAmT + q_col) = ra[j];
    }
    __syncthreads();  // lmx_s and sym_s are visible
    // per-symbol product: the pairs with a symbol among this wave's columns ...
    bool in = false;
    if (lane < pairs)
      in = (unsigned)(sym_s[2 * lane] - c_lo) < 32u || (unsigned)(sym_s[2 * lane + 1] - c_lo) < 32u;
    unsigned long long wanted = __ballot(in);
    // ... and this lane's gx[k][t] of pair i (k = 2 i + half, t = the wave's frame r32):
    // nothing for the masked frame, past T or past the last symbol
    const int hot_t = t_tile + wt + r32;
    const bool hot_ok = hot_t < T && hot_t != t_mask;
    auto hot_value = [&](int i) {
      const int k = k0 + 2 * i + half;
      return (hot_ok && k < S) ? gxb[(long)k * T1 + hot_t] : 0.f;
    };
    int ahead[kAmHotAhead];
    float ahead_v[kAmHotAhead];
#pragma unroll
    for (int u = 0; u < kAmHotAhead; ++u) {
      ahead[u] = -1;
      ahead_v[u] = 0.f;
      if (wanted) {
        ahead[u] = __builtin_ctzll(wanted);
        wanted &= wanted - 1;
        ahead_v[u] = hot_value(ahead[u]);
      }
    }
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const int k = q_row + 16 * j, c = c_tile + q_col;
      if (k >= 2 * pairs) continue;
      const float mx = lmx_s[k];
      floatx4 e;
#pragma unroll
      for (int i = 0; i < 4; ++i) e[i] = (k < rows && c + i < C) ? __expf(rb[j][i] - mx) : 0.f;
      *reinterpret_cast<floatx4 *>(Bs + k * kAmC + q_col) = e;
    }
    // the next pass's panels are on their way while this one is multiplied
    if (k0 + rows_cap < k_lim) request(k0 + rows_cap);
    __syncthreads();
    // dense product
    const float *ap = As + half * kAmT + wt + r32;
    const float *bp = Bs + half * kAmC + wc + r32;
#pragma unroll 4
    for (int i = 0; i < pairs; ++i)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ap[2 * i * kAmT], bp[2 * i * kAmC], acc, 0, 0, 0);
    // per-symbol product
#pragma unroll
    for (int u = 0; u < kAmHotAhead; ++u) {
      if (ahead[u] < 0) continue;
      const float h = (sym_s[2 * ahead[u] + half] == c_lo + r32) ? 1.f : 0.f;
      hot = __builtin_amdgcn_mfma_f32_32x32x2f32(ahead_v[u], h, hot, 0, 0, 0);
    }
    while (wanted) {
      const int i = __builtin_ctzll(wanted);
      wanted &= wanted - 1;
      const float h = (sym_s[2 * i + half] == c_lo + r32) ? 1.f : 0.f;
      hot = __builtin_amdgcn_mfma_f32_32x32x2f32(hot_value(i), h, hot, 0, 0, 0);
    }
  }
  // results through LDS, so that they leave as whole row segments
  __syncthreads();
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = wt + 8 * (v / 4) + 4 * half + (v % 4);
    out_acc[row * kAmOutPitch + wc + r32] = acc[v];
    out_hot[row * kAmOutPitch + wc + r32] = hot[v];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kAmT / 16; ++j) {
    const int row = q_row + 16 * j, t = t_tile + row, c = c_tile + q_col;
    if (t >= T || c >= C) continue;
    const floatx4 sum = *reinterpret_cast<const floatx4 *>(out_acc + row * kAmOutPitch + q_col);
    const floatx4 one = *reinterpret_cast<const floatx4 *>(out_hot + row * kAmOutPitch + q_col);
    const float shift = shift_s[row], extra = extra_s[row];
    floatx4 res;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      res[i] = __expf(am_in[j][i] - shift) * sum[i] + one[i];
      if (c + i == term) res[i] += extra;
      if (t >= t_lim) res[i] = 0.f;
    }
    float *dst = am_grad + ((long)b * T + t) * C + c;
    if (c + 4 <= C) {
      *reinterpret_cast<floatx4u *>(dst) = floatx4u{res[0], res[1], res[2], res[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (c + i < C) dst[i] = res[i];
    }
  }
}

// launchers: float goes to the slab / panel kernels, double to the LDS-tiled ones

void launch_fwd_gemm(const float *lm, const float *am, const int64_t *symbols,
                     const int64_t *boundary, float *lm_max, float *am_max, float *px,
                     float *py, float *norm_raw, const int64_t *window, int B, int S, int T,
                     int C, int term, int rnnt_type, hipStream_t stream) {
  launch_normalizer_f32(lm, am, symbols, boundary, lm_max, am_max, px, py, norm_raw, window, B, S,
                        T, C, term, rnnt_type, stream);
}
void launch_fwd_gemm(const double *lm, const double *am, const int64_t *symbols,
                     const int64_t *boundary, const double *lm_max, const double *am_max,
                     double *px, double *py, double *norm_raw, const int64_t *, int B, int S,
                     int T, int C, int term, int rnnt_type, hipStream_t stream) {
  // (the double kernels compute the whole lattice whether or not a window is given)
  const int t_tiles = T > 0 ? (T + kTileN - 1) / kTileN : 1;
  const dim3 grid(t_tiles, (S + 1 + kTileM - 1) / kTileM, B);
  hipLaunchKernelGGL(simple_fwd_kernel<double>, grid, dim3(kGemmThreads), 0, stream, lm, am,
                     symbols, boundary, lm_max, am_max, px, py, norm_raw, S, T, C, term,
                     rnnt_type);
}
template <int kS, int kK>
__global__ void __launch_bounds__(kLmThreads, 2)
    simple_bwd_lm_slab_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                              const int64_t *__restrict__ symbols,
                              const float *__restrict__ lm_max,
                              const float *__restrict__ am_max, const float *__restrict__ dmat,
                              const float *__restrict__ row_x, const float *__restrict__ row_y,
                              float *__restrict__ lm_grad, const int64_t *__restrict__ window,
                              int B, int S, int T, int C, int ldd, int term, int part_shift) {
  simple_bwd_lm_slab_body<kS, kK>((int)blockIdx.x, lm, am, symbols, lm_max, am_max, dmat, row_x,
                                  row_y, lm_grad, window, B, S, T, C, ldd, term, part_shift);
}
template <int kCap, int kPerCu>
__global__ void __launch_bounds__(256, kPerCu)
    simple_bwd_am_panel_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                               const int64_t *__restrict__ symbols,
                               const int64_t *__restrict__ boundary,
                               const float *__restrict__ lm_max,
                               const float *__restrict__ am_max, const float *__restrict__ dmat,
                               const float *__restrict__ gpx, const float *__restrict__ row_x,
                               const float *__restrict__ col_y, float *__restrict__ am_grad,
                               const int64_t *__restrict__ window, int B, int S, int T, int C,
                               int ldd, int term, int rnnt_type, int rows_cap, int part_shift) {
  simple_bwd_am_panel_body<kCap>((int)blockIdx.x, lm, am, symbols, boundary, lm_max, am_max, dmat,
                                 gpx, row_x, col_y, am_grad, window, B, S, T, C, ldd, term,
                                 rnnt_type, rows_cap, part_shift);
}
// Both gradient products in one launch: the first lm_blocks workgroups take tiles of
// lm.grad, the rest tiles of am.grad.  The two only read what the prep kernel left, so
// their workgroups share the chip.  The order matters: the am tiles are short and mostly
// wait for memory, and fill the end of the launch better than the lm tiles do (c2 shape:
// 30.4 us with the lm tiles first, 33.2 with the am tiles first, 36.9 with the two kinds
// dealt out alternately).  lm_blocks is a multiple of 8, so a workgroup's XCD is the same
// in both numberings.
static_assert(kLmThreads == 256, "the two kinds of workgroup must have the same size");
template <int kS, int kK>
__global__ void __launch_bounds__(256, 2)
    simple_bwd_am_lm_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                            const int64_t *__restrict__ symbols,
                            const int64_t *__restrict__ boundary,
                            const float *__restrict__ lm_max, const float *__restrict__ am_max,
                            const float *__restrict__ dmat, const float *__restrict__ gpx,
                            const float *__restrict__ row_x, const float *__restrict__ row_y,
                            const float *__restrict__ col_y, float *__restrict__ lm_grad,
                            float *__restrict__ am_grad, const int64_t *__restrict__ window, int B,
                            int S, int T, int C, int ldd, int term, int rnnt_type, int rows_cap,
                            int lm_blocks, int lm_part_shift, int am_part_shift) {
  if ((int)blockIdx.x < lm_blocks)
    simple_bwd_lm_slab_body<kS, kK>((int)blockIdx.x, lm, am, symbols, lm_max, am_max, dmat, row_x,
                                    row_y, lm_grad, window, B, S, T, C, ldd, term, lm_part_shift);
  else
    simple_bwd_am_panel_body<kAmCap>((int)blockIdx.x - lm_blocks, lm, am, symbols, boundary, lm_max,
                                     am_max, dmat, gpx, row_x, col_y, am_grad, window, B, S, T, C,
                                     ldd, term, rnnt_type, rows_cap, am_part_shift);
}
// lm.grad and am.grad together (float only)
void launch_bwd_both(const float *lm, const float *am, const int64_t *symbols,
                     const int64_t *boundary, const float *lm_max, const float *am_max,
                     const float *dmat, const float *gpx, const float *row_x, const float *row_y,
                     const float *col_y, float *lm_grad, float *am_grad, const int64_t *window,
                     int B, int S, int T, int C, int ldd, int term, int rnnt_type,
                     hipStream_t stream) {
  const int S1 = S + 1;
  const bool rows96 = (S1 + 95) / 96 * 96 < (S1 + 127) / 128 * 128;
  const int rows = rows96 ? 96 : 128;
  const int lm_c = (C + kLmC - 1) / kLmC, am_c = (C + kAmC - 1) / kAmC;
  const int lm_shift = part_shift_for(B, lm_c), am_shift = part_shift_for(B, am_c);
  const int rows_cap = am_rows_per_pass(S);
  // (frames in slabs of 16 here also for the 96-row form: its LDS is then 50 KB, not 67,
  // and three workgroups fit on a CU whichever product they work on: 33.4 us against 36.2)
  const size_t lm_lds = rows96 ? LmShape<96, 16>::kLdsBytes : LmShape<128, 16>::kLdsBytes;
  const size_t lds = std::max(lm_lds, am_panel_lds_bytes(rows_cap));
  const unsigned am_blocks = placed_grid(am_c, (T + kAmT - 1) / kAmT, B, am_shift);
  const unsigned lm_blocks = placed_grid(lm_c, (S1 + rows - 1) / rows, B, lm_shift);
  auto kernel = rows96 ? simple_bwd_am_lm_kernel<96, 16> : simple_bwd_am_lm_kernel<128, 16>;
  (void)allow_lds(reinterpret_cast<const void *>(kernel), lds);
  hipLaunchKernelGGL(kernel, dim3(am_blocks + lm_blocks), dim3(256), lds, stream, lm, am, symbols,
                     boundary, lm_max, am_max, dmat, gpx, row_x, row_y, col_y, lm_grad, am_grad,
                     window, B, S, T, C, ldd, term, rnnt_type, rows_cap, (int)lm_blocks, lm_shift,
                     am_shift);
}
void launch_bwd_both(const double *, const double *, const int64_t *, const int64_t *,
                     const double *, const double *, const double *, const double *,
                     const double *, const double *, const double *, double *, double *,
                     const int64_t *, int, int, int, int, int, int, int, hipStream_t) {}
void launch_bwd_lm(const float *lm, const float *am, const int64_t *symbols, const float *lm_max,
                   const float *am_max, const float *dmat, const float *row_x, const float *row_y,
                   float *lm_grad, const int64_t *window, int B, int S, int T, int C, int ldd,
                   int term, hipStream_t stream) {
  // the row count per workgroup that leaves fewer padding rows; 128 on a tie
  const int S1 = S + 1;
  const bool rows96 = (S1 + 95) / 96 * 96 < (S1 + 127) / 128 * 128;
  const int rows = rows96 ? 96 : 128;
  const int c_tiles = (C + kLmC - 1) / kLmC, shift = part_shift_for(B, c_tiles);
  auto kernel = rows96 ? simple_bwd_lm_slab_kernel<96, 32> : simple_bwd_lm_slab_kernel<128, 16>;
  const size_t lds = rows96 ? LmShape<96, 32>::kLdsBytes : LmShape<128, 16>::kLdsBytes;
  (void)allow_lds(reinterpret_cast<const void *>(kernel), lds);
  hipLaunchKernelGGL(kernel, dim3(placed_grid(c_tiles, (S1 + rows - 1) / rows, B, shift)),
                     dim3(kLmThreads), lds, stream, lm, am, symbols, lm_max, am_max, dmat, row_x,
                     row_y, lm_grad, window, B, S, T, C, ldd, term, shift);
}
void launch_bwd_lm(const double *lm, const double *am, const int64_t *symbols,
                   const double *lm_max, const double *am_max, const double *dmat,
                   const double *row_x, const double *row_y, double *lm_grad, const int64_t *, int B,
                   int S, int T, int C, int ldd, int term, hipStream_t stream) {
  const dim3 grid((C + kTileN - 1) / kTileN, (S + 1 + kTileM - 1) / kTileM, B);
  hipLaunchKernelGGL(simple_bwd_lm_kernel<double>, grid, dim3(kGemmThreads), 0, stream, lm, am,
                     symbols, lm_max, am_max, dmat, row_x, row_y, lm_grad, S, T, C, ldd, term);
}
void launch_bwd_am(const float *lm, const float *am, const int64_t *symbols,
                   const int64_t *boundary, const float *lm_max, const float *am_max,
                   const float *dmat, const float *gpx, const float *row_x, const float *col_y,
                   float *am_grad, const int64_t *window, int B, int S, int T, int C, int ldd,
                   int term, int rnnt_type, hipStream_t stream) {
  const int c_tiles = (C + kAmC - 1) / kAmC, shift = part_shift_for(B, c_tiles);
  // rows of k held in LDS per pass: all of them when they fit
  // Rows of k held in LDS per pass: at most 64, in passes of equal size.  The workgroup's
  // phases (panels in, exp, products, results out) do not overlap inside it, so the compute
  // unit needs several of them; 64 rows of panels leave room for four (128 rows: two), and the
  // next pass's panels are requested before the current one is multiplied (B = 16, S + 1 = 121,
  // T = 400, C = 5000: 154 us with one pass of 122 rows, 138 with two of 64 as three workgroups
  // per compute unit).
  const int rows_cap = am_rows_per_pass(S);
  const size_t lds = am_panel_lds_bytes(rows_cap);
  // (the 16-byte accesses need no alignment)
  auto kernel = simple_bwd_am_panel_kernel<kAmCap, 4>;
  (void)allow_lds(reinterpret_cast<const void *>(kernel), lds);
  hipLaunchKernelGGL(kernel, dim3(placed_grid(c_tiles, (T + kAmT - 1) / kAmT, B, shift)), dim3(256),
                     lds, stream, lm, am, symbols, boundary, lm_max, am_max, dmat, gpx, row_x, col_y,
                     am_grad, window, B, S, T, C, ldd, term, rnnt_type, rows_cap, shift);
}
void launch_bwd_am(const double *lm, const double *am, const int64_t *symbols,
                   const int64_t *boundary, const double *lm_max, const double *am_max,
                   const double *dmat, const double *gpx, const double *, const double *col_y,
                   double *am_grad, const int64_t *, int B, int S, int T, int C, int ldd, int term,
                   int rnnt_type, hipStream_t stream) {
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
             int rnnt_type, int window_only, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "simple_logprobs_fwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2)
    return fail(FRNNT_EINVAL, "simple_logprobs_fwd: rnnt_type must be 0, 1 or 2");
  if (term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "simple_logprobs_fwd: termination symbol outside [0, C)");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !px || !py || !lm_max || !am_max)
    return fail(FRNNT_EINVAL, "simple_logprobs_fwd: null pointer");
  // (the float32 kernel addresses an utterance's lm / am rows by 32-bit byte offsets)
  if (std::is_same<R, float>::value &&
      ((long)(S + 1) * C * 4 >= (1L << 31) || (long)T * C * 4 >= (1L << 31)))
    return fail(FRNNT_ELIMIT, "simple_logprobs_fwd: one utterance's lm or am exceeds 2 GiB");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long n_lm = (long)B * (S + 1), n_am = (long)B * T;
  const long rows = n_lm + n_am;
  // (the fp32 GEMM kernel finds the row maxima itself)
  if (!std::is_same<R, float>::value)
    hipLaunchKernelGGL(row_max_kernel<R>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream,
                       lm, am, lm_max, am_max, n_lm, n_am, C);
  {
    // (the grid always has at least one column of tiles, so that the -inf column of
    // an empty-frame regular lattice is still written)
    launch_fwd_gemm(lm, am, symbols, boundary, lm_max, am_max, px, py, norm_raw,
                    window_only ? boundary : nullptr, B, S, T, C, term, rnnt_type, stream);
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
             const R *lm_max, const R *am_max, const R *norm_raw, const R *score_grad,
             int score_grad_stride, double score_grad_scale, R *px_grad, R *py_grad, R *dmat,
             R *row_x, R *row_y, R *col_y, R *lm_grad, R *am_grad, int B, int S, int T, int C,
             int term, int rnnt_type, int window_only, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || C < 1) return fail(FRNNT_EINVAL, "simple_logprobs_bwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "simple_logprobs_bwd: bad rnnt_type or termination symbol");
  if (B == 0) return FRNNT_OK;
  if (!lm || !am || (!symbols && S > 0) || !lm_max || !am_max || !norm_raw || !px_grad ||
      !py_grad || !dmat || !row_x || !row_y || !col_y)
    return fail(FRNNT_EINVAL, "simple_logprobs_bwd: null pointer");
  // (the float32 kernels address an utterance's lm / am / D rows by 32-bit byte offsets)
  if (std::is_same<R, float>::value &&
      ((long)(S + 1) * C * 4 >= (1L << 31) || (long)T * C * 4 >= (1L << 31) ||
       (long)(S + 1) * (T + 3) * 4 >= (1L << 31)))
    return fail(FRNNT_ELIMIT, "simple_logprobs_bwd: one utterance's lm, am or lattice exceeds 2 GiB");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (score_grad) {
    if (score_grad_stride != 0 && score_grad_stride != 1)
      return fail(FRNNT_EINVAL, "simple_logprobs_bwd: score_grad_stride must be 0 or 1");
    const int T1 = rnnt_type == kRegular ? T + 1 : T;
    const int per_x = S * T1, per_y = (S + 1) * T;
    const int x_blocks = (per_x + 1023) / 1024, y_blocks = (per_y + 1023) / 1024;
    if (x_blocks + y_blocks > 0)
      hipLaunchKernelGGL(scale_by_batch_kernel<R>, dim3(x_blocks + y_blocks, B), dim3(256), 0,
                         stream, px_grad, py_grad, score_grad, score_grad_stride,
                         (R)score_grad_scale, per_x, per_y, x_blocks);
  }
  const int ldd = (T + 3) & ~3;  // leading dimension of dmat: 16-byte rows
  // (the double kernels ignore the window: they take the whole lattice as it is)
  const int64_t *window = (window_only && std::is_same<R, float>::value) ? boundary : nullptr;
  const long prep_blocks = ((long)B * (S + 1) + 3) / 4 + (long)B * ((T + kWave - 1) / kWave) + 1;
  hipLaunchKernelGGL(simple_bwd_prep_kernel<R>, dim3((unsigned)prep_blocks), dim3(256), 0, stream,
                     px_grad, py_grad, norm_raw, boundary, window, dmat, row_x, row_y, col_y, B, S, T,
                     ldd, rnnt_type);
  // (one launch for both products while they are short: at B (S+1) T C = 3.2e8 it saves
  // about 1 us of 37; at 3.9e9 the common LDS and register budget costs 8 %)
  if (std::is_same<R, float>::value && lm_grad && am_grad && T > 0 &&
      (double)B * (S + 1) * T * C < 1e9) {
    launch_bwd_both(lm, am, symbols, boundary, lm_max, am_max, dmat, px_grad, row_x, row_y, col_y,
                    lm_grad, am_grad, window, B, S, T, C, ldd, term, rnnt_type, stream);
    return check_launch("simple_logprobs_bwd");
  }
  if (lm_grad)
    launch_bwd_lm(lm, am, symbols, lm_max, am_max, dmat, row_x, row_y, lm_grad, window, B, S, T, C,
                  ldd, term, stream);
  if (am_grad && T > 0)
    launch_bwd_am(lm, am, symbols, boundary, lm_max, am_max, dmat, px_grad, row_x, col_y, am_grad, window,
                  B, S, T, C, ldd, term, rnnt_type, stream);
  return check_launch("simple_logprobs_bwd");
}

// px_grad[b] and py_grad[b] times score_grad_scale * score_grad[b * stride], in place: the
// scaling step of the recursion's autograd backward (mutual_information.py:173-181).
template <typename R>
int scale_grads_impl(R *px_grad, R *py_grad, const R *score_grad, int score_grad_stride,
                     double score_grad_scale, int B, int S, int T, int modified, void *stream) {
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "mi_scale_grads: negative size");
  if (score_grad_stride != 0 && score_grad_stride != 1)
    return fail(FRNNT_EINVAL, "mi_scale_grads: score_grad_stride must be 0 or 1");
  if (B == 0) return FRNNT_OK;
  if (!px_grad || !py_grad || !score_grad)
    return fail(FRNNT_EINVAL, "mi_scale_grads: null pointer");
  const int T1 = modified ? T : T + 1;
  const int per_x = S * T1, per_y = (S + 1) * T;
  const int x_blocks = (per_x + 1023) / 1024, y_blocks = (per_y + 1023) / 1024;
  if (x_blocks + y_blocks > 0)
    hipLaunchKernelGGL(scale_by_batch_kernel<R>, dim3(x_blocks + y_blocks, B), dim3(256), 0,
                       static_cast<hipStream_t>(stream), px_grad, py_grad, score_grad,
                       score_grad_stride, (R)score_grad_scale, per_x, per_y, x_blocks);
  return check_launch("mi_scale_grads");
}

template <typename R>
int reduce_impl(const R *scores, R *loss, int B, int reduction, void *stream) {
  if (B < 0 || reduction < 0 || reduction > 2)
    return fail(FRNNT_EINVAL, "loss_reduce: bad size or reduction");
  if (!loss || (B > 0 && !scores)) return fail(FRNNT_EINVAL, "loss_reduce: null pointer");
  if (B == 0 && reduction == 0) return FRNNT_OK;
  hipLaunchKernelGGL(loss_reduce_kernel<R>, dim3(1), dim3(kWave), 0,
                     static_cast<hipStream_t>(stream), scores, loss, B, reduction);
  return check_launch("loss_reduce");
}

// ---- scratch that the library owns: for callers that cannot allocate --------------------
// One array per GPU, part of the code object, held until the process ends.  In host code
// the array's name is only a handle: its device address is looked up once per device
// (with that device current) and kept; kernels and everything else get that address.
constexpr size_t kOwnScratchFloats = (size_t)4 << 20;  // 16 MiB
static __device__ __align__(256) float own_scratch[kOwnScratchFloats];
constexpr int kMaxDevices = 64;

float *own_scratch_address() {
  static std::mutex guard;
  static float *address[kMaxDevices] = {nullptr};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(guard);
  if (!address[device]) {
    void *found = nullptr;
    if (hipGetSymbolAddress(&found, HIP_SYMBOL(own_scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    address[device] = static_cast<float *>(found);
  }
  return address[device];
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_simple_logprobs_bwd_noalloc_f32(const float *lm, const float *am, const int64_t *symbols,
                                          const int64_t *boundary, const float *lm_max,
                                          const float *am_max, const float *norm_raw,
                                          const float *score_grad, int score_grad_stride,
                                          double score_grad_scale, float *px_grad,
                                          float *py_grad, float *lm_grad, float *am_grad, int B,
                                          int S, int T, int C, int termination_symbol,
                                          int rnnt_type, int window_only, void *stream) {
  using frnnt::fail;
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "simple_logprobs_bwd_noalloc: bad size");
  // dmat | row_x | row_y | col_y, each starting 16-byte aligned
  const size_t ldd = ((size_t)T + 3) & ~(size_t)3;
  const size_t n_rows = ((size_t)B * (S + 1) + 3) & ~(size_t)3;
  const size_t n_cols = ((size_t)B * T + 3) & ~(size_t)3;
  const size_t n_dmat = (size_t)B * (S + 1) * ldd;
  const size_t need = n_dmat + 2 * n_rows + n_cols;
  if (need > frnnt::kOwnScratchFloats)
    return fail(FRNNT_ELIMIT,
                "simple_logprobs_bwd_noalloc: B=%d S=%d T=%d needs %zu bytes of scratch, the "
                "library's own buffer holds %zu; use frnnt_simple_logprobs_bwd_f32 with a "
                "caller-provided workspace",
                B, S, T, need * sizeof(float), frnnt::kOwnScratchFloats * sizeof(float));
  // the array is the current device's copy: the buffers must live on that device
  if (px_grad) {
    hipPointerAttribute_t where;
    int current = -1;
    if (hipPointerGetAttributes(&where, px_grad) != hipSuccess) {
      (void)hipGetLastError();
      return fail(FRNNT_EINVAL, "simple_logprobs_bwd_noalloc: px_grad is not a device pointer");
    }
    if (hipGetDevice(&current) != hipSuccess || where.device != current)
      return fail(FRNNT_EINVAL,
                  "simple_logprobs_bwd_noalloc: the buffers live on device %d but device %d is "
                  "current; make the buffers' device current before the call",
                  where.device, current);
  }
  float *base = frnnt::own_scratch_address();
  if (!base) return fail(FRNNT_ELAUNCH, "simple_logprobs_bwd_noalloc: hipGetSymbolAddress failed");
  float *dmat = base, *row_x = dmat + n_dmat, *row_y = row_x + n_rows, *col_y = row_y + n_rows;
  return frnnt::bwd_impl<float>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, score_grad,
                                score_grad_stride, score_grad_scale, px_grad, py_grad, dmat, row_x,
                                row_y, col_y, lm_grad, am_grad, B, S, T, C, termination_symbol,
                                rnnt_type, window_only, stream);
}

int frnnt_simple_logprobs_fwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                  const int64_t *boundary, float *px, float *py, float *lm_max,
                                  float *am_max, float *norm_raw, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream) {
  return frnnt::fwd_impl<float>(lm, am, symbols, boundary, px, py, lm_max, am_max, norm_raw, B, S,
                                T, C, termination_symbol, rnnt_type, window_only, stream);
}
int frnnt_simple_logprobs_fwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, double *px, double *py, double *lm_max,
                                  double *am_max, double *norm_raw, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream) {
  return frnnt::fwd_impl<double>(lm, am, symbols, boundary, px, py, lm_max, am_max, norm_raw, B, S,
                                 T, C, termination_symbol, rnnt_type, window_only, stream);
}
int frnnt_simple_logprobs_bwd_f32(const float *lm, const float *am, const int64_t *symbols,
                                  const int64_t *boundary, const float *lm_max,
                                  const float *am_max, const float *norm_raw,
                                  const float *score_grad, int score_grad_stride,
                                  double score_grad_scale, float *px_grad, float *py_grad,
                                  float *dmat, float *row_x, float *row_y, float *col_y,
                                  float *lm_grad, float *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream) {
  return frnnt::bwd_impl<float>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, score_grad,
                                score_grad_stride, score_grad_scale, px_grad, py_grad, dmat, row_x,
                                row_y, col_y, lm_grad, am_grad, B, S, T, C, termination_symbol,
                                rnnt_type, window_only, stream);
}
int frnnt_simple_logprobs_bwd_f64(const double *lm, const double *am, const int64_t *symbols,
                                  const int64_t *boundary, const double *lm_max,
                                  const double *am_max, const double *norm_raw,
                                  const double *score_grad, int score_grad_stride,
                                  double score_grad_scale, double *px_grad, double *py_grad,
                                  double *dmat, double *row_x, double *row_y, double *col_y,
                                  double *lm_grad, double *am_grad, int B, int S, int T, int C,
                                  int termination_symbol, int rnnt_type, int window_only,
                                  void *stream) {
  return frnnt::bwd_impl<double>(lm, am, symbols, boundary, lm_max, am_max, norm_raw, score_grad,
                                 score_grad_stride, score_grad_scale, px_grad, py_grad, dmat,
                                 row_x, row_y, col_y, lm_grad, am_grad, B, S, T, C,
                                 termination_symbol, rnnt_type, window_only, stream);
}

int frnnt_mi_scale_grads_f32(float *px_grad, float *py_grad, const float *score_grad,
                             int score_grad_stride, double score_grad_scale, int B, int S, int T,
                             int modified, void *stream) {
  return frnnt::scale_grads_impl<float>(px_grad, py_grad, score_grad, score_grad_stride,
                                        score_grad_scale, B, S, T, modified, stream);
}
int frnnt_mi_scale_grads_f64(double *px_grad, double *py_grad, const double *score_grad,
                             int score_grad_stride, double score_grad_scale, int B, int S, int T,
                             int modified, void *stream) {
  return frnnt::scale_grads_impl<double>(px_grad, py_grad, score_grad, score_grad_stride,
                                         score_grad_scale, B, S, T, modified, stream);
}
int frnnt_loss_reduce_f32(const float *scores, float *loss, int B, int reduction, void *stream) {
  return frnnt::reduce_impl<float>(scores, loss, B, reduction, stream);
}
int frnnt_loss_reduce_f64(const double *scores, double *loss, int B, int reduction, void *stream) {
  return frnnt::reduce_impl<double>(scores, loss, B, reduction, stream);
}

}  // extern "C"
