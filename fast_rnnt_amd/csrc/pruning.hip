// Pruning bounds and the pruning gather of the pruned RNN-T loss.
//
// prune_ranges (fast_rnnt/python/fast_rnnt/rnnt_loss.py:638-777, helpers
// :550-632): for every frame pick the window start s that maximises
//   sum_{j<R} py_grad[b,s+j,t] - px_grad[b,s-1,t]        (0 for s = 0)
// with the window sum formed in the input precision in the order of the reference's
// torch.sum on the CPU (left to right up to 16 values, in stretches of 16 beyond: see
// window_sum below) and ties resolved to the first maximum, replace the starts of frames at or beyond
// T_b - 1 by max(S_b - R + 1, 0), then make the starts non-decreasing, starting
// at 0, with steps smaller than r (r = R for the regular lattice, 2 otherwise)
// by two suffix-minimum passes.  Two kernels: one lane per frame for the window
// starts (left in ranges[b][t][0]), then one wave per utterance for the two passes,
// with the starts in LDS and the suffix minima as a chunked wave scan.
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

// The sum of the s_range values of one window, in the order in which the reference's
// torch.sum adds them on the CPU (rnnt_loss.py:726-734 reduces a strided view over the
// window axis; ATen's outer-sum loop, SumKernel.cpp multi_row_sum): left to right in
// stretches of 16, each stretch's sum added to a second accumulator, that one to a third
// after 16 stretches and to a fourth after 256, the remainder left to right, and at the
// end the four added in order.  Up to 16 values that is plain left to right.  The order
// matters: when the window is wider than the band of the lattice that holds the
// alignment's mass, neighbouring window starts tie up to rounding, and the first maximum
// among them is whatever the rounding makes it.  `at(j)` is the window's j-th value.
template <typename R, typename F>
__device__ __forceinline__ R window_sum(int width, F at) {
  if (width <= 16) {
    R sum = at(0);
    for (int j = 1; j < width; ++j) sum = sum + at(j);
    return sum;
  }
  R a1 = 0, a2 = 0, a3 = 0;
  int i = 0;
  while (i + 16 <= width) {
    R c = at(i);
#pragma unroll
    for (int j = 1; j < 16; ++j) c = c + at(i + j);
    i += 16;
    a1 = a1 + c;
    if ((i & 0xF0) == 0) {
      a2 = a2 + a1;
      a1 = 0;
      if ((i & 0xF00) == 0) {
        a3 = a3 + a2;
        a2 = 0;
      }
    }
  }
  R rest = 0;
  for (; i < width; ++i) rest = rest + at(i);
  return ((rest + a1) + a2) + a3;
}

// Step 1, one lane per frame: the best window start of frame (b, t), left in
// ranges[b][t][0].
template <typename R>
__global__ void __launch_bounds__(kWave)
    prune_starts_kernel(const R *__restrict__ px_grad, const R *__restrict__ py_grad,
                        const int64_t *__restrict__ boundary, int64_t *__restrict__ ranges, int S,
                        int T, int T1, int Rr) {
  const int b = blockIdx.y, t = blockIdx.x * kWave + threadIdx.x;
  if (t >= T) return;
  const R *gx = px_grad + (long)b * S * T1 + t;
  const R *gy = py_grad + (long)b * (S + 1) * T + t;
  const int n = S + 2 - Rr;  // candidate window starts
  const int64_t Sb = boundary[4 * b + 2], Tb = boundary[4 * b + 3];
  int64_t tail = Sb - Rr + 1;
  if (tail < 0) tail = 0;
  int best = 0;
  R best_score = 0;
  // first maximum wins; a NaN score counts as the maximum, like torch.argmax
  auto consider = [&](int s, R score) {
    if (s == 0 || score > best_score || (score != score && best_score == best_score)) {
      best = s;
      best_score = score;
    }
  };
  auto score_of = [&](int s) {
    const R sum = window_sum<R>(Rr, [&](int j) { return gy[(long)(s + j) * T]; });
    const R below = s >= 1 ? gx[(long)(s - 1) * T1] : (R)0;
    return sum - below;
  };
  int s = 0;
  for (; s + 4 <= n; s += 4) {
    // four independent windows in flight
    const R a0 = score_of(s), a1 = score_of(s + 1), a2 = score_of(s + 2), a3 = score_of(s + 3);
    consider(s, a0);
    consider(s + 1, a1);
    consider(s + 2, a2);
    consider(s + 3, a3);
  }
  for (; s < n; ++s) consider(s, score_of(s));
  ranges[((long)b * T + t) * Rr] = ((int64_t)t < Tb - 1) ? (int64_t)best : tail;
}

// The same with the 64 frames' columns of py_grad and px_grad staged in LDS first: every
// load of the tile is in flight at once (the kernel above walks the rows with a few loads
// in flight), and the four waves share the candidate starts, each scanning a contiguous
// quarter; wave 0 then takes the quarters' winners in order under the same rule, which
// is the sequential scan's result.
template <typename R>
__global__ void __launch_bounds__(256)
    prune_starts_tile_kernel(const R *__restrict__ px_grad, const R *__restrict__ py_grad,
                             const int64_t *__restrict__ boundary, int64_t *__restrict__ ranges,
                             int S, int T, int T1, int Rr) {
  extern __shared__ unsigned char tile_raw[];
  __shared__ int seg_best[4][kWave];
  __shared__ R seg_score[4][kWave];
  R *ty = reinterpret_cast<R *>(tile_raw);  // [S + 1][64]
  R *tx = ty + (S + 1) * kWave;             // [S][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = blockIdx.y, t = blockIdx.x * kWave + lane;
  const bool ok = t < T;
  // (a frame past the end reads the last frame's column: no branch around the loads, so
  // that eight rows are requested before the first is stored)
  const int t_read = ok ? t : T - 1;
  const R *gx = px_grad + (long)b * S * T1 + t_read;
  const R *gy = py_grad + (long)b * (S + 1) * T + t_read;
  for (int s0 = wave; s0 <= S; s0 += 32) {
    R v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = gy[(long)min(s0 + 4 * u, S) * T];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + 4 * u <= S) ty[(s0 + 4 * u) * kWave + lane] = ok ? v[u] : (R)0;
  }
  for (int s0 = wave; s0 < S; s0 += 32) {
    R v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = gx[(long)min(s0 + 4 * u, S - 1) * T1];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + 4 * u < S) tx[(s0 + 4 * u) * kWave + lane] = ok ? v[u] : (R)0;
  }
  __syncthreads();
  const int n = S + 2 - Rr;  // candidate window starts
  const int per = (n + 3) / 4, lo = wave * per, hi = min(n, lo + per);
  int best = -1;
  R best_score = 0;
  // first maximum wins; a NaN score counts as the maximum, like torch.argmax
  auto consider = [&](int s, R score) {
    if (best < 0 || score > best_score || (score != score && best_score == best_score)) {
      best = s;
      best_score = score;
    }
  };
  for (int s = lo; s < hi; ++s) {
    const R sum = window_sum<R>(Rr, [&](int j) { return ty[(s + j) * kWave + lane]; });
    const R below = s >= 1 ? tx[(s - 1) * kWave + lane] : (R)0;
    consider(s, sum - below);
  }
  seg_best[wave][lane] = best;
  seg_score[wave][lane] = best_score;
  __syncthreads();
  if (wave != 0 || !ok) return;
  for (int w = 1; w < 4; ++w)
    if (seg_best[w][lane] >= 0) consider(seg_best[w][lane], seg_score[w][lane]);
  const int64_t Sb = boundary[4 * b + 2], Tb = boundary[4 * b + 3];
  int64_t tail = Sb - Rr + 1;
  if (tail < 0) tail = 0;
  ranges[((long)b * T + t) * Rr] = ((int64_t)t < Tb - 1) ? (int64_t)best : tail;
}

// Step 2, one wave per utterance: the starts are made non-decreasing with bounded
// steps by two suffix-minimum passes and expanded to the R entries of each frame.
__global__ void __launch_bounds__(kWave)
    prune_monotone_kernel(int64_t *__restrict__ ranges, int T, int r, int Rr) {
  extern __shared__ int start[];  // [T]
  const int b = blockIdx.x, lane = threadIdx.x;
  int64_t *rb = ranges + (long)b * T * Rr;
  for (int t = lane; t < T; t += kWave) start[t] = (int)rb[(long)t * Rr];
  __syncthreads();
  suffix_min_inplace(start, T, lane);
  for (int t = lane; t < T; t += kWave) start[t] = (r - 1) * t - start[t];
  __syncthreads();
  suffix_min_inplace(start, T, lane);
  for (int t = lane; t < T; t += kWave) {
    const int y = max(start[t], 0);
    const int64_t s0 = (int64_t)(r - 1) * t - y;
    int64_t *out = rb + (long)t * Rr;
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
    typedef typename AccOf<R>::type A;
    for (int c = lane; c < C; c += kWave) dst[c] = (R)std::numeric_limits<A>::quiet_NaN();
    return;
  }
  const R *src = lm + (b * S1 + s) * C;
  for (int c = lane; c < C; c += kWave) dst[c] = src[c];
}

// The same for rows of 4-byte elements whose length is a multiple of 4 (at most
// 256 * kVecs): the whole row is requested at once, 16 bytes per lane and load, and
// leaves as 16-byte stores.
typedef int words4 __attribute__((ext_vector_type(4), aligned(4)));
template <int kVecs>
__global__ void __launch_bounds__(256)
    prune_gather_vec_kernel(const int *__restrict__ lm, const int64_t *__restrict__ ranges,
                            int *__restrict__ out, long rows, int TR, int S1, int C,
                            int nan_bits) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register
  const long row = (long)blockIdx.x * 4 + wave;
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const long b = row / TR;
  const int64_t s = ranges[row];
  const bool valid = s >= 0 && s < S1;
  const int *src = lm + (b * S1 + (valid ? s : 0)) * C;
  words4 v[kVecs];
#pragma unroll
  for (int i = 0; i < kVecs; ++i) {
    const int c = 4 * (lane + kWave * i);
    v[i] = words4{nan_bits, nan_bits, nan_bits, nan_bits};
    if (valid && c < C) v[i] = *reinterpret_cast<const words4 *>(src + c);
  }
  int *dst = out + row * C;
#pragma unroll
  for (int i = 0; i < kVecs; ++i) {
    const int c = 4 * (lane + kWave * i);
    if (c < C) *reinterpret_cast<words4 *>(dst + c) = v[i];
  }
}

// adjoint: one block per lm row (b, s).  The block first lists, in order, the entries
// of ranges[b] that point at s (an ordered compaction through LDS; only a few dozen of
// the T * R entries match), then sums those rows of the incoming gradient -- in that
// order (shared out over the block's waves in a fixed way), so the result is
// deterministic -- with coalesced loads.  For the listing a
// thread takes kScanPerThread consecutive entries (all requested at once), and one
// prefix sum over the threads' counts places everybody's matches.
constexpr int kHitCapacity = 4096;   // matches listed per round
constexpr int kScanPerThread = 8;
constexpr int kScanChunk = 256 * kScanPerThread;
// a round must be able to take a whole chunk of matches, or it would make no progress
static_assert(kHitCapacity >= kScanChunk, "a chunk of matches must fit in the list");

// With `act_out` (the tanh outputs the gradient belongs to, same shape as grad) every
// gradient entry is first multiplied by the activation's derivative 1 - out^2: the adjoint
// of the fused joiner input below, which never materialises the gathered rows.
template <typename R>
__global__ void __launch_bounds__(256)
    prune_scatter_kernel(const R *__restrict__ grad, const R *__restrict__ act_out,
                         const int64_t *__restrict__ ranges, R *__restrict__ lm_grad, int TR,
                         int S1, int C) {
  __shared__ int hits[kHitCapacity];
  __shared__ int wave_count[4];
  __shared__ __align__(16) float meet[4 * 512];  // the four waves' sums of 512 columns
  const int b = blockIdx.x / S1, s = blockIdx.x % S1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t *rb = ranges + (long)b * TR;
  const R *gb = grad + (long)b * TR * C;
  const R *ob = act_out ? act_out + (long)b * TR * C : nullptr;
  R *dst = lm_grad + ((long)b * S1 + s) * C;
  bool first_round = true;
  int k_next = 0;
  // rounds only repeat when more than kHitCapacity entries point at s
  do {
    int listed = 0;  // the same in every thread
    int k0 = k_next;
    for (; k0 < TR; k0 += kScanChunk) {
      const int mine = k0 + tid * kScanPerThread;
      int64_t v[kScanPerThread];
#pragma unroll
      for (int u = 0; u < kScanPerThread; ++u) v[u] = mine + u < TR ? rb[mine + u] : (int64_t)-1;
      unsigned found = 0;
#pragma unroll
      for (int u = 0; u < kScanPerThread; ++u) found |= (v[u] == s ? 1u : 0u) << u;
      const int count = __popc(found);
      // exclusive prefix of the counts: over the wave, then over the four waves
      int upto = count;
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) {
        const int o = __shfl_up(upto, off, kWave);
        if (lane >= off) upto += o;
      }
      __syncthreads();  // the previous chunk's wave_count has been read
      if (lane == kWave - 1) wave_count[wave] = upto;
      __syncthreads();
      int before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (w < wave) before += wave_count[w];
        total += wave_count[w];
      }
      if (listed + total > kHitCapacity) break;  // (uniform) this chunk waits for the next round
      int at = listed + before + upto - count;
#pragma unroll
      for (int u = 0; u < kScanPerThread; ++u)
        if (found & (1u << u)) hits[at++] = mine + u;
      listed += total;
    }
    k_next = k0;
    __syncthreads();
    const int n = listed;
    if (sizeof(R) == 4 && C % 4 == 0 && (long)TR * C * 4 < (1L << 31)) {
      // The four waves share the listed rows (wave w takes rows w, w + 4, ...), a lane
      // reads 16 bytes of a row at a time, two stretches of 256 columns and four rows
      // per request round; the waves' sums meet in LDS in a fixed order.
      // Loads go through a buffer resource over the utterance's gradient rows: a lane
      // with nothing to read passes an offset outside it and gets 0 -- no branch around
      // the load, so that all loads of a round are in flight together.
      typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
      typedef int intx4 __attribute__((ext_vector_type(4)));
      const __amdgpu_buffer_rsrc_t g_rs = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<float *>(reinterpret_cast<const float *>(gb)), 0, TR * C * 4, 0x00020000);
      // (without activation outputs the second resource is empty: its loads return 0)
      const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<float *>(reinterpret_cast<const float *>(ob ? ob : gb)), 0,
          ob ? TR * C * 4 : 0, 0x00020000);
      constexpr int kNowhere = (int)0x80000000;
      auto row_piece = [&](int byte_offset) {
        const intx4 w = __builtin_amdgcn_raw_buffer_load_b128(g_rs, byte_offset, 0, 0);
        const intx4 o = __builtin_amdgcn_raw_buffer_load_b128(o_rs, byte_offset, 0, 0);
        f4 g = f4{__int_as_float(w[0]), __int_as_float(w[1]), __int_as_float(w[2]),
                  __int_as_float(w[3])};
        const f4 y = f4{__int_as_float(o[0]), __int_as_float(o[1]), __int_as_float(o[2]),
                        __int_as_float(o[3])};
        return g * (1.f - y * y);  // y = 0 without an activation
      };
      float *df = reinterpret_cast<float *>(dst);
      f4 *meet4 = reinterpret_cast<f4 *>(meet);
      for (int c0 = 0; c0 < C; c0 += 512) {
        const int ca = c0 + 4 * lane, cb = ca + 256;
        f4 a = {0, 0, 0, 0}, b2 = {0, 0, 0, 0};
        for (int i = wave; i < n; i += 16) {
          f4 va[4], vb[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int at = i + 4 * u;
            const int row = hits[at < n ? at : i] * C * 4;  // byte offset of the row
            va[u] = row_piece((at < n && ca < C) ? row + ca * 4 : kNowhere);
            vb[u] = row_piece((at < n && cb < C) ? row + cb * 4 : kNowhere);
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) a += va[u], b2 += vb[u];
        }
        meet4[wave * 128 + lane] = a;
        meet4[wave * 128 + 64 + lane] = b2;
        __syncthreads();
        if (tid < 128) {
          const int c = c0 + 4 * tid;
          if (c < C) {
            f4 sum = (meet4[tid] + meet4[128 + tid]) + (meet4[256 + tid] + meet4[384 + tid]);
            if (!first_round) sum += *reinterpret_cast<const f4 *>(df + c);
            *reinterpret_cast<f4 *>(df + c) = sum;
          }
        }
        __syncthreads();
      }
    } else {
      for (int c0 = 0; c0 < C; c0 += 256) {
        const int c = c0 + tid;
        if (c >= C) continue;
        // (2-byte elements are summed in float32; a sum that takes several rounds --
        // more than kHitCapacity rows -- is rounded to the element type between rounds)
        typedef typename AccOf<R>::type A;
        A acc = first_round ? (A)0 : (A)dst[c];
        auto entry = [&](int i) -> A {
          const long at = (long)hits[i] * C + c;
          const A g = (A)gb[at];
          if (!ob) return g;
          const A y = (A)ob[at];
          return g * ((A)1 - y * y);
        };
        int i = 0;
        for (; i + 8 <= n; i += 8) {
          A g[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) g[u] = entry(i + u);
#pragma unroll
          for (int u = 0; u < 8; ++u) acc += g[u];
        }
        if (i + 4 <= n) {
          A g[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) g[u] = entry(i + u);
#pragma unroll
          for (int u = 0; u < 4; ++u) acc += g[u];
          i += 4;
        }
        for (; i < n; ++i) acc += entry(i);
        dst[c] = (R)acc;
      }
    }
    first_round = false;
    __syncthreads();
  } while (k_next < TR);
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
  if (!allow_lds(reinterpret_cast<const void *>(prune_monotone_kernel), lds))
    return check_launch("prune_ranges: hipFuncSetAttribute");
  const int T1 = modified ? T : T + 1;
  const size_t tile_lds = (size_t)(2 * S + 1) * kWave * sizeof(R);
  if (tile_lds <= 144 * 1024 &&
      allow_lds(reinterpret_cast<const void *>(prune_starts_tile_kernel<R>), tile_lds))
    hipLaunchKernelGGL(prune_starts_tile_kernel<R>, dim3((T + kWave - 1) / kWave, B), dim3(256),
                       tile_lds, static_cast<hipStream_t>(stream), px_grad, py_grad, boundary,
                       ranges, S, T, T1, s_range);
  else
    hipLaunchKernelGGL(prune_starts_kernel<R>, dim3((T + kWave - 1) / kWave, B), dim3(kWave), 0,
                       static_cast<hipStream_t>(stream), px_grad, py_grad, boundary, ranges, S, T,
                       T1, s_range);
  hipLaunchKernelGGL(prune_monotone_kernel, dim3(B), dim3(kWave), lds,
                     static_cast<hipStream_t>(stream), ranges, T, modified ? 2 : s_range, s_range);
  return check_launch("prune_ranges");
}

// nan_words: a quiet NaN of the element type as a 4-byte word (twice, for 2-byte elements)
template <typename R>
int gather_impl(const R *lm, const int64_t *ranges, R *out, int B, int S, int T, int Rr, int C,
                int nan_words, void *stream) {
  if (B < 0 || S < 0 || T < 0 || Rr < 0 || C < 0)
    return fail(FRNNT_EINVAL, "prune_gather: negative size");
  const long rows = (long)B * T * Rr;
  if (rows == 0 || C == 0) return FRNNT_OK;
  if (!lm || !ranges || !out) return fail(FRNNT_EINVAL, "prune_gather: null pointer");
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  // rows as 4-byte words: the elements themselves, or 2-byte elements in pairs
  const int W = sizeof(R) == 4 ? C : (sizeof(R) == 2 && C % 2 == 0 ? C / 2 : 0);
  if (W > 0 && W % 4 == 0 && W <= 256 * 16 &&
      ((reinterpret_cast<uintptr_t>(lm) | reinterpret_cast<uintptr_t>(out)) & 3) == 0) {
    const int *src = reinterpret_cast<const int *>(lm);
    int *dst = reinterpret_cast<int *>(out);
#define FRNNT_GATHER(V)                                                                          \
  hipLaunchKernelGGL(prune_gather_vec_kernel<V>, grid, block, 0, static_cast<hipStream_t>(stream), \
                     src, ranges, dst, rows, T * Rr, S + 1, W, nan_words)
    if (W <= 256)
      FRNNT_GATHER(1);
    else if (W <= 512)
      FRNNT_GATHER(2);
    else if (W <= 1024)
      FRNNT_GATHER(4);
    else if (W <= 2048)
      FRNNT_GATHER(8);
    else
      FRNNT_GATHER(16);
#undef FRNNT_GATHER
  } else {
    hipLaunchKernelGGL(prune_gather_kernel<R>, grid, block, 0, static_cast<hipStream_t>(stream), lm,
                       ranges, out, rows, T * Rr, S + 1, C);
  }
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
                     static_cast<hipStream_t>(stream), grad, (const R *)nullptr, ranges, lm_grad,
                     T * Rr, S + 1, C);
  return check_launch("prune_gather_bwd");
}

// ---- the joiner's input without the gathered copy ------------------------------------------
// out[b,t,j,:] = act(am[b,t,:] + lm[b, ranges[b,t,j], :]) in one pass: what a joiner of the
// usual form does first with the two tensors do_rnnt_pruning returns (README "pruned
// rnnt loss" recipe: logits = joiner(am_pruned, lm_pruned)), without lm_pruned [B,T,R,C]
// ever existing.  One wave per output row; 16-byte accesses when the rows allow.
enum { kActNone = 0, kActTanh = 1 };
__device__ __forceinline__ float act_tanh(float x) { return tanhf(x); }
__device__ __forceinline__ double act_tanh(double x) { return tanh(x); }

template <typename R>
__global__ void __launch_bounds__(256)
    joiner_input_kernel(const R *__restrict__ am, const R *__restrict__ lm,
                        const int64_t *__restrict__ ranges, R *__restrict__ out, long rows, int Rr,
                        int TR, int S1, int C, int activation) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register
  const long row = (long)blockIdx.x * 4 + wave;
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const long b = row / TR;
  const int64_t s = ranges[row];
  const bool valid = s >= 0 && s < S1;
  const R *a = am + (row / Rr) * C;
  const R *l = lm + (b * S1 + (valid ? s : 0)) * C;
  R *dst = out + row * C;
  const R nan = std::numeric_limits<R>::quiet_NaN();
  constexpr int kPer = 16 / (int)sizeof(R);
  typedef R Piece __attribute__((ext_vector_type(kPer), aligned(sizeof(R))));
  if (C % kPer == 0) {
    // two pieces per lane in flight from each source
    for (int c0 = kPer * lane; c0 < C; c0 += 2 * kPer * kWave) {
      const int c1 = c0 + kPer * kWave;
      const bool second = c1 < C;
      const Piece a0 = *reinterpret_cast<const Piece *>(a + c0);
      const Piece l0 = *reinterpret_cast<const Piece *>(l + c0);
      Piece a1 = a0, l1 = l0;
      if (second) {
        a1 = *reinterpret_cast<const Piece *>(a + c1);
        l1 = *reinterpret_cast<const Piece *>(l + c1);
      }
      Piece y0, y1;
#pragma unroll
      for (int e = 0; e < kPer; ++e) {
        const R v0 = a0[e] + l0[e], v1 = a1[e] + l1[e];
        y0[e] = !valid ? nan : (activation == kActTanh ? act_tanh(v0) : v0);
        y1[e] = !valid ? nan : (activation == kActTanh ? act_tanh(v1) : v1);
      }
      *reinterpret_cast<Piece *>(dst + c0) = y0;
      if (second) *reinterpret_cast<Piece *>(dst + c1) = y1;
    }
  } else {
    for (int c = lane; c < C; c += kWave) {
      const R v = a[c] + l[c];
      dst[c] = !valid ? nan : (activation == kActTanh ? act_tanh(v) : v);
    }
  }
}

// am.grad[b,t,:] = sum_j grad[b,t,j,:] * act'(out[b,t,j,:]), j in order: one wave per frame.
template <typename R>
__global__ void __launch_bounds__(256)
    joiner_input_am_grad_kernel(const R *__restrict__ grad, const R *__restrict__ act_out,
                                R *__restrict__ am_grad, long frames, int Rr, int C) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long frame = (long)blockIdx.x * 4 + wave;
  const int lane = threadIdx.x & 63;
  if (frame >= frames) return;
  const R *g = grad + frame * Rr * C;
  const R *o = act_out ? act_out + frame * Rr * C : nullptr;
  R *dst = am_grad + frame * C;
  constexpr int kPer = 16 / (int)sizeof(R);
  typedef R Piece __attribute__((ext_vector_type(kPer), aligned(sizeof(R))));
  if (C % kPer == 0) {
    for (int c = kPer * lane; c < C; c += kPer * kWave) {
      Piece acc;
#pragma unroll
      for (int e = 0; e < kPer; ++e) acc[e] = 0;
      int j = 0;
      for (; j + 4 <= Rr; j += 4) {  // four rows in flight
        Piece gv[4], ov[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          gv[u] = *reinterpret_cast<const Piece *>(g + (long)(j + u) * C + c);
          if (o) ov[u] = *reinterpret_cast<const Piece *>(o + (long)(j + u) * C + c);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int e = 0; e < kPer; ++e)
            acc[e] += o ? gv[u][e] * ((R)1 - ov[u][e] * ov[u][e]) : gv[u][e];
      }
      for (; j < Rr; ++j) {
        const Piece gv = *reinterpret_cast<const Piece *>(g + (long)j * C + c);
        Piece ov = gv;
        if (o) ov = *reinterpret_cast<const Piece *>(o + (long)j * C + c);
#pragma unroll
        for (int e = 0; e < kPer; ++e) acc[e] += o ? gv[e] * ((R)1 - ov[e] * ov[e]) : gv[e];
      }
      *reinterpret_cast<Piece *>(dst + c) = acc;
    }
  } else {
    for (int c = lane; c < C; c += kWave) {
      R acc = 0;
      for (int j = 0; j < Rr; ++j) {
        const R gv = g[(long)j * C + c];
        acc += o ? gv * ((R)1 - o[(long)j * C + c] * o[(long)j * C + c]) : gv;
      }
      dst[c] = acc;
    }
  }
}

template <typename R>
int joiner_fwd_impl(const R *am, const R *lm, const int64_t *ranges, R *out, int B, int S, int T,
                    int Rr, int C, int activation, void *stream) {
  if (B < 0 || S < 0 || T < 0 || Rr < 0 || C < 0)
    return fail(FRNNT_EINVAL, "pruned_joiner_fwd: negative size");
  if (activation != kActNone && activation != kActTanh)
    return fail(FRNNT_EINVAL, "pruned_joiner_fwd: activation must be 0 (none) or 1 (tanh)");
  const long rows = (long)B * T * Rr;
  if (rows == 0 || C == 0) return FRNNT_OK;
  if (!am || !lm || !ranges || !out) return fail(FRNNT_EINVAL, "pruned_joiner_fwd: null pointer");
  hipLaunchKernelGGL(joiner_input_kernel<R>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), am, lm, ranges, out, rows, Rr, T * Rr, S + 1,
                     C, activation);
  return check_launch("pruned_joiner_fwd");
}

template <typename R>
int joiner_bwd_impl(const R *grad, const R *out, const int64_t *ranges, R *am_grad, R *lm_grad,
                    int B, int S, int T, int Rr, int C, int activation, void *stream) {
  if (B < 0 || S < 0 || T < 0 || Rr < 0 || C < 0)
    return fail(FRNNT_EINVAL, "pruned_joiner_bwd: negative size");
  if (activation != kActNone && activation != kActTanh)
    return fail(FRNNT_EINVAL, "pruned_joiner_bwd: activation must be 0 (none) or 1 (tanh)");
  if (B == 0 || C == 0) return FRNNT_OK;
  const long frames = (long)B * T;
  if ((long)T * Rr > 0 && (!grad || !ranges || (activation == kActTanh && !out)))
    return fail(FRNNT_EINVAL, "pruned_joiner_bwd: null pointer");
  const R *act_out = activation == kActTanh ? out : nullptr;
  if (am_grad && frames > 0)
    hipLaunchKernelGGL(joiner_input_am_grad_kernel<R>, dim3((unsigned)((frames + 3) / 4)), dim3(256),
                       0, static_cast<hipStream_t>(stream), grad, act_out, am_grad, frames, Rr, C);
  if (lm_grad)
    hipLaunchKernelGGL(prune_scatter_kernel<R>, dim3((unsigned)(B * (S + 1))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), grad, act_out, ranges, lm_grad, T * Rr,
                       S + 1, C);
  return check_launch("pruned_joiner_bwd");
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
  return frnnt::gather_impl<float>(lm, ranges, lm_pruned, B, S, T, R, C, 0x7fc00000, stream);
}
int frnnt_prune_gather_f64(const double *lm, const int64_t *ranges, double *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream) {
  return frnnt::gather_impl<double>(lm, ranges, lm_pruned, B, S, T, R, C, 0, stream);
}
int frnnt_prune_gather_bwd_f32(const float *grad, const int64_t *ranges, float *lm_grad, int B,
                               int S, int T, int R, int C, void *stream) {
  return frnnt::scatter_impl<float>(grad, ranges, lm_grad, B, S, T, R, C, stream);
}
int frnnt_prune_gather_bwd_f64(const double *grad, const int64_t *ranges, double *lm_grad, int B,
                               int S, int T, int R, int C, void *stream) {
  return frnnt::scatter_impl<double>(grad, ranges, lm_grad, B, S, T, R, C, stream);
}
int frnnt_prune_gather_f16(const void *lm, const int64_t *ranges, void *lm_pruned, int B, int S,
                           int T, int R, int C, void *stream) {
  return frnnt::gather_impl<frnnt::f16_t>(static_cast<const frnnt::f16_t *>(lm), ranges,
                                          static_cast<frnnt::f16_t *>(lm_pruned), B, S, T, R, C,
                                          0x7e007e00, stream);
}
int frnnt_prune_gather_bf16(const void *lm, const int64_t *ranges, void *lm_pruned, int B, int S,
                            int T, int R, int C, void *stream) {
  return frnnt::gather_impl<frnnt::bf16_t>(static_cast<const frnnt::bf16_t *>(lm), ranges,
                                           static_cast<frnnt::bf16_t *>(lm_pruned), B, S, T, R, C,
                                           0x7fc07fc0, stream);
}
int frnnt_prune_gather_bwd_f16(const void *grad, const int64_t *ranges, void *lm_grad, int B, int S,
                               int T, int R, int C, void *stream) {
  return frnnt::scatter_impl<frnnt::f16_t>(static_cast<const frnnt::f16_t *>(grad), ranges,
                                           static_cast<frnnt::f16_t *>(lm_grad), B, S, T, R, C,
                                           stream);
}
int frnnt_prune_gather_bwd_bf16(const void *grad, const int64_t *ranges, void *lm_grad, int B,
                                int S, int T, int R, int C, void *stream) {
  return frnnt::scatter_impl<frnnt::bf16_t>(static_cast<const frnnt::bf16_t *>(grad), ranges,
                                            static_cast<frnnt::bf16_t *>(lm_grad), B, S, T, R, C,
                                            stream);
}
int frnnt_pruned_joiner_fwd_f32(const float *am, const float *lm, const int64_t *ranges, float *out,
                                int B, int S, int T, int R, int C, int activation, void *stream) {
  return frnnt::joiner_fwd_impl<float>(am, lm, ranges, out, B, S, T, R, C, activation, stream);
}
int frnnt_pruned_joiner_fwd_f64(const double *am, const double *lm, const int64_t *ranges,
                                double *out, int B, int S, int T, int R, int C, int activation,
                                void *stream) {
  return frnnt::joiner_fwd_impl<double>(am, lm, ranges, out, B, S, T, R, C, activation, stream);
}
int frnnt_pruned_joiner_bwd_f32(const float *grad, const float *out, const int64_t *ranges,
                                float *am_grad, float *lm_grad, int B, int S, int T, int R, int C,
                                int activation, void *stream) {
  return frnnt::joiner_bwd_impl<float>(grad, out, ranges, am_grad, lm_grad, B, S, T, R, C,
                                       activation, stream);
}
int frnnt_pruned_joiner_bwd_f64(const double *grad, const double *out, const int64_t *ranges,
                                double *am_grad, double *lm_grad, int B, int S, int T, int R, int C,
                                int activation, void *stream) {
  return frnnt::joiner_bwd_impl<double>(grad, out, ranges, am_grad, lm_grad, B, S, T, R, C,
                                        activation, stream);
}

}  // extern "C"
