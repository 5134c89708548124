// Lattice ("mutual information") recursion, forward and backward, for gfx950.
//
// Mapping: one workgroup per utterance, one lane per lattice row.  A wave owns
// 64 consecutive rows and sweeps the lattice along anti-diagonals: at local
// step e lane L works on column e - L, so the "up" neighbour is what lane L-1
// produced one step earlier (regular lattice) or two steps earlier (modified
// lattice) and arrives through a DPP wave shift, and the "left" neighbour is the
// lane's own previous result.  Rows beyond 64 go to further waves of the same
// workgroup; wave w+1 consumes the last row of wave w through an LDS seam row
// guarded by a monotone progress counter, so waves run skewed by a chunk or two
// instead of meeting at a barrier every step.  Lattices taller than the
// workgroup are swept band after band with the same seam mechanism.
//
// The arithmetic follows the CPU reference operation for operation
// (fast_rnnt/csrc/mutual_information_cpu.cu:89-121 forward, :179-252 backward,
// log-add from fast_rnnt/csrc/mutual_information.h:36-65); only exp/log1p come
// from the GPU's own units.
#include "common.hip.h"

namespace frnnt {
namespace {

constexpr int kMaxWaves = 16;  // 1024 threads
constexpr int kChunk = 8;      // steps per prefetch / seam hand-over chunk
constexpr int kSpinLimit = 1 << 24;

struct Window {
  int s0, t0, ns, nt;  // origin and extent (ns = s_end - s_begin, ...)
  bool ok;
};

__device__ __forceinline__ Window load_window(const int64_t *boundary, int b, int S, int T) {
  Window w{0, 0, S, T, true};
  if (boundary) {
    const int64_t a = boundary[4 * b + 0], c = boundary[4 * b + 1];
    const int64_t d = boundary[4 * b + 2], e = boundary[4 * b + 3];
    w.ok = (0 <= a) && (a <= d) && (d <= S) && (0 <= c) && (c <= e) && (e <= T);
    w.s0 = (int)a;
    w.t0 = (int)c;
    w.ns = (int)(d - a);
    w.nt = (int)(e - c);
  }
  return w;
}

// Blocks until the producer's counter reaches `target`; gives up (returns false)
// after a bounded number of polls so that no wave can spin forever.
__device__ __forceinline__ bool wait_for(const int *counter, int target) {
  int spins = 0;
  while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
    __builtin_amdgcn_s_sleep(1);
    if (++spins > kSpinLimit) return false;
  }
  return true;
}

template <typename R, bool kModified, int kBlock>
__global__ void __launch_bounds__(kBlock)
    mi_forward_kernel(const R *__restrict__ px, const R *__restrict__ py,
                      const int64_t *__restrict__ boundary, R *__restrict__ p,
                      R *__restrict__ ans, int S, int T) {
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ int ready[kMaxWaves];
  R *seam = reinterpret_cast<R *>(dyn_lds);

  const int b = blockIdx.x;
  const int nw = blockDim.x / kWave;
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int T1 = kModified ? T : T + 1;
  const int TP = T + 1;
  const R ninf = Num<R>::neg_inf();

  const Window win = load_window(boundary, b, S, T);
  if (!win.ok) {
    if (threadIdx.x == 0) ans[b] = std::numeric_limits<R>::quiet_NaN();
    return;
  }
  if (threadIdx.x < kMaxWaves) ready[threadIdx.x] = 0;
  __syncthreads();

  const int NS = win.ns, NT = win.nt, cols = NT + 1;
  const R *pxb = px + (size_t)b * S * T1;
  const R *pyb = py + (size_t)b * (S + 1) * T;
  R *pb = p + (size_t)b * (S + 1) * TP;
  const int band_rows = kWave * nw;
  const int prev = (w + nw - 1) % nw;
  R *my_seam = seam + (size_t)w * TP;
  const R *up_seam = seam + (size_t)prev * TP;

  for (int band = 0; band * band_rows <= NS; ++band) {
    const int row0 = band * band_rows + kWave * w;
    if (row0 > NS) break;
    const int i = row0 + lane;  // lattice row relative to the window
    const int s = win.s0 + i;
    const bool row_ok = i <= NS;
    const int nrows = min(kWave, NS + 1 - row0);
    const bool has_up = row0 > 0;
    const int up_base = (w > 0 ? band : band - 1) * cols;
    const int my_base = band * cols;
    const long x_off = (long)(s - 1) * T1 + win.t0;  // px row feeding this lattice row
    const long y_off = (long)s * T + win.t0;
    const long p_off = (long)s * TP + win.t0;
    const int x_last = kModified ? NT - 1 : NT;
    const int nsteps = NT + nrows;

    R xn[kChunk], yn[kChunk];
    auto fetch = [&](int e0) {
#pragma unroll
      for (int k = 0; k < kChunk; ++k) {
        const int j = e0 + k - lane;
        const int jj = kModified ? j - 1 : j;
        xn[k] = (row_ok && i >= 1 && jj >= 0 && jj <= x_last) ? pxb[x_off + jj] : ninf;
        yn[k] = (row_ok && j >= 1 && j <= NT) ? pyb[y_off + j - 1] : ninf;
      }
    };
    fetch(0);

    R own = ninf, own2 = ninf;
    for (int e0 = 0; e0 < nsteps; e0 += kChunk) {
      R xc[kChunk], yc[kChunk];
#pragma unroll
      for (int k = 0; k < kChunk; ++k) {
        xc[k] = xn[k];
        yc[k] = yn[k];
      }
      if (e0 + kChunk < nsteps) fetch(e0 + kChunk);

      R handed = ninf;  // lane k holds the seam value lane 0 needs at step e0 + k
      if (has_up) {
        const int need = min(e0 + kChunk - (kModified ? 1 : 0), cols);
        if (need > 0 && !wait_for(&ready[prev], up_base + need)) return;
        const int col = e0 + lane - (kModified ? 1 : 0);
        if (lane < kChunk && col >= 0 && col <= NT) handed = up_seam[col];
      }

#pragma unroll
      for (int k = 0; k < kChunk; ++k) {
        const int j = e0 + k - lane;
        const int jj = kModified ? j - 1 : j;
        R up = from_lane_below(kModified ? own2 : own, ninf);
        if (has_up) {
          const R first = lane_value(handed, k);
          if (lane == 0) up = first;
        }
        const R a = (i > 0 && jj >= 0) ? up + xc[k] : ninf;
        const R c = (j > 0) ? own + yc[k] : ninf;
        R v = log_add(a, c);
        if (i == 0 && j == 0) v = 0;
        if (row_ok && j >= 0 && j <= NT) {
          pb[p_off + j] = v;
          if (lane == kWave - 1) my_seam[j] = v;
          if (i == NS && j == NT) ans[b] = v;
        }
        own2 = own;
        own = v;
      }

      if (nrows == kWave && lane == kWave - 1) {
        const int done = max(0, min(e0 + kChunk - (kWave - 1), cols));
        __hip_atomic_store(&ready[w], my_base + done, __ATOMIC_RELEASE,
                           __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
  }
}

// Reverse sweep.  Rows and columns are counted from the end of the window
// (r = NS - i, c = NT - j); lane L of a wave owns reversed row r and works on
// reversed column e - L at local step e.  Each cell adds what its upper
// neighbour hands down (d1 share) and what its right neighbour hands left
// (d2 share), then splits the sum for its own two predecessors.
template <typename R, bool kModified, int kBlock>
__global__ void __launch_bounds__(kBlock)
    mi_backward_kernel(const R *__restrict__ px, const int64_t *__restrict__ boundary,
                       const R *__restrict__ p, R *ans_grad, R *__restrict__ px_grad,
                       R *__restrict__ py_grad, int S, int T, int overwrite_ans_grad) {
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ int ready[kMaxWaves];
  R *seam = reinterpret_cast<R *>(dyn_lds);

  const int b = blockIdx.x;
  const int nw = blockDim.x / kWave;
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int T1 = kModified ? T : T + 1;
  const int TP = T + 1;
  const int shift = kModified ? 1 : 0;

  const Window win = load_window(boundary, b, S, T);
  R *gxb = px_grad + (size_t)b * S * T1;
  R *gyb = py_grad + (size_t)b * (S + 1) * T;

  // exact zeros everywhere the sweep below does not write
  if (boundary) {
    const int s_lo = win.s0, s_hi = win.s0 + win.ns;  // window rows  [s_lo, s_hi]
    const int t_lo = win.t0, t_hi = win.t0 + win.nt;  // window cols  [t_lo, t_hi]
    for (int idx = threadIdx.x; idx < S * T1; idx += blockDim.x) {
      const int s = idx / T1, t = idx - s * T1;
      const bool inside = win.ok && s >= s_lo && s < s_hi && t >= t_lo && t <= t_hi - shift;
      if (!inside) gxb[idx] = 0;
    }
    for (int idx = threadIdx.x; idx < (S + 1) * T; idx += blockDim.x) {
      const int s = idx / T, t = idx - s * T;
      const bool inside = win.ok && s >= s_lo && s <= s_hi && t >= t_lo && t < t_hi;
      if (!inside) gyb[idx] = 0;
    }
  }
  if (!win.ok) return;
  if (threadIdx.x < kMaxWaves) ready[threadIdx.x] = 0;
  __syncthreads();

  const int NS = win.ns, NT = win.nt, cols = NT + 1;
  const R *pxb = px + (size_t)b * S * T1;
  const R *pb = p + (size_t)b * (S + 1) * TP;
  const R seed = ans_grad[b];
  const int band_rows = kWave * nw;
  const int prev = (w + nw - 1) % nw;
  R *my_seam = seam + (size_t)w * TP;
  const R *up_seam = seam + (size_t)prev * TP;

  for (int band = 0; band * band_rows <= NS; ++band) {
    const int row0 = band * band_rows + kWave * w;
    if (row0 > NS) break;
    const int r = row0 + lane;  // reversed row
    const int i = NS - r;       // lattice row relative to the window (may be < 0)
    const int s = win.s0 + i;
    const bool row_ok = r <= NS;
    const int nrows = min(kWave, NS + 1 - row0);
    const bool has_up = row0 > 0;
    const int up_base = (w > 0 ? band : band - 1) * cols;
    const int my_base = band * cols;
    const long here_off = (long)s * TP + win.t0;          // p[s][t0 + j]
    const long below_off = (long)(s - 1) * TP + win.t0;   // p[s-1][t0 + j - shift]
    const long x_off = (long)(s - 1) * T1 + win.t0;       // px[s-1][t0 + j - shift]
    const long gy_off = (long)s * T + win.t0;             // py_grad[s][t0 + j - 1]
    const int nsteps = NT + nrows;

    // d1 / d2 shares of each cell of the chunk (independent of the gradient,
    // so they stay off the serial chain)
    R d1n[kChunk], d2n[kChunk];
    auto shares = [&](int e0) {
#pragma unroll
      for (int k = 0; k < kChunk; ++k) {
        const int c = e0 + k - lane;
        const int j = NT - c;
        R d1 = 0, d2 = 0;
        if (row_ok && c >= 0 && c <= NT) {
          if (i > 0 && j > 0) {
            const R term1 = pb[below_off + j - shift] + pxb[x_off + j - shift];
            R total = pb[here_off + j];
            if (total - total != 0) total = 0;
            d1 = Num<R>::exp_(term1 - total);
            d2 = (R)1 - d1;
            if (d1 - d1 != 0) d1 = d2 = 0;
          } else if (i == 0 && j > 0) {
            d2 = 1;
          } else if (i > 0 && j == 0 && !kModified) {
            d1 = 1;
          }
        }
        d1n[k] = d1;
        d2n[k] = d2;
      }
    };
    shares(0);

    R to_below = 0, to_below2 = 0, to_left = 0;
    for (int e0 = 0; e0 < nsteps; e0 += kChunk) {
      R d1c[kChunk], d2c[kChunk];
#pragma unroll
      for (int k = 0; k < kChunk; ++k) {
        d1c[k] = d1n[k];
        d2c[k] = d2n[k];
      }
      if (e0 + kChunk < nsteps) shares(e0 + kChunk);

      R handed = 0;
      if (has_up) {
        const int need = min(e0 + kChunk - shift, cols);
        if (need > 0 && !wait_for(&ready[prev], up_base + need)) return;
        const int col = e0 + lane - shift;
        if (lane < kChunk && col >= 0 && col <= NT) handed = up_seam[col];
      }

#pragma unroll
      for (int k = 0; k < kChunk; ++k) {
        const int c = e0 + k - lane;
        const int j = NT - c;
        R from_above = from_lane_below(kModified ? to_below2 : to_below, (R)0);
        if (has_up) {
          const R first = lane_value(handed, k);
          if (lane == 0) from_above = first;
        }
        const bool live = row_ok && c >= 0 && c <= NT;
        R g = 0;
        if (r > 0 && c - shift >= 0) g = from_above;
        if (c > 0) g += to_left;
        if (r == 0 && c == 0) g = seed;
        const R down = d1c[k] * g;
        const R left = d2c[k] * g;
        to_below2 = to_below;
        to_below = live ? down : (R)0;
        to_left = live ? left : (R)0;
        if (live) {
          if (i > 0 && (j > 0 || !kModified)) gxb[x_off + j - shift] = down;
          if (j > 0) gyb[gy_off + j - 1] = left;
          if (lane == kWave - 1) my_seam[c] = down;
          if (i == 0 && j == 0 && overwrite_ans_grad) ans_grad[b] = g;
        }
      }

      if (nrows == kWave && lane == kWave - 1) {
        const int done = max(0, min(e0 + kChunk - (kWave - 1), cols));
        __hip_atomic_store(&ready[w], my_base + done, __ATOMIC_RELEASE,
                           __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
  }
}

// Waves per workgroup: enough for every row when the seam rows fit in LDS.
int pick_waves(int S, int T, size_t elem, size_t lds_budget) {
  int nw = (S + 1 + kWave - 1) / kWave;
  if (nw < 1) nw = 1;
  if (nw > kMaxWaves) nw = kMaxWaves;
  while (nw > 1 && (size_t)nw * (T + 1) * elem > lds_budget) --nw;
  return nw;
}

constexpr size_t kLdsBudget = 150 * 1024;

template <typename R>
int forward_impl(const R *px, const R *py, const int64_t *boundary, R *p, R *ans, int B, int S,
                 int T, int modified, void *stream) {
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "mi_forward: negative size");
  if (B == 0) return FRNNT_OK;
  if (!px || !py || !p || !ans) return fail(FRNNT_EINVAL, "mi_forward: null pointer");
  if (modified && S > 0 && T == 0) { /* px has zero columns; still fine */ }
  const int nw = pick_waves(S, T, sizeof(R), kLdsBudget);
  const size_t lds = (size_t)nw * (T + 1) * sizeof(R);
  if (lds > kLdsBudget) return fail(FRNNT_ELIMIT, "mi_forward: T=%d needs %zu bytes of LDS", T, lds);
  // two register budgets: workgroups of up to 4 waves may use 512 VGPRs per lane
  auto kernel = nw <= 4 ? (modified ? mi_forward_kernel<R, true, 256> : mi_forward_kernel<R, false, 256>)
                        : (modified ? mi_forward_kernel<R, true, 1024>
                                    : mi_forward_kernel<R, false, 1024>);
  if (lds > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return check_launch("mi_forward: hipFuncSetAttribute");
  }
  hipLaunchKernelGGL(kernel, dim3(B), dim3(nw * kWave), lds, static_cast<hipStream_t>(stream), px,
                     py, boundary, p, ans, S, T);
  return check_launch("mi_forward");
}

template <typename R>
int backward_impl(const R *px, const R *py, const int64_t *boundary, const R *p, R *ans_grad,
                  R *px_grad, R *py_grad, int B, int S, int T, int modified,
                  int overwrite_ans_grad, void *stream) {
  (void)py;  // the d2 = 1 - d1 split needs only p and px
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "mi_backward: negative size");
  if (B == 0) return FRNNT_OK;
  if (!px || !p || !ans_grad || !px_grad || !py_grad)
    return fail(FRNNT_EINVAL, "mi_backward: null pointer");
  const int nw = pick_waves(S, T, sizeof(R), kLdsBudget);
  const size_t lds = (size_t)nw * (T + 1) * sizeof(R);
  if (lds > kLdsBudget)
    return fail(FRNNT_ELIMIT, "mi_backward: T=%d needs %zu bytes of LDS", T, lds);
  auto kernel = nw <= 4 ? (modified ? mi_backward_kernel<R, true, 256>
                                    : mi_backward_kernel<R, false, 256>)
                        : (modified ? mi_backward_kernel<R, true, 1024>
                                    : mi_backward_kernel<R, false, 1024>);
  if (lds > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return check_launch("mi_backward: hipFuncSetAttribute");
  }
  hipLaunchKernelGGL(kernel, dim3(B), dim3(nw * kWave), lds, static_cast<hipStream_t>(stream), px,
                     boundary, p, ans_grad, px_grad, py_grad, S, T, overwrite_ans_grad);
  return check_launch("mi_backward");
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_mi_forward_f32(const float *px, const float *py, const int64_t *boundary, float *p,
                         float *ans, int B, int S, int T, int modified, void *stream) {
  return frnnt::forward_impl<float>(px, py, boundary, p, ans, B, S, T, modified, stream);
}
int frnnt_mi_forward_f64(const double *px, const double *py, const int64_t *boundary, double *p,
                         double *ans, int B, int S, int T, int modified, void *stream) {
  return frnnt::forward_impl<double>(px, py, boundary, p, ans, B, S, T, modified, stream);
}
int frnnt_mi_backward_f32(const float *px, const float *py, const int64_t *boundary,
                          const float *p, float *ans_grad, float *px_grad, float *py_grad, int B,
                          int S, int T, int modified, int overwrite_ans_grad, void *stream) {
  return frnnt::backward_impl<float>(px, py, boundary, p, ans_grad, px_grad, py_grad, B, S, T,
                                     modified, overwrite_ans_grad, stream);
}
int frnnt_mi_backward_f64(const double *px, const double *py, const int64_t *boundary,
                          const double *p, double *ans_grad, double *px_grad, double *py_grad,
                          int B, int S, int T, int modified, int overwrite_ans_grad,
                          void *stream) {
  return frnnt::backward_impl<double>(px, py, boundary, p, ans_grad, px_grad, py_grad, B, S, T,
                                      modified, overwrite_ans_grad, stream);
}

}  // extern "C"
