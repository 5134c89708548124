// px / py from joiner logits: the unpruned loss (logits [B][T][S+1][C],
// fast_rnnt/python/fast_rnnt/rnnt_loss.py:343-449) and the pruned loss
// (logits [B][T][R][C] plus ranges [B][T][R], rnnt_loss.py:856-1024) share one
// set of kernels; the unpruned case is R = S+1 with every range starting at 0.
//
// Forward, HBM-streaming: one wave per logits row (b, t, j) makes one pass for
// the maximum and one for sum exp(x - max) (the second pass hits L1/L2), then
// emits norm = logsumexp and the two picked log-probs
//   xr[b,t,j] = logits[b,t,j,sym(b, ranges[b,t,j])] - norm   (sym(b, S) = termination symbol)
//   yr[b,t,j] = logits[b,t,j,term] - norm.
// A second, small kernel lays them out as px [B][S][T1] / py [B][S+1][T]: row
// j of frame t lands at lattice row (j + ranges[b,t,0]) mod (S+1), everything
// else is -inf, plus the -inf columns of the regular lattice and the constrained
// "px += py[:, 1:]" step.
//
// Backward, HBM-streaming: one wave per logits row,
//   dlogits[c] = -softmax[c] * (gx + gy) + [c = sym] gx + [c = term] gy
// with gx / gy the px / py gradients of the lattice cell the row was placed at.
#include "common.hip.h"

namespace frnnt {
namespace {

enum { kRegular = 0, kModified = 1, kConstrained = 2 };

template <typename R>
__device__ __forceinline__ R wave_max_all(R v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const R o = __shfl_xor(v, off, 64);
    v = (o > v || o != o) ? o : v;
  }
  return v;
}
template <typename R>
__device__ __forceinline__ R wave_sum_all(R v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <typename R>
__device__ __forceinline__ R exp_acc(R x);
template <>
__device__ __forceinline__ float exp_acc<float>(float x) {
  return __expf(x);
}
template <>
__device__ __forceinline__ double exp_acc<double>(double x) {
  return exp(x);
}
template <typename R>
__device__ __forceinline__ R log_acc(R x);
template <>
__device__ __forceinline__ float log_acc<float>(float x) {
  return logf(x);
}
template <>
__device__ __forceinline__ double log_acc<double>(double x) {
  return log(x);
}

// Symbol scored by row j of frame (b, t): symbols[b][s] for s < S, the
// termination symbol for s == S; -1 if the range entry is out of [0, S].
__device__ __forceinline__ int64_t row_symbol(const int64_t *symbols, const int64_t *ranges,
                                              long row, int b, int j, int S, int term) {
  const int64_t s = ranges ? ranges[row] : j;
  if (s < 0 || s > S) return -1;
  return s == S ? (int64_t)term : symbols[(long)b * S + s];
}

// Lattice row that logits row `row` = (frame, j) is placed at: j without ranges, else
// (ranges[frame][0] + j) mod (S + 1) -- the roll of rnnt_loss.py:968-984, the rule the assembly
// and the gradient kernels follow, whatever the frame's other range entries hold (the
// reference accepts ranges that are not consecutive and rolls by the first entry alone).
__device__ __forceinline__ int64_t placed_row(const int64_t *ranges, long row, int Rr, int S) {
  const int j = (int)(row % Rr);
  if (!ranges) return j;
  int64_t s = ((int64_t)j + ranges[row - j]) % (S + 1);
  return s < 0 ? s + S + 1 : s;
}

// True when the logits row (b, t) x lattice row s lies outside utterance b's boundary
// window [s_begin, s_end] x [t_begin, t_end): the recursion never looks at its px / py
// and hands it a gradient of exact zeros.  Callers that go on to the recursion with the
// same boundary (the loss functions) let the kernels skip such rows -- about a third of
// a ragged batch.  `s` < 0 stands for "not known", only the frame is tested then.
__device__ __forceinline__ bool outside_window(const int64_t *boundary, int b, int t, int64_t s) {
  const int64_t s_begin = boundary[4 * b + 0], t_begin = boundary[4 * b + 1];
  const int64_t s_end = boundary[4 * b + 2], t_end = boundary[4 * b + 3];
  return t < t_begin || t >= t_end || (s >= 0 && (s < s_begin || s > s_end));
}

// 4 rows per 256-thread block.
template <typename R>
__global__ void __launch_bounds__(256)
    row_norm_kernel(const R *__restrict__ logits, const int64_t *__restrict__ symbols,
                    const int64_t *__restrict__ ranges, const int64_t *__restrict__ window,
                    R *__restrict__ norm, R *__restrict__ xr, R *__restrict__ yr, long rows, int T,
                    int Rr, int S, int C, int term) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  if (window &&
      outside_window(window, (int)(row / ((long)Rr * T)), (int)((row / Rr) % T),
                     placed_row(ranges, row, Rr, S)))
    return;
  const R *x = logits + row * C;
  R m = Num<R>::neg_inf();
  for (int c = lane; c < C; c += kWave) {
    const R v = x[c];
    m = (v > m || v != v) ? v : m;
  }
  m = wave_max_all(m);
  const R shift = (m - m == 0) ? m : (R)0;  // torch.logsumexp: infinite max -> shift by 0
  R sum = 0;
  for (int c = lane; c < C; c += kWave) sum += exp_acc<R>(x[c] - shift);
  sum = wave_sum_all(sum);
  const R lse = log_acc<R>(sum) + shift;
  if (lane == 0) {
    const int j = (int)(row % Rr);
    const int b = (int)(row / ((long)Rr * T));
    const int64_t sym = row_symbol(symbols, ranges, row, b, j, S, term);
    norm[row] = lse;
    xr[row] = (sym >= 0 && sym < C) ? x[sym] - lse : std::numeric_limits<R>::quiet_NaN();
    yr[row] = x[term] - lse;
  }
}

// The same with the rows held in registers (fp32, C a multiple of 4, at most
// 256 * kVecs entries).  A wave takes kRows consecutive rows (the launchers use 1: more
// rows per wave were slower).  The rows are fetched through a raw buffer resource
// that covers just the wave's rows -- 16 bytes per lane and load, every load of every row
// in flight before the first is used; a row that needs no work (past the end, or outside
// the boundary window when the caller asked for that) and a piece past the end of a row
// get an offset outside the resource, which reads as 0 and moves no data: no branch
// stands between the loads.  The two entries a row contributes to px / py are taken from
// the registers that hold them (selects under wave-uniform conditions, then a read of
// the owning lane), not read again from memory.  `kStream`: the logits exceed what the
// last-level cache holds, so they are read with the non-temporal hint.
typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
constexpr int kOutOfRange = (int)0x80000000;  // an offset outside every buffer resource
template <int kVecs>
__device__ __forceinline__ float row_entry(const floatx4u (&v)[kVecs], int c) {
  // c is wave-uniform and inside the row
  const int piece = c >> 2, e = c & 3, vec = piece / kWave, owner = piece % kWave;
  float cand = v[0][0];
#pragma unroll
  for (int i = 0; i < kVecs; ++i)
#pragma unroll
    for (int k = 0; k < 4; ++k) cand = (i == vec && k == e) ? v[i][k] : cand;
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cand), owner));
}
__device__ __forceinline__ floatx4u as_floats(intx4 raw) {
  return floatx4u{__int_as_float(raw[0]), __int_as_float(raw[1]), __int_as_float(raw[2]),
                  __int_as_float(raw[3])};
}
// which rows of the wave's group need work (bit r), wave-uniform
template <int kRows>
__device__ __forceinline__ unsigned live_rows(long first, long rows, const int64_t *ranges,
                                              const int64_t *window, int T, int Rr, int S) {
  unsigned live = 0;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const long row = first + r;
    if (row >= rows) break;
    bool needed = true;
    if (window)
      needed = !outside_window(window, (int)(row / ((long)Rr * T)), (int)((row / Rr) % T),
                               placed_row(ranges, row, Rr, S));
    live |= needed ? 1u << r : 0u;
  }
  return live;
}
template <int kVecs, int kRows, bool kStream>
__global__ void __launch_bounds__(256)
    row_norm_regs_kernel(const float *__restrict__ logits, const int64_t *__restrict__ symbols,
                         const int64_t *__restrict__ ranges,
                         const int64_t *__restrict__ window, float *__restrict__ norm,
                         float *__restrict__ xr, float *__restrict__ yr, long rows, int T, int Rr,
                         int S, int C, int term) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register
  const long first = ((long)blockIdx.x * 4 + wave) * kRows;
  const int lane = threadIdx.x & 63;
  if (first >= rows) return;
  const unsigned live = live_rows<kRows>(first, rows, ranges, window, T, Rr, S);
  if (live == 0) return;
  const long here = rows - first < kRows ? rows - first : kRows;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(logits + first * C), 0, (int)(here * C * 4), 0x00020000);
  constexpr int kAux = kStream ? 2 : 0;
  floatx4u v[kRows][kVecs];
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
      const int c = 4 * (lane + kWave * i);
      const bool wanted = ((live >> r) & 1) && c < C;
      v[r][i] = as_floats(
          __builtin_amdgcn_raw_buffer_load_b128(rs, wanted ? (r * C + c) * 4 : kOutOfRange, 0, kAux));
    }
  const float ninf = -__builtin_huge_valf();
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    if (!((live >> r) & 1)) continue;  // wave-uniform
    const long row = first + r;
    // what lies past the end of the row takes no part
#pragma unroll
    for (int i = 0; i < kVecs; ++i)
      if (4 * (lane + kWave * i) >= C) v[r][i] = floatx4u{ninf, ninf, ninf, ninf};
    const int j = (int)(row % Rr);
    const int b = (int)(row / ((long)Rr * T));
    const int64_t sym = row_symbol(symbols, ranges, row, b, j, S, term);
    float m = ninf;
#pragma unroll
    for (int i = 0; i < kVecs; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) m = (v[r][i][e] > m || v[r][i][e] != v[r][i][e]) ? v[r][i][e] : m;
    m = wave_max_all(m);
    const float shift = (m - m == 0) ? m : 0.f;  // torch.logsumexp: infinite max -> shift by 0
    float sum = 0;
#pragma unroll
    for (int i = 0; i < kVecs; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) sum += __expf(v[r][i][e] - shift);  // padding is -inf: adds 0
    sum = wave_sum_all(sum);
    const float lse = logf(sum) + shift;
    const float at_sym = (sym >= 0 && sym < C) ? row_entry<kVecs>(v[r], (int)sym) - lse
                                               : std::numeric_limits<float>::quiet_NaN();
    const float at_term = row_entry<kVecs>(v[r], term) - lse;
    if (lane == 0) {
      norm[row] = lse;
      xr[row] = at_sym;
      yr[row] = at_term;
    }
  }
}

// Logits beyond this many bytes do not stay in the last-level cache between the forward
// and the backward pass: they are streamed (non-temporal hint), which leaves the cache to
// what is used again.  Below it the hint costs (a 80 MB gradient pass: 23.8 -> 26.6 us).
constexpr long kStreamBytes = 192L << 20;

template <typename R>
bool launch_row_norm_regs(const R *, const int64_t *, const int64_t *, const int64_t *, R *, R *,
                          R *, long, int, int, int, int, int, hipStream_t) {
  return false;
}
template <>
bool launch_row_norm_regs<float>(const float *logits, const int64_t *symbols, const int64_t *ranges,
                                 const int64_t *window, float *norm, float *xr, float *yr, long rows,
                                 int T, int Rr, int S, int C, int term, hipStream_t stream) {
  if (C % 4 != 0 || C > 256 * 16) return false;
  const bool big = rows * C * 4 > kStreamBytes;
#define FRNNT_ROW_NORM(V, N)                                                                     \
  do {                                                                                           \
    const dim3 grid((unsigned)((rows + 4 * N - 1) / (4 * N))), block(256);                       \
    if (big)                                                                                     \
      hipLaunchKernelGGL((row_norm_regs_kernel<V, N, true>), grid, block, 0, stream, logits,     \
                         symbols, ranges, window, norm, xr, yr, rows, T, Rr, S, C, term);        \
    else                                                                                         \
      hipLaunchKernelGGL((row_norm_regs_kernel<V, N, false>), grid, block, 0, stream, logits,    \
                         symbols, ranges, window, norm, xr, yr, rows, T, Rr, S, C, term);        \
  } while (0)
  // (one row per wave: two or four rows per wave were measured 3 to 10 % slower on
  // 390 MB and on 80 MB of logits)
  if (C <= 256)
    FRNNT_ROW_NORM(1, 1);
  else if (C <= 512)
    FRNNT_ROW_NORM(2, 1);
  else if (C <= 1024)
    FRNNT_ROW_NORM(4, 1);
  else if (C <= 2048)
    FRNNT_ROW_NORM(8, 1);
  else
    FRNNT_ROW_NORM(16, 1);
#undef FRNNT_ROW_NORM
  return true;
}

// One thread per px / py element, t fastest (coalesced stores).
template <typename R>
__global__ void __launch_bounds__(256)
    assemble_kernel(const R *__restrict__ xr, const R *__restrict__ yr,
                    const int64_t *__restrict__ ranges, const int64_t *__restrict__ boundary,
                    R *__restrict__ px, R *__restrict__ py, int B, int S, int T, int Rr,
                    int rnnt_type) {
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int S1 = S + 1;
  const long n_px = (long)B * S * T1, n_py = (long)B * S1 * T;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const R ninf = Num<R>::neg_inf();
  // value of the staged row that the roll places at lattice row s of frame t
  auto placed = [&](const R *src, int b, int s, int t) -> R {
    const long frame = ((long)b * T + t) * Rr;
    const int64_t r0 = ranges ? ranges[frame] : 0;
    int64_t rel = ((int64_t)s - r0) % S1;
    if (rel < 0) rel += S1;
    return rel < Rr ? src[frame + rel] : ninf;
  };
  if (idx < n_px) {
    const int b = (int)(idx / ((long)S * T1));
    const long rem = idx - (long)b * S * T1;
    const int s = (int)(rem / T1), t = (int)(rem % T1);
    R v = ninf;
    if (t < T) {
      v = placed(xr, b, s, t);
      if (rnnt_type == kRegular && boundary && boundary[4 * b + 3] == t) v = ninf;
      if (rnnt_type == kConstrained) v += placed(yr, b, s + 1, t);
    }
    px[idx] = v;
  } else if (idx < n_px + n_py) {
    const long k = idx - n_px;
    const int b = (int)(k / ((long)S1 * T));
    const long rem = k - (long)b * S1 * T;
    const int s = (int)(rem / T), t = (int)(rem % T);
    py[k] = placed(yr, b, s, t);
  }
}

// One wave per logits row.
template <typename R>
__global__ void __launch_bounds__(256)
    row_grad_kernel(const R *__restrict__ logits, const int64_t *__restrict__ symbols,
                    const int64_t *__restrict__ ranges, const int64_t *__restrict__ boundary,
                    const int64_t *__restrict__ window, const R *__restrict__ norm,
                    const R *__restrict__ gpx, const R *__restrict__ gpy, R *__restrict__ glogits,
                    long rows, int S, int T, int Rr, int C, int term, int rnnt_type) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  if (window &&
      outside_window(window, (int)(row / ((long)Rr * T)), (int)((row / Rr) % T),
                     placed_row(ranges, row, Rr, S))) {
    for (int c = lane; c < C; c += kWave) glogits[row * C + c] = 0;
    return;
  }
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int j = (int)(row % Rr);
  const long frame = row / Rr;
  const int t = (int)(frame % T), b = (int)(frame / T);
  const int64_t r0 = ranges ? ranges[frame * Rr] : 0;
  // lattice row this logits row was placed at; rows the roll pushes past S+1 wrap
  // around exactly as in the forward pass
  int64_t s64 = ((int64_t)j + r0) % S1;
  if (s64 < 0) s64 += S1;
  const int s = (int)s64;
  const bool masked = rnnt_type == kRegular && boundary && boundary[4 * b + 3] == t;
  auto gx_at = [&](int ss) -> R {
    if (ss < 0 || ss >= S || masked) return (R)0;
    return gpx[((long)b * S + ss) * T1 + t];
  };
  const R gx = gx_at(s);
  R gy = gpy[((long)b * S1 + s) * T + t];
  if (rnnt_type == kConstrained) gy += gx_at(s - 1);
  const int64_t sym = row_symbol(symbols, ranges, row, b, j, S, term);
  const R lse = norm[row];
  const R w = -(gx + gy);
  const R *x = logits + row * C;
  R *g = glogits + row * C;
  for (int c = lane; c < C; c += kWave) {
    R v = exp_acc<R>(x[c] - lse) * w;
    if (c == sym) v += gx;
    if (c == term) v += gy;
    g[c] = v;
  }
}

// The same with the rows held in registers (fp32, C a multiple of 4, at most
// 256 * kVecs entries), kRows consecutive rows per wave as in row_norm_regs_kernel: every
// load of every row is in flight (branch-free, through a buffer resource over the wave's
// rows) while the rows' scalars (range, gradients, normalizer) are looked up; the gradient
// leaves as 16-byte stores.  A row outside the window (when the caller says the gradients
// vanish there) is not read: exact zeros are stored.
template <int kVecs, int kRows, bool kStream>
__global__ void __launch_bounds__(256)
    row_grad_regs_kernel(const float *__restrict__ logits, const int64_t *__restrict__ symbols,
                         const int64_t *__restrict__ ranges, const int64_t *__restrict__ boundary,
                         const int64_t *__restrict__ window, const float *__restrict__ norm,
                         const float *__restrict__ gpx, const float *__restrict__ gpy,
                         float *__restrict__ glogits, long rows, int S, int T, int Rr, int C,
                         int term, int rnnt_type) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register
  const long first = ((long)blockIdx.x * 4 + wave) * kRows;
  const int lane = threadIdx.x & 63;
  if (first >= rows) return;
  const unsigned live = live_rows<kRows>(first, rows, ranges, window, T, Rr, S);
  const long here = rows - first < kRows ? rows - first : kRows;
  const __amdgpu_buffer_rsrc_t in_rs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(logits + first * C), 0, (int)(here * C * 4), 0x00020000);
  const __amdgpu_buffer_rsrc_t out_rs =
      __builtin_amdgcn_make_buffer_rsrc(glogits + first * C, 0, (int)(here * C * 4), 0x00020000);
  constexpr int kAux = kStream ? 2 : 0;
  floatx4u v[kRows][kVecs];
#pragma unroll
  for (int r = 0; r < kRows; ++r)
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
      const int c = 4 * (lane + kWave * i);
      const bool wanted = ((live >> r) & 1) && c < C;
      v[r][i] = as_floats(
          __builtin_amdgcn_raw_buffer_load_b128(in_rs, wanted ? (r * C + c) * 4 : kOutOfRange, 0, kAux));
    }
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const long row = first + r;
    if (row >= rows) break;
    float gx = 0.f, gy = 0.f, lse = 0.f;
    int sym = -1;
    if ((live >> r) & 1) {  // wave-uniform
      const int j = (int)(row % Rr);
      const long frame = row / Rr;
      const int t = (int)(frame % T), b = (int)(frame / T);
      const int64_t r0 = ranges ? ranges[frame * Rr] : 0;
      int64_t s64 = ((int64_t)j + r0) % S1;
      if (s64 < 0) s64 += S1;
      const int s = (int)s64;
      const bool masked = rnnt_type == kRegular && boundary && boundary[4 * b + 3] == t;
      auto gx_at = [&](int ss) -> float {
        if (ss < 0 || ss >= S || masked) return 0.f;
        return gpx[((long)b * S + ss) * T1 + t];
      };
      gx = gx_at(s);
      gy = gpy[((long)b * S1 + s) * T + t];
      if (rnnt_type == kConstrained) gy += gx_at(s - 1);
      sym = (int)row_symbol(symbols, ranges, row, b, j, S, term);
      lse = norm[row];
    }
    const float w = -(gx + gy);
    const bool zero = !((live >> r) & 1);
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
      const int c = 4 * (lane + kWave * i);
      intx4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float g = __expf(v[r][i][e] - lse) * w;
        if (c + e == sym) g += gx;
        if (c + e == term) g += gy;
        o[e] = zero ? 0 : __float_as_int(g);  // (term may equal an entry of a skipped row)
      }
      __builtin_amdgcn_raw_buffer_store_b128(o, out_rs, c < C ? (r * C + c) * 4 : kOutOfRange, 0,
                                             kAux);
    }
  }
}

template <typename R>
bool launch_row_grad_regs(const R *, const int64_t *, const int64_t *, const int64_t *,
                          const int64_t *, const R *, const R *, const R *, R *, long, int, int, int,
                          int, int, int, hipStream_t) {
  return false;
}
template <>
bool launch_row_grad_regs<float>(const float *logits, const int64_t *symbols, const int64_t *ranges,
                                 const int64_t *boundary, const int64_t *window, const float *norm,
                                 const float *gpx, const float *gpy, float *glogits, long rows,
                                 int S, int T, int Rr, int C, int term, int rnnt_type,
                                 hipStream_t stream) {
  if (C % 4 != 0 || C > 256 * 16) return false;
  const bool big = rows * C * 4 > kStreamBytes;
#define FRNNT_ROW_GRAD(V, N)                                                                     \
  do {                                                                                           \
    const dim3 grid((unsigned)((rows + 4 * N - 1) / (4 * N))), block(256);                       \
    if (big)                                                                                     \
      hipLaunchKernelGGL((row_grad_regs_kernel<V, N, true>), grid, block, 0, stream, logits,     \
                         symbols, ranges, boundary, window, norm, gpx, gpy, glogits, rows, S, T, \
                         Rr, C, term, rnnt_type);                                                \
    else                                                                                         \
      hipLaunchKernelGGL((row_grad_regs_kernel<V, N, false>), grid, block, 0, stream, logits,    \
                         symbols, ranges, boundary, window, norm, gpx, gpy, glogits, rows, S, T, \
                         Rr, C, term, rnnt_type);                                                \
  } while (0)
  if (C <= 256)
    FRNNT_ROW_GRAD(1, 1);
  else if (C <= 512)
    FRNNT_ROW_GRAD(2, 1);
  else if (C <= 1024)
    FRNNT_ROW_GRAD(4, 1);
  else if (C <= 2048)
    FRNNT_ROW_GRAD(8, 1);
  else
    FRNNT_ROW_GRAD(16, 1);
#undef FRNNT_ROW_GRAD
  return true;
}

// ---- 2-byte logits (float16 / bfloat16) ----------------------------------------------
// The reference's recursion has no half-precision form (mutual_information_cuda.cu:37-38
// notes the missing half LogAdd), so half or bfloat16 logits there need a float32 copy
// first.  Here they are read as they are -- half the bytes of the dominant stream -- and
// everything after the load is float32: the normalizer, the picked log-probs, px / py, the
// recursion and its gradients.  Only logits.grad goes back out in the 2-byte type.
// the eight values of a 16-byte piece
template <typename IO>
__device__ __forceinline__ void unpack8(intx4 raw, float (&out)[8]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    out[2 * k] = IO::load((uint16_t)((unsigned)raw[k] & 0xffffu));
    out[2 * k + 1] = IO::load((uint16_t)((unsigned)raw[k] >> 16));
  }
}
// entry c of a row held as 8-value pieces (c wave-uniform and inside the row)
template <int kVecs>
__device__ __forceinline__ float row_entry8(const float (&v)[kVecs][8], int c) {
  const int piece = c >> 3, e = c & 7, vec = piece / kWave, owner = piece % kWave;
  float cand = v[0][0];
#pragma unroll
  for (int i = 0; i < kVecs; ++i)
#pragma unroll
    for (int k = 0; k < 8; ++k) cand = (i == vec && k == e) ? v[i][k] : cand;
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cand), owner));
}

// One wave per row, the row in registers as float32 (C a multiple of 8, at most
// 512 * kVecs entries): the 2-byte counterpart of row_norm_regs_kernel.
template <typename IO, int kVecs, bool kStream>
__global__ void __launch_bounds__(256)
    row_norm_narrow_kernel(const uint16_t *__restrict__ logits, const int64_t *__restrict__ symbols,
                           const int64_t *__restrict__ ranges, const int64_t *__restrict__ window,
                           float *__restrict__ norm, float *__restrict__ xr, float *__restrict__ yr,
                           long rows, int T, int Rr, int S, int C, int term) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long row = (long)blockIdx.x * 4 + wave;
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  if (live_rows<1>(row, rows, ranges, window, T, Rr, S) == 0) return;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t *>(logits + row * C), 0, C * 2, 0x00020000);
  constexpr int kAux = kStream ? 2 : 0;
  intx4 raw[kVecs];
#pragma unroll
  for (int i = 0; i < kVecs; ++i) {
    const int c = 8 * (lane + kWave * i);
    raw[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, c < C ? c * 2 : kOutOfRange, 0, kAux);
  }
  const float ninf = -__builtin_huge_valf();
  float v[kVecs][8];
#pragma unroll
  for (int i = 0; i < kVecs; ++i) {
    unpack8<IO>(raw[i], v[i]);
    if (8 * (lane + kWave * i) >= C) {  // what lies past the end of the row takes no part
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] = ninf;
    }
  }
  const int j = (int)(row % Rr);
  const int b = (int)(row / ((long)Rr * T));
  const int64_t sym = row_symbol(symbols, ranges, row, b, j, S, term);
  float m = ninf;
#pragma unroll
  for (int i = 0; i < kVecs; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) m = (v[i][e] > m || v[i][e] != v[i][e]) ? v[i][e] : m;
  m = wave_max_all(m);
  const float shift = (m - m == 0) ? m : 0.f;  // torch.logsumexp: infinite max -> shift by 0
  float sum = 0;
#pragma unroll
  for (int i = 0; i < kVecs; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += __expf(v[i][e] - shift);
  sum = wave_sum_all(sum);
  const float lse = logf(sum) + shift;
  const float at_sym = (sym >= 0 && sym < C) ? row_entry8<kVecs>(v, (int)sym) - lse
                                             : std::numeric_limits<float>::quiet_NaN();
  const float at_term = row_entry8<kVecs>(v, term) - lse;
  if (lane == 0) {
    norm[row] = lse;
    xr[row] = at_sym;
    yr[row] = at_term;
  }
}

// any row length: lanes stride over the row, two passes (the second hits the cache)
template <typename IO>
__global__ void __launch_bounds__(256)
    row_norm_narrow_any_kernel(const uint16_t *__restrict__ logits,
                               const int64_t *__restrict__ symbols,
                               const int64_t *__restrict__ ranges,
                               const int64_t *__restrict__ window, float *__restrict__ norm,
                               float *__restrict__ xr, float *__restrict__ yr, long rows, int T,
                               int Rr, int S, int C, int term) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  if (live_rows<1>(row, rows, ranges, window, T, Rr, S) == 0) return;
  const uint16_t *x = logits + row * C;
  float m = -__builtin_huge_valf();
  for (int c = lane; c < C; c += kWave) {
    const float v = IO::load(x[c]);
    m = (v > m || v != v) ? v : m;
  }
  m = wave_max_all(m);
  const float shift = (m - m == 0) ? m : 0.f;
  float sum = 0;
  for (int c = lane; c < C; c += kWave) sum += __expf(IO::load(x[c]) - shift);
  sum = wave_sum_all(sum);
  const float lse = logf(sum) + shift;
  if (lane == 0) {
    const int j = (int)(row % Rr);
    const int b = (int)(row / ((long)Rr * T));
    const int64_t sym = row_symbol(symbols, ranges, row, b, j, S, term);
    norm[row] = lse;
    xr[row] = (sym >= 0 && sym < C) ? IO::load(x[sym]) - lse
                                    : std::numeric_limits<float>::quiet_NaN();
    yr[row] = IO::load(x[term]) - lse;
  }
}

// What the gradient of a logits row needs besides the row (all wave-uniform): the px / py
// gradients of the lattice cell the row was placed at, its symbol and its normalizer.
struct RowScalars {
  float gx, gy, lse;
  int sym;
};
__device__ __forceinline__ RowScalars row_scalars(long row, const int64_t *symbols,
                                                  const int64_t *ranges, const int64_t *boundary,
                                                  const float *norm, const float *gpx,
                                                  const float *gpy, int S, int T, int Rr, int term,
                                                  int rnnt_type) {
  const int S1 = S + 1;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const int j = (int)(row % Rr);
  const long frame = row / Rr;
  const int t = (int)(frame % T), b = (int)(frame / T);
  const int64_t r0 = ranges ? ranges[frame * Rr] : 0;
  int64_t s64 = ((int64_t)j + r0) % S1;
  if (s64 < 0) s64 += S1;
  const int s = (int)s64;
  const bool masked = rnnt_type == kRegular && boundary && boundary[4 * b + 3] == t;
  auto gx_at = [&](int ss) -> float {
    if (ss < 0 || ss >= S || masked) return 0.f;
    return gpx[((long)b * S + ss) * T1 + t];
  };
  RowScalars r;
  r.gx = gx_at(s);
  r.gy = gpy[((long)b * S1 + s) * T + t];
  if (rnnt_type == kConstrained) r.gy += gx_at(s - 1);
  r.sym = (int)row_symbol(symbols, ranges, row, b, j, S, term);
  r.lse = norm[row];
  return r;
}

template <typename IO, int kVecs, bool kStream>
__global__ void __launch_bounds__(256)
    row_grad_narrow_kernel(const uint16_t *__restrict__ logits, const int64_t *__restrict__ symbols,
                           const int64_t *__restrict__ ranges, const int64_t *__restrict__ boundary,
                           const int64_t *__restrict__ window, const float *__restrict__ norm,
                           const float *__restrict__ gpx, const float *__restrict__ gpy,
                           uint16_t *__restrict__ glogits, long rows, int S, int T, int Rr, int C,
                           int term, int rnnt_type) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long row = (long)blockIdx.x * 4 + wave;
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  const bool live = live_rows<1>(row, rows, ranges, window, T, Rr, S) != 0;  // wave-uniform
  const __amdgpu_buffer_rsrc_t in_rs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t *>(logits + row * C), 0, C * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t out_rs =
      __builtin_amdgcn_make_buffer_rsrc(glogits + row * C, 0, C * 2, 0x00020000);
  constexpr int kAux = kStream ? 2 : 0;
  intx4 raw[kVecs];
#pragma unroll
  for (int i = 0; i < kVecs; ++i) {
    const int c = 8 * (lane + kWave * i);
    raw[i] = __builtin_amdgcn_raw_buffer_load_b128(in_rs, (live && c < C) ? c * 2 : kOutOfRange, 0,
                                                   kAux);
  }
  RowScalars k{0.f, 0.f, 0.f, -1};
  if (live)
    k = row_scalars(row, symbols, ranges, boundary, norm, gpx, gpy, S, T, Rr, term, rnnt_type);
  const float w = -(k.gx + k.gy);
#pragma unroll
  for (int i = 0; i < kVecs; ++i) {
    const int c = 8 * (lane + kWave * i);
    float v[8];
    unpack8<IO>(raw[i], v);
    intx4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      unsigned packed = 0;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int e = 2 * q + h;
        float g = __expf(v[e] - k.lse) * w;
        if (c + e == k.sym) g += k.gx;
        if (c + e == term) g += k.gy;
        // a row outside the window is not read and gets exact zeros
        packed |= (unsigned)(live ? IO::store(g) : (uint16_t)0) << (16 * h);
      }
      o[q] = (int)packed;
    }
    __builtin_amdgcn_raw_buffer_store_b128(o, out_rs, c < C ? c * 2 : kOutOfRange, 0, kAux);
  }
}

template <typename IO>
__global__ void __launch_bounds__(256)
    row_grad_narrow_any_kernel(const uint16_t *__restrict__ logits,
                               const int64_t *__restrict__ symbols,
                               const int64_t *__restrict__ ranges,
                               const int64_t *__restrict__ boundary,
                               const int64_t *__restrict__ window, const float *__restrict__ norm,
                               const float *__restrict__ gpx, const float *__restrict__ gpy,
                               uint16_t *__restrict__ glogits, long rows, int S, int T, int Rr,
                               int C, int term, int rnnt_type) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  uint16_t *g = glogits + row * C;
  if (live_rows<1>(row, rows, ranges, window, T, Rr, S) == 0) {
    for (int c = lane; c < C; c += kWave) g[c] = 0;
    return;
  }
  const RowScalars k =
      row_scalars(row, symbols, ranges, boundary, norm, gpx, gpy, S, T, Rr, term, rnnt_type);
  const float w = -(k.gx + k.gy);
  const uint16_t *x = logits + row * C;
  for (int c = lane; c < C; c += kWave) {
    float v = __expf(IO::load(x[c]) - k.lse) * w;
    if (c == k.sym) v += k.gx;
    if (c == term) v += k.gy;
    g[c] = IO::store(v);
  }
}

template <typename IO>
int narrow_fwd_impl(const void *logits_, const int64_t *symbols, const int64_t *ranges,
                    const int64_t *boundary, float *px, float *py, float *norm, float *xr,
                    float *yr, int B, int S, int T, int Rr, int C, int term, int rnnt_type,
                    int window_only, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || Rr < 1 || C < 1)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: bad size");
  if (Rr > S + 1) return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: more range rows than S + 1");
  if (!ranges && Rr != S + 1)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: without ranges the logits need S + 1 rows");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: bad rnnt_type or termination symbol");
  if (B == 0) return FRNNT_OK;
  if (!logits_ || (!symbols && S > 0) || !px || !py || !norm || !xr || !yr)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: null pointer");
  const uint16_t *logits = static_cast<const uint16_t *>(logits_);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long rows = (long)B * T * Rr;
  const int64_t *window = window_only ? boundary : nullptr;
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const bool big = rows * C * 2 > kStreamBytes;
#define FRNNT_NARROW_NORM(V)                                                                     \
  do {                                                                                           \
    if (big)                                                                                     \
      hipLaunchKernelGGL((row_norm_narrow_kernel<IO, V, true>), grid, block, 0, stream, logits,  \
                         symbols, ranges, window, norm, xr, yr, rows, T, Rr, S, C, term);        \
    else                                                                                         \
      hipLaunchKernelGGL((row_norm_narrow_kernel<IO, V, false>), grid, block, 0, stream, logits, \
                         symbols, ranges, window, norm, xr, yr, rows, T, Rr, S, C, term);        \
  } while (0)
  if (rows > 0) {
    if (C % 8 != 0 || C > 512 * 8 || (reinterpret_cast<uintptr_t>(logits) & 15))
      hipLaunchKernelGGL(row_norm_narrow_any_kernel<IO>, grid, block, 0, stream, logits, symbols,
                         ranges, window, norm, xr, yr, rows, T, Rr, S, C, term);
    else if (C <= 512)
      FRNNT_NARROW_NORM(1);
    else if (C <= 1024)
      FRNNT_NARROW_NORM(2);
    else if (C <= 2048)
      FRNNT_NARROW_NORM(4);
    else
      FRNNT_NARROW_NORM(8);
  }
#undef FRNNT_NARROW_NORM
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const long total = (long)B * S * T1 + (long)B * (S + 1) * T;
  if (total > 0)
    hipLaunchKernelGGL(assemble_kernel<float>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       stream, xr, yr, ranges, boundary, px, py, B, S, T, Rr, rnnt_type);
  return check_launch("lattice_logprobs_fwd");
}

template <typename IO>
int narrow_bwd_impl(const void *logits_, const int64_t *symbols, const int64_t *ranges,
                    const int64_t *boundary, const float *norm, const float *px_grad,
                    const float *py_grad, void *logits_grad_, int B, int S, int T, int Rr, int C,
                    int term, int rnnt_type, int window_only, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || Rr < 1 || C < 1 || Rr > S + 1 || (!ranges && Rr != S + 1))
    return fail(FRNNT_EINVAL, "lattice_logprobs_bwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "lattice_logprobs_bwd: bad rnnt_type or termination symbol");
  if (B == 0 || T == 0) return FRNNT_OK;
  if (!logits_ || (!symbols && S > 0) || !norm || !px_grad || !py_grad || !logits_grad_)
    return fail(FRNNT_EINVAL, "lattice_logprobs_bwd: null pointer");
  const uint16_t *logits = static_cast<const uint16_t *>(logits_);
  uint16_t *glogits = static_cast<uint16_t *>(logits_grad_);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long rows = (long)B * T * Rr;
  const int64_t *window = window_only ? boundary : nullptr;
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const bool big = rows * C * 2 > kStreamBytes;
#define FRNNT_NARROW_GRAD(V)                                                                      \
  do {                                                                                            \
    if (big)                                                                                      \
      hipLaunchKernelGGL((row_grad_narrow_kernel<IO, V, true>), grid, block, 0, stream, logits,   \
                         symbols, ranges, boundary, window, norm, px_grad, py_grad, glogits,      \
                         rows, S, T, Rr, C, term, rnnt_type);                                     \
    else                                                                                          \
      hipLaunchKernelGGL((row_grad_narrow_kernel<IO, V, false>), grid, block, 0, stream, logits,  \
                         symbols, ranges, boundary, window, norm, px_grad, py_grad, glogits,      \
                         rows, S, T, Rr, C, term, rnnt_type);                                     \
  } while (0)
  if (C % 8 != 0 || C > 512 * 8 ||
      ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(glogits)) & 15))
    hipLaunchKernelGGL(row_grad_narrow_any_kernel<IO>, grid, block, 0, stream, logits, symbols,
                       ranges, boundary, window, norm, px_grad, py_grad, glogits, rows, S, T, Rr,
                       C, term, rnnt_type);
  else if (C <= 512)
    FRNNT_NARROW_GRAD(1);
  else if (C <= 1024)
    FRNNT_NARROW_GRAD(2);
  else if (C <= 2048)
    FRNNT_NARROW_GRAD(4);
  else
    FRNNT_NARROW_GRAD(8);
#undef FRNNT_NARROW_GRAD
  return check_launch("lattice_logprobs_bwd");
}

template <typename R>
int fwd_impl(const R *logits, const int64_t *symbols, const int64_t *ranges,
             const int64_t *boundary, R *px, R *py, R *norm, R *xr, R *yr, int B, int S, int T,
             int Rr, int C, int term, int rnnt_type, int window_only, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || Rr < 1 || C < 1)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: bad size");
  if (Rr > S + 1) return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: more range rows than S + 1");
  if (!ranges && Rr != S + 1)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: without ranges the logits need S + 1 rows");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: bad rnnt_type or termination symbol");
  if (B == 0) return FRNNT_OK;
  if (!logits || (!symbols && S > 0) || !px || !py || !norm || !xr || !yr)
    return fail(FRNNT_EINVAL, "lattice_logprobs_fwd: null pointer");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long rows = (long)B * T * Rr;
  const int64_t *window = window_only ? boundary : nullptr;
  if (rows > 0)
    if (!launch_row_norm_regs<R>(logits, symbols, ranges, window, norm, xr, yr, rows, T, Rr, S, C,
                                 term, stream))
      hipLaunchKernelGGL(row_norm_kernel<R>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                         stream, logits, symbols, ranges, window, norm, xr, yr, rows, T, Rr, S, C,
                         term);
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  const long total = (long)B * S * T1 + (long)B * (S + 1) * T;
  if (total > 0)
    hipLaunchKernelGGL(assemble_kernel<R>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       stream, xr, yr, ranges, boundary, px, py, B, S, T, Rr, rnnt_type);
  return check_launch("lattice_logprobs_fwd");
}

template <typename R>
int bwd_impl(const R *logits, const int64_t *symbols, const int64_t *ranges,
             const int64_t *boundary, const R *norm, const R *px_grad, const R *py_grad,
             R *logits_grad, int B, int S, int T, int Rr, int C, int term, int rnnt_type,
             int window_only, void *stream_) {
  if (B < 0 || S < 0 || T < 0 || Rr < 1 || C < 1 || Rr > S + 1 || (!ranges && Rr != S + 1))
    return fail(FRNNT_EINVAL, "lattice_logprobs_bwd: bad size");
  if (rnnt_type < 0 || rnnt_type > 2 || term < 0 || term >= C)
    return fail(FRNNT_EINVAL, "lattice_logprobs_bwd: bad rnnt_type or termination symbol");
  if (B == 0 || T == 0) return FRNNT_OK;
  if (!logits || (!symbols && S > 0) || !norm || !px_grad || !py_grad || !logits_grad)
    return fail(FRNNT_EINVAL, "lattice_logprobs_bwd: null pointer");
  const long rows = (long)B * T * Rr;
  const int64_t *window = window_only ? boundary : nullptr;
  if (!launch_row_grad_regs<R>(logits, symbols, ranges, boundary, window, norm, px_grad, py_grad,
                               logits_grad, rows, S, T, Rr, C, term, rnnt_type,
                               static_cast<hipStream_t>(stream_)))
    hipLaunchKernelGGL(row_grad_kernel<R>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                       static_cast<hipStream_t>(stream_), logits, symbols, ranges, boundary, window,
                       norm, px_grad, py_grad, logits_grad, rows, S, T, Rr, C, term, rnnt_type);
  return check_launch("lattice_logprobs_bwd");
}

}  // namespace
}  // namespace frnnt

extern "C" {

int frnnt_lattice_logprobs_fwd_f32(const float *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary, float *px,
                                   float *py, float *norm, float *xr, float *yr, int B, int S,
                                   int T, int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream) {
  return frnnt::fwd_impl<float>(logits, symbols, ranges, boundary, px, py, norm, xr, yr, B, S, T, R,
                                C, termination_symbol, rnnt_type, window_only, stream);
}
int frnnt_lattice_logprobs_fwd_f64(const double *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary, double *px,
                                   double *py, double *norm, double *xr, double *yr, int B, int S,
                                   int T, int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream) {
  return frnnt::fwd_impl<double>(logits, symbols, ranges, boundary, px, py, norm, xr, yr, B, S, T,
                                 R, C, termination_symbol, rnnt_type, window_only, stream);
}
int frnnt_lattice_logprobs_bwd_f32(const float *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary,
                                   const float *norm, const float *px_grad, const float *py_grad,
                                   float *logits_grad, int B, int S, int T, int R, int C,
                                   int termination_symbol, int rnnt_type, int window_only,
                                   void *stream) {
  return frnnt::bwd_impl<float>(logits, symbols, ranges, boundary, norm, px_grad, py_grad,
                                logits_grad, B, S, T, R, C, termination_symbol, rnnt_type,
                                window_only, stream);
}
int frnnt_lattice_logprobs_bwd_f64(const double *logits, const int64_t *symbols,
                                   const int64_t *ranges, const int64_t *boundary,
                                   const double *norm, const double *px_grad,
                                   const double *py_grad, double *logits_grad, int B, int S, int T,
                                   int R, int C, int termination_symbol, int rnnt_type,
                                   int window_only, void *stream) {
  return frnnt::bwd_impl<double>(logits, symbols, ranges, boundary, norm, px_grad, py_grad,
                                 logits_grad, B, S, T, R, C, termination_symbol, rnnt_type,
                                 window_only, stream);
}


#define FRNNT_NARROW_ENTRY(sfx, IO)                                                              \
  int frnnt_lattice_logprobs_fwd_##sfx(                                                          \
      const void *logits, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary, \
      float *px, float *py, float *norm, float *xr, float *yr, int B, int S, int T, int R, int C, \
      int termination_symbol, int rnnt_type, int window_only, void *stream) {                    \
    return frnnt::narrow_fwd_impl<frnnt::IO>(logits, symbols, ranges, boundary, px, py, norm, xr, \
                                             yr, B, S, T, R, C, termination_symbol, rnnt_type,    \
                                             window_only, stream);                                \
  }                                                                                              \
  int frnnt_lattice_logprobs_bwd_##sfx(                                                          \
      const void *logits, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary, \
      const float *norm, const float *px_grad, const float *py_grad, void *logits_grad, int B,    \
      int S, int T, int R, int C, int termination_symbol, int rnnt_type, int window_only,         \
      void *stream) {                                                                            \
    return frnnt::narrow_bwd_impl<frnnt::IO>(logits, symbols, ranges, boundary, norm, px_grad,    \
                                             py_grad, logits_grad, B, S, T, R, C,                 \
                                             termination_symbol, rnnt_type, window_only, stream); \
  }
FRNNT_NARROW_ENTRY(f16, HalfIO)
FRNNT_NARROW_ENTRY(bf16, Bf16IO)
#undef FRNNT_NARROW_ENTRY

}  // extern "C"
