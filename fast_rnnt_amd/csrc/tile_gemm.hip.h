// LDS-tiled batched GEMM building blocks on the CDNA matrix cores.
//
// A workgroup of 256 threads (4 waves, 2 x 2) produces a 64 x 64 output tile;
// each wave owns a 32 x 32 quadrant held in MFMA accumulators
// (v_mfma_f32_32x32x2_f32 for float, 2 x 2 v_mfma_f64_16x16x4_f64 for double).
// Operand tiles are staged in LDS as [k][row] with an odd row pitch so that both
// the transposing stores of the loaders and the per-lane operand reads are free
// of bank conflicts.  Loaders apply an optional exp(x - rowmax) while the tile
// is in registers, so the exponentiated operands never exist in HBM.
#pragma once

#include "common.hip.h"

namespace frnnt {

constexpr int kTileM = 64;
constexpr int kTileN = 64;
constexpr int kGemmThreads = 256;
constexpr int kPitch = kTileM + 1;  // floats/doubles per LDS k-row

template <typename R>
struct TileK;
template <>
struct TileK<float> {
  static constexpr int value = 32;
};
template <>
struct TileK<double> {
  static constexpr int value = 16;
};

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef double doublex4 __attribute__((ext_vector_type(4)));

template <typename R>
__device__ __forceinline__ R fast_exp(R x);
template <>
__device__ __forceinline__ float fast_exp<float>(float x) {
  return __expf(x);
}
template <>
__device__ __forceinline__ double fast_exp<double>(double x) {
  return exp(x);
}

// ---- accumulators ------------------------------------------------------------
// acc.step(As, Bs) consumes one staged k-tile; acc.for_each(f) visits every
// element of the wave's 32 x 32 quadrant as f(row_in_tile, col_in_tile, value),
// consecutive lanes walking consecutive columns.
template <typename R>
struct WaveAcc;

template <>
struct WaveAcc<float> {
  floatx16 c;
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int v = 0; v < 16; ++v) c[v] = 0.f;
  }
  __device__ __forceinline__ void step(const float *As, const float *Bs, int m0, int n0,
                                       int lane) {
    const int half = lane >> 5, col = lane & 31;
#pragma unroll
    for (int kk = 0; kk < TileK<float>::value; kk += 2) {
      const float a = As[(kk + half) * kPitch + m0 + col];
      const float b = Bs[(kk + half) * kPitch + n0 + col];
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
  }
  template <typename F>
  __device__ __forceinline__ void for_each(int m0, int n0, int lane, F f) const {
    const int half = lane >> 5, col = lane & 31;
#pragma unroll
    for (int v = 0; v < 16; ++v) f(m0 + 8 * (v / 4) + 4 * half + (v % 4), n0 + col, c[v]);
  }
};

template <>
struct WaveAcc<double> {
  doublex4 c[2][2];
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v) c[a][b][v] = 0.0;
  }
  __device__ __forceinline__ void step(const double *As, const double *Bs, int m0, int n0,
                                       int lane) {
    const int quad = lane >> 4, col = lane & 15;
#pragma unroll
    for (int kk = 0; kk < TileK<double>::value; kk += 4) {
      double a[2], b[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        a[h] = As[(kk + quad) * kPitch + m0 + 16 * h + col];
        b[h] = Bs[(kk + quad) * kPitch + n0 + 16 * h + col];
      }
#pragma unroll
      for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int y = 0; y < 2; ++y)
          c[x][y] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[x], b[y], c[x][y], 0, 0, 0);
    }
  }
  template <typename F>
  __device__ __forceinline__ void for_each(int m0, int n0, int lane, F f) const {
    const int quad = lane >> 4, col = lane & 15;
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
      for (int y = 0; y < 2; ++y)
#pragma unroll
        for (int v = 0; v < 4; ++v) f(m0 + 16 * x + 4 * v + quad, n0 + 16 * y + col, c[x][y][v]);
  }
};

// ---- operand loaders -------------------------------------------------------------
// Each loader moves one [64 rows] x [TileK] operand tile: fetch() pulls it from
// global memory into registers (issued early), stash() transforms and writes it
// to the LDS tile laid out [k][row].

// Source is row-major [rows][K] (k fastest): e.g. lm / am in the forward GEMM.
template <typename R, bool kExp>
struct LoaderKFast {
  static constexpr int BK = TileK<R>::value;
  static constexpr int kPerThread = kTileM * BK / kGemmThreads;  // 8 (float) / 4 (double)
  R reg[kPerThread];
  // thread -> (row, k) pairs: k index fastest across threads so that a row's
  // BK values are fetched by neighbouring lanes
  __device__ __forceinline__ void fetch(const R *src, long ld, int row0, int nrows, int k0, int K,
                                        int tid) {
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
      const int e = q * kGemmThreads + tid;
      const int row = e / BK, k = e % BK;
      const bool ok = (row0 + row < nrows) && (k0 + k < K);
      reg[q] = ok ? src[(long)(row0 + row) * ld + k0 + k] : (R)0;
    }
  }
  __device__ __forceinline__ void stash(R *tile, const R *rowmax, int row0, int nrows, int k0,
                                        int K, int tid) const {
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
      const int e = q * kGemmThreads + tid;
      const int row = e / BK, k = e % BK;
      R v = reg[q];
      if (kExp) {
        const bool ok = (row0 + row < nrows) && (k0 + k < K);
        v = ok ? fast_exp<R>(v - rowmax[row0 + row]) : (R)0;
      }
      tile[k * kPitch + row] = v;
    }
  }
};

// Source is row-major [K][rows] (row index fastest): e.g. am as the B operand of
// the lm-gradient GEMM, where k runs over frames; rowmax is indexed by k.
template <typename R, bool kExp>
struct LoaderRowFast {
  static constexpr int BK = TileK<R>::value;
  static constexpr int kPerThread = kTileM * BK / kGemmThreads;
  R reg[kPerThread];
  __device__ __forceinline__ void fetch(const R *src, long ld, int row0, int nrows, int k0, int K,
                                        int tid) {
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
      const int e = q * kGemmThreads + tid;
      const int k = e / kTileM, row = e % kTileM;
      const bool ok = (row0 + row < nrows) && (k0 + k < K);
      reg[q] = ok ? src[(long)(k0 + k) * ld + row0 + row] : (R)0;
    }
  }
  __device__ __forceinline__ void stash(R *tile, const R *kmax, int row0, int nrows, int k0, int K,
                                        int tid) const {
#pragma unroll
    for (int q = 0; q < kPerThread; ++q) {
      const int e = q * kGemmThreads + tid;
      const int k = e / kTileM, row = e % kTileM;
      R v = reg[q];
      if (kExp) {
        const bool ok = (row0 + row < nrows) && (k0 + k < K);
        v = ok ? fast_exp<R>(v - kmax[k0 + k]) : (R)0;
      }
      tile[k * kPitch + row] = v;
    }
  }
};

// One 64 x 64 output tile: C = A * B over K, double-buffered through LDS.
// LA / LB are loader types; a_* / b_* describe the operands; returns the wave's
// accumulators.  `lds` must hold 4 * TileK * kPitch elements.
template <typename R, typename LA, typename LB>
__device__ __forceinline__ void tile_matmul(WaveAcc<R> &acc, R *lds, const R *a_src, long a_ld,
                                            const R *a_max, int m_tile0, int M, const R *b_src,
                                            long b_ld, const R *b_max, int n_tile0, int N, int K) {
  constexpr int BK = TileK<R>::value;
  R *As[2] = {lds, lds + BK * kPitch};
  R *Bs[2] = {lds + 2 * BK * kPitch, lds + 3 * BK * kPitch};
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = (wave >> 1) * 32, n0 = (wave & 1) * 32;
  LA la;
  LB lb;
  acc.clear();
  la.fetch(a_src, a_ld, m_tile0, M, 0, K, tid);
  lb.fetch(b_src, b_ld, n_tile0, N, 0, K, tid);
  la.stash(As[0], a_max, m_tile0, M, 0, K, tid);
  lb.stash(Bs[0], b_max, n_tile0, N, 0, K, tid);
  __syncthreads();
  const int nk = (K + BK - 1) / BK;
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      la.fetch(a_src, a_ld, m_tile0, M, (kt + 1) * BK, K, tid);
      lb.fetch(b_src, b_ld, n_tile0, N, (kt + 1) * BK, K, tid);
    }
    acc.step(As[cur], Bs[cur], m0, n0, lane);
    if (more) {
      la.stash(As[cur ^ 1], a_max, m_tile0, M, (kt + 1) * BK, K, tid);
      lb.stash(Bs[cur ^ 1], b_max, n_tile0, N, (kt + 1) * BK, K, tid);
    }
    __syncthreads();
  }
}

}  // namespace frnnt
