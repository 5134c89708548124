// Register-direct batched fp32 GEMM pieces for the matrix cores (gfx950).
//
// Each wave keeps a 32 x 64 output tile in two v_mfma_f32_32x32x2_f32
// accumulators.  With a long K the waves of a workgroup split the K range of ONE
// tile between them (wave w takes k-blocks w, w+W, ...) and the partial sums
// meet in LDS once, at the end; with a short K every wave owns its own tile.
// In the main loop nothing goes through LDS and there is no barrier: every lane
// fetches its own MFMA operands straight
// from global memory into registers, applies exp(x - max) there, and feeds the
// matrix core.  That works because the order in which k is summed is free: in
// MFMA instruction i of a 32-wide k-block, lanes 0-31 supply k = 16*0 + i and
// lanes 32-63 supply k = 16*1 + i (for both operands), so
//   - a k-contiguous operand (row-major [rows][K]) is 16 consecutive floats per
//     lane: four 16-byte loads;
//   - a row-contiguous operand (row-major [K][rows]) is one float per lane and
//     instruction, 32 consecutive floats per half-wave: fully coalesced.
// Loads for the next k-block are issued before the current one is consumed.
#pragma once

#include "common.hip.h"

namespace frnnt {
namespace dgemm {

constexpr int kBM = 32;   // output rows per workgroup
constexpr int kBN = 64;   // output columns per workgroup (two 32-wide MFMA tiles)
constexpr int kBK = 32;   // k-block: 16 MFMA instructions of depth 2
constexpr int kXcds = 8;  // workgroup i is dispatched to XCD i % 8; each XCD has its own L2

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct Frag {
  float v[16];
};

// Operand fetches address memory as (uniform base pointer) + (32-bit element
// offset), which lets the compiler use the scalar-base addressing form and keep
// one VGPR per address instead of two; a per-utterance operand has far fewer than
// 2^31 elements.

// 16 consecutive k of the row that starts at element offset `row_off` of a
// k-contiguous matrix; `ok` false (row out of range) gives `fill` everywhere.
template <bool kVec>
__device__ __forceinline__ void load_kfast(Frag &f, const float *base, int row_off, bool ok,
                                           int k0, int K, float fill) {
  if (kVec && ok && k0 + 16 <= K) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const floatx4 t = *reinterpret_cast<const floatx4 *>(base + (row_off + k0 + 4 * q));
      f.v[4 * q + 0] = t[0];
      f.v[4 * q + 1] = t[1];
      f.v[4 * q + 2] = t[2];
      f.v[4 * q + 3] = t[3];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) f.v[i] = (ok && k0 + i < K) ? base[row_off + k0 + i] : fill;
  }
}

// element `col` of 16 consecutive rows k0.. of a row-major [K][ld] matrix; `ok`
// false (column out of range) gives `fill` everywhere.
__device__ __forceinline__ void load_rowfast(Frag &f, const float *base, int ld, int col, bool ok,
                                             int k0, int K, float fill) {
#pragma unroll
  for (int i = 0; i < 16; ++i) f.v[i] = (ok && k0 + i < K) ? base[(k0 + i) * ld + col] : fill;
}

__device__ __forceinline__ void exp_shift_each(Frag &f, const Frag &shift) {
#pragma unroll
  for (int i = 0; i < 16; ++i) f.v[i] = __expf(f.v[i] - shift.v[i]);
}

struct Acc {
  floatx16 c[2];
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int v = 0; v < 16; ++v) c[t][v] = 0.f;
  }
  __device__ __forceinline__ void mma(const Frag &a, const Frag &b0, const Frag &b1) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      c[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b0.v[i], c[0], 0, 0, 0);
      c[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b1.v[i], c[1], 0, 0, 0);
    }
  }
};

// Epilogues run in two passes: `pre(row, col)` fetches whatever the element needs
// from global memory (all fetches of a thread are issued back to back), then
// `post(row, col, sum, fetched)` computes and stores.  A single pass would
// serialise one memory round trip per element, because a store may alias the next
// element's load and therefore pins it in program order.

// Sums the partial tiles of kW waves through LDS (kW x 32 x 64 floats);
// consecutive threads walk consecutive columns.
template <int kW, typename Pre, typename Post>
__device__ __forceinline__ void reduce_and_emit(const Acc &acc, float *lds, Pre pre, Post post) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  float *mine = lds + wave * (kBM * kBN);
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v)
      mine[(8 * (v / 4) + 4 * half + (v % 4)) * kBN + 32 * t + col] = acc.c[t][v];
  constexpr int kPer = kBM * kBN / (kW * kWave);
  float fetched[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int e = j * (kW * kWave) + tid;
    fetched[j] = pre(e / kBN, e % kBN);
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int e = j * (kW * kWave) + tid;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kW; ++w) sum += lds[w * kBM * kBN + e];
    post(e / kBN, e % kBN, sum, fetched[j]);
  }
}

// XCD-aware decode of a 1-D grid: all tiles of batch element b run on XCD b % 8,
// so one XCD's L2 holds the operands of only B/8 utterances.  The grid must have
// kXcds * ceil(B / kXcds) * tiles workgroups; returns false for padding ones.
__device__ __forceinline__ bool decode_block(int tiles, int B, int &b, int &tile) {
  const int id = blockIdx.x;
  const int xcd = id % kXcds, slot = id / kXcds;
  b = xcd + kXcds * (slot / tiles);
  tile = slot % tiles;
  return b < B;
}
inline unsigned xcd_grid(int tiles, int B) {
  return (unsigned)(kXcds * ((B + kXcds - 1) / kXcds) * tiles);
}

}  // namespace dgemm
}  // namespace frnnt
