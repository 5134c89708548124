// Vector types of the fp32 MFMA kernels and the XCD-aware mapping of a 1-D grid onto
// (utterance, tile) for gfx950: workgroup i is dispatched to XCD i % 8 and every XCD
// has its own L2, so all tiles of one utterance are given ids that land on one XCD.
#pragma once

#include "common.hip.h"

namespace frnnt {
namespace dgemm {

constexpr int kXcds = 8;

typedef float floatx16 __attribute__((ext_vector_type(16)));  // a 32 x 32 MFMA accumulator
typedef float floatx4 __attribute__((ext_vector_type(4)));

// All tiles of batch element b run on XCD b % 8, so one XCD's L2 holds the operands
// of only B/8 utterances.  The grid must have kXcds * ceil(B / kXcds) * tiles
// workgroups; returns false for the padding ones.
__device__ __forceinline__ bool decode_block(int id, int tiles, int B, int &b, int &tile) {
  const int xcd = id % kXcds, slot = id / kXcds;
  b = xcd + kXcds * (slot / tiles);
  tile = slot % tiles;
  return b < B;
}
__device__ __forceinline__ bool decode_block(int tiles, int B, int &b, int &tile) {
  return decode_block((int)blockIdx.x, tiles, B, b, tile);
}
inline unsigned xcd_grid(int tiles, int B) {
  return (unsigned)(kXcds * ((B + kXcds - 1) / kXcds) * tiles);
}

}  // namespace dgemm
}  // namespace frnnt
