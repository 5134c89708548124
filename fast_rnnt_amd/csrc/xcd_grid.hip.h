// Vector types of the fp32 MFMA kernels and the XCD count of gfx950: workgroup i of a 1-D
// grid is dispatched to XCD i % 8 and every XCD has its own L2, so the kernels give all
// tiles of one utterance (or of one part of it) ids that land on one XCD (place_block and
// place_frames in simple_logprobs.hip).
#pragma once

#include "common.hip.h"

namespace frnnt {
namespace dgemm {

constexpr int kXcds = 8;

typedef float floatx16 __attribute__((ext_vector_type(16)));  // a 32 x 32 MFMA accumulator
typedef float floatx4 __attribute__((ext_vector_type(4)));

}  // namespace dgemm
}  // namespace frnnt
