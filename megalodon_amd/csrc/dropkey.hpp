// DropKey mask shared by the attention softmax kernels of every element type.
#pragma once

#include "common.hpp"

namespace mega {

// ---- DropKey (softmax.cuh:135-196) ----------------------------------------------
// With probability `p` a key is taken out of a row (its score becomes -inf)
// before the softmax; the survivors are not rescaled, and the backward needs no
// mask because a dropped key has probability 0.  The reference draws from
// curand's Philox stream of the thread that holds the element; here the draw of
// element (row i, column j) is a pure function of its position, so it does not
// depend on the kernel flavour or the element type: Philox4x32-10 with counter
// (j / 4, i, offset_lo, offset_hi) and key (seed_lo, seed_hi) gives four words,
// element j takes word j % 4, u = (word >> 8) * 2^-24, dropped iff u < p.
// i counts rows over all matrices (i = matrix * L1 + r < 2^32).
struct DropKey {
  float p;
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
};

// drops[e] for the four columns 4 * quad .. 4 * quad + 3 of row i
__device__ __forceinline__ void dropkey_quad(const DropKey& dk, uint32_t i, uint32_t quad, bool* drops) {
  uint32_t w[4];
  philox4x32_10(quad, i, dk.off_lo, dk.off_hi, dk.seed_lo, dk.seed_hi, w);
#pragma unroll
  for (int e = 0; e < 4; ++e) drops[e] = static_cast<float>(w[e] >> 8) * 0x1p-24f < dk.p;
}

}  // namespace mega
