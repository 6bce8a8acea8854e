// Powers of the CEMA decay factors, shared by the kernel-generation and the
// chunked-recurrence kernels.
#pragma once

#include "common.hpp"

namespace mega {

// q^j for log q = (a, phi), evaluated directly.
__device__ __forceinline__ cf qpow(float a, float phi, int64_t j) {
  if (j == 0) return {1.0f, 0.0f};
  const double jj = static_cast<double>(j);
  const double turns = static_cast<double>(phi) * 0.15915494309189535 * jj;
  const double fr = turns - rint(turns);  // in [-0.5, 0.5]
  float s, c;
  sincospif(2.0f * static_cast<float>(fr), &s, &c);
  // |q|^j = 2^t, t = a j log2(e): the integer part of t goes into the exponent
  // exactly, the fraction (|f| <= 0.5, rounded to float: 3e-8) through exp2f
  const double t = fmax(static_cast<double>(a) * jj * 1.4426950408889634, -1000.0);
  const double ti = rint(t);
  const float mag = ldexpf(exp2f(static_cast<float>(t - ti)), static_cast<int>(ti));
  return {mag * c, mag * s};
}

}  // namespace mega
