// Dropout whose mask is a pure function of (seed, offset, element index).
//
// Replaces megalodon/modules/fused_ops/memory_efficient_dropout.py:39-96: the
// reference saves the generator state in the forward and replays the generator
// in the backward to rebuild the same Bernoulli noise without keeping it.  Here
// the mask needs no generator: element e is kept iff word e % 4 of
// Philox4x32-10 with counter (e / 4, offset) and key seed, taken as
// u = (word >> 8) * 2^-24, satisfies u >= p.  Forward and backward are the same
// launch (on x and on dy): out = keep ? in / (1 - p) : 0.
#include "common.hpp"

namespace mega {
namespace {

constexpr int kThreads = 256;

struct DropState {
  float p, inv_keep;
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
};

__device__ __forceinline__ void keep_quad(const DropState& st, uint64_t quad, float* scale) {
  uint32_t w[4];
  philox4x32_10(static_cast<uint32_t>(quad), static_cast<uint32_t>(quad >> 32), st.off_lo, st.off_hi,
                st.seed_lo, st.seed_hi, w);
#pragma unroll
  for (int e = 0; e < 4; ++e)
    scale[e] = static_cast<float>(w[e] >> 8) * 0x1p-24f < st.p ? 0.f : st.inv_keep;
}

// 8 elements per lane and step; n8 = number of whole groups of 8.  16-bit types
// move 16 bytes per lane, float 32.
template <int DT>
__global__ __launch_bounds__(kThreads) void dropout_vec_kernel(const typename Elem<DT>::type* in,
                                                              typename Elem<DT>::type* out,
                                                              int64_t n8, DropState st) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; g < n8; g += stride) {
    float sc[8];
    keep_quad(st, static_cast<uint64_t>(g) * 2, sc);
    keep_quad(st, static_cast<uint64_t>(g) * 2 + 1, sc + 4);
    if (DT == MEGA_F32) {
      const float4* src = reinterpret_cast<const float4*>(in) + g * 2;
      float4* dst = reinterpret_cast<float4*>(out) + g * 2;
      const float4 a = src[0], b = src[1];
      float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      // a dropped element is 0 whatever it held (0 * inf would be NaN)
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = sc[e] == 0.f ? 0.f : v[e] * sc[e];
      dst[0] = make_float4(v[0], v[1], v[2], v[3]);
      dst[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
      float v[8];
      unpack8<DT>(reinterpret_cast<const uint4*>(in)[g], v);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = sc[e] == 0.f ? 0.f : v[e] * sc[e];
      reinterpret_cast<uint4*>(out)[g] = pack8<DT>(v);
    }
  }
}

// elements [first, n) one by one (tails and unaligned tensors)
template <int DT>
__global__ __launch_bounds__(kThreads) void dropout_scalar_kernel(const typename Elem<DT>::type* in,
                                                                 typename Elem<DT>::type* out,
                                                                 int64_t first, int64_t n, DropState st) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  for (int64_t e = first + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; e < n; e += stride) {
    float sc[4];
    keep_quad(st, static_cast<uint64_t>(e) >> 2, sc);
    const float s = sc[e & 3];
    Elem<DT>::store(out + e, s == 0.f ? 0.f : Elem<DT>::load(in + e) * s);
  }
}

template <int DT>
int launch_dropout(const void* in, void* out, int64_t n, const DropState& st, hipStream_t s) {
  using T = typename Elem<DT>::type;
  const T* src = static_cast<const T*>(in);
  T* dst = static_cast<T*>(out);
  const int align = DT == MEGA_F32 ? 32 : 16;
  const bool vec = reinterpret_cast<uintptr_t>(in) % align == 0 && reinterpret_cast<uintptr_t>(out) % align == 0;
  const int64_t n8 = vec ? n / 8 : 0;
  if (n8 > 0) {
    const int64_t blocks = (n8 + kThreads - 1) / kThreads;
    dropout_vec_kernel<DT><<<static_cast<unsigned>(blocks < 65536 ? blocks : 65536), kThreads, 0, s>>>(src, dst, n8, st);
    MEGA_CHECK_LAUNCH();
  }
  const int64_t rest = n - n8 * 8;
  if (rest > 0) {
    const int64_t blocks = (rest + kThreads - 1) / kThreads;
    dropout_scalar_kernel<DT><<<static_cast<unsigned>(blocks < 65536 ? blocks : 65536), kThreads, 0, s>>>(
        src, dst, n8 * 8, n, st);
    MEGA_CHECK_LAUNCH();
  }
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_dropout(const void* in, int dtype, int64_t n, double p, uint64_t seed,
                            uint64_t offset, void* out, void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_dropout: unknown dtype %d", dtype);
  MEGA_CHECK_ARG(n >= 0, "mega_dropout: negative size");
  MEGA_CHECK_ARG(p >= 0.0 && p <= 1.0, "mega_dropout: dropout probability has to be between 0 and 1");
  if (n == 0) return MEGA_OK;
  MEGA_CHECK_ARG(in && out, "mega_dropout: null pointer");
  DropState st;
  st.p = static_cast<float>(p);
  st.inv_keep = p < 1.0 ? static_cast<float>(1.0 / (1.0 - p)) : 0.f;
  st.seed_lo = static_cast<uint32_t>(seed);
  st.seed_hi = static_cast<uint32_t>(seed >> 32);
  st.off_lo = static_cast<uint32_t>(offset);
  st.off_hi = static_cast<uint32_t>(offset >> 32);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32) return launch_dropout<MEGA_F32>(in, out, n, st, s);
  if (dtype == MEGA_BF16) return launch_dropout<MEGA_BF16>(in, out, n, st, s);
  return launch_dropout<MEGA_F16>(in, out, n, st, s);
}
