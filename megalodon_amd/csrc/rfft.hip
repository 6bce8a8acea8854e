// Real FFT of zero-padded rows: y = rfft(x, n = 2 M), M = max(2^ceil(log2 L), 32).
//
// Replaces rfft(x, flip) (megalodon/csrc/ops/fftconv.cc:6-8,22,
// fftconv_kernel.cu:23-32,170-215): the reference uses it to bring a 16-bit
// convolution kernel into the frequency domain for its fused operator
// (fused_ops/fftconv.py:88-91).  The convolution path of this library takes the
// kernel in the time domain, so nothing here depends on this operator; it is a
// plain one-workgroup-per-row transform for callers that want the spectrum:
// the row is packed z[n] = x[2n] + i x[2n+1], an M-point radix-2 FFT runs in
// LDS in float32 (twiddles from sincospi), and the even / odd parts are
// recombined into the M + 1 bins of the 2 M-point real transform.
#include "common.hpp"

namespace mega {
namespace {

constexpr int kThreads = 1024;

__device__ __forceinline__ float2 cmulf(float2 a, float2 b) {
  return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x);
}

template <int DT>
__global__ __launch_bounds__(kThreads) void rfft_kernel(const typename Elem<DT>::type* x, float2* y,
                                                        int L, int logm, int flip) {
  extern __shared__ float2 z[];
  const int M = 1 << logm, tid = threadIdx.x;
  const typename Elem<DT>::type* xr = x + static_cast<int64_t>(blockIdx.x) * L;
  float2* yr = y + static_cast<int64_t>(blockIdx.x) * (M + 1);
  // packed, zero-padded, stored in bit-reversed order for the in-place passes
  for (int n = tid; n < M; n += kThreads) {
    const int i0 = 2 * n, i1 = 2 * n + 1;
    const float a = i0 < L ? Elem<DT>::load(xr + (flip ? L - 1 - i0 : i0)) : 0.f;
    const float b = i1 < L ? Elem<DT>::load(xr + (flip ? L - 1 - i1 : i1)) : 0.f;
    z[__brev(static_cast<unsigned>(n)) >> (32 - logm)] = make_float2(a, b);
  }
  __syncthreads();
  for (int s = 1; s <= logm; ++s) {
    const int half = 1 << (s - 1);
    for (int j = tid; j < M / 2; j += kThreads) {
      const int pos = j & (half - 1), i = ((j >> (s - 1)) << s) + pos, k = i + half;
      float sn, cs;
      sincospif(-static_cast<float>(pos) / static_cast<float>(half), &sn, &cs);  // exp(-2 pi i pos / 2^s)
      const float2 u = z[i], t = cmulf(z[k], make_float2(cs, sn));
      z[i] = make_float2(u.x + t.x, u.y + t.y);
      z[k] = make_float2(u.x - t.x, u.y - t.y);
    }
    __syncthreads();
  }
  // X[k] = E[k] + exp(-i pi k / M) O[k], E = (Z[k] + conj Z[M-k]) / 2, O = (Z[k] - conj Z[M-k]) / (2 i)
  for (int k = tid; k <= M; k += kThreads) {
    const float2 a = z[k & (M - 1)], b = z[(M - k) & (M - 1)];
    const float2 e = make_float2(0.5f * (a.x + b.x), 0.5f * (a.y - b.y));
    const float2 o = make_float2(0.5f * (a.y + b.y), -0.5f * (a.x - b.x));
    float sn, cs;
    sincospif(-static_cast<float>(k) / static_cast<float>(M), &sn, &cs);
    const float2 t = cmulf(o, make_float2(cs, sn));
    yr[k] = make_float2(e.x + t.x, e.y + t.y);
  }
}

template <int DT>
int launch_rfft(const void* x, float2* y, int64_t rows, int L, int logm, int flip, hipStream_t s) {
  const size_t lds = sizeof(float2) << logm;
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&rfft_kernel<DT>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
  rfft_kernel<DT><<<static_cast<unsigned>(rows), kThreads, lds, s>>>(
      static_cast<const typename Elem<DT>::type*>(x), y, L, logm, flip);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int64_t mega_rfft_bins(int64_t L) {
  if (L < 1) return 0;
  int64_t m = 32;
  while (m < L) m <<= 1;
  return m + 1;
}

extern "C" int mega_rfft(const void* x, int dtype, int64_t rows, int64_t L, int flip, void* y, void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_rfft: unknown dtype %d", dtype);
  MEGA_CHECK_ARG(rows >= 0 && L >= 1, "mega_rfft: bad sizes");
  if (L > 16384)
    return set_error(MEGA_ERR_UNSUPPORTED, "mega_rfft: rows longer than 16384 samples are not supported");
  MEGA_CHECK_ARG(rows < (1ll << 31), "mega_rfft: too many rows");
  if (rows == 0) return MEGA_OK;
  MEGA_CHECK_ARG(x && y, "mega_rfft: null pointer");
  int logm = 5;
  while ((1ll << logm) < L) ++logm;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float2* out = static_cast<float2*>(y);
  if (dtype == MEGA_F32) return launch_rfft<MEGA_F32>(x, out, rows, (int)L, logm, flip, s);
  if (dtype == MEGA_BF16) return launch_rfft<MEGA_BF16>(x, out, rows, (int)L, logm, flip, s);
  return launch_rfft<MEGA_F16>(x, out, rows, (int)L, logm, flip, s);
}
