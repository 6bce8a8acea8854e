// The CEMA operators on float64 tensors: kernel generation, its backward sums and
// the causal convolution.
//
// The reference instantiates these operators for double as well
// (megalodon/csrc/ops/ema_parameters_kernel.cu:1227: p float64, log_q / gamma
// complex128; fftconv_kernel.cu:468-476,487-499: x float64 with complex128
// spectra); nothing in the model runs them.  These are the double-precision
// flavours: the defining sums evaluated directly in double on the vector ALUs --
// every power q^j from its own exp / sincos, the convolution as the triangular sum
// it is (exact up to rounding, no transform) -- for checking results, not for
// speed.
#include "common.hpp"

namespace mega {
namespace {

struct cd {
  double x, y;
};
__device__ __forceinline__ cd cmul(cd a, cd b) { return cd{a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x}; }
// exp(j * lq)
__device__ __forceinline__ cd qpow(cd lq, double j) {
  double s, c;
  sincos(j * lq.y, &s, &c);
  const double m = exp(j * lq.x);
  return cd{m * c, m * s};
}

constexpr int kThreads = 256;

// w[r, j] = sum_n Re(p[r, n] gamma[r, n] q[r, n]^j)   (ema_parameters.cc:17-52)
__global__ __launch_bounds__(kThreads) void ema_weight_fwd_f64_kernel(const double* __restrict__ p,
                                                                      const cd* __restrict__ log_q,
                                                                      const cd* __restrict__ gamma, int N, int64_t L,
                                                                      double* __restrict__ w) {
  const int64_t r = blockIdx.y;
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j >= L) return;
  double acc = 0.0;
  for (int n = 0; n < N; ++n) {
    const double pv = p[r * N + n];
    const cd g = gamma[r * N + n];
    const cd z = qpow(log_q[r * N + n], static_cast<double>(j));
    acc += pv * (g.x * z.x - g.y * z.y);
  }
  w[r * L + j] = acc;
}

// S2 = sum_j dw[j] q^j, S1 = sum_j j dw[j] q^(j-1); dp = Re(S2 gamma), dq = conj(S1 p gamma),
// dgamma = conj(S2 p)   (ema_parameters.cc:80-98,141-156).  One workgroup per (row, mode).
__global__ __launch_bounds__(kThreads) void ema_weight_bwd_f64_kernel(const double* __restrict__ dw,
                                                                      const double* __restrict__ p,
                                                                      const cd* __restrict__ log_q,
                                                                      const cd* __restrict__ gamma, int N, int64_t L,
                                                                      double* __restrict__ dp, cd* __restrict__ dq,
                                                                      cd* __restrict__ dgamma) {
  __shared__ double red[4][kThreads];
  const int64_t r = blockIdx.y;
  const int n = blockIdx.x, tid = threadIdx.x;
  const cd lq = log_q[r * N + n];
  cd s1{0.0, 0.0}, s2{0.0, 0.0};
  for (int64_t j = tid; j < L; j += kThreads) {
    const double d = dw[r * L + j];
    const cd z = qpow(lq, static_cast<double>(j));
    s2.x = fma(d, z.x, s2.x);
    s2.y = fma(d, z.y, s2.y);
    if (j > 0) {
      const cd z1 = qpow(lq, static_cast<double>(j - 1));
      const double dj = d * static_cast<double>(j);
      s1.x = fma(dj, z1.x, s1.x);
      s1.y = fma(dj, z1.y, s1.y);
    }
  }
  red[0][tid] = s1.x;
  red[1][tid] = s1.y;
  red[2][tid] = s2.x;
  red[3][tid] = s2.y;
  __syncthreads();
  for (int half = kThreads / 2; half > 0; half >>= 1) {
    if (tid < half)
      for (int c = 0; c < 4; ++c) red[c][tid] += red[c][tid + half];
    __syncthreads();
  }
  if (tid == 0) {
    const cd S1{red[0][0], red[1][0]}, S2{red[2][0], red[3][0]};
    const double pv = p[r * N + n];
    const cd g = gamma[r * N + n];
    dp[r * N + n] = S2.x * g.x - S2.y * g.y;
    const cd t = cmul(S1, g);
    dq[r * N + n] = cd{pv * t.x, -pv * t.y};
    dgamma[r * N + n] = cd{pv * S2.x, -pv * S2.y};
  }
}

// out[r, t] = sum_{s <= t} a[r % rows_a, s] b[r, t - s]: the causal convolution
// (fused_ops/fftconv.py:30-50 computes the same sum through rfft / irfft).  A workgroup owns
// 256 outputs of a row; a and the window of b that meets it pass through LDS 256 lags at a time.
__global__ __launch_bounds__(kThreads) void causal_conv_f64_kernel(const double* __restrict__ a,
                                                                   const double* __restrict__ b, int64_t rows_a,
                                                                   int64_t L, double* __restrict__ out) {
  __shared__ double sa[kThreads], sb[2 * kThreads];
  const int64_t r = blockIdx.y;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kThreads;
  const int tid = threadIdx.x;
  const double* ar = a + (r % rows_a) * L;
  const double* br = b + r * L;
  const int64_t t = t0 + tid;
  double acc = 0.0;
  // lags s0 .. s0 + 255 meet b[t - s], t in the tile: indices t0 - s0 - 255 .. t0 - s0 + 255
  for (int64_t s0 = 0; s0 <= t0 + kThreads - 1 && s0 < L; s0 += kThreads) {
    const int64_t base = t0 - s0 - (kThreads - 1);
    sa[tid] = s0 + tid < L ? ar[s0 + tid] : 0.0;
    for (int i = tid; i < 2 * kThreads; i += kThreads) {
      const int64_t idx = base + i;
      sb[i] = (idx >= 0 && idx < L) ? br[idx] : 0.0;
    }
    __syncthreads();
    // b[t - s] with s = s0 + e sits at sb[t - s - base] = sb[tid + 255 - e]
#pragma unroll 8
    for (int e = 0; e < kThreads; ++e) acc = fma(sa[e], sb[tid + (kThreads - 1) - e], acc);
    __syncthreads();
  }
  if (t < L) out[r * L + t] = acc;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_ema_weight_fwd_f64(const double* p, const double* log_q, const double* gamma, int64_t D,
                                       int64_t N, int64_t L, double* w, void* stream) {
  MEGA_CHECK_ARG(D >= 0 && N >= 1 && N <= 32 && L >= 0, "mega_ema_weight_fwd_f64: bad sizes (1 <= N <= 32)");
  MEGA_CHECK_ARG(D <= 65535 * 64ll && L <= (1ll << 31), "mega_ema_weight_fwd_f64: too many rows or steps");
  if (D == 0 || L == 0) return MEGA_OK;
  MEGA_CHECK_ARG(p && log_q && gamma && w, "mega_ema_weight_fwd_f64: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // the row index rides on gridDim.y (at most 65535): rows in slices
  for (int64_t r0 = 0; r0 < D; r0 += 65535) {
    const int64_t rows = D - r0 < 65535 ? D - r0 : 65535;
    ema_weight_fwd_f64_kernel<<<dim3((unsigned)((L + kThreads - 1) / kThreads), (unsigned)rows), kThreads, 0, s>>>(
        p + r0 * N, reinterpret_cast<const cd*>(log_q) + r0 * N, reinterpret_cast<const cd*>(gamma) + r0 * N, (int)N, L,
        w + r0 * L);
    MEGA_CHECK_LAUNCH();
  }
  return MEGA_OK;
}

extern "C" int mega_ema_weight_bwd_f64(const double* dw, const double* p, const double* log_q, const double* gamma,
                                       int64_t D, int64_t N, int64_t L, double* dp, double* dq, double* dgamma,
                                       void* stream) {
  MEGA_CHECK_ARG(D >= 0 && N >= 1 && N <= 32 && L >= 0, "mega_ema_weight_bwd_f64: bad sizes (1 <= N <= 32)");
  if (D == 0) return MEGA_OK;
  MEGA_CHECK_ARG(p && log_q && gamma && dp && dq && dgamma && (dw || L == 0), "mega_ema_weight_bwd_f64: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (int64_t r0 = 0; r0 < D; r0 += 65535) {
    const int64_t rows = D - r0 < 65535 ? D - r0 : 65535;
    ema_weight_bwd_f64_kernel<<<dim3((unsigned)N, (unsigned)rows), kThreads, 0, s>>>(
        dw + r0 * L, p + r0 * N, reinterpret_cast<const cd*>(log_q) + r0 * N,
        reinterpret_cast<const cd*>(gamma) + r0 * N, (int)N, L, dp + r0 * N, reinterpret_cast<cd*>(dq) + r0 * N,
        reinterpret_cast<cd*>(dgamma) + r0 * N);
    MEGA_CHECK_LAUNCH();
  }
  return MEGA_OK;
}

extern "C" int mega_causal_conv_f64(const double* a, const double* b, int64_t rows_a, int64_t rows, int64_t L,
                                    double* out, void* stream) {
  MEGA_CHECK_ARG(rows_a >= 1 && rows >= 0 && L >= 0 && rows % rows_a == 0,
                 "mega_causal_conv_f64: bad sizes (rows must be a multiple of rows_a)");
  MEGA_CHECK_ARG(L <= (1ll << 31), "mega_causal_conv_f64: rows too long");
  if (rows == 0 || L == 0) return MEGA_OK;
  MEGA_CHECK_ARG(a && b && out, "mega_causal_conv_f64: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // slices of 65535 * rows_a-aligned rows keep r % rows_a right
  const int64_t slice = (65535 / rows_a) * rows_a;
  MEGA_CHECK_ARG(slice > 0, "mega_causal_conv_f64: more than 65535 kernel rows");
  for (int64_t r0 = 0; r0 < rows; r0 += slice) {
    const int64_t n = rows - r0 < slice ? rows - r0 : slice;
    causal_conv_f64_kernel<<<dim3((unsigned)((L + kThreads - 1) / kThreads), (unsigned)n), kThreads, 0, s>>>(
        a, b + r0 * L, rows_a, L, out + r0 * L);
    MEGA_CHECK_LAUNCH();
  }
  return MEGA_OK;
}
