// CEMA coefficients from the raw parameters and their gradients, one launch each.
//
// Follows MultiHeadComplexEMA._calc_coeffs
// (megalodon/modules/complex_exponential_moving_average.py:100-117):
//   a = sigmoid(alpha), d = sigmoid(delta), t = sigmoid(theta)
//   p = a,  q = rho e^(i phi) with rho = 1 - a d, phi = n t 2 pi / N  (n = 1 .. N)
//   gamma_hat = (gamma_0 + i gamma_1) sqrt(1 / N)
// The weight operator wants log q, which is (ln rho, phi): it is written
// directly, no complex logarithm.  In the reference (and in the module's
// general path here) these are ~30 elementwise PyTorch kernels on (D, N)
// tensors per training step, forward and backward, each bound by its launch.
//
// Backward: with (dq_r, dq_i) the gradient of the loss w.r.t. (Re q, Im q)
// (PyTorch's convention for complex gradients), dp real, dgamma_hat complex,
//   drho = dq_r cos phi + dq_i sin phi,     dphi = rho (dq_i cos phi - dq_r sin phi)
//   dalpha = (dp - d drho) a (1 - a),       ddelta = -a drho d (1 - d)
//   dtheta = t (1 - t) (2 pi / N) sum_n n dphi_n
//   dgamma = sqrt(1 / N) (Re dgamma_hat, Im dgamma_hat)
#include "common.hpp"

namespace mega {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float sigmoidf(float v) { return 1.f / (1.f + expf(-v)); }

__global__ __launch_bounds__(kThreads) void cema_coeffs_fwd_kernel(
    const float* __restrict__ alpha, const float* __restrict__ delta,
    const float* __restrict__ theta, const float* __restrict__ gamma, int64_t D, int N,
    float* __restrict__ p, float* __restrict__ log_q, float* __restrict__ gamma_hat) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= D * N) return;
  const int64_t ch = i / N;
  const int n = static_cast<int>(i % N);
  const float a = sigmoidf(alpha[i]), d = sigmoidf(delta[i]), t = sigmoidf(theta[ch]);
  const float scale = sqrtf(1.f / static_cast<float>(N));
  p[i] = a;
  // log |q| = log(1 - a d) without forming 1 - a d: rounded to float32 that difference loses
  // the decay rate's low bits when a d is small (6e-4 of it at a d = 1e-4)
  log_q[2 * i] = log1pf(-a * d);
  log_q[2 * i + 1] = static_cast<float>(n + 1) * (t * (6.283185307179586f / static_cast<float>(N)));
  gamma_hat[2 * i] = gamma[2 * i] * scale;
  gamma_hat[2 * i + 1] = gamma[2 * i + 1] * scale;
}

// one thread per (channel, mode); the sum over the modes of a channel runs
// through LDS (N <= 64, a workgroup holds whole channels)
__global__ __launch_bounds__(kThreads) void cema_coeffs_bwd_kernel(
    const float* __restrict__ dp, const float* __restrict__ dq, const float* __restrict__ dgamma_hat,
    const float* __restrict__ alpha, const float* __restrict__ delta,
    const float* __restrict__ theta, int64_t D, int N, int ch_per_block,
    float* __restrict__ dalpha, float* __restrict__ ddelta, float* __restrict__ dtheta,
    float* __restrict__ dgamma) {
  __shared__ float s_phi[kThreads];
  const int local_ch = threadIdx.x / N, n = threadIdx.x % N;
  const int64_t ch = static_cast<int64_t>(blockIdx.x) * ch_per_block + local_ch;
  const bool on = local_ch < ch_per_block && ch < D;
  float contrib = 0.f;
  if (on) {
    const int64_t i = ch * N + n;
    const float a = sigmoidf(alpha[i]), d = sigmoidf(delta[i]), t = sigmoidf(theta[ch]);
    const float rho = 1.f - a * d;
    const float phi = static_cast<float>(n + 1) * (t * (6.283185307179586f / static_cast<float>(N)));
    float sn, cs;
    sincosf(phi, &sn, &cs);
    const float qr = dq[2 * i], qi = dq[2 * i + 1];
    const float drho = qr * cs + qi * sn;
    const float dphi = rho * (qi * cs - qr * sn);
    dalpha[i] = (dp[i] - d * drho) * a * (1.f - a);
    ddelta[i] = -a * drho * d * (1.f - d);
    const float scale = sqrtf(1.f / static_cast<float>(N));
    dgamma[2 * i] = dgamma_hat[2 * i] * scale;
    dgamma[2 * i + 1] = dgamma_hat[2 * i + 1] * scale;
    contrib = static_cast<float>(n + 1) * dphi;
  }
  s_phi[threadIdx.x] = contrib;
  __syncthreads();
  if (on && n == 0) {
    float s = 0.f;
    for (int k = 0; k < N; ++k) s += s_phi[local_ch * N + k];
    const float t = sigmoidf(theta[ch]);
    dtheta[ch] = t * (1.f - t) * (6.283185307179586f / static_cast<float>(N)) * s;
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_cema_coeffs_fwd(const float* alpha, const float* delta, const float* theta,
                                    const float* gamma, int64_t D, int64_t N, float* p,
                                    float* log_q, float* gamma_hat, void* stream) {
  MEGA_CHECK_ARG(alpha && delta && theta && gamma && p && log_q && gamma_hat,
                 "mega_cema_coeffs_fwd: null pointer");
  MEGA_CHECK_ARG(D >= 0 && N >= 1 && N <= 64, "mega_cema_coeffs_fwd: need D >= 0 and 1 <= N <= 64");
  if (D == 0) return MEGA_OK;
  MEGA_CHECK_ARG(D * N <= (1ll << 40), "mega_cema_coeffs_fwd: too many elements");
  const int64_t blocks = (D * N + kThreads - 1) / kThreads;
  cema_coeffs_fwd_kernel<<<dim3(static_cast<unsigned>(blocks)), kThreads, 0,
                           static_cast<hipStream_t>(stream)>>>(alpha, delta, theta, gamma, D,
                                                                static_cast<int>(N), p, log_q,
                                                                gamma_hat);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

extern "C" int mega_cema_coeffs_bwd(const float* dp, const float* dq, const float* dgamma_hat,
                                    const float* alpha, const float* delta, const float* theta,
                                    int64_t D, int64_t N, float* dalpha, float* ddelta,
                                    float* dtheta, float* dgamma, void* stream) {
  MEGA_CHECK_ARG(dp && dq && dgamma_hat && alpha && delta && theta && dalpha && ddelta && dtheta &&
                     dgamma,
                 "mega_cema_coeffs_bwd: null pointer");
  MEGA_CHECK_ARG(D >= 0 && N >= 1 && N <= 64, "mega_cema_coeffs_bwd: need D >= 0 and 1 <= N <= 64");
  if (D == 0) return MEGA_OK;
  const int cpb = kThreads / static_cast<int>(N);
  const int64_t blocks = (D + cpb - 1) / cpb;
  MEGA_CHECK_ARG(blocks <= 0x7fffffff, "mega_cema_coeffs_bwd: too many channels");
  cema_coeffs_bwd_kernel<<<dim3(static_cast<unsigned>(blocks)), kThreads, 0,
                           static_cast<hipStream_t>(stream)>>>(dp, dq, dgamma_hat, alpha, delta, theta,
                                                                D, static_cast<int>(N), cpb, dalpha,
                                                                ddelta, dtheta, dgamma);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}
