// Thin extern "C" driver over the reference's own C++ CPU operators, compiled
// from the sources where they lie under /root/reference (see oracle/Makefile).
// TEST INFRASTRUCTURE ONLY: used to validate the oracle restatements and,
// optionally, as the timed CPU baseline.  Only the reference's *CPU* entry
// points are called (EMAParametersCPUFwd/Bwd, EMAHiddenCPUFwd/Bwd, GroupTimestepNormCPUFwd/Bwd,
// GroupSequenceNormCPUFwd/Bwd, declared in megalodon/csrc/ops/ema_parameters.h:19-49,
// timestep_norm.h and sequence_norm.h:57-83).
#include <torch/torch.h>

#include "ops/ema_hidden.h"
#include "ops/ema_parameters.h"
#include "ops/sequence_norm.h"
#include "ops/timestep_norm.h"

namespace mo = megalodon::ops;

static torch::Tensor f32(const float* p, std::vector<int64_t> shape) {
  return torch::from_blob(const_cast<float*>(p), shape, torch::kFloat32);
}
static torch::Tensor c64(const float* p, std::vector<int64_t> shape) {
  return torch::from_blob(const_cast<float*>(p), shape, torch::kComplexFloat);
}

extern "C" __attribute__((visibility("default"))) int ref_ema_weight_fwd(const float* p, const float* log_q, const float* gamma,
                                  int64_t D, int64_t N, int64_t L, float* w) {
  auto out = mo::EMAParametersCPUFwd(f32(p, {D, N}), c64(log_q, {D, N}), c64(gamma, {D, N}),
                                     c10::nullopt, L);
  std::memcpy(w, std::get<0>(out).data_ptr<float>(), sizeof(float) * D * L);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ref_ema_weight_bwd(const float* dw, const float* p, const float* log_q,
                                  const float* gamma, int64_t D, int64_t N, int64_t L, float* dp,
                                  float* dq, float* dgamma) {
  auto out = mo::EMAParametersCPUBwd(f32(dw, {D, L}), c10::nullopt, f32(p, {D, N}),
                                     c64(log_q, {D, N}), c64(gamma, {D, N}), c10::nullopt,
                                     c10::nullopt);
  std::memcpy(dp, std::get<0>(out).data_ptr<float>(), sizeof(float) * D * N);
  std::memcpy(dq, std::get<1>(out).data_ptr(), sizeof(float) * 2 * D * N);
  std::memcpy(dgamma, std::get<2>(out).data_ptr(), sizeof(float) * 2 * D * N);
  return 0;
}

// float32 tensors throughout; mask may be null.
extern "C" __attribute__((visibility("default"))) int ref_group_timestep_norm_fwd(const float* x, const int64_t* prev_count,
                                           const float* prev_mean, const float* prev_var,
                                           const float* gamma, const float* beta,
                                           const uint8_t* mask, int64_t B, int64_t L, int64_t H,
                                           int64_t G, double eps, float* y, int64_t* count,
                                           float* mean, float* var, float* cummean,
                                           float* cumrstd) {
  c10::optional<torch::Tensor> m = c10::nullopt;
  if (mask) m = torch::from_blob(const_cast<uint8_t*>(mask), {B, L}, torch::kBool);
  auto pc = torch::from_blob(const_cast<int64_t*>(prev_count), {B}, torch::kInt64);
  auto out = mo::GroupTimestepNormCPUFwd(f32(x, {B, L, H}), pc, f32(prev_mean, {B, G}),
                                         f32(prev_var, {B, G}), f32(gamma, {H}), f32(beta, {H}),
                                         m, G, eps);
  std::memcpy(y, std::get<0>(out).data_ptr<float>(), sizeof(float) * B * L * H);
  std::memcpy(count, std::get<1>(out).data_ptr<int64_t>(), sizeof(int64_t) * B);
  std::memcpy(mean, std::get<2>(out).data_ptr<float>(), sizeof(float) * B * G);
  std::memcpy(var, std::get<3>(out).data_ptr<float>(), sizeof(float) * B * G);
  std::memcpy(cummean, std::get<4>(out).data_ptr<float>(), sizeof(float) * B * L * G);
  std::memcpy(cumrstd, std::get<5>(out).data_ptr<float>(), sizeof(float) * B * L * G);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ref_group_timestep_norm_bwd(const float* dy, const float* dmean, const float* dvar,
                                           const float* x, const float* prev_mean,
                                           const int64_t* count, const float* cummean,
                                           const float* cumrstd, const float* gamma,
                                           const uint8_t* mask, int64_t B, int64_t L, int64_t H,
                                           int64_t G, float* dx, float* dprev_mean,
                                           float* dprev_var, float* dgamma, float* dbeta) {
  c10::optional<torch::Tensor> m = c10::nullopt;
  if (mask) m = torch::from_blob(const_cast<uint8_t*>(mask), {B, L}, torch::kBool);
  auto cnt = torch::from_blob(const_cast<int64_t*>(count), {B}, torch::kInt64);
  auto out = mo::GroupTimestepNormCPUBwd(f32(dy, {B, L, H}), f32(dmean, {B, G}), f32(dvar, {B, G}),
                                         f32(x, {B, L, H}), f32(prev_mean, {B, G}), cnt,
                                         f32(cummean, {B, L, G}), f32(cumrstd, {B, L, G}),
                                         f32(gamma, {H}), m, G);
  std::memcpy(dx, std::get<0>(out).data_ptr<float>(), sizeof(float) * B * L * H);
  std::memcpy(dprev_mean, std::get<1>(out).data_ptr<float>(), sizeof(float) * B * G);
  std::memcpy(dprev_var, std::get<2>(out).data_ptr<float>(), sizeof(float) * B * G);
  std::memcpy(dgamma, std::get<3>(out).data_ptr<float>(), sizeof(float) * H);
  std::memcpy(dbeta, std::get<4>(out).data_ptr<float>(), sizeof(float) * H);
  return 0;
}

// ---- carried state: bias branch of ema_parameters and ema_hidden (float32) -------
// h (B, D, N) complex; b, b_grad (B, D, L).  w_grad is taken as zeros so that the
// returned gradients are the bias contributions alone.
extern "C" __attribute__((visibility("default"))) int ref_ema_bias_fwd(
    const float* p, const float* log_q, const float* gamma, const float* h, int64_t B, int64_t D,
    int64_t N, int64_t L, float* b) {
  auto out = mo::EMAParametersCPUFwd(f32(p, {D, N}), c64(log_q, {D, N}), c64(gamma, {D, N}),
                                     c10::make_optional(c64(h, {B, D, N})), L);
  std::memcpy(b, std::get<1>(out)->data_ptr<float>(), sizeof(float) * B * D * L);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ref_ema_bias_bwd(
    const float* b_grad, const float* p, const float* log_q, const float* gamma, const float* h,
    int64_t B, int64_t D, int64_t N, int64_t L, float* dq, float* dgamma, float* dh) {
  auto out = mo::EMAParametersCPUBwd(torch::zeros({D, L}, torch::kFloat32),
                                     c10::make_optional(f32(b_grad, {B, D, L})), f32(p, {D, N}),
                                     c64(log_q, {D, N}), c64(gamma, {D, N}),
                                     c10::make_optional(c64(h, {B, D, N})), c10::nullopt);
  std::memcpy(dq, std::get<1>(out).data_ptr(), sizeof(float) * 2 * D * N);
  std::memcpy(dgamma, std::get<2>(out).data_ptr(), sizeof(float) * 2 * D * N);
  std::memcpy(dh, std::get<3>(out)->data_ptr(), sizeof(float) * 2 * B * D * N);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ref_ema_hidden_fwd(
    const float* x, const float* p, const float* log_q, const float* h, int64_t B, int64_t D,
    int64_t N, int64_t L, float* y) {
  c10::optional<torch::Tensor> hh = c10::nullopt;
  if (h) hh = c64(h, {B, D, N});
  auto out = mo::EMAHiddenCPUFwd(f32(x, {B, D, L}), f32(p, {D, N}), c64(log_q, {D, N}), hh);
  std::memcpy(y, std::get<0>(out).data_ptr(), sizeof(float) * 2 * B * D * N);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ref_ema_hidden_bwd(
    const float* y_grad, const float* x, const float* p, const float* log_q, const float* h,
    int64_t B, int64_t D, int64_t N, int64_t L, float* dx, float* dp, float* dq, float* dh) {
  c10::optional<torch::Tensor> hh = c10::nullopt;
  if (h) hh = c64(h, {B, D, N});
  auto out = mo::EMAHiddenCPUBwd(c64(y_grad, {B, D, N}), f32(x, {B, D, L}), f32(p, {D, N}),
                                 c64(log_q, {D, N}), hh, c10::nullopt);
  std::memcpy(dx, std::get<0>(out).data_ptr<float>(), sizeof(float) * B * D * L);
  std::memcpy(dp, std::get<1>(out).data_ptr<float>(), sizeof(float) * D * N);
  std::memcpy(dq, std::get<2>(out).data_ptr(), sizeof(float) * 2 * D * N);
  if (h) std::memcpy(dh, std::get<3>(out)->data_ptr(), sizeof(float) * 2 * B * D * N);
  return 0;
}

// ---- whole-sequence group normalisation (float32) ---------------------------------
// x, y, dy, dx: (B, L, H), or (B, H, L) when length_last; mean, rstd (B, G).
extern "C" __attribute__((visibility("default"))) int ref_group_sequence_norm_fwd(
    const float* x, const float* gamma, const float* beta, const uint8_t* mask, int64_t B, int64_t L, int64_t H,
    int64_t G, double eps, int length_last, float* y, int64_t* count, float* mean, float* rstd) {
  c10::optional<torch::Tensor> m = c10::nullopt;
  if (mask) m = torch::from_blob(const_cast<uint8_t*>(mask), {B, L}, torch::kBool);
  const std::vector<int64_t> shape = length_last ? std::vector<int64_t>{B, H, L} : std::vector<int64_t>{B, L, H};
  auto out = mo::GroupSequenceNormCPUFwd(f32(x, shape), f32(gamma, {H}), f32(beta, {H}), m, G, eps,
                                         length_last != 0);
  std::memcpy(y, std::get<0>(out).data_ptr<float>(), sizeof(float) * B * L * H);
  std::memcpy(count, std::get<1>(out).data_ptr<int64_t>(), sizeof(int64_t) * B);
  std::memcpy(mean, std::get<2>(out).data_ptr<float>(), sizeof(float) * B * G);
  std::memcpy(rstd, std::get<3>(out).data_ptr<float>(), sizeof(float) * B * G);
  return 0;
}

extern "C" __attribute__((visibility("default"))) int ref_group_sequence_norm_bwd(
    const float* dy, const float* x, const int64_t* count, const float* mean, const float* rstd, const float* gamma,
    const uint8_t* mask, int64_t B, int64_t L, int64_t H, int64_t G, int length_last, float* dx, float* dgamma,
    float* dbeta) {
  c10::optional<torch::Tensor> m = c10::nullopt;
  if (mask) m = torch::from_blob(const_cast<uint8_t*>(mask), {B, L}, torch::kBool);
  const std::vector<int64_t> shape = length_last ? std::vector<int64_t>{B, H, L} : std::vector<int64_t>{B, L, H};
  auto cnt = torch::from_blob(const_cast<int64_t*>(count), {B}, torch::kInt64);
  auto out = mo::GroupSequenceNormCPUBwd(f32(dy, shape), f32(x, shape), cnt, f32(mean, {B, G}), f32(rstd, {B, G}),
                                         f32(gamma, {H}), m, G, length_last != 0);
  std::memcpy(dx, std::get<0>(out).data_ptr<float>(), sizeof(float) * B * L * H);
  std::memcpy(dgamma, std::get<1>(out).data_ptr<float>(), sizeof(float) * H);
  std::memcpy(dbeta, std::get<2>(out).data_ptr<float>(), sizeof(float) * H);
  return 0;
}
