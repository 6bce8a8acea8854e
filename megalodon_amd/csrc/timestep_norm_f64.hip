// Group TimestepNorm on float64 tensors.
//
// The reference instantiates its TimestepNorm kernels for double as well
// (megalodon/csrc/ops/timestep_norm_kernel.cu:1567-1576, accumulate type double:
// cummean / cumrstd are float64 then); nothing in the model runs it.  This is the
// double-precision flavour of mega_group_timestep_norm_fwd/bwd: the same
// recurrences (timestep_norm.cc:218-316 forward, :318-450 backward), storage and
// arithmetic in double, one wavefront per (batch, group) chain walking the
// sequence step by step -- the plain form of the operator, with no tiles, no
// look-back and no workspace records.
#include "common.hpp"

namespace mega {
namespace {

__device__ __forceinline__ double wsum(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

struct Tsn64 {
  const double* x;
  const double* dy;
  double* y;  // y (forward) or dx (backward)
  const int64_t* prev_count;  // forward: the carried-in count; backward: the forward's output count
  int64_t* count;
  const double* prev_mean;
  const double* prev_var;
  const double* dmean;
  const double* dvar;
  const double* gamma;
  const double* beta;
  const uint8_t* mask;
  double* mean;  // forward: final mean / var; backward: dprev_mean / dprev_var
  double* var;
  double* cummean;
  double* cumrstd;
  const double* cummean_in;
  const double* cumrstd_in;
  double* part_g;  // (B, D) partial sums of dgamma / dbeta
  double* part_b;
  int B, L, D, G, Dg;
  double eps;
};

// Forward (timestep_norm.cc:218-316): per step the group's mean and biased variance over its
// Dg features, merged into the running (count, mean, var) by Welford's rule (utils.h:154-164);
// a masked step leaves the state alone and writes 0.
__global__ __launch_bounds__(kWave) void tsn64_fwd_kernel(const Tsn64 p) {
  const int chain = blockIdx.x, b = chain / p.G, g = chain % p.G, lane = threadIdx.x;
  const double inv_dg = 1.0 / static_cast<double>(p.Dg);
  int64_t m0 = p.prev_count[b];
  double u = p.prev_mean[chain], v = p.prev_var[chain];
  for (int t = 0; t < p.L; ++t) {
    const int64_t row = (static_cast<int64_t>(b) * p.L + t) * p.D + static_cast<int64_t>(g) * p.Dg;
    const bool valid = p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0;
    double s = 0.0;
    for (int i = lane; i < p.Dg; i += kWave) s += p.x[row + i];
    const double mu = wsum(s) * inv_dg;
    double s2 = 0.0;
    for (int i = lane; i < p.Dg; i += kWave) {
      const double d = p.x[row + i] - mu;
      s2 = fma(d, d, s2);
    }
    const double var = wsum(s2) * inv_dg;
    if (valid) {
      const double m1 = static_cast<double>(m0 + 1);
      const double c1 = static_cast<double>(m0) / m1, c2 = 1.0 / m1;
      const double delta = mu - u;
      u = c1 * u + c2 * mu;
      v = c1 * v + c2 * var + c1 * c2 * delta * delta;
      ++m0;
    }
    const double rstd = 1.0 / sqrt(v + p.eps);
    if (lane == 0) {
      const int64_t o = (static_cast<int64_t>(b) * p.L + t) * p.G + g;
      p.cummean[o] = u;
      p.cumrstd[o] = rstd;
    }
    for (int i = lane; i < p.Dg; i += kWave) {
      const int h = g * p.Dg + i;
      p.y[row + i] = valid ? (p.x[row + i] - u) * rstd * p.gamma[h] + p.beta[h] : 0.0;
    }
  }
  if (lane == 0) {
    p.mean[chain] = u;
    p.var[chain] = v;
    if (g == 0) p.count[b] = m0;
  }
}

// Backward (timestep_norm.cc:385-430), in reverse time: carried gradients (ug, vg) of the
// running mean and variance; per step c1 = (m0 - 1) / m0, c2 = 1 / m0 with m0 the count
// after that step.
__global__ __launch_bounds__(kWave) void tsn64_bwd_kernel(const Tsn64 p) {
  const int chain = blockIdx.x, b = chain / p.G, g = chain % p.G, lane = threadIdx.x;
  const double inv_dg = 1.0 / static_cast<double>(p.Dg);
  double ug = p.dmean[chain], vg = p.dvar[chain];
  int64_t m0 = p.prev_count[b];
  // this lane's features keep their dgamma / dbeta sums in registers across the sequence
  // when the group is at most 4 * 64 wide; wider groups accumulate in memory
  constexpr int kKeep = 4;
  const bool keep = p.Dg <= kKeep * kWave;
  double ag[kKeep] = {0.0, 0.0, 0.0, 0.0}, ab[kKeep] = {0.0, 0.0, 0.0, 0.0};
  if (!keep)
    for (int i = lane; i < p.Dg; i += kWave) {
      p.part_g[static_cast<int64_t>(b) * p.D + g * p.Dg + i] = 0.0;
      p.part_b[static_cast<int64_t>(b) * p.D + g * p.Dg + i] = 0.0;
    }
  for (int t = p.L - 1; t >= 0; --t) {
    const int64_t row = (static_cast<int64_t>(b) * p.L + t) * p.D + static_cast<int64_t>(g) * p.Dg;
    const bool valid = p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0;
    if (!valid) {
      for (int i = lane; i < p.Dg; i += kWave) p.y[row + i] = 0.0;
      continue;
    }
    const int64_t so = (static_cast<int64_t>(b) * p.L + t) * p.G + g;
    const double u = p.cummean_in[so], r = p.cumrstd_in[so];
    const double prev_u = t == 0 ? p.prev_mean[chain] : p.cummean_in[so - p.G];
    const double c1 = static_cast<double>(m0 - 1) / static_cast<double>(m0);
    const double c2 = 1.0 / static_cast<double>(m0);
    --m0;
    double sx = 0.0, sds = 0.0, sdb = 0.0;
    for (int i = lane; i < p.Dg; i += kWave) {
      const double xx = p.x[row + i], d = p.dy[row + i], w = p.gamma[g * p.Dg + i];
      sx += xx;
      sds = fma(d * (xx - u), w, sds);
      sdb = fma(d, w, sdb);
    }
    const double ux = wsum(sx) * inv_dg;
    const double ds = wsum(sds), db = wsum(sdb);
    const double du = ug - r * db;
    const double dvv = vg - 0.5 * r * r * r * ds;
    const double dux = c2 * du + 2.0 * c1 * c2 * dvv * (ux - prev_u);
    const double dvx = c2 * dvv;
    if (keep) {
#pragma unroll
      for (int slot = 0; slot < kKeep; ++slot) {
        const int i = lane + kWave * slot;
        if (i < p.Dg) {
          const double xx = p.x[row + i], d = p.dy[row + i], w = p.gamma[g * p.Dg + i];
          p.y[row + i] = d * r * w + (dux + 2.0 * dvx * (xx - ux)) * inv_dg;
          ag[slot] = fma(d * (xx - u), r, ag[slot]);
          ab[slot] += d;
        }
      }
    } else {
      for (int i = lane; i < p.Dg; i += kWave) {
        const double xx = p.x[row + i], d = p.dy[row + i], w = p.gamma[g * p.Dg + i];
        p.y[row + i] = d * r * w + (dux + 2.0 * dvx * (xx - ux)) * inv_dg;
        p.part_g[static_cast<int64_t>(b) * p.D + g * p.Dg + i] += d * (xx - u) * r;
        p.part_b[static_cast<int64_t>(b) * p.D + g * p.Dg + i] += d;
      }
    }
    ug = c1 * du - 2.0 * c1 * c2 * dvv * (ux - prev_u);
    vg = c1 * dvv;
  }
  if (keep) {
#pragma unroll
    for (int slot = 0; slot < kKeep; ++slot) {
      const int i = lane + kWave * slot;
      if (i < p.Dg) {
        p.part_g[static_cast<int64_t>(b) * p.D + g * p.Dg + i] = ag[slot];
        p.part_b[static_cast<int64_t>(b) * p.D + g * p.Dg + i] = ab[slot];
      }
    }
  }
  if (lane == 0) {
    p.mean[chain] = ug;
    p.var[chain] = vg;
  }
}

// dgamma[h] = sum_b part_g[b][h], dbeta likewise (fixed order: deterministic)
__global__ void tsn64_param_grad_kernel(const double* part_g, const double* part_b, int B, int D, double* dgamma,
                                        double* dbeta) {
  const int h = blockIdx.x * blockDim.x + threadIdx.x;
  if (h >= D) return;
  double a = 0.0, c = 0.0;
  for (int b = 0; b < B; ++b) {
    a += part_g[static_cast<int64_t>(b) * D + h];
    c += part_b[static_cast<int64_t>(b) * D + h];
  }
  dgamma[h] = a;
  dbeta[h] = c;
}

int check(const char* who, int64_t B, int64_t L, int64_t D, int64_t G) {
  MEGA_CHECK_ARG(B >= 0 && L >= 0 && D >= 1 && G >= 1 && D % G == 0, "%s: bad sizes (D must be a multiple of G)", who);
  MEGA_CHECK_ARG(B * G <= 0x7fffffff && L <= 0x7fffffff && D <= 0x7fffffff, "%s: sizes exceed 2^31", who);
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_group_timestep_norm_fwd_f64(const double* x, const int64_t* prev_count, const double* prev_mean,
                                                const double* prev_var, const double* gamma, const double* beta,
                                                const uint8_t* padding_mask, int64_t B, int64_t L, int64_t D,
                                                int64_t G, double eps, double* y, int64_t* count, double* mean,
                                                double* var, double* cummean, double* cumrstd, void* stream) {
  int rc = check("mega_group_timestep_norm_fwd_f64", B, L, D, G);
  if (rc != MEGA_OK) return rc;
  if (B == 0) return MEGA_OK;
  MEGA_CHECK_ARG(prev_count && prev_mean && prev_var && gamma && beta && count && mean && var,
                 "mega_group_timestep_norm_fwd_f64: null pointer");
  MEGA_CHECK_ARG(L == 0 || (x && y && cummean && cumrstd), "mega_group_timestep_norm_fwd_f64: null pointer");
  Tsn64 p{};
  p.x = x; p.y = y; p.prev_count = prev_count; p.count = count; p.prev_mean = prev_mean; p.prev_var = prev_var;
  p.gamma = gamma; p.beta = beta; p.mask = padding_mask; p.mean = mean; p.var = var;
  p.cummean = cummean; p.cumrstd = cumrstd;
  p.B = (int)B; p.L = (int)L; p.D = (int)D; p.G = (int)G; p.Dg = (int)(D / G); p.eps = eps;
  tsn64_fwd_kernel<<<dim3((unsigned)(B * G)), kWave, 0, static_cast<hipStream_t>(stream)>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

extern "C" int mega_group_timestep_norm_bwd_f64(const double* dy, const double* dmean, const double* dvar,
                                                const double* x, const double* prev_mean, const int64_t* count,
                                                const double* cummean, const double* cumrstd, const double* gamma,
                                                const uint8_t* padding_mask, int64_t B, int64_t L, int64_t D,
                                                int64_t G, double* dx, double* dprev_mean, double* dprev_var,
                                                double* dgamma, double* dbeta, double* workspace, void* stream) {
  int rc = check("mega_group_timestep_norm_bwd_f64", B, L, D, G);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG(dgamma && dbeta, "mega_group_timestep_norm_bwd_f64: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B > 0) {
    MEGA_CHECK_ARG(dmean && dvar && prev_mean && count && gamma && dprev_mean && dprev_var && workspace,
                   "mega_group_timestep_norm_bwd_f64: null pointer");
    MEGA_CHECK_ARG(L == 0 || (dy && x && dx && cummean && cumrstd), "mega_group_timestep_norm_bwd_f64: null pointer");
    Tsn64 p{};
    p.x = x; p.dy = dy; p.y = dx; p.prev_count = count; p.prev_mean = prev_mean; p.dmean = dmean; p.dvar = dvar;
    p.gamma = gamma; p.mask = padding_mask; p.mean = dprev_mean; p.var = dprev_var;
    p.cummean_in = cummean; p.cumrstd_in = cumrstd; p.part_g = workspace; p.part_b = workspace + B * D;
    p.B = (int)B; p.L = (int)L; p.D = (int)D; p.G = (int)G; p.Dg = (int)(D / G);
    tsn64_bwd_kernel<<<dim3((unsigned)(B * G)), kWave, 0, s>>>(p);
    MEGA_CHECK_LAUNCH();
  }
  tsn64_param_grad_kernel<<<dim3((unsigned)((D + 255) / 256)), 256, 0, s>>>(workspace, workspace + B * D, (int)B, (int)D,
                                                                            dgamma, dbeta);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}
