/*
 * C / OpenMP restatement of the reference's CPU loop nests for the hot path.
 * TEST INFRASTRUCTURE ONLY (checker for tests and the timed `cpu_baseline` of
 * bench.py); nothing in the product links or loads this file.
 *
 * Parallel structure is kept as in the reference: `ema_parameters` over
 * channels D (ema_parameters.cc:37), TimestepNorm group moments over B*L*G
 * (timestep_norm.cc:252) and the time scan over the batch only (:264).
 * Arithmetic is float32 with float32 accumulation (at::opmath_type<float>).
 */
#include <complex.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* w[d,j] = sum_n Re(p*gamma * exp(log_q * j))      ema_parameters.cc:17-52 */
void oracle_ema_weight_fwd(const float* p, const float* log_q, const float* gamma, int64_t D,
                           int64_t N, int64_t L, float* w) {
  const float complex* lq = (const float complex*)log_q;
  const float complex* gm = (const float complex*)gamma;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < D; ++i) {
    for (int64_t j = 0; j < L; ++j) {
      float sum = 0.f;
      for (int64_t k = 0; k < N; ++k) {
        const float complex c = p[i * N + k] * gm[i * N + k];
        const float complex qw = cexpf(lq[i * N + k] * (float)j);
        sum += crealf(c * qw);
      }
      w[i * L + j] = sum;
    }
  }
}

/* (dp, dq, dgamma)                                   ema_parameters.cc:80-98,141-156 */
void oracle_ema_weight_bwd(const float* dw, const float* p, const float* log_q, const float* gamma,
                           int64_t D, int64_t N, int64_t L, float* dp, float* dq, float* dgamma) {
  const float complex* lq = (const float complex*)log_q;
  const float complex* gm = (const float complex*)gamma;
  float complex* dqc = (float complex*)dq;
  float complex* dgc = (float complex*)dgamma;
#pragma omp parallel for schedule(static)
  for (int64_t d = 0; d < D; ++d) {
    for (int64_t n = 0; n < N; ++n) {
      const float complex l = lq[d * N + n];
      const float complex q = cexpf(l);
      float complex sum1 = 0.f, sum2 = 0.f;
      for (int64_t i = 0; i < L; ++i) {
        const float g = dw[d * L + i];
        const float complex qw1 = i == 0 ? 0.f : cexpf(l * (float)(i - 1));
        const float complex qw2 = i == 0 ? 1.f : qw1 * q;
        sum1 += g * qw1 * (float)i;
        sum2 += g * qw2;
      }
      dp[d * N + n] = crealf(sum2 * gm[d * N + n]);
      dqc[d * N + n] = conjf(sum1 * p[d * N + n] * gm[d * N + n]);
      dgc[d * N + n] = conjf(sum2 * p[d * N + n]);
    }
  }
}

/* WelfordCombine                                      utils.h:154-164 */
static inline void welford_combine(int64_t a0, float a1, float a2, int64_t b0, float b1, float b2,
                                   float* m1, float* m2) {
  const int64_t m0 = a0 + b0;
  const float c1 = m0 == 0 ? 0.f : (float)a0 / (float)m0;
  const float c2 = m0 == 0 ? 0.f : (float)b0 / (float)m0;
  const float delta = b1 - a1;
  *m1 = c1 * a1 + c2 * b1;
  *m2 = c1 * a2 + c2 * b2 + (c1 * delta) * (c2 * delta);
}

/* GroupTimestepNorm forward                           timestep_norm.cc:218-316
 * x, y (B, L, H); gamma, beta (H); prev_mean/var, mean/var (B, G); mask (B, L)
 * or NULL (1 = padding); cummean, cumrstd (B, L, G).  At masked steps the
 * stored cummean/cumrstd are those of the UNCHANGED state, as the reference's
 * CUDA kernel does (timestep_norm_kernel.cu:621-626); its CPU loop stores the
 * would-be-updated value instead (timestep_norm.cc:294-297) -- the two agree
 * wherever the mask is trailing padding. */
void oracle_group_timestep_norm_fwd(const float* x, const int64_t* prev_count,
                                    const float* prev_mean, const float* prev_var,
                                    const float* gamma, const float* beta, const uint8_t* mask,
                                    int64_t B, int64_t L, int64_t H, int64_t G, double eps,
                                    float* y, int64_t* count, float* mean, float* var,
                                    float* cummean, float* cumrstd) {
  const int64_t Dg = H / G;
  float* gmean = (float*)malloc(sizeof(float) * B * L * G);
  float* gvar = (float*)malloc(sizeof(float) * B * L * G);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * L * G; ++i) {
    /* sequential Welford update over the group (utils.h:143-152) */
    const float* xp = x + i * Dg;
    float m1 = 0.f, m2 = 0.f;
    for (int64_t k = 0; k < Dg; ++k) {
      const float coef = 1.f / (float)(k + 1);
      const float d1 = xp[k] - m1;
      m1 += coef * d1;
      const float d2 = d1 * (xp[k] - m1) - m2;
      m2 += coef * d2;
    }
    gmean[i] = m1;
    gvar[i] = m2;
  }
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < B; ++b) {
    int64_t m0 = prev_count[b];
    float* u = (float*)malloc(sizeof(float) * G);
    float* v = (float*)malloc(sizeof(float) * G);
    for (int64_t g = 0; g < G; ++g) {
      u[g] = prev_mean[b * G + g];
      v[g] = prev_var[b * G + g];
    }
    for (int64_t j = 0; j < L; ++j) {
      const int msk = mask != NULL && mask[b * L + j];
      for (int64_t g = 0; g < G; ++g) {
        float m1, m2;
        welford_combine(m0, u[g], v[g], 1, gmean[(b * L + j) * G + g], gvar[(b * L + j) * G + g],
                        &m1, &m2);
        if (!msk) {
          u[g] = m1;
          v[g] = m2;
        }
        const float rstd = 1.f / sqrtf(v[g] + (float)eps);
        cummean[(b * L + j) * G + g] = u[g];
        cumrstd[(b * L + j) * G + g] = rstd;
        for (int64_t k = 0; k < Dg; ++k) {
          const int64_t o = (b * L + j) * H + g * Dg + k;
          y[o] = msk ? 0.f : (x[o] - u[g]) * rstd * gamma[g * Dg + k] + beta[g * Dg + k];
        }
      }
      m0 += msk ? 0 : 1;
    }
    count[b] = m0;
    for (int64_t g = 0; g < G; ++g) {
      mean[b * G + g] = u[g];
      var[b * G + g] = v[g];
    }
    free(u);
    free(v);
  }
  free(gmean);
  free(gvar);
}

/* GroupTimestepNorm backward                          timestep_norm.cc:318-450 */
void oracle_group_timestep_norm_bwd(const float* dy, const float* dmean, const float* dvar,
                                    const float* x, const float* prev_mean, const int64_t* count,
                                    const float* cummean, const float* cumrstd,
                                    const float* gamma, const uint8_t* mask, int64_t B, int64_t L,
                                    int64_t H, int64_t G, float* dx, float* dprev_mean,
                                    float* dprev_var, float* dgamma, float* dbeta) {
  const int64_t Dg = H / G;
  const float cg = 1.f / (float)Dg;
  float* wg = (float*)calloc(B * H, sizeof(float));
  float* bg = (float*)calloc(B * H, sizeof(float));
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < B; ++b) {
    int64_t m0 = count[b];
    float* ug = (float*)malloc(sizeof(float) * G);
    float* vg = (float*)malloc(sizeof(float) * G);
    for (int64_t g = 0; g < G; ++g) {
      ug[g] = dmean[b * G + g];
      vg[g] = dvar[b * G + g];
    }
    for (int64_t j = L - 1; j >= 0; --j) {
      const int msk = mask != NULL && mask[b * L + j];
      const float c1 = (float)(m0 - 1) / (float)m0;
      const float c2 = 1.f / (float)m0;
      m0 -= msk ? 0 : 1;
      for (int64_t g = 0; g < G; ++g) {
        const float prev_u = j == 0 ? prev_mean[b * G + g] : cummean[(b * L + j - 1) * G + g];
        const float u = cummean[(b * L + j) * G + g];
        const float r = cumrstd[(b * L + j) * G + g];
        float ux = 0.f, ds = 0.f, db = 0.f;
        for (int64_t k = 0; k < Dg; ++k) {
          const int64_t o = (b * L + j) * H + g * Dg + k;
          const float w = gamma[g * Dg + k];
          ux += x[o];
          ds += dy[o] * (x[o] - u) * w;
          db += dy[o] * w;
        }
        ux /= (float)Dg;
        const float du = ug[g] - r * db;
        const float dv = vg[g] - 0.5f * r * r * r * ds;
        const float dux = c2 * du + 2.f * c1 * c2 * dv * (ux - prev_u);
        const float dvx = c2 * dv;
        for (int64_t k = 0; k < Dg; ++k) {
          const int64_t o = (b * L + j) * H + g * Dg + k;
          const float w = gamma[g * Dg + k];
          const float v = dy[o] * r * w + dux * cg + 2.f * dvx * cg * (x[o] - ux);
          dx[o] = msk ? 0.f : v;
          wg[b * H + g * Dg + k] += msk ? 0.f : dy[o] * (x[o] - u) * r;
          bg[b * H + g * Dg + k] += msk ? 0.f : dy[o];
        }
        if (!msk) {
          ug[g] = c1 * du - 2.f * c1 * c2 * dv * (ux - prev_u);
          vg[g] = c1 * dv;
        }
      }
    }
    for (int64_t g = 0; g < G; ++g) {
      dprev_mean[b * G + g] = ug[g];
      dprev_var[b * G + g] = vg[g];
    }
    free(ug);
    free(vg);
  }
  for (int64_t h = 0; h < H; ++h) {
    float s1 = 0.f, s2 = 0.f;
    for (int64_t b = 0; b < B; ++b) {
      s1 += wg[b * H + h];
      s2 += bg[b * H + h];
    }
    dgamma[h] = s1;
    dbeta[h] = s2;
  }
  free(wg);
  free(bg);
}
