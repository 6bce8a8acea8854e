// CPU emulation of the register-FFT convolution engine (fftconv_core.hpp):
// the lanes of one workgroup are run one after another, phase by phase, with
// LDS as a plain array.  Built by tests/test_fftconv_engine_cpu.py with g++.
#include <cmath>
#include <cstring>
#include <vector>

#include "../../megalodon_amd/csrc/fftconv_core.hpp"

using namespace mega::fftc;

template <int LOGM>
static void build_tables(std::vector<c32>& tab) {
  tab.resize(Cfg<LOGM>::TABLE);
  fill_tables<LOGM>(tab.data());
}

static float seq_at(const float* s, int L, int m, int flip) {
  if (m >= L) return 0.f;
  return flip ? s[L - 1 - m] : s[m];
}

template <int LOGM, int H>
static void forward(std::vector<float>& re, std::vector<float>& im, std::vector<float>& lre,
                    std::vector<float>& lim, const Tables& tb) {
  using C = Cfg<LOGM>;
  for (int t = 0; t < C::T; ++t) fwd_pass1<LOGM, H>(&re[t * 32], &im[t * 32], t, tb);
  for (int t = 0; t < C::T; ++t) x1_write<LOGM>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) x1_read<LOGM>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) fwd_pass2<LOGM>(&re[t * 32], &im[t * 32], t, tb);
  for (int t = 0; t < C::T; ++t) x2_write<LOGM>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) x2_read<LOGM, H>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) fwd_pass3<LOGM>(&re[t * 32], &im[t * 32]);
}

template <int LOGM, int H>
static void inverse(std::vector<float>& re, std::vector<float>& im, std::vector<float>& lre,
                    std::vector<float>& lim, const Tables& tb) {
  using C = Cfg<LOGM>;
  for (int t = 0; t < C::T; ++t) inv_pass3<LOGM, H>(&re[t * 32], &im[t * 32], t, tb);
  for (int t = 0; t < C::T; ++t) ix2_write<LOGM, H>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) ix2_read<LOGM>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) inv_pass2<LOGM, H>(&re[t * 32], &im[t * 32], t, tb);
  for (int t = 0; t < C::T; ++t) ix1_write<LOGM>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) ix1_read<LOGM>(&re[t * 32], &im[t * 32], t, lre.data(), lim.data());
  for (int t = 0; t < C::T; ++t) inv_pass1<H>(&re[t * 32], &im[t * 32]);
}

template <int LOGM>
static void load(std::vector<float>& re, std::vector<float>& im, const float* s, int L, int flip) {
  using C = Cfg<LOGM>;
  for (int t = 0; t < C::T; ++t)
    for (int j = 0; j < 32; ++j) {
      const int n = t + C::T * j;
      re[t * 32 + j] = seq_at(s, L, 2 * n, flip);
      im[t * 32 + j] = seq_at(s, L, 2 * n + 1, flip);
    }
}

template <int LOGM, int H>
static void half(const float* a, const float* b, int L, int flip_a, std::vector<float>& ore,
                 std::vector<float>& oim, const Tables& tb) {
  using C = Cfg<LOGM>;
  std::vector<float> re(C::M), im(C::M), pre(C::M), pim(C::M), lre(C::PLANE), lim(C::PLANE);
  load<LOGM>(pre, pim, b, L, 0);
  forward<LOGM, H>(pre, pim, lre, lim, tb);
  const float scale = 1.0f / (8.0f * C::M);  // 1 / (4 N)
  for (auto& v : pre) v *= scale;
  for (auto& v : pim) v *= scale;
  load<LOGM>(re, im, a, L, flip_a);
  forward<LOGM, H>(re, im, lre, lim, tb);
  for (int t = 0; t < C::T; ++t) pointwise<LOGM, H>(&re[t * 32], &im[t * 32], &pre[t * 32], &pim[t * 32], t, tb);
  inverse<LOGM, H>(re, im, lre, lim, tb);
  for (int t = 0; t < C::T; ++t)
    for (int j = 0; j < 32; ++j) {
      ore[t * 32 + j] += re[t * 32 + out_pos<H>(j)];
      oim[t * 32 + j] += im[t * 32 + out_pos<H>(j)];
    }
}

template <int LOGM>
static int run(const float* a, const float* b, int L, int flip_a, int flip_out, float* y) {
  using C = Cfg<LOGM>;
  if (L > 2 * C::M) return 1;
  std::vector<c32> tab;
  build_tables<LOGM>(tab);
  const Tables tb = make_tables<LOGM>(tab.data());
  std::vector<float> ore(C::M, 0.f), oim(C::M, 0.f);
  half<LOGM, 0>(a, b, L, flip_a, ore, oim, tb);
  half<LOGM, 1>(a, b, L, flip_a, ore, oim, tb);
  for (int t = 0; t < C::T; ++t)
    for (int j = 0; j < 32; ++j) {
      const int n = t + C::T * j;
      const int m0 = 2 * n, m1 = 2 * n + 1;
      if (m0 < L) y[flip_out ? L - 1 - m0 : m0] = ore[t * 32 + j];
      if (m1 < L) y[flip_out ? L - 1 - m1 : m1] = oim[t * 32 + j];
    }
  return 0;
}

// y = conv(flip_a ? reverse(a) : a, b)[:L], optionally reversed on output
extern "C" int emu_fftconv(int logm, const float* a, const float* b, int L, int flip_a,
                           int flip_out, float* y) {
  switch (logm) {
    case 11: return run<11>(a, b, L, flip_a, flip_out, y);
    case 12: return run<12>(a, b, L, flip_a, flip_out, y);
    case 13: return run<13>(a, b, L, flip_a, flip_out, y);
    case 14: return run<14>(a, b, L, flip_a, flip_out, y);
  }
  return 2;
}

// plain M-point transforms through the engine, for testing the passes alone:
// out[a] = sum_n in[n] W_M^(n a) (H=0) or with the extra W_N^n modulation (H=1),
// returned in natural bin order.
template <int LOGM, int H>
static void run_fwd(const float* inr, const float* ini, float* outr, float* outi) {
  using C = Cfg<LOGM>;
  std::vector<c32> tab;
  build_tables<LOGM>(tab);
  const Tables tb = make_tables<LOGM>(tab.data());
  std::vector<float> re(C::M), im(C::M), lre(C::PLANE), lim(C::PLANE);
  for (int t = 0; t < C::T; ++t)
    for (int j = 0; j < 32; ++j) {
      re[t * 32 + j] = inr[t + C::T * j];
      im[t * 32 + j] = ini[t + C::T * j];
    }
  forward<LOGM, H>(re, im, lre, lim, tb);
  constexpr int LR = ilog2(C::R3);
  for (int t = 0; t < C::T; ++t)
    for (int u = 0; u < C::NSLOT; ++u) {
      int c[2];
      slot_residues<H>(t + C::T * u, c[0], c[1]);
      for (int w = 0; w < 2; ++w)
        for (int a0 = 0; a0 < C::R3; ++a0) {
          int br = 0;
          for (int i = 0; i < LR; ++i) br |= ((a0 >> i) & 1) << (LR - 1 - i);
          const int bin = c[w] + 1024 * a0;
          outr[bin] = re[t * 32 + (u * 2 + w) * C::R3 + br];
          outi[bin] = im[t * 32 + (u * 2 + w) * C::R3 + br];
        }
    }
}
extern "C" int emu_fft_half(int logm, int h, const float* inr, const float* ini, float* outr,
                            float* outi) {
  if (logm == 11 && h == 0) run_fwd<11, 0>(inr, ini, outr, outi);
  else if (logm == 11 && h == 1) run_fwd<11, 1>(inr, ini, outr, outi);
  else if (logm == 12 && h == 0) run_fwd<12, 0>(inr, ini, outr, outi);
  else if (logm == 12 && h == 1) run_fwd<12, 1>(inr, ini, outr, outi);
  else if (logm == 13 && h == 0) run_fwd<13, 0>(inr, ini, outr, outi);
  else if (logm == 13 && h == 1) run_fwd<13, 1>(inr, ini, outr, outi);
  else if (logm == 14 && h == 0) run_fwd<14, 0>(inr, ini, outr, outi);
  else if (logm == 14 && h == 1) run_fwd<14, 1>(inr, ini, outr, outi);
  else return 1;
  return 0;
}
