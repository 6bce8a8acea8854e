// Register-resident FFT engine for the causal convolution (gfx950).
//
// Plain C++17 with no HIP dependency in the algorithmic part, so the same
// phases run under g++ in a CPU harness (threads emulated one after another,
// LDS as an ordinary array) and under hipcc inside the kernel.
//
// Problem.  y = irfft(rfft(a, 2N) * rfft(b, 2N))[:L] with N = 2^n >= L
// (megalodon/modules/fused_ops/fftconv.py:30-50).  Both real sequences are
// split into even/odd samples, z[n] = s[2n] + i s[2n+1], n < M = N/2 (the
// upper half of the N-point z sequence is the zero padding).  The N-point
// spectrum Z[r] then splits by parity of r into two independent M-point
// transforms that never need the zeros:
//     Z[2a]   = FFT_M(z[n])[a]            ("even half", H = 0)
//     Z[2a+1] = FFT_M(z[n] W_N^n)[a]      ("odd half",  H = 1)
// With E = (Z[r] + conj Z[N-r])/2 (spectrum of the even samples) and
// O = -i (Z[r] - conj Z[N-r])/2 (odd samples) the product is the polyphase
// identity   Ey = Ea Eb + W_N^r Oa Ob,   Oy = Ea Ob + Oa Eb,   Zy = Ey + i Oy,
// and only the first M outputs of the inverse are needed (the [:L] crop):
//     zy[n] = IFFT_M(Zy[2a])[n] + W_N^-n IFFT_M(Zy[2a+1])[n].
//
// Engine.  One workgroup of T = M/32 lanes transforms one M-point half with 32
// complex points per lane in registers: M = 32 * 32 * R3 (R3 = M/1024 in
// {2,4,8,16}); pass 1 radix-32 over the top digit, LDS exchange, pass 2
// radix-32, LDS exchange, pass 3 radix-R3 (32/R3 butterflies per lane).  The
// residues handled by one lane in pass 3 are chosen in conjugate pairs
// (c, 1024-c) / (c, 1023-c), so both Z[r] and Z[N-r] of every bin sit in the
// same lane and the pointwise stage needs no further exchange.  The inverse is
// the mirror image (decimation-in-time first pass, then the same radix-32
// passes on swapped re/im).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define MEGA_HD __host__ __device__ __forceinline__
#else
#define MEGA_HD inline
#endif
// keeps the compiler from issuing every table load of a pass at once
#define MEGA_MEM_FENCE() asm volatile("" ::: "memory")

namespace mega {
namespace fftc {

struct c32 {
  float x, y;
};
struct alignas(8) f2 {
  float x, y;
};

// cos/sin of 2*pi*k/64
constexpr float kC64[64] = {
    1.f, 0.99518472667219693f, 0.98078528040323043f, 0.95694033573220882f, 0.92387953251128674f, 0.88192126434835505f, 0.83146961230254524f, 0.77301045336273699f, 0.70710678118654757f, 0.63439328416364549f, 0.55557023301960229f, 0.47139673682599781f, 0.38268343236508984f, 0.29028467725446233f, 0.19509032201612833f, 0.09801714032956077f,
    0.f, -0.098017140329560645f, -0.19509032201612819f, -0.29028467725446216f, -0.38268343236508973f, -0.4713967368259977f, -0.55557023301960196f, -0.63439328416364538f, -0.70710678118654746f, -0.77301045336273699f, -0.83146961230254535f, -0.88192126434835494f, -0.92387953251128674f, -0.95694033573220882f, -0.98078528040323043f, -0.99518472667219682f,
    -1.f, -0.99518472667219693f, -0.98078528040323043f, -0.95694033573220894f, -0.92387953251128685f, -0.88192126434835505f, -0.83146961230254546f, -0.7730104533627371f, -0.70710678118654768f, -0.63439328416364593f, -0.55557023301960218f, -0.47139673682599786f, -0.38268343236509034f, -0.29028467725446244f, -0.19509032201612866f, -0.098017140329560451f,
    0.f, 0.09801714032956009f, 0.1950903220161283f, 0.29028467725446205f, 0.38268343236509f, 0.47139673682599759f, 0.55557023301960184f, 0.6343932841636456f, 0.70710678118654735f, 0.77301045336273666f, 0.83146961230254524f, 0.88192126434835483f, 0.92387953251128652f, 0.95694033573220882f, 0.98078528040323032f, 0.99518472667219693f};
constexpr float kS64[64] = {
    0.f, 0.098017140329560604f, 0.19509032201612825f, 0.29028467725446233f, 0.38268343236508978f, 0.47139673682599764f, 0.55557023301960218f, 0.63439328416364549f, 0.70710678118654746f, 0.77301045336273699f, 0.83146961230254524f, 0.88192126434835494f, 0.92387953251128674f, 0.95694033573220894f, 0.98078528040323043f, 0.99518472667219682f,
    1.f, 0.99518472667219693f, 0.98078528040323043f, 0.95694033573220894f, 0.92387953251128674f, 0.88192126434835505f, 0.83146961230254546f, 0.7730104533627371f, 0.70710678118654757f, 0.63439328416364549f, 0.55557023301960218f, 0.47139673682599786f, 0.38268343236508989f, 0.29028467725446239f, 0.19509032201612861f, 0.098017140329560826f,
    0.f, -0.09801714032956059f, -0.19509032201612836f, -0.29028467725446211f, -0.38268343236508967f, -0.47139673682599764f, -0.55557023301960196f, -0.63439328416364527f, -0.70710678118654746f, -0.77301045336273666f, -0.83146961230254524f, -0.88192126434835494f, -0.92387953251128652f, -0.95694033573220882f, -0.98078528040323032f, -0.99518472667219693f,
    -1.f, -0.99518472667219693f, -0.98078528040323043f, -0.95694033573220894f, -0.92387953251128663f, -0.88192126434835505f, -0.83146961230254546f, -0.77301045336273688f, -0.70710678118654768f, -0.63439328416364593f, -0.55557023301960218f, -0.47139673682599792f, -0.38268343236509039f, -0.2902846772544625f, -0.19509032201612872f, -0.098017140329560506f};

constexpr float kRsqrt2 = 0.70710678118654752f;

template <int BITS>
constexpr int bitrev(int x) {
  int r = 0;
  for (int i = 0; i < BITS; ++i) r |= ((x >> i) & 1) << (BITS - 1 - i);
  return r;
}
constexpr int ilog2(int x) { return x <= 1 ? 0 : 1 + ilog2(x >> 1); }

// v *= W_R^i with W_R = exp(-2 pi i / R), i < R/2 ... general k in [0, R)
template <int R>
MEGA_HD void mul_w(float& xr, float& xi, int k) {
  // callers pass compile-time k after unrolling
  const int q = (k * (64 / R)) & 63;
  const float c = kC64[q], s = kS64[q];  // W = c - i s
  const float r = xr * c + xi * s;
  const float i = xi * c - xr * s;
  xr = r;
  xi = i;
}

// In-place radix-2 decimation-in-frequency DFT (kernel exp(-2 pi i nk/R)) over
// v[0], v[S], ..., v[(R-1)S]; output index k ends at position bitrev(k)*S.
template <int R, int S>
MEGA_HD void dif(float* re, float* im) {
  if constexpr (R > 1) {
    constexpr int H = R / 2;
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const float ar = re[i * S], ai = im[i * S];
      const float br = re[(i + H) * S], bi = im[(i + H) * S];
      re[i * S] = ar + br;
      im[i * S] = ai + bi;
      const float dr = ar - br, di = ai - bi;
      float orr, oi;
      if (i == 0) {
        orr = dr;
        oi = di;
      } else if (4 * i == R) {  // -i
        orr = di;
        oi = -dr;
      } else if (8 * i == R) {  // (1 - i)/sqrt2
        orr = (dr + di) * kRsqrt2;
        oi = (di - dr) * kRsqrt2;
      } else if (8 * i == 3 * R) {  // (-1 - i)/sqrt2
        orr = (di - dr) * kRsqrt2;
        oi = -(dr + di) * kRsqrt2;
      } else {
        orr = dr;
        oi = di;
        mul_w<R>(orr, oi, i);
      }
      re[(i + H) * S] = orr;
      im[(i + H) * S] = oi;
    }
    dif<H, S>(re, im);
    dif<H, S>(re + H * S, im + H * S);
  }
}

// Transpose of dif: input index k at position bitrev(k)*S, output natural order.
template <int R, int S>
MEGA_HD void dit(float* re, float* im) {
  if constexpr (R > 1) {
    constexpr int H = R / 2;
    dit<H, S>(re, im);
    dit<H, S>(re + H * S, im + H * S);
#pragma unroll
    for (int i = 0; i < H; ++i) {
      const float ar = re[i * S], ai = im[i * S];
      float br = re[(i + H) * S], bi = im[(i + H) * S];
      if (i == 0) {
      } else if (4 * i == R) {
        const float t = br;
        br = bi;
        bi = -t;
      } else if (8 * i == R) {
        const float t = (br + bi) * kRsqrt2;
        bi = (bi - br) * kRsqrt2;
        br = t;
      } else if (8 * i == 3 * R) {
        const float t = (bi - br) * kRsqrt2;
        bi = -(br + bi) * kRsqrt2;
        br = t;
      } else {
        mul_w<R>(br, bi, i);
      }
      re[i * S] = ar + br;
      im[i * S] = ai + bi;
      re[(i + H) * S] = ar - br;
      im[(i + H) * S] = ai - bi;
    }
  }
}

// V[a] = sum_n v[n] W_64^(n (2a+1)), n, a < 32 (odd bins of a 64-point DFT of
// v padded with zeros).  Natural input; V[a] ends at position bitrev5(a).
MEGA_HD void shifted_dif32(float* re, float* im) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float ar = re[i], ai = im[i], br = re[i + 16], bi = im[i + 16];
    // g = W_64^i (a - i b), h = W_64^(3i) (a + i b)
    float gr = ar + bi, gi = ai - br;
    float hr = ar - bi, hi = ai + br;
    if (i != 0) {
      mul_w<64>(gr, gi, i);
      mul_w<64>(hr, hi, 3 * i);
    }
    re[i] = gr;
    im[i] = gi;
    re[i + 16] = hr;
    im[i + 16] = hi;
  }
  dif<16, 1>(re, im);
  dif<16, 1>(re + 16, im + 16);
}

// P[n] = sum_a u[a] W_64^((2a+1) n), the transpose of shifted_dif32.  Natural
// input; P[n] ends at position 2*bitrev4(n) for n < 16 and 1 + 2*bitrev4(n-16)
// otherwise.
MEGA_HD void shifted_dit32(float* re, float* im) {
  dif<16, 2>(re, im);          // G over even a
  dif<16, 2>(re + 1, im + 1);  // H over odd a
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int pg = 2 * bitrev<4>(i), ph = pg + 1;
    float gr = re[pg], gi = im[pg], hr = re[ph], hi = im[ph];
    if (i != 0) {
      mul_w<64>(gr, gi, i);
      mul_w<64>(hr, hi, 3 * i);
    }
    re[pg] = gr + hr;
    im[pg] = gi + hi;
    const float dr = gr - hr, di = gi - hi;  // P[i+16] = -i (g - h)
    re[ph] = di;
    im[ph] = -dr;
  }
}
MEGA_HD constexpr int shifted_dit32_pos(int n) {
  return n < 16 ? 2 * bitrev<4>(n) : 1 + 2 * bitrev<4>(n - 16);
}

// ---------------------------------------------------------------------------
template <int LOGM>
struct Cfg {
  static constexpr int M = 1 << LOGM;       // complex points of one half
  static constexpr int T = M / 32;          // lanes per workgroup
  static constexpr int R3 = M / 1024;       // radix of the third pass
  static constexpr int NSLOT = 16 / R3;     // residue pairs per lane
  static constexpr int LD1 = T + R3;        // row pitch of exchange 1 (floats)
  static constexpr int LD2 = R3 + (R3 >= 4 ? 2 : 0);  // pitch of exchange 2
  static constexpr int PLANE = (32 * LD1 > 1024 * LD2) ? 32 * LD1 : 1024 * LD2;
  static constexpr int TABLE = 4 * T + R3 + 96 + 2048;  // c32 entries
  static_assert(LOGM >= 11 && LOGM <= 14, "M must be 2048..16384");
};

// Per-lane twiddle seeds for one M (device memory, W_X^k = exp(-2 pi i k / X)).
// Every twiddle of a pass is a geometric sequence base * ratio^k whose base
// and ratio depend only on the lane, so a pass loads two seeds and generates
// the rest with multiplications instead of 31 dependent table loads.
//   kr[t]   = W_M^t                      ratio, forward pass 1 (t = lane)
//   kbo[t]  = W_N^t                      base,  forward pass 1, odd half
//   kp2[n0] = W_T^n0                     ratio, forward pass 2
//   ki3[a1] = W_T^a1                     ratio, inverse pass 3
//   kbe[t]  = W_M^(n0 a2)                base,  inverse pass 2, even (t = a2*R3 + n0)
//   kre[a2] = W_M^(R3 a2)                ratio, inverse pass 2, even
//   kbo2[t] = W_N^(n0 (2 a2 + 1))        base,  inverse pass 2, odd
//   kro[a2] = W_N^(R3 (2 a2 + 1))        ratio, inverse pass 2, odd
//   pw[h*1024 + c] = W_N^(2c + h)        pointwise twiddle
struct Tables {
  const c32* kr;
  const c32* kbo;
  const c32* kp2;
  const c32* ki3;
  const c32* kbe;
  const c32* kre;
  const c32* kbo2;
  const c32* kro;
  const c32* pw;
};

template <int LOGM>
MEGA_HD Tables make_tables(const c32* base) {
  using C = Cfg<LOGM>;
  Tables tb;
  tb.kr = base;
  tb.kbo = tb.kr + C::T;
  tb.kbe = tb.kbo + C::T;
  tb.kbo2 = tb.kbe + C::T;
  tb.kp2 = tb.kbo2 + C::T;
  tb.ki3 = tb.kp2 + C::R3;
  tb.kre = tb.ki3 + 32;
  tb.kro = tb.kre + 32;
  tb.pw = tb.kro + 32;
  return tb;
}

// Host-side fill of the seed table (float64 trigonometry, exact argument reduction).
template <int LOGM>
inline void fill_tables(c32* out) {
  using C = Cfg<LOGM>;
  const double N = 2.0 * C::M;
  auto w = [](double num, double den) {
    const double fr = __builtin_fmod(num, den) / den;
    const double a = -6.283185307179586476925286766559 * fr;
    return c32{static_cast<float>(__builtin_cos(a)), static_cast<float>(__builtin_sin(a))};
  };
  c32* p = out;
  for (int t = 0; t < C::T; ++t) *p++ = w(t, C::M);
  for (int t = 0; t < C::T; ++t) *p++ = w(t, N);
  for (int t = 0; t < C::T; ++t) *p++ = w(static_cast<double>(t % C::R3) * (t / C::R3), C::M);
  for (int t = 0; t < C::T; ++t) *p++ = w(static_cast<double>(t % C::R3) * (2 * (t / C::R3) + 1), N);
  for (int n0 = 0; n0 < C::R3; ++n0) *p++ = w(n0, C::T);
  for (int a1 = 0; a1 < 32; ++a1) *p++ = w(a1, C::T);
  for (int a2 = 0; a2 < 32; ++a2) *p++ = w(static_cast<double>(C::R3) * a2, C::M);
  for (int a2 = 0; a2 < 32; ++a2) *p++ = w(static_cast<double>(C::R3) * (2 * a2 + 1), N);
  for (int h = 0; h < 2; ++h)
    for (int c = 0; c < 1024; ++c) *p++ = w(2.0 * c + h, N);
}

// table[idx] addressed as uniform base + 32-bit unsigned byte offset (lets the
// compiler use the scalar-base addressing form instead of a 64-bit lane address)
MEGA_HD c32 ldc(const c32* base, unsigned idx) {
  return *reinterpret_cast<const c32*>(reinterpret_cast<const char*>(base) + idx * 8u);
}

MEGA_HD c32 cmulv(c32 a, c32 b) { return c32{a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x}; }
MEGA_HD c32 csqv(c32 a) { return c32{a.x * a.x - a.y * a.y, 2.f * a.x * a.y}; }
MEGA_HD c32 conjv(c32 a) { return c32{a.x, -a.y}; }

// Calls f(k, base * r^k) for k = 0..COUNT-1.  Powers are built in blocks of 8
// (block seeds by r^8, then a chain of 7), so no twiddle is more than 10
// multiplications away from a table value.
template <int COUNT, typename F>
MEGA_HD void geo_twiddles(c32 base, c32 r, F&& f) {
  const c32 r8 = csqv(csqv(csqv(r)));
  c32 blk = base;
#pragma unroll
  for (int a = 0; a < COUNT; a += 8) {
    c32 s = blk;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      if (a + b < COUNT) {
        f(a + b, s);
        if (b + 1 < 8 && a + b + 1 < COUNT) s = cmulv(s, r);
      }
    }
    if (a + 8 < COUNT) blk = cmulv(blk, r8);
  }
}

MEGA_HD void cmul_ip(float& xr, float& xi, c32 w) {
  const float r = xr * w.x - xi * w.y;
  xi = xr * w.y + xi * w.x;
  xr = r;
}
MEGA_HD void cmulc_ip(float& xr, float& xi, c32 w) {  // times conj(w)
  const float r = xr * w.x + xi * w.y;
  xi = xi * w.x - xr * w.y;
  xr = r;
}

// residues of slot s for half H
template <int H>
MEGA_HD void slot_residues(int s, int& c0, int& c1) {
  if (H == 0) {
    c0 = s;
    c1 = s == 0 ? 512 : 1024 - s;
  } else {
    c0 = s;
    c1 = 1023 - s;
  }
}

// ------------------------------ forward ------------------------------------
// F1: pass 1 on natural-order input v[j] = z[t + T j]; leaves the twiddled
// outputs in registers (output a2 at position bitrev5(a2)).
template <int LOGM, int H>
MEGA_HD void fwd_pass1(float* re, float* im, int t, const Tables& tb) {
  const c32 r = ldc(tb.kr, t);
  const c32 base = H == 0 ? c32{1.f, 0.f} : ldc(tb.kbo, t);
  if (H == 0) dif<32, 1>(re, im); else shifted_dif32(re, im);
  // W_M^(t a2) (even) or W_N^(t (2 a2 + 1)) = W_N^t (W_M^t)^a2 (odd)
  geo_twiddles<32>(base, r, [&](int a2, c32 w) {
    if (H == 0 && a2 == 0) return;
    const int pos = bitrev<5>(a2);
    cmul_ip(re[pos], im[pos], w);
  });
}
template <int LOGM>
MEGA_HD void x1_write(const float* re, const float* im, int t, float* lre, float* lim) {
  using C = Cfg<LOGM>;
#pragma unroll
  for (int a2 = 0; a2 < 32; ++a2) {
    const int pos = bitrev<5>(a2);
    lre[a2 * C::LD1 + t] = re[pos];
    lim[a2 * C::LD1 + t] = im[pos];
  }
}
// lane (a2', n0') = (t / R3, t % R3) gathers n1 = 0..31
template <int LOGM>
MEGA_HD void x1_read(float* re, float* im, int t, const float* lre, const float* lim) {
  using C = Cfg<LOGM>;
  const int a2p = t / C::R3, n0p = t % C::R3;
#pragma unroll
  for (int n1 = 0; n1 < 32; ++n1) {
    re[n1] = lre[a2p * C::LD1 + n1 * C::R3 + n0p];
    im[n1] = lim[a2p * C::LD1 + n1 * C::R3 + n0p];
  }
}
template <int LOGM>
MEGA_HD void fwd_pass2(float* re, float* im, int t, const Tables& tb) {
  using C = Cfg<LOGM>;
  const c32 r = ldc(tb.kp2, t % C::R3);  // W_T^n0'
  dif<32, 1>(re, im);
  geo_twiddles<32>(c32{1.f, 0.f}, r, [&](int a1, c32 w) {
    if (a1 == 0) return;
    const int pos = bitrev<5>(a1);
    cmul_ip(re[pos], im[pos], w);
  });
}
// element (a2', a1, n0') goes to residue c = a2' + 32 a1
template <int LOGM>
MEGA_HD void x2_write(const float* re, const float* im, int t, float* lre, float* lim) {
  using C = Cfg<LOGM>;
  const int a2p = t / C::R3, n0p = t % C::R3;
#pragma unroll
  for (int a1 = 0; a1 < 32; ++a1) {
    const int pos = bitrev<5>(a1);
    const int c = a2p + 32 * a1;
    lre[c * C::LD2 + n0p] = re[pos];
    lim[c * C::LD2 + n0p] = im[pos];
  }
}
// register index of (slot u, member w, element e)
template <int LOGM>
MEGA_HD constexpr int sidx(int u, int w, int e) {
  return (u * 2 + w) * Cfg<LOGM>::R3 + e;
}
template <int LOGM, int H>
MEGA_HD void x2_read(float* re, float* im, int t, const float* lre, const float* lim) {
  using C = Cfg<LOGM>;
#pragma unroll
  for (int u = 0; u < C::NSLOT; ++u) {
    int c[2];
    slot_residues<H>(t + C::T * u, c[0], c[1]);
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const f2* pr = reinterpret_cast<const f2*>(lre + c[w] * C::LD2);
      const f2* pi = reinterpret_cast<const f2*>(lim + c[w] * C::LD2);
#pragma unroll
      for (int e = 0; e < C::R3 / 2; ++e) {
        const f2 a = pr[e], b = pi[e];
        re[sidx<LOGM>(u, w, 2 * e)] = a.x;
        re[sidx<LOGM>(u, w, 2 * e + 1)] = a.y;
        im[sidx<LOGM>(u, w, 2 * e)] = b.x;
        im[sidx<LOGM>(u, w, 2 * e + 1)] = b.y;
      }
    }
  }
}
// pass 3: bin a0 of (u, w) ends at register sidx(u, w, bitrev(a0))
template <int LOGM>
MEGA_HD void fwd_pass3(float* re, float* im) {
  using C = Cfg<LOGM>;
#pragma unroll
  for (int g = 0; g < 2 * C::NSLOT; ++g) dif<C::R3, 1>(re + g * C::R3, im + g * C::R3);
}

// ------------------------------ pointwise ----------------------------------
// One conjugate pair of bins (r, r' = N - r).  (ar, ai) = Za[r], (apr, api) =
// Za[r'], same for b; w = W_N^r.  Returns Zy[r] in (ar, ai), Zy[r'] in (apr, api).
MEGA_HD void pair_product(float& ar, float& ai, float& apr, float& api, float br, float bi,
                          float bpr, float bpi, float wr, float wi) {
  // 2E = Z[r] + conj Z[r'];  2O = -i (Z[r] - conj Z[r'])
  const float ear = ar + apr, eai = ai - api;
  const float oar = ai + api, oai = apr - ar;
  const float ebr = br + bpr, ebi = bi - bpi;
  const float obr = bi + bpi, obi = bpr - br;
  // t = Oa Ob
  const float tr = oar * obr - oai * obi, ti = oar * obi + oai * obr;
  // Ey = Ea Eb + w t
  float eyr = ear * ebr - eai * ebi, eyi = ear * ebi + eai * ebr;
  eyr += wr * tr - wi * ti;
  eyi += wr * ti + wi * tr;
  // Oy = Ea Ob + Oa Eb
  const float oyr = ear * obr - eai * obi + oar * ebr - oai * ebi;
  const float oyi = ear * obi + eai * obr + oar * ebi + oai * ebr;
  ar = eyr - oyi;
  ai = eyi + oyr;
  apr = eyr + oyi;
  api = oyr - eyi;
}

// a (in flight) times parked b, both in pass-3 register layout; result Zy in a.
template <int LOGM, int H>
MEGA_HD void pointwise(float* re, float* im, const float* bre, const float* bim, int t,
                       const Tables& tb) {
  using C = Cfg<LOGM>;
  constexpr int R3 = C::R3;
  constexpr int LR = ilog2(R3);
#pragma unroll
  for (int u = 0; u < C::NSLOT; ++u) {
    const int s = t + C::T * u;
    const bool self = (H == 0) && (u == 0) && (s == 0);
    if (!self) {
      const c32 pw = ldc(tb.pw, H * 1024 + s);  // W_N^(2 c0 + H)
#pragma unroll
      for (int a0 = 0; a0 < R3; ++a0) {
        const int i0 = sidx<LOGM>(u, 0, bitrev<LR>(a0));
        const int i1 = sidx<LOGM>(u, 1, bitrev<LR>(R3 - 1 - a0));
        float wr = pw.x, wi = pw.y;
        if (a0 != 0) mul_w<R3>(wr, wi, a0);
        pair_product(re[i0], im[i0], re[i1], im[i1], bre[i0], bim[i0], bre[i1], bim[i1], wr, wi);
      }
    } else if (u == 0) {
      // slot 0 of the even half: residues 0 and 512 pair with themselves
      float nr[2 * R3], ni[2 * R3];
      const c32 pw512 = ldc(tb.pw, 512);  // W_N^1024
#pragma unroll
      for (int w = 0; w < 2; ++w) {
#pragma unroll
        for (int a0 = 0; a0 < R3; ++a0) {
          const int pa = w == 0 ? (R3 - a0) % R3 : R3 - 1 - a0;
          const int i0 = sidx<LOGM>(0, w, bitrev<LR>(a0));
          const int i1 = sidx<LOGM>(0, w, bitrev<LR>(pa));
          float wr = w == 0 ? 1.f : pw512.x, wi = w == 0 ? 0.f : pw512.y;
          if (a0 != 0) mul_w<R3>(wr, wi, a0);
          float ar = re[i0], ai = im[i0], apr = re[i1], api = im[i1];
          pair_product(ar, ai, apr, api, bre[i0], bim[i0], bre[i1], bim[i1], wr, wi);
          nr[w * R3 + a0] = ar;
          ni[w * R3 + a0] = ai;
        }
      }
#pragma unroll
      for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int a0 = 0; a0 < R3; ++a0) {
          re[sidx<LOGM>(0, w, bitrev<LR>(a0))] = nr[w * R3 + a0];
          im[sidx<LOGM>(0, w, bitrev<LR>(a0))] = ni[w * R3 + a0];
        }
    }
  }
}

// ------------------------------ inverse ------------------------------------
// pass 3': inverse radix-R3 over a0 (swapped re/im), then conj pass-2 twiddle
template <int LOGM, int H>
MEGA_HD void inv_pass3(float* re, float* im, int t, const Tables& tb) {
  using C = Cfg<LOGM>;
  c32 rr[2 * C::NSLOT];
#pragma unroll
  for (int u = 0; u < C::NSLOT; ++u) {
    int c[2];
    slot_residues<H>(t + C::T * u, c[0], c[1]);
    rr[2 * u] = conjv(ldc(tb.ki3, c[0] >> 5));
    rr[2 * u + 1] = conjv(ldc(tb.ki3, c[1] >> 5));
  }
#pragma unroll
  for (int g = 0; g < 2 * C::NSLOT; ++g) dit<C::R3, 1>(im + g * C::R3, re + g * C::R3);
#pragma unroll
  for (int g = 0; g < 2 * C::NSLOT; ++g) {
    // conj(W_T^(n0 a1)), a1 = residue >> 5
    geo_twiddles<C::R3>(c32{1.f, 0.f}, rr[g], [&](int n0, c32 w) {
      if (n0 == 0) return;
      const int i = g * C::R3 + n0;
      cmul_ip(re[i], im[i], w);
    });
  }
}
template <int LOGM, int H>
MEGA_HD void ix2_write(const float* re, const float* im, int t, float* lre, float* lim) {
  using C = Cfg<LOGM>;
#pragma unroll
  for (int u = 0; u < C::NSLOT; ++u) {
    int c[2];
    slot_residues<H>(t + C::T * u, c[0], c[1]);
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      f2* pr = reinterpret_cast<f2*>(lre + c[w] * C::LD2);
      f2* pi = reinterpret_cast<f2*>(lim + c[w] * C::LD2);
#pragma unroll
      for (int e = 0; e < C::R3 / 2; ++e) {
        pr[e] = f2{re[sidx<LOGM>(u, w, 2 * e)], re[sidx<LOGM>(u, w, 2 * e + 1)]};
        pi[e] = f2{im[sidx<LOGM>(u, w, 2 * e)], im[sidx<LOGM>(u, w, 2 * e + 1)]};
      }
    }
  }
}
template <int LOGM>
MEGA_HD void ix2_read(float* re, float* im, int t, const float* lre, const float* lim) {
  using C = Cfg<LOGM>;
  const int a2p = t / C::R3, n0p = t % C::R3;
#pragma unroll
  for (int a1 = 0; a1 < 32; ++a1) {
    const int c = a2p + 32 * a1;
    re[a1] = lre[c * C::LD2 + n0p];
    im[a1] = lim[c * C::LD2 + n0p];
  }
}
// pass 2': inverse radix-32 over a1 -> n1 at bitrev5(n1); conj pass-1 twiddle
// conj(W^((n1 R3 + n0') ...)) = conj(base) conj(ratio)^n1
template <int LOGM, int H>
MEGA_HD void inv_pass2(float* re, float* im, int t, const Tables& tb) {
  using C = Cfg<LOGM>;
  const int a2p = t / C::R3;
  const c32 base = conjv(ldc(H == 0 ? tb.kbe : tb.kbo2, t));
  const c32 r = conjv(ldc(H == 0 ? tb.kre : tb.kro, a2p));
  dif<32, 1>(im, re);
  geo_twiddles<32>(base, r, [&](int n1, c32 w) {
    const int pos = bitrev<5>(n1);
    cmul_ip(re[pos], im[pos], w);
  });
}
template <int LOGM>
MEGA_HD void ix1_write(const float* re, const float* im, int t, float* lre, float* lim) {
  using C = Cfg<LOGM>;
  const int a2p = t / C::R3, n0p = t % C::R3;
#pragma unroll
  for (int n1 = 0; n1 < 32; ++n1) {
    const int pos = bitrev<5>(n1);
    lre[a2p * C::LD1 + n1 * C::R3 + n0p] = re[pos];
    lim[a2p * C::LD1 + n1 * C::R3 + n0p] = im[pos];
  }
}
template <int LOGM>
MEGA_HD void ix1_read(float* re, float* im, int t, const float* lre, const float* lim) {
  using C = Cfg<LOGM>;
#pragma unroll
  for (int a2 = 0; a2 < 32; ++a2) {
    re[a2] = lre[a2 * C::LD1 + t];
    im[a2] = lim[a2 * C::LD1 + t];
  }
}
// pass 1': inverse radix-32 over a2; zy[t + T n2] ends at register out_pos<H>(n2)
template <int H>
MEGA_HD void inv_pass1(float* re, float* im) {
  if (H == 0) dif<32, 1>(im, re); else shifted_dit32(im, re);
}
template <int H>
MEGA_HD constexpr int out_pos(int n2) {
  return H == 0 ? bitrev<5>(n2) : shifted_dit32_pos(n2);
}

}  // namespace fftc
}  // namespace mega
