// CEMA convolution-kernel generation for gfx950: w[d,j] = sum_n Re(c_n q_n^j)
// and its backward reductions.
//
// Follows the math of the reference weight path
//   megalodon/csrc/ops/ema_parameters.cc:17-52 (forward), :80-98 (backward)
// with a different evaluation scheme: every power q^j is factored as
// q^(T*h) * q^lo with both factors taken from small per-channel tables whose
// entries are evaluated directly (phase reduced in float64 "turns", so the
// angle j*arg(q) never loses bits for j up to 2^31), instead of the
// reference's repeated multiplication (ema_parameters_kernel.cu:115-117) or
// fp32 exp(log_q*j) (ema_parameters.cc:45-46).
//
// Forward: one workgroup per (channel, 64-tile slab).  Each lane keeps the 4
// (or 2) consecutive low powers q^lo of all N modes in registers, reads the
// per-tile factor c*q^(T*h) from LDS (wave-uniform broadcast) and emits one
// float4 (float2) per tile: 2 FMA per (element, mode), one coalesced store.
//
// Backward: same factorisation turned into per-lane partial sums
//   A[lo] = sum_h dw[h,lo] q^(T h),  B[lo] = sum_h j dw[h,lo] q^(T h)
// followed by one multiplication with q^lo and a workgroup reduction.
#include "common.hpp"
#include "cema_pow.hpp"

namespace mega {
namespace {

constexpr int kThreads = 256;
constexpr int kSlab = 64;  // tiles handled per table fill

template <int NMAX, int PT>
struct LowTables {
  cf p1[NMAX][64];  // q^b, b < 64
  cf p2[NMAX][(kThreads * PT) / 64];  // q^(64 a)
};

template <int NMAX, int PT>
__device__ __forceinline__ void fill_low_tables(LowTables<NMAX, PT>& t, const cf* lq, int N) {
  constexpr int kA = (kThreads * PT) / 64;
  for (int i = threadIdx.x; i < NMAX * 64; i += kThreads) {
    const int n = i >> 6, b = i & 63;
    t.p1[n][b] = n < N ? qpow(lq[n].x, lq[n].y, b) : cf{0.f, 0.f};
  }
  for (int i = threadIdx.x; i < NMAX * kA; i += kThreads) {
    const int n = i / kA, a = i % kA;
    t.p2[n][a] = n < N ? qpow(lq[n].x, lq[n].y, 64 * a) : cf{0.f, 0.f};
  }
}

// ------------------------------ forward ------------------------------------
template <int NMAX, int PT, bool VEC>
__global__ __launch_bounds__(kThreads) void ema_weight_fwd_kernel(
    const float* __restrict__ p, const cf* __restrict__ log_q,
    const cf* __restrict__ gamma, int N, int64_t L, float* __restrict__ w) {
  constexpr int kTile = kThreads * PT;
  __shared__ LowTables<NMAX, PT> low;
  __shared__ cf hi[kSlab][NMAX];  // c_n * q_n^(kTile * h)

  const int64_t d = blockIdx.x;
  const int64_t h0 = static_cast<int64_t>(blockIdx.y) * kSlab;
  const int64_t n_tiles = (L + kTile - 1) / kTile;
  const int nh = static_cast<int>(min<int64_t>(kSlab, n_tiles - h0));
  const cf* lq = log_q + d * N;

  fill_low_tables<NMAX, PT>(low, lq, N);
  for (int i = threadIdx.x; i < nh * NMAX; i += kThreads) {
    const int h = i / NMAX, n = i % NMAX;
    cf v{0.f, 0.f};
    if (n < N) {
      const cf g = gamma[d * N + n];
      const float pp = p[d * N + n];
      v = cmul(cf{pp * g.x, pp * g.y}, qpow(lq[n].x, lq[n].y, (h0 + h) * kTile));
    }
    hi[h][n] = v;
  }
  __syncthreads();

  float qx[PT][NMAX], qny[PT][NMAX];  // Re(q^lo), -Im(q^lo)
#pragma unroll
  for (int r = 0; r < PT; ++r) {
    const int lo = threadIdx.x * PT + r;
#pragma unroll
    for (int n = 0; n < NMAX; ++n) {
      const cf v = cmul(low.p2[n][lo >> 6], low.p1[n][lo & 63]);
      qx[r][n] = v.x;
      qny[r][n] = -v.y;
    }
  }

  float* wrow = w + d * L;
  for (int h = 0; h < nh; ++h) {
    float acc[PT];
#pragma unroll
    for (int r = 0; r < PT; ++r) acc[r] = 0.f;
#pragma unroll
    for (int n = 0; n < NMAX; ++n) {
      const cf t = hi[h][n];
#pragma unroll
      for (int r = 0; r < PT; ++r) {
        acc[r] = fmaf(t.x, qx[r][n], acc[r]);
        acc[r] = fmaf(t.y, qny[r][n], acc[r]);
      }
    }
    const int64_t j0 = (h0 + h) * kTile + static_cast<int64_t>(threadIdx.x) * PT;
    if (VEC && j0 + PT <= L) {
      if constexpr (PT == 4) {
        *reinterpret_cast<float4*>(wrow + j0) = make_float4(acc[0], acc[1], acc[2], acc[3]);
      } else {
        *reinterpret_cast<float2*>(wrow + j0) = make_float2(acc[0], acc[1]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < PT; ++r)
        if (j0 + r < L) wrow[j0 + r] = acc[r];
    }
  }
}

// ------------------------------ backward -----------------------------------
template <int NMAX, int PT, bool VEC>
__global__ __launch_bounds__(kThreads) void ema_weight_bwd_kernel(
    const float* __restrict__ dw, const float* __restrict__ p,
    const cf* __restrict__ log_q, const cf* __restrict__ gamma, int N,
    int64_t L, float* __restrict__ dp, cf* __restrict__ dq,
    cf* __restrict__ dgamma) {
  constexpr int kTile = kThreads * PT;
  __shared__ LowTables<NMAX, PT> low;
  __shared__ cf hi[kSlab][NMAX];                // q_n^(kTile * h)
  __shared__ float red[kThreads / kWave][4 * NMAX];

  const int64_t d = blockIdx.x;
  const cf* lq = log_q + d * N;
  const float* drow = dw + d * L;
  const int64_t n_tiles = (L + kTile - 1) / kTile;

  fill_low_tables<NMAX, PT>(low, lq, N);

  float ax[PT][NMAX], ay[PT][NMAX], bx[PT][NMAX], by[PT][NMAX];
#pragma unroll
  for (int r = 0; r < PT; ++r)
#pragma unroll
    for (int n = 0; n < NMAX; ++n) ax[r][n] = ay[r][n] = bx[r][n] = by[r][n] = 0.f;

  for (int64_t h0 = 0; h0 < n_tiles; h0 += kSlab) {
    const int nh = static_cast<int>(min<int64_t>(kSlab, n_tiles - h0));
    __syncthreads();  // previous slab fully consumed (also orders the low-table fill)
    for (int i = threadIdx.x; i < nh * NMAX; i += kThreads) {
      const int h = i / NMAX, n = i % NMAX;
      hi[h][n] = n < N ? qpow(lq[n].x, lq[n].y, (h0 + h) * kTile) : cf{0.f, 0.f};
    }
    __syncthreads();
    for (int h = 0; h < nh; ++h) {
      const int64_t j0 = (h0 + h) * kTile + static_cast<int64_t>(threadIdx.x) * PT;
      float g[PT];
      if (VEC && PT == 2 && j0 + PT <= L) {
        const float2 v = *reinterpret_cast<const float2*>(drow + j0);
        g[0] = v.x;
        g[PT - 1] = v.y;
      } else {
#pragma unroll
        for (int r = 0; r < PT; ++r) g[r] = j0 + r < L ? drow[j0 + r] : 0.f;
      }
      float gj[PT];
#pragma unroll
      for (int r = 0; r < PT; ++r) gj[r] = g[r] * static_cast<float>(j0 + r);
#pragma unroll
      for (int n = 0; n < NMAX; ++n) {
        const cf t = hi[h][n];
#pragma unroll
        for (int r = 0; r < PT; ++r) {
          ax[r][n] = fmaf(g[r], t.x, ax[r][n]);
          ay[r][n] = fmaf(g[r], t.y, ay[r][n]);
          bx[r][n] = fmaf(gj[r], t.x, bx[r][n]);
          by[r][n] = fmaf(gj[r], t.y, by[r][n]);
        }
      }
    }
  }

  // fold in q^lo, then reduce over the workgroup
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
  for (int n = 0; n < NMAX; ++n) {
    cf s2{0.f, 0.f}, s1{0.f, 0.f};
#pragma unroll
    for (int r = 0; r < PT; ++r) {
      const int lo = threadIdx.x * PT + r;
      const cf ql = cmul(low.p2[n][lo >> 6], low.p1[n][lo & 63]);
      s2 = cadd(s2, cmul(ql, cf{ax[r][n], ay[r][n]}));
      s1 = cadd(s1, cmul(ql, cf{bx[r][n], by[r][n]}));
    }
    const float v0 = wave_sum(s2.x), v1 = wave_sum(s2.y);
    const float v2 = wave_sum(s1.x), v3 = wave_sum(s1.y);
    if (lane == 0) {
      red[wave][4 * n + 0] = v0;
      red[wave][4 * n + 1] = v1;
      red[wave][4 * n + 2] = v2;
      red[wave][4 * n + 3] = v3;
    }
  }
  __syncthreads();
  if (threadIdx.x < N) {
    const int n = threadIdx.x;
    cf s2{0.f, 0.f}, s1q{0.f, 0.f};
#pragma unroll
    for (int wv = 0; wv < kThreads / kWave; ++wv) {
      s2.x += red[wv][4 * n + 0];
      s2.y += red[wv][4 * n + 1];
      s1q.x += red[wv][4 * n + 2];
      s1q.y += red[wv][4 * n + 3];
    }
    // S1 = sum_j j dw_j q^(j-1) = (sum_j j dw_j q^j) / q
    const cf s1 = cmul(s1q, qpow(lq[n].x, lq[n].y, -1));
    const cf g = gamma[d * N + n];
    const float pp = p[d * N + n];
    dp[d * N + n] = s2.x * g.x - s2.y * g.y;
    const cf t = cmul(s1, cf{pp * g.x, pp * g.y});
    dq[d * N + n] = cf{t.x, -t.y};
    dgamma[d * N + n] = cf{s2.x * pp, -s2.y * pp};
  }
}


// ---- backward on the matrix cores (N <= 16) -----------------------------------
// With j = 64 lo + h the two sums over the row become one small GEMM per channel,
//   C[lo][.] = sum_h dw[64 lo + h] * Q[h][.],  Q[h] = (q_n^h, h q_n^h) for the 16 modes,
// followed by a weighted column sum with q_n^(64 lo):
//   S2 = sum_lo q^(64 lo) A[lo],   sum_j j dw_j q^j = sum_lo q^(64 lo) (64 lo A[lo] + B[lo]).
// The products run as bf16 MFMAs with both operands split into high and low
// halves (hi*hi + hi*lo + lo*hi): 16 significant bits per factor, fp32
// accumulation, which keeps the fp32 tolerance of the operator.
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ floatx16 mfma_bf16(u32x4 a, u32x4 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
// 8 floats -> packed bf16 high parts and packed bf16 residuals
__device__ __forceinline__ void split8(const float* v, u32x4& hi, u32x4& lo) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t h = pack_bf16x2(v[2 * e], v[2 * e + 1]);
    const float r0 = v[2 * e] - __uint_as_float(h << 16);
    const float r1 = v[2 * e + 1] - __uint_as_float(h & 0xffff0000u);
    hi[e] = h;
    lo[e] = pack_bf16x2(r0, r1);
  }
}

// ---- forward on the matrix cores (N <= 16) ------------------------------------
// With j = 1024 h + lo the kernel row of a channel is a small GEMM,
//   w[1024 h + lo] = sum_c T[h][c] Q[lo][c],  c = 2 n + part,
//   T[h] = (Re, Im)(c_n q_n^(1024 h)),  Q[lo] = (Re, -Im)(q_n^lo),
// 32 rows h x 1024 columns lo x 32 values c per workgroup: the VALU version
// spends 2 FMA per (element, mode) and is bound by them, this one by its
// stores.  Same split-bf16 products as the backward kernel.
__global__ __launch_bounds__(kThreads) void ema_weight_fwd_mfma_kernel(
    const float* __restrict__ p, const cf* __restrict__ log_q, const cf* __restrict__ gamma, int N,
    int64_t L, float* __restrict__ w) {
  __shared__ LowTables<16, 4> low;  // q^b (b < 64), q^(64 a) (a < 16)
  __shared__ cf hi[32][16];         // c_n q_n^(1024 h) for the 32 rows of this workgroup
  const int64_t d = blockIdx.x;
  const int64_t h0 = static_cast<int64_t>(blockIdx.y) * 32;
  const cf* lq = log_q + d * N;
  fill_low_tables<16, 4>(low, lq, N);
  for (int i = threadIdx.x; i < 32 * 16; i += kThreads) {
    const int h = i >> 4, n = i & 15;
    cf v{0.f, 0.f};
    if (n < N && (h0 + h) * 1024 < L) {
      const cf g = gamma[d * N + n];
      const float pp = p[d * N + n];
      v = cmul(cf{pp * g.x, pp * g.y}, qpow(lq[n].x, lq[n].y, (h0 + h) * 1024));
    }
    hi[h][n] = v;
  }
  __syncthreads();

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane >> 5, col = lane & 31;
  // A operand: lane <-> row h = col, k = c = 16 s + 8 g + e  ->  modes 8 s + 4 g + e / 2
  u32x4 ahi[2], alo[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    float v[8];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const cf t = hi[col][8 * s + 4 * g + m];
      v[2 * m] = t.x;
      v[2 * m + 1] = t.y;
    }
    split8(v, ahi[s], alo[s]);
  }
  float* wrow = w + d * L + h0 * 1024;
  const int64_t left = L - h0 * 1024;  // samples of this workgroup's rows
  for (int lt = wave; lt < 32; lt += kThreads / kWave) {
    const int lo = 32 * lt + col;
    u32x4 bhi[2], blo[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      float v[8];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int n = 8 * s + 4 * g + m;
        const cf q = cmul(low.p2[n][lo >> 6], low.p1[n][lo & 63]);
        v[2 * m] = q.x;
        v[2 * m + 1] = -q.y;
      }
      split8(v, bhi[s], blo[s]);
    }
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      acc = mfma_bf16(ahi[s], bhi[s], acc);
      acc = mfma_bf16(ahi[s], blo[s], acc);
      acc = mfma_bf16(alo[s], bhi[s], acc);
    }
    // result: lane <-> column lo, register r <-> row h = 8 (r / 4) + 4 g + r % 4
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int64_t j = static_cast<int64_t>(8 * (r >> 2) + 4 * g + (r & 3)) * 1024 + lo;
      if (j < left) wrow[j] = acc[r];
    }
  }
}

__global__ __launch_bounds__(kThreads) void ema_weight_bwd_mfma_kernel(
    const float* __restrict__ dw, const float* __restrict__ p, const cf* __restrict__ log_q,
    const cf* __restrict__ gamma, int N, int64_t L, float* __restrict__ dp, cf* __restrict__ dq,
    cf* __restrict__ dgamma) {
  __shared__ float red[kThreads][4];
  __shared__ u32x4 qop[4][4][kWave];  // [k-step][re hi, re lo, im hi, im lo][lane]
  static_assert(kThreads / kWave == 4, "one wave per k-step of the B operand");
  const int64_t d = blockIdx.x;
  const cf* lq = log_q + d * N;
  const float* drow = dw + d * L;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int g = lane >> 5, col = lane & 31;
  const int n = col & 15, kind = col >> 4;  // kind 0: q^h, kind 1: h q^h
  const bool live = n < N;
  const float la = live ? lq[n].x : 0.f, lphi = live ? lq[n].y : 0.f;

  const int64_t rows = (L + 63) / 64;
  const int64_t mtiles = (rows + 31) / 32;
  auto load_tile = [&](int64_t mt, float (*raw)[8]) {
    const int64_t j0 = (32 * mt + col) * 64 + 8 * g;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int64_t j = j0 + 16 * s;
      if (j + 8 <= L) {
        const float4 u = *reinterpret_cast<const float4*>(drow + j);
        const float4 v = *reinterpret_cast<const float4*>(drow + j + 4);
        raw[s][0] = u.x; raw[s][1] = u.y; raw[s][2] = u.z; raw[s][3] = u.w;
        raw[s][4] = v.x; raw[s][5] = v.y; raw[s][6] = v.z; raw[s][7] = v.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) raw[s][e] = j + e < L ? drow[j + e] : 0.f;
      }
    }
  };

  // the first tile's loads fly while the operand below is built (a second
  // tile in flight per wave costs the third workgroup per CU and runs 6 % slower)
  float raw[4][8];
  if (wave < mtiles) load_tile(wave, raw);

  // B operand: lane <-> column (kind, n), k = h = 16 s + 8 g + e; real and
  // imaginary parts are the two 32-column tiles.  It is the same for the four
  // waves: wave s builds k-step s and the operand lives in LDS (64 registers
  // less per lane, one more workgroup per CU).
  {
    const int s = wave;
    const cf q1 = qpow(la, lphi, 1);
    float vr[8], vi[8];
    cf v = qpow(la, lphi, 16 * s + 8 * g);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sc = !live ? 0.f : (kind ? static_cast<float>(16 * s + 8 * g + e) : 1.f);
      vr[e] = v.x * sc;
      vi[e] = v.y * sc;
      v = cmul(v, q1);
    }
    u32x4 rh, rl, ih, il;
    split8(vr, rh, rl);
    split8(vi, ih, il);
    qop[s][0][lane] = rh;
    qop[s][1][lane] = rl;
    qop[s][2][lane] = ih;
    qop[s][3][lane] = il;
  }
  __syncthreads();
  // q^(64 lo) for the rows a lane meets: lo = 32 mt + 8 qd + 4 g + e
  const cf st1 = qpow(la, lphi, 64), st2 = cmul(st1, st1), st3 = cmul(st2, st1);
  const cf st8 = qpow(la, lphi, 512);

  cf s2{0.f, 0.f}, s1{0.f, 0.f};

  for (int64_t mt = wave; mt < mtiles; mt += kThreads / kWave) {
    u32x4 ahi[4], alo[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) split8(raw[s], ahi[s], alo[s]);
    if (mt + kThreads / kWave < mtiles) load_tile(mt + kThreads / kWave, raw);  // next tile in flight
    floatx16 cr, ci;
#pragma unroll
    for (int r = 0; r < 16; ++r) cr[r] = ci[r] = 0.f;
    // re-read per tile: left to itself the compiler hoists these 64 registers
    // out of the loop again
    int ql = lane;
    asm volatile("" : "+v"(ql));
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const u32x4 qre_hi = qop[s][0][ql], qre_lo = qop[s][1][ql];
      const u32x4 qim_hi = qop[s][2][ql], qim_lo = qop[s][3][ql];
      cr = mfma_bf16(ahi[s], qre_hi, cr);
      ci = mfma_bf16(ahi[s], qim_hi, ci);
      cr = mfma_bf16(ahi[s], qre_lo, cr);
      ci = mfma_bf16(ahi[s], qim_lo, ci);
      cr = mfma_bf16(alo[s], qre_hi, cr);
      ci = mfma_bf16(alo[s], qim_hi, ci);
    }
    // result: lane <-> column, register r <-> row lo = 32 mt + 8 (r / 4) + 4 g + r % 4
    const int64_t lo0 = 32 * mt + 4 * g;
    cf qq = qpow(la, lphi, 64 * lo0);
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
      const cf w4[4] = {qq, cmul(qq, st1), cmul(qq, st2), cmul(qq, st3)};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * qd + e;
        const cf t = cmul(w4[e], cf{cr[r], ci[r]});
        const float jlo = static_cast<float>(64 * (lo0 + 8 * qd + e));
        const float c2 = kind ? 0.f : 1.f, c1 = kind ? 1.f : jlo;
        s2.x = fmaf(c2, t.x, s2.x);
        s2.y = fmaf(c2, t.y, s2.y);
        s1.x = fmaf(c1, t.x, s1.x);
        s1.y = fmaf(c1, t.y, s1.y);
      }
      qq = cmul(qq, st8);
    }
  }
  red[threadIdx.x][0] = s2.x;
  red[threadIdx.x][1] = s2.y;
  red[threadIdx.x][2] = s1.x;
  red[threadIdx.x][3] = s1.y;
  __syncthreads();
  if (threadIdx.x < N) {
    const int m = threadIdx.x;
    cf t2{0.f, 0.f}, s1q{0.f, 0.f};
    for (int wv = 0; wv < kThreads / kWave; ++wv)
      for (int c = 0; c < 4; ++c) {
        const float* r = red[wv * kWave + m + 16 * c];
        t2.x += r[0];
        t2.y += r[1];
        s1q.x += r[2];
        s1q.y += r[3];
      }
    // S1 = sum_j j dw_j q^(j-1) = (sum_j j dw_j q^j) / q
    const cf sq = cmul(s1q, qpow(lq[m].x, lq[m].y, -1));
    const cf gm = gamma[d * N + m];
    const float pp = p[d * N + m];
    dp[d * N + m] = t2.x * gm.x - t2.y * gm.y;
    const cf t = cmul(sq, cf{pp * gm.x, pp * gm.y});
    dq[d * N + m] = cf{t.x, -t.y};
    dgamma[d * N + m] = cf{t2.x * pp, -t2.y * pp};
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_ema_weight_fwd(const float* p, const float* log_q,
                                   const float* gamma, int64_t D, int64_t N,
                                   int64_t L, float* w, void* stream) {
  MEGA_CHECK_ARG(p && log_q && gamma && w, "mega_ema_weight_fwd: null pointer");
  MEGA_CHECK_ARG(D >= 0 && L >= 0, "mega_ema_weight_fwd: negative size");
  MEGA_CHECK_ARG(N >= 1 && N <= 32, "mega_ema_weight_fwd: N=%lld outside [1,32]", (long long)N);
  MEGA_CHECK_ARG(D <= 0x7fffffff, "mega_ema_weight_fwd: D too large");
  if (D == 0 || L == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const cf* lq = reinterpret_cast<const cf*>(log_q);
  const cf* gm = reinterpret_cast<const cf*>(gamma);
  const bool vec = (L % 4 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0);
  if (N <= 16 && (L + 1023) / 1024 <= 32 * 65535) {
    const int64_t hrows = (L + 1023) / 1024;
    dim3 grid(static_cast<unsigned>(D), static_cast<unsigned>((hrows + 31) / 32));
    ema_weight_fwd_mfma_kernel<<<grid, kThreads, 0, s>>>(p, lq, gm, (int)N, L, w);
  } else if (N <= 16) {
    constexpr int kTile = kThreads * 4;
    const int64_t tiles = (L + kTile - 1) / kTile;
    dim3 grid(static_cast<unsigned>(D), static_cast<unsigned>((tiles + kSlab - 1) / kSlab));
    if (vec)
      ema_weight_fwd_kernel<16, 4, true><<<grid, kThreads, 0, s>>>(p, lq, gm, (int)N, L, w);
    else
      ema_weight_fwd_kernel<16, 4, false><<<grid, kThreads, 0, s>>>(p, lq, gm, (int)N, L, w);
  } else {
    constexpr int kTile = kThreads * 2;
    const int64_t tiles = (L + kTile - 1) / kTile;
    dim3 grid(static_cast<unsigned>(D), static_cast<unsigned>((tiles + kSlab - 1) / kSlab));
    if (vec)
      ema_weight_fwd_kernel<32, 2, true><<<grid, kThreads, 0, s>>>(p, lq, gm, (int)N, L, w);
    else
      ema_weight_fwd_kernel<32, 2, false><<<grid, kThreads, 0, s>>>(p, lq, gm, (int)N, L, w);
  }
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

extern "C" int mega_ema_weight_bwd(const float* dw, const float* p,
                                   const float* log_q, const float* gamma,
                                   int64_t D, int64_t N, int64_t L, float* dp,
                                   float* dq, float* dgamma, void* stream) {
  MEGA_CHECK_ARG(dw && p && log_q && gamma && dp && dq && dgamma,
                 "mega_ema_weight_bwd: null pointer");
  MEGA_CHECK_ARG(D >= 0 && L >= 0, "mega_ema_weight_bwd: negative size");
  MEGA_CHECK_ARG(N >= 1 && N <= 32, "mega_ema_weight_bwd: N=%lld outside [1,32]", (long long)N);
  MEGA_CHECK_ARG(D <= 0x7fffffff, "mega_ema_weight_bwd: D too large");
  MEGA_CHECK_ARG(L <= 0x7fffffff, "mega_ema_weight_bwd: L too large");
  if (D == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const cf* lq = reinterpret_cast<const cf*>(log_q);
  const cf* gm = reinterpret_cast<const cf*>(gamma);
  cf* dqc = reinterpret_cast<cf*>(dq);
  cf* dgc = reinterpret_cast<cf*>(dgamma);
  const bool vec = (L % 2 == 0) && (reinterpret_cast<uintptr_t>(dw) % 8 == 0);
  dim3 grid(static_cast<unsigned>(D));
  if (N <= 16 && L >= 1 && reinterpret_cast<uintptr_t>(dw) % 16 == 0 && L % 4 == 0) {
    ema_weight_bwd_mfma_kernel<<<grid, kThreads, 0, s>>>(dw, p, lq, gm, (int)N, L, dp, dqc, dgc);
  } else if (N <= 16) {
    if (vec)
      ema_weight_bwd_kernel<16, 2, true><<<grid, kThreads, 0, s>>>(dw, p, lq, gm, (int)N, L, dp, dqc, dgc);
    else
      ema_weight_bwd_kernel<16, 2, false><<<grid, kThreads, 0, s>>>(dw, p, lq, gm, (int)N, L, dp, dqc, dgc);
  } else {
    ema_weight_bwd_kernel<32, 1, false><<<grid, kThreads, 0, s>>>(dw, p, lq, gm, (int)N, L, dp, dqc, dgc);
  }
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}
