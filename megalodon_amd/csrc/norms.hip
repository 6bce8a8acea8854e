// LayerNorm / RMSNorm over the last axis with the reference's parameterisation:
// the stored weight is gamma - 1 (megalodon/modules/layer_norm.py:14-66 adds 1
// before calling apex's fused_layer_norm_cuda, which is not part of the
// reference tree).  y = (x - mean) * rstd * (weight + 1) + bias with biased
// variance and rstd = 1 / sqrt(var + eps); RMSNorm drops the mean and the bias
// and uses mean(x^2).  Rows are independent, so the kernels are streaming:
// a row (or 2-4 short rows) sits in the registers of one wavefront, x is read
// once and y written once; the backward reads x and dy once, writes dx once and
// leaves per-workgroup column sums for the parameter gradients, which a second
// small kernel reduces in a fixed order (no float atomics).
#include "common.hpp"

namespace mega {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxGroups = 1024;  // workgroups of the backward = partial-sum rows


// hides a register from common-subexpression elimination: values derived from it
// afterwards are recomputed instead of being kept alive across the row reduction
__device__ __forceinline__ void opaque(uint4& q) {
  asm volatile("" : "+v"(q.x), "+v"(q.y), "+v"(q.z), "+v"(q.w));
}

struct NormParams {
  const void* x;
  const void* dy;
  const void* weight;  // gamma - 1, may be null (gamma = 1)
  const void* bias;    // may be null
  void* y;             // forward: y, backward: dx
  float* mean;         // per row (unused for RMS)
  float* rstd;         // per row
  float* part_w;       // backward: (groups, D) partial sums of dy * xhat
  float* part_b;       // backward: (groups, D) partial sums of dy
  int64_t rows;
  int D;
  float eps;
};

// ---- rows in registers: D = LPR * 8 * NCH, 64 / LPR rows per wavefront --------
template <int DT, int LPR, int NCH, bool RMS>
__global__ __launch_bounds__(kThreads) void norm_fwd_vec_kernel(NormParams p) {
  constexpr int RPW = kWave / LPR;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lr = lane % LPR, slot = lane / LPR;
  const uint16_t* x = static_cast<const uint16_t*>(p.x);
  uint16_t* y = static_cast<uint16_t*>(p.y);
  const float inv_d = 1.f / static_cast<float>(p.D);
  // weight and bias stay packed (one register per element pair)
  uint4 gq[NCH], bq[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = (lr + LPR * i) * 8;
    gq[i] = make_uint4(0, 0, 0, 0);
    bq[i] = make_uint4(0, 0, 0, 0);
    if (p.weight) gq[i] = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p.weight) + c);
    if (!RMS && p.bias) bq[i] = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p.bias) + c);
  }
  const int64_t step = static_cast<int64_t>(gridDim.x) * kWaves * RPW;
  for (int64_t row = (static_cast<int64_t>(blockIdx.x) * kWaves + wave) * RPW + slot;
       row - slot < p.rows; row += step) {
    const bool live = row < p.rows;
    float v[NCH][8];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      uint4 q = make_uint4(0, 0, 0, 0);
      if (live) q = *reinterpret_cast<const uint4*>(x + row * p.D + (lr + LPR * i) * 8);
      unpack8<DT>(q, v[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += RMS ? v[i][e] * v[i][e] : v[i][e];
    }
    s = group_sum<LPR>(s) * inv_d;
    float mu = 0.f, var = s;
    if (!RMS) {
      mu = s;
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[i][e] -= mu;
          ss += v[i][e] * v[i][e];
        }
      var = group_sum<LPR>(ss) * inv_d;
    }
    const float r = rsqrtf(var + p.eps);
    if (live) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        float g[8], b[8];
        opaque(gq[i]);  // unpacked per row, not hoisted out of the row loop
        unpack8<DT>(gq[i], g);
        if (!RMS) {
          opaque(bq[i]);
          unpack8<DT>(bq[i], b);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] * r * (g[e] + 1.f) + (RMS ? 0.f : b[e]);
        *reinterpret_cast<uint4*>(y + row * p.D + (lr + LPR * i) * 8) = pack8<DT>(v[i]);
      }
      if (lr == 0) {
        p.rstd[row] = r;
        if (!RMS) p.mean[row] = mu;
      }
    }
  }
}

template <int DT, int LPR, int NCH, bool RMS>
__global__ __launch_bounds__(kThreads) void norm_bwd_vec_kernel(NormParams p) {
  constexpr int RPW = kWave / LPR;
  extern __shared__ float acc[];  // D floats (x 2 with a bias)
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int lr = lane % LPR, slot = lane / LPR;
  const uint16_t* x = static_cast<const uint16_t*>(p.x);
  const uint16_t* dy = static_cast<const uint16_t*>(p.dy);
  uint16_t* dx = static_cast<uint16_t*>(p.y);
  const float inv_d = 1.f / static_cast<float>(p.D);
  // weights stay packed; x and dy of the row stay packed too and are unpacked once
  // for the row sums and once more for dx, so that the two accumulator sets
  // (2 x D / 64 floats per lane) fit beside them
  uint4 gq[NCH];
  float aw[NCH][8], ab[RMS ? 1 : NCH][8];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    gq[i] = make_uint4(0, 0, 0, 0);
    if (p.weight)
      gq[i] = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p.weight) + (lr + LPR * i) * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      aw[i][e] = 0.f;
      if (!RMS) ab[i][e] = 0.f;
    }
  }
  const int64_t step = static_cast<int64_t>(gridDim.x) * kWaves * RPW;
  for (int64_t row = (static_cast<int64_t>(blockIdx.x) * kWaves + wave) * RPW + slot;
       row - slot < p.rows; row += step) {
    const bool live = row < p.rows;
    const float r = live ? p.rstd[row] : 0.f;
    const float mu = (!RMS && live) ? p.mean[row] : 0.f;
    uint4 qx[NCH], qg[NCH];
    float s1 = 0.f, s0 = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      qx[i] = make_uint4(0, 0, 0, 0);
      qg[i] = make_uint4(0, 0, 0, 0);
      if (live) {
        qx[i] = *reinterpret_cast<const uint4*>(x + row * p.D + (lr + LPR * i) * 8);
        qg[i] = *reinterpret_cast<const uint4*>(dy + row * p.D + (lr + LPR * i) * 8);
      }
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      float xh[8], gy[8], g[8];
      unpack8<DT>(qx[i], xh);
      unpack8<DT>(qg[i], gy);
      opaque(gq[i]);  // unpacked per row, not hoisted out of the row loop
      unpack8<DT>(gq[i], g);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float h = (xh[e] - mu) * r;
        aw[i][e] += gy[e] * h;
        if (!RMS) ab[i][e] += gy[e];
        const float gw = gy[e] * (g[e] + 1.f);
        s1 += gw * h;
        if (!RMS) s0 += gw;
      }
    }
    s1 = group_sum<LPR>(s1) * inv_d;
    if (!RMS) s0 = group_sum<LPR>(s0) * inv_d;
    if (live) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        opaque(qx[i]);
        opaque(qg[i]);
        opaque(gq[i]);
        float xh[8], gy[8], g[8];
        unpack8<DT>(qx[i], xh);
        unpack8<DT>(qg[i], gy);
        unpack8<DT>(gq[i], g);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          gy[e] = r * (gy[e] * (g[e] + 1.f) - (xh[e] - mu) * r * s1 - s0);
        *reinterpret_cast<uint4*>(dx + row * p.D + (lr + LPR * i) * 8) = pack8<DT>(gy);
      }
    }
  }
  if (p.part_w == nullptr) return;  // no affine parameters
  // column sums of this workgroup, added slot by slot in a fixed order
  for (int s = 0; s < kWaves * RPW; ++s) {
    if (wave * RPW + slot == s) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = (lr + LPR * i) * 8 + e;
          if (s == 0) {
            acc[c] = aw[i][e];
            if (!RMS) acc[p.D + c] = ab[i][e];
          } else {
            acc[c] += aw[i][e];
            if (!RMS) acc[p.D + c] += ab[i][e];
          }
        }
    }
    __syncthreads();
  }
  for (int c = threadIdx.x; c < p.D; c += kThreads) {
    p.part_w[static_cast<int64_t>(blockIdx.x) * p.D + c] = acc[c];
    if (!RMS && p.part_b) p.part_b[static_cast<int64_t>(blockIdx.x) * p.D + c] = acc[p.D + c];
  }
}

// ---- any D, any element type: one wavefront per row, row re-read from cache ----
template <int DT, bool RMS>
__global__ __launch_bounds__(kThreads) void norm_fwd_any_kernel(NormParams p) {
  using T = typename Elem<DT>::type;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const T* x = static_cast<const T*>(p.x);
  const T* w = static_cast<const T*>(p.weight);
  const T* b = static_cast<const T*>(p.bias);
  T* y = static_cast<T*>(p.y);
  const float inv_d = 1.f / static_cast<float>(p.D);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + wave; row < p.rows;
       row += static_cast<int64_t>(gridDim.x) * kWaves) {
    const T* xr = x + row * p.D;
    float mu = 0.f;
    if (!RMS) {
      float s = 0.f;
      for (int c = lane; c < p.D; c += kWave) s += Elem<DT>::load(xr + c);
      mu = wave_sum(s) * inv_d;
    }
    float ss = 0.f;
    for (int c = lane; c < p.D; c += kWave) {
      const float d = Elem<DT>::load(xr + c) - mu;
      ss += d * d;
    }
    const float r = rsqrtf(wave_sum(ss) * inv_d + p.eps);
    for (int c = lane; c < p.D; c += kWave) {
      const float gm = w ? Elem<DT>::load(w + c) + 1.f : 1.f;
      const float bs = (!RMS && b) ? Elem<DT>::load(b + c) : 0.f;
      Elem<DT>::store(y + row * p.D + c, (Elem<DT>::load(xr + c) - mu) * r * gm + bs);
    }
    if (lane == 0) {
      p.rstd[row] = r;
      if (!RMS) p.mean[row] = mu;
    }
  }
}

template <int DT, bool RMS>
__global__ __launch_bounds__(kThreads) void norm_bwd_any_kernel(NormParams p, int active) {
  using T = typename Elem<DT>::type;
  extern __shared__ float acc[];  // `active` stripes of D floats (x 2 with a bias), one per working wave
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const T* x = static_cast<const T*>(p.x);
  const T* dy = static_cast<const T*>(p.dy);
  const T* w = static_cast<const T*>(p.weight);
  T* dx = static_cast<T*>(p.y);
  const float inv_d = 1.f / static_cast<float>(p.D);
  const int nacc = RMS ? 1 : 2;
  float* mine = acc + static_cast<int64_t>(wave) * nacc * p.D;
  if (p.part_w && wave < active)
    for (int c = lane; c < nacc * p.D; c += kWave) mine[c] = 0.f;
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * active + wave; wave < active && row < p.rows;
       row += static_cast<int64_t>(gridDim.x) * active) {
    const T* xr = x + row * p.D;
    const T* gr = dy + row * p.D;
    const float r = p.rstd[row], mu = RMS ? 0.f : p.mean[row];
    float s1 = 0.f, s0 = 0.f;
    for (int c = lane; c < p.D; c += kWave) {
      const float xh = (Elem<DT>::load(xr + c) - mu) * r;
      const float go = Elem<DT>::load(gr + c);
      const float gw = go * (w ? Elem<DT>::load(w + c) + 1.f : 1.f);
      s1 += gw * xh;
      s0 += gw;
      if (p.part_w) {
        mine[c] += go * xh;
        if (!RMS) mine[p.D + c] += go;
      }
    }
    s1 = wave_sum(s1) * inv_d;
    s0 = RMS ? 0.f : wave_sum(s0) * inv_d;
    for (int c = lane; c < p.D; c += kWave) {
      const float xh = (Elem<DT>::load(xr + c) - mu) * r;
      const float gw = Elem<DT>::load(gr + c) * (w ? Elem<DT>::load(w + c) + 1.f : 1.f);
      Elem<DT>::store(dx + row * p.D + c, r * (gw - xh * s1 - s0));
    }
  }
  if (p.part_w == nullptr) return;
  __syncthreads();
  for (int c = threadIdx.x; c < p.D; c += kThreads) {
    float sw = 0.f, sb = 0.f;
    for (int v = 0; v < active; ++v) {
      sw += acc[static_cast<int64_t>(v) * nacc * p.D + c];
      if (!RMS) sb += acc[static_cast<int64_t>(v) * nacc * p.D + p.D + c];
    }
    p.part_w[static_cast<int64_t>(blockIdx.x) * p.D + c] = sw;
    if (!RMS && p.part_b) p.part_b[static_cast<int64_t>(blockIdx.x) * p.D + c] = sb;
  }
}

// out[c] = sum over `groups` rows (`stride` floats apart) of part[., c], c < D:
// 64 columns x 16 row slices per workgroup
template <int DT>
__global__ __launch_bounds__(1024) void norm_param_grad_kernel(const float* part, int groups, int D,
                                                              int stride, typename Elem<DT>::type* out) {
  __shared__ float red[16][65];
  const int cx = threadIdx.x % 64, sy = threadIdx.x / 64;
  const int c = blockIdx.x * 64 + cx;
  float s = 0.f;
  if (c < D)
    for (int gidx = sy; gidx < groups; gidx += 16) s += part[static_cast<int64_t>(gidx) * stride + c];
  red[sy][cx] = s;
  __syncthreads();
  if (sy == 0 && c < D) {
    float t = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) t += red[v][cx];
    Elem<DT>::store(out + c, t);
  }
}


// ---- z -> (q, k): per-head RMSNorm, the two affine maps, rotary ----------------
// megalodon/modules/moving_average_gated_attention.py:319-330 (znorm over each
// head of z, `z.unsqueeze(2) * (gamma + 1) / sqrt(Dh) + beta`, unbind into q, k)
// followed by the rotary product of
// megalodon/modules/rotary_positional_embedding.py:53-77 on both: neighbouring
// elements (2i, 2i+1) of a head are one complex number that is multiplied by
// freqs[p][i], p = (row % L) % P the position inside the chunk.  One wavefront
// holds a row of S = 512 * NCH elements, G = Dh / 8 lanes per head; z is read
// once and q, k are written once.  The backward undoes the rotation with the
// conjugate factor, forms the gradients of the affine parameters as column
// sums (per-workgroup partials, reduced in a fixed order afterwards) and the
// RMSNorm gradient per head.
struct QkParams {
  const uint16_t* z;
  const uint16_t* gamma;  // (2, S) as stored: the factor is (gamma + 1) / sqrt(Dh)
  const uint16_t* beta;   // (2, S)
  const float* freqs;     // (P, Dh / 2, 2) cos, sin; null = no rotary
  const uint16_t* dq;
  const uint16_t* dk;
  uint16_t* q;  // forward: q, backward: dz
  uint16_t* k;
  float* rstd;  // (rows, S / Dh)
  float* part;  // backward: (groups, 4 S): dgamma_q | dgamma_k | dbeta_q | dbeta_k
  int64_t rows;
  int L, P, S, Dh;
  float eps, inv_sqrt_dh;
};

__device__ __forceinline__ void rotate8(float* u, const float4& f0, const float4& f1, bool conj) {
  const float c[4] = {f0.x, f0.z, f1.x, f1.z};
  const float sn[4] = {f0.y, f0.w, f1.y, f1.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float s = conj ? -sn[i] : sn[i];
    const float a = u[2 * i], b = u[2 * i + 1];
    u[2 * i] = a * c[i] - b * s;
    u[2 * i + 1] = a * s + b * c[i];
  }
}

template <int DT, int G, int NCH>
__global__ __launch_bounds__(kThreads) void qk_fwd_kernel(QkParams p) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int heads = p.S / p.Dh;
  const float inv_dh = 1.f / static_cast<float>(p.Dh);
  uint4 gq[NCH], gk[NCH], bq[NCH], bk[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = (lane + kWave * i) * 8;
    gq[i] = *reinterpret_cast<const uint4*>(p.gamma + c);
    gk[i] = *reinterpret_cast<const uint4*>(p.gamma + p.S + c);
    bq[i] = *reinterpret_cast<const uint4*>(p.beta + c);
    bk[i] = *reinterpret_cast<const uint4*>(p.beta + p.S + c);
  }
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + wave; row < p.rows;
       row += static_cast<int64_t>(gridDim.x) * kWaves) {
    const int pos = static_cast<int>(row % p.L) % p.P;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = (lane + kWave * i) * 8;
      float v[8], uq[8], uk[8], g[8], b[8];
      unpack8<DT>(*reinterpret_cast<const uint4*>(p.z + row * p.S + c), v);
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
      const float r = rsqrtf(group_sum<G>(ss) * inv_dh + p.eps);
      if (lane % G == 0) p.rstd[row * heads + c / p.Dh] = r;
      opaque(gq[i]); opaque(bq[i]); opaque(gk[i]); opaque(bk[i]);
      unpack8<DT>(gq[i], g);
      unpack8<DT>(bq[i], b);
#pragma unroll
      for (int e = 0; e < 8; ++e) uq[e] = v[e] * r * ((g[e] + 1.f) * p.inv_sqrt_dh) + b[e];
      unpack8<DT>(gk[i], g);
      unpack8<DT>(bk[i], b);
#pragma unroll
      for (int e = 0; e < 8; ++e) uk[e] = v[e] * r * ((g[e] + 1.f) * p.inv_sqrt_dh) + b[e];
      if (p.freqs) {
        const float4* f = reinterpret_cast<const float4*>(p.freqs + (static_cast<int64_t>(pos) * p.Dh + c % p.Dh));
        const float4 f0 = f[0], f1 = f[1];
        rotate8(uq, f0, f1, false);
        rotate8(uk, f0, f1, false);
      }
      *reinterpret_cast<uint4*>(p.q + row * p.S + c) = pack8<DT>(uq);
      *reinterpret_cast<uint4*>(p.k + row * p.S + c) = pack8<DT>(uk);
    }
  }
}

template <int DT, int G, int NCH>
__global__ __launch_bounds__(kThreads) void qk_bwd_kernel(QkParams p) {
  extern __shared__ float acc[];  // 4 S floats
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int heads = p.S / p.Dh;
  const float inv_dh = 1.f / static_cast<float>(p.Dh);
  uint4 gq[NCH], gk[NCH];
  float a_gq[NCH][8], a_gk[NCH][8], a_bq[NCH][8], a_bk[NCH][8];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = (lane + kWave * i) * 8;
    gq[i] = *reinterpret_cast<const uint4*>(p.gamma + c);
    gk[i] = *reinterpret_cast<const uint4*>(p.gamma + p.S + c);
#pragma unroll
    for (int e = 0; e < 8; ++e) a_gq[i][e] = 0.f, a_gk[i][e] = 0.f, a_bq[i][e] = 0.f, a_bk[i][e] = 0.f;
  }
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + wave; row < p.rows;
       row += static_cast<int64_t>(gridDim.x) * kWaves) {
    const int pos = static_cast<int>(row % p.L) % p.P;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = (lane + kWave * i) * 8;
      float zn[8], dq[8], dk[8], g[8], dzn[8];
      unpack8<DT>(*reinterpret_cast<const uint4*>(p.z + row * p.S + c), zn);
      unpack8<DT>(*reinterpret_cast<const uint4*>(p.dq + row * p.S + c), dq);
      unpack8<DT>(*reinterpret_cast<const uint4*>(p.dk + row * p.S + c), dk);
      const float r = p.rstd[row * heads + c / p.Dh];
      if (p.freqs) {
        const float4* f = reinterpret_cast<const float4*>(p.freqs + (static_cast<int64_t>(pos) * p.Dh + c % p.Dh));
        const float4 f0 = f[0], f1 = f[1];
        rotate8(dq, f0, f1, true);
        rotate8(dk, f0, f1, true);
      }
      opaque(gq[i]); opaque(gk[i]);
      unpack8<DT>(gq[i], g);
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        zn[e] *= r;
        a_gq[i][e] += dq[e] * zn[e];
        a_bq[i][e] += dq[e];
        dzn[e] = dq[e] * ((g[e] + 1.f) * p.inv_sqrt_dh);
      }
      unpack8<DT>(gk[i], g);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        a_gk[i][e] += dk[e] * zn[e];
        a_bk[i][e] += dk[e];
        dzn[e] += dk[e] * ((g[e] + 1.f) * p.inv_sqrt_dh);
        s += dzn[e] * zn[e];
      }
      s = group_sum<G>(s) * inv_dh;
#pragma unroll
      for (int e = 0; e < 8; ++e) dzn[e] = r * (dzn[e] - zn[e] * s);
      *reinterpret_cast<uint4*>(p.q + row * p.S + c) = pack8<DT>(dzn);
    }
  }
  // column sums of this workgroup, wave by wave in a fixed order
  for (int w = 0; w < kWaves; ++w) {
    if (wave == w) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = (lane + kWave * i) * 8 + e;
          const float vg0 = a_gq[i][e] * p.inv_sqrt_dh, vg1 = a_gk[i][e] * p.inv_sqrt_dh;
          if (w == 0) {
            acc[c] = vg0; acc[p.S + c] = vg1; acc[2 * p.S + c] = a_bq[i][e]; acc[3 * p.S + c] = a_bk[i][e];
          } else {
            acc[c] += vg0; acc[p.S + c] += vg1; acc[2 * p.S + c] += a_bq[i][e]; acc[3 * p.S + c] += a_bk[i][e];
          }
        }
    }
    __syncthreads();
  }
  for (int c = threadIdx.x; c < 4 * p.S; c += kThreads)
    p.part[static_cast<int64_t>(blockIdx.x) * 4 * p.S + c] = acc[c];
}

template <int DT, bool BWD>
int launch_qk(const QkParams& p, int groups, hipStream_t s) {
  const int G = p.Dh / 8, nch = p.S / 512;
  const size_t lds = BWD ? static_cast<size_t>(4) * p.S * sizeof(float) : 0;
  bool hit = false;
#define MEGA_QK(GG, NN)                                                      \
  if (G == GG && nch == NN) {                                                \
    hit = true;                                                              \
    if (BWD)                                                                 \
      qk_bwd_kernel<DT, GG, NN><<<groups, kThreads, lds, s>>>(p);            \
    else                                                                     \
      qk_fwd_kernel<DT, GG, NN><<<groups, kThreads, 0, s>>>(p);              \
  }
#define MEGA_QK_G(GG) MEGA_QK(GG, 1) MEGA_QK(GG, 2) MEGA_QK(GG, 4) MEGA_QK(GG, 8)
  MEGA_QK_G(8) MEGA_QK_G(16) MEGA_QK_G(32) MEGA_QK_G(64)
#undef MEGA_QK_G
#undef MEGA_QK
  if (!hit) return set_error(MEGA_ERR_UNSUPPORTED, "qk_norm_rotary: unsupported head size / width");
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

// How a row is split over a wavefront: `lpr` lanes per row, `nch` 16-byte chunks
// per lane (D = lpr * 8 * nch); lpr == 0: no register-resident variant.
struct Shape {
  int lpr, nch;
};
Shape vec_shape(int dtype, int64_t D, const NormParams& p) {
  if (dtype == MEGA_F32) return {0, 0};
  for (const void* q : {p.x, p.dy, p.weight, p.bias, static_cast<const void*>(p.y)})
    if (reinterpret_cast<uintptr_t>(q) % 16 != 0) return {0, 0};
  for (int nch : {1, 2, 4, 8})
    if (D == 512 * nch) return {64, nch};  // one row per wavefront
  if (D == 256) return {32, 1};            // two rows per wavefront
  if (D == 128) return {16, 1};            // four
  return {0, 0};
}

int groups_for(int64_t rows, int rows_per_group) {
  const int64_t g = (rows + rows_per_group - 1) / rows_per_group;
  return static_cast<int>(g < 1 ? 1 : (g > kMaxGroups ? kMaxGroups : g));
}

template <int DT, bool RMS, bool BWD>
int launch_vec(const NormParams& p, Shape sh, int groups, hipStream_t s) {
  const size_t lds = BWD && p.part_w ? static_cast<size_t>(p.D) * (RMS ? 1 : 2) * sizeof(float) : 0;
#define MEGA_NORM(LPR, NCH)                                                                  \
  if (sh.lpr == LPR && sh.nch == NCH) {                                                      \
    if (BWD)                                                                                 \
      norm_bwd_vec_kernel<DT, LPR, NCH, RMS><<<groups, kThreads, lds, s>>>(p);               \
    else                                                                                     \
      norm_fwd_vec_kernel<DT, LPR, NCH, RMS><<<groups, kThreads, 0, s>>>(p);                 \
  }
  MEGA_NORM(64, 1) MEGA_NORM(64, 2) MEGA_NORM(64, 4) MEGA_NORM(64, 8)
  MEGA_NORM(32, 1) MEGA_NORM(16, 1)
#undef MEGA_NORM
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT, bool RMS>
int run_fwd(const NormParams& p, int dtype, hipStream_t s) {
  const Shape sh = vec_shape(dtype, p.D, p);
  if constexpr (DT != MEGA_F32) {
    if (sh.lpr) {
      const int rpg = kWaves * (kWave / sh.lpr);
      const int64_t g = (p.rows + rpg - 1) / rpg;
      return launch_vec<DT, RMS, false>(p, sh, static_cast<int>(g > 16384 ? 16384 : g), s);
    }
  }
  const int64_t g = (p.rows + kWaves - 1) / kWaves;
  norm_fwd_any_kernel<DT, RMS><<<static_cast<int>(g > 16384 ? 16384 : g), kThreads, 0, s>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

static int check_norm(const char* who, int dtype, int64_t rows, int64_t D) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "%s: unknown dtype %d", who, dtype);
  MEGA_CHECK_ARG(rows >= 0 && D >= 1, "%s: bad sizes", who);
  MEGA_CHECK_ARG(D <= 65536, "%s: rows longer than 65536 elements are not supported", who);
  return MEGA_OK;
}

extern "C" int64_t mega_layer_norm_workspace_bytes(int64_t rows, int64_t D) {
  if (rows < 0 || D < 1) return 16;
  return 2 * static_cast<int64_t>(kMaxGroups) * D * static_cast<int64_t>(sizeof(float));
}

extern "C" int mega_layer_norm_fwd(const void* x, const void* weight, const void* bias, int dtype,
                                   int64_t rows, int64_t D, double eps, int rms, void* y,
                                   float* mean, float* rstd, void* stream) {
  int rc = check_norm("mega_layer_norm_fwd", dtype, rows, D);
  if (rc != MEGA_OK) return rc;
  if (rows == 0) return MEGA_OK;
  MEGA_CHECK_ARG(x && y && rstd && (rms || mean), "mega_layer_norm_fwd: null pointer");
  NormParams p{};
  p.x = x; p.weight = weight; p.bias = rms ? nullptr : bias; p.y = y; p.mean = mean; p.rstd = rstd;
  p.rows = rows; p.D = static_cast<int>(D); p.eps = static_cast<float>(eps);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define MEGA_DISPATCH(DT)                                   \
  return rms ? run_fwd<DT, true>(p, dtype, s) : run_fwd<DT, false>(p, dtype, s);
  if (dtype == MEGA_F32) { MEGA_DISPATCH(MEGA_F32) }
  if (dtype == MEGA_BF16) { MEGA_DISPATCH(MEGA_BF16) }
  MEGA_DISPATCH(MEGA_F16)
#undef MEGA_DISPATCH
}

template <int DT, bool RMS>
static int run_bwd(NormParams p, int dtype, void* dweight, void* dbias, float* ws, hipStream_t s) {
  using T = typename Elem<DT>::type;
  const bool affine = dweight != nullptr;
  const Shape sh = vec_shape(dtype, p.D, p);
  const int rpg = sh.lpr ? kWaves * (kWave / sh.lpr) : kWaves;
  const int groups = groups_for(p.rows, rpg);
  p.part_w = affine ? ws : nullptr;
  p.part_b = (affine && !RMS && dbias) ? ws + static_cast<int64_t>(kMaxGroups) * p.D : nullptr;
  bool done = false;
  if constexpr (DT != MEGA_F32) {
    if (sh.lpr) {
      int rc = launch_vec<DT, RMS, true>(p, sh, groups, s);
      if (rc != MEGA_OK) return rc;
      done = true;
    }
  }
  if (!done) {
    // one stripe of column sums per active wave, as many waves as 64 KB of LDS hold
    const size_t stripe = static_cast<size_t>(p.D) * (RMS ? 1 : 2) * sizeof(float);
    int active = kWaves;
    while (affine && active > 1 && active * stripe > 64 * 1024) active /= 2;
    MEGA_CHECK_ARG(!affine || active * stripe <= 64 * 1024,
                   "mega_layer_norm_bwd: parameter gradients for rows of %d elements do not fit", p.D);
    norm_bwd_any_kernel<DT, RMS><<<groups, kThreads, affine ? active * stripe : 0, s>>>(p, active);
    MEGA_CHECK_LAUNCH();
  }
  if (affine) {
    const int blocks = (p.D + 63) / 64;
    norm_param_grad_kernel<DT><<<blocks, 1024, 0, s>>>(p.part_w, groups, p.D, p.D, static_cast<T*>(dweight));
    MEGA_CHECK_LAUNCH();
    if (p.part_b) {
      norm_param_grad_kernel<DT><<<blocks, 1024, 0, s>>>(p.part_b, groups, p.D, p.D, static_cast<T*>(dbias));
      MEGA_CHECK_LAUNCH();
    }
  }
  return MEGA_OK;
}

extern "C" int mega_layer_norm_bwd(const void* dy, const void* x, const void* weight, const float* mean,
                                   const float* rstd, int dtype, int64_t rows, int64_t D, int rms,
                                   void* dx, void* dweight, void* dbias, void* workspace,
                                   void* stream) {
  int rc = check_norm("mega_layer_norm_bwd", dtype, rows, D);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG(rows >= 1, "mega_layer_norm_bwd: no rows");
  MEGA_CHECK_ARG(dy && x && dx && rstd && (rms || mean), "mega_layer_norm_bwd: null pointer");
  MEGA_CHECK_ARG(!dweight || workspace, "mega_layer_norm_bwd: parameter gradients need the workspace");
  MEGA_CHECK_ARG(!dbias || dweight, "mega_layer_norm_bwd: dbias without dweight");
  NormParams p{};
  p.x = x; p.dy = dy; p.weight = weight; p.y = dx; p.mean = const_cast<float*>(mean);
  p.rstd = const_cast<float*>(rstd); p.rows = rows; p.D = static_cast<int>(D);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
#define MEGA_DISPATCH(DT)                                                                       \
  return rms ? run_bwd<DT, true>(p, dtype, dweight, dbias, ws, s)                               \
             : run_bwd<DT, false>(p, dtype, dweight, dbias, ws, s);
  if (dtype == MEGA_F32) { MEGA_DISPATCH(MEGA_F32) }
  if (dtype == MEGA_BF16) { MEGA_DISPATCH(MEGA_BF16) }
  MEGA_DISPATCH(MEGA_F16)
#undef MEGA_DISPATCH
}

// ---- z -> (q, k) -------------------------------------------------------------------
static int check_qk(const char* who, int dtype, int64_t rows, int64_t L, int64_t P, int64_t S, int64_t Dh,
                    const void* freqs) {
  if (dtype != MEGA_BF16 && dtype != MEGA_F16)
    return set_error(MEGA_ERR_UNSUPPORTED, "%s: only bfloat16 / float16 tensors are supported", who);
  MEGA_CHECK_ARG(rows >= 0 && (rows == 0 || L >= 1) && S >= 1 && Dh >= 1, "%s: bad sizes", who);
  MEGA_CHECK_ARG(!freqs || P >= 1, "%s: rotary factors without positions", who);
  if (!(Dh == 64 || Dh == 128 || Dh == 256 || Dh == 512) || S % Dh != 0 ||
      !(S == 512 || S == 1024 || S == 2048 || S == 4096))
    return set_error(MEGA_ERR_UNSUPPORTED,
                     "%s: needs a head size of 64, 128, 256 or 512 and a width of 512, 1024, 2048 or 4096 "
                     "(got %lld, %lld)", who, (long long)Dh, (long long)S);
  return MEGA_OK;
}

extern "C" int64_t mega_qk_norm_rotary_workspace_bytes(int64_t S) {
  return S < 1 ? 16 : static_cast<int64_t>(kMaxGroups) * 4 * S * static_cast<int64_t>(sizeof(float));
}

extern "C" int mega_qk_norm_rotary_fwd(const void* z, const void* gamma, const void* beta,
                                       const float* freqs, int dtype, int64_t rows, int64_t L, int64_t P,
                                       int64_t S, int64_t Dh, double eps, void* q, void* k, float* rstd,
                                       void* stream) {
  int rc = check_qk("mega_qk_norm_rotary_fwd", dtype, rows, L, P, S, Dh, freqs);
  if (rc != MEGA_OK) return rc;
  if (rows == 0) return MEGA_OK;
  MEGA_CHECK_ARG(z && gamma && beta && q && k && rstd, "mega_qk_norm_rotary_fwd: null pointer");
  for (const void* ptr : {z, gamma, beta, static_cast<const void*>(freqs), static_cast<const void*>(q),
                          static_cast<const void*>(k)})
    MEGA_CHECK_ARG(reinterpret_cast<uintptr_t>(ptr) % 16 == 0, "mega_qk_norm_rotary_fwd: buffers must be 16-byte aligned");
  QkParams p{};
  p.z = static_cast<const uint16_t*>(z); p.gamma = static_cast<const uint16_t*>(gamma);
  p.beta = static_cast<const uint16_t*>(beta); p.freqs = freqs;
  p.q = static_cast<uint16_t*>(q); p.k = static_cast<uint16_t*>(k); p.rstd = rstd;
  p.rows = rows; p.L = (int)L; p.P = freqs ? (int)P : 1; p.S = (int)S; p.Dh = (int)Dh;
  p.eps = static_cast<float>(eps); p.inv_sqrt_dh = static_cast<float>(1.0 / sqrt(static_cast<double>(Dh)));
  const int64_t g = (rows + kWaves - 1) / kWaves;
  const int groups = static_cast<int>(g > 16384 ? 16384 : g);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == MEGA_BF16 ? launch_qk<MEGA_BF16, false>(p, groups, s) : launch_qk<MEGA_F16, false>(p, groups, s);
}

extern "C" int mega_qk_norm_rotary_bwd(const void* dq, const void* dk, const void* z, const void* gamma,
                                       const float* rstd, const float* freqs, int dtype, int64_t rows,
                                       int64_t L, int64_t P, int64_t S, int64_t Dh, void* dz, void* dgamma,
                                       void* dbeta, void* workspace, void* stream) {
  int rc = check_qk("mega_qk_norm_rotary_bwd", dtype, rows, L, P, S, Dh, freqs);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG(rows >= 1, "mega_qk_norm_rotary_bwd: no rows");
  MEGA_CHECK_ARG(dq && dk && z && gamma && rstd && dz && dgamma && dbeta && workspace,
                 "mega_qk_norm_rotary_bwd: null pointer");
  for (const void* ptr : {dq, dk, z, gamma, static_cast<const void*>(freqs), static_cast<const void*>(dz)})
    MEGA_CHECK_ARG(reinterpret_cast<uintptr_t>(ptr) % 16 == 0, "mega_qk_norm_rotary_bwd: buffers must be 16-byte aligned");
  QkParams p{};
  p.z = static_cast<const uint16_t*>(z); p.gamma = static_cast<const uint16_t*>(gamma); p.freqs = freqs;
  p.dq = static_cast<const uint16_t*>(dq); p.dk = static_cast<const uint16_t*>(dk);
  p.q = static_cast<uint16_t*>(dz); p.rstd = const_cast<float*>(rstd); p.part = static_cast<float*>(workspace);
  p.rows = rows; p.L = (int)L; p.P = freqs ? (int)P : 1; p.S = (int)S; p.Dh = (int)Dh;
  p.inv_sqrt_dh = static_cast<float>(1.0 / sqrt(static_cast<double>(Dh)));
  const int groups = groups_for(rows, kWaves);
  hipStream_t s = static_cast<hipStream_t>(stream);
  rc = dtype == MEGA_BF16 ? launch_qk<MEGA_BF16, true>(p, groups, s) : launch_qk<MEGA_F16, true>(p, groups, s);
  if (rc != MEGA_OK) return rc;
  const int cols = 2 * static_cast<int>(S), blocks = (cols + 63) / 64;
  if (dtype == MEGA_BF16) {
    norm_param_grad_kernel<MEGA_BF16><<<blocks, 1024, 0, s>>>(p.part, groups, cols, 2 * cols, static_cast<uint16_t*>(dgamma));
    norm_param_grad_kernel<MEGA_BF16><<<blocks, 1024, 0, s>>>(p.part + cols, groups, cols, 2 * cols, static_cast<uint16_t*>(dbeta));
  } else {
    norm_param_grad_kernel<MEGA_F16><<<blocks, 1024, 0, s>>>(p.part, groups, cols, 2 * cols, static_cast<uint16_t*>(dgamma));
    norm_param_grad_kernel<MEGA_F16><<<blocks, 1024, 0, s>>>(p.part + cols, groups, cols, 2 * cols, static_cast<uint16_t*>(dbeta));
  }
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}
