// Whole-sequence (non-causal) group normalisation for gfx950.
//
// For every sequence b and feature group g the mean and the biased variance
// are taken over the unmasked time steps and the D = H / G features of the
// group; y = (x - mean) * rstd * gamma + beta, zero at masked steps.  G = H is
// the per-feature operator.  Two layouts: features last (B, L, H) and length
// last (B, H, L).
// Reference semantics: megalodon/csrc/ops/sequence_norm.cc:258-372 (forward),
// :374-529 (backward), :531-842 (group variants).
//
// Both directions run as partial sums over tiles of the time axis, a small
// per-(b, g) combine, and one elementwise pass:
//   forward   moments_kernel  -> (mean, M2) of every (b, tile, feature)
//             finalize_fwd    -> mean, rstd, count (pairwise combination of
//                                the partial moments, no E[x^2] - E[x]^2)
//             apply_fwd       -> y
//   backward  moments_kernel  -> sum dy (x - mean), sum dy per (b, tile, feature)
//             finalize_bwd    -> the two per-group coefficients of dx and the
//                                per-(b, feature) terms of dgamma, dbeta
//             param_grad      -> dgamma, dbeta (sum over b)
//             apply_bwd       -> dx
#include "common.hpp"

namespace mega {
namespace {

constexpr int kThreads = 256;
constexpr int kTileFeatLast = 64;    // time steps per partial, (B, L, H)
constexpr int kTileLenLast = 2048;   // time steps per partial, (B, H, L)

// (n, mean, M2) <- combination with (n2, mean2, M2_2); M2 = sum (x - mean)^2
__device__ __forceinline__ void merge(float& n, float& m, float& s, float n2, float m2, float s2) {
  const float nn = n + n2;
  if (nn == 0.f) return;
  const float d = m2 - m;
  const float f = n2 / nn;
  m += d * f;
  s += s2 + d * d * n * f;
  n = nn;
}

__device__ __forceinline__ void block_merge(float& n, float& m, float& s, float* lds) {
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const float n2 = __shfl_xor(n, o), m2 = __shfl_xor(m, o), s2 = __shfl_xor(s, o);
    merge(n, m, s, n2, m2, s2);
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) {
    lds[3 * wave] = n;
    lds[3 * wave + 1] = m;
    lds[3 * wave + 2] = s;
  }
  __syncthreads();
  n = lds[0], m = lds[1], s = lds[2];
  for (int w = 1; w < kThreads / kWave; ++w) merge(n, m, s, lds[3 * w], lds[3 * w + 1], lds[3 * w + 2]);
}

__device__ __forceinline__ void block_sum2(float& a, float& b, float* lds) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) {
    lds[2 * wave] = a;
    lds[2 * wave + 1] = b;
  }
  __syncthreads();
  a = b = 0.f;
  for (int w = 0; w < kThreads / kWave; ++w) a += lds[2 * w], b += lds[2 * w + 1];
}

// One 16-byte access of `dtype` elements as floats.
template <int DT> struct Vec {
  static constexpr int N = DT == MEGA_F32 ? 4 : 8;  // elements of one 16-byte access
  static __device__ __forceinline__ void load(const typename Elem<DT>::type* p, float* v) {
    const uint4 q = *reinterpret_cast<const uint4*>(p);
    if constexpr (DT == MEGA_F32) {
      v[0] = __uint_as_float(q.x), v[1] = __uint_as_float(q.y), v[2] = __uint_as_float(q.z),
      v[3] = __uint_as_float(q.w);
    } else {
      unpack8<DT>(q, v);
    }
  }
  static __device__ __forceinline__ void store(typename Elem<DT>::type* p, const float* v) {
    if constexpr (DT == MEGA_F32) {
      *reinterpret_cast<uint4*>(p) =
          make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3]));
    } else {
      *reinterpret_cast<uint4*>(p) = pack8<DT>(v);
    }
  }
};

// Features last.  A thread owns V consecutive features (one 16-byte load per
// step when V > 1) and walks the tile's time steps; the padding mask is per
// step, so the branch is uniform.
//   BWD == false: part = (mean, M2) of the unmasked steps, cnt = their number
//   BWD == true : part = (sum dy (x - mean_g), sum dy)
template <int DT, bool BWD, int V>
__global__ __launch_bounds__(kThreads) void moments_feat_last_kernel(
    const typename Elem<DT>::type* __restrict__ x, const typename Elem<DT>::type* __restrict__ dy,
    const uint8_t* __restrict__ mask, const float* __restrict__ mean, int64_t L, int64_t H, int G, int D, int tiles,
    float2* __restrict__ part, int* __restrict__ cnt) {
  const int64_t h = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * V;
  const int tile = blockIdx.y;
  const int64_t b = blockIdx.z;
  const int64_t l0 = static_cast<int64_t>(tile) * kTileFeatLast;
  const int64_t l1 = l0 + kTileFeatLast < L ? l0 + kTileFeatLast : L;
  const bool live = h < H;  // V > 1 is only used when H % V == 0
  const uint8_t* mrow = mask ? mask + b * L : nullptr;
  float u[V], x0[V], s1[V], s2[V];
  int64_t sg = b * G + h / D;
  int rem = static_cast<int>(h % D);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    if (e > 0 && ++rem == D) rem = 0, ++sg;
    u[e] = (BWD && live) ? mean[sg] : 0.f;
    x0[e] = s1[e] = s2[e] = 0.f;
  }
  int n = 0;
  // U steps per round: their loads are issued together, then summed in order
  constexpr int U = BWD ? 4 : 8;
  for (int64_t l = l0; l < l1; l += U) {
    float v[U][V], g[U][V];
    bool ok[U];
#pragma unroll
    for (int i = 0; i < U; ++i) {
      ok[i] = l + i < l1 && !(mrow && mrow[l + i]);
      if (!(ok[i] && live)) continue;
      const int64_t at = (b * L + l + i) * H + h;
      if constexpr (V == 1) {
        v[i][0] = Elem<DT>::load(x + at);
        if (BWD) g[i][0] = Elem<DT>::load(dy + at);
      } else {
        Vec<DT>::load(x + at, v[i]);
        if (BWD) Vec<DT>::load(dy + at, g[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < U; ++i) {
      if (!ok[i]) continue;
      if (live) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          if (BWD) {
            s1[e] += g[i][e] * (v[i][e] - u[e]);
            s2[e] += g[i][e];
          } else {
            if (n == 0) x0[e] = v[i][e];
            const float d = v[i][e] - x0[e];
            s1[e] += d;
            s2[e] += d * d;
          }
        }
      }
      ++n;
    }
  }
  if (live) {
    const float inv = n > 0 ? 1.f / static_cast<float>(n) : 0.f;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float2 out = BWD ? make_float2(s1[e], s2[e])
                             : make_float2(x0[e] + s1[e] * inv, fmaxf(s2[e] - s1[e] * s1[e] * inv, 0.f));
      part[(b * tiles + tile) * H + h + e] = out;
    }
  }
  if (!BWD && blockIdx.x == 0 && threadIdx.x == 0) cnt[b * tiles + tile] = n;
}

// Length last.  A workgroup owns one tile of one (b, feature) row; lanes run
// along the time axis, V consecutive steps per load (V > 1 needs L % V == 0).
template <int DT, bool BWD, int V>
__global__ __launch_bounds__(kThreads) void moments_len_last_kernel(
    const typename Elem<DT>::type* __restrict__ x, const typename Elem<DT>::type* __restrict__ dy,
    const uint8_t* __restrict__ mask, const float* __restrict__ mean, int64_t L, int64_t H, int G, int D, int tiles,
    float2* __restrict__ part, int* __restrict__ cnt) {
  __shared__ float lds[3 * kThreads / kWave];
  const int tile = blockIdx.x;
  const int64_t h = blockIdx.y;
  const int64_t b = blockIdx.z;
  const int64_t l0 = static_cast<int64_t>(tile) * kTileLenLast;
  const int64_t l1 = l0 + kTileLenLast < L ? l0 + kTileLenLast : L;
  const int64_t row = (b * H + h) * L;
  const uint8_t* mrow = mask ? mask + b * L : nullptr;
  const float u = BWD ? mean[b * G + h / D] : 0.f;
  float n = 0.f, x0 = 0.f, s1 = 0.f, s2 = 0.f;
  for (int64_t l = l0 + static_cast<int64_t>(threadIdx.x) * V; l < l1; l += kThreads * V) {
    float v[V], g[V];
    if constexpr (V == 1) {
      v[0] = Elem<DT>::load(x + row + l);
      if (BWD) g[0] = Elem<DT>::load(dy + row + l);
    } else {
      Vec<DT>::load(x + row + l, v);
      if (BWD) Vec<DT>::load(dy + row + l, g);
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if (mrow && mrow[l + e]) continue;
      if (BWD) {
        s1 += g[e] * (v[e] - u);
        s2 += g[e];
      } else {
        if (n == 0.f) x0 = v[e];
        const float d = v[e] - x0;
        s1 += d;
        s2 += d * d;
        n += 1.f;
      }
    }
  }
  if (BWD) {
    block_sum2(s1, s2, lds);
    if (threadIdx.x == 0) part[(b * tiles + tile) * H + h] = make_float2(s1, s2);
  } else {
    float m = 0.f, s = 0.f;
    if (n > 0.f) {
      const float inv = 1.f / n;
      m = x0 + s1 * inv;
      s = fmaxf(s2 - s1 * s1 * inv, 0.f);
    }
    block_merge(n, m, s, lds);
    if (threadIdx.x == 0) {
      part[(b * tiles + tile) * H + h] = make_float2(m, s);
      if (h == 0) cnt[b * tiles + tile] = static_cast<int>(n + 0.5f);
    }
  }
}

// Sum of the per-tile step counts of one batch entry, by the whole workgroup
// (every thread must call it; thread 0 holds the result).
__device__ __forceinline__ long long block_count(const int* __restrict__ cnt, int tiles, long long* lds) {
  long long c = 0;
  for (int t = threadIdx.x; t < tiles; t += kThreads) c += cnt[t];
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) c += __shfl_down(c, o);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  __syncthreads();
  if (lane == 0) lds[wave] = c;
  __syncthreads();
  c = 0;
  for (int w = 0; w < kThreads / kWave; ++w) c += lds[w];
  return c;
}

// Shape of the combination passes: 16 threads along features, 16 along tiles.
constexpr int kColFeat = 16;                      // neighbouring features (128 bytes of float2) per pass
constexpr int kColSlices = kThreads / kColFeat;   // tile slices per workgroup
constexpr int kColAhead = 8;                  // loads issued before their merges

// One workgroup per (b, g): combine the (tile, feature) partial moments.
__global__ __launch_bounds__(kThreads) void finalize_fwd_kernel(const float2* __restrict__ part,
                                                                const int* __restrict__ cnt, int64_t H, int G, int D,
                                                                int tiles, float eps, int64_t* __restrict__ count,
                                                                float* __restrict__ mean, float* __restrict__ rstd) {
  __shared__ float lds[3 * kThreads / kWave];
  const int g = blockIdx.x;
  const int64_t b = blockIdx.y;
  const int lane = threadIdx.x % kColFeat, slice = threadIdx.x / kColFeat;
  float n = 0.f, m = 0.f, s = 0.f;
  for (int k0 = 0; k0 < D; k0 += kColFeat) {
    const bool live = k0 + lane < D;
    const int64_t h = static_cast<int64_t>(g) * D + k0 + lane;
    for (int t0 = slice; t0 < tiles; t0 += kColSlices * kColAhead) {
      float2 p[kColAhead];
      int ct[kColAhead];
#pragma unroll
      for (int i = 0; i < kColAhead; ++i) {
        const int t = t0 + i * kColSlices;
        const bool ok = live && t < tiles;
        p[i] = ok ? part[(b * tiles + t) * H + h] : make_float2(0.f, 0.f);
        ct[i] = ok ? cnt[b * tiles + t] : 0;
      }
#pragma unroll
      for (int i = 0; i < kColAhead; ++i) merge(n, m, s, static_cast<float>(ct[i]), p[i].x, p[i].y);
    }
  }
  block_merge(n, m, s, lds);
  if (threadIdx.x == 0) {
    const float var = n > 0.f ? s / n : 0.f;
    mean[b * G + g] = m;
    rstd[b * G + g] = 1.f / sqrtf(var + eps);
  }
  if (g == 0) {
    __shared__ long long cl[kThreads / kWave];
    const long long c = block_count(cnt + b * tiles, tiles, cl);
    if (threadIdx.x == 0) count[b] = c;
  }
}

// One workgroup per (b, g): per-feature sums over the tiles, the group's
// gamma-weighted sums, and from them the two coefficients of dx:
//   dx = rstd gamma dy - (x - mean) c1 - c2,
//   c1 = rstd^3 sum_g(gamma dy (x - mean)) / (count D),  c2 = rstd sum_g(gamma dy) / (count D)
template <int DT>
__global__ __launch_bounds__(kThreads) void finalize_bwd_kernel(
    const float2* __restrict__ part, const int64_t* __restrict__ count, const float* __restrict__ rstd,
    const typename Elem<DT>::type* __restrict__ gamma, int64_t H, int G, int D, int tiles, float2* __restrict__ col,
    float2* __restrict__ coef) {
  __shared__ float lds[2 * kThreads / kWave];
  __shared__ float cols[kColSlices][2][kColFeat];
  const int g = blockIdx.x;
  const int64_t b = blockIdx.y;
  const float r = rstd[b * G + g];
  const int lane = threadIdx.x % kColFeat, slice = threadIdx.x / kColFeat;
  float A = 0.f, Bs = 0.f;
  for (int k0 = 0; k0 < D; k0 += kColFeat) {
    const bool live = k0 + lane < D;
    const int64_t h = static_cast<int64_t>(g) * D + k0 + lane;
    float a = 0.f, c = 0.f;
    for (int t0 = slice; t0 < tiles; t0 += kColSlices * kColAhead) {
      float2 p[kColAhead];
#pragma unroll
      for (int i = 0; i < kColAhead; ++i) {
        const int t = t0 + i * kColSlices;
        p[i] = (live && t < tiles) ? part[(b * tiles + t) * H + h] : make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int i = 0; i < kColAhead; ++i) a += p[i].x, c += p[i].y;
    }
    cols[slice][0][lane] = a, cols[slice][1][lane] = c;
    __syncthreads();
    if (slice == 0 && live) {
      for (int w = 1; w < kColSlices; ++w) a += cols[w][0][lane], c += cols[w][1][lane];
      col[b * H + h] = make_float2(r * a, c);
      const float w = Elem<DT>::load(gamma + h);
      A += w * a;
      Bs += w * c;
    }
    __syncthreads();
  }
  block_sum2(A, Bs, lds);
  if (threadIdx.x == 0) {
    const int64_t c = count[b];
    const float k = c > 0 ? 1.f / (static_cast<float>(c) * static_cast<float>(D)) : 0.f;
    coef[b * G + g] = make_float2(k * r * r * r * A, k * r * Bs);
  }
}

// The per-feature operator (D == 1): a workgroup owns 16 neighbouring features
// of one batch entry; slice w walks tiles w, w + 16, ... (eight loads in flight
// per thread), the partial results are combined in slice order through LDS.

__global__ __launch_bounds__(kThreads) void finalize_fwd_cols_kernel(const float2* __restrict__ part,
                                                                     const int* __restrict__ cnt, int64_t H, int tiles,
                                                                     float eps, int64_t* __restrict__ count,
                                                                     float* __restrict__ mean,
                                                                     float* __restrict__ rstd) {
  __shared__ float lds[kColSlices][3][kColFeat];
  const int lane = threadIdx.x % kColFeat, slice = threadIdx.x / kColFeat;
  const int64_t h = static_cast<int64_t>(blockIdx.x) * kColFeat + lane;
  const int64_t b = blockIdx.y;
  const bool live = h < H;
  float n = 0.f, m = 0.f, s = 0.f;
  for (int t0 = slice; t0 < tiles; t0 += kColSlices * kColAhead) {
    float2 p[kColAhead];
    int ct[kColAhead];
#pragma unroll
    for (int i = 0; i < kColAhead; ++i) {
      const int t = t0 + i * kColSlices;
      const bool ok = live && t < tiles;
      p[i] = ok ? part[(b * tiles + t) * H + h] : make_float2(0.f, 0.f);
      ct[i] = ok ? cnt[b * tiles + t] : 0;
    }
#pragma unroll
    for (int i = 0; i < kColAhead; ++i) merge(n, m, s, static_cast<float>(ct[i]), p[i].x, p[i].y);
  }
  lds[slice][0][lane] = n, lds[slice][1][lane] = m, lds[slice][2][lane] = s;
  __syncthreads();
  if (blockIdx.x == 0) {
    __shared__ long long cl[kThreads / kWave];
    const long long c = block_count(cnt + b * tiles, tiles, cl);
    if (threadIdx.x == 0) count[b] = c;
  }
  if (slice != 0 || !live) return;
  for (int w = 1; w < kColSlices; ++w) merge(n, m, s, lds[w][0][lane], lds[w][1][lane], lds[w][2][lane]);
  mean[b * H + h] = m;
  rstd[b * H + h] = 1.f / sqrtf((n > 0.f ? s / n : 0.f) + eps);
}

template <int DT>
__global__ __launch_bounds__(kThreads) void finalize_bwd_cols_kernel(
    const float2* __restrict__ part, const int64_t* __restrict__ count, const float* __restrict__ rstd,
    const typename Elem<DT>::type* __restrict__ gamma, int64_t H, int tiles, float2* __restrict__ col,
    float2* __restrict__ coef) {
  __shared__ float lds[kColSlices][2][kColFeat];
  const int lane = threadIdx.x % kColFeat, slice = threadIdx.x / kColFeat;
  const int64_t h = static_cast<int64_t>(blockIdx.x) * kColFeat + lane;
  const int64_t b = blockIdx.y;
  const bool live = h < H;
  float a = 0.f, c = 0.f;
  for (int t0 = slice; t0 < tiles; t0 += kColSlices * kColAhead) {
    float2 p[kColAhead];
#pragma unroll
    for (int i = 0; i < kColAhead; ++i) {
      const int t = t0 + i * kColSlices;
      p[i] = (live && t < tiles) ? part[(b * tiles + t) * H + h] : make_float2(0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < kColAhead; ++i) a += p[i].x, c += p[i].y;
  }
  lds[slice][0][lane] = a, lds[slice][1][lane] = c;
  __syncthreads();
  if (slice != 0 || !live) return;
  for (int w = 1; w < kColSlices; ++w) a += lds[w][0][lane], c += lds[w][1][lane];
  const float r = rstd[b * H + h];
  const float w = Elem<DT>::load(gamma + h);
  const int64_t cn = count[b];
  const float k = cn > 0 ? 1.f / static_cast<float>(cn) : 0.f;
  col[b * H + h] = make_float2(r * a, c);
  coef[b * H + h] = make_float2(k * r * r * r * w * a, k * r * w * c);
}

template <int DT>
__global__ __launch_bounds__(kThreads) void param_grad_kernel(const float2* __restrict__ col, int64_t B, int64_t H,
                                                              typename Elem<DT>::type* __restrict__ dgamma,
                                                              typename Elem<DT>::type* __restrict__ dbeta) {
  const int64_t h = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (h >= H) return;
  float a = 0.f, c = 0.f;
  for (int64_t b = 0; b < B; ++b) {
    const float2 p = col[b * H + h];
    a += p.x;
    c += p.y;
  }
  Elem<DT>::store(dgamma + h, a);
  Elem<DT>::store(dbeta + h, c);
}

// ---- elementwise passes -------------------------------------------------------
// y (BWD == false) or dx (BWD == true) for V consecutive elements per thread.
// V = Vec<DT>::N needs the V elements to lie in one step (features last:
// H % V == 0) or one row (length last: L % V == 0) and 16-byte aligned
// pointers; V = 1 is the general path.
template <int DT, bool LAST, bool BWD, int V>
__global__ __launch_bounds__(kThreads) void apply_kernel(
    const typename Elem<DT>::type* __restrict__ x, const typename Elem<DT>::type* __restrict__ dy,
    const typename Elem<DT>::type* __restrict__ gamma, const typename Elem<DT>::type* __restrict__ beta,
    const uint8_t* __restrict__ mask, const float* __restrict__ mean, const float* __restrict__ rstd,
    const float2* __restrict__ coef, int64_t L, int64_t H, int G, int D, int64_t total,
    typename Elem<DT>::type* __restrict__ out) {
  const int64_t at = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * V;
  if (at >= total) return;
  int64_t b, h, l;
  if (LAST) {
    l = at % L;
    const int64_t bh = at / L;
    h = bh % H;
    b = bh / H;
  } else {
    h = at % H;
    const int64_t bl = at / H;
    l = bl % L;
    b = bl / L;
  }
  // statistics of each element's group: shared by the V elements when they
  // lie in one row (length last) or one group (D % V == 0)
  float uv[V], rv[V], c1v[V], c2v[V];
  const bool shared = LAST || V == 1 || D % V == 0;
  // group of element e: one division, then a running remainder
  int64_t sg = b * G + h / D;
  int rem = static_cast<int>(h % D);
  // one feature per group: the V statistics are V neighbouring floats
  const bool rowwise = !LAST && V > 1 && D == 1 &&
                       ((reinterpret_cast<uintptr_t>(mean) | reinterpret_cast<uintptr_t>(rstd)) & 15) == 0;
  if (rowwise) {
#pragma unroll
    for (int e = 0; e < V; e += 4) {
      const float4 u4 = *reinterpret_cast<const float4*>(mean + sg + e);
      const float4 r4 = *reinterpret_cast<const float4*>(rstd + sg + e);
      uv[e] = u4.x, uv[e + 1 < V ? e + 1 : e] = u4.y, uv[e + 2 < V ? e + 2 : e] = u4.z, uv[e + 3 < V ? e + 3 : e] = u4.w;
      rv[e] = r4.x, rv[e + 1 < V ? e + 1 : e] = r4.y, rv[e + 2 < V ? e + 2 : e] = r4.z, rv[e + 3 < V ? e + 3 : e] = r4.w;
    }
#pragma unroll
    for (int e = 0; e < V; e += 2) {
      float4 c4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (BWD) c4 = *reinterpret_cast<const float4*>(coef + sg + e);
      c1v[e] = c4.x, c2v[e] = c4.y, c1v[e + 1 < V ? e + 1 : e] = c4.z, c2v[e + 1 < V ? e + 1 : e] = c4.w;
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) {
    if (rowwise) break;
    if (e > 0 && shared) {
      uv[e] = uv[0], rv[e] = rv[0], c1v[e] = c1v[0], c2v[e] = c2v[0];
      continue;
    }
    if (e > 0 && ++rem == D) rem = 0, ++sg;
    uv[e] = mean[sg], rv[e] = rstd[sg];
    c1v[e] = c2v[e] = 0.f;
    if (BWD) {
      const float2 c = coef[sg];
      c1v[e] = c.x, c2v[e] = c.y;
    }
  }
  float xv[V], gv[V], wv[V], bv[V], ov[V];
  if constexpr (V == 1) {
    xv[0] = Elem<DT>::load(x + at);
    if (BWD) gv[0] = Elem<DT>::load(dy + at);
    wv[0] = Elem<DT>::load(gamma + h);
    bv[0] = BWD ? 0.f : Elem<DT>::load(beta + h);
  } else {
    Vec<DT>::load(x + at, xv);
    if (BWD) Vec<DT>::load(dy + at, gv);
    if (LAST) {
      const float w = Elem<DT>::load(gamma + h);
      const float bb = BWD ? 0.f : Elem<DT>::load(beta + h);
#pragma unroll
      for (int e = 0; e < V; ++e) wv[e] = w, bv[e] = bb;
    } else {
      Vec<DT>::load(gamma + h, wv);
      if (!BWD) Vec<DT>::load(beta + h, bv);
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const bool masked = mask && mask[b * L + (LAST ? l + e : l)];
    const float v = BWD ? rv[e] * wv[e] * gv[e] - (xv[e] - uv[e]) * c1v[e] - c2v[e]
                        : (xv[e] - uv[e]) * rv[e] * wv[e] + bv[e];
    ov[e] = masked ? 0.f : v;
  }
  if constexpr (V == 1) {
    Elem<DT>::store(out + at, ov[0]);
  } else {
    Vec<DT>::store(out + at, ov);
  }
}

struct Shape {
  int64_t B, L, H;
  int G, D, tiles, last;
};

inline int64_t align256(int64_t v) { return (v + 255) & ~int64_t(255); }
inline int tiles_of(int64_t L, int last) {
  const int t = last ? kTileLenLast : kTileFeatLast;
  return static_cast<int>((L + t - 1) / t);
}

struct Workspace {
  float2* part;
  int* cnt;
  float2* col;
  float2* coef;
  int64_t bytes;
};
inline Workspace carve(void* base, int64_t B, int64_t H, int G, int tiles) {
  Workspace w;
  char* p = static_cast<char*>(base);
  int64_t off = 0;
  w.part = reinterpret_cast<float2*>(p + off);
  off += align256(B * tiles * H * 8);
  w.cnt = reinterpret_cast<int*>(p + off);
  off += align256(B * tiles * 4);
  w.col = reinterpret_cast<float2*>(p + off);
  off += align256(B * H * 8);
  w.coef = reinterpret_cast<float2*>(p + off);
  off += align256(B * G * 8);
  w.bytes = off;
  return w;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int DT, bool BWD>
int launch_moments(const Shape& s, const void* x, const void* dy, const uint8_t* mask, const float* mean,
                   const Workspace& w, hipStream_t st) {
  using T = typename Elem<DT>::type;
  constexpr int V = Vec<DT>::N;
  if (s.tiles == 0) return MEGA_OK;  // empty sequences: nothing to sum
  const T* xp = static_cast<const T*>(x);
  const T* gp = static_cast<const T*>(dy);
  const bool vec = aligned16(x) && (!BWD || aligned16(dy)) && (s.last ? s.L : s.H) % V == 0;
#define MEGA_MOMENTS(KERNEL_, V_, GRID_) \
  KERNEL_<DT, BWD, V_><<<GRID_, kThreads, 0, st>>>(xp, gp, mask, mean, s.L, s.H, s.G, s.D, s.tiles, w.part, w.cnt)
  if (s.last) {
    const dim3 grid(s.tiles, static_cast<unsigned>(s.H), static_cast<unsigned>(s.B));
    if (vec) MEGA_MOMENTS(moments_len_last_kernel, V, grid); else MEGA_MOMENTS(moments_len_last_kernel, 1, grid);
  } else {
    const int64_t per = static_cast<int64_t>(kThreads) * (vec ? V : 1);
    const dim3 grid(static_cast<unsigned>((s.H + per - 1) / per), s.tiles, static_cast<unsigned>(s.B));
    if (vec) MEGA_MOMENTS(moments_feat_last_kernel, V, grid); else MEGA_MOMENTS(moments_feat_last_kernel, 1, grid);
  }
#undef MEGA_MOMENTS
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT, bool BWD>
int launch_apply(const Shape& s, const void* x, const void* dy, const void* gamma, const void* beta,
                 const uint8_t* mask, const float* mean, const float* rstd, const float2* coef, void* out,
                 hipStream_t st) {
  using T = typename Elem<DT>::type;
  constexpr int V = Vec<DT>::N;
  const int64_t total = s.B * s.L * s.H;
  if (total == 0) return MEGA_OK;
  bool vec = aligned16(x) && aligned16(out) && (!BWD || aligned16(dy));
  if (s.last)
    vec = vec && s.L % V == 0;
  else
    vec = vec && s.H % V == 0 && aligned16(gamma) && (BWD || aligned16(beta));
  const int64_t threads = vec ? total / V : total;
  const int64_t blocks = (threads + kThreads - 1) / kThreads;
  MEGA_CHECK_ARG(blocks < (1ll << 31), "mega_group_sequence_norm: tensor too large");
  const T* xp = static_cast<const T*>(x);
  const T* gp = static_cast<const T*>(dy);
  const T* wp = static_cast<const T*>(gamma);
  const T* bp = static_cast<const T*>(beta);
  T* op = static_cast<T*>(out);
  const unsigned nb = static_cast<unsigned>(blocks);
#define MEGA_APPLY(LAST_, V_)                                                                                   \
  apply_kernel<DT, LAST_, BWD, V_><<<nb, kThreads, 0, st>>>(xp, gp, wp, bp, mask, mean, rstd, coef, s.L, s.H, s.G, \
                                                            s.D, total, op)
  if (s.last) {
    if (vec) MEGA_APPLY(true, V); else MEGA_APPLY(true, 1);
  } else {
    if (vec) MEGA_APPLY(false, V); else MEGA_APPLY(false, 1);
  }
#undef MEGA_APPLY
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT>
int run_fwd(const Shape& s, const void* x, const void* gamma, const void* beta, const uint8_t* mask, float eps,
            void* y, int64_t* count, float* mean, float* rstd, void* workspace, hipStream_t st) {
  const Workspace w = carve(workspace, s.B, s.H, s.G, s.tiles);
  if (int rc = launch_moments<DT, false>(s, x, nullptr, mask, nullptr, w, st)) return rc;
  if (s.D == 1)
    finalize_fwd_cols_kernel<<<dim3(static_cast<unsigned>((s.H + kColFeat - 1) / kColFeat),
                                    static_cast<unsigned>(s.B)), kThreads, 0, st>>>(w.part, w.cnt, s.H, s.tiles, eps,
                                                                                     count, mean, rstd);
  else
    finalize_fwd_kernel<<<dim3(s.G, static_cast<unsigned>(s.B)), kThreads, 0, st>>>(w.part, w.cnt, s.H, s.G, s.D,
                                                                                     s.tiles, eps, count, mean, rstd);
  MEGA_CHECK_LAUNCH();
  return launch_apply<DT, false>(s, x, nullptr, gamma, beta, mask, mean, rstd, nullptr, y, st);
}

template <int DT>
int run_bwd(const Shape& s, const void* dy, const void* x, const int64_t* count, const float* mean, const float* rstd,
            const void* gamma, const uint8_t* mask, void* dx, void* dgamma, void* dbeta, void* workspace,
            hipStream_t st) {
  using T = typename Elem<DT>::type;
  const Workspace w = carve(workspace, s.B, s.H, s.G, s.tiles);
  if (s.B == 0) {  // no sequences: the parameter gradients are zero
    param_grad_kernel<DT><<<static_cast<unsigned>((s.H + kThreads - 1) / kThreads), kThreads, 0, st>>>(
        w.col, 0, s.H, static_cast<T*>(dgamma), static_cast<T*>(dbeta));
    MEGA_CHECK_LAUNCH();
    return MEGA_OK;
  }
  if (int rc = launch_moments<DT, true>(s, x, dy, mask, mean, w, st)) return rc;
  if (s.D == 1)
    finalize_bwd_cols_kernel<DT><<<dim3(static_cast<unsigned>((s.H + kColFeat - 1) / kColFeat),
                                        static_cast<unsigned>(s.B)), kThreads, 0, st>>>(
        w.part, count, rstd, static_cast<const T*>(gamma), s.H, s.tiles, w.col, w.coef);
  else
    finalize_bwd_kernel<DT><<<dim3(s.G, static_cast<unsigned>(s.B)), kThreads, 0, st>>>(
        w.part, count, rstd, static_cast<const T*>(gamma), s.H, s.G, s.D, s.tiles, w.col, w.coef);
  MEGA_CHECK_LAUNCH();
  param_grad_kernel<DT><<<static_cast<unsigned>((s.H + kThreads - 1) / kThreads), kThreads, 0, st>>>(
      w.col, s.B, s.H, static_cast<T*>(dgamma), static_cast<T*>(dbeta));
  MEGA_CHECK_LAUNCH();
  return launch_apply<DT, true>(s, x, dy, gamma, nullptr, mask, mean, rstd, w.coef, dx, st);
}

int check_shape(const char* who, int dtype, int64_t B, int64_t L, int64_t H, int64_t G, int last, Shape* s) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "%s: unknown dtype %d", who, dtype);
  MEGA_CHECK_ARG(B >= 0 && L >= 0 && H >= 1, "%s: bad sizes B=%lld L=%lld H=%lld", who, (long long)B, (long long)L,
                 (long long)H);
  MEGA_CHECK_ARG(G >= 1 && H % G == 0, "%s: num_groups %lld does not divide H=%lld", who, (long long)G,
                 (long long)H);
  MEGA_CHECK_ARG(B <= 65535 && H < (1ll << 31), "%s: B <= 65535 and H < 2^31 required", who);
  MEGA_CHECK_ARG(!last || H <= 65535, "%s: length-last layout needs H <= 65535", who);
  const int tiles = tiles_of(L, last);
  MEGA_CHECK_ARG(L < (1ll << 31) && (last || tiles <= 65535), "%s: sequence too long", who);
  s->B = B, s->L = L, s->H = H;
  s->G = static_cast<int>(G), s->D = static_cast<int>(H / G);
  s->tiles = tiles, s->last = last ? 1 : 0;
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int64_t mega_group_sequence_norm_workspace_bytes(int64_t B, int64_t L, int64_t H, int64_t num_groups,
                                                            int length_last) {
  if (B < 0 || L < 0 || H < 1 || num_groups < 1) return 0;
  return carve(nullptr, B, H, static_cast<int>(num_groups), tiles_of(L, length_last)).bytes;
}

extern "C" int mega_group_sequence_norm_fwd(const void* x, const void* gamma, const void* beta,
                                            const uint8_t* padding_mask, int dtype, int64_t B, int64_t L, int64_t H,
                                            int64_t num_groups, double eps, int length_last, void* y, int64_t* count,
                                            float* mean, float* rstd, void* workspace, void* stream) {
  Shape s;
  if (int rc = check_shape("mega_group_sequence_norm_fwd", dtype, B, L, H, num_groups, length_last, &s)) return rc;
  if (B == 0) return MEGA_OK;
  MEGA_CHECK_ARG(gamma && beta && count && mean && rstd && workspace,
                 "mega_group_sequence_norm_fwd: null pointer");
  MEGA_CHECK_ARG(L == 0 || (x && y), "mega_group_sequence_norm_fwd: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float e = static_cast<float>(eps);
  if (dtype == MEGA_F32)
    return run_fwd<MEGA_F32>(s, x, gamma, beta, padding_mask, e, y, count, mean, rstd, workspace, st);
  if (dtype == MEGA_BF16)
    return run_fwd<MEGA_BF16>(s, x, gamma, beta, padding_mask, e, y, count, mean, rstd, workspace, st);
  return run_fwd<MEGA_F16>(s, x, gamma, beta, padding_mask, e, y, count, mean, rstd, workspace, st);
}

extern "C" int mega_group_sequence_norm_bwd(const void* dy, const void* x, const int64_t* count, const float* mean,
                                            const float* rstd, const void* gamma, const uint8_t* padding_mask,
                                            int dtype, int64_t B, int64_t L, int64_t H, int64_t num_groups,
                                            int length_last, void* dx, void* dgamma, void* dbeta, void* workspace,
                                            void* stream) {
  Shape s;
  if (int rc = check_shape("mega_group_sequence_norm_bwd", dtype, B, L, H, num_groups, length_last, &s)) return rc;
  MEGA_CHECK_ARG(dgamma && dbeta, "mega_group_sequence_norm_bwd: null pointer");
  MEGA_CHECK_ARG(B == 0 || (count && mean && rstd && gamma && workspace),
                 "mega_group_sequence_norm_bwd: null pointer");
  MEGA_CHECK_ARG(B == 0 || L == 0 || (dy && x && dx), "mega_group_sequence_norm_bwd: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32)
    return run_bwd<MEGA_F32>(s, dy, x, count, mean, rstd, gamma, padding_mask, dx, dgamma, dbeta, workspace, st);
  if (dtype == MEGA_BF16)
    return run_bwd<MEGA_BF16>(s, dy, x, count, mean, rstd, gamma, padding_mask, dx, dgamma, dbeta, workspace, st);
  return run_bwd<MEGA_F16>(s, dy, x, count, mean, rstd, gamma, padding_mask, dx, dgamma, dbeta, workspace, st);
}
