// Memory-bound glue of the Megalodon block that the reference leaves to
// PyTorch's generic kernels:
//
//  * transposing (B, L, D) <-> (B, D, L) around the EMA convolution
//    (megalodon/modules/moving_average_gated_attention.py:299-300,314:
//    `out_tsn.transpose(1, 2)` ... `out_cema.transpose(1, 2)`, each followed by
//    a strided copy when the next operator asks for contiguous memory);
//  * the gates `silu(a) * b` (moving_average_gated_attention.py:333-336,
//    normalized_feedforward_network.py:82) with their backward.
//
// Both are pure streaming kernels: 16-byte accesses on both sides, one read
// and one write of every element.
#include "common.hpp"

#include <algorithm>

namespace mega {
namespace {

constexpr int kThreads = 256;

// ---- (Z, R, C) -> (Z, C, R) for 16-bit elements ---------------------------------
// A workgroup moves a 128 x 128 tile through LDS.  The tile is stored
// transposed ([c][r], 64 words per c) by 2-byte LDS writes and read back in
// 16-byte runs along r.  Word w of row c sits at w ^ (((c >> 3) & 15) << 2):
// the 16 lanes that hold the 16 column groups of one input row then write to
// 16 different banks, and the 16-byte runs stay contiguous.
constexpr int kTT = 128;

__global__ __launch_bounds__(kThreads) void transpose16_kernel(const uint16_t* in, uint16_t* out,
                                                              int R, int C, int tiles_c, int tiles_r) {
  __shared__ uint32_t tile[kTT * kTT / 2];
  uint16_t* t16 = reinterpret_cast<uint16_t*>(tile);
  const int per_z = tiles_c * tiles_r;
  const int z = blockIdx.x / per_z;
  const int tr = (blockIdx.x % per_z) / tiles_c, tc = blockIdx.x % tiles_c;
  const int r0 = tr * kTT, c0 = tc * kTT;
  const uint16_t* src = in + static_cast<int64_t>(z) * R * C;
  uint16_t* dst = out + static_cast<int64_t>(z) * R * C;
  const int m = threadIdx.x % 16, q = threadIdx.x / 16;
  // load: thread (q, m) takes columns c0 + 8m .. +7 of rows r0 + q + 16 * pass
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int rl = q + 16 * pass;
    const int r = r0 + rl, c = c0 + 8 * m;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (r < R && c < C) v = *reinterpret_cast<const uint4*>(src + static_cast<int64_t>(r) * C + c);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
    const int w = ((rl >> 1) ^ (m << 2)) * 2 + (rl & 1);
#pragma unroll
    for (int k = 0; k < 8; ++k)
      t16[(8 * m + k) * kTT + w] = static_cast<uint16_t>(k & 1 ? u[k >> 1] >> 16 : u[k >> 1] & 0xffffu);
  }
  __syncthreads();
  // store: thread (q, m) writes rows r0 + 8m .. +7 of output row c0 + q + 16 * pass
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int cl = q + 16 * pass;
    const int c = c0 + cl, r = r0 + 8 * m;
    if (c < C && r < R) {
      const int w = (4 * m) ^ (((cl >> 3) & 15) << 2);
      const uint4 v = *reinterpret_cast<const uint4*>(tile + cl * (kTT / 2) + w);
      *reinterpret_cast<uint4*>(dst + static_cast<int64_t>(c) * R + r) = v;
    }
  }
}

// any element size, any shape: 32 x 32 tiles, one element per access
template <typename T>
__global__ __launch_bounds__(kThreads) void transpose_any_kernel(const T* in, T* out, int R, int C,
                                                                int tiles_c, int tiles_r) {
  __shared__ T tile[32][33];
  const int per_z = tiles_c * tiles_r;
  const int z = blockIdx.x / per_z;
  const int tr = (blockIdx.x % per_z) / tiles_c, tc = blockIdx.x % tiles_c;
  const T* src = in + static_cast<int64_t>(z) * R * C;
  T* dst = out + static_cast<int64_t>(z) * R * C;
  const int x = threadIdx.x % 32, y = threadIdx.x / 32;
  for (int i = y; i < 32; i += kThreads / 32) {
    const int r = tr * 32 + i, c = tc * 32 + x;
    if (r < R && c < C) tile[i][x] = src[static_cast<int64_t>(r) * C + c];
  }
  __syncthreads();
  for (int i = y; i < 32; i += kThreads / 32) {
    const int c = tc * 32 + i, r = tr * 32 + x;
    if (r < R && c < C) dst[static_cast<int64_t>(c) * R + r] = tile[x][i];
  }
}

// ---- gates ------------------------------------------------------------------

__device__ __forceinline__ float sigmoidf(float a) { return 1.f / (1.f + __expf(-a)); }
__device__ __forceinline__ float gate_fwd(float a, float b) { return a * sigmoidf(a) * b; }
__device__ __forceinline__ void gate_bwd(float g, float a, float b, float* da, float* db) {
  const float s = sigmoidf(a);
  *db = g * a * s;
  *da = g * b * s * (1.f + a * (1.f - s));
}

// out = silu(a) * b over n elements; [first, n) one by one when VEC is false
template <int DT, bool VEC>
__global__ __launch_bounds__(kThreads) void silu_mul_fwd_kernel(const typename Elem<DT>::type* a,
                                                               const typename Elem<DT>::type* b,
                                                               typename Elem<DT>::type* out,
                                                               int64_t first, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  const int64_t i0 = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (VEC) {
    // n counts groups of 8 (16-bit) / 4 (float) elements
    for (int64_t g = i0; g < n; g += stride) {
      if (DT == MEGA_F32) {
        const float4 x = reinterpret_cast<const float4*>(a)[g], y = reinterpret_cast<const float4*>(b)[g];
        reinterpret_cast<float4*>(out)[g] =
            make_float4(gate_fwd(x.x, y.x), gate_fwd(x.y, y.y), gate_fwd(x.z, y.z), gate_fwd(x.w, y.w));
      } else {
        float x[8], y[8];
        unpack8<DT>(reinterpret_cast<const uint4*>(a)[g], x);
        unpack8<DT>(reinterpret_cast<const uint4*>(b)[g], y);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = gate_fwd(x[e], y[e]);
        reinterpret_cast<uint4*>(out)[g] = pack8<DT>(x);
      }
    }
  } else {
    for (int64_t e = first + i0; e < n; e += stride)
      Elem<DT>::store(out + e, gate_fwd(Elem<DT>::load(a + e), Elem<DT>::load(b + e)));
  }
}

template <int DT, bool VEC>
__global__ __launch_bounds__(kThreads) void silu_mul_bwd_kernel(const typename Elem<DT>::type* dout,
                                                               const typename Elem<DT>::type* a,
                                                               const typename Elem<DT>::type* b,
                                                               typename Elem<DT>::type* da,
                                                               typename Elem<DT>::type* db,
                                                               int64_t first, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
  const int64_t i0 = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (VEC) {
    for (int64_t g = i0; g < n; g += stride) {
      if (DT == MEGA_F32) {
        const float4 go = reinterpret_cast<const float4*>(dout)[g];
        const float4 x = reinterpret_cast<const float4*>(a)[g], y = reinterpret_cast<const float4*>(b)[g];
        float4 ga, gb;
        gate_bwd(go.x, x.x, y.x, &ga.x, &gb.x);
        gate_bwd(go.y, x.y, y.y, &ga.y, &gb.y);
        gate_bwd(go.z, x.z, y.z, &ga.z, &gb.z);
        gate_bwd(go.w, x.w, y.w, &ga.w, &gb.w);
        reinterpret_cast<float4*>(da)[g] = ga;
        reinterpret_cast<float4*>(db)[g] = gb;
      } else {
        float go[8], x[8], y[8], ga[8], gb[8];
        unpack8<DT>(reinterpret_cast<const uint4*>(dout)[g], go);
        unpack8<DT>(reinterpret_cast<const uint4*>(a)[g], x);
        unpack8<DT>(reinterpret_cast<const uint4*>(b)[g], y);
#pragma unroll
        for (int e = 0; e < 8; ++e) gate_bwd(go[e], x[e], y[e], &ga[e], &gb[e]);
        reinterpret_cast<uint4*>(da)[g] = pack8<DT>(ga);
        reinterpret_cast<uint4*>(db)[g] = pack8<DT>(gb);
      }
    }
  } else {
    for (int64_t e = first + i0; e < n; e += stride) {
      float ga, gb;
      gate_bwd(Elem<DT>::load(dout + e), Elem<DT>::load(a + e), Elem<DT>::load(b + e), &ga, &gb);
      Elem<DT>::store(da + e, ga);
      Elem<DT>::store(db + e, gb);
    }
  }
}

inline unsigned grid_for(int64_t items) {
  const int64_t blocks = (items + kThreads - 1) / kThreads;
  return static_cast<unsigned>(blocks < 1 ? 1 : (blocks > (1 << 20) ? (1 << 20) : blocks));
}

template <int DT>
int launch_silu_mul(const void* dout, const void* a, const void* b, void* o0, void* o1, int64_t n,
                    hipStream_t s) {
  using T = typename Elem<DT>::type;
  const int per = DT == MEGA_F32 ? 4 : 8;
  bool vec = true;
  for (const void* p : {dout, a, b, static_cast<const void*>(o0), static_cast<const void*>(o1)})
    vec = vec && reinterpret_cast<uintptr_t>(p) % 16 == 0;
  const int64_t groups = vec ? n / per : 0;
  const T* pa = static_cast<const T*>(a);
  const T* pb = static_cast<const T*>(b);
  const T* pg = static_cast<const T*>(dout);
  if (groups > 0) {
    if (dout == nullptr)
      silu_mul_fwd_kernel<DT, true><<<grid_for(groups), kThreads, 0, s>>>(pa, pb, static_cast<T*>(o0), 0, groups);
    else
      silu_mul_bwd_kernel<DT, true><<<grid_for(groups), kThreads, 0, s>>>(pg, pa, pb, static_cast<T*>(o0),
                                                                          static_cast<T*>(o1), 0, groups);
    MEGA_CHECK_LAUNCH();
  }
  const int64_t first = groups * per;
  if (first < n) {
    if (dout == nullptr)
      silu_mul_fwd_kernel<DT, false><<<grid_for(n - first), kThreads, 0, s>>>(pa, pb, static_cast<T*>(o0), first, n);
    else
      silu_mul_bwd_kernel<DT, false><<<grid_for(n - first), kThreads, 0, s>>>(pg, pa, pb, static_cast<T*>(o0),
                                                                              static_cast<T*>(o1), first, n);
    MEGA_CHECK_LAUNCH();
  }
  return MEGA_OK;
}

// ---- a float32 / float16 tensor as the sum of two bfloat16 tensors ------------------------
// hi = bf16(v), lo = bf16(v - hi): 16 significant bits of a float32 value, all 11 of a float16
// one.  The backward of the CEMA recurrence is linear in dy and, for the parameter gradients,
// in x, and runs on such pieces (mega_cema_scan_bwd_wide).  8 elements per lane and pass.
template <int DT>
__global__ __launch_bounds__(kThreads) void split_bf16_kernel(const void* __restrict__ src, uint16_t* __restrict__ hi,
                                                             uint16_t* __restrict__ lo, int64_t n8) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n8;
       i += static_cast<int64_t>(gridDim.x) * kThreads) {
    float v[8];
    if (DT == MEGA_F32) {
      const float4 a = reinterpret_cast<const float4*>(src)[2 * i], b = reinterpret_cast<const float4*>(src)[2 * i + 1];
      v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
      unpack8<MEGA_F16>(reinterpret_cast<const uint4*>(src)[i], v);
    }
    uint32_t h[4], l[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      h[e] = pack_bf16x2(v[2 * e], v[2 * e + 1]);
      l[e] = pack_bf16x2(v[2 * e] - __uint_as_float(h[e] << 16), v[2 * e + 1] - __uint_as_float(h[e] & 0xffff0000u));
    }
    reinterpret_cast<uint4*>(hi)[i] = make_uint4(h[0], h[1], h[2], h[3]);
    reinterpret_cast<uint4*>(lo)[i] = make_uint4(l[0], l[1], l[2], l[3]);
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_transpose(const void* in, int dtype, int64_t Z, int64_t R, int64_t C, void* out,
                              void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_transpose: unknown dtype %d", dtype);
  MEGA_CHECK_ARG(Z >= 0 && R >= 0 && C >= 0, "mega_transpose: negative size");
  if (Z == 0 || R == 0 || C == 0) return MEGA_OK;
  MEGA_CHECK_ARG(in && out && in != out, "mega_transpose: null or aliased pointers");
  MEGA_CHECK_ARG(R < (1ll << 31) && C < (1ll << 31), "mega_transpose: matrix side above 2^31");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool fast = dtype != MEGA_F32 && R % 8 == 0 && C % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int64_t side = fast ? kTT : 32;
  const int64_t tiles_r = (R + side - 1) / side, tiles_c = (C + side - 1) / side;
  MEGA_CHECK_ARG(Z * tiles_r * tiles_c < (1ll << 31), "mega_transpose: too many tiles");
  const unsigned grid = static_cast<unsigned>(Z * tiles_r * tiles_c);
  if (fast)
    transpose16_kernel<<<grid, kThreads, 0, s>>>(static_cast<const uint16_t*>(in), static_cast<uint16_t*>(out),
                                                 (int)R, (int)C, (int)tiles_c, (int)tiles_r);
  else if (dtype == MEGA_F32)
    transpose_any_kernel<float><<<grid, kThreads, 0, s>>>(static_cast<const float*>(in), static_cast<float*>(out),
                                                          (int)R, (int)C, (int)tiles_c, (int)tiles_r);
  else
    transpose_any_kernel<uint16_t><<<grid, kThreads, 0, s>>>(static_cast<const uint16_t*>(in),
                                                             static_cast<uint16_t*>(out), (int)R, (int)C,
                                                             (int)tiles_c, (int)tiles_r);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

extern "C" int mega_silu_mul_fwd(const void* a, const void* b, int dtype, int64_t n, void* out,
                                 void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_silu_mul_fwd: unknown dtype %d", dtype);
  MEGA_CHECK_ARG(n >= 0, "mega_silu_mul_fwd: negative size");
  if (n == 0) return MEGA_OK;
  MEGA_CHECK_ARG(a && b && out, "mega_silu_mul_fwd: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32) return launch_silu_mul<MEGA_F32>(nullptr, a, b, out, nullptr, n, s);
  if (dtype == MEGA_BF16) return launch_silu_mul<MEGA_BF16>(nullptr, a, b, out, nullptr, n, s);
  return launch_silu_mul<MEGA_F16>(nullptr, a, b, out, nullptr, n, s);
}

extern "C" int mega_silu_mul_bwd(const void* dout, const void* a, const void* b, int dtype, int64_t n,
                                 void* da, void* db, void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_silu_mul_bwd: unknown dtype %d", dtype);
  MEGA_CHECK_ARG(n >= 0, "mega_silu_mul_bwd: negative size");
  if (n == 0) return MEGA_OK;
  MEGA_CHECK_ARG(dout && a && b && da && db, "mega_silu_mul_bwd: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32) return launch_silu_mul<MEGA_F32>(dout, a, b, da, db, n, s);
  if (dtype == MEGA_BF16) return launch_silu_mul<MEGA_BF16>(dout, a, b, da, db, n, s);
  return launch_silu_mul<MEGA_F16>(dout, a, b, da, db, n, s);
}

extern "C" int mega_split_bf16(const void* src, int dtype, int64_t n, void* hi, void* lo, void* stream) {
  MEGA_CHECK_ARG(dtype == MEGA_F32 || dtype == MEGA_F16, "mega_split_bf16: float32 or float16 input");
  MEGA_CHECK_ARG(n >= 0 && n % 8 == 0, "mega_split_bf16: the element count must be a multiple of 8");
  if (n == 0) return MEGA_OK;
  MEGA_CHECK_ARG(src && hi && lo, "mega_split_bf16: null pointer");
  const auto al = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  MEGA_CHECK_ARG(al(src) && al(hi) && al(lo), "mega_split_bf16: operands must be 16-byte aligned");
  const int64_t n8 = n / 8;
  const unsigned grid = static_cast<unsigned>(std::min<int64_t>((n8 + kThreads - 1) / kThreads, 16384));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32)
    split_bf16_kernel<MEGA_F32><<<grid, kThreads, 0, s>>>(src, static_cast<uint16_t*>(hi), static_cast<uint16_t*>(lo), n8);
  else
    split_bf16_kernel<MEGA_F16><<<grid, kThreads, 0, s>>>(src, static_cast<uint16_t*>(hi), static_cast<uint16_t*>(lo), n8);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}
