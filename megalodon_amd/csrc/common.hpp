// Shared host/device helpers for the gfx950 kernels of libmegalodon_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/megalodon_hip.h"

namespace mega {

constexpr int kWave = 64;  // gfx950 wavefront width

// ---- error reporting --------------------------------------------------
char* last_error_buf();  // thread-local, 512 bytes
int set_error(int code, const char* fmt, ...);

#define MEGA_CHECK_ARG(cond, ...)                                  \
  do {                                                             \
    if (!(cond)) return mega::set_error(MEGA_ERR_INVALID_ARG, __VA_ARGS__); \
  } while (0)

#define MEGA_CHECK_HIP(expr)                                               \
  do {                                                                     \
    hipError_t e_ = (expr);                                                \
    if (e_ != hipSuccess)                                                  \
      return mega::set_error(MEGA_ERR_HIP, "%s failed: %s", #expr,         \
                             hipGetErrorString(e_));                       \
  } while (0)

#define MEGA_CHECK_LAUNCH() MEGA_CHECK_HIP(hipGetLastError())

// ---- 16-bit element conversion (bit-level, round-to-nearest-even) -------
__device__ __forceinline__ float bf16_bits_to_float(uint16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}
// gfx950 converts in hardware (v_cvt_pk_bf16_f32, round to nearest even)
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const bf16x2_t v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float f16_bits_to_float(uint16_t v) {
  return __half2float(__ushort_as_half(v));
}
__device__ __forceinline__ uint16_t float_to_f16_bits(float f) {
  return __half_as_ushort(__float2half_rn(f));
}

// Element traits: storage type + conversion to/from float.
template <int DT> struct Elem;
template <> struct Elem<MEGA_F32> {
  using type = float;
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<MEGA_BF16> {
  using type = uint16_t;
  static __device__ __forceinline__ float load(const uint16_t* p) { return bf16_bits_to_float(*p); }
  static __device__ __forceinline__ void store(uint16_t* p, float v) { *p = float_to_bf16_bits(v); }
};
template <> struct Elem<MEGA_F16> {
  using type = uint16_t;
  static __device__ __forceinline__ float load(const uint16_t* p) { return f16_bits_to_float(*p); }
  static __device__ __forceinline__ void store(uint16_t* p, float v) { *p = float_to_f16_bits(v); }
};

// ---- eight 16-bit elements <-> float -------------------------------------------
// One 16-byte load holds 8 bfloat16 / float16 values; element 2e is the low
// half of word e.
template <int DT>
__device__ __forceinline__ void unpack8(const uint4& q, float* v) {
  const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (DT == MEGA_BF16) {
      v[2 * e] = __uint_as_float(u[e] << 16);
      v[2 * e + 1] = __uint_as_float(u[e] & 0xffff0000u);
    } else {
      v[2 * e] = f16_bits_to_float(static_cast<uint16_t>(u[e] & 0xffffu));
      v[2 * e + 1] = f16_bits_to_float(static_cast<uint16_t>(u[e] >> 16));
    }
  }
}
template <int DT>
__device__ __forceinline__ uint4 pack8(const float* v) {
  uint32_t u[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (DT == MEGA_BF16) {
      u[e] = pack_bf16x2(v[2 * e], v[2 * e + 1]);
    } else {
      u[e] = static_cast<uint32_t>(float_to_f16_bits(v[2 * e])) |
             (static_cast<uint32_t>(float_to_f16_bits(v[2 * e + 1])) << 16);
    }
  }
  return make_uint4(u[0], u[1], u[2], u[3]);
}

inline int elem_size(int dt) { return dt == MEGA_F32 ? 4 : 2; }
inline bool valid_dtype(int dt) { return dt == MEGA_F32 || dt == MEGA_BF16 || dt == MEGA_F16; }

// ---- complex helpers ------------------------------------------------------
struct cf {
  float x, y;
};
__device__ __forceinline__ cf cmul(cf a, cf b) {
  return {a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x};
}
__device__ __forceinline__ cf cmulc(cf a, cf b) {  // a * conj(b)
  return {a.x * b.x + a.y * b.y, a.y * b.x - a.x * b.y};
}
__device__ __forceinline__ cf cadd(cf a, cf b) { return {a.x + b.x, a.y + b.y}; }
__device__ __forceinline__ cf csub(cf a, cf b) { return {a.x - b.x, a.y - b.y}; }

// ---- DPP row reductions --------------------------------------------------------
// v + (v moved by a DPP pattern inside the 16-lane row); folds into one
// v_add_f32_dpp.  0xB1 / 0x4E = quad_perm [1,0,3,2] / [2,3,0,1], 0x141 =
// row_half_mirror, 0x140 = row_mirror.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v),
                                                                    CTRL, 0xf, 0xf, true));
}
// sum over aligned groups of W lanes (W = 2..64), result in every lane of the group
template <int W>
__device__ __forceinline__ float group_sum(float v) {
  if (W >= 2) v = dpp_add<0xB1>(v);
  if (W >= 4) v = dpp_add<0x4E>(v);
  if (W >= 8) v = dpp_add<0x141>(v);
  if (W >= 16) v = dpp_add<0x140>(v);
  if (W >= 32) v += __shfl_xor(v, 16, 64);
  if (W >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// ---- wave64 reductions ------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// ---- counter-based random numbers -------------------------------------------
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
// SC'11): four 32-bit words as a pure function of a 128-bit counter and a
// 64-bit key.
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                              uint32_t k0, uint32_t k1, uint32_t* out) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// 16-byte accesses with the non-temporal hint: for tensors a kernel writes once in whole
// 128-byte lines and does not read again (stores), or reads once (loads).  Such stores do not
// displace what the kernel still reads; partial lines written with the hint are slow.
typedef uint32_t nt_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_streaming(void* ptr, uint4 v) {
  nt_u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, static_cast<nt_u32x4*>(ptr));
}
__device__ __forceinline__ uint4 load_once(const void* ptr) {
  const nt_u32x4 v = __builtin_nontemporal_load(static_cast<const nt_u32x4*>(ptr));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

}  // namespace mega
