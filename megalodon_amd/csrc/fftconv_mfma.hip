// Causal convolution of 16-bit rows with the DFT stages on the matrix cores.
//
// One workgroup (8 waves) owns one row at a time.  The zero-padded real row of
// 2N = 65536 samples is packed as z[n] = s[2n] + i s[2n+1], n < N = 32768, and
// kept in LDS as fp16 re and im values (rows of a, re half then im half).  The N-point transform is three
// radix-32 stages over the digits of n = 1024 a + 32 b + c:
//     forward  F1 over a, F2 over b, F3 over c  -> Z[k1 + 32 k2 + 1024 k3] at (k1, k2, k3)
//     inverse  I1 over c, I2 over b, I3 over a  -> z[n] back at (a, b, c)
// (the inverse undoes the forward steps in reverse order, conjugated)
// every stage in place: a wave takes a 32 x 32 tile (32 transform points x 32
// bystanders), multiplies it by the 32 x 32 DFT matrix with 8 MFMAs
// (v_mfma_f32_32x32x16_f16, complex = 4 real products, K = 32), applies the
// stage's twiddle in fp32, rounds to fp16 and writes the tile back.  The DFT
// matrices carry 1/sqrt(32), so each stage is unitary and values keep their
// magnitude; rows are pre-scaled by a power of two so that fp16 neither
// overflows nor flushes the row to zero.  The spectrum of the second operand
// (the kernel row) waits in registers while the first operand is transformed;
// the real-signal product is formed on conjugate bin pairs (k, N - k).
//
// Used for bf16 / fp16 rows with 16384 < L <= 32768 and L % 8 == 0; everything else
// stays with the fp32 VALU engine of fftconv.hip.
#include "common.hpp"
#include "fftconv_mfma.hpp"

namespace mega {
namespace fftm {
namespace {

constexpr int kN = 32768;             // complex points per transform
// LDS: row a holds its 1024 re values, 16 elements of padding, then its 1024 im
// values and padding.  The a-stride of 1040 dwords is 16 mod 64 banks, and the
// im value of an element sits a constant 2080 bytes after its re value, which
// every access folds into the instruction's immediate offset.
constexpr int kIm = 1024 + 16;        // elements from a re value to its im value
constexpr int kRS = 2 * kIm;          // elements between consecutive a
constexpr int kPlane = 16 * kRS;      // half of the LDS elements (two "planes" of 32 half rows)
constexpr int kThreads = 512;         // 8 waves, two per SIMD
constexpr int kWaves = kThreads / kWave;
constexpr size_t kLdsBytes = sizeof(uint16_t) * 2 * kPlane + 64;

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// LDS element offset of digit triple (a, b, c).  Bits 3-4 of c are XORed with
// two bits taken from a and b so that both the 8-byte tile writes (lanes along
// a or b) and the transposing reads (4 consecutive a or b) spread over the banks.
__device__ __forceinline__ int pos(int a, int b, int c) {
  return a * kRS + 32 * b + (c ^ ((((a >> 2) ^ (b >> 2)) & 3) << 3));
}

__device__ __forceinline__ floatx16 mfma(u32x4 a, u32x4 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                __builtin_bit_cast(half8, b), c, 0, 0, 0);
}
__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) {
  const half2v v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ void unpack_h2(uint32_t u, float& lo, float& hi) {
  const half2v v = __builtin_bit_cast(half2v, u);
  lo = static_cast<float>(v[0]);
  hi = static_cast<float>(v[1]);
}
__device__ __forceinline__ float h2f(uint16_t u) {
  return static_cast<float>(__builtin_bit_cast(_Float16, u));
}
__device__ __forceinline__ uint16_t f2h(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}
// Makes a lane-derived value opaque to the optimiser.  Twiddles, LDS offsets and
// bin-pair indices depend only on the lane and the tile, not on the row: left
// alone they are hoisted out of the persistent row loop into hundreds of
// spilled registers.  Recomputing them per tile is cheaper than reloading them.
__device__ __forceinline__ int opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}
// Workgroup barrier that waits for this wave's LDS traffic only: global loads
// issued earlier (the prefetch of the next operand row) stay in flight.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// (cos, sin)(2 pi j / 2^logn) from the hardware's revolution-based sin / cos
__device__ __forceinline__ void cis(int j, float inv_n, float& c, float& s) {
  const float x = static_cast<float>(j) * inv_n;
  c = __builtin_amdgcn_cosf(x);
  s = __builtin_amdgcn_sinf(x);
}
// transposing 8-byte LDS read: lane t of a 16-lane group receives column t of
// the 4 rows its group's source lanes point at (source lane 4a + b: row a,
// columns 4b .. 4b+3)
__device__ __forceinline__ uint2 lds_read_tr(const uint16_t* q) {
  const short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) short4v*)(q));
  return __builtin_bit_cast(uint2, v);
}

// The 32 x 32 DFT matrix W[k][j] = exp(-2 pi i k j / 32) / sqrt(32) in MFMA operand
// form (lane l: j = l % 32, k = 16 s + 8 (l / 32) + e).  W is symmetric, so the
// same registers serve as the A or the B operand.
struct Dft {
  u32x4 re[2], im[2], nim[2];  // cos, -sin, +sin
};
__device__ __forceinline__ Dft make_dft(int lane) {
  Dft w;
  const int j = lane & 31, g = lane >> 5;
  const float sc = 0.17677669529663687f;  // 1 / sqrt(32)
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    float c[8], sn[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      cis(((16 * s + 8 * g + e) * j) & 31, 1.f / 32.f, c[e], sn[e]);
      c[e] *= sc;
      sn[e] *= sc;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      w.re[s][e] = pack_h2(c[2 * e], c[2 * e + 1]);
      w.im[s][e] = pack_h2(-sn[2 * e], -sn[2 * e + 1]);
      w.nim[s][e] = pack_h2(sn[2 * e], sn[2 * e + 1]);
    }
  }
  return w;
}

// D = X W (X as the A operand: rows = bystanders, k = transform index).
// Result: lane <-> output frequency, registers <-> bystanders.
template <bool INV, int KSTEPS>
__device__ __forceinline__ void dft_xa(const u32x4* xr, const u32x4* xi, const Dft& w,
                                       floatx16& dr, floatx16& di) {
#pragma unroll
  for (int r = 0; r < 16; ++r) dr[r] = di[r] = 0.f;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    dr = mfma(xr[s], w.re[s], dr);
    dr = mfma(xi[s], INV ? w.im[s] : w.nim[s], dr);  // -Xi Wi
    di = mfma(xr[s], INV ? w.nim[s] : w.im[s], di);
    di = mfma(xi[s], w.re[s], di);
  }
}
// D = W X (X as the B operand: columns = bystanders).  Result: lane <->
// bystander, registers <-> output frequency.
template <bool INV>
__device__ __forceinline__ void dft_xb(const u32x4* xr, const u32x4* xi, const Dft& w,
                                       floatx16& dr, floatx16& di) {
#pragma unroll
  for (int r = 0; r < 16; ++r) dr[r] = di[r] = 0.f;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    dr = mfma(w.re[s], xr[s], dr);
    dr = mfma(INV ? w.im[s] : w.nim[s], xi[s], dr);
    di = mfma(INV ? w.nim[s] : w.im[s], xr[s], di);
    di = mfma(w.re[s], xi[s], di);
  }
}

// exp(+i 2 pi c m / N) for the 16 values c = 8 qd + 4 g + e a lane holds after a
// stage (register 4 qd + e), from three sin/cos pairs and complex products:
// W^(c m) = W^(4 g m) (W^(8 m))^qd (W^m)^e.
struct Tw16 {
  float c[16], s[16];
};
__device__ __forceinline__ void cmul(float ar, float ai, float br, float bi, float& cr, float& ci) {
  cr = ar * br - ai * bi;
  ci = ar * bi + ai * br;
}
__device__ __forceinline__ Tw16 twiddles16(int m, int g) {
  Tw16 t;
  float t1c, t1s, t2c, t2s, t3c, t3s, bc, bs, s8c, s8s;
  cis(m & (kN - 1), 1.f / kN, t1c, t1s);
  cis((4 * g * m) & (kN - 1), 1.f / kN, bc, bs);
  cis((8 * m) & (kN - 1), 1.f / kN, s8c, s8s);
  cmul(t1c, t1s, t1c, t1s, t2c, t2s);
  cmul(t2c, t2s, t1c, t1s, t3c, t3s);
  float qc = bc, qs = bs;
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    t.c[4 * qd] = qc;
    t.s[4 * qd] = qs;
    cmul(qc, qs, t1c, t1s, t.c[4 * qd + 1], t.s[4 * qd + 1]);
    cmul(qc, qs, t2c, t2s, t.c[4 * qd + 2], t.s[4 * qd + 2]);
    cmul(qc, qs, t3c, t3s, t.c[4 * qd + 3], t.s[4 * qd + 3]);
    if (qd < 3) {
      float nc, ns;
      cmul(qc, qs, s8c, s8s, nc, ns);
      qc = nc;
      qs = ns;
    }
  }
  return t;
}
// v *= exp(-i theta) (forward) or exp(+i theta) (CONJ), theta given by (c, s)
template <bool CONJ>
__device__ __forceinline__ void apply_tw(floatx16& dr, floatx16& di, const Tw16& t) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float vr = dr[r], vi = di[r], tc = t.c[r], ts = CONJ ? -t.s[r] : t.s[r];
    dr[r] = vr * tc + vi * ts;
    di[r] = vi * tc - vr * ts;
  }
}

// Per-lane pieces of the LDS offsets (elements), computed once per stage call.
// A tile adds its own digit (wave-uniform, scalar) and XORs its swizzle bits.
struct LaneGeo {
  int g, f;         // lane / 32, lane % 32
  int rd[2];        // transposing read, h = 0, 1: row part + swizzled source column
  int wr;           // tile write: lane part
};
// quad slot q of a tile write lands at 8 (q ^ x): x = swizzle bits of (tile digit, lane digit)
__device__ __forceinline__ void write_tile_x(uint16_t* pre, const floatx16& dr, const floatx16& di,
                                             int base, int x) {
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    uint16_t* q = pre + base + ((qd ^ x) << 3);
    *reinterpret_cast<uint2*>(q) =
        make_uint2(pack_h2(dr[4 * qd], dr[4 * qd + 1]), pack_h2(dr[4 * qd + 2], dr[4 * qd + 3]));
    *reinterpret_cast<uint2*>(q + kIm) =
        make_uint2(pack_h2(di[4 * qd], di[4 * qd + 1]), pack_h2(di[4 * qd + 2], di[4 * qd + 3]));
  }
}
template <int KSTEPS, int SSTRIDE>
__device__ __forceinline__ void read_tile_tr(const uint16_t* pre, int o0, int o1, u32x4* xr,
                                             u32x4* xi) {
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const uint2 r0 = lds_read_tr(pre + o0 + s * SSTRIDE), r1 = lds_read_tr(pre + o1 + s * SSTRIDE);
    const uint2 i0 = lds_read_tr(pre + o0 + s * SSTRIDE + kIm);
    const uint2 i1 = lds_read_tr(pre + o1 + s * SSTRIDE + kIm);
    xr[s] = u32x4{r0.x, r0.y, r1.x, r1.y};
    xi[s] = u32x4{i0.x, i0.y, i1.x, i1.y};
  }
}

// ---- stages over a (F1 / I3): tile = fixed b, rows a, bystander c -------------
// F1 (a -> k1): only a < 16 holds data (zero padding) -> one k-step; then
// twiddle W_1024^(b k1), one factor per lane.  I3 (k1 -> a): all 32 rows, no twiddle.
template <bool INV>
__device__ __forceinline__ void stage_a(uint16_t* pre, const Dft& w, int wave, int lane) {
  lane = opaque(lane) & 63;
  const int g = lane >> 5, f = lane & 31;
  const int rsrc = 8 * g + ((lane & 15) >> 2), csrc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  // pos(16 s + rsrc + 4 h, b, csrc): the row's swizzle bits are (2 g + h) & 3
  const int rd0 = rsrc * kRS + (csrc ^ (((2 * g) & 3) << 3));
  const int rd1 = (rsrc + 4) * kRS + (csrc ^ (((2 * g + 1) & 3) << 3));
  const int wr = f * kRS + 4 * g, fx = (f >> 2) & 3;
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  for (int b = wv; b < 32; b += kWaves) {
    const int bx = ((b >> 2) & 3) << 3;
    u32x4 xr[2], xi[2];
    read_tile_tr<INV ? 2 : 1, 16 * kRS>(pre, (rd0 ^ bx) + 32 * b, (rd1 ^ bx) + 32 * b, xr, xi);
    floatx16 dr, di;
    dft_xa<INV, INV ? 2 : 1>(xr, xi, w, dr, di);
    if (!INV) {
      float tc, ts;
      cis((b * f) & 1023, 1.f / 1024.f, tc, ts);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float vr = dr[r], vi = di[r];
        dr[r] = vr * tc + vi * ts;  // (vr + i vi)(tc - i ts)
        di[r] = vi * tc - vr * ts;
      }
    }
    write_tile_x(pre, dr, di, wr + 32 * b, fx ^ (bx >> 3));
  }
}

// ---- stages over b (F2 / I2): tile = fixed a, rows b, bystander c -------------
// F2 (b -> k2): then twiddle W_N^(c (a + 32 k2)).  I2 (k2 -> n2): undoes F1's
// twiddle, conj W_1024^(n2 a), one factor per lane.
template <bool INV>
__device__ __forceinline__ void stage_b(uint16_t* pre, const Dft& w, int wave, int lane) {
  lane = opaque(lane) & 63;
  const int g = lane >> 5, f = lane & 31;
  const int rsrc = 8 * g + ((lane & 15) >> 2), csrc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int rd0 = 32 * rsrc + (csrc ^ (((2 * g) & 3) << 3));
  const int rd1 = 32 * (rsrc + 4) + (csrc ^ (((2 * g + 1) & 3) << 3));
  const int wr = 32 * f + 4 * g, fx = (f >> 2) & 3;
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  for (int a = wv; a < 32; a += kWaves) {
    const int ax = ((a >> 2) & 3) << 3;
    u32x4 xr[2], xi[2];
    read_tile_tr<2, 512>(pre, (rd0 ^ ax) + a * kRS, (rd1 ^ ax) + a * kRS, xr, xi);
    floatx16 dr, di;
    dft_xa<INV, 2>(xr, xi, w, dr, di);
    if (!INV) {
      const Tw16 t = twiddles16(a + 32 * f, g);
      apply_tw<false>(dr, di, t);
    } else {
      float tc, ts;
      cis((a * f) & 1023, 1.f / 1024.f, tc, ts);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float vr = dr[r], vi = di[r];
        dr[r] = vr * tc - vi * ts;  // (vr + i vi)(tc + i ts)
        di[r] = vi * tc + vr * ts;
      }
    }
    write_tile_x(pre, dr, di, wr + a * kRS, fx ^ (ax >> 3));
  }
}

// ---- stages over c (F3 / I1): tile = fixed a, lanes b, rows c (contiguous) ----
// F3 (c -> k3): no twiddle.  I1 (k3 -> n3): then undoes F2's twiddle,
// conj W_N^(n3 (a + 32 b)).
template <bool INV>
__device__ __forceinline__ void stage_c(uint16_t* pre, const Dft& w, int wave, int lane) {
  lane = opaque(lane) & 63;
  const int g = lane >> 5, b = lane & 31;
  const int bx = (b >> 2) & 3, row = 32 * b;
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  for (int a = wv; a < 32; a += kWaves) {
    const int x = bx ^ ((a >> 2) & 3);
    // pos(a, b, 16 s + 8 g) = row part + 8 ((2 s + g) ^ x)
    const int base = a * kRS + row;
    u32x4 xr[2], xi[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint16_t* q = pre + base + (((2 * s + g) ^ x) << 3);
      xr[s] = *reinterpret_cast<const u32x4*>(q);
      xi[s] = *reinterpret_cast<const u32x4*>(q + kIm);
    }
    floatx16 dr, di;
    dft_xb<INV>(xr, xi, w, dr, di);
    if (INV) {
      const Tw16 t = twiddles16(a + 32 * b, g);
      apply_tw<true>(dr, di, t);
    }
    write_tile_x(pre, dr, di, base + 4 * g, x);
  }
}

template <bool INV>
__device__ __forceinline__ void transform(uint16_t* pre, uint16_t* pim, const Dft& w, int wave,
                                          int lane) {
  if (!INV) {
    stage_a<false>(pre, w, wave, lane);
    lds_barrier();
    stage_b<false>(pre, w, wave, lane);
    lds_barrier();
    stage_c<false>(pre, w, wave, lane);
    lds_barrier();
  } else {
    stage_c<true>(pre, w, wave, lane);
    lds_barrier();
    stage_b<true>(pre, w, wave, lane);
    lds_barrier();
    stage_a<true>(pre, w, wave, lane);
    lds_barrier();
  }
}

// ---- rows in and out -------------------------------------------------------
// Four consecutive sample pairs (s[2n], s[2n+1]), n = n0 .. n0+3, as one access.
template <int DT> struct QuadIo;
template <> struct QuadIo<MEGA_F32> {
  struct Raw { f32x4 u, v; };
  static __device__ __forceinline__ Raw fetch(const void* row, unsigned n0) {
    const f32x4* p = reinterpret_cast<const f32x4*>(static_cast<const char*>(row) + n0 * 8u);
    return Raw{p[0], p[1]};
  }
  static __device__ __forceinline__ Raw zero() { return Raw{f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}}; }
  static __device__ __forceinline__ void unpack(const Raw& r, float* lo, float* hi) {
    lo[0] = r.u[0]; hi[0] = r.u[1]; lo[1] = r.u[2]; hi[1] = r.u[3];
    lo[2] = r.v[0]; hi[2] = r.v[1]; lo[3] = r.v[2]; hi[3] = r.v[3];
  }
  static __device__ __forceinline__ void load(const void* row, unsigned n0, float* lo, float* hi) {
    unpack(fetch(row, n0), lo, hi);
  }
  static __device__ __forceinline__ void store(void* row, unsigned n0, const float* lo, const float* hi) {
    float4* p = reinterpret_cast<float4*>(static_cast<char*>(row) + n0 * 8u);
    p[0] = make_float4(lo[0], hi[0], lo[1], hi[1]);
    p[1] = make_float4(lo[2], hi[2], lo[3], hi[3]);
  }
};
template <> struct QuadIo<MEGA_BF16> {
  typedef u32x4 Raw;
  static __device__ __forceinline__ Raw fetch(const void* row, unsigned n0) {
    return *reinterpret_cast<const u32x4*>(static_cast<const char*>(row) + n0 * 4u);
  }
  static __device__ __forceinline__ Raw zero() { return u32x4{0u, 0u, 0u, 0u}; }
  static __device__ __forceinline__ void unpack(const Raw& u, float* lo, float* hi) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = __uint_as_float(u[e] << 16);
      hi[e] = __uint_as_float(u[e] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void load(const void* row, unsigned n0, float* lo, float* hi) {
    unpack(fetch(row, n0), lo, hi);
  }
  static __device__ __forceinline__ void store(void* row, unsigned n0, const float* lo, const float* hi) {
    *reinterpret_cast<uint4*>(static_cast<char*>(row) + n0 * 4u) =
        make_uint4(pack_bf16x2(lo[0], hi[0]), pack_bf16x2(lo[1], hi[1]), pack_bf16x2(lo[2], hi[2]),
                   pack_bf16x2(lo[3], hi[3]));
  }
};
template <> struct QuadIo<MEGA_F16> {
  typedef u32x4 Raw;
  static __device__ __forceinline__ Raw fetch(const void* row, unsigned n0) {
    return *reinterpret_cast<const u32x4*>(static_cast<const char*>(row) + n0 * 4u);
  }
  static __device__ __forceinline__ Raw zero() { return u32x4{0u, 0u, 0u, 0u}; }
  static __device__ __forceinline__ void unpack(const Raw& v, float* lo, float* hi) {
#pragma unroll
    for (int e = 0; e < 4; ++e) unpack_h2(v[e], lo[e], hi[e]);
  }
  static __device__ __forceinline__ void load(const void* row, unsigned n0, float* lo, float* hi) {
    unpack(fetch(row, n0), lo, hi);
  }
  static __device__ __forceinline__ void store(void* row, unsigned n0, const float* lo, const float* hi) {
    *reinterpret_cast<uint4*>(static_cast<char*>(row) + n0 * 4u) =
        make_uint4(pack_h2(lo[0], hi[0]), pack_h2(lo[1], hi[1]), pack_h2(lo[2], hi[2]),
                   pack_h2(lo[3], hi[3]));
  }
};

// A row in flight: a thread's 8 quads n0 = 4 (tid + 512 j) of sample pairs
// (reversed order when flip), as loaded.  L % 8 == 0 keeps quads whole.
template <int DT>
struct RowRegs {
  typename QuadIo<DT>::Raw q[8];
};
template <int DT>
__device__ __forceinline__ void fetch_row(RowRegs<DT>& r, const void* row, int L, bool flip,
                                          int tid) {
  const unsigned half = static_cast<unsigned>(L) >> 1;
  tid = opaque(tid) & (kThreads - 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const unsigned n0 = 4u * (static_cast<unsigned>(tid) + kThreads * j);
    r.q[j] = QuadIo<DT>::zero();
    if (n0 < half) r.q[j] = QuadIo<DT>::fetch(row, flip ? half - 4u - n0 : n0);
  }
}
// Writes the fetched row to the planes as z[n] = s[2n] + i s[2n+1], n < 16384
// (zeros beyond the row), scaled by a power of two so that max |s| lands in
// [1/8, 1/4).  Returns the scale.  `red` is 8 floats of LDS.  Ends with a barrier.
template <int DT>
__device__ __forceinline__ float place_row(uint16_t* pre, uint16_t* pim, float* red,
                                           const RowRegs<DT>& r, bool flip, int tid) {
  tid = opaque(tid) & (kThreads - 1);
  float re[8][4], im[8][4];
  float m = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float lo[4], hi[4];
    QuadIo<DT>::unpack(r.q[j], lo, hi);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      re[j][e] = flip ? hi[3 - e] : lo[e];
      im[j][e] = flip ? lo[3 - e] : hi[e];
      m = fmaxf(m, fmaxf(fabsf(re[j][e]), fabsf(im[j][e])));
    }
  }
  m = wave_max(m);
  if ((tid & (kWave - 1)) == 0) red[tid / kWave] = m;
  lds_barrier();
  m = red[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) m = fmaxf(m, red[i]);
  // 2^-(e+2) with m = f 2^e, f in [0.5, 1); finite non-zero m only
  float scale = 1.f;
  if (m > 0.f && m < 3.0e38f) {
    int e;
    (void)frexpf(m, &e);
    scale = ldexpf(1.f, -(e + 2));
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int n0 = 4 * (tid + kThreads * j);
    const int o = pos(n0 >> 10, (n0 >> 5) & 31, n0 & 31);
    *reinterpret_cast<uint2*>(pre + o) = make_uint2(pack_h2(re[j][0] * scale, re[j][1] * scale),
                                                    pack_h2(re[j][2] * scale, re[j][3] * scale));
    *reinterpret_cast<uint2*>(pim + o) = make_uint2(pack_h2(im[j][0] * scale, im[j][1] * scale),
                                                    pack_h2(im[j][2] * scale, im[j][3] * scale));
  }
  lds_barrier();
  return scale;
}

// out[2n] = re z[n] * scale (+ w res[2n]), out[2n+1] likewise, n < L/2
// (reversed when flip); ACC adds to what is there (fp32 rows).
template <int DT, bool ACC>
__device__ __forceinline__ void store_row(const uint16_t* pre, const uint16_t* pim, void* row,
                                          int L, bool flip, float scale, const void* res, float w,
                                          int tid) {
  const unsigned half = static_cast<unsigned>(L) >> 1;
  tid = opaque(tid) & (kThreads - 1);
#pragma unroll 2
  for (int j = 0; j < 8; ++j) {
    const unsigned n0 = 4u * (static_cast<unsigned>(tid) + kThreads * j);
    if (n0 < half) {
      const int o = pos(n0 >> 10, (n0 >> 5) & 31, n0 & 31);
      const uint2 ur = *reinterpret_cast<const uint2*>(pre + o);
      const uint2 ui = *reinterpret_cast<const uint2*>(pim + o);
      float zr[4], zi[4], lo[4], hi[4];
      unpack_h2(ur.x, zr[0], zr[1]);
      unpack_h2(ur.y, zr[2], zr[3]);
      unpack_h2(ui.x, zi[0], zi[1]);
      unpack_h2(ui.y, zi[2], zi[3]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = (flip ? zi[3 - e] : zr[e]) * scale;
        hi[e] = (flip ? zr[3 - e] : zi[e]) * scale;
      }
      const unsigned m0 = flip ? half - 4u - n0 : n0;
      if (ACC) {
        float plo[4], phi[4];
        QuadIo<DT>::load(row, m0, plo, phi);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] += plo[e];
          hi[e] += phi[e];
        }
      }
      if (res != nullptr) {
        float rlo[4], rhi[4];
        QuadIo<DT>::load(res, m0, rlo, rhi);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] = fmaf(w, rlo[e], lo[e]);
          hi[e] = fmaf(w, rhi[e], hi[e]);
        }
      }
      QuadIo<DT>::store(row, m0, lo, hi);
    }
  }
}

// ---- conjugate bin pairs ------------------------------------------------------
// Bin k = k1 + 32 k2 + 1024 k3 sits at (k1, k2, k3); its partner N - k at the
// mirrored row (k1', k2') = (32 - k1, 31 - k2) (k1 != 0) or (0, 32 - k2), with
// k3' = 31 - k3.  Row (0, 0) is its own mirror with k3' = (32 - k3) % 32 and is
// handled apart.  The other 1023 rows form 511 pairs plus the self-mirrored row
// (0, 16): row pair q of 512 is
//   q < 480: (1 + q / 32, q % 32);  480..495: (16, q - 480);  496..510: (0, q - 495);  511: (0, 16).
// A lane takes one quad of a row pair: bins k3 = 4u .. 4u+3 of the row and the
// reversed quad 7 - u of the mirror row; task T = tid + 512 i -> q = T / 8, u = T % 8.
struct RowPair {
  int ok, om;   // LDS offsets of the two quads
  int k0;       // bin index of the quad's first element: k1 + 32 k2 + 4096 u
  bool writes;  // false for the duplicate lanes of the self-mirrored row
};
__device__ __forceinline__ RowPair row_pair(int task) {
  const int q = task >> 3, u = task & 7;
  int k1, k2;
  if (q < 480) {
    k1 = 1 + (q >> 5);
    k2 = q & 31;
  } else if (q < 496) {
    k1 = 16;
    k2 = q - 480;
  } else if (q < 511) {
    k1 = 0;
    k2 = q - 495;
  } else {
    k1 = 0;
    k2 = 16;
  }
  const int m1 = k1 != 0 ? 32 - k1 : 0;
  const int m2 = k1 != 0 ? 31 - k2 : 32 - k2;
  RowPair r;
  r.ok = pos(k1, k2, 4 * u);
  r.om = pos(m1, m2, 4 * (7 - u));
  r.k0 = k1 + 32 * k2 + 4096 * u;
  r.writes = q != 511 || u < 4;
  return r;
}
__device__ __forceinline__ void read_quad(const uint16_t* p, float* v) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  unpack_h2(u.x, v[0], v[1]);
  unpack_h2(u.y, v[2], v[3]);
}
__device__ __forceinline__ void write_quad(uint16_t* p, const float* v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]));
}

// E = (Z(k) + conj Z(m)) / 2,  O = (Z(k) - conj Z(m)) / (2i)
__device__ __forceinline__ void untangle(float zkr, float zki, float zmr, float zmi, float& er,
                                         float& ei, float& orr, float& oi) {
  er = 0.5f * (zkr + zmr);
  ei = 0.5f * (zki - zmi);
  orr = 0.5f * (zki + zmi);
  oi = 0.5f * (zmr - zkr);
}
// Zy(k) = Ey + i Oy and Zy(m) = conj Ey + i conj Oy with
// Ey = Ea Eb + W_N^k Oa Ob, Oy = Ea Ob + Oa Eb;  W_N^k = wc - i ws
__device__ __forceinline__ void bin_product(float ar, float ai, float pr, float pi, float br,
                                            float bi, float qr, float qi, float wc, float ws,
                                            float& zkr, float& zki, float& zmr, float& zmi) {
  const float oor = pr * qr - pi * qi, ooi = pr * qi + pi * qr;  // Oa Ob
  const float eyr = ar * br - ai * bi + (oor * wc + ooi * ws);
  const float eyi = ar * bi + ai * br + (ooi * wc - oor * ws);
  const float oyr = ar * qr - ai * qi + pr * br - pi * bi;
  const float oyi = ar * qi + ai * qr + pr * bi + pi * br;
  zkr = eyr - oyi;
  zki = eyi + oyr;
  zmr = eyr + oyi;
  zmi = oyr - eyi;
}

struct Spectrum {
  uint32_t e[8][4], o[8][4];  // E(k), O(k) of the parked operand per task and element, fp16 (re, im)
  uint32_t e0, o0;            // row (0, 0), lane = k3 (threads 0..31)
};

__device__ __forceinline__ void capture_spectrum(const uint16_t* pre, const uint16_t* pim,
                                                 Spectrum& sp, int tid) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    tid = opaque(tid) & (kThreads - 1);
    const RowPair rp = row_pair(tid + kThreads * i);
    float kr[4], ki[4], mr[4], mi[4];
    read_quad(pre + rp.ok, kr);
    read_quad(pim + rp.ok, ki);
    read_quad(pre + rp.om, mr);
    read_quad(pim + rp.om, mi);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float er, ei, orr, oi;
      untangle(kr[e], ki[e], mr[3 - e], mi[3 - e], er, ei, orr, oi);
      sp.e[i][e] = pack_h2(er, ei);
      sp.o[i][e] = pack_h2(orr, oi);
    }
  }
  sp.e0 = sp.o0 = 0u;
  tid = opaque(tid) & (kThreads - 1);
  if (tid < 32) {
    const int ok = pos(0, 0, tid), om = pos(0, 0, (32 - tid) & 31);
    float er, ei, orr, oi;
    untangle(h2f(pre[ok]), h2f(pim[ok]), h2f(pre[om]), h2f(pim[om]), er, ei, orr, oi);
    sp.e0 = pack_h2(er, ei);
    sp.o0 = pack_h2(orr, oi);
  }
}

// the product of the two real signals' spectra, written over Za
__device__ __forceinline__ void pointwise(uint16_t* pre, uint16_t* pim, const Spectrum& sp,
                                          int tid) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    tid = opaque(tid) & (kThreads - 1);
    const RowPair rp = row_pair(tid + kThreads * i);
    float kr[4], ki[4], mr[4], mi[4];
    read_quad(pre + rp.ok, kr);
    read_quad(pim + rp.ok, ki);
    read_quad(pre + rp.om, mr);
    read_quad(pim + rp.om, mi);
    float w0c, w0s;
    cis(rp.k0, 1.f / kN, w0c, w0s);
    // W_N^(k0 + 1024 e) = W_N^k0 W_32^e
    const float c32[4] = {1.f, 0.98078528040323043f, 0.92387953251128674f, 0.83146961230254524f};
    const float s32[4] = {0.f, 0.19509032201612825f, 0.38268343236508978f, 0.55557023301960218f};
    float okr[4], oki[4], omr[4], omi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float ar, ai, pr, pi, br, bi, qr, qi, wc, ws;
      untangle(kr[e], ki[e], mr[3 - e], mi[3 - e], ar, ai, pr, pi);
      unpack_h2(sp.e[i][e], br, bi);
      unpack_h2(sp.o[i][e], qr, qi);
      cmul(w0c, w0s, c32[e], s32[e], wc, ws);
      bin_product(ar, ai, pr, pi, br, bi, qr, qi, wc, ws, okr[e], oki[e], omr[3 - e], omi[3 - e]);
    }
    if (rp.writes) {
      write_quad(pre + rp.ok, okr);
      write_quad(pim + rp.ok, oki);
      write_quad(pre + rp.om, omr);
      write_quad(pim + rp.om, omi);
    }
  }
  tid = opaque(tid) & (kThreads - 1);
  if (tid < 32) {
    const int m3 = (32 - tid) & 31;
    const int ok = pos(0, 0, tid), om = pos(0, 0, m3);
    float ar, ai, pr, pi, br, bi, qr, qi, wc, ws, zkr, zki, zmr, zmi;
    untangle(h2f(pre[ok]), h2f(pim[ok]), h2f(pre[om]), h2f(pim[om]), ar, ai, pr, pi);
    unpack_h2(sp.e0, br, bi);
    unpack_h2(sp.o0, qr, qi);
    cis(1024 * tid, 1.f / kN, wc, ws);
    bin_product(ar, ai, pr, pi, br, bi, qr, qi, wc, ws, zkr, zki, zmr, zmi);
    if (tid <= m3) {
      pre[ok] = f2h(zkr);
      pim[ok] = f2h(zki);
      pre[om] = f2h(zmr);
      pim[om] = f2h(zmi);
    }
  }
}

// MODE 0: out[b,d,:] = conv(a[b,d,:], k[d,:]) (+ omega[d] a[b,d,:]); `flip`
//         reverses a on load and the result on store (backward dx); k fp32.
// MODE 1: out[d,:] (+)= reverse(conv(reverse(a[b0,d,:]), x[b0,d,:])), fp32 out,
//         `flip` != 0 accumulates (backward dk, one batch index per launch).
template <int DT, int MODE>
__global__ __launch_bounds__(kThreads) void fftconv_mfma_kernel(
    const void* __restrict__ a, const void* __restrict__ b, void* __restrict__ out, int rows,
    int D, int L, int flip, const float* __restrict__ omega) {
  extern __shared__ __align__(16) uint16_t lds[];
  uint16_t* pre = lds;
  uint16_t* pim = lds + kIm;
  float* red = reinterpret_cast<float*>(lds + 2 * kPlane);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const Dft w = make_dft(lane);
  const int64_t esz = 2;

  // Software pipeline over the rows of this workgroup: the first-operand row is
  // fetched while the second operand is transformed, and the next row's second
  // operand while the inverse transform runs.
  typedef RowRegs<MODE == 0 ? MEGA_F32 : DT> RegsB;
  auto brow_of = [&](int64_t row) -> const void* {
    if (MODE == 0) return static_cast<const float*>(b) + (row % D) * L;
    return static_cast<const char*>(b) + row * L * esz;
  };
  RegsB rb;
  if (blockIdx.x < rows) fetch_row(rb, brow_of(blockIdx.x), L, false, tid);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const int64_t d = row % D;
    const char* arow = static_cast<const char*>(a) + row * L * esz;
    const bool flip_a = MODE == 1 || flip != 0;
    const float sb = place_row(pre, pim, red, rb, false, tid);
    RowRegs<DT> ra;
    fetch_row(ra, arow, L, flip_a, tid);
    transform<false>(pre, pim, w, wave, lane);
    Spectrum sp;
    capture_spectrum(pre, pim, sp, tid);
    lds_barrier();
    const float sa = place_row(pre, pim, red, ra, flip_a, tid);
    transform<false>(pre, pim, w, wave, lane);
    pointwise(pre, pim, sp, tid);
    lds_barrier();
    if (row + gridDim.x < rows) fetch_row(rb, brow_of(row + gridDim.x), L, false, tid);
    transform<true>(pre, pim, w, wave, lane);
    const float scale = 181.01933598375618f / (sa * sb);  // sqrt(N) / (row scales)
    if (MODE == 0) {
      store_row<DT, false>(pre, pim, static_cast<char*>(out) + row * L * esz, L, flip != 0, scale,
                           omega != nullptr ? arow : nullptr, omega != nullptr ? omega[d] : 0.f, tid);
    } else {
      float* orow = static_cast<float*>(out) + row * L;
      if (flip)
        store_row<MEGA_F32, true>(pre, pim, orow, L, true, scale, nullptr, 0.f, tid);
      else
        store_row<MEGA_F32, false>(pre, pim, orow, L, true, scale, nullptr, 0.f, tid);
    }
    lds_barrier();  // the planes are rewritten by the next row's operand
  }
}

// Backward of one channel in one pass: dy is transformed once and its spectrum
// parked; then k (-> dx) and x (-> dk) are each transformed, multiplied with
// it and transformed back.
//   dx[b,d,:] = reverse(conv(reverse(dy[b,d,:]), k[d,:])) (+ omega[d] dy[b,d,:])
//   dk[d,:]   = sum_b reverse(conv(reverse(dy[b,d,:]), x[b,d,:]))
// A workgroup owns channels d = blockIdx.x, + gridDim.x, ... and walks the batch
// itself, so dk accumulates in order without atomics.
template <int DT>
__global__ __launch_bounds__(kThreads) void fftconv_mfma_bwd_kernel(
    const void* __restrict__ dy, const void* __restrict__ x, const float* __restrict__ k,
    void* __restrict__ dx, float* __restrict__ dk, int B, int D, int L,
    const float* __restrict__ omega) {
  extern __shared__ __align__(16) uint16_t lds[];
  uint16_t* pre = lds;
  uint16_t* pim = lds + kIm;
  float* red = reinterpret_cast<float*>(lds + 2 * kPlane);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const Dft w = make_dft(lane);
  const int64_t rows = static_cast<int64_t>(B) * D;  // visited as (d, b), b fastest
  const int64_t total = (static_cast<int64_t>(D) - blockIdx.x + gridDim.x - 1) / gridDim.x * B;
  auto row_of = [&](int64_t it) -> int64_t {  // it-th row of this workgroup
    const int64_t d = blockIdx.x + (it / B) * gridDim.x, bb = it % B;
    return bb * D + d;
  };
  (void)rows;
  RowRegs<DT> rdy;
  if (total > 0) fetch_row(rdy, static_cast<const char*>(dy) + row_of(0) * L * 2, L, true, tid);
  for (int64_t it = 0; it < total; ++it) {
    const int64_t row = row_of(it), d = row % D;
    const bool first = it % B == 0;
    const char* dyrow = static_cast<const char*>(dy) + row * L * 2;
    const float sdy = place_row(pre, pim, red, rdy, true, tid);
    transform<false>(pre, pim, w, wave, lane);
    RowRegs<MEGA_F32> rk;
    fetch_row(rk, k + d * L, L, false, tid);
    Spectrum sp;
    capture_spectrum(pre, pim, sp, tid);
    lds_barrier();
    // dx
    const float sk = place_row(pre, pim, red, rk, false, tid);
    transform<false>(pre, pim, w, wave, lane);
    pointwise(pre, pim, sp, tid);
    lds_barrier();
    RowRegs<DT> rx;
    fetch_row(rx, static_cast<const char*>(x) + row * L * 2, L, false, tid);
    transform<true>(pre, pim, w, wave, lane);
    store_row<DT, false>(pre, pim, static_cast<char*>(dx) + row * L * 2, L, true,
                         181.01933598375618f / (sdy * sk), omega != nullptr ? dyrow : nullptr,
                         omega != nullptr ? omega[d] : 0.f, tid);
    lds_barrier();
    // dk
    const float sx = place_row(pre, pim, red, rx, false, tid);
    transform<false>(pre, pim, w, wave, lane);
    pointwise(pre, pim, sp, tid);
    lds_barrier();
    if (it + 1 < total)
      fetch_row(rdy, static_cast<const char*>(dy) + row_of(it + 1) * L * 2, L, true, tid);
    transform<true>(pre, pim, w, wave, lane);
    float* krow = dk + d * L;
    const float sc = 181.01933598375618f / (sdy * sx);
    if (first)
      store_row<MEGA_F32, false>(pre, pim, krow, L, true, sc, nullptr, 0.f, tid);
    else
      store_row<MEGA_F32, true>(pre, pim, krow, L, true, sc, nullptr, 0.f, tid);
    lds_barrier();
  }
}

template <int DT>
int launch_bwd(const void* dy, const void* x, const float* k, void* dx, float* dk, int64_t B,
               int64_t D, int64_t L, const float* omega, hipStream_t stream) {
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&fftconv_mfma_bwd_kernel<DT>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     static_cast<int>(kLdsBytes)));
  MEGA_CHECK_ARG(B * D <= 0x7fffffff, "fftconv: too many rows");
  const unsigned grid = static_cast<unsigned>(D < cus ? D : cus);
  fftconv_mfma_bwd_kernel<DT><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
      dy, x, k, dx, dk, static_cast<int>(B), static_cast<int>(D), static_cast<int>(L), omega);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT, int MODE>
int launch(const void* a, const void* b, void* out, int64_t B, int64_t D, int64_t L, int flip,
           const float* omega, hipStream_t stream) {
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&fftconv_mfma_kernel<DT, MODE>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     static_cast<int>(kLdsBytes)));
  if (MODE == 0) {
    const int64_t rows = B * D;
    MEGA_CHECK_ARG(rows <= 0x7fffffff, "fftconv: too many rows");
    const unsigned grid = static_cast<unsigned>(rows < cus ? rows : cus);
    fftconv_mfma_kernel<DT, MODE><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
        a, b, out, static_cast<int>(rows), static_cast<int>(D), static_cast<int>(L), flip, omega);
    MEGA_CHECK_LAUNCH();
  } else {
    const unsigned grid = static_cast<unsigned>(D < cus ? D : cus);
    for (int64_t bb = 0; bb < B; ++bb) {
      const char* ab = static_cast<const char*>(a) + bb * D * L * 2;
      const char* xb = static_cast<const char*>(b) + bb * D * L * 2;
      fftconv_mfma_kernel<DT, MODE><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
          ab, xb, out, static_cast<int>(D), static_cast<int>(D), static_cast<int>(L),
          bb > 0 ? 1 : 0, nullptr);
      MEGA_CHECK_LAUNCH();
    }
  }
  return MEGA_OK;
}

}  // namespace

bool applicable(int dtype, int64_t L, const void* a, const void* b, const void* out) {
  const auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  return (dtype == MEGA_BF16 || dtype == MEGA_F16) && L > 16384 && L <= 32768 && L % 8 == 0 &&
         al(a) && al(b) && al(out);
}

int launch_conv(int dtype, int mode, const void* a, const void* b, void* out, int64_t B,
                int64_t D, int64_t L, int flip, const float* omega, hipStream_t stream) {
  if (dtype == MEGA_BF16)
    return mode == 0 ? launch<MEGA_BF16, 0>(a, b, out, B, D, L, flip, omega, stream)
                     : launch<MEGA_BF16, 1>(a, b, out, B, D, L, flip, omega, stream);
  return mode == 0 ? launch<MEGA_F16, 0>(a, b, out, B, D, L, flip, omega, stream)
                   : launch<MEGA_F16, 1>(a, b, out, B, D, L, flip, omega, stream);
}

int launch_backward(int dtype, const void* dy, const void* x, const float* k, void* dx, float* dk,
                    int64_t B, int64_t D, int64_t L, const float* omega, hipStream_t stream) {
  if (dtype == MEGA_BF16) return launch_bwd<MEGA_BF16>(dy, x, k, dx, dk, B, D, L, omega, stream);
  return launch_bwd<MEGA_F16>(dy, x, k, dx, dk, B, D, L, omega, stream);
}

}  // namespace fftm
}  // namespace mega
