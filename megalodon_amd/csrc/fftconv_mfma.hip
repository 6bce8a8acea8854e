// Causal convolution of 16-bit rows with the DFT stages on the matrix cores.
//
// One workgroup (8 waves) owns one row at a time (the longest rows; shorter
// rows go 2, 4 or 8 to a pass, see Geo below).  The zero-padded real row of
// 2N = 65536 samples is packed as z[n] = s[2n] + i s[2n+1], n < N = 32768, and
// kept in LDS as fp16 re and im values (rows of a, re half then im half).  The
// N-point transform is three radix-32 stages over the digits of n = 1024 a + 32 b + c:
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
// Used for bf16 / fp16 rows with 2048 < L <= 32768 and L % 8 == 0; everything else
// stays with the fp32 VALU engine of fftconv.hip.  Rows that share a pass are
// independent for finite data; a NaN or Inf in one of them spreads to the
// others of its pass (0 x NaN in the block-diagonal stage).
#include "common.hpp"
#include "fftconv_mfma.hpp"

namespace mega {
namespace fftm {
namespace {

// Row lengths: a row of L samples needs N' = 1024 A complex points with
// A = 32, 16, 8 or 4 digits a (L <= N').  The LDS always holds 32 values of a:
// a workgroup pass takes R = 32 / A rows side by side, row r owning a = r A ..
// r A + A - 1; the stage over a multiplies by the block-diagonal matrix of R
// DFT-A blocks, every other stage is unchanged (the row index rides along as a
// bystander).
template <int LOGA>
struct Geo {
  static constexpr int A = 1 << LOGA;       // digits a per row
  static constexpr int R = 32 / A;          // rows per workgroup pass
  static constexpr int NP = A * 1024;       // complex points of a row's transform
  static constexpr int HALF = NP / 2;       // packed points a row can fill (the rest is padding)
  static constexpr int JSH = LOGA - 2;      // quad j of a thread belongs to row j >> JSH
  static __device__ __forceinline__ int row_of_quad(int j) { return LOGA == 5 ? 0 : (j >> JSH); }
};
// LDS: row a holds its 1024 re values, 16 elements of padding, then its 1024 im
// values and padding.  The a-stride of 1040 dwords is 16 mod 64 banks, and the
// im value of an element sits a constant 2080 bytes after its re value, which
// every access folds into the instruction's immediate offset.
constexpr int kIm = 1024 + 16;        // elements from a re value to its im value
constexpr int kRS = 2 * kIm;          // elements between consecutive a
static_assert(kRS % 32 == 0, "the stages XOR swizzle bits 3-4 into offsets that include a * kRS");
constexpr int kPlane = 16 * kRS;      // half of the LDS elements (two "planes" of 32 half rows)
constexpr int kThreads = 512;         // 8 waves, two per SIMD
constexpr int kWaves = kThreads / kWave;
constexpr size_t kLdsBytes = sizeof(uint16_t) * 2 * kPlane + 256;  // + 8 x 8 floats for row maxima

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

// exp(+i 2 pi c m / N') for the 16 values c = 8 qd + 4 g + e a lane holds after a
// stage (register 4 qd + e), from three sin/cos pairs and complex products:
// W^(c m) = W^(4 g m) (W^(8 m))^qd (W^m)^e.
struct Tw16 {
  float c[16], s[16];
};
__device__ __forceinline__ void cmul(float ar, float ai, float br, float bi, float& cr, float& ci) {
  cr = ar * br - ai * bi;
  ci = ar * bi + ai * br;
}
template <int LOGA>
__device__ __forceinline__ Tw16 twiddles16(int m, int g) {
  constexpr int kN = Geo<LOGA>::NP;
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

// The block-diagonal matrix of 32 / A DFT-A blocks in MFMA operand form (lane l:
// j = l % 32 the output digit, k = 16 s + 8 (l / 32) + e the input digit),
// scaled by 1 / sqrt(A).
template <int LOGA>
__device__ __forceinline__ Dft make_dft_a(int lane) {
  constexpr int A = Geo<LOGA>::A;
  Dft w;
  const int j = lane & 31, g = lane >> 5;
  const float sc = LOGA == 4 ? 0.25f : (LOGA == 3 ? 0.35355339059327379f : 0.5f);
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    float c[8], sn[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = 16 * s + 8 * g + e;
      const bool on = (k >> LOGA) == (j >> LOGA);
      cis(((k & (A - 1)) * (j & (A - 1))) & (A - 1), 1.f / A, c[e], sn[e]);
      c[e] = on ? c[e] * sc : 0.f;
      sn[e] = on ? sn[e] * sc : 0.f;
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

// ---- stages over a (F1 / I3): tile = fixed b, rows a, bystander c -------------
// F1 (a -> k1): then twiddle W_(32 A)^(b k1), one factor per lane.  With A = 32
// only a < 16 holds data (zero padding) -> one k-step; shorter rows have their
// padding written as zeros and take both.  I3 (k1 -> a): no twiddle.
template <int LOGA, bool INV, bool PF>
__device__ __forceinline__ void stage_a(uint16_t* pre, const Dft& w32, int wave, int lane) {
  constexpr int A = Geo<LOGA>::A;
  constexpr int KS = (INV || LOGA < 5) ? 2 : 1;
  lane = opaque(lane) & 63;
  const Dft w = LOGA == 5 ? w32 : make_dft_a<LOGA>(lane);
  const int g = lane >> 5, f = lane & 31;
  const int rsrc = 8 * g + ((lane & 15) >> 2), csrc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  // pos(16 s + rsrc + 4 h, b, csrc): the row's swizzle bits are (2 g + h) & 3
  const int rd0 = rsrc * kRS + (csrc ^ (((2 * g) & 3) << 3));
  const int rd1 = (rsrc + 4) * kRS + (csrc ^ (((2 * g + 1) & 3) << 3));
  const int wr = f * kRS + 4 * g, fx = (f >> 2) & 3;
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  // PF: the operands of the wave's next tile are read before this tile's
  // twiddles and write-back (tiles are disjoint, but the compiler cannot move
  // LDS reads over LDS writes by itself); the loop is then fully unrolled.
  u32x4 xr[2], xi[2], nr[2], ni[2];
  if (PF) read_tile_tr<KS, 16 * kRS>(pre, (rd0 ^ (((wv >> 2) & 3) << 3)) + 32 * wv,
                                     (rd1 ^ (((wv >> 2) & 3) << 3)) + 32 * wv, xr, xi);
#pragma unroll(PF ? 4 : 1)
  for (int b = wv; b < 32; b += kWaves) {
    const int bx = ((b >> 2) & 3) << 3;
    if (!PF) {
      read_tile_tr<KS, 16 * kRS>(pre, (rd0 ^ bx) + 32 * b, (rd1 ^ bx) + 32 * b, xr, xi);
    } else if (b + kWaves < 32) {
      const int b2 = b + kWaves, bx2 = ((b2 >> 2) & 3) << 3;
      read_tile_tr<KS, 16 * kRS>(pre, (rd0 ^ bx2) + 32 * b2, (rd1 ^ bx2) + 32 * b2, nr, ni);
    }
    floatx16 dr, di;
    dft_xa<INV, KS>(xr, xi, w, dr, di);
    if (!INV) {
      float tc, ts;
      cis((b * (f & (A - 1))) & (32 * A - 1), 1.f / (32 * A), tc, ts);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float vr = dr[r], vi = di[r];
        dr[r] = vr * tc + vi * ts;  // (vr + i vi)(tc - i ts)
        di[r] = vi * tc - vr * ts;
      }
    }
    write_tile_x(pre, dr, di, wr + 32 * b, fx ^ (bx >> 3));
    if (PF) {
#pragma unroll
      for (int s = 0; s < KS; ++s) xr[s] = nr[s], xi[s] = ni[s];
    }
  }
}

// ---- stages over b (F2 / I2): tile = fixed a, rows b, bystander c -------------
// With k1 = a % A: F2 (b -> k2): then twiddle W_N'^(c (k1 + A k2)).  I2 (k2 ->
// n2): undoes F1's twiddle, conj W_(32 A)^(n2 k1), one factor per lane.
template <int LOGA, bool INV, bool PF>
__device__ __forceinline__ void stage_b(uint16_t* pre, const Dft& w, int wave, int lane) {
  constexpr int A = Geo<LOGA>::A;
  lane = opaque(lane) & 63;
  const int g = lane >> 5, f = lane & 31;
  const int rsrc = 8 * g + ((lane & 15) >> 2), csrc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int rd0 = 32 * rsrc + (csrc ^ (((2 * g) & 3) << 3));
  const int rd1 = 32 * (rsrc + 4) + (csrc ^ (((2 * g + 1) & 3) << 3));
  const int wr = 32 * f + 4 * g, fx = (f >> 2) & 3;
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  u32x4 xr[2], xi[2], nr[2], ni[2];
  if (PF) read_tile_tr<2, 512>(pre, (rd0 ^ (((wv >> 2) & 3) << 3)) + wv * kRS,
                               (rd1 ^ (((wv >> 2) & 3) << 3)) + wv * kRS, xr, xi);
#pragma unroll(PF ? 4 : 1)
  for (int a = wv; a < 32; a += kWaves) {
    const int ax = ((a >> 2) & 3) << 3, k1 = a & (A - 1);
    if (!PF) {
      read_tile_tr<2, 512>(pre, (rd0 ^ ax) + a * kRS, (rd1 ^ ax) + a * kRS, xr, xi);
    } else if (a + kWaves < 32) {
      const int a2 = a + kWaves, ax2 = ((a2 >> 2) & 3) << 3;
      read_tile_tr<2, 512>(pre, (rd0 ^ ax2) + a2 * kRS, (rd1 ^ ax2) + a2 * kRS, nr, ni);
    }
    floatx16 dr, di;
    dft_xa<INV, 2>(xr, xi, w, dr, di);
    if (!INV) {
      const Tw16 t = twiddles16<LOGA>(k1 + A * f, g);
      apply_tw<false>(dr, di, t);
    } else {
      float tc, ts;
      cis((k1 * f) & (32 * A - 1), 1.f / (32 * A), tc, ts);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float vr = dr[r], vi = di[r];
        dr[r] = vr * tc - vi * ts;  // (vr + i vi)(tc + i ts)
        di[r] = vi * tc + vr * ts;
      }
    }
    write_tile_x(pre, dr, di, wr + a * kRS, fx ^ (ax >> 3));
    if (PF) {
#pragma unroll
      for (int s = 0; s < 2; ++s) xr[s] = nr[s], xi[s] = ni[s];
    }
  }
}

// ---- stages over c (F3 / I1): tile = fixed a, lanes b, rows c (contiguous) ----
// F3 (c -> k3): no twiddle.  I1 (k3 -> n3): then undoes F2's twiddle,
// conj W_N'^(n3 (k1 + A b)).
template <int LOGA, bool INV, bool PF>
__device__ __forceinline__ void stage_c(uint16_t* pre, const Dft& w, int wave, int lane) {
  constexpr int A = Geo<LOGA>::A;
  lane = opaque(lane) & 63;
  const int g = lane >> 5, b = lane & 31;
  const int bx = (b >> 2) & 3, row = 32 * b;
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  // pos(a, b, 16 s + 8 g) = row part + 8 ((2 s + g) ^ x), x = bx ^ bits 2-3 of a
  auto read_tile = [&](int a, u32x4* r, u32x4* i) {
    const int x = bx ^ ((a >> 2) & 3);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const uint16_t* q = pre + a * kRS + row + (((2 * s + g) ^ x) << 3);
      r[s] = *reinterpret_cast<const u32x4*>(q);
      i[s] = *reinterpret_cast<const u32x4*>(q + kIm);
    }
  };
  u32x4 xr[2], xi[2], nr[2], ni[2];
  if (PF) read_tile(wv, xr, xi);
#pragma unroll(PF ? 4 : 1)
  for (int a = wv; a < 32; a += kWaves) {
    const int x = bx ^ ((a >> 2) & 3);
    const int base = a * kRS + row;
    if (!PF) {
      read_tile(a, xr, xi);
    } else if (a + kWaves < 32) {
      read_tile(a + kWaves, nr, ni);
    }
    floatx16 dr, di;
    dft_xb<INV>(xr, xi, w, dr, di);
    if (INV) {
      const Tw16 t = twiddles16<LOGA>((a & (A - 1)) + A * b, g);
      apply_tw<true>(dr, di, t);
    }
    write_tile_x(pre, dr, di, base + 4 * g, x);
    if (PF) {
#pragma unroll
      for (int s = 0; s < 2; ++s) xr[s] = nr[s], xi[s] = ni[s];
    }
  }
}

// PF: every stage reads the operands of a wave's next tile before it twiddles
// and writes back the current one: 16 more live registers, worth ~5 % where they
// are free.  The kernels that hold a parked spectrum plus prefetched rows sit at
// the 256-register limit already and leave it off.
template <int LOGA, bool INV, bool PF = false>
__device__ __forceinline__ void transform(uint16_t* pre, const Dft& w, int wave, int lane) {
  if (!INV) {
    stage_a<LOGA, false, PF>(pre, w, wave, lane);
    lds_barrier();
    stage_b<LOGA, false, PF>(pre, w, wave, lane);
    lds_barrier();
    stage_c<LOGA, false, PF>(pre, w, wave, lane);
    lds_barrier();
  } else {
    stage_c<LOGA, true, PF>(pre, w, wave, lane);
    lds_barrier();
    stage_b<LOGA, true, PF>(pre, w, wave, lane);
    lds_barrier();
    stage_a<LOGA, true, PF>(pre, w, wave, lane);
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

// The rows of a pass in flight: a thread's 8 quads of sample pairs, as loaded.
// Quad j belongs to row j >> JSH of the pass and covers the packed points
// n0 .. n0 + 3, n0 = 4 (tid + 512 j) mod (N' / 2) (reversed order when flip).
// L % 8 == 0 keeps quads whole.  Absent rows (null pointer) read as zeros.
template <int DT>
struct RowRegs {
  typename QuadIo<DT>::Raw q[8];
};
template <int LOGA>
struct RowPtrs {
  const char* p[Geo<LOGA>::R];
};
template <int LOGA>
__device__ __forceinline__ unsigned quad_n0(int tid, int j) {
  return (4u * (static_cast<unsigned>(tid) + kThreads * j)) & (Geo<LOGA>::HALF - 1);
}
template <int LOGA, int DT>
__device__ __forceinline__ void fetch_rows(RowRegs<DT>& r, const RowPtrs<LOGA>& rows, int L,
                                           bool flip, int tid) {
  const unsigned half = static_cast<unsigned>(L) >> 1;
  tid = opaque(tid) & (kThreads - 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const unsigned n0 = quad_n0<LOGA>(tid, j);
    const char* row = rows.p[Geo<LOGA>::row_of_quad(j)];
    r.q[j] = QuadIo<DT>::zero();
    if (n0 < half && row != nullptr) r.q[j] = QuadIo<DT>::fetch(row, flip ? half - 4u - n0 : n0);
  }
}
// Writes the fetched rows to the LDS as z[n] = s[2n] + i s[2n+1], n < N' / 2
// (zeros beyond the row), each row scaled by a power of two so that its max |s|
// lands in [1/8, 1/4); `scale` receives the R scales.  Rows of fewer than 32
// digits a also have their padding half written as zeros (A = 32 never reads
// it).  `red` is 8 R floats of LDS.  Ends with a barrier.
template <int LOGA, int DT>
__device__ __forceinline__ void place_rows(uint16_t* pre, float* red, const RowRegs<DT>& r,
                                           bool flip, int tid, float* scale) {
  constexpr int A = Geo<LOGA>::A, R = Geo<LOGA>::R;
  tid = opaque(tid) & (kThreads - 1);
  float re[8][4], im[8][4];
  float m[R];
#pragma unroll
  for (int i = 0; i < R; ++i) m[i] = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    float lo[4], hi[4];
    QuadIo<DT>::unpack(r.q[j], lo, hi);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      re[j][e] = flip ? hi[3 - e] : lo[e];
      im[j][e] = flip ? lo[3 - e] : hi[e];
      m[Geo<LOGA>::row_of_quad(j)] = fmaxf(m[Geo<LOGA>::row_of_quad(j)], fmaxf(fabsf(re[j][e]), fabsf(im[j][e])));
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    m[i] = wave_max(m[i]);
    if ((tid & (kWave - 1)) == 0) red[(tid / kWave) * R + i] = m[i];
  }
  lds_barrier();
#pragma unroll
  for (int i = 0; i < R; ++i) {
    float v = red[i];
#pragma unroll
    for (int wv = 1; wv < kWaves; ++wv) v = fmaxf(v, red[wv * R + i]);
    // 2^-(e+2) with v = f 2^e, f in [0.5, 1); finite non-zero v only
    float sc = 1.f;
    if (v > 0.f && v < 3.0e38f) {
      int e;
      (void)frexpf(v, &e);
      sc = ldexpf(1.f, -(e + 2));
    }
    scale[i] = sc;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int n0 = static_cast<int>(quad_n0<LOGA>(tid, j));
    const float sc = scale[Geo<LOGA>::row_of_quad(j)];
    const int a = Geo<LOGA>::row_of_quad(j) * A + (n0 >> 10);
    const int o = pos(a, (n0 >> 5) & 31, n0 & 31);
    *reinterpret_cast<uint2*>(pre + o) =
        make_uint2(pack_h2(re[j][0] * sc, re[j][1] * sc), pack_h2(re[j][2] * sc, re[j][3] * sc));
    *reinterpret_cast<uint2*>(pre + o + kIm) =
        make_uint2(pack_h2(im[j][0] * sc, im[j][1] * sc), pack_h2(im[j][2] * sc, im[j][3] * sc));
    if (LOGA < 5) {
      const int oz = pos(a + A / 2, (n0 >> 5) & 31, n0 & 31);
      *reinterpret_cast<uint2*>(pre + oz) = make_uint2(0u, 0u);
      *reinterpret_cast<uint2*>(pre + oz + kIm) = make_uint2(0u, 0u);
    }
  }
  lds_barrier();
}

// Row r of the pass: out[2n] = re z[n] * scale[r] (+ w[r] res[r][2n]), out[2n+1]
// likewise, n < L/2 (reversed when flip); ACC adds to what is there (fp32 rows).
// Absent rows (null pointer) are skipped.
template <int LOGA, int DT, bool ACC>
__device__ __forceinline__ void store_rows(const uint16_t* pre, const RowPtrs<LOGA>& rows, int L,
                                           bool flip, const float* scale,
                                           const RowPtrs<LOGA>* res, const float* w, int tid) {
  constexpr int A = Geo<LOGA>::A;
  const unsigned half = static_cast<unsigned>(L) >> 1;
  tid = opaque(tid) & (kThreads - 1);
#pragma unroll(LOGA == 5 ? 2 : 8)
  for (int j = 0; j < 8; ++j) {
    const unsigned n0 = quad_n0<LOGA>(tid, j);
    char* row = const_cast<char*>(rows.p[Geo<LOGA>::row_of_quad(j)]);
    if (n0 < half && row != nullptr) {
      const float sc = scale[Geo<LOGA>::row_of_quad(j)];
      const int o = pos(Geo<LOGA>::row_of_quad(j) * A + static_cast<int>(n0 >> 10), (n0 >> 5) & 31, n0 & 31);
      const uint2 ur = *reinterpret_cast<const uint2*>(pre + o);
      const uint2 ui = *reinterpret_cast<const uint2*>(pre + o + kIm);
      float zr[4], zi[4], lo[4], hi[4];
      unpack_h2(ur.x, zr[0], zr[1]);
      unpack_h2(ur.y, zr[2], zr[3]);
      unpack_h2(ui.x, zi[0], zi[1]);
      unpack_h2(ui.y, zi[2], zi[3]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = (flip ? zi[3 - e] : zr[e]) * sc;
        hi[e] = (flip ? zr[3 - e] : zi[e]) * sc;
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
        QuadIo<DT>::load(res->p[Geo<LOGA>::row_of_quad(j)], m0, rlo, rhi);
        const float wt = w[Geo<LOGA>::row_of_quad(j)];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] = fmaf(wt, rlo[e], lo[e]);
          hi[e] = fmaf(wt, rhi[e], hi[e]);
        }
      }
      QuadIo<DT>::store(row, m0, lo, hi);
    }
  }
}

// ---- conjugate bin pairs ------------------------------------------------------
// Bin k = k1 + A k2 + 32 A k3 of row r sits at (r A + k1, k2, k3); its partner
// N' - k at the mirrored LDS row (k1', k2') = (A - k1, 31 - k2) (k1 != 0) or
// (0, 32 - k2), with k3' = 31 - k3.  LDS row (0, 0) is its own mirror with
// k3' = (32 - k3) % 32 and is handled apart.  The other 32 A - 1 LDS rows of a
// row form 16 A - 1 pairs plus the self-mirrored (0, 16): pair q of 16 A is
//   q < 32 (A/2 - 1): (1 + q / 32, q % 32);  the next 16: (A/2, 0..15);
//   the next 15: (0, 1..15);  the last: (0, 16).
// A lane takes one quad of a pair: bins k3 = 4u .. 4u+3 and the reversed quad
// 7 - u of the mirror; task T = tid + 512 i -> row T / (128 A), q = T / 8 % (16 A), u = T % 8.
struct RowPair {
  int ok, om;   // LDS offsets of the two quads
  int k0;       // bin index of the quad's first element: k1 + A k2 + 128 A u
  bool writes;  // false for the duplicate lanes of the self-mirrored row
};
template <int LOGA>
__device__ __forceinline__ RowPair row_pair(int task) {
  constexpr int A = Geo<LOGA>::A;
  const int r = task >> (LOGA + 7), q = (task >> 3) & (16 * A - 1), u = task & 7;
  constexpr int kBulk = 32 * (A / 2 - 1);
  int k1, k2;
  if (q < kBulk) {
    k1 = 1 + (q >> 5);
    k2 = q & 31;
  } else if (q < kBulk + 16) {
    k1 = A / 2;
    k2 = q - kBulk;
  } else if (q < kBulk + 31) {
    k1 = 0;
    k2 = q - (kBulk + 15);
  } else {
    k1 = 0;
    k2 = 16;
  }
  const int m1 = k1 != 0 ? A - k1 : 0;
  const int m2 = k1 != 0 ? 31 - k2 : 32 - k2;
  RowPair rp;
  rp.ok = pos(r * A + k1, k2, 4 * u);
  rp.om = pos(r * A + m1, m2, 4 * (7 - u));
  rp.k0 = k1 + A * k2 + 128 * A * u;
  rp.writes = q != 16 * A - 1 || u < 4;
  return rp;
}
__device__ __forceinline__ void write_quad(uint16_t* p, const float* v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]));
}

// Twice the even / odd spectra of a real signal packed as z = even + i odd:
// 2E = Z(k) + conj Z(m), 2O = (Z(k) - conj Z(m)) / i, m the mirror bin.  The
// factors of two of both operands are taken out again by the final scale.
__device__ __forceinline__ void untangle(float zkr, float zki, float zmr, float zmi, float& er,
                                         float& ei, float& orr, float& oi) {
  er = zkr + zmr;
  ei = zki - zmi;
  orr = zki + zmi;
  oi = zmr - zkr;
}
// The same on a quad of bins (elements 0..3 of the re and im runs) and the
// reversed quad of mirror bins, in packed fp16: element e pairs with mirror
// element 3 - e.  Results: index 0 holds elements (0, 1), index 1 elements (2, 3).
struct Quad2 {
  half2v er[2], ei[2], orr[2], oi[2];
};
__device__ __forceinline__ half2v as_h2(uint32_t u) { return __builtin_bit_cast(half2v, u); }
__device__ __forceinline__ half2v swap_h2(half2v v) { return __builtin_shufflevector(v, v, 1, 0); }
__device__ __forceinline__ Quad2 untangle_quads(uint2 kr, uint2 ki, uint2 mr, uint2 mi) {
  const half2v mr0 = swap_h2(as_h2(mr.y)), mr1 = swap_h2(as_h2(mr.x));  // mirror of elements (0,1), (2,3)
  const half2v mi0 = swap_h2(as_h2(mi.y)), mi1 = swap_h2(as_h2(mi.x));
  Quad2 q;
  q.er[0] = as_h2(kr.x) + mr0;
  q.er[1] = as_h2(kr.y) + mr1;
  q.ei[0] = as_h2(ki.x) - mi0;
  q.ei[1] = as_h2(ki.y) - mi1;
  q.orr[0] = as_h2(ki.x) + mi0;
  q.orr[1] = as_h2(ki.y) + mi1;
  q.oi[0] = mr0 - as_h2(kr.x);
  q.oi[1] = mr1 - as_h2(kr.y);
  return q;
}
__device__ __forceinline__ uint2 read_quad_raw(const uint16_t* p) {
  return *reinterpret_cast<const uint2*>(p);
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
  // 2E(k), 2O(k) of the parked operand per task, packed fp16:
  // e = (re of elements 0,1), (re 2,3), (im 0,1), (im 2,3); o likewise
  uint32_t e[8][4], o[8][4];
  uint32_t e0, o0;  // row (0, 0), lane = k3 (threads 0..31), fp16 (re, im)
};

// A spectrum kept in memory between the forward and the backward launch: the
// registers of `Spectrum` as they are, per pass
//   [task 0..7][thread 0..511][8 words]  then  [thread][e0, o0]  then  8 row scales (float).
constexpr int kSpecRowWords = 8 * kThreads * 8;              // offset of the (e0, o0) pairs
constexpr int kSpecScaleWords = kSpecRowWords + kThreads * 2;  // offset of the scales
constexpr int kSpecWords = kSpecScaleWords + 8;              // words per pass (a multiple of 4)

__device__ __forceinline__ void store_spec_task(uint32_t* spec, int i, int tid, const uint32_t* e,
                                                const uint32_t* o) {
  u32x4* q = reinterpret_cast<u32x4*>(spec + (static_cast<size_t>(i) * kThreads + tid) * 8);
  q[0] = u32x4{e[0], e[1], e[2], e[3]};
  q[1] = u32x4{o[0], o[1], o[2], o[3]};
}
__device__ __forceinline__ void store_spectrum(uint32_t* spec, const Spectrum& sp, int tid) {
#pragma unroll
  for (int i = 0; i < 8; ++i) store_spec_task(spec, i, tid, sp.e[i], sp.o[i]);
  *reinterpret_cast<uint2*>(spec + kSpecRowWords + 2 * tid) = make_uint2(sp.e0, sp.o0);
}

template <int LOGA>
__device__ __forceinline__ void capture_spectrum(const uint16_t* pre, Spectrum& sp, int tid) {
  constexpr int A = Geo<LOGA>::A, R = Geo<LOGA>::R;
  const uint16_t* pim = pre + kIm;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    tid = opaque(tid) & (kThreads - 1);
    const RowPair rp = row_pair<LOGA>(tid + kThreads * i);
    const Quad2 q = untangle_quads(read_quad_raw(pre + rp.ok), read_quad_raw(pim + rp.ok),
                                   read_quad_raw(pre + rp.om), read_quad_raw(pim + rp.om));
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      sp.e[i][h] = __builtin_bit_cast(uint32_t, q.er[h]);
      sp.e[i][2 + h] = __builtin_bit_cast(uint32_t, q.ei[h]);
      sp.o[i][h] = __builtin_bit_cast(uint32_t, q.orr[h]);
      sp.o[i][2 + h] = __builtin_bit_cast(uint32_t, q.oi[h]);
    }
  }
  sp.e0 = sp.o0 = 0u;
  tid = opaque(tid) & (kThreads - 1);
  if (tid < 32 * R) {
    const int a0 = (tid >> 5) * A, k3 = tid & 31;
    const int ok = pos(a0, 0, k3), om = pos(a0, 0, (32 - k3) & 31);
    float er, ei, orr, oi;
    untangle(h2f(pre[ok]), h2f(pim[ok]), h2f(pre[om]), h2f(pim[om]), er, ei, orr, oi);
    sp.e0 = pack_h2(er, ei);
    sp.o0 = pack_h2(orr, oi);
  }
}

// the product of the two real signals' spectra, written over Za
// `save` != nullptr: the untangled spectrum of the operand in LDS is also
// written out in the saved-spectrum layout.
template <int LOGA>
__device__ __forceinline__ void pointwise(uint16_t* pre, const Spectrum& sp, int tid,
                                          uint32_t* save = nullptr) {
  constexpr int A = Geo<LOGA>::A, R = Geo<LOGA>::R, NP = Geo<LOGA>::NP;
  uint16_t* pim = pre + kIm;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    tid = opaque(tid) & (kThreads - 1);
    const RowPair rp = row_pair<LOGA>(tid + kThreads * i);
    const Quad2 qa = untangle_quads(read_quad_raw(pre + rp.ok), read_quad_raw(pim + rp.ok),
                                    read_quad_raw(pre + rp.om), read_quad_raw(pim + rp.om));
    if (save != nullptr) {
      const uint32_t se[4] = {__builtin_bit_cast(uint32_t, qa.er[0]), __builtin_bit_cast(uint32_t, qa.er[1]),
                              __builtin_bit_cast(uint32_t, qa.ei[0]), __builtin_bit_cast(uint32_t, qa.ei[1])};
      const uint32_t so[4] = {__builtin_bit_cast(uint32_t, qa.orr[0]), __builtin_bit_cast(uint32_t, qa.orr[1]),
                              __builtin_bit_cast(uint32_t, qa.oi[0]), __builtin_bit_cast(uint32_t, qa.oi[1])};
      store_spec_task(save, i, tid, se, so);
    }
    float w0c, w0s;
    cis(rp.k0, 1.f / NP, w0c, w0s);
    // W_N'^(k0 + 32 A e) = W_N'^k0 W_32^e
    const float c32[4] = {1.f, 0.98078528040323043f, 0.92387953251128674f, 0.83146961230254524f};
    const float s32[4] = {0.f, 0.19509032201612825f, 0.38268343236508978f, 0.55557023301960218f};
    float okr[4], oki[4], omr[4], omi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int hp = e >> 1, hh = e & 1;  // which packed pair, which half of it
      const float ar = static_cast<float>(qa.er[hp][hh]), ai = static_cast<float>(qa.ei[hp][hh]);
      const float pr = static_cast<float>(qa.orr[hp][hh]), pi = static_cast<float>(qa.oi[hp][hh]);
      const float br = static_cast<float>(as_h2(sp.e[i][hp])[hh]);
      const float bi = static_cast<float>(as_h2(sp.e[i][2 + hp])[hh]);
      const float qr = static_cast<float>(as_h2(sp.o[i][hp])[hh]);
      const float qi = static_cast<float>(as_h2(sp.o[i][2 + hp])[hh]);
      float wc, ws;
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
  if (tid < 32 * R) {
    const int a0 = (tid >> 5) * A, k3 = tid & 31, m3 = (32 - k3) & 31;
    const int ok = pos(a0, 0, k3), om = pos(a0, 0, m3);
    float ar, ai, pr, pi, br, bi, qr, qi, wc, ws, zkr, zki, zmr, zmi;
    untangle(h2f(pre[ok]), h2f(pim[ok]), h2f(pre[om]), h2f(pim[om]), ar, ai, pr, pi);
    if (save != nullptr)
      *reinterpret_cast<uint2*>(save + kSpecRowWords + 2 * tid) = make_uint2(pack_h2(ar, ai), pack_h2(pr, pi));
    unpack_h2(sp.e0, br, bi);
    unpack_h2(sp.o0, qr, qi);
    cis(k3, 1.f / 32.f, wc, ws);
    bin_product(ar, ai, pr, pi, br, bi, qr, qi, wc, ws, zkr, zki, zmr, zmi);
    if (k3 <= m3) {
      pre[ok] = f2h(zkr);
      pim[ok] = f2h(zki);
      pre[om] = f2h(zmr);
      pim[om] = f2h(zmi);
    }
  } else if (save != nullptr) {
    *reinterpret_cast<uint2*>(save + kSpecRowWords + 2 * tid) = make_uint2(0u, 0u);
  }
}

// The same product with both spectra untangled already: `sa` in registers, the
// other read from a saved spectrum; the result goes to the LDS planes.
template <int LOGA>
__device__ __forceinline__ void pointwise_saved(uint16_t* pre, const Spectrum& sa,
                                                const uint32_t* __restrict__ spec, int tid) {
  constexpr int A = Geo<LOGA>::A, R = Geo<LOGA>::R, NP = Geo<LOGA>::NP;
  uint16_t* pim = pre + kIm;
  // the saved spectrum is read two tasks ahead of its use
  const u32x4* q = reinterpret_cast<const u32x4*>(spec) + static_cast<size_t>(tid) * 2;
  const uint2 b0 = *reinterpret_cast<const uint2*>(spec + kSpecRowWords + 2 * tid);
  u32x4 be_n = q[0], bo_n = q[1];
  u32x4 be_nn = q[2 * kThreads], bo_nn = q[2 * kThreads + 1];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    tid = opaque(tid) & (kThreads - 1);
    const RowPair rp = row_pair<LOGA>(tid + kThreads * i);
    const u32x4 be = be_n, bo = bo_n;
    be_n = be_nn;
    bo_n = bo_nn;
    if (i + 2 < 8) {
      be_nn = q[static_cast<size_t>(i + 2) * 2 * kThreads];
      bo_nn = q[static_cast<size_t>(i + 2) * 2 * kThreads + 1];
    }
    float w0c, w0s;
    cis(rp.k0, 1.f / NP, w0c, w0s);
    const float c32[4] = {1.f, 0.98078528040323043f, 0.92387953251128674f, 0.83146961230254524f};
    const float s32[4] = {0.f, 0.19509032201612825f, 0.38268343236508978f, 0.55557023301960218f};
    float okr[4], oki[4], omr[4], omi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int hp = e >> 1, hh = e & 1;
      const float ar = static_cast<float>(as_h2(sa.e[i][hp])[hh]);
      const float ai = static_cast<float>(as_h2(sa.e[i][2 + hp])[hh]);
      const float pr = static_cast<float>(as_h2(sa.o[i][hp])[hh]);
      const float pi = static_cast<float>(as_h2(sa.o[i][2 + hp])[hh]);
      const float br = static_cast<float>(as_h2(be[hp])[hh]), bi = static_cast<float>(as_h2(be[2 + hp])[hh]);
      const float qr = static_cast<float>(as_h2(bo[hp])[hh]), qi = static_cast<float>(as_h2(bo[2 + hp])[hh]);
      float wc, ws;
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
  if (tid < 32 * R) {
    const int a0 = (tid >> 5) * A, k3 = tid & 31, m3 = (32 - k3) & 31;
    const int ok = pos(a0, 0, k3), om = pos(a0, 0, m3);
    float ar, ai, pr, pi, br, bi, qr, qi, wc, ws, zkr, zki, zmr, zmi;
    unpack_h2(sa.e0, ar, ai);
    unpack_h2(sa.o0, pr, pi);
    unpack_h2(b0.x, br, bi);
    unpack_h2(b0.y, qr, qi);
    cis(k3, 1.f / 32.f, wc, ws);
    bin_product(ar, ai, pr, pi, br, bi, qr, qi, wc, ws, zkr, zki, zmr, zmi);
    if (k3 <= m3) {
      pre[ok] = f2h(zkr);
      pim[ok] = f2h(zki);
      pre[om] = f2h(zmr);
      pim[om] = f2h(zmi);
    }
  }
}

// sqrt(N') / 4 / (the two operands' row scales): undoes the three unitary transforms
template <int LOGA>
__device__ __forceinline__ void final_scales(const float* sa, const float* sb, float* out) {
  // sqrt(N') / 4: the spectra of both operands are carried at twice their size
  constexpr float root = 0.25f * (LOGA == 5 ? 181.01933598375618f
                                            : (LOGA == 4 ? 128.f : (LOGA == 3 ? 90.509667991878086f : 64.f)));
#pragma unroll
  for (int i = 0; i < Geo<LOGA>::R; ++i) out[i] = root / (sa[i] * sb[i]);
}

// A pass takes R consecutive rows (R = 1 for the longest rows).
// MODE 0: out[b,d,:] = conv(a[b,d,:], k[d,:]) (+ omega[d] a[b,d,:]); `flip`
//         reverses a on load and the result on store (backward dx); k fp32.
// MODE 1: out[d,:] (+)= reverse(conv(reverse(a[b0,d,:]), x[b0,d,:])), fp32 out,
//         `flip` != 0 accumulates (backward dk, one batch index per launch).
template <int DT, int MODE, int LOGA>
__global__ __launch_bounds__(kThreads) void fftconv_mfma_kernel(
    const void* __restrict__ a, const void* __restrict__ b, void* __restrict__ out, int rows,
    int D, int L, int flip, const float* __restrict__ omega, uint32_t* __restrict__ spec_a,
    uint32_t* __restrict__ spec_b) {
  constexpr int R = Geo<LOGA>::R;
  extern __shared__ __align__(16) uint16_t lds[];
  uint16_t* pre = lds;
  float* red = reinterpret_cast<float*>(lds + 2 * kPlane);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const Dft w = make_dft(lane);
  const int64_t esz = 2;
  const int passes = (rows + R - 1) / R;
  // spec_a / spec_b (both or neither): the untangled spectra of the two
  // operands of every pass and their row scales are kept for the backward launch

  // Software pipeline over the passes of this workgroup: the first-operand rows
  // are fetched while the second operand is transformed, and the next pass's
  // second operand while the inverse transform runs.
  typedef RowRegs<MODE == 0 ? MEGA_F32 : DT> RegsB;
  auto brows_of = [&](int pass) {
    RowPtrs<LOGA> p;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int64_t row = static_cast<int64_t>(pass) * R + i;
      p.p[i] = row >= rows ? nullptr
               : MODE == 0 ? reinterpret_cast<const char*>(static_cast<const float*>(b) + (row % D) * L)
                           : static_cast<const char*>(b) + row * L * esz;
    }
    return p;
  };
  RegsB rb;
  if (static_cast<int>(blockIdx.x) < passes)
    fetch_rows<LOGA>(rb, brows_of(blockIdx.x), L, false, tid);
  for (int pass = blockIdx.x; pass < passes; pass += gridDim.x) {
    RowPtrs<LOGA> arows, orows;
    float wres[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int64_t row = static_cast<int64_t>(pass) * R + i;
      const bool on = row < rows;
      arows.p[i] = on ? static_cast<const char*>(a) + row * L * esz : nullptr;
      orows.p[i] = !on ? nullptr
                   : MODE == 0 ? static_cast<const char*>(out) + row * L * esz
                               : reinterpret_cast<const char*>(static_cast<float*>(out) + row * L);
      wres[i] = (MODE == 0 && omega != nullptr && on) ? omega[row % D] : 0.f;
    }
    const bool flip_a = MODE == 1 || flip != 0;
    float sb[R], sa[R], scale[R];
    place_rows<LOGA>(pre, red, rb, false, tid, sb);
    RowRegs<DT> ra;
    fetch_rows<LOGA>(ra, arows, L, flip_a, tid);
    transform<LOGA, false>(pre, w, wave, lane);
    Spectrum sp;
    capture_spectrum<LOGA>(pre, sp, tid);
    uint32_t* const save_a = spec_a == nullptr ? nullptr : spec_a + static_cast<size_t>(pass) * kSpecWords;
    lds_barrier();
    place_rows<LOGA>(pre, red, ra, flip_a, tid, sa);
    transform<LOGA, false>(pre, w, wave, lane);
    if (spec_b != nullptr) {
      // Stores go here, after the wait for the first operand's rows and with
      // no wait on memory before the next pass: issued right after the capture
      // they would be waited for in front of place_rows (loads and stores
      // share one in-order counter).
      // The second operand depends on the channel only: its spectrum is kept
      // once per channel group, by the pass of batch index 0.
      if (static_cast<int64_t>(pass) * R < D) {
        uint32_t* const save_b = spec_b + static_cast<size_t>(pass) * kSpecWords;
        store_spectrum(save_b, sp, tid);
#pragma unroll
        for (int i = 0; i < R; ++i)
          if (tid == i) reinterpret_cast<float*>(save_b + kSpecScaleWords)[i] = sb[i];
      }
#pragma unroll
      for (int i = 0; i < R; ++i)
        if (tid == i) reinterpret_cast<float*>(save_a + kSpecScaleWords)[i] = sa[i];
    }
    pointwise<LOGA>(pre, sp, tid, save_a);
    lds_barrier();
    if (pass + static_cast<int>(gridDim.x) < passes)
      fetch_rows<LOGA>(rb, brows_of(pass + gridDim.x), L, false, tid);
    transform<LOGA, true>(pre, w, wave, lane);
    final_scales<LOGA>(sa, sb, scale);
    if (MODE == 0) {
      store_rows<LOGA, DT, false>(pre, orows, L, flip != 0, scale,
                                  omega != nullptr ? &arows : nullptr, wres, tid);
    } else {
      if (flip)
        store_rows<LOGA, MEGA_F32, true>(pre, orows, L, true, scale, nullptr, wres, tid);
      else
        store_rows<LOGA, MEGA_F32, false>(pre, orows, L, true, scale, nullptr, wres, tid);
    }
    lds_barrier();  // the planes are rewritten by the next pass's operand
  }
}

// Backward of R channels in one pass: dy is transformed once and its spectrum
// parked; then k (-> dx) and x (-> dk) are each transformed, multiplied with
// it and transformed back.
//   dx[b,d,:] = reverse(conv(reverse(dy[b,d,:]), k[d,:])) (+ omega[d] dy[b,d,:])
//   dk[d,:]   = sum_b reverse(conv(reverse(dy[b,d,:]), x[b,d,:]))
// A workgroup owns the channel groups blockIdx.x, + gridDim.x, ... (R channels
// each) and walks the batch itself, so dk accumulates in order without atomics.
template <int DT, int LOGA>
__global__ __launch_bounds__(kThreads) void fftconv_mfma_bwd_kernel(
    const void* __restrict__ dy, const void* __restrict__ x, const float* __restrict__ k,
    void* __restrict__ dx, float* __restrict__ dk, int B, int D, int L,
    const float* __restrict__ omega) {
  constexpr int R = Geo<LOGA>::R;
  extern __shared__ __align__(16) uint16_t lds[];
  uint16_t* pre = lds;
  float* red = reinterpret_cast<float*>(lds + 2 * kPlane);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const Dft w = make_dft(lane);
  const int64_t groups = (static_cast<int64_t>(D) + R - 1) / R;
  const int64_t total = (groups - blockIdx.x + gridDim.x - 1) / gridDim.x * B;
  // rows of this workgroup's it-th pass: channels d0 .. d0 + R - 1 of batch index bb
  auto rows_of = [&](int64_t it, const void* base, int64_t esz, bool batched) {
    const int64_t d0 = (blockIdx.x + (it / B) * gridDim.x) * R, bb = it % B;
    RowPtrs<LOGA> p;
#pragma unroll
    for (int i = 0; i < R; ++i)
      p.p[i] = d0 + i < D ? static_cast<const char*>(base) + ((batched ? bb * D : 0) + d0 + i) * L * esz
                          : nullptr;
    return p;
  };
  RowRegs<DT> rdy;
  if (total > 0) fetch_rows<LOGA>(rdy, rows_of(0, dy, 2, true), L, true, tid);
  for (int64_t it = 0; it < total; ++it) {
    const int64_t d0 = (blockIdx.x + (it / B) * gridDim.x) * R;
    const bool first = it % B == 0;
    const RowPtrs<LOGA> dyrows = rows_of(it, dy, 2, true);
    float wres[R];
#pragma unroll
    for (int i = 0; i < R; ++i) wres[i] = (omega != nullptr && d0 + i < D) ? omega[d0 + i] : 0.f;
    float sdy[R], sk[R], sx[R], scale[R];
    place_rows<LOGA>(pre, red, rdy, true, tid, sdy);
    transform<LOGA, false>(pre, w, wave, lane);
    RowRegs<MEGA_F32> rk;
    fetch_rows<LOGA>(rk, rows_of(it, k, 4, false), L, false, tid);
    Spectrum sp;
    capture_spectrum<LOGA>(pre, sp, tid);
    lds_barrier();
    // dx
    place_rows<LOGA>(pre, red, rk, false, tid, sk);
    transform<LOGA, false>(pre, w, wave, lane);
    pointwise<LOGA>(pre, sp, tid);
    lds_barrier();
    RowRegs<DT> rx;
    fetch_rows<LOGA>(rx, rows_of(it, x, 2, true), L, false, tid);
    transform<LOGA, true>(pre, w, wave, lane);
    final_scales<LOGA>(sdy, sk, scale);
    store_rows<LOGA, DT, false>(pre, rows_of(it, dx, 2, true), L, true, scale,
                                omega != nullptr ? &dyrows : nullptr, wres, tid);
    lds_barrier();
    // dk
    place_rows<LOGA>(pre, red, rx, false, tid, sx);
    transform<LOGA, false>(pre, w, wave, lane);
    pointwise<LOGA>(pre, sp, tid);
    lds_barrier();
    if (it + 1 < total) fetch_rows<LOGA>(rdy, rows_of(it + 1, dy, 2, true), L, true, tid);
    transform<LOGA, true>(pre, w, wave, lane);
    final_scales<LOGA>(sdy, sx, scale);
    const RowPtrs<LOGA> krows = rows_of(it, dk, 4, false);
    if (first)
      store_rows<LOGA, MEGA_F32, false>(pre, krows, L, true, scale, nullptr, wres, tid);
    else
      store_rows<LOGA, MEGA_F32, true>(pre, krows, L, true, scale, nullptr, wres, tid);
    lds_barrier();
  }
}

// Backward from the spectra the forward launch kept (those of x and k, one pass
// = R consecutive channels of one batch index, D % R == 0): dy is transformed
// once, multiplied with either spectrum and transformed back -- three
// transforms per pass instead of five, and neither x nor k is read.
//   dx[b,d,:] = reverse(conv(reverse(dy[b,d,:]), k[d,:])) (+ omega[d] dy[b,d,:])
//   dk[d,:]   = sum_b reverse(conv(reverse(dy[b,d,:]), x[b,d,:]))
// As in the kernel above a workgroup owns channel groups and walks the batch.
template <int DT, int LOGA>
__global__ __launch_bounds__(kThreads) void fftconv_mfma_bwd_saved_kernel(
    const void* __restrict__ dy, const uint32_t* __restrict__ spec_x,
    const uint32_t* __restrict__ spec_k, void* __restrict__ dx, float* __restrict__ dk, int B,
    int D, int L, const float* __restrict__ omega) {
  constexpr int R = Geo<LOGA>::R;
  extern __shared__ __align__(16) uint16_t lds[];
  uint16_t* pre = lds;
  float* red = reinterpret_cast<float*>(lds + 2 * kPlane);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const Dft w = make_dft(lane);
  const int64_t groups = D / R;
  const int64_t total = (groups - blockIdx.x + gridDim.x - 1) / gridDim.x * B;
  auto rows_of = [&](int64_t it, const void* base, int64_t esz, bool batched) {
    const int64_t d0 = (blockIdx.x + (it / B) * gridDim.x) * R, bb = it % B;
    RowPtrs<LOGA> p;
#pragma unroll
    for (int i = 0; i < R; ++i)
      p.p[i] = static_cast<const char*>(base) + ((batched ? bb * D : 0) + d0 + i) * L * esz;
    return p;
  };
  RowRegs<DT> rdy;
  if (total > 0) fetch_rows<LOGA>(rdy, rows_of(0, dy, 2, true), L, true, tid);
  for (int64_t it = 0; it < total; ++it) {
    const int64_t d0 = (blockIdx.x + (it / B) * gridDim.x) * R, bb = it % B;
    const bool first = bb == 0;
    // the forward's pass of rows (bb, d0 .. d0 + R - 1)
    const size_t pass = static_cast<size_t>((bb * D + d0) / R);
    const uint32_t* sx = spec_x + pass * kSpecWords;
    const uint32_t* sk = spec_k + static_cast<size_t>(d0 / R) * kSpecWords;  // one per channel group
    const RowPtrs<LOGA> dyrows = rows_of(it, dy, 2, true);
    float wres[R], sdy[R], s2[R], scale[R];
#pragma unroll
    for (int i = 0; i < R; ++i) wres[i] = omega != nullptr ? omega[d0 + i] : 0.f;
    place_rows<LOGA>(pre, red, rdy, true, tid, sdy);
    transform<LOGA, false>(pre, w, wave, lane);
    Spectrum sp;
    capture_spectrum<LOGA>(pre, sp, tid);
    lds_barrier();
    // dx
    pointwise_saved<LOGA>(pre, sp, sk, tid);
    lds_barrier();
    transform<LOGA, true>(pre, w, wave, lane);
#pragma unroll
    for (int i = 0; i < R; ++i) s2[i] = reinterpret_cast<const float*>(sk + kSpecScaleWords)[i];
    final_scales<LOGA>(sdy, s2, scale);
    store_rows<LOGA, DT, false>(pre, rows_of(it, dx, 2, true), L, true, scale,
                                omega != nullptr ? &dyrows : nullptr, wres, tid);
    lds_barrier();
    // dk
    pointwise_saved<LOGA>(pre, sp, sx, tid);
    lds_barrier();
    if (it + 1 < total) fetch_rows<LOGA>(rdy, rows_of(it + 1, dy, 2, true), L, true, tid);
    transform<LOGA, true>(pre, w, wave, lane);
#pragma unroll
    for (int i = 0; i < R; ++i) s2[i] = reinterpret_cast<const float*>(sx + kSpecScaleWords)[i];
    final_scales<LOGA>(sdy, s2, scale);
    const RowPtrs<LOGA> krows = rows_of(it, dk, 4, false);
    if (first)
      store_rows<LOGA, MEGA_F32, false>(pre, krows, L, true, scale, nullptr, wres, tid);
    else
      store_rows<LOGA, MEGA_F32, true>(pre, krows, L, true, scale, nullptr, wres, tid);
    lds_barrier();
  }
}

// Forward for B > 1: the kernel row k[d, :] is the same for every batch index,
// so a workgroup owns channel groups (as the backward kernels do) and walks
// the batch itself: k is transformed once per channel group and its spectrum
// stays parked while the B rows of x are transformed, multiplied and
// transformed back -- 2 transforms per row instead of 3.  spec_x / spec_k as
// in fftconv_mfma_kernel (both or neither).
template <int DT, int LOGA>
__global__ __launch_bounds__(kThreads) void fftconv_mfma_fwd_batch_kernel(
    const void* __restrict__ x, const float* __restrict__ k, void* __restrict__ y, int B, int D, int L,
    const float* __restrict__ omega, uint32_t* __restrict__ spec_x, uint32_t* __restrict__ spec_k) {
  constexpr int R = Geo<LOGA>::R;
  extern __shared__ __align__(16) uint16_t lds[];
  uint16_t* pre = lds;
  float* red = reinterpret_cast<float*>(lds + 2 * kPlane);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const Dft w = make_dft(lane);
  const int64_t groups = (static_cast<int64_t>(D) + R - 1) / R;
  const int64_t total = (groups - blockIdx.x + gridDim.x - 1) / gridDim.x * B;
  auto rows_of = [&](int64_t it, const void* base, int64_t esz, bool batched) {
    const int64_t d0 = (blockIdx.x + (it / B) * gridDim.x) * R, bb = it % B;
    RowPtrs<LOGA> p;
#pragma unroll
    for (int i = 0; i < R; ++i)
      p.p[i] = d0 + i < D ? static_cast<const char*>(base) + ((batched ? bb * D : 0) + d0 + i) * L * esz
                          : nullptr;
    return p;
  };
  RowRegs<DT> rx;
  if (total > 0) fetch_rows<LOGA>(rx, rows_of(0, x, 2, true), L, false, tid);
  Spectrum spk;
  float sk[R];
  for (int64_t it = 0; it < total; ++it) {
    const int64_t d0 = (blockIdx.x + (it / B) * gridDim.x) * R, bb = it % B;
    if (bb == 0) {
      // a new channel group: its kernel rows, transformed once
      RowRegs<MEGA_F32> rk;
      fetch_rows<LOGA>(rk, rows_of(it, k, 4, false), L, false, tid);
      place_rows<LOGA>(pre, red, rk, false, tid, sk);
      transform<LOGA, false, LOGA == 5>(pre, w, wave, lane);
      capture_spectrum<LOGA>(pre, spk, tid);
      if (spec_k != nullptr) {
        uint32_t* const save_k = spec_k + static_cast<size_t>(d0 / R) * kSpecWords;
        store_spectrum(save_k, spk, tid);
#pragma unroll
        for (int i = 0; i < R; ++i)
          if (tid == i) reinterpret_cast<float*>(save_k + kSpecScaleWords)[i] = sk[i];
      }
      lds_barrier();
    }
    const RowPtrs<LOGA> xrows = rows_of(it, x, 2, true);
    float wres[R], sx[R], scale[R];
#pragma unroll
    for (int i = 0; i < R; ++i) wres[i] = (omega != nullptr && d0 + i < D) ? omega[d0 + i] : 0.f;
    place_rows<LOGA>(pre, red, rx, false, tid, sx);
    transform<LOGA, false, LOGA == 5>(pre, w, wave, lane);
    uint32_t* save_x = nullptr;
    if (spec_x != nullptr) {
      save_x = spec_x + static_cast<size_t>((bb * D + d0) / R) * kSpecWords;
#pragma unroll
      for (int i = 0; i < R; ++i)
        if (tid == i) reinterpret_cast<float*>(save_x + kSpecScaleWords)[i] = sx[i];
    }
    pointwise<LOGA>(pre, spk, tid, save_x);
    lds_barrier();
    if (it + 1 < total) fetch_rows<LOGA>(rx, rows_of(it + 1, x, 2, true), L, false, tid);
    transform<LOGA, true, LOGA == 5>(pre, w, wave, lane);
    final_scales<LOGA>(sx, sk, scale);
    store_rows<LOGA, DT, false>(pre, rows_of(it, y, 2, true), L, false, scale,
                                omega != nullptr ? &xrows : nullptr, wres, tid);
    lds_barrier();
  }
}

// digits a per row for a row of L samples: the smallest of 4, 8, 16, 32 with L <= 1024 A
inline int loga_of(int64_t L) { return L > 16384 ? 5 : (L > 8192 ? 4 : (L > 4096 ? 3 : 2)); }

template <int DT, int LOGA>
int launch_bwd(const void* dy, const void* x, const float* k, void* dx, float* dk, int64_t B,
               int64_t D, int64_t L, const float* omega, hipStream_t stream) {
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  MEGA_CHECK_HIP(hipFuncSetAttribute(
      reinterpret_cast<const void*>(&fftconv_mfma_bwd_kernel<DT, LOGA>),
      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsBytes)));
  MEGA_CHECK_ARG(B * D <= 0x7fffffff, "fftconv: too many rows");
  const int64_t groups = (D + Geo<LOGA>::R - 1) / Geo<LOGA>::R;
  const unsigned grid = static_cast<unsigned>(groups < cus ? groups : cus);
  fftconv_mfma_bwd_kernel<DT, LOGA><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
      dy, x, k, dx, dk, static_cast<int>(B), static_cast<int>(D), static_cast<int>(L), omega);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT, int LOGA>
int launch_bwd_saved(const void* dy, const uint32_t* spec_x, const uint32_t* spec_k, void* dx,
                     float* dk, int64_t B, int64_t D, int64_t L, const float* omega,
                     hipStream_t stream) {
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  MEGA_CHECK_HIP(hipFuncSetAttribute(
      reinterpret_cast<const void*>(&fftconv_mfma_bwd_saved_kernel<DT, LOGA>),
      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsBytes)));
  MEGA_CHECK_ARG(B * D <= 0x7fffffff, "fftconv: too many rows");
  const int64_t groups = D / Geo<LOGA>::R;
  const unsigned grid = static_cast<unsigned>(groups < cus ? groups : cus);
  fftconv_mfma_bwd_saved_kernel<DT, LOGA><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
      dy, spec_x, spec_k, dx, dk, static_cast<int>(B), static_cast<int>(D), static_cast<int>(L), omega);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT, int MODE, int LOGA>
int launch(const void* a, const void* b, void* out, int64_t B, int64_t D, int64_t L, int flip,
           const float* omega, hipStream_t stream, uint32_t* spec_a = nullptr,
           uint32_t* spec_b = nullptr) {
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  MEGA_CHECK_HIP(hipFuncSetAttribute(
      reinterpret_cast<const void*>(&fftconv_mfma_kernel<DT, MODE, LOGA>),
      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsBytes)));
  constexpr int R = Geo<LOGA>::R;
  if (MODE == 0 && B >= 2 && flip == 0 && 2 * ((D + R - 1) / R) >= cus) {
    // enough channel groups to fill the chip: one transform of k per group instead of one per row
    MEGA_CHECK_HIP(hipFuncSetAttribute(
        reinterpret_cast<const void*>(&fftconv_mfma_fwd_batch_kernel<DT, LOGA>),
        hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kLdsBytes)));
    MEGA_CHECK_ARG(B * D <= 0x7fffffff, "fftconv: too many rows");
    const int64_t groups = (D + R - 1) / R;
    const unsigned grid = static_cast<unsigned>(groups < cus ? groups : cus);
    fftconv_mfma_fwd_batch_kernel<DT, LOGA><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
        a, static_cast<const float*>(b), out, static_cast<int>(B), static_cast<int>(D),
        static_cast<int>(L), omega, spec_a, spec_b);
    MEGA_CHECK_LAUNCH();
    return MEGA_OK;
  }
  if (MODE == 0) {
    const int64_t rows = B * D;
    MEGA_CHECK_ARG(rows <= 0x7fffffff, "fftconv: too many rows");
    const int64_t passes = (rows + R - 1) / R;
    const unsigned grid = static_cast<unsigned>(passes < cus ? passes : cus);
    fftconv_mfma_kernel<DT, MODE, LOGA><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
        a, b, out, static_cast<int>(rows), static_cast<int>(D), static_cast<int>(L), flip, omega,
        spec_a, spec_b);
    MEGA_CHECK_LAUNCH();
  } else {
    const int64_t passes = (D + R - 1) / R;
    const unsigned grid = static_cast<unsigned>(passes < cus ? passes : cus);
    for (int64_t bb = 0; bb < B; ++bb) {
      const char* ab = static_cast<const char*>(a) + bb * D * L * 2;
      const char* xb = static_cast<const char*>(b) + bb * D * L * 2;
      fftconv_mfma_kernel<DT, MODE, LOGA><<<dim3(grid), kThreads, kLdsBytes, stream>>>(
          ab, xb, out, static_cast<int>(D), static_cast<int>(D), static_cast<int>(L),
          bb > 0 ? 1 : 0, nullptr, nullptr, nullptr);
      MEGA_CHECK_LAUNCH();
    }
  }
  return MEGA_OK;
}

template <int DT, int MODE>
int launch_len(const void* a, const void* b, void* out, int64_t B, int64_t D, int64_t L, int flip,
               const float* omega, hipStream_t stream, uint32_t* spec_a = nullptr,
               uint32_t* spec_b = nullptr) {
  switch (loga_of(L)) {
    case 5: return launch<DT, MODE, 5>(a, b, out, B, D, L, flip, omega, stream, spec_a, spec_b);
    case 4: return launch<DT, MODE, 4>(a, b, out, B, D, L, flip, omega, stream, spec_a, spec_b);
    case 3: return launch<DT, MODE, 3>(a, b, out, B, D, L, flip, omega, stream, spec_a, spec_b);
    default: return launch<DT, MODE, 2>(a, b, out, B, D, L, flip, omega, stream, spec_a, spec_b);
  }
}
template <int DT>
int launch_bwd_saved_len(const void* dy, const uint32_t* spec_x, const uint32_t* spec_k, void* dx,
                         float* dk, int64_t B, int64_t D, int64_t L, const float* omega,
                         hipStream_t stream) {
  switch (loga_of(L)) {
    case 5: return launch_bwd_saved<DT, 5>(dy, spec_x, spec_k, dx, dk, B, D, L, omega, stream);
    case 4: return launch_bwd_saved<DT, 4>(dy, spec_x, spec_k, dx, dk, B, D, L, omega, stream);
    case 3: return launch_bwd_saved<DT, 3>(dy, spec_x, spec_k, dx, dk, B, D, L, omega, stream);
    default: return launch_bwd_saved<DT, 2>(dy, spec_x, spec_k, dx, dk, B, D, L, omega, stream);
  }
}
template <int DT>
int launch_bwd_len(const void* dy, const void* x, const float* k, void* dx, float* dk, int64_t B,
                   int64_t D, int64_t L, const float* omega, hipStream_t stream) {
  switch (loga_of(L)) {
    case 5: return launch_bwd<DT, 5>(dy, x, k, dx, dk, B, D, L, omega, stream);
    case 4: return launch_bwd<DT, 4>(dy, x, k, dx, dk, B, D, L, omega, stream);
    case 3: return launch_bwd<DT, 3>(dy, x, k, dx, dk, B, D, L, omega, stream);
    default: return launch_bwd<DT, 2>(dy, x, k, dx, dk, B, D, L, omega, stream);
  }
}

}  // namespace

bool applicable(int dtype, int64_t L, const void* a, const void* b, const void* out) {
  const auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  return (dtype == MEGA_BF16 || dtype == MEGA_F16) && L > 2048 && L <= 32768 && L % 8 == 0 &&
         al(a) && al(b) && al(out);
}

int launch_conv(int dtype, int mode, const void* a, const void* b, void* out, int64_t B,
                int64_t D, int64_t L, int flip, const float* omega, hipStream_t stream) {
  if (dtype == MEGA_BF16)
    return mode == 0 ? launch_len<MEGA_BF16, 0>(a, b, out, B, D, L, flip, omega, stream)
                     : launch_len<MEGA_BF16, 1>(a, b, out, B, D, L, flip, omega, stream);
  return mode == 0 ? launch_len<MEGA_F16, 0>(a, b, out, B, D, L, flip, omega, stream)
                   : launch_len<MEGA_F16, 1>(a, b, out, B, D, L, flip, omega, stream);
}

int64_t spectrum_bytes(int dtype, int64_t B, int64_t D, int64_t L) {
  if ((dtype != MEGA_BF16 && dtype != MEGA_F16) || L <= 2048 || L > 32768 || L % 8 != 0) return 0;
  const int64_t R = 32 >> loga_of(L);
  if (D % R != 0) return 0;
  return B * D / R * kSpecWords * 4;
}

int launch_forward_saving(int dtype, const void* x, const float* k, void* y, int64_t B, int64_t D,
                          int64_t L, const float* omega, void* spec_x, void* spec_k,
                          hipStream_t stream) {
  uint32_t* sx = static_cast<uint32_t*>(spec_x);
  uint32_t* sk = static_cast<uint32_t*>(spec_k);
  if (dtype == MEGA_BF16) return launch_len<MEGA_BF16, 0>(x, k, y, B, D, L, 0, omega, stream, sx, sk);
  return launch_len<MEGA_F16, 0>(x, k, y, B, D, L, 0, omega, stream, sx, sk);
}

int launch_backward_saved(int dtype, const void* dy, const void* spec_x, const void* spec_k, void* dx,
                          float* dk, int64_t B, int64_t D, int64_t L, const float* omega,
                          hipStream_t stream) {
  const uint32_t* sx = static_cast<const uint32_t*>(spec_x);
  const uint32_t* sk = static_cast<const uint32_t*>(spec_k);
  if (dtype == MEGA_BF16)
    return launch_bwd_saved_len<MEGA_BF16>(dy, sx, sk, dx, dk, B, D, L, omega, stream);
  return launch_bwd_saved_len<MEGA_F16>(dy, sx, sk, dx, dk, B, D, L, omega, stream);
}

int launch_backward(int dtype, const void* dy, const void* x, const float* k, void* dx, float* dk,
                    int64_t B, int64_t D, int64_t L, const float* omega, hipStream_t stream) {
  if (dtype == MEGA_BF16)
    return launch_bwd_len<MEGA_BF16>(dy, x, k, dx, dk, B, D, L, omega, stream);
  return launch_bwd_len<MEGA_F16>(dy, x, k, dx, dk, B, D, L, omega, stream);
}

}  // namespace fftm
}  // namespace mega
