// The CEMA layer as a chunked linear recurrence on the matrix cores.
//
// The layer's convolution kernel is a sum of N damped complex exponentials,
//   k[j] = Re sum_n c_n q_n^j,  c_n = p_n gamma_n
// (megalodon/csrc/ops/ema_parameters.cc:37-52), so
//   y = fftconv(x, k) + omega x  (+ the bias of a carried state)
// (megalodon/modules/complex_exponential_moving_average.py:127-147) is the
// output of the recurrence h[t] = q h[t-1] + p x[t], y[t] = Re sum_n gamma_n
// h_n[t] + omega x[t] (the same states ema_hidden.cc:31-61 returns).  Neither k
// nor any spectrum is formed.  A row is cut into chunks of T = 64 steps; with
// X[c][j] = x[64 c + j]:
//   S[c]    = P X[c],          P[m][j]  = (Re, Im)(p_n q_n^(63-j)),  m = 2 n + part   (local state)
//   H[c]    = q^64 H[c-1] + S[c],  H[-1] = carried state                             (scan over chunks)
//   Y[c]    = K X[c] + Q H[c-1],  K[i][j] = k[i-j] (i >= j),  Q[i][m] = (Re, -Im)(gamma_n q_n^(i+1))
// The three products are MFMAs with the chunks of a tile as the 32 columns
// (v_mfma_f32_32x32x16_bf16); a row of x is read from memory once, straight
// into operand registers (a lane's 16-byte load is 8 consecutive steps of one
// chunk), and y is written once from the accumulators.  Parameter matrices are
// float32 values split into two bf16 pieces (hi + lo, 16 significant bits); x in
// bf16 is exact, fp16 x is split into two exact bf16 pieces; the states are
// float32 and split the same way; accumulation is float32.
//
// One workgroup of four waves owns a row; a segment of 128 NT chunks is
// resident at a time: wave w holds chunk tiles NT w .. NT w + NT - 1 of it
// (NT = 1 is what the entry point launches: 8192 steps per segment).
#include "common.hpp"
#include "cema_pow.hpp"

#include <type_traits>

namespace mega {
namespace {

constexpr int kT = 64;         // steps per chunk
constexpr int kThreads = 256;  // four waves
constexpr int kWaves = kThreads / kWave;
constexpr int kHP = 36;        // floats per state row in LDS: 32 + 4 (16-byte rows 8 lanes apart hit 32 banks)
constexpr int kSubs = 16;      // sub-segments of the chunk scan (one per 16 threads)

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
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// a <-> b between the two halves of the wave (v_permlane32_swap_b32): afterwards
// the low half holds (its own a, the high half's a), the high half (the low
// half's b, its own b).  Written as inline assembly: the compiler's builtin
// returned the first result for both outputs here.  The compiler does not
// see what the assembly reads, so it guards none of the hazards: the s_nop
// covers the wait states after a vector write of an operand, and operands
// that come out of an MFMA must first pass through an ordinary vector
// instruction (`settle`), which the compiler does schedule behind the MFMA.
__device__ __forceinline__ void half_swap(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void half_swap(uint32_t& a, uint32_t& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// two floats -> one word of two 16-bit elements of type DT
template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if (DT == MEGA_BF16) return pack_bf16x2(lo, hi);
  return static_cast<uint32_t>(float_to_f16_bits(lo)) | (static_cast<uint32_t>(float_to_f16_bits(hi)) << 16);
}
// An accumulator tile (lane <-> chunk, register 4 qd + e <-> step 8 qd + 4 g + e of a 32-step
// row tile) rounded to 16 bits and regrouped so that the lane of half g holds the 8
// consecutive steps 16 pr + 8 g .. + 7: the rounding is the ordinary vector instruction
// that separates the MFMA from the swaps (see half_swap).
template <int DT>
__device__ __forceinline__ uint4 octet_of(const floatx16& acc, int pr) {
  uint32_t a0 = pack2<DT>(acc[8 * pr], acc[8 * pr + 1]), a1 = pack2<DT>(acc[8 * pr + 2], acc[8 * pr + 3]);
  uint32_t b0 = pack2<DT>(acc[8 * pr + 4], acc[8 * pr + 5]), b1 = pack2<DT>(acc[8 * pr + 6], acc[8 * pr + 7]);
  half_swap(a0, b0);
  half_swap(a1, b1);
  return make_uint4(a0, a1, b0, b1);
}
// Makes a lane-derived value opaque to the optimiser.  Offsets, masks and converted indices
// depend only on the lane, not on the row: left alone they are hoisted out of the persistent
// row loop into hundreds of spilled registers; recomputing them per item is cheaper.
__device__ __forceinline__ int opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}
// 1.0f the optimiser cannot see through
__device__ __forceinline__ float opaque_one() {
  float one = 1.0f;
  asm volatile("" : "+v"(one));
  return one;
}

// Eight consecutive steps of a row as a matrix operand: XP bf16 pieces whose sum
// is the data exactly (bf16: the data itself; fp16: two pieces).
template <int DT> struct XOp;
template <> struct XOp<MEGA_BF16> {
  static constexpr int XP = 1;
  u32x4 pc[1];
  __device__ __forceinline__ void load(const void* row, int64_t elem, bool on) {
    pc[0] = on ? *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(row) + elem) : u32x4{0u, 0u, 0u, 0u};
  }
  __device__ __forceinline__ void values(float* v) const {
    unpack8<MEGA_BF16>(make_uint4(pc[0][0], pc[0][1], pc[0][2], pc[0][3]), v);
  }
};
template <> struct XOp<MEGA_F16> {
  static constexpr int XP = 2;
  u32x4 pc[2];
  __device__ __forceinline__ void load(const void* row, int64_t elem, bool on) {
    float v[8];
    uint4 raw = make_uint4(0u, 0u, 0u, 0u);
    if (on) raw = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(row) + elem);
    unpack8<MEGA_F16>(raw, v);
    split8(v, pc[0], pc[1]);
  }
  __device__ __forceinline__ void values(float* v) const {
    float a[8], b[8];
    unpack8<MEGA_BF16>(make_uint4(pc[0][0], pc[0][1], pc[0][2], pc[0][3]), a);
    unpack8<MEGA_BF16>(make_uint4(pc[1][0], pc[1][1], pc[1][2], pc[1][3]), b);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = a[e] + b[e];
  }
};

// float32 rows: the two leading bf16 pieces (16 significant bits, what the parameter matrices
// carry as well); the rest, 2^-17 of a value, is left out
template <> struct XOp<MEGA_F32> {
  static constexpr int XP = 2;
  u32x4 pc[2];
  __device__ __forceinline__ void load(const void* row, int64_t elem, bool on) {
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
    if (on) {
      const float4* src = reinterpret_cast<const float4*>(static_cast<const float*>(row) + elem);
      a = src[0];
      b = src[1];
    }
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    split8(v, pc[0], pc[1]);
  }
};

// acc += (A_hi + A_lo) * x with the lo * lo term of a two-piece x left out
template <int XP>
__device__ __forceinline__ floatx16 mma_split(const u32x4* a, const u32x4* x, floatx16 acc) {
  acc = mfma_bf16(a[0], x[0], acc);
  acc = mfma_bf16(a[1], x[0], acc);
  if (XP == 2) acc = mfma_bf16(a[0], x[1], acc);
  return acc;
}

// Operand blocks of the forward kernel (each 64 lanes x 8 values, two pieces):
//   0..3   P, k-step s:            rows m, steps j = 16 s + 8 g + e
//   4..7   K by offset o = 16 (b - 5): rows r, lag = o + r - 8 g - e (zero where negative)
//   8..11  Q, (row tile it, k-step s2): rows i = 32 it + r, state columns m = 16 s2 + 8 g + e
constexpr int kFwdBlocks = 12;

template <int NT>
struct FwdSmem {
  static constexpr int NC = kWaves * NT * 32;  // chunks per segment
  float klocal[kT];                            // k[0 .. 63] (+ omega at lag 0)
  float pn[16];
  cf gn[16];
  cf sub_end[kSubs][16];                       // local end state of each sub-segment (4 per wave)
  cf wave_end[2][kWaves][16];                  // local end state of each wave's 4 sub-segments, by item parity
  float wave_cin[kWaves][32];                  // state in front of each wave's first chunk
  cf carry[2][16];
  cf pw[12][16];                               // q^(4 k), q^(16 k) (k < 4), q, q^64, q^(64 CPS), q^(256 CPS)
  u32x4 aop[kFwdBlocks][2][kWave];
  // row 1 + c: state after chunk c of the segment; while a row is set up the buffer holds the
  // power table q_n^e, e = 0 .. 64 (16 x 66 complex), from which the operand blocks are built
  float H[(NC + 1) * kHP];
};
static_assert(sizeof(cf) * 16 * (kT + 2) <= sizeof(float) * (kWaves * 32 + 1) * kHP, "the power table fits the state buffer");

// LDS traffic of one wave is processed in order: a wave that has written rows
// and waits for its own LDS operations can read what its other lanes wrote.
__device__ __forceinline__ void wave_sync() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

template <int DT, int NT>
__global__ __launch_bounds__(kThreads, NT == 1 ? 3 : 2) void cema_scan_fwd_kernel(
    const void* __restrict__ x, void* __restrict__ y, const float* __restrict__ p,
    const cf* __restrict__ log_q, const cf* __restrict__ gamma, const float* __restrict__ omega,
    const cf* __restrict__ h0, cf* __restrict__ h_last, int64_t rows, int D, int N, int64_t L) {
  using Smem = FwdSmem<NT>;
  constexpr int NC = Smem::NC, CPS = NC / kSubs, XP = XOp<DT>::XP;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
  cf (*qp)[kT + 2] = reinterpret_cast<cf(*)[kT + 2]>(sm.H);  // while a row is set up
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int g = lane >> 5, r = lane & 31;
  // scan roles: mode sn; sub-segment sa = 4 wave + sl of CPS chunks, inside the wave's own tiles
  const int sn = tid & 15, sa = tid >> 4, sl = sa & 3;
  const int64_t C = (L + kT - 1) / kT;

  // The workgroup walks (row, segment) items: rows blockIdx.x, + gridDim.x, ...,
  // the segments of a row in time order.  The x tiles of the next item and the
  // parameters of the next row are requested ahead (two register sets for the
  // tiles, swapped by taking the item body twice per loop turn).
  auto load_tiles = [&](XOp<DT> (&t)[NT][4], int64_t row, int64_t seg0) {
    const typename Elem<DT>::type* xrow = static_cast<const typename Elem<DT>::type*>(x) + row * L;
#pragma unroll
    for (int ctl = 0; ctl < NT; ++ctl) {
      const int64_t chunk = seg0 + (wave * NT + ctl) * 32 + r;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int64_t elem = chunk * kT + 16 * s + 8 * g;
        t[ctl][s].load(xrow, elem, row < rows && elem + 8 <= L);
      }
    }
  };
  struct RowParams {
    cf lq, gv, hv;
    float pv, w;
  };
  auto fetch_params = [&](int64_t row) {
    RowParams rp{cf{0.f, 0.f}, cf{0.f, 0.f}, cf{0.f, 0.f}, 0.f, 0.f};
    if (row < rows) {
      const int d = static_cast<int>(row % D);
      if (sn < N) {
        rp.lq = log_q[d * N + sn];
        rp.gv = gamma[d * N + sn];
        rp.pv = p[d * N + sn];
        if (h0 != nullptr && tid < 16) rp.hv = h0[row * N + sn];
      }
      if (omega != nullptr) rp.w = omega[d];
    }
    return rp;
  };

  cf qT{0.f, 0.f}, qS{0.f, 0.f}, qW{0.f, 0.f};
  int cur = 0, par = 0;
  RowParams rp = fetch_params(blockIdx.x);

  // tables, operand blocks and scan multipliers of a row's channel, from the
  // parameters fetched ahead; then the next row's parameters are requested
  auto setup_row = [&](int64_t row) {
    // the few powers that are evaluated directly (phase reduced in float64): 12 per mode;
    // everything else is a product of two of them and a short chain of multiplications
    cf direct{0.f, 0.f};
    if (tid < 12 * 16 && sn < N) {
      const int k = tid >> 4;
      const int e = k < 4 ? 4 * k
                          : (k < 8 ? 16 * (k - 4) : (k == 8 ? 1 : (k == 9 ? kT : (k == 10 ? kT * CPS : 4 * kT * CPS))));
      direct = qpow(rp.lq.x, rp.lq.y, e);
    }
    __syncthreads();  // every wave is done with the previous row's tables and carried state
    if (tid < 12 * 16) sm.pw[tid >> 4][sn] = direct;
    if (tid < 16) {
      sm.pn[tid] = rp.pv;
      sm.gn[tid] = rp.gv;
      sm.carry[0][tid] = rp.hv;
    }
    cur = 0;
    __syncthreads();
    {
      // q^(4 sa + e), e < 4, and this mode's share of k at those lags, summed over the
      // 16 modes (the 16 lanes of a row): the skip term omega x rides on k[0]
      cf v = cmul(sm.pw[sa & 3][sn], sm.pw[4 + (sa >> 2)][sn]);
      const cf q1 = sm.pw[8][sn];
      const cf c{rp.pv * rp.gv.x, rp.pv * rp.gv.y};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        qp[sn][4 * sa + e] = v;
        const float kl = group_sum<16>(c.x * v.x - c.y * v.y);
        if (sn == 0) sm.klocal[4 * sa + e] = (sa == 0 && e == 0) ? kl + rp.w : kl;
        v = cmul(v, q1);
      }
      if (sa == 15) qp[sn][kT] = sm.pw[9][sn];
      qT = sm.pw[9][sn];
      qS = sm.pw[10][sn];
      qW = sm.pw[11][sn];
    }
    const RowParams next_rp = fetch_params(row + gridDim.x);
    __syncthreads();
    for (int item = tid; item < kFwdBlocks * kWave; item += kThreads) {
      const int blk = item >> 6, ln = item & 63, rr = ln & 31, gg = ln >> 5;
      float v[8];
      if (blk < 4) {
        const int n = rr >> 1, part = rr & 1;
        const float pp = sm.pn[n];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const cf w = qp[n][kT - 1 - (16 * blk + 8 * gg + e)];
          v[e] = pp * (part ? w.y : w.x);
        }
      } else if (blk < 8) {
        const int o = 16 * (blk - 5);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int lag = o + rr - 8 * gg - e;
          const float kv = sm.klocal[lag >= 0 ? lag : 0];  // read, then masked: no branch around the load
          v[e] = lag >= 0 ? kv : 0.f;
        }
      } else {
        const int it = (blk - 8) >> 1, s2 = (blk - 8) & 1, i = 32 * it + rr;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int m = 16 * s2 + 8 * gg + e, n = m >> 1;
          const cf w = cmul(sm.gn[n], qp[n][i + 1]);
          v[e] = (m & 1) ? -w.y : w.x;
        }
      }
      u32x4 hi, lo;
      split8(v, hi, lo);
      sm.aop[blk][0][ln] = hi;
      sm.aop[blk][1][ln] = lo;
    }
    __syncthreads();
    rp = next_rp;
  };
  // The operand blocks stay in LDS and are read where a phase needs them (P for the local
  // states, K and Q for the outputs): held in registers across the whole item they cost
  // 96 registers and spill.
  auto load_block = [&](int b, u32x4* dst) {
    dst[0] = sm.aop[b][0][lane];
    dst[1] = sm.aop[b][1][lane];
  };

  // One (row, segment) item.  The item's x tiles were requested by the previous item (or
  // the prologue); everything that reads them -- the local states and the K X part of the
  // outputs -- comes first, then the same registers are reloaded with the next item's tiles
  // while the scan and the state part of the outputs run.
  XOp<DT> xb[NT][4];
  auto item = [&](int64_t row, int64_t seg0) {
    if (seg0 == 0) setup_row(row);
    typename Elem<DT>::type* yrow = static_cast<typename Elem<DT>::type*>(y) + row * L;
    const int nc = static_cast<int>(C - seg0 < NC ? C - seg0 : NC);
    floatx16 yacc[NT][2];
    // ---- local states S = P X, into this wave's own rows of the state buffer ----------
    {
      u32x4 P[4][2];
#pragma unroll
      for (int s = 0; s < 4; ++s) load_block(s, P[s]);
#pragma unroll
      for (int ctl = 0; ctl < NT; ++ctl) {
        const int c0 = (wave * NT + ctl) * 32;
        if (c0 < nc) {
          floatx16 acc;
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
          for (int s = 0; s < 4; ++s) acc = mma_split<XP>(P[s], xb[ctl][s].pc, acc);
          float* dst = sm.H + (1 + c0 + r) * kHP + 4 * g;
#pragma unroll
          for (int qd = 0; qd < 4; ++qd)
            *reinterpret_cast<float4*>(dst + 8 * qd) =
                make_float4(acc[4 * qd], acc[4 * qd + 1], acc[4 * qd + 2], acc[4 * qd + 3]);
        }
      }
    }
    // ---- the within-chunk part of the outputs, K X (omega x included: K carries omega on
    //      its diagonal); the accumulators wait for the state part ------------------------
    {
      u32x4 K[4][2];
#pragma unroll
      for (int b = 0; b < 4; ++b) load_block(4 + b, K[b]);
#pragma unroll
      for (int ctl = 0; ctl < NT; ++ctl)
#pragma unroll
        for (int it = 0; it < 2; ++it) {
#pragma unroll
          for (int i = 0; i < 16; ++i) yacc[ctl][it][i] = 0.f;
          if ((wave * NT + ctl) * 32 < nc) {
#pragma unroll
            for (int s = 0; s < 2 + 2 * it; ++s)
              yacc[ctl][it] = mma_split<XP>(K[1 + 2 * it - s], xb[ctl][s].pc, yacc[ctl][it]);
          }
        }
    }
    {
      int64_t nrow = row, nseg = seg0 + NC;
      if (nseg >= C) {
        nrow = row + gridDim.x;
        nseg = 0;
      }
      load_tiles(xb, nrow, nseg);
    }
    wave_sync();
    // ---- scan over the chunks of the segment: a sub-segment per 16 lanes, the wave's four
    //      sub-segments are its own chunks; one workgroup barrier hands over the waves' ends -----
    {
      float* col = sm.H + kHP + 2 * sn;  // state column n of row 1 + c
      float2 sv[CPS];                    // the sub-segment's local states, kept for the second pass
#pragma unroll
      for (int i = 0; i < CPS; ++i) {
        const int c = sa * CPS + i;
        const float2 s0 = *reinterpret_cast<const float2*>(col + c * kHP);  // read, then masked
        sv[i] = c < nc ? s0 : make_float2(0.f, 0.f);
      }
      cf h{0.f, 0.f};
#pragma unroll
      for (int i = 0; i < CPS; ++i) h = cadd(cmul(qT, h), cf{sv[i].x, sv[i].y});
      sm.sub_end[sa][sn] = h;
      wave_sync();
      if (sl == 3) {
        cf e = sm.sub_end[sa - 3][sn];
        e = cadd(cmul(qS, e), sm.sub_end[sa - 2][sn]);
        e = cadd(cmul(qS, e), sm.sub_end[sa - 1][sn]);
        sm.wave_end[par][wave][sn] = cadd(cmul(qS, e), h);
      }
      lds_barrier();
      cf cin = sm.carry[cur][sn];
#pragma unroll
      for (int w = 0; w < kWaves - 1; ++w) {
        const cf e = sm.wave_end[par][w][sn];
        if (w < wave) cin = cadd(cmul(qW, cin), e);
      }
      if (sa == kSubs - 1) sm.carry[cur ^ 1][sn] = cadd(cmul(qW, cin), sm.wave_end[par][kWaves - 1][sn]);
      if (sl == 0) *reinterpret_cast<float2*>(sm.wave_cin[wave] + 2 * sn) = make_float2(cin.x, cin.y);
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        const cf e = sm.sub_end[4 * wave + s][sn];
        if (s < sl) cin = cadd(cmul(qS, cin), e);
      }
      h = cin;
#pragma unroll
      for (int i = 0; i < CPS; ++i) {
        const int c = sa * CPS + i;
        h = cadd(cmul(qT, h), cf{sv[i].x, sv[i].y});
        if (c < nc) *reinterpret_cast<float2*>(col + c * kHP) = make_float2(h.x, h.y);
      }
    }
    wave_sync();
    // ---- the state part of the outputs, Q H[c-1], and the stores ------------------------------
    {
      u32x4 Q[4][2];
#pragma unroll
      for (int b = 0; b < 4; ++b) load_block(8 + b, Q[b]);
#pragma unroll
      for (int ctl = 0; ctl < NT; ++ctl) {
        const int c0 = (wave * NT + ctl) * 32;
        if (c0 < nc) {
          u32x4 hb[2][2];
          // the state in front of chunk c0 + r: the previous row of the buffer, or, for the
          // wave's first chunk, what the scan left in wave_cin
          const float* hrow = (ctl == 0 && r == 0) ? sm.wave_cin[wave] : sm.H + (c0 + r) * kHP;
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const float* src = hrow + 16 * s2 + 8 * g;
            const float4 u = *reinterpret_cast<const float4*>(src);
            const float4 w = *reinterpret_cast<const float4*>(src + 4);
            const float v[8] = {u.x, u.y, u.z, u.w, w.x, w.y, w.z, w.w};
            split8(v, hb[s2][0], hb[s2][1]);
          }
          const int64_t chunk = seg0 + c0 + r;
#pragma unroll
          for (int it = 0; it < 2; ++it) {
            floatx16 acc = yacc[ctl][it];
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
              acc = mfma_bf16(Q[2 * it + s2][0], hb[s2][0], acc);
              acc = mfma_bf16(Q[2 * it + s2][1], hb[s2][0], acc);
              acc = mfma_bf16(Q[2 * it + s2][0], hb[s2][1], acc);
            }
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
              if constexpr (DT == MEGA_F32) {
                // registers 8 pr + 4 h + e hold the steps 16 pr + 8 h + 4 g + e: two 16-byte stores
                // per lane, no exchange between the halves of the wave
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                  const int64_t elem = chunk * kT + 16 * (2 * it + pr) + 8 * h + 4 * g;
                  if (elem + 4 <= L)
                    *reinterpret_cast<float4*>(yrow + elem) = make_float4(acc[8 * pr + 4 * h], acc[8 * pr + 4 * h + 1],
                                                                          acc[8 * pr + 4 * h + 2], acc[8 * pr + 4 * h + 3]);
                }
              } else {
                const uint4 oct = octet_of<DT>(acc, pr);
                const int64_t elem = chunk * kT + 16 * (2 * it + pr) + 8 * g;
                if (elem + 8 <= L) *reinterpret_cast<uint4*>(yrow + elem) = oct;
              }
            }
          }
        }
      }
    }
    cur ^= 1;
    par ^= 1;
    if (seg0 + NC >= C && h_last != nullptr) {
      // the row's last segment: the state after step L - 1 (the last chunk may be partial)
      lds_barrier();
      if (tid < N) {
        const typename Elem<DT>::type* xrow = static_cast<const typename Elem<DT>::type*>(x) + row * L;
        const int rem = static_cast<int>(L - (C - 1) * kT);  // 1 .. 64 steps in the last chunk
        const int cl = static_cast<int>(C - 1 - seg0);       // the last chunk inside this segment
        cf h;
        if (rem == kT) {
          const float* lastrow = sm.H + (1 + cl) * kHP + 2 * tid;
          h = cf{lastrow[0], lastrow[1]};
        } else {
          // H[C-2]: the row in front of the last chunk, or the wave's carried-in state
          const float* prev = (cl % (NT * 32) == 0) ? sm.wave_cin[cl / (NT * 32)] + 2 * tid
                                                    : sm.H + cl * kHP + 2 * tid;
          // the recurrence itself over the last chunk's steps (the power table has made way for
          // the states by now): h <- q h + p x
          h = cf{prev[0], prev[1]};
          const cf q1 = sm.pw[8][tid];
          const float pp = sm.pn[tid];
          for (int j = 0; j < rem; ++j) {
            const float xv = Elem<DT>::load(xrow + (C - 1) * kT + j) * pp;
            h = cmul(q1, h);
            h.x += xv;
          }
        }
        h_last[row * N + tid] = h;
      }
    }
  };

  load_tiles(xb, blockIdx.x, 0);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x)
    for (int64_t seg0 = 0; seg0 < C; seg0 += NC) item(row, seg0);
}

template <int DT, int NT>
int launch_fwd(const void* x, void* y, const float* p, const cf* log_q, const cf* gamma,
               const float* omega, const cf* h0, cf* h_last, int64_t B, int64_t D, int64_t N,
               int64_t L, hipStream_t stream) {
  const size_t lds = sizeof(FwdSmem<NT>);
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&cema_scan_fwd_kernel<DT, NT>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  const int64_t rows = B * D, slots = (NT == 1 ? 3 : 2) * static_cast<int64_t>(cus);  // workgroups that fit a compute unit
  const unsigned grid = static_cast<unsigned>(rows < slots ? rows : slots);
  cema_scan_fwd_kernel<DT, NT><<<dim3(grid), kThreads, lds, stream>>>(
      x, y, p, log_q, gamma, omega, h0, h_last, rows, static_cast<int>(D), static_cast<int>(N), L);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}


// ------------------------------ backward ------------------------------------
// With c_n = p_n gamma_n and, per mode,
//   A = sum_{t >= s} dy[t] x[s] q^(t-s),   B = dA / dq
// the gradients the reference forms from dk (ema_parameters.cc:80-98 after
// fftconv.py:53-75) are dp = Re(A gamma), dq = conj(B p gamma), dgamma = conj(A p),
// domega = sum dy x, and dx[s] = sum_{t >= s} k[t-s] dy[t] + omega dy[s].  By chunks, in
// reverse time (DY[c][i] = dy[64 c + i], XR[c][j'] = x[64 c + 63 - j']):
//   (G, G')[c]   = Pg DY[c],     Pg = rows (Re, Im)(q^i), then (Re, Im)(i q^(i-1)), i < 64
//   R[c]  = G[c] + q^64 R[c+1],   R'[c] = G'[c] + 64 q^63 R[c+1] + q^64 R'[c+1]      (scan)
//   (X, X')[c]   = Pg XR[c]
//   W  = sum_c X[c] R[c+1],   W' = sum_c (X'[c] R[c+1] + X[c] R'[c+1])
//   DX[c] = K^T DY[c] + Qd R[c+1],   Qd[j][m] = (Re, -Im)(c_n q_n^(64-j)),  omega on the diagonal of K
//   M     = sum_c DY[c]^T X[c]   (64 x 64, rows i >= columns j), dkin[l] = sum_j M[j+l][j]
//   A = sum_l q^l dkin[l] + q W,   B = sum_l l q^(l-1) dkin[l] + W + q W'
// Segments of 128 chunks are taken from the end of the row to its start; a
// wave holds one chunk tile of the segment.  The chunk-contracted product M
// needs operands with chunks along k: the wave parks its DY and X tiles in a
// private LDS tile and reads them back with the transposing LDS read; the same
// tile hands out the time-reversed x operand.  Everything that reads the dy
// and x tiles comes before the scan, so the next item's tiles load under it.
constexpr int kRP = 68;       // floats per row of the reverse-state buffer: (R, R') = 64 + 4
constexpr int kSP = 72;       // 16-bit elements per row of a wave's staging tile: 64 + 8
constexpr int kBwdNC = kWaves * 32;  // chunks per segment
constexpr int kBwdCPS = kBwdNC / kSubs;
constexpr int kBwdBlocks = 16;  // Pg 0..7 (kind, k-step), K^T 8..11 (by offset), Qd 12..15 (row tile, k-step)

typedef short short4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_read_tr(const uint16_t* q) {
  const short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) short4v*)(q));
  return __builtin_bit_cast(uint2, v);
}

struct BwdSmem {
  u32x4 aop[kBwdBlocks][2][kWave];       // operand blocks, two pieces
  // row c: (R, R') at the start of chunk c of the segment.  A wave's own 32 rows double as its
  // private tile for the parked dy / x data before they are written; between rows the buffer
  // holds the power table (setup) and the reduction scratch (finish).
  float R[kBwdNC * kRP];
  float klocal[kT];
  float pn[16];
  cf gn[16];
  cf pw[14][16];                         // powers evaluated directly (see setup_row)
  cf sub_end[kSubs][2][16];              // local (R, R') at the start of each sub-segment
  cf wave_end[2][kWaves][2][16];         // the same for each wave's four sub-segments, by item parity
  float wave_cin[kWaves][64];            // (R, R') behind each wave's last chunk
  cf carry[2][2][16];
  float red[kWaves][2][32];
  float dpart[kWaves][kT];
  float dkin[kT];
};
static_assert(sizeof(cf) * 16 * (kT + 2) + sizeof(cf) * 16 * 2 * 16 <= sizeof(float) * kBwdNC * kRP,
              "the power table and the final partial sums live in the state buffer");
static_assert(32 * kSP * 2 <= 32 * kRP * 4 && 16 * kWave * 4 <= 32 * kRP * 4 && kWave * 33 <= 32 * kRP,
              "a wave's parked tile and one accumulator tile fit its own rows of the state buffer");
static_assert(sizeof(BwdSmem) <= 80 * 1024, "two workgroups per compute unit");

// (h, h') <- (g, g') + [[m, 0], [md, m]] (h, h'): one step of the reverse scan, over a chunk
// (m = q^64, md = 64 q^63), a sub-segment or a wave's chunks (the same form with larger powers)
__device__ __forceinline__ void rstep(cf& h, cf& hd, cf g, cf gd, cf m, cf md) {
  const cf nd = cadd(gd, cadd(cmul(md, h), cmul(m, hd)));
  h = cadd(g, cmul(m, h));
  hd = nd;
}

// DX32: dx is written in float32 (or, with a null pointer, not at all) instead of the rows'
// own type -- for callers that add up the backward of several bfloat16 pieces of one tensor;
// DX32 == 2 adds to what dx holds instead of overwriting it.
template <int DT, int DX32>
__global__ __launch_bounds__(kThreads, 2) void cema_scan_bwd_kernel(
    const void* __restrict__ dy, const void* __restrict__ x, void* __restrict__ dx,
    const float* __restrict__ p, const cf* __restrict__ log_q, const cf* __restrict__ gamma,
    const float* __restrict__ omega, const cf* __restrict__ h0, float* __restrict__ dp, cf* __restrict__ dq,
    cf* __restrict__ dgamma, float* __restrict__ domega, cf* __restrict__ dh0, int64_t rows, int D, int N,
    int64_t L) {
  static_assert(XOp<DT>::XP == 1, "the backward kernel takes bfloat16 rows");
  constexpr int NC = kBwdNC, CPS = kBwdCPS;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  BwdSmem& sm = *reinterpret_cast<BwdSmem*>(smem_raw);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  // lane-derived indices, re-derived from an opaque thread id wherever a phase starts
#define MEGA_LANE_IDS                                                          \
  const int tid = opaque(threadIdx.x) & (kThreads - 1), lane = tid & (kWave - 1); \
  const int g = lane >> 5, r = lane & 31, sn = tid & 15, sa = tid >> 4, sl = sa & 3; \
  (void)g; (void)r; (void)sn; (void)sa; (void)sl; (void)lane;                   \
  float* const myrows = sm.R + wave * 32 * kRP;                                \
  uint16_t* const stage = reinterpret_cast<uint16_t*>(myrows);                 \
  (void)stage
  cf (*qp)[kT + 2] = reinterpret_cast<cf(*)[kT + 2]>(sm.R);                 // setup and finish only
  cf (*ab)[2][16] = reinterpret_cast<cf(*)[2][16]>(sm.R + 2 * 16 * (kT + 2));  // finish only, behind the table
  const int64_t C = (L + kT - 1) / kT;
  const int64_t seg_last = (C - 1) / NC * NC;

  XOp<DT> db[4], xb[4], dn[4];  // dn: the next item's dy tile on its way
  auto load_dy = [&](int64_t row, int64_t seg0) {
    MEGA_LANE_IDS;
    const uint16_t* dyrow = static_cast<const uint16_t*>(dy) + row * L;
    const int64_t chunk = seg0 + wave * 32 + r;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int64_t elem = chunk * kT + 16 * s + 8 * g;
      dn[s].load(dyrow, elem, row < rows && elem + 8 <= L);
    }
  };
  auto load_x = [&](int64_t row, int64_t seg0) {
    MEGA_LANE_IDS;
    const uint16_t* xrow = static_cast<const uint16_t*>(x) + row * L;
    const int64_t chunk = seg0 + wave * 32 + r;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int64_t elem = chunk * kT + 16 * s + 8 * g;
      xb[s].load(xrow, elem, row < rows && elem + 8 <= L);
    }
  };
  struct RowParams {
    cf lq, gv;
    float pv, w;
  };
  auto fetch_params = [&](int64_t row) {
    MEGA_LANE_IDS;
    RowParams rp{cf{0.f, 0.f}, cf{0.f, 0.f}, 0.f, 0.f};
    if (row < rows) {
      const int d = static_cast<int>(row % D);
      if (sn < N) {
        rp.lq = log_q[d * N + sn];
        rp.gv = gamma[d * N + sn];
        rp.pv = p[d * N + sn];
      }
      if (omega != nullptr) rp.w = omega[d];
    }
    return rp;
  };
  auto load_block = [&](int b, u32x4* dst, int lane) {
    dst[0] = sm.aop[b][0][lane];
    dst[1] = sm.aop[b][1][lane];
  };

  // scan multipliers of this thread's mode: over a chunk, a sub-segment, a wave's chunks
  cf qT{0.f, 0.f}, qTd{0.f, 0.f}, q1{0.f, 0.f};
  int cur = 0, par = 0;
  RowParams rp = fetch_params(blockIdx.x);


  // per-row accumulators
  floatx16 macc[3];      // M tiles (0,0), (1,0), (1,1) over this wave's chunks
  cf wacc[8], wdacc[8];  // W, W' of modes n = 4 qd + 2 g + b at index 2 qd + b, over this lane's chunks

  auto setup_row = [&](int64_t row) {
    MEGA_LANE_IDS;
    // powers evaluated directly (phase reduced in float64), 14 per mode: q^(4 k), q^(16 k)
    // (k < 4), q, q^64, q^(64 CPS), q^(64 CPS - 1), q^(256 CPS), q^(256 CPS - 1)
    cf direct{0.f, 0.f};
    if (tid < 14 * 16 && sn < N) {
      const int k = tid >> 4;
      const int tab[6] = {1, kT, kT * CPS, kT * CPS - 1, 4 * kT * CPS, 4 * kT * CPS - 1};
      const int e = k < 4 ? 4 * k : (k < 8 ? 16 * (k - 4) : tab[k - 8]);
      direct = qpow(rp.lq.x, rp.lq.y, e);
    }
    __syncthreads();  // every wave is done with the previous row's tables and reductions
    if (tid < 14 * 16) sm.pw[tid >> 4][sn] = direct;
    if (tid < 16) {
      sm.pn[tid] = rp.pv;
      sm.gn[tid] = rp.gv;
      sm.carry[0][0][tid] = cf{0.f, 0.f};
      sm.carry[0][1][tid] = cf{0.f, 0.f};
    }
    cur = 0;
    __syncthreads();
    {
      cf v = cmul(sm.pw[sa & 3][sn], sm.pw[4 + (sa >> 2)][sn]);
      q1 = sm.pw[8][sn];
      const cf c{rp.pv * rp.gv.x, rp.pv * rp.gv.y};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        qp[sn][4 * sa + e] = v;
        const float kl = group_sum<16>(c.x * v.x - c.y * v.y);
        if (sn == 0) sm.klocal[4 * sa + e] = (sa == 0 && e == 0) ? kl + rp.w : kl;  // omega on the diagonal
        v = cmul(v, q1);
      }
      if (sa == 15) qp[sn][kT] = sm.pw[9][sn];
      qT = sm.pw[9][sn];
    }
    __syncthreads();
    // 64 q^63
    qTd = cf{kT * qp[sn][kT - 1].x, kT * qp[sn][kT - 1].y};
    for (int item = tid; item < kBwdBlocks * kWave; item += kThreads) {
      const int blk = item >> 6, ln = item & 63, rr = ln & 31, gg = ln >> 5;
      float v[8];
      if (blk < 8) {
        const int kind = blk >> 2, s = blk & 3, n = rr >> 1, part = rr & 1;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int i = 16 * s + 8 * gg + e;
          const cf w = qp[n][kind ? (i > 0 ? i - 1 : 0) : i];
          const float sc = kind ? static_cast<float>(i) : 1.f;
          v[e] = sc * (part ? w.y : w.x);
        }
      } else if (blk < 12) {
        const int o = 16 * (blk - 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int lag = o - rr + 8 * gg + e;
          const float kv = sm.klocal[lag >= 0 ? lag : 0];  // read, then masked: no branch around the load
          v[e] = lag >= 0 ? kv : 0.f;
        }
      } else {
        const int jt = (blk - 12) >> 1, s2 = (blk - 12) & 1, j = 32 * jt + rr;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int m = 16 * s2 + 8 * gg + e, n = m >> 1;
          const cf c = cf{sm.pn[n] * sm.gn[n].x, sm.pn[n] * sm.gn[n].y};
          const cf w = cmul(c, qp[n][kT - j]);
          v[e] = (m & 1) ? -w.y : w.x;
        }
      }
      u32x4 hi, lo;
      split8(v, hi, lo);
      sm.aop[blk][0][ln] = hi;
      sm.aop[blk][1][ln] = lo;
    }
#pragma unroll
    for (int t = 0; t < 3; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) macc[t][i] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) wacc[i] = wdacc[i] = cf{0.f, 0.f};
    __syncthreads();
    rp = fetch_params(row + gridDim.x);
  };

  // the row's reductions and its five gradient outputs
  auto finish_row = [&](int64_t row) {
    MEGA_LANE_IDS;
    // W, W': over the 32 lanes (chunks) of a half wave, then over the waves.  A lane holds 32
    // partial sums (8 modes x (W, W') x (re, im)) and each half of the wave its own 8 modes: the
    // wave transposes them through its rows of the state buffer ([lane][value], pitch 33), and
    // lane (g, t) adds up value t of half g.
    wave_sync();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float* dst = myrows + lane * 33 + 4 * i;
      dst[0] = wacc[i].x;
      dst[1] = wacc[i].y;
      dst[2] = wdacc[i].x;
      dst[3] = wdacc[i].y;
    }
    wave_sync();
    {
      float part[32];
#pragma unroll
      for (int j = 0; j < 32; ++j) part[j] = myrows[(32 * g + j) * 33 + r];
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < 32; ++j) acc += part[j];
      sm.red[wave][g][r] = acc;
    }
    // dkin[l] = sum_j M[j + l][j]: each wave sums the diagonals of its own M, one 32 x 32 tile
    // at a time through its own rows of the state buffer ([i][j], pitch 33).  Lane (g, t) walks
    // the wrapped diagonal tile[(j + t) mod 32][j] over its 16 columns j = 16 g .. 16 g + 15:
    // the part with j + t < 32 belongs to the diagonal d = t, the rest to d = t - 32.  The tiles
    // (0,0) and (1,1) hold the same lags d >= 0 (their d < 0 is not asked for) and are added
    // first; the tile (1,0) holds lag 32 + d for both signs of d.
    {
      float lo[2], hi[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        wave_sync();
#pragma unroll
        for (int i = 0; i < 16; ++i)
          myrows[(8 * (i >> 2) + 4 * g + (i & 3)) * 33 + r] = t == 0 ? macc[0][i] + macc[2][i] : macc[1][i];
        wave_sync();
        float v[16];
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) {
          const int j = 16 * g + jj;
          v[jj] = myrows[((j + r) & 31) * 33 + j];
        }
        lo[t] = hi[t] = 0.f;
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) {
          const bool below = 16 * g + jj + r < 32;
          lo[t] += below ? v[jj] : 0.f;
          hi[t] += below ? 0.f : v[jj];
        }
      }
      // the two halves of the wave took different columns
      const float same = lo[0] + __shfl_xor(lo[0], 32, 64);
      const float cross_lo = lo[1] + __shfl_xor(lo[1], 32, 64);
      const float cross_hi = hi[1] + __shfl_xor(hi[1], 32, 64);
      // lag l <= 31: same[d = l] + cross[d = l - 32]; lag l >= 32: cross[d = l - 32]
      sm.dpart[wave][lane] = g == 0 ? same + cross_hi : cross_lo;
    }
    __syncthreads();  // every wave is done with the state buffer: it takes the power table again
    if (tid < kT) sm.dkin[tid] = (sm.dpart[0][tid] + sm.dpart[1][tid]) + (sm.dpart[2][tid] + sm.dpart[3][tid]);
    {
      cf v = cmul(sm.pw[sa & 3][sn], sm.pw[4 + (sa >> 2)][sn]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        qp[sn][4 * sa + e] = v;
        v = cmul(v, q1);
      }
    }
    __syncthreads();
    {
      // A_in = sum_l q^l dkin[l], B_in = sum_l l q^(l-1) dkin[l]: thread (n, a) takes l = 4 a .. 4 a + 3
      cf ain{0.f, 0.f}, bin{0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int l = 4 * sa + e;
        const float dk = sm.dkin[l];
        const cf v = qp[sn][l];
        ain.x = fmaf(dk, v.x, ain.x);
        ain.y = fmaf(dk, v.y, ain.y);
        if (l > 0) {
          const cf u = qp[sn][l - 1];
          const float dl = dk * static_cast<float>(l);
          bin.x = fmaf(dl, u.x, bin.x);
          bin.y = fmaf(dl, u.y, bin.y);
        }
      }
      ab[sa][0][sn] = ain;
      ab[sa][1][sn] = bin;
    }
    __syncthreads();
    if (tid < N) {
      const int n = tid;
      cf ain{0.f, 0.f}, bin{0.f, 0.f};
      for (int a = 0; a < 16; ++a) {
        ain = cadd(ain, ab[a][0][n]);
        bin = cadd(bin, ab[a][1][n]);
      }
      // mode n sits in half g = (n >> 1) & 1 at index 2 (n >> 2) + (n & 1)
      const int hg = (n >> 1) & 1, idx = 2 * (n >> 2) + (n & 1);
      cf w{0.f, 0.f}, wd{0.f, 0.f};
      for (int wv = 0; wv < kWaves; ++wv) {
        w.x += sm.red[wv][hg][4 * idx];
        w.y += sm.red[wv][hg][4 * idx + 1];
        wd.x += sm.red[wv][hg][4 * idx + 2];
        wd.y += sm.red[wv][hg][4 * idx + 3];
      }
      const cf qq = sm.pw[8][n];
      const cf A = cadd(ain, cmul(qq, w));
      const cf Bq = cadd(cadd(bin, w), cmul(qq, wd));
      const cf gm = sm.gn[n];
      const float pp = sm.pn[n];
      dp[row * N + n] = A.x * gm.x - A.y * gm.y;
      const cf t = cmul(Bq, cf{pp * gm.x, pp * gm.y});
      cf dqv{t.x, -t.y}, dgv{A.x * pp, -A.y * pp};
      if (h0 != nullptr) {
        // A carried state h0 adds b[t] = Re(gamma q^(t+1) h0) to the output (ema_parameters.cc:56-77).
        // With R0 = sum_t dy[t] q^t and R0' = dR0 / dq -- what the reverse scan has carried to the
        // start of the row -- its gradients are (ema_parameters.cc:158-188, PyTorch's convention)
        //   dgamma += conj(q h0 R0),  dq += conj(gamma h0 (R0 + q R0')),  dh0 = conj(gamma q R0).
        const cf r0 = sm.carry[cur][0][n], r0d = sm.carry[cur][1][n];
        const cf h = h0[row * N + n];
        const cf e1 = cmul(cmul(qq, h), r0);
        dgv.x += e1.x;
        dgv.y -= e1.y;
        const cf e2 = cmul(cmul(gm, h), cadd(r0, cmul(qq, r0d)));
        dqv.x += e2.x;
        dqv.y -= e2.y;
        if (dh0 != nullptr) {
          const cf e3 = cmul(cmul(gm, qq), r0);
          dh0[row * N + n] = cf{e3.x, -e3.y};
        }
      }
      dq[row * N + n] = dqv;
      dgamma[row * N + n] = dgv;
    }
    // the skip term sat on the diagonal of K, not in M: domega = sum dy x = dkin[0]
    if (tid == 0) domega[row] = sm.dkin[0];
  };

  auto item = [&](int64_t row, int64_t seg0) {
    MEGA_LANE_IDS;
    // transposing read of the parked tile: row tile tt (32 time steps), k-step ks (16 chunks)
    const int tr_base = (8 * g + ((lane & 15) >> 2)) * kSP + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    auto read_tr = [&](int tt, int ks) {
      const uint16_t* q = stage + tr_base + 16 * ks * kSP + 32 * tt;
      const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * kSP);
      return u32x4{lo.x, lo.y, hi.x, hi.y};
    };
    if (seg0 == seg_last) setup_row(row);
    using dx_t = typename std::conditional<DX32 != 0, float, uint16_t>::type;
    dx_t* dxrow = static_cast<dx_t*>(dx) + row * L;
    const int nc = static_cast<int>(C - seg0 < NC ? C - seg0 : NC);
    const int c0 = wave * 32;
    const bool on = c0 < nc;
    u32x4 xr[4];  // time-reversed x as an operand: steps 63 - (16 s + 8 g + e)
    // the next item of this workgroup: its x tile is requested as soon as this item's has been
    // consumed, its dy tile at the end of the item
    int64_t nrow = row, nseg = seg0 - NC;
    if (nseg < 0) {
      nrow = row + gridDim.x;
      nseg = seg_last;
    }
    if (on) {
      // ---- the wave's private tile: X parked first (it arrived an item ago), read back with
      //      chunks along k and time-reversed; then DY, whose loads were issued last ------------
      uint16_t* mine = stage + r * kSP + 8 * g;
#pragma unroll
      for (int s = 0; s < 4; ++s) *reinterpret_cast<u32x4*>(mine + 16 * s) = xb[s].pc[0];
      wave_sync();
      u32x4 xt[2][2];
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) xt[jt][ks] = read_tr(jt, ks);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(stage + r * kSP + 56 - 16 * s - 8 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) xr[s][e] = __builtin_amdgcn_alignbit(v[3 - e], v[3 - e], 16);
      }
      wave_sync();
#pragma unroll
      for (int s = 0; s < 4; ++s) *reinterpret_cast<u32x4*>(mine + 16 * s) = db[s].pc[0];
      wave_sync();
      // M += DY^T X over the tile's 32 chunks
#pragma unroll
      for (int it = 0; it < 2; ++it)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const u32x4 dyt = read_tr(it, ks);
          if (it == 0) macc[0] = mfma_bf16(dyt, xt[0][ks], macc[0]);
          if (it == 1) {
            macc[1] = mfma_bf16(dyt, xt[0][ks], macc[1]);
            macc[2] = mfma_bf16(dyt, xt[1][ks], macc[2]);
          }
        }
      wave_sync();  // the tile has been read: its place takes the wave's rows of (G, G')
    }
    load_x(nrow, nseg);
    if (on) {
      // ---- (G, G') = Pg DY, into this wave's own rows of the state buffer ----------------
#pragma unroll
      for (int kind = 0; kind < 2; ++kind) {
        floatx16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          u32x4 a[2];
          load_block(kind * 4 + s, a, lane);
          acc = mma_split<1>(a, db[s].pc, acc);
        }
        float* dst = myrows + r * kRP + 32 * kind + 4 * g;
#pragma unroll
        for (int qd = 0; qd < 4; ++qd)
          *reinterpret_cast<float4*>(dst + 8 * qd) =
              make_float4(acc[4 * qd], acc[4 * qd + 1], acc[4 * qd + 2], acc[4 * qd + 3]);
      }
    }
    wave_sync();
    load_dy(nrow, nseg);
    // ---- reverse scan over the chunks of the segment; a wave's four sub-segments are its own
    //      chunks, one workgroup barrier hands over the waves' ends ---------------------------------
    {
      float* col = sm.R + 2 * sn;
      float2 gv[CPS], gd[CPS];
#pragma unroll
      for (int i = 0; i < CPS; ++i) {
        const int c = sa * CPS + i;
        const bool live = c < nc;
        const float2 a0 = *reinterpret_cast<const float2*>(col + c * kRP);
        const float2 b0 = *reinterpret_cast<const float2*>(col + c * kRP + 32);
        gv[i] = live ? a0 : make_float2(0.f, 0.f);
        gd[i] = live ? b0 : make_float2(0.f, 0.f);
      }
      cf e{0.f, 0.f}, ed{0.f, 0.f};
#pragma unroll
      for (int i = CPS - 1; i >= 0; --i) rstep(e, ed, cf{gv[i].x, gv[i].y}, cf{gd[i].x, gd[i].y}, qT, qTd);
      sm.sub_end[sa][0][sn] = e;
      sm.sub_end[sa][1][sn] = ed;
      wave_sync();
      // multipliers over a sub-segment and over a wave's chunks
      const cf qS = sm.pw[10][sn], qW = sm.pw[12][sn];
      const cf qSd{(kT * CPS) * sm.pw[11][sn].x, (kT * CPS) * sm.pw[11][sn].y};
      const cf qWd{(4 * kT * CPS) * sm.pw[13][sn].x, (4 * kT * CPS) * sm.pw[13][sn].y};
      if (sl == 0) {
        // the wave's chunks from zero: sub-segments 3, 2, 1, then this one
        cf h = sm.sub_end[sa + 3][0][sn], hd = sm.sub_end[sa + 3][1][sn];
        rstep(h, hd, sm.sub_end[sa + 2][0][sn], sm.sub_end[sa + 2][1][sn], qS, qSd);
        rstep(h, hd, sm.sub_end[sa + 1][0][sn], sm.sub_end[sa + 1][1][sn], qS, qSd);
        rstep(h, hd, e, ed, qS, qSd);
        sm.wave_end[par][wave][0][sn] = h;
        sm.wave_end[par][wave][1][sn] = hd;
      }
      lds_barrier();
      cf h = sm.carry[cur][0][sn], hd = sm.carry[cur][1][sn];
#pragma unroll
      for (int w = kWaves - 1; w >= 1; --w) {
        const cf we = sm.wave_end[par][w][0][sn], wed = sm.wave_end[par][w][1][sn];
        if (w > wave) rstep(h, hd, we, wed, qW, qWd);
      }
      if (sa == 0) {
        // through wave 0's chunks too: the state at the start of the segment, the next item's carry
        cf ch = h, chd = hd;
        rstep(ch, chd, sm.wave_end[par][0][0][sn], sm.wave_end[par][0][1][sn], qW, qWd);
        sm.carry[cur ^ 1][0][sn] = ch;
        sm.carry[cur ^ 1][1][sn] = chd;
      }
      if (sl == 3) {  // (R, R') behind the wave's last chunk
        *reinterpret_cast<float2*>(sm.wave_cin[wave] + 2 * sn) = make_float2(h.x, h.y);
        *reinterpret_cast<float2*>(sm.wave_cin[wave] + 32 + 2 * sn) = make_float2(hd.x, hd.y);
      }
#pragma unroll
      for (int s = 3; s >= 1; --s) {
        const cf se = sm.sub_end[4 * wave + s][0][sn], sed = sm.sub_end[4 * wave + s][1][sn];
        if (s > sl) rstep(h, hd, se, sed, qS, qSd);
      }
#pragma unroll
      for (int i = CPS - 1; i >= 0; --i) {
        const int c = sa * CPS + i;
        rstep(h, hd, cf{gv[i].x, gv[i].y}, cf{gd[i].x, gd[i].y}, qT, qTd);
        if (c < nc) {
          *reinterpret_cast<float2*>(col + c * kRP) = make_float2(h.x, h.y);
          *reinterpret_cast<float2*>(col + c * kRP + 32) = make_float2(hd.x, hd.y);
        }
      }
    }
    wave_sync();
    if (on) {
      // (R, R')[c + 1]: the next row of the buffer, or, for the wave's last chunk, wave_cin;
      // chunks past the end of the row have X = 0 and DY = 0, their rows may hold anything
      const bool live = c0 + r < nc;
      const float* rnext = (r == 31) ? sm.wave_cin[wave] : myrows + (r + 1) * kRP;
      const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
      // the stores of dX go out first: they have the (X, X') products and the next item's
      // staging to retire under before the next loads are issued behind them
      // ---- DX = K^T DY + Qd R[c+1] (omega dy included: K carries omega on its diagonal) -------------
      u32x4 hb[2][2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const float* src = rnext + 16 * s2 + 8 * g;
        const float4 u0 = *reinterpret_cast<const float4*>(src);
        const float4 w0 = *reinterpret_cast<const float4*>(src + 4);
        const float4 u = live ? u0 : zero4;
        const float4 w = live ? w0 : zero4;
        const float v[8] = {u.x, u.y, u.z, u.w, w.x, w.y, w.z, w.w};
        split8(v, hb[s2][0], hb[s2][1]);
      }
      const int64_t chunk = seg0 + c0 + r;
#pragma unroll
      for (int jt = 0; jt < 2; ++jt) {
        floatx16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 2 * jt; s < 4; ++s) {
          u32x4 a[2];
          load_block(8 + s - 2 * jt, a, lane);
          acc = mma_split<1>(a, db[s].pc, acc);
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          u32x4 a[2];
          load_block(12 + 2 * jt + s2, a, lane);
          acc = mfma_bf16(a[0], hb[s2][0], acc);
          acc = mfma_bf16(a[1], hb[s2][0], acc);
          acc = mfma_bf16(a[0], hb[s2][1], acc);
        }
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
          if constexpr (DX32) {
            // registers 8 pr + 4 h + e hold the steps 16 pr + 8 h + 4 g + e
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const int64_t elem = chunk * kT + 16 * (2 * jt + pr) + 8 * h + 4 * g;
              if (dx != nullptr && elem + 4 <= L) {
                float4 v = make_float4(acc[8 * pr + 4 * h], acc[8 * pr + 4 * h + 1], acc[8 * pr + 4 * h + 2],
                                       acc[8 * pr + 4 * h + 3]);
                if constexpr (DX32 == 2) {
                  const float4 o = *reinterpret_cast<const float4*>(dxrow + elem);
                  v = make_float4(v.x + o.x, v.y + o.y, v.z + o.z, v.w + o.w);
                }
                *reinterpret_cast<float4*>(dxrow + elem) = v;
              }
            }
          } else {
            const uint4 oct = octet_of<DT>(acc, pr);
            const int64_t elem = chunk * kT + 16 * (2 * jt + pr) + 8 * g;
            if (elem + 8 <= L) *reinterpret_cast<uint4*>(dxrow + elem) = oct;
          }
        }
      }
      // ---- (X, X') = Pg XR;  W += X R[c+1], W' += X' R[c+1] + X R'[c+1] ---------------------------
      {
        floatx16 xacc[2];
#pragma unroll
        for (int kind = 0; kind < 2; ++kind) {
#pragma unroll
          for (int i = 0; i < 16; ++i) xacc[kind][i] = 0.f;
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            u32x4 a[2];
            load_block(kind * 4 + s, a, lane);
            xacc[kind] = mma_split<1>(a, &xr[s], xacc[kind]);
          }
        }
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          // loaded whatever the row holds, then masked: a conditional load is split into
          // single-word reads under an execution mask
          const float4 rv0 = *reinterpret_cast<const float4*>(rnext + 4 * g + 8 * qd);
          const float4 rd0 = *reinterpret_cast<const float4*>(rnext + 32 + 4 * g + 8 * qd);
          const float4 rv = live ? rv0 : zero4;
          const float4 rd = live ? rd0 : zero4;
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            const cf xv{xacc[0][4 * qd + 2 * b], xacc[0][4 * qd + 2 * b + 1]};
            const cf xd{xacc[1][4 * qd + 2 * b], xacc[1][4 * qd + 2 * b + 1]};
            const cf rr_ = b ? cf{rv.z, rv.w} : cf{rv.x, rv.y};
            const cf rdd = b ? cf{rd.z, rd.w} : cf{rd.x, rd.y};
            wacc[2 * qd + b] = cadd(wacc[2 * qd + b], cmul(xv, rr_));
            wdacc[2 * qd + b] = cadd(wdacc[2 * qd + b], cadd(cmul(xd, rr_), cmul(xv, rdd)));
          }
        }
      }
    }
    cur ^= 1;
    par ^= 1;
    if (seg0 == 0) finish_row(row);
#pragma unroll
    for (int s = 0; s < 4; ++s) db[s] = dn[s];
  };

  load_x(blockIdx.x, seg_last);
  load_dy(blockIdx.x, seg_last);
#pragma unroll
  for (int s = 0; s < 4; ++s) db[s] = dn[s];
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x)
    for (int64_t seg0 = seg_last; seg0 >= 0; seg0 -= NC) item(row, seg0);
#undef MEGA_LANE_IDS
}

template <int DX32>
int launch_bwd(const void* dy, const void* x, void* dx, const float* p, const cf* log_q,
               const cf* gamma, const float* omega, const cf* h0, float* dp, cf* dq, cf* dgamma, float* domega,
               cf* dh0, int64_t B, int64_t D, int64_t N, int64_t L, hipStream_t stream) {
  const int lds = static_cast<int>(sizeof(BwdSmem));
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&cema_scan_bwd_kernel<MEGA_BF16, DX32>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  const int64_t rows = B * D, slots = 2 * static_cast<int64_t>(cus);  // two workgroups fit a compute unit
  const unsigned grid = static_cast<unsigned>(rows < slots ? rows : slots);
  cema_scan_bwd_kernel<MEGA_BF16, DX32><<<dim3(grid), kThreads, lds, stream>>>(
      dy, x, dx, p, log_q, gamma, omega, h0, dp, dq, dgamma, domega, dh0, rows, static_cast<int>(D),
      static_cast<int>(N), L);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_cema_scan_supported(int dtype, int64_t N, int64_t L) {
  return valid_dtype(dtype) && N >= 1 && N <= 16 && L >= 8 && L % 8 == 0;
}

extern "C" int mega_cema_scan_fwd(const void* x, int dtype, const float* p, const float* log_q,
                                  const float* gamma, const float* omega, const float* h0,
                                  int64_t B, int64_t D, int64_t N, int64_t L, void* y, float* h_last,
                                  void* stream) {
  const char* who = "mega_cema_scan_fwd";
  MEGA_CHECK_ARG(x && p && log_q && gamma && y, "%s: null pointer", who);
  MEGA_CHECK_ARG(B >= 0 && D >= 0 && L >= 0, "%s: negative size", who);
  MEGA_CHECK_ARG(B * D <= 0x7fffffff, "%s: too many rows", who);
  if (!mega_cema_scan_supported(dtype, N, L))
    return set_error(MEGA_ERR_UNSUPPORTED,
                     "%s: needs N <= 16 and L a multiple of 8 (dtype %d, N %lld, L %lld)",
                     who, dtype, (long long)N, (long long)L);
  MEGA_CHECK_ARG(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0,
                 "%s: x and y must be 16-byte aligned", who);
  if (B == 0 || D == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const cf* lq = reinterpret_cast<const cf*>(log_q);
  const cf* gm = reinterpret_cast<const cf*>(gamma);
  const cf* h0c = reinterpret_cast<const cf*>(h0);
  cf* hl = reinterpret_cast<cf*>(h_last);
  // one chunk tile per wave (segments of 128 chunks) measured 5 % faster than two for bfloat16 rows as well
  if (dtype == MEGA_BF16) return launch_fwd<MEGA_BF16, 1>(x, y, p, lq, gm, omega, h0c, hl, B, D, N, L, s);
  if (dtype == MEGA_F32) return launch_fwd<MEGA_F32, 1>(x, y, p, lq, gm, omega, h0c, hl, B, D, N, L, s);
  return launch_fwd<MEGA_F16, 1>(x, y, p, lq, gm, omega, h0c, hl, B, D, N, L, s);
}

extern "C" int mega_cema_scan_bwd_supported(int dtype, int64_t N, int64_t L) {
  return dtype == MEGA_BF16 && N >= 1 && N <= 16 && L >= 8 && L % 8 == 0;
}

extern "C" int mega_cema_scan_bwd_state(const void* dy, const void* x, int dtype, const float* p,
                                        const float* log_q, const float* gamma, const float* omega,
                                        const float* h0, int64_t B, int64_t D, int64_t N, int64_t L, void* dx,
                                        float* dp, float* dq, float* dgamma, float* domega, float* dh0,
                                        void* stream) {
  const char* who = "mega_cema_scan_bwd";
  MEGA_CHECK_ARG(dy && x && p && log_q && gamma && dx && dp && dq && dgamma && domega, "%s: null pointer", who);
  MEGA_CHECK_ARG(B >= 0 && D >= 0 && L >= 0, "%s: negative size", who);
  MEGA_CHECK_ARG(B * D <= 0x7fffffff, "%s: too many rows", who);
  if (!mega_cema_scan_bwd_supported(dtype, N, L))
    return set_error(MEGA_ERR_UNSUPPORTED,
                     "%s: needs bfloat16 rows, N <= 16 and L a multiple of 8 (dtype %d, N %lld, L %lld)", who,
                     dtype, (long long)N, (long long)L);
  const auto al = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  MEGA_CHECK_ARG(al(dy) && al(x) && al(dx), "%s: dy, x and dx must be 16-byte aligned", who);
  if (B == 0 || D == 0) return MEGA_OK;
  MEGA_CHECK_ARG(dh0 == nullptr || h0 != nullptr, "%s: dh0 without h0", who);
  return launch_bwd<0>(dy, x, dx, p, reinterpret_cast<const cf*>(log_q), reinterpret_cast<const cf*>(gamma),
                           omega, reinterpret_cast<const cf*>(h0), dp, reinterpret_cast<cf*>(dq),
                           reinterpret_cast<cf*>(dgamma), domega, reinterpret_cast<cf*>(dh0), B, D, N, L,
                           static_cast<hipStream_t>(stream));
}

extern "C" int mega_cema_scan_bwd(const void* dy, const void* x, int dtype, const float* p,
                                  const float* log_q, const float* gamma, const float* omega,
                                  int64_t B, int64_t D, int64_t N, int64_t L, void* dx, float* dp,
                                  float* dq, float* dgamma, float* domega, void* stream) {
  return mega_cema_scan_bwd_state(dy, x, dtype, p, log_q, gamma, omega, nullptr, B, D, N, L, dx, dp, dq, dgamma,
                                  domega, nullptr, stream);
}

extern "C" int mega_cema_scan_bwd_wide(const void* dy, const void* x, const float* p, const float* log_q,
                                       const float* gamma, const float* omega, const float* h0, int64_t B,
                                       int64_t D, int64_t N, int64_t L, float* dx, int accumulate_dx, float* dp,
                                       float* dq, float* dgamma, float* domega, float* dh0, void* stream) {
  const char* who = "mega_cema_scan_bwd_wide";
  MEGA_CHECK_ARG(dy && x && p && log_q && gamma && dp && dq && dgamma && domega, "%s: null pointer", who);
  MEGA_CHECK_ARG(B >= 0 && D >= 0 && L >= 0, "%s: negative size", who);
  MEGA_CHECK_ARG(B * D <= 0x7fffffff, "%s: too many rows", who);
  if (!mega_cema_scan_bwd_supported(MEGA_BF16, N, L))
    return set_error(MEGA_ERR_UNSUPPORTED, "%s: needs N <= 16 and L a multiple of 8 (N %lld, L %lld)", who,
                     (long long)N, (long long)L);
  const auto al = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  MEGA_CHECK_ARG(al(dy) && al(x) && al(dx), "%s: dy, x and dx must be 16-byte aligned", who);
  if (B == 0 || D == 0) return MEGA_OK;
  MEGA_CHECK_ARG(dh0 == nullptr || h0 != nullptr, "%s: dh0 without h0", who);
  if (accumulate_dx && dx != nullptr)
    return launch_bwd<2>(dy, x, dx, p, reinterpret_cast<const cf*>(log_q), reinterpret_cast<const cf*>(gamma),
                         omega, reinterpret_cast<const cf*>(h0), dp, reinterpret_cast<cf*>(dq),
                         reinterpret_cast<cf*>(dgamma), domega, reinterpret_cast<cf*>(dh0), B, D, N, L,
                         static_cast<hipStream_t>(stream));
  return launch_bwd<1>(dy, x, dx, p, reinterpret_cast<const cf*>(log_q), reinterpret_cast<const cf*>(gamma),
                       omega, reinterpret_cast<const cf*>(h0), dp, reinterpret_cast<cf*>(dq),
                       reinterpret_cast<cf*>(dgamma), domega, reinterpret_cast<cf*>(dh0), B, D, N, L,
                       static_cast<hipStream_t>(stream));
}
