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
// One workgroup of four waves owns a row; a segment of 256 chunks (16384
// steps) is resident at a time: wave w holds chunk tiles 2 w, 2 w + 1 of it.
#include "common.hpp"
#include "cema_pow.hpp"

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
// returned the first result for both outputs here.  The s_nop covers the wait
// states the instruction needs after a vector write of its operands.
__device__ __forceinline__ void half_swap(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
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
  cf qp[16][kT + 2];                           // q_n^e, e = 0 .. 64
  float klocal[kT];                            // k[0 .. 63]
  float pn[16];
  cf gn[16];
  cf sub_end[kSubs][16];
  cf carry[2][16];
  u32x4 aop[kFwdBlocks][2][kWave];
  float H[(NC + 1) * kHP];                     // row 0: state before the segment, row 1 + c: after chunk c
};

template <int DT, int NT>
__global__ __launch_bounds__(kThreads) void cema_scan_fwd_kernel(
    const void* __restrict__ x, void* __restrict__ y, const float* __restrict__ p,
    const cf* __restrict__ log_q, const cf* __restrict__ gamma, const float* __restrict__ omega,
    const cf* __restrict__ h0, cf* __restrict__ h_last, int D, int N, int64_t L) {
  using Smem = FwdSmem<NT>;
  constexpr int NC = Smem::NC, CPS = NC / kSubs, XP = XOp<DT>::XP;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int g = lane >> 5, r = lane & 31;
  const int64_t row = blockIdx.x;
  const int d = static_cast<int>(row % D);
  const uint16_t* xrow = static_cast<const uint16_t*>(x) + row * L;
  uint16_t* yrow = static_cast<uint16_t*>(y) + row * L;
  const float wres = omega != nullptr ? omega[d] : 0.f;
  const int64_t C = (L + kT - 1) / kT;

  // the first segment's rows are requested before the tables are built
  XOp<DT> xb[NT][4];
  auto load_tiles = [&](int64_t seg0) {
#pragma unroll
    for (int ctl = 0; ctl < NT; ++ctl) {
      const int64_t chunk = seg0 + (wave * NT + ctl) * 32 + r;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int64_t elem = chunk * kT + 16 * s + 8 * g;
        xb[ctl][s].load(xrow, elem, elem + 8 <= L);
      }
    }
  };
  load_tiles(0);

  // ---- per-row tables ---------------------------------------------------------
  const int sn = tid & 15, sa = tid >> 4;  // mode, and: power group here, sub-segment in the scan
  {
    cf v{0.f, 0.f}, q1{0.f, 0.f};
    if (sn < N) {
      const cf lq = log_q[d * N + sn];
      v = qpow(lq.x, lq.y, 4 * sa);
      q1 = qpow(lq.x, lq.y, 1);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      sm.qp[sn][4 * sa + e] = v;
      v = cmul(v, q1);
    }
    if (sa == 15) sm.qp[sn][kT] = v;
    if (tid < 16) {
      sm.pn[tid] = tid < N ? p[d * N + tid] : 0.f;
      sm.gn[tid] = tid < N ? gamma[d * N + tid] : cf{0.f, 0.f};
      sm.carry[0][tid] = (h0 != nullptr && tid < N) ? h0[row * N + tid] : cf{0.f, 0.f};
    }
  }
  // q^64 and q^(64 CPS) for the scan
  cf qT{0.f, 0.f}, qS{0.f, 0.f};
  if (sn < N) {
    const cf lq = log_q[d * N + sn];
    qT = qpow(lq.x, lq.y, kT);
    qS = qpow(lq.x, lq.y, kT * CPS);
  }
  __syncthreads();
  if (tid < kT) {
    float acc = 0.f;
#pragma unroll
    for (int n = 0; n < 16; ++n) {
      const cf c = cmul(cf{sm.pn[n] * sm.gn[n].x, sm.pn[n] * sm.gn[n].y}, sm.qp[n][tid]);
      acc += c.x;
    }
    sm.klocal[tid] = acc;
  }
  __syncthreads();
  for (int item = tid; item < kFwdBlocks * kWave; item += kThreads) {
    const int blk = item >> 6, ln = item & 63, rr = ln & 31, gg = ln >> 5;
    float v[8];
    if (blk < 4) {
      const int n = rr >> 1, part = rr & 1;
      const float pp = sm.pn[n];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const cf w = sm.qp[n][kT - 1 - (16 * blk + 8 * gg + e)];
        v[e] = pp * (part ? w.y : w.x);
      }
    } else if (blk < 8) {
      const int o = 16 * (blk - 5);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int lag = o + rr - 8 * gg - e;
        v[e] = lag >= 0 ? sm.klocal[lag] : 0.f;
      }
    } else {
      const int it = (blk - 8) >> 1, s2 = (blk - 8) & 1, i = 32 * it + rr;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int m = 16 * s2 + 8 * gg + e, n = m >> 1;
        const cf w = cmul(sm.gn[n], sm.qp[n][i + 1]);
        v[e] = (m & 1) ? -w.y : w.x;
      }
    }
    u32x4 hi, lo;
    split8(v, hi, lo);
    sm.aop[blk][0][ln] = hi;
    sm.aop[blk][1][ln] = lo;
  }
  __syncthreads();
  u32x4 A[kFwdBlocks][2];
#pragma unroll
  for (int b = 0; b < kFwdBlocks; ++b) {
    A[b][0] = sm.aop[b][0][lane];
    A[b][1] = sm.aop[b][1][lane];
  }

  int cur = 0;
  for (int64_t seg0 = 0; seg0 < C; seg0 += NC) {
    const int nc = static_cast<int>(C - seg0 < NC ? C - seg0 : NC);
    // ---- local states S = P X ---------------------------------------------------
#pragma unroll
    for (int ctl = 0; ctl < NT; ++ctl) {
      const int c0 = (wave * NT + ctl) * 32;
      if (c0 < nc) {
        floatx16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < 4; ++s) acc = mma_split<XP>(A[s], xb[ctl][s].pc, acc);
        float* dst = sm.H + (1 + c0 + r) * kHP + 4 * g;
#pragma unroll
        for (int qd = 0; qd < 4; ++qd)
          *reinterpret_cast<float4*>(dst + 8 * qd) =
              make_float4(acc[4 * qd], acc[4 * qd + 1], acc[4 * qd + 2], acc[4 * qd + 3]);
      }
    }
    lds_barrier();
    // ---- scan over the chunks of the segment --------------------------------------
    {
      float* col = sm.H + kHP + 2 * sn;  // state column n of row 1 + c
      cf h{0.f, 0.f};
#pragma unroll 4
      for (int i = 0; i < CPS; ++i) {
        const int c = sa * CPS + i;
        if (c < nc) {
          const float2 s = *reinterpret_cast<const float2*>(col + c * kHP);
          h = cadd(cmul(qT, h), cf{s.x, s.y});
        }
      }
      sm.sub_end[sa][sn] = h;
      lds_barrier();
      cf cin = sm.carry[cur][sn];
      for (int s = 0; s < sa; ++s) cin = cadd(cmul(qS, cin), sm.sub_end[s][sn]);
      if (sa == 0) *reinterpret_cast<float2*>(sm.H + 2 * sn) = make_float2(cin.x, cin.y);
      h = cin;
#pragma unroll 4
      for (int i = 0; i < CPS; ++i) {
        const int c = sa * CPS + i;
        if (c < nc) {
          const float2 s = *reinterpret_cast<const float2*>(col + c * kHP);
          h = cadd(cmul(qT, h), cf{s.x, s.y});
          *reinterpret_cast<float2*>(col + c * kHP) = make_float2(h.x, h.y);
        }
      }
      if (sa == kSubs - 1) sm.carry[cur ^ 1][sn] = h;
    }
    lds_barrier();
    // ---- Y = K X + Q H[c-1] (+ omega x), written from the accumulators ---------------
#pragma unroll
    for (int ctl = 0; ctl < NT; ++ctl) {
      const int c0 = (wave * NT + ctl) * 32;
      if (c0 < nc) {
        u32x4 hb[2][2];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const float* src = sm.H + (c0 + r) * kHP + 16 * s2 + 8 * g;
          const float4 u = *reinterpret_cast<const float4*>(src);
          const float4 w = *reinterpret_cast<const float4*>(src + 4);
          const float v[8] = {u.x, u.y, u.z, u.w, w.x, w.y, w.z, w.w};
          split8(v, hb[s2][0], hb[s2][1]);
        }
        const int64_t chunk = seg0 + c0 + r;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
          floatx16 acc;
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
          for (int s = 0; s < 2 + 2 * it; ++s) acc = mma_split<XP>(A[5 + 2 * it - s], xb[ctl][s].pc, acc);
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            acc = mfma_bf16(A[8 + 2 * it + s2][0], hb[s2][0], acc);
            acc = mfma_bf16(A[8 + 2 * it + s2][1], hb[s2][0], acc);
            acc = mfma_bf16(A[8 + 2 * it + s2][0], hb[s2][1], acc);
          }
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            float oct[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              oct[e] = acc[8 * pr + e];
              oct[4 + e] = acc[8 * pr + 4 + e];
              half_swap(oct[e], oct[4 + e]);
            }
            const int s = 2 * it + pr;
            float xv[8];
            xb[ctl][s].values(xv);
#pragma unroll
            for (int e = 0; e < 8; ++e) oct[e] = fmaf(wres, xv[e], oct[e]);
            const int64_t elem = chunk * kT + 16 * s + 8 * g;
            if (elem + 8 <= L) *reinterpret_cast<uint4*>(yrow + elem) = pack8<DT>(oct);
          }
        }
      }
    }
    cur ^= 1;
    if (seg0 + NC < C) {
      load_tiles(seg0 + NC);
      lds_barrier();  // the next segment's local states overwrite the rows read above
    }
  }

  if (h_last != nullptr) {
    __syncthreads();
    if (tid < N) {
      // state after step L - 1: the last chunk may be partial
      const int64_t seg_last = (C - 1) / NC * NC;
      const int rem = static_cast<int>(L - (C - 1) * kT);  // 1 .. 64 steps in the last chunk
      // row C - 1 - seg_last of the state buffer is H[C-2], the next one H[C-1]
      const float* prev = sm.H + static_cast<int>(C - 1 - seg_last) * kHP + 2 * tid;
      cf h;
      if (rem == kT) {
        h = cf{prev[kHP], prev[kHP + 1]};
      } else {
        h = cmul(sm.qp[tid][rem], cf{prev[0], prev[1]});
        const float pp = sm.pn[tid];
        for (int j = 0; j < rem; ++j) {
          const float xv = Elem<DT>::load(xrow + (C - 1) * kT + j) * pp;
          const cf w = sm.qp[tid][rem - 1 - j];
          h.x = fmaf(xv, w.x, h.x);
          h.y = fmaf(xv, w.y, h.y);
        }
      }
      h_last[row * N + tid] = h;
    }
  }
}

template <int DT, int NT>
int launch_fwd(const void* x, void* y, const float* p, const cf* log_q, const cf* gamma,
               const float* omega, const cf* h0, cf* h_last, int64_t B, int64_t D, int64_t N,
               int64_t L, hipStream_t stream) {
  const size_t lds = sizeof(FwdSmem<NT>);
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&cema_scan_fwd_kernel<DT, NT>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
  cema_scan_fwd_kernel<DT, NT><<<dim3(static_cast<unsigned>(B * D)), kThreads, lds, stream>>>(
      x, y, p, log_q, gamma, omega, h0, h_last, static_cast<int>(D), static_cast<int>(N), L);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_cema_scan_supported(int dtype, int64_t N, int64_t L) {
  return (dtype == MEGA_BF16 || dtype == MEGA_F16) && N >= 1 && N <= 16 && L >= 8 && L % 8 == 0;
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
                     "%s: needs bfloat16 / float16 rows, N <= 16 and L a multiple of 8 (dtype %d, N %lld, L %lld)",
                     who, dtype, (long long)N, (long long)L);
  MEGA_CHECK_ARG(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0,
                 "%s: x and y must be 16-byte aligned", who);
  if (B == 0 || D == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const cf* lq = reinterpret_cast<const cf*>(log_q);
  const cf* gm = reinterpret_cast<const cf*>(gamma);
  const cf* h0c = reinterpret_cast<const cf*>(h0);
  cf* hl = reinterpret_cast<cf*>(h_last);
  if (dtype == MEGA_BF16) return launch_fwd<MEGA_BF16, 2>(x, y, p, lq, gm, omega, h0c, hl, B, D, N, L, s);
  return launch_fwd<MEGA_F16, 1>(x, y, p, lq, gm, omega, h0c, hl, B, D, N, L, s);
}
