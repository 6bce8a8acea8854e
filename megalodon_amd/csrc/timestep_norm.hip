// Group TimestepNorm for gfx950: cumulative (over time) group mean / variance
// normalisation, forward and backward, one pass over the activations.
//
// Math follows megalodon/csrc/ops/timestep_norm.cc:218-316 (forward) and
// :318-450 (backward), merge operator megalodon/csrc/utils.h:154-164; masked
// steps behave as in the reference's CUDA kernels (state unchanged, y = dx = 0,
// stored statistics are those of the unchanged state,
// timestep_norm_kernel.cu:621-626).
//
// Design.  The reference scans time in B*ceil(G/32) blocks and reads x two to
// three times.  Here the (batch, group) chains are cut into tiles of 64
// timesteps; a workgroup loads one tile (64 rows x D/G features) into
// registers, reduces every row to its moments, scans the 64 rows inside one
// wavefront (lane = timestep) and obtains the carry of all earlier tiles by a
// decoupled look-back over per-tile records in device memory (aggregate /
// inclusive-prefix words published with relaxed device-scope atomics, two
// floats per 64-bit word, all ones meaning "not written yet").  Groups of at
// most 16 lanes per row (128 bf16 features) give every wavefront a tile of its
// own in the forward pass, with no workgroup barrier after the ticket.
// The tile is then normalised from registers:
// x is read once and y written once.  The backward pass runs the same scheme
// in reverse time with 2x2 upper-triangular affine maps as the carried
// quantity (the reverse recurrence on (dmean, dvar) is affine in the state).
// A workgroup's chain is fixed by its index; the tile of that chain it works on
// comes from the chain's own ticket counter, so tiles of a chain start in time
// order and every tile a workgroup waits for is already resident or finished.
// (One counter for all chains would do too, but atomics on one address from
// different workgroups retire at ~11 ns each on this part: 16384 tiles would
// cost 190 us in tickets alone.)
#include "common.hpp"

#include <atomic>
#include <mutex>

#include <algorithm>

namespace mega {
namespace {

constexpr int kTL = 64;        // timesteps per tile = lanes per wavefront
constexpr int kThreads = 256;  // 4 wavefronts
constexpr int kWaves = kThreads / kWave;
constexpr int kTicketStride = 16;  // ints between ticket counters: one 64-byte line each
constexpr int kStatusSlot = 1;     // the status word lives in the unused part of the first ticket's line

struct TsnParams {
  const void* x;
  const void* dy;          // backward only
  const void* gamma;
  const void* beta;        // forward only
  const uint8_t* mask;     // (B, L) or null; 1 = padding
  const int64_t* prev_count;  // forward: (B); backward: final count (B)
  const void* prev_mean;
  const void* prev_var;    // forward only
  const void* dmean;       // backward only
  const void* dvar;
  const float* cummean_in;  // backward
  const float* cumrstd_in;
  void* y;                 // forward y / backward dx
  int64_t* count;
  void* mean;              // forward mean / backward dprev_mean
  void* var;               // forward var / backward dprev_var
  float* cummean;
  float* cumrstd;
  float* part_g;           // backward partial sums (B*NT, D)
  float* part_b;
  int* ticket;             // one counter per chain, kTicketStride ints apart (the per-wave forward kernel uses the first)
  const int* nbefore;      // (B, NT+1) unmasked steps before tile j
  unsigned long long* rec; // per (chain, tile) records
  unsigned int* status;    // one word: bit 0 = a look-back wait ran into spin_limit
  long long spin_limit;    // polls of one record before a wait is given up
  int mute_tile;           // test hook: this tile index publishes nothing (-1: none)
  int B, L, D, G, Dg, NT;
  // element strides of cummean / cumrstd: (B, L, G) as the reference stores them, or (B, G, L)
  int64_t st_b, st_t, st_g;
  float eps;
};

__device__ __forceinline__ int64_t stat_index(const TsnParams& p, int b, int64_t t, int g) {
  return b * p.st_b + t * p.st_t + g * p.st_g;
}

// A wait for another tile's record is bounded: tiles of a chain start in time
// order, so in a healthy launch the record arrives within the predecessor's own
// run time.  A wave that has polled spin_limit times sets bit 0 of the status
// word, takes NaN as the missing value (every output that depends on it shows
// it) and goes on, so the grid always drains;
// mega_group_timestep_norm_status reports the word to the host.
constexpr long long kDefaultSpinLimit = 1ll << 22;  // >= 2 s of polling on this part
constexpr unsigned int kStatusGaveUp = 1u;
__device__ __forceinline__ void give_up(const TsnParams& p) {
  __hip_atomic_fetch_or(p.status, kStatusGaveUp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- 64-bit record words: two floats published together -------------------------
// A word that nobody has written yet holds kEmpty (all ones).  A published word
// never does: a float whose bits are all ones (one of the NaN encodings) is
// stored as the default NaN instead.
constexpr unsigned long long kEmpty = ~0ull;
constexpr int kWin = 32;  // records polled per look-back round (lanes 0 .. kWin-1)
__device__ __forceinline__ uint32_t word_bits(float v) {
  const uint32_t b = __float_as_uint(v);
  return b == 0xffffffffu ? 0x7fc00000u : b;
}
__device__ __forceinline__ void put_pair(unsigned long long* p, float lo, float hi) {
  const unsigned long long w = (static_cast<unsigned long long>(word_bits(hi)) << 32) | word_bits(lo);
  __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool get_pair(const unsigned long long* p, float& lo, float& hi) {
  const unsigned long long w =
      __hip_atomic_load(const_cast<unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  lo = __uint_as_float(static_cast<uint32_t>(w));
  hi = __uint_as_float(static_cast<uint32_t>(w >> 32));
  return w != kEmpty;
}

// ---- Welford triple ----------------------------------------------------------
struct Wel {
  float n, u, v;
};
// Two empty operands (a prior of count zero and masked steps, or the identity)
// keep the prior's mean and variance: at most one of them is not all zeros.
__device__ __forceinline__ Wel wel_merge(Wel a, Wel b) {  // utils.h:154-164
  const float n = a.n + b.n;
  const float inv = n > 0.f ? 1.f / n : 0.f;
  const float c1 = a.n * inv, c2 = b.n * inv;
  const float d = b.u - a.u;
  const float u = c1 * a.u + c2 * b.u, v = c1 * a.v + c2 * b.v + (c1 * d) * (c2 * d);
  return Wel{n, n > 0.f ? u : a.u + b.u, n > 0.f ? v : a.v + b.v};
}
__device__ __forceinline__ Wel wel_shfl_up(Wel a, int d) {
  return Wel{__shfl_up(a.n, d, 64), __shfl_up(a.u, d, 64), __shfl_up(a.v, d, 64)};
}
__device__ __forceinline__ Wel wel_shfl_xor(Wel a, int d) {
  return Wel{__shfl_xor(a.n, d, 64), __shfl_xor(a.u, d, 64), __shfl_xor(a.v, d, 64)};
}

// ---- affine map on the carried gradient (ug, vg) -----------------------------
//   ug' = a ug + e vg + bu,   vg' = a vg + bv
struct Aff {
  float a, e, bu, bv;
};
// apply x first (later time), then y (earlier time)
__device__ __forceinline__ Aff aff_compose(Aff y, Aff x) {
  return Aff{y.a * x.a, y.a * x.e + y.e * x.a, y.a * x.bu + y.e * x.bv + y.bu, y.a * x.bv + y.bv};
}
__device__ __forceinline__ Aff aff_shfl_down(Aff m, int d) {
  return Aff{__shfl_down(m.a, d, 64), __shfl_down(m.e, d, 64), __shfl_down(m.bu, d, 64),
             __shfl_down(m.bv, d, 64)};
}
__device__ __forceinline__ Aff aff_shfl_up(Aff m, int d) {
  return Aff{__shfl_up(m.a, d, 64), __shfl_up(m.e, d, 64), __shfl_up(m.bu, d, 64),
             __shfl_up(m.bv, d, 64)};
}

// ---- element vectors (16 bytes) -----------------------------------------------
template <int DT> struct Vec;
template <> struct Vec<MEGA_F32> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(const uint4& r, float* f) {
    f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y);
    f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                      __float_as_uint(f[3]));
  }
};
template <> struct Vec<MEGA_BF16> {
  static constexpr int N = 8;
  // sum and sum of squares of the 8 elements, products exact, fp32 accumulation
  // (v_dot2c_f32_bf16: no unpacking)
  static __device__ __forceinline__ void moments(const uint4& r, float& s1, float& s2) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 one = __builtin_bit_cast(bf16x2, 0x3f803f80u);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
    s1 = s2 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bf16x2 v = __builtin_bit_cast(bf16x2, w[i]);
      s1 = __builtin_amdgcn_fdot2_f32_bf16(v, one, s1, false);
      s2 = __builtin_amdgcn_fdot2_f32_bf16(v, v, s2, false);
    }
  }
  static __device__ __forceinline__ void unpack(const uint4& r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    return make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                      pack_bf16x2(f[6], f[7]));
  }
};
template <> struct Vec<MEGA_F16> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(const uint4& r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = f16_bits_to_float(static_cast<uint16_t>(w[i] & 0xffffu));
      f[2 * i + 1] = f16_bits_to_float(static_cast<uint16_t>(w[i] >> 16));
    }
  }
  static __device__ __forceinline__ uint4 pack(const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = static_cast<uint32_t>(float_to_f16_bits(f[2 * i])) |
             (static_cast<uint32_t>(float_to_f16_bits(f[2 * i + 1])) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
  }
};

template <int DT>
__device__ __forceinline__ float ldT(const void* p, int64_t i) {
  return Elem<DT>::load(static_cast<const typename Elem<DT>::type*>(p) + i);
}
template <int DT>
__device__ __forceinline__ void stT(void* p, int64_t i, float v) {
  Elem<DT>::store(static_cast<typename Elem<DT>::type*>(p) + i, v);
}

// Streamed accesses (store_streaming / load_once).  y (dx) is written once, in whole 128-byte lines, and read by another
// kernel much later: stored with the non-temporal hint it does not displace what the kernel
// still reads (config 2, forward 0.129 -> 0.104 ms, backward 0.193 -> 0.185 ms).  dy in the
// backward is read once: loaded with the hint, 0.185 -> 0.175 ms.  x is left alone (with the
// hint on its loads the forward is 0.114 ms, the backward 0.179 ms), and so are the statistics:
// they leave four bytes per lane, and partial lines written with the hint are slow (forward
// 0.167 ms).

// Hides a loaded vector from common-subexpression elimination: the unpacked
// floats of an earlier phase are recomputed instead of being kept in registers.
__device__ __forceinline__ uint4 reload(uint4 v) {
  asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
  return v;
}

template <int LPR>
__device__ __forceinline__ float row_sum(float v) {  // sum over the LPR lanes of a row
  if (LPR <= 16) return group_sum<LPR>(v);  // inside one 16-lane DPP row
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---- preparation: clear ticket / records, count unmasked steps per tile --------
__global__ void tsn_prep_kernel(int* ticket, int n_tickets, unsigned long long* rec, int64_t rec_words,
                                const uint8_t* mask, int* nbefore, int B, int L, int NT) {
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = gid; i < rec_words; i += stride) rec[i] = kEmpty;
  for (int64_t i = gid; i < n_tickets; i += stride) ticket[i * kTicketStride] = 0;
  if (gid == 0) ticket[kStatusSlot] = 0;  // the status word of this launch
  // block b (< B) also builds nbefore[b][0..NT]: thread i counts the unmasked
  // steps of tiles i per .. i per + per - 1, a block-wide exclusive scan turns
  // the counts into starting values
  if (blockIdx.x < static_cast<unsigned>(B)) {
    __shared__ int wsum[4];
    const int b = blockIdx.x;
    const uint8_t* mrow = mask == nullptr ? nullptr : mask + static_cast<int64_t>(b) * L;
    const bool vec_ok = mrow != nullptr && reinterpret_cast<uintptr_t>(mrow) % 16 == 0;
    auto tile_count = [&](int j) -> int {
      const int tb = j * kTL, te = min(tb + kTL, L);
      if (mrow == nullptr) return te - tb;
      int c = 0;
      if (vec_ok && te - tb == kTL) {
#pragma unroll
        for (int i = 0; i < kTL / 16; ++i) {
          const uint4 v = *reinterpret_cast<const uint4*>(mrow + tb + 16 * i);
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int sh = 0; sh < 32; sh += 8) c += ((w[k] >> sh) & 0xffu) == 0u ? 1 : 0;
        }
      } else {
        for (int t = tb; t < te; ++t) c += mrow[t] == 0 ? 1 : 0;
      }
      return c;
    };
    const int per = (NT + 255) / 256;  // tiles per thread
    const int j0 = threadIdx.x * per;
    int local = 0;
    for (int j = j0; j < j0 + per && j < NT; ++j) local += tile_count(j);
    const int lane = threadIdx.x % kWave, wv = threadIdx.x / kWave;
    int inc = local;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int o = __shfl_up(inc, d, kWave);
      if (lane >= d) inc += o;
    }
    if (lane == kWave - 1) wsum[wv] = inc;
    __syncthreads();
    int run = inc - local;
    for (int i = 0; i < wv; ++i) run += wsum[i];
    for (int j = j0; j < j0 + per && j < NT; ++j) {
      nbefore[b * (NT + 1) + j] = run;
      run += per == 1 ? local : tile_count(j);
      if (j == NT - 1) nbefore[b * (NT + 1) + NT] = run;
    }
  }
}

// the serial kernels never wait: their launches only reset the workspace's status word
__global__ void tsn_clear_status_kernel(int* ticket) { ticket[kStatusSlot] = 0; }

// ------------------------------ forward ---------------------------------------
constexpr int kFwdWords = 2;  // aggregate (u, v), inclusive prefix (u, v)

// carry of all tiles before tile j of this chain (wave 0 only)
__device__ __forceinline__ Wel fwd_lookback(const TsnParams& p, int b, int g, int j, int lane,
                                            Wel prior) {
  const int64_t chain = static_cast<int64_t>(b) * p.G + g;
  const unsigned long long* rec = p.rec + chain * p.NT * kFwdWords;
  const int* nb = p.nbefore + b * (p.NT + 1);
  Wel total{0.f, 0.f, 0.f};
  int base = j - 1;
  while (true) {
    const int idx = base - lane;
    int kind = 3;  // 1 aggregate, 2 inclusive prefix, 3 beyond the chain start or outside the window
    Wel val{0.f, 0.f, 0.f};
    if (lane < kWin) {
      if (idx >= 0) {
        const unsigned long long* r = rec + static_cast<int64_t>(idx) * kFwdWords;
        long long polls = 0;
        while (true) {
          // both words in one round trip: the aggregate counts only if the
          // inclusive prefix is not there yet
          float iu, iv, au, av;
          const bool fi = get_pair(r + 1, iu, iv);
          const bool fa = get_pair(r + 0, au, av);
          if (fi) {
            kind = 2;
            val = Wel{prior.n + static_cast<float>(nb[idx + 1]), iu, iv};
            break;
          }
          if (fa) {
            kind = 1;
            val = Wel{static_cast<float>(nb[idx + 1] - nb[idx]), au, av};
            break;
          }
          if (++polls >= p.spin_limit) {
            give_up(p);
            kind = 2;
            val = Wel{prior.n + static_cast<float>(nb[idx + 1]), __builtin_nanf(""), __builtin_nanf("")};
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
      } else if (idx == -1) {
        kind = 2;
        val = prior;
      }
    }
    const unsigned long long m2 = __ballot(kind == 2);
    const int k = m2 ? __ffsll(static_cast<long long>(m2)) - 1 : 64;
    if (lane > k || kind == 3) val = Wel{0.f, 0.f, 0.f};
#pragma unroll
    for (int off = kWin / 2; off > 0; off >>= 1) val = wel_merge(val, wel_shfl_xor(val, off));
    val = Wel{__shfl(val.n, 0, 64), __shfl(val.u, 0, 64), __shfl(val.v, 0, 64)};
    total = wel_merge(val, total);
    if (m2) break;
    base -= kWin;
  }
  return total;
}

template <int DT, int LPR>
__global__ __launch_bounds__(kThreads) void tsn_fwd_kernel(const TsnParams p) {
  constexpr int VEC = Vec<DT>::N;
  constexpr int RPW = kWave / LPR;         // rows per wave per pass
  constexpr int RPP = RPW * kWaves;        // rows per pass
  constexpr int P = kTL / RPP;             // passes
  __shared__ float s_a[kTL], s_b[kTL];
  __shared__ int s_valid[kTL];
  __shared__ int s_ticket;

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int NC = p.B * p.G;
  const int chain = static_cast<int>(blockIdx.x % static_cast<unsigned>(NC));
  if (threadIdx.x == 0) s_ticket = atomicAdd(p.ticket + chain * kTicketStride, 1);
  __syncthreads();
  const int j = s_ticket;  // the grid holds NT workgroups per chain
  const int b = chain / p.G, g = chain % p.G;
  const int t0 = j * kTL;
  const int col = lane % LPR;
  const bool col_ok = col * VEC < p.Dg;
  const float inv_dg = 1.f / static_cast<float>(p.Dg);

  // everything the tile needs from memory is requested up front: the rows, the
  // affine parameters of the last phase and the chain's prior state
  // bit r of `live`: row r of the tile is a real, unmasked step; padding rows
  // are never read
  unsigned long long live;
  {
    const int t = t0 + lane;
    live = __ballot(t < p.L && (p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0));
  }
  uint4 xv[P];
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPP + wave * RPW + lane / LPR;
    const int t = t0 + r;
    xv[q] = make_uint4(0, 0, 0, 0);
    if (((live >> r) & 1) && col_ok) {
      const int64_t off = (static_cast<int64_t>(b) * p.L + t) * p.D + g * p.Dg + col * VEC;
      xv[q] = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.x) + off);
    }
  }
  uint4 gmv = make_uint4(0, 0, 0, 0), btv = make_uint4(0, 0, 0, 0);
  if (col_ok) {
    gmv = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.gamma) + g * p.Dg + col * VEC);
    btv = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.beta) + g * p.Dg + col * VEC);
  }
  const int64_t chain64 = static_cast<int64_t>(b) * p.G + g;
  const Wel prior{static_cast<float>(p.prev_count[b]), ldT<DT>(p.prev_mean, chain64),
                  ldT<DT>(p.prev_var, chain64)};
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPP + wave * RPW + lane / LPR;
    float f[VEC];
    Vec<DT>::unpack(xv[q], f);
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < VEC; ++e) s += f[e];
    const float mu = row_sum<LPR>(s) * inv_dg;
    float s2 = 0.f;
    if (col_ok) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) s2 += (f[e] - mu) * (f[e] - mu);
    }
    const float var = row_sum<LPR>(s2) * inv_dg;
    if (col == 0) {
      s_a[r] = mu;
      s_b[r] = var;
    }
  }
  __syncthreads();

  if (wave == 0) {
    const int t = t0 + lane;
    const bool valid = t < p.L && (p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0);
    Wel me{valid ? 1.f : 0.f, valid ? s_a[lane] : 0.f, valid ? s_b[lane] : 0.f};
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const Wel o = wel_shfl_up(me, d);
      if (lane >= d) me = wel_merge(o, me);
    }
    unsigned long long* rec = p.rec + (chain64 * p.NT + j) * kFwdWords;
    const Wel agg{__shfl(me.n, 63, 64), __shfl(me.u, 63, 64), __shfl(me.v, 63, 64)};
    if (lane == 0 && j + 1 < p.NT && j != p.mute_tile) {
      put_pair(rec + 0, agg.u, agg.v);
    }
    const Wel prefix = j == 0 ? prior : fwd_lookback(p, b, g, j, lane, prior);
    if (lane == 0 && j + 1 < p.NT && j != p.mute_tile) {
      const Wel inc = wel_merge(prefix, agg);
      put_pair(rec + 1, inc.u, inc.v);
    }
    const Wel st = wel_merge(prefix, me);
    const float rstd = 1.f / sqrtf(st.v + p.eps);
    if (t < p.L) {
      const int64_t o = stat_index(p, b, t, g);
      p.cummean[o] = st.u;
      p.cumrstd[o] = rstd;
    }
    s_valid[lane] = valid ? 1 : 0;
    if (j == p.NT - 1 && lane == 63) {
      stT<DT>(p.mean, chain64, st.u);
      stT<DT>(p.var, chain64, st.v);
      if (g == 0) p.count[b] = p.prev_count[b] + p.nbefore[b * (p.NT + 1) + p.NT];
    }
    // s_a/s_b reads retired before they are overwritten (LDS only: the stores
    // above need not have landed)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    s_a[lane] = st.u;
    s_b[lane] = rstd;
  }
  __syncthreads();

  float gm[VEC], bt[VEC];
  Vec<DT>::unpack(gmv, gm);
  Vec<DT>::unpack(btv, bt);
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPP + wave * RPW + lane / LPR;
    const int t = t0 + r;
    if (t < p.L && col_ok) {
      float f[VEC], o[VEC];
      Vec<DT>::unpack(xv[q], f);
      const float u = s_a[r], rs = s_b[r];
      const bool valid = s_valid[r] != 0;
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[e] = valid ? (f[e] - u) * rs * gm[e] + bt[e] : 0.f;
      const int64_t off = (static_cast<int64_t>(b) * p.L + t) * p.D + g * p.Dg + col * VEC;
      store_streaming(static_cast<typename Elem<DT>::type*>(p.y) + off, Vec<DT>::pack(o));
    }
  }
}

// Narrow groups (at most 32 lanes per row): every wavefront owns a tile of its
// own -- it loads the 64 rows, reduces, scans, looks back and normalises
// without a workgroup barrier, so a slow tile holds up nobody else and each
// wave keeps a whole tile's loads in flight.  The workgroup's four waves share
// one ticket (a single counter here: with a quarter of the tickets its cost
// stays below the kernel's time, and the pacing it gives the workgroups'
// starts measured 7 % faster than per-group counters): tiles 4 ticket ..
// 4 ticket + 3 in time order, which only ever wait for tiles of smaller or
// equal ticket.
template <int DT, int LPR>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4)))
void tsn_fwd_wave_kernel(const TsnParams p, int tiles) {
  constexpr int VEC = Vec<DT>::N;
  constexpr int RPW = kWave / LPR;  // rows per pass
  constexpr int P = LPR;            // passes: kTL / RPW
  __shared__ float s_a[kWaves][kTL], s_b[kWaves][kTL];
  __shared__ int s_valid[kWaves][kTL];
  __shared__ int s_ticket;

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  if (threadIdx.x == 0) s_ticket = atomicAdd(p.ticket, 1);
  __syncthreads();
  const int tile = s_ticket * kWaves + wave;
  if (tile >= tiles) return;  // no workgroup barrier below
  const int NC = p.B * p.G;
  const int j = tile / NC;
  const int chain = tile % NC;
  const int b = chain / p.G, g = chain % p.G;
  const int t0 = j * kTL;
  const int col = lane % LPR;
  const bool col_ok = col * VEC < p.Dg;
  const float inv_dg = 1.f / static_cast<float>(p.Dg);
  float* sa = s_a[wave];
  float* sb = s_b[wave];
  int* sv = s_valid[wave];

  // element offset of this lane's vector in pass 0; a pass advances RPW rows
  const int64_t off0 =
      (static_cast<int64_t>(b) * p.L + t0 + lane / LPR) * p.D + g * p.Dg + col * VEC;
  const int64_t pass_stride = static_cast<int64_t>(RPW) * p.D;
  const int rows_left = p.L - t0 - lane / LPR;  // pass q is in range iff q * RPW < rows_left
  const typename Elem<DT>::type* xp = static_cast<const typename Elem<DT>::type*>(p.x) + off0;
  // lane <-> time step for the scan; bit r of `live` says that row r of the
  // tile is a real, unmasked step.  Padding rows are never read: their
  // output is zero and they leave the statistics alone.
  const int t = t0 + lane;
  const bool valid = t < p.L && (p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0);
  const unsigned long long live = __ballot(valid);
  uint4 xv[P];
#pragma unroll
  for (int q = 0; q < P; ++q) {
    xv[q] = make_uint4(0, 0, 0, 0);
    if (((live >> (q * RPW + lane / LPR)) & 1) && col_ok) xv[q] = *reinterpret_cast<const uint4*>(xp + q * pass_stride);
  }
  uint4 gmv = make_uint4(0, 0, 0, 0), btv = make_uint4(0, 0, 0, 0);
  if (col_ok) {
    gmv = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.gamma) + g * p.Dg + col * VEC);
    btv = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.beta) + g * p.Dg + col * VEC);
  }
  const int64_t chain64 = static_cast<int64_t>(b) * p.G + g;
  const Wel prior{static_cast<float>(p.prev_count[b]), ldT<DT>(p.prev_mean, chain64),
                  ldT<DT>(p.prev_var, chain64)};
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPW + lane / LPR;
    float mu, var;
    if (DT == MEGA_BF16) {
      // one pass over the packed words.  E[x^2] - mu^2 in fp32 is exact to
      // ~1e-7 (1 + mu^2 / var), and bf16 data cannot hold |mu| / sigma > 256
      float s1, s2;
      Vec<MEGA_BF16>::moments(xv[q], s1, s2);  // lanes past the group hold zeros
      mu = row_sum<LPR>(s1) * inv_dg;
      var = fmaxf(row_sum<LPR>(s2) * inv_dg - mu * mu, 0.f);
    } else {
      float f[VEC];
      Vec<DT>::unpack(xv[q], f);
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < VEC; ++e) s += f[e];
      mu = row_sum<LPR>(s) * inv_dg;
      float s2 = 0.f;
      if (col_ok) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) s2 += (f[e] - mu) * (f[e] - mu);
      }
      var = row_sum<LPR>(s2) * inv_dg;
    }
    if (col == 0) {
      sa[r] = mu;
      sb[r] = var;
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();

  Wel me{valid ? 1.f : 0.f, valid ? sa[lane] : 0.f, valid ? sb[lane] : 0.f};
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const Wel o = wel_shfl_up(me, d);
    if (lane >= d) me = wel_merge(o, me);
  }
  unsigned long long* rec = p.rec + (chain64 * p.NT + j) * kFwdWords;
  const Wel agg{__shfl(me.n, 63, 64), __shfl(me.u, 63, 64), __shfl(me.v, 63, 64)};
  if (lane == 0 && j + 1 < p.NT && j != p.mute_tile) {
    put_pair(rec + 0, agg.u, agg.v);
  }
  const Wel prefix = j == 0 ? prior : fwd_lookback(p, b, g, j, lane, prior);
  if (lane == 0 && j + 1 < p.NT && j != p.mute_tile) {
    const Wel inc = wel_merge(prefix, agg);
    put_pair(rec + 1, inc.u, inc.v);
  }
  const Wel st = wel_merge(prefix, me);
  const float rstd = 1.f / sqrtf(st.v + p.eps);
  if (t < p.L) {
    const int64_t o = stat_index(p, b, t, g);
    p.cummean[o] = st.u;
    p.cumrstd[o] = rstd;
  }
  if (j == p.NT - 1 && lane == 63) {
    stT<DT>(p.mean, chain64, st.u);
    stT<DT>(p.var, chain64, st.v);
    if (g == 0) p.count[b] = p.prev_count[b] + p.nbefore[b * (p.NT + 1) + p.NT];
  }
  // the row moments were read before the scan (the shuffles above depend on
  // them); a wave runs in program order, so they can be overwritten now
  // y = x rstd - mean rstd per row (then gamma, beta per column); masked rows
  // get the zero map and are cleared after packing
  sa[lane] = valid ? -st.u * rstd : 0.f;
  sb[lane] = valid ? rstd : 0.f;
  sv[lane] = valid ? 1 : 0;
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();

  float gm[VEC], bt[VEC];
  Vec<DT>::unpack(gmv, gm);
  Vec<DT>::unpack(btv, bt);
  typename Elem<DT>::type* yp = static_cast<typename Elem<DT>::type*>(p.y) + off0;
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPW + lane / LPR;
    if (q * RPW < rows_left && col_ok) {
      float f[VEC], o[VEC];
      Vec<DT>::unpack(reload(xv[q]), f);
      const float nur = sa[r], rs = sb[r];
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[e] = fmaf(fmaf(f[e], rs, nur), gm[e], bt[e]);
      uint4 packed = Vec<DT>::pack(o);
      if (sv[r] == 0) packed = make_uint4(0, 0, 0, 0);
      store_streaming(yp + q * pass_stride, packed);
    }
  }
}

// Any shape: one wavefront per (batch, group) walks the sequence step by step.
template <int DT>
__global__ __launch_bounds__(kWave) void tsn_fwd_serial_kernel(const TsnParams p) {
  const int chain = blockIdx.x;
  const int b = chain / p.G, g = chain % p.G;
  const int lane = threadIdx.x;
  const float inv_dg = 1.f / static_cast<float>(p.Dg);
  Wel st{static_cast<float>(p.prev_count[b]), ldT<DT>(p.prev_mean, chain), ldT<DT>(p.prev_var, chain)};
  int64_t cnt = p.prev_count[b];
  for (int t = 0; t < p.L; ++t) {
    const int64_t row = (static_cast<int64_t>(b) * p.L + t) * p.D + g * p.Dg;
    const bool valid = p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0;
    float s = 0.f;
    for (int i = lane; i < p.Dg; i += kWave) s += ldT<DT>(p.x, row + i);
    const float mu = wave_sum(s) * inv_dg;
    float s2 = 0.f;
    for (int i = lane; i < p.Dg; i += kWave) {
      const float d = ldT<DT>(p.x, row + i) - mu;
      s2 += d * d;
    }
    const float var = wave_sum(s2) * inv_dg;
    if (valid) {
      st = wel_merge(st, Wel{1.f, mu, var});
      ++cnt;
    }
    const float rstd = 1.f / sqrtf(st.v + p.eps);
    if (lane == 0) {
      const int64_t o = stat_index(p, b, t, g);
      p.cummean[o] = st.u;
      p.cumrstd[o] = rstd;
    }
    for (int i = lane; i < p.Dg; i += kWave) {
      const float xx = ldT<DT>(p.x, row + i);
      const float o = valid ? (xx - st.u) * rstd * ldT<DT>(p.gamma, g * p.Dg + i) +
                                  ldT<DT>(p.beta, g * p.Dg + i)
                            : 0.f;
      stT<DT>(p.y, row + i, o);
    }
  }
  if (lane == 0) {
    stT<DT>(p.mean, chain, st.u);
    stT<DT>(p.var, chain, st.v);
    if (g == 0) p.count[b] = cnt;
  }
}

// ------------------------------ backward --------------------------------------
constexpr int kBwdWords = 3;  // aggregate (a, e), (bu, bv), outgoing state (ug, vg)

struct State2 {
  float ug, vg;
};
__device__ __forceinline__ State2 aff_apply(Aff m, State2 s) {
  return State2{m.a * s.ug + m.e * s.vg + m.bu, m.a * s.vg + m.bv};
}

// state entering tile j from the later tiles of this chain (wave 0 only)
__device__ __forceinline__ State2 bwd_lookahead(const TsnParams& p, int64_t chain, int j, int lane,
                                                State2 init) {
  const unsigned long long* rec = p.rec + chain * p.NT * kBwdWords;
  Aff total{1.f, 0.f, 0.f, 0.f};
  int base = j + 1;
  while (true) {
    const int idx = base + lane;
    int kind = 3;
    Aff val{1.f, 0.f, 0.f, 0.f};
    State2 sv{0.f, 0.f};
    if (lane < kWin) {
      if (idx < p.NT) {
        const unsigned long long* r = rec + static_cast<int64_t>(idx) * kBwdWords;
        long long polls = 0;
        while (true) {
          // all three words in one round trip
          float a, e, bu, bv, ug, vg;
          const bool fs = get_pair(r + 2, ug, vg);
          const bool f0 = get_pair(r + 0, a, e), f1 = get_pair(r + 1, bu, bv);
          if (fs) {
            kind = 2;
            sv = State2{ug, vg};
            break;
          }
          if (f0 & f1) {
            kind = 1;
            val = Aff{a, e, bu, bv};
            break;
          }
          if (++polls >= p.spin_limit) {
            give_up(p);
            kind = 2;
            sv = State2{__builtin_nanf(""), __builtin_nanf("")};
            break;
          }
          __builtin_amdgcn_s_sleep(2);
        }
      } else if (idx == p.NT) {
        kind = 2;
        sv = init;
      }
    }
    const unsigned long long m2 = __ballot(kind == 2);
    const int k = m2 ? __ffsll(static_cast<long long>(m2)) - 1 : 64;
    if (lane >= k || kind != 1) val = Aff{1.f, 0.f, 0.f, 0.f};
    // ordered prefix composition: lane l holds A_base o ... o A_(base+l)
#pragma unroll
    for (int d = 1; d < kWin; d <<= 1) {
      const Aff o = aff_shfl_up(val, d);
      if (lane >= d) val = aff_compose(o, val);
    }
    const Aff win{__shfl(val.a, kWin - 1, 64), __shfl(val.e, kWin - 1, 64),
                  __shfl(val.bu, kWin - 1, 64), __shfl(val.bv, kWin - 1, 64)};
    total = aff_compose(total, win);
    if (m2) {
      const State2 s{__shfl(sv.ug, k, 64), __shfl(sv.vg, k, 64)};
      return aff_apply(total, s);
    }
    base += kWin;
  }
}

template <int DT, int LPR>
__global__ __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(LPR <= 16 ? 4 : (LPR == 32 ? 2 : 1))))  // at least this many waves per SIMD
void tsn_bwd_kernel(const TsnParams p) {
  constexpr int VEC = Vec<DT>::N;
  constexpr int RPW = kWave / LPR;
  constexpr int RPP = RPW * kWaves;
  constexpr int P = kTL / RPP;
  __shared__ float s_ux[kTL], s_ds[kTL], s_db[kTL];   // row stats, then (ux, dux, dvx)
  __shared__ float s_u[kTL], s_r[kTL];
  __shared__ int s_valid[kTL];
  __shared__ float s_pg[kWaves][LPR * VEC], s_pb[kWaves][LPR * VEC];
  __shared__ int s_ticket;

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int NC = p.B * p.G;
  const int chain = static_cast<int>(blockIdx.x % static_cast<unsigned>(NC));
  if (threadIdx.x == 0) s_ticket = atomicAdd(p.ticket + chain * kTicketStride, 1);
  __syncthreads();
  const int j = p.NT - 1 - s_ticket;  // later tiles first; the grid holds NT workgroups per chain
  const int b = chain / p.G, g = chain % p.G;
  const int t0 = j * kTL;
  const int col = lane % LPR;
  const bool col_ok = col * VEC < p.Dg;
  const float inv_dg = 1.f / static_cast<float>(p.Dg);

  // everything the tile needs from memory is requested up front: the rows of x
  // and dy, gamma, the saved statistics and the chain's boundary values
  // bit r of `live`: row r of the tile is a real, unmasked step.  Padding rows
  // are never read (dx = 0 there and they add nothing to any sum).
  unsigned long long live;
  {
    const int t = t0 + lane;
    live = __ballot(t < p.L && (p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0));
  }
  uint4 xv[P], dv[P];
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPP + wave * RPW + lane / LPR;
    const int t = t0 + r;
    xv[q] = make_uint4(0, 0, 0, 0);
    dv[q] = make_uint4(0, 0, 0, 0);
    if (((live >> r) & 1) && col_ok) {
      const int64_t off = (static_cast<int64_t>(b) * p.L + t) * p.D + g * p.Dg + col * VEC;
      xv[q] = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.x) + off);
      dv[q] = load_once(static_cast<const typename Elem<DT>::type*>(p.dy) + off);
    }
  }
  uint4 gmv = make_uint4(0, 0, 0, 0);
  if (col_ok)
    gmv = *reinterpret_cast<const uint4*>(static_cast<const typename Elem<DT>::type*>(p.gamma) + g * p.Dg + col * VEC);
  const int64_t chain64 = static_cast<int64_t>(b) * p.G + g;
  // wave 0 only uses these; loading them in every wave keeps the code uniform
  const float before_u = t0 == 0 ? ldT<DT>(p.prev_mean, chain64)
                                 : p.cummean_in[stat_index(p, b, t0 - 1, g)];
  const State2 init{ldT<DT>(p.dmean, chain64), ldT<DT>(p.dvar, chain64)};
  const int* nb = p.nbefore + b * (p.NT + 1);
  const int64_t n0 = p.prev_count[b] - nb[p.NT];  // prior count
  const int nbj = nb[j];

  // statistics saved by the forward pass, one row per lane
  {
    const int t = t0 + lane;
    if (wave == 0) {
      const bool in = t < p.L;
      const int64_t o = stat_index(p, b, in ? t : 0, g);
      s_u[lane] = in ? p.cummean_in[o] : 0.f;
      s_r[lane] = in ? p.cumrstd_in[o] : 0.f;
      s_valid[lane] = (in && (p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0)) ? 1 : 0;
    }
  }
  __syncthreads();
  float gm[VEC];
  Vec<DT>::unpack(gmv, gm);

#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPP + wave * RPW + lane / LPR;
    float f[VEC], d[VEC];
    Vec<DT>::unpack(xv[q], f);
    Vec<DT>::unpack(dv[q], d);
    // ds = sum dy gamma (x - u) = sum (dy gamma) x - u sum (dy gamma): lanes past
    // the group hold zeros and add nothing
    float sx = 0.f, sa = 0.f, sdb = 0.f;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float dg = d[e] * gm[e];
      sx += f[e];
      sa = fmaf(dg, f[e], sa);
      sdb += dg;
    }
    sx = row_sum<LPR>(sx);
    sa = row_sum<LPR>(sa);
    sdb = row_sum<LPR>(sdb);
    if (col == 0) {
      s_ux[r] = sx * inv_dg;
      s_ds[r] = sa - s_u[r] * sdb;
      s_db[r] = sdb;
    }
  }
  __syncthreads();

  if (wave == 0) {
    const bool valid = s_valid[lane] != 0;
    // n_t = number of valid steps up to and including t, prior included
    const unsigned long long vm = __ballot(valid);
    const int incl = __popcll(vm & ((lane == 63) ? ~0ull : ((1ull << (lane + 1)) - 1ull)));
    const float nt = static_cast<float>(n0 + nbj + incl);
    const float c1 = valid ? (nt - 1.f) / nt : 0.f;
    const float c2 = valid ? 1.f / nt : 0.f;
    const float r = s_r[lane], ux = s_ux[lane];
    const float prev_u = lane == 0 ? before_u : s_u[lane - 1];
    const float delta = ux - prev_u;
    const float pu = -r * s_db[lane];
    const float pv = -0.5f * r * r * r * s_ds[lane];
    const float e = -2.f * c1 * c2 * delta;
    const Aff mine = valid ? Aff{c1, e, c1 * pu + e * pv, c1 * pv} : Aff{1.f, 0.f, 0.f, 0.f};
    // inclusive suffix composition: I_i = X_i o X_(i+1) o ... o X_63
    Aff inc = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const Aff o = aff_shfl_down(inc, d);
      if (lane + d < 64) inc = aff_compose(inc, o);
    }
    unsigned long long* rec = p.rec + (chain64 * p.NT + j) * kBwdWords;
    if (lane == 0 && j > 0 && j != p.mute_tile) {
      put_pair(rec + 0, inc.a, inc.e);
      put_pair(rec + 1, inc.bu, inc.bv);
    }
    const State2 sin = j == p.NT - 1 ? init : bwd_lookahead(p, chain64, j, lane, init);
    // state entering row i = (X_(i+1) o ... o X_63)(sin)
    Aff exc = aff_shfl_down(inc, 1);
    if (lane == 63) exc = Aff{1.f, 0.f, 0.f, 0.f};
    const State2 si = aff_apply(exc, sin);
    if (lane == 0) {
      const State2 sout = aff_apply(inc, sin);
      if (j > 0) {
        if (j != p.mute_tile) put_pair(rec + 2, sout.ug, sout.vg);
      } else {
        stT<DT>(p.mean, chain64, sout.ug);
        stT<DT>(p.var, chain64, sout.vg);
      }
    }
    const float du = si.ug + pu;
    const float dvv = si.vg + pv;
    const float dux = c2 * du + 2.f * c1 * c2 * dvv * delta;
    const float dvx = c2 * dvv;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // LDS reads above retired
    __builtin_amdgcn_wave_barrier();
    // dx = dy gamma r + c0 + c1 x with c1 = 2 dvx / Dg, c0 = (dux - 2 dvx ux) / Dg;
    // masked rows get the zero map (their x and dy are cleared before use, so
    // whatever the padding holds stays out of dx and the parameter sums)
    s_ds[lane] = valid ? (dux - 2.f * dvx * ux) * inv_dg : 0.f;
    s_db[lane] = valid ? 2.f * dvx * inv_dg : 0.f;
    s_r[lane] = valid ? r : 0.f;
  }
  __syncthreads();

  float pg[VEC], pb[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) pg[e] = pb[e] = 0.f;
#pragma unroll
  for (int q = 0; q < P; ++q) {
    const int r = q * RPP + wave * RPW + lane / LPR;
    const int t = t0 + r;
    if (t < p.L && col_ok) {
      float f[VEC], d[VEC], o[VEC];
      uint4 xq = xv[q], dq = dv[q];
      if (s_valid[r] == 0) xq = dq = make_uint4(0, 0, 0, 0);
      Vec<DT>::unpack(xq, f);
      Vec<DT>::unpack(dq, d);
      const float u = s_u[r], rs = s_r[r], c0 = s_ds[r], c1 = s_db[r];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        o[e] = fmaf(d[e] * gm[e], rs, fmaf(c1, f[e], c0));
        pg[e] = fmaf(d[e] * rs, f[e] - u, pg[e]);
        pb[e] += d[e];
      }
      const int64_t off = (static_cast<int64_t>(b) * p.L + t) * p.D + g * p.Dg + col * VEC;
      store_streaming(static_cast<typename Elem<DT>::type*>(p.y) + off, Vec<DT>::pack(o));
    }
  }
  // per-tile column sums of the gamma / beta gradients
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) {
      pg[e] += __shfl_xor(pg[e], off, 64);
      pb[e] += __shfl_xor(pb[e], off, 64);
    }
    if (lane < LPR) {
      s_pg[wave][col * VEC + e] = pg[e];
      s_pb[wave][col * VEC + e] = pb[e];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < LPR * VEC; i += kThreads) {
    if (i < p.Dg) {
      float a = 0.f, c = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        a += s_pg[w][i];
        c += s_pb[w][i];
      }
      const int64_t o = (static_cast<int64_t>(b) * p.NT + j) * p.D + g * p.Dg + i;
      p.part_g[o] = a;
      p.part_b[o] = c;
    }
  }
}

template <int DT>
__global__ __launch_bounds__(kWave) void tsn_bwd_serial_kernel(const TsnParams p) {
  const int chain = blockIdx.x;
  const int b = chain / p.G, g = chain % p.G;
  const int lane = threadIdx.x;
  const float inv_dg = 1.f / static_cast<float>(p.Dg);
  float ug = ldT<DT>(p.dmean, chain), vg = ldT<DT>(p.dvar, chain);
  int64_t m0 = p.prev_count[b];
  // per-(batch) partial sums live in part_g/part_b rows [b] (NT == 1 layout)
  for (int i = lane; i < p.Dg; i += kWave) {
    p.part_g[static_cast<int64_t>(b) * p.D + g * p.Dg + i] = 0.f;
    p.part_b[static_cast<int64_t>(b) * p.D + g * p.Dg + i] = 0.f;
  }
  for (int t = p.L - 1; t >= 0; --t) {
    const int64_t row = (static_cast<int64_t>(b) * p.L + t) * p.D + g * p.Dg;
    const bool valid = p.mask == nullptr || p.mask[static_cast<int64_t>(b) * p.L + t] == 0;
    if (!valid) {
      for (int i = lane; i < p.Dg; i += kWave) stT<DT>(p.y, row + i, 0.f);
      continue;
    }
    const int64_t so = stat_index(p, b, t, g);
    const float u = p.cummean_in[so], r = p.cumrstd_in[so];
    const float prev_u = t == 0 ? ldT<DT>(p.prev_mean, chain) : p.cummean_in[so - p.st_t];
    const float c1 = static_cast<float>(m0 - 1) / static_cast<float>(m0);
    const float c2 = 1.f / static_cast<float>(m0);
    --m0;
    float sx = 0.f, sds = 0.f, sdb = 0.f;
    for (int i = lane; i < p.Dg; i += kWave) {
      const float xx = ldT<DT>(p.x, row + i), d = ldT<DT>(p.dy, row + i);
      const float w = ldT<DT>(p.gamma, g * p.Dg + i);
      sx += xx;
      sds += d * (xx - u) * w;
      sdb += d * w;
    }
    const float ux = wave_sum(sx) * inv_dg;
    const float ds = wave_sum(sds), db = wave_sum(sdb);
    const float du = ug - r * db;
    const float dvv = vg - 0.5f * r * r * r * ds;
    const float dux = c2 * du + 2.f * c1 * c2 * dvv * (ux - prev_u);
    const float dvx = c2 * dvv;
    for (int i = lane; i < p.Dg; i += kWave) {
      const float xx = ldT<DT>(p.x, row + i), d = ldT<DT>(p.dy, row + i);
      const float w = ldT<DT>(p.gamma, g * p.Dg + i);
      stT<DT>(p.y, row + i, d * r * w + (dux + 2.f * dvx * (xx - ux)) * inv_dg);
      p.part_g[static_cast<int64_t>(b) * p.D + g * p.Dg + i] += d * (xx - u) * r;
      p.part_b[static_cast<int64_t>(b) * p.D + g * p.Dg + i] += d;
    }
    ug = c1 * du - 2.f * c1 * c2 * dvv * (ux - prev_u);
    vg = c1 * dvv;
  }
  if (lane == 0) {
    stT<DT>(p.mean, chain, ug);
    stT<DT>(p.var, chain, vg);
  }
}

// dgamma[h] = sum_rows part_g[row][h] (same for dbeta), rows = B*NT.  A workgroup
// owns 64 columns; its 16 waves split the rows (Kahan-compensated partial sums
// in a fixed order: deterministic), then combine through LDS.
constexpr int kPgWaves = 16;
template <int DT>
__global__ __launch_bounds__(kPgWaves * 64) void tsn_param_grad_kernel(
    const float* part_g, const float* part_b, int rows, int D, void* dgamma, void* dbeta) {
  __shared__ float sg[kPgWaves][64], sb[kPgWaves][64];
  const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
  const int h = blockIdx.x * 64 + lane;
  float a = 0.f, c = 0.f, ca = 0.f, cc = 0.f;
  if (h < D) {
    constexpr int U = 8;  // rows in flight per wave
    int r = w;
    for (; r + (U - 1) * kPgWaves < rows; r += U * kPgWaves) {
      float va[U], vc[U];
#pragma unroll
      for (int i = 0; i < U; ++i) {
        va[i] = part_g[static_cast<int64_t>(r + i * kPgWaves) * D + h];
        vc[i] = part_b[static_cast<int64_t>(r + i * kPgWaves) * D + h];
      }
#pragma unroll
      for (int i = 0; i < U; ++i) {
        const float ya = va[i] - ca;
        const float ta = a + ya;
        ca = (ta - a) - ya;
        a = ta;
        const float yc = vc[i] - cc;
        const float tc = c + yc;
        cc = (tc - c) - yc;
        c = tc;
      }
    }
    for (; r < rows; r += kPgWaves) {
      const float ya = part_g[static_cast<int64_t>(r) * D + h] - ca;
      const float ta = a + ya;
      ca = (ta - a) - ya;
      a = ta;
      const float yc = part_b[static_cast<int64_t>(r) * D + h] - cc;
      const float tc = c + yc;
      cc = (tc - c) - yc;
      c = tc;
    }
  }
  sg[w][lane] = a;
  sb[w][lane] = c;
  __syncthreads();
  if (w == 0 && h < D) {
    float ta = 0.f, tc = 0.f;
#pragma unroll
    for (int i = 0; i < kPgWaves; ++i) {
      ta += sg[i][lane];
      tc += sb[i][lane];
    }
    stT<DT>(dgamma, h, ta);
    stT<DT>(dbeta, h, tc);
  }
}

// ------------------------------ host side --------------------------------------
inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Test hooks (mega_test_timestep_norm_lookback): the poll limit of the look-back
// waits and a tile index that publishes no record, for the launches that follow.
std::atomic<long long> g_spin_limit{kDefaultSpinLimit};
std::atomic<int> g_mute_tile{-1};

struct WsLayout {
  int64_t ticket_off, nbefore_off, rec_off, rec_words, part_off, total;
};
WsLayout ws_layout(int64_t B, int64_t L, int64_t D, int64_t G, int words, bool partials) {
  const int64_t NT = (L + kTL - 1) / kTL;
  WsLayout w;
  w.ticket_off = 0;  // one counter per (batch, group) chain
  w.nbefore_off = align_up(B * G * kTicketStride * 4, 256);
  w.rec_off = align_up(w.nbefore_off + B * (NT + 1) * 4, 256);
  w.rec_words = B * G * NT * words;
  w.part_off = align_up(w.rec_off + w.rec_words * 8, 256);
  w.total = w.part_off + (partials ? 2 * B * NT * D * 4 : 0);
  return w;
}

bool fast_path_ok(int dtype, int64_t D, int64_t Dg, const void* a, const void* b, const void* c) {
  const int vec = dtype == MEGA_F32 ? 4 : 8;
  const auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  return Dg % vec == 0 && D % vec == 0 && Dg / vec <= 64 && al(a) && (b == nullptr || al(b)) &&
         (c == nullptr || al(c));
}

template <int DT, bool FWD>
int launch_fast(const TsnParams& p, int64_t tiles, hipStream_t s) {
  const int vec = DT == MEGA_F32 ? 4 : 8;
  const int lanes = p.Dg / vec;
  const dim3 grid(static_cast<unsigned>(tiles));  // NT workgroups per chain
  // forward, narrow groups: one tile per wavefront
  const dim3 wgrid(static_cast<unsigned>((tiles + kWaves - 1) / kWaves));
  const int nt = static_cast<int>(tiles);
  // Fewer resident workgroups than the registers allow move the bytes faster: a wave asks for
  // its whole tile at once, and with every wave slot filled (256 KB requested per compute unit)
  // the memory system delivers 5.0 TB/s to a copy of this tile shape, with half of them 5.6.
  // Unused dynamic LDS caps the residency: three workgroups per compute unit for the
  // tile-per-wave forward kernel (config 2: 0.137 -> 0.130 ms), four for the backward kernel
  // of narrow groups (0.204 -> 0.196 ms); measured optima, flat within +-8 KB.
  constexpr size_t kFwdWavePad = 44 * 1024, kBwdPad = 28 * 1024;
#define MEGA_TSN_LAUNCH(LPR)                                              \
  do {                                                                    \
    if (FWD) tsn_fwd_kernel<DT, LPR><<<grid, kThreads, 0, s>>>(p);        \
    else tsn_bwd_kernel<DT, LPR><<<grid, kThreads, (LPR) <= 16 ? kBwdPad : 0, s>>>(p); \
  } while (0)
#define MEGA_TSN_LAUNCH_WAVE(LPR) tsn_fwd_wave_kernel<DT, LPR><<<wgrid, kThreads, kFwdWavePad, s>>>(p, nt)
  if (!FWD) {  // two operand tiles per wave leave too few waves resident
    if (lanes <= 4) MEGA_TSN_LAUNCH(4);
    else if (lanes <= 8) MEGA_TSN_LAUNCH(8);
    else if (lanes <= 16) MEGA_TSN_LAUNCH(16);
    else if (lanes <= 32) MEGA_TSN_LAUNCH(32);
    else MEGA_TSN_LAUNCH(64);
  } else
  if (lanes <= 4) MEGA_TSN_LAUNCH_WAVE(4);
  else if (lanes <= 8) MEGA_TSN_LAUNCH_WAVE(8);
  else if (lanes <= 16) MEGA_TSN_LAUNCH_WAVE(16);
  else if (lanes <= 32) MEGA_TSN_LAUNCH(32);
  else MEGA_TSN_LAUNCH(64);
#undef MEGA_TSN_LAUNCH
#undef MEGA_TSN_LAUNCH_WAVE
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT>
int tsn_fwd_impl(TsnParams p, void* workspace, hipStream_t s) {
  const int64_t NT = p.NT;
  if (fast_path_ok(DT, p.D, p.Dg, p.x, p.y, nullptr) && fast_path_ok(DT, p.D, p.Dg, p.gamma, p.beta, nullptr)) {
    const WsLayout w = ws_layout(p.B, p.L, p.D, p.G, kFwdWords, false);
    char* ws = static_cast<char*>(workspace);
    p.ticket = reinterpret_cast<int*>(ws + w.ticket_off);
    p.status = reinterpret_cast<unsigned int*>(p.ticket + kStatusSlot);
    p.spin_limit = g_spin_limit.load();
    p.mute_tile = g_mute_tile.load();
    int* nbefore = reinterpret_cast<int*>(ws + w.nbefore_off);
    p.nbefore = nbefore;
    p.rec = reinterpret_cast<unsigned long long*>(ws + w.rec_off);
    const int prep_blocks = static_cast<int>(std::max<int64_t>(p.B, std::min<int64_t>(1024, (w.rec_words + 255) / 256)));
    tsn_prep_kernel<<<prep_blocks, 256, 0, s>>>(p.ticket, p.B * p.G, p.rec, w.rec_words, p.mask, nbefore, p.B,
                                                p.L, static_cast<int>(NT));
    MEGA_CHECK_LAUNCH();
    return launch_fast<DT, true>(p, static_cast<int64_t>(p.B) * p.G * NT, s);
  }
  tsn_clear_status_kernel<<<1, 1, 0, s>>>(static_cast<int*>(workspace));
  tsn_fwd_serial_kernel<DT><<<p.B * p.G, kWave, 0, s>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT>
int tsn_bwd_impl(TsnParams p, void* dgamma, void* dbeta, void* workspace, hipStream_t s) {
  const int64_t NT = p.NT;
  char* ws = static_cast<char*>(workspace);
  const WsLayout w = ws_layout(p.B, p.L, p.D, p.G, kBwdWords, true);
  p.part_g = reinterpret_cast<float*>(ws + w.part_off);
  p.part_b = p.part_g + static_cast<int64_t>(p.B) * NT * p.D;
  int rows;
  if (fast_path_ok(DT, p.D, p.Dg, p.x, p.y, p.dy) && fast_path_ok(DT, p.D, p.Dg, p.gamma, nullptr, nullptr)) {
    p.ticket = reinterpret_cast<int*>(ws + w.ticket_off);
    p.status = reinterpret_cast<unsigned int*>(p.ticket + kStatusSlot);
    p.spin_limit = g_spin_limit.load();
    p.mute_tile = g_mute_tile.load();
    int* nbefore = reinterpret_cast<int*>(ws + w.nbefore_off);
    p.nbefore = nbefore;
    p.rec = reinterpret_cast<unsigned long long*>(ws + w.rec_off);
    const int prep_blocks = static_cast<int>(std::max<int64_t>(p.B, std::min<int64_t>(1024, (w.rec_words + 255) / 256)));
    tsn_prep_kernel<<<prep_blocks, 256, 0, s>>>(p.ticket, p.B * p.G, p.rec, w.rec_words, p.mask, nbefore, p.B,
                                                p.L, static_cast<int>(NT));
    MEGA_CHECK_LAUNCH();
    const int rc = launch_fast<DT, false>(p, static_cast<int64_t>(p.B) * p.G * NT, s);
    if (rc != MEGA_OK) return rc;
    rows = static_cast<int>(p.B * NT);
  } else {
    tsn_clear_status_kernel<<<1, 1, 0, s>>>(static_cast<int*>(workspace));
    tsn_bwd_serial_kernel<DT><<<p.B * p.G, kWave, 0, s>>>(p);
    MEGA_CHECK_LAUNCH();
    rows = p.B;
  }
  tsn_param_grad_kernel<DT><<<(p.D + 63) / 64, kPgWaves * 64, 0, s>>>(p.part_g, p.part_b, rows, p.D, dgamma, dbeta);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int64_t mega_group_timestep_norm_workspace_bytes(int64_t B, int64_t L, int64_t D,
                                                            int64_t G, int backward) {
  if (B <= 0 || L <= 0 || D <= 0 || G <= 0) return 256;
  return ws_layout(B, L, D, G, backward ? kBwdWords : kFwdWords, backward != 0).total;
}

static int check_dims(const char* who, int64_t B, int64_t L, int64_t D, int64_t G) {
  MEGA_CHECK_ARG(B >= 0 && L >= 0 && D >= 1 && G >= 1, "%s: bad sizes", who);
  MEGA_CHECK_ARG(D % G == 0, "%s: num_features %lld not divisible by num_groups %lld", who,
                 (long long)D, (long long)G);
  MEGA_CHECK_ARG(B * G <= 0x7fffffff && L <= 0x7fffffff && D <= 0x7fffffff, "%s: size too large", who);
  MEGA_CHECK_ARG(B * G * ((L + kTL - 1) / kTL) <= 0x7fffffff, "%s: too many tiles", who);
  return MEGA_OK;
}

// time_last: cummean / cumrstd are (B, G, L) instead of the reference's (B, L, G)
static void set_stat_strides(TsnParams& p, bool time_last) {
  if (time_last) {
    p.st_b = static_cast<int64_t>(p.G) * p.L; p.st_g = p.L; p.st_t = 1;
  } else {
    p.st_b = static_cast<int64_t>(p.L) * p.G; p.st_t = p.G; p.st_g = 1;
  }
}

static int tsn_fwd_entry(bool time_last, const void* x, int dtype, const int64_t* prev_count,
                         const void* prev_mean, const void* prev_var, const void* gamma, const void* beta,
                         const uint8_t* padding_mask, int64_t B, int64_t L, int64_t D, int64_t G, double eps,
                         void* y, int64_t* count, void* mean, void* var, float* cummean, float* cumrstd,
                         void* workspace, void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_group_timestep_norm_fwd: bad dtype %d", dtype);
  int rc = check_dims("mega_group_timestep_norm_fwd", B, L, D, G);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG(x && prev_count && prev_mean && prev_var && gamma && beta && y && count && mean &&
                     var && cummean && cumrstd && workspace,
                 "mega_group_timestep_norm_fwd: null pointer");
  if (B == 0) return MEGA_OK;
  TsnParams p{};
  p.x = x; p.gamma = gamma; p.beta = beta; p.mask = padding_mask; p.prev_count = prev_count;
  p.prev_mean = prev_mean; p.prev_var = prev_var; p.y = y; p.count = count; p.mean = mean;
  p.var = var; p.cummean = cummean; p.cumrstd = cumrstd;
  p.B = (int)B; p.L = (int)L; p.D = (int)D; p.G = (int)G; p.Dg = (int)(D / G);
  p.NT = (int)((L + kTL - 1) / kTL); p.eps = (float)eps;
  set_stat_strides(p, time_last);
  hipStream_t s = static_cast<hipStream_t>(stream);
  MEGA_CHECK_ARG(L >= 1, "mega_group_timestep_norm_fwd: empty sequence");
  switch (dtype) {
    case MEGA_F32: return tsn_fwd_impl<MEGA_F32>(p, workspace, s);
    case MEGA_BF16: return tsn_fwd_impl<MEGA_BF16>(p, workspace, s);
    default: return tsn_fwd_impl<MEGA_F16>(p, workspace, s);
  }
}

extern "C" int mega_group_timestep_norm_fwd(const void* x, int dtype, const int64_t* prev_count,
                                            const void* prev_mean, const void* prev_var,
                                            const void* gamma, const void* beta,
                                            const uint8_t* padding_mask, int64_t B, int64_t L,
                                            int64_t D, int64_t G, double eps, void* y,
                                            int64_t* count, void* mean, void* var, float* cummean,
                                            float* cumrstd, void* workspace, void* stream) {
  return tsn_fwd_entry(false, x, dtype, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, B, L, D, G,
                       eps, y, count, mean, var, cummean, cumrstd, workspace, stream);
}

extern "C" int mega_group_timestep_norm_fwd_tl(const void* x, int dtype, const int64_t* prev_count,
                                               const void* prev_mean, const void* prev_var,
                                               const void* gamma, const void* beta,
                                               const uint8_t* padding_mask, int64_t B, int64_t L,
                                               int64_t D, int64_t G, double eps, void* y,
                                               int64_t* count, void* mean, void* var, float* cummean,
                                               float* cumrstd, void* workspace, void* stream) {
  return tsn_fwd_entry(true, x, dtype, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, B, L, D, G,
                       eps, y, count, mean, var, cummean, cumrstd, workspace, stream);
}

static int tsn_bwd_entry(bool time_last, const void* dy, const void* dmean, const void* dvar, const void* x,
                         int dtype, const void* prev_mean, const int64_t* count, const float* cummean,
                         const float* cumrstd, const void* gamma, const uint8_t* padding_mask, int64_t B,
                         int64_t L, int64_t D, int64_t G, void* dx, void* dprev_mean, void* dprev_var,
                         void* dgamma, void* dbeta, void* workspace, void* stream) {
  MEGA_CHECK_ARG(valid_dtype(dtype), "mega_group_timestep_norm_bwd: bad dtype %d", dtype);
  int rc = check_dims("mega_group_timestep_norm_bwd", B, L, D, G);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG(dy && dmean && dvar && x && prev_mean && count && cummean && cumrstd && gamma &&
                     dx && dprev_mean && dprev_var && dgamma && dbeta && workspace,
                 "mega_group_timestep_norm_bwd: null pointer");
  MEGA_CHECK_ARG(B >= 1 && L >= 1, "mega_group_timestep_norm_bwd: empty input");
  TsnParams p{};
  p.x = x; p.dy = dy; p.gamma = gamma; p.mask = padding_mask; p.prev_count = count;
  p.prev_mean = prev_mean; p.dmean = dmean; p.dvar = dvar; p.cummean_in = cummean;
  p.cumrstd_in = cumrstd; p.y = dx; p.mean = dprev_mean; p.var = dprev_var;
  p.B = (int)B; p.L = (int)L; p.D = (int)D; p.G = (int)G; p.Dg = (int)(D / G);
  p.NT = (int)((L + kTL - 1) / kTL);
  set_stat_strides(p, time_last);
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MEGA_F32: return tsn_bwd_impl<MEGA_F32>(p, dgamma, dbeta, workspace, s);
    case MEGA_BF16: return tsn_bwd_impl<MEGA_BF16>(p, dgamma, dbeta, workspace, s);
    default: return tsn_bwd_impl<MEGA_F16>(p, dgamma, dbeta, workspace, s);
  }
}

extern "C" int mega_group_timestep_norm_bwd(const void* dy, const void* dmean, const void* dvar,
                                            const void* x, int dtype, const void* prev_mean,
                                            const int64_t* count, const float* cummean,
                                            const float* cumrstd, const void* gamma,
                                            const uint8_t* padding_mask, int64_t B, int64_t L,
                                            int64_t D, int64_t G, void* dx, void* dprev_mean,
                                            void* dprev_var, void* dgamma, void* dbeta,
                                            void* workspace, void* stream) {
  return tsn_bwd_entry(false, dy, dmean, dvar, x, dtype, prev_mean, count, cummean, cumrstd, gamma, padding_mask,
                       B, L, D, G, dx, dprev_mean, dprev_var, dgamma, dbeta, workspace, stream);
}

extern "C" int mega_group_timestep_norm_bwd_tl(const void* dy, const void* dmean, const void* dvar,
                                               const void* x, int dtype, const void* prev_mean,
                                               const int64_t* count, const float* cummean,
                                               const float* cumrstd, const void* gamma,
                                               const uint8_t* padding_mask, int64_t B, int64_t L,
                                               int64_t D, int64_t G, void* dx, void* dprev_mean,
                                               void* dprev_var, void* dgamma, void* dbeta,
                                               void* workspace, void* stream) {
  return tsn_bwd_entry(true, dy, dmean, dvar, x, dtype, prev_mean, count, cummean, cumrstd, gamma, padding_mask,
                       B, L, D, G, dx, dprev_mean, dprev_var, dgamma, dbeta, workspace, stream);
}

// Test hook: look-back poll limit (<= 0 restores the default) and a tile index
// that publishes no record (-1: none) for the launches that follow.
extern "C" void mega_test_timestep_norm_lookback(long long spin_limit, int mute_tile) {
  g_spin_limit.store(spin_limit > 0 ? spin_limit : kDefaultSpinLimit);
  g_mute_tile.store(mute_tile);
}

// ---- forward without a caller workspace: a static device buffer ---------------------
// Callers that may not allocate (graph capture, serving loops) get the
// forward's scratch (tickets, per-tile counts, look-back records) from a
// file-scope device array instead of a workspace argument.  Each GPU holds its
// own copy of the array until the process ends; `scratch` itself is only the
// host-side name of the symbol, so its device address is looked up once per
// device and that pointer is what the kernels receive.
constexpr int64_t kStaticScratchBytes = 2 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kScratchDevices = 64;
void* g_scratch_ptr[kScratchDevices] = {};
std::mutex g_scratch_mu;

int static_scratch(void** out) {
  int dev = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_ARG(dev >= 0 && dev < kScratchDevices, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    MEGA_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MEGA_OK;
}
}  // namespace

// Status of the last fast-path launch that used `workspace`: waits for the
// stream, reads the launch's status word and returns MEGA_OK, or
// MEGA_ERR_TIMEOUT when a look-back wait was given up (the outputs that
// depended on the missing record are NaN).  The serial kernels never wait.
// A null `workspace` means the static buffer of mega_group_timestep_norm_fwd_static
// on the current device.
extern "C" int mega_group_timestep_norm_status(const void* workspace, void* stream) {
  if (workspace == nullptr) {
    void* ptr = nullptr;
    const int rc = static_scratch(&ptr);
    if (rc != MEGA_OK) return rc;
    workspace = ptr;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  unsigned int word = 0;
  MEGA_CHECK_HIP(hipMemcpyAsync(&word, static_cast<const int*>(workspace) + kStatusSlot, sizeof(word),
                                hipMemcpyDeviceToHost, s));
  MEGA_CHECK_HIP(hipStreamSynchronize(s));
  if (word & kStatusGaveUp)
    return set_error(MEGA_ERR_TIMEOUT,
                     "TimestepNorm: a tile gave up waiting for an earlier tile's record after %lld polls; "
                     "the outputs that depend on it are NaN",
                     g_spin_limit.load());
  return MEGA_OK;
}

extern "C" int64_t mega_group_timestep_norm_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int mega_group_timestep_norm_fwd_static(const void* x, int dtype, const int64_t* prev_count,
                                                   const void* prev_mean, const void* prev_var,
                                                   const void* gamma, const void* beta,
                                                   const uint8_t* padding_mask, int64_t B, int64_t L,
                                                   int64_t D, int64_t G, double eps, void* y,
                                                   int64_t* count, void* mean, void* var,
                                                   float* cummean, float* cumrstd, void* stream) {
  int rc = check_dims("mega_group_timestep_norm_fwd_static", B, L, D, G);
  if (rc != MEGA_OK) return rc;
  const int64_t need = mega_group_timestep_norm_workspace_bytes(B, L, D, G, 0);
  if (need > kStaticScratchBytes)
    return set_error(MEGA_ERR_UNSUPPORTED,
                     "mega_group_timestep_norm_fwd_static: this shape needs %lld bytes of scratch, the static "
                     "buffer holds %lld; use mega_group_timestep_norm_fwd with a workspace",
                     (long long)need, (long long)kStaticScratchBytes);
  void* ptr = nullptr;
  rc = static_scratch(&ptr);
  if (rc != MEGA_OK) return rc;
  return mega_group_timestep_norm_fwd(x, dtype, prev_count, prev_mean, prev_var, gamma, beta, padding_mask,
                                      B, L, D, G, eps, y, count, mean, var, cummean, cumrstd, ptr, stream);
}
