// Scores and softmax of the chunk attention in one kernel (bf16 / fp16 on MFMA).
//
// What it computes is the first half of the reference's forward
//   megalodon/csrc/ops/attention_kernel.cu:78-98 (S = scale Q K^T) and
//   megalodon/csrc/softmax.cuh:86-131 (P = causal softmax of S in float32):
// w[z][r][c] = P[r][c] for the keys c <= r + (L2 - L1) of query row r, zero for the other keys
// it writes.  The reference stores S in the element type and reads it back for the softmax;
// here S never leaves the registers (the scores enter the exponential in float32), so the
// triangle of S is neither written nor re-read: the only HBM traffic is Q, K and P.
//
// Shape of the kernel.  A workgroup of eight waves owns 256 query rows of one (batch, head);
// wave v holds its 32 rows of Q as MFMA operands in registers for the whole kernel
// (H1 / 16 fragments).  The keys pass by in tiles of 64: K tiles are sent from memory straight
// into an LDS ring of eight slabs (`global_load_lds_dwordx4`, six to seven slabs in flight), every wave
// reads the same key fragments and multiplies them with its own rows, so a wave's accumulators
// are 32 rows x 64 keys and a row lives in two lanes (l, l + 32), 16 keys of a 32-key block
// each.  The softmax needs a row's maximum and sum before the first probability can be written,
// so the tiles are walked twice:
//   pass 1, keys ascending:  per lane a running (max, sum of exp) over its own columns -- no
//                            cross-lane traffic at all; the two lanes of a row are merged once
//                            at the end of the pass;
//   pass 2, keys descending: the tile is computed again (K = H1 is short: the product is an
//                            eighth of P V), p = exp(s - max) / sum is rounded to the element
//                            type, the two lane halves swap register pairs so that a lane holds
//                            8 consecutive keys, and the tile leaves in 16-byte stores.
// The vector work of a tile (about six issue slots per score and pass, four of them the
// quarter-rate exponential) costs as much as its matrix work, so the two are overlapped inside
// each wave: there are two accumulator sets, and while the products of tile t fill one set the
// wave works through the finished tile t - 1 in the other, one 32-key block per slab, a piece
// of it per k-step.
// Measured on the way (8 chunks x 4 heads, 4096 x 4096, head width 256; this kernel 0.31 ms
// against 0.27 + 0.23 ms for product and softmax as two kernels).  With parts switched off
// (timing only): no stores 0.27 ms, neither barrier nor slab requests 0.26 ms, neither of the
// two 0.24 ms -- the products and the passes themselves, at the clock the part sustains with
// every matrix pipe busy; a quarter of the (batch, head) pairs, half the compute units idle,
// runs the same code a quarter faster per row block.  A wave's `s_waitcnt vmcnt` counts its
// stores of P with its slab requests, so the waits for slabs also wait for stores; letting four
// waves request for all eight changed nothing.  The same tile staged through LDS and stored as
// whole lines was slower (0.38 ms), non-temporal stores of the 32-byte pieces three times
// slower; four waves per workgroup and two workgroups per compute unit 0.33 ms; taking the
// (batch, head) pairs of an XCD two at a time instead of all at once 0.33 -> 0.31 ms.
// On this part an MFMA of this shape holds the matrix pipe for 32 clocks and its wave's issue
// for about 14; beside it a SIMD issues six ordinary vector instructions (v_exp_f32 counts
// two) per MFMA before the vector port, not the matrix pipe, sets the pace.
#include "common.hpp"

#include <type_traits>

namespace mega {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ floatx16 mma16(u32x4 a, u32x4 b, floatx16 c) {
  if constexpr (DT == MEGA_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DT == MEGA_BF16) return pack_bf16x2(lo, hi);
  return static_cast<uint32_t>(float_to_f16_bits(lo)) | (static_cast<uint32_t>(float_to_f16_bits(hi)) << 16);
}

// a <-> b between the two halves of the wave (v_permlane32_swap_b32): afterwards the low half
// holds (its own a, the high half's a), the high half (the low half's b, its own b).  The
// operands must come out of ordinary vector instructions (not straight out of an MFMA); the
// s_nop covers the wait states after a vector write of an operand.
__device__ __forceinline__ void half_swap(uint32_t& a, uint32_t& b) {
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void half_swap(float& a, float& b) {
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}

// One request: lane l's 16 bytes at base + offset go to LDS bytes lds_dst + 16 l .. + 15
// (lds_dst wave-uniform, in M0).  Assembly, so that the compiler does not see a vector memory
// instruction that writes LDS (it would wait for every request in flight in front of each LDS
// read); the waits for these requests are the explicit `s_waitcnt vmcnt` below.
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t offset, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(offset), "s"(base), "s"(lds_dst));
}

constexpr int kWaves = 8;                    // waves of a workgroup (two per SIMD)
constexpr int kRows = 32 * kWaves;           // query rows of a workgroup
constexpr int kKeys = 64;                    // keys of a tile
constexpr int kRing = 8;                     // slab buffers in LDS (128 KB at head width 128 and 256)

struct ProbsParams {
  const uint16_t* q;
  const uint16_t* k;
  uint16_t* w;
  int L1, L2, NH, Z, MT;
  int causal, off;
  int fill;  // also write zeros from the last tile to the end of every row
  float sl;  // scale * log2(e)
};

enum { kStats = 0, kWrite = 1 };

template <int DT, int H1>
__global__ __launch_bounds__(64 * kWaves) void attn_probs_kernel(const ProbsParams p) {
  constexpr int KW = H1 >= 128 ? 128 : 64;  // k values of a slab
  constexpr int NS = H1 / KW;               // slabs of a tile
  constexpr int KST = KW / 16;              // MFMA k-steps of a slab
  constexpr int QF = H1 / 16;               // fragments of a row of Q
  constexpr int CPR = KW / 8;               // 16-byte chunks of a slab row
  constexpr int RPP = 1024 / (KW * 2);      // slab rows in a 1 KB piece
  constexpr int PPW = kKeys / RPP / kWaves; // pieces of a slab a wave requests
  constexpr int SLAB = kKeys * KW;          // elements of a slab
  static_assert(NS == 1 || NS == 2, "one or two slabs per tile");
  static_assert(KST % 4 == 0 && PPW >= 1, "four fragment sets, reused every four k-steps");
  extern __shared__ __align__(16) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform for the compiler too
  const int r = lane & 31, h = lane >> 5;

  // work item: heavy row blocks first (a block's work grows with its index).  With a multiple of
  // eight (batch, head) pairs each XCD keeps its own pairs and takes them two at a time, so that the
  // K of the workgroups running together (2 MB per pair at 4096 keys of 256) fits its 4 MB L2;
  // the heavy blocks of the next two pairs fall to the units the light blocks of these two free.
  int z, mt;
  {
    const int idx = static_cast<int>(blockIdx.x);
    if (p.Z % 8 == 0) {
      const int zper = p.Z / 8, xcd = idx & 7, j = idx >> 3;
      const int gs = zper % 2 == 0 ? 2 : 1;
      const int g = j / (gs * p.MT), jj = j % (gs * p.MT);
      mt = p.MT - 1 - jj / gs;
      z = xcd * zper + g * gs + jj % gs;
    } else {
      mt = p.MT - 1 - idx / p.Z;
      z = idx % p.Z;
    }
  }
  const int b = z / p.NH, hd = z % p.NH;
  const int m0 = mt * kRows, r0 = m0 + 32 * wave, row = r0 + r;
  const int ld = p.NH * H1;
  const uint16_t* Q = p.q + (static_cast<int64_t>(b) * p.L1) * ld + hd * H1;
  const uint16_t* K = p.k + (static_cast<int64_t>(b) * p.L2) * ld + hd * H1;

  // the wave's rows of Q: lane (r, h) holds row r0 + r, k = 16 f + 8 h .. + 7 of fragment f
  u32x4 qf[QF];
  {
    const uint16_t* qr = Q + static_cast<int64_t>(min(row, p.L1 - 1)) * ld + 8 * h;
#pragma unroll
    for (int f = 0; f < QF; ++f) qf[f] = *reinterpret_cast<const u32x4*>(qr + 16 * f);
  }

  const int rows_end = min(m0 + kRows, p.L1);
  const int kend = p.causal ? min(p.L2, rows_end + p.off) : p.L2;  // keys the block's rows can see
  const int nb = (kend + kKeys - 1) / kKeys;                       // tiles of a pass
  const int ntile = 2 * nb, nslab = ntile * NS;
  const int lim_row = p.causal ? min(row + p.off, p.L2 - 1) : p.L2 - 1;   // last key of this lane's row
  const int lim_wave = p.causal ? min(r0 + p.off, p.L2 - 1) : p.L2 - 1;  // ... of the wave's first row
  const bool rows_full = r0 + 31 < p.L1;
  const auto tile_keys = [&](int t) { return (t < nb ? t : ntile - 1 - t) * kKeys; };

  // memory side: piece pc = wave + kWaves i of a slab is RPP rows; lane l of the piece fetches what
  // belongs at byte 16 l of it: row pc RPP + l / CPR, position l % CPR, which holds k chunk
  // position ^ swizzle(row) (sixteen consecutive rows of one k chunk then cover sixteen
  // different 16-byte bank groups for the fragment reads)
  int drow[PPW], dcol[PPW];
#pragma unroll
  for (int i = 0; i < PPW; ++i) {
    const int rs = (wave + kWaves * i) * RPP + lane / CPR, pos = lane % CPR;
    const int sw = CPR == 16 ? (rs & 15) : ((rs >> 1) & 7);
    drow[i] = rs;
    dcol[i] = (pos ^ sw) * 16;  // bytes
  }
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)(smem))));
  // slab s of the stream (tile s / NS, k values (s % NS) KW .. + KW - 1) into buffer s % kRing;
  // slabs past the end ask for the last one again, so that every step issues the same requests
  const auto request = [&](int s) {
    const int sc = min(s, nslab - 1);
    const int c0 = tile_keys(sc / NS), k0 = (sc % NS) * KW;
    const uint32_t dst = lds0 + static_cast<uint32_t>((s % kRing) * SLAB * 2 + wave * 1024);
#pragma unroll
    for (int i = 0; i < PPW; ++i) {
      const int key = min(c0 + drow[i], p.L2 - 1);
      load_to_lds16(K, static_cast<uint32_t>(key * (ld * 2) + k0 * 2 + dcol[i]), dst + i * kWaves * 1024);
    }
  };

  // fragment side: k-step ks of a slab, key block j: lane (r, h) reads key row 32 j + r,
  // k chunk 2 ks + h, which sits at position (2 ks + h) ^ swizzle = ((h ^ swizzle) ^ 2 ks)
  const int sw_r = CPR == 16 ? (r & 15) : ((r >> 1) & 7);
  uint32_t fro[KST];  // byte offsets inside a slab
#pragma unroll
  for (int ks = 0; ks < KST; ++ks) fro[ks] = static_cast<uint32_t>(((r * KW + ((h ^ sw_r) * 8)) ^ (ks * 16)) * 2);
  const auto fread = [&](u32x4* f, uint32_t bufoff, int ks) {
    const char* base = reinterpret_cast<const char*>(smem) + (bufoff + fro[ks]);
    f[0] = *reinterpret_cast<const u32x4*>(base);
    f[1] = *reinterpret_cast<const u32x4*>(base + 32 * KW * 2);
  };

  floatx16 acc[2][2];  // [set][key block]
  u32x4 fr[4][2];      // fragment sets: k-step ks of a slab lives in set ks % 4
  float m = -1e30f, l = 0.f;   // this lane's running maximum (raw score) and sum of exp
  float nm = 0.f;              // pass 1: -(block max) * sl; after it: -(max * sl + log2(sum)) of the whole row
  uint16_t* wrow = p.w + (static_cast<int64_t>(z) * p.L1 + min(row, p.L1 - 1)) * p.L2;
  const bool row_ok = row < p.L1;

  // The pass over one 32-key block of a finished tile (16 scores per lane, element i = key
  // x0 + 8 (i / 4) + i % 4 of the tile) is a list of 17 small operations, cut into `nparts` pieces
  // that run beside the products, one piece per k-step:
  //   pass 1: operation 0 takes the block's maximum into the running one and rescales the running
  //           sum, operation 1 + i forms exp(s_i - max) and adds it up;
  //   pass 2: operation i turns score i into its probability (in place), operation 16 rounds them,
  //           swaps register pairs between the wave's halves so that a lane holds 8 consecutive
  //           keys, and stores 16 bytes per lane.
  const auto stats_part = [&](floatx16& a, int x0, auto mask_c, int lim, int part, int nparts) {
    constexpr bool MASK = decltype(mask_c)::value;
#pragma unroll
    for (int op = 0; op < 17; ++op) {
      if (op < part * 17 / nparts || op >= (part + 1) * 17 / nparts) continue;
      if (op == 0) {
        if constexpr (MASK) {
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (x0 + 8 * (i >> 2) + (i & 3) > lim) a[i] = -INFINITY;
        }
        float tm = m;
#pragma unroll
        for (int i = 0; i < 16; ++i) tm = fmaxf(tm, a[i]);
        l *= __builtin_amdgcn_exp2f((m - tm) * p.sl);
        m = tm;
        nm = -tm * p.sl;
      } else {
        // the sum runs two elements behind the exponentials, so that no addition waits for the
        // transcendental unit
        const int i = op - 1;
        a[i] = __builtin_amdgcn_exp2f(fmaf(a[i], p.sl, nm));
        if (i >= 2) l += a[i - 2];
        if (i == 15) l += a[14] + a[15];
      }
    }
  };
  const auto write_part = [&](floatx16& a, int x0, auto mask_c, int lim, int c0, int part, int nparts) {
    constexpr bool MASK = decltype(mask_c)::value;
#pragma unroll
    for (int op = 0; op < 17; ++op) {
      if (op < part * 17 / nparts || op >= (part + 1) * 17 / nparts) continue;
      if (op < 16) {
        float s = a[op];
        if constexpr (MASK)
          if (x0 + 8 * (op >> 2) + (op & 3) > lim) s = -INFINITY;
        a[op] = __builtin_amdgcn_exp2f(fmaf(s, p.sl, nm));
      } else {
        uint32_t px[4], py[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          px[g] = pack2<DT>(a[4 * g], a[4 * g + 1]);
          py[g] = pack2<DT>(a[4 * g + 2], a[4 * g + 3]);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          half_swap(px[2 * u], px[2 * u + 1]);
          half_swap(py[2 * u], py[2 * u + 1]);
          const u32x4 o = {px[2 * u], py[2 * u], px[2 * u + 1], py[2 * u + 1]};
          const int col = c0 + x0 + 16 * u + 8 * h;
          if (!MASK || (row_ok && col < p.L2)) *reinterpret_cast<u32x4*>(wrow + col) = o;
        }
      }
    }
  };

  // One tile: NS slab steps of products into set SET while the finished tile in the other set goes
  // through its pass (KIND).  A slab step starts with the barrier: this wave's pieces of the slab
  // have landed (the requests of the kRing - 2 slabs behind it may still be in flight) and every
  // wave has read the slab before to its end, so that buffer takes the request for the slab
  // kRing - 1 ahead.  What a wave has read it need not have multiplied: the products of a slab's
  // last two k-steps run after the barrier, under the latency of the first fragment reads of the
  // new slab, so a step is the k-steps KST - 2, KST - 1 of the slab before and 0 .. KST - 3 of its
  // own (at a tile's first step the two old k-steps complete the tile before, whose pass therefore
  // starts with the third).  Fragments are read four k-steps ahead of their products into four
  // register sets.  Every k-step is a scheduling region of its own, in the order
  //   MFMA / half of the pass's piece / MFMA / the other half / the fragment reads:
  // a wave issues in order, an MFMA holds the matrix pipe for 32 clocks while the wave goes on, so
  // the vector work runs in the shadow of the products.  (Left to itself the compiler put every
  // fragment read directly in front of the MFMA that needs it, a full LDS latency per product.)
#define MEGA_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
  const auto tile = [&](auto set_c, auto kind_c, auto mask_c, int s0, int c0p, int limp) {
    constexpr int SET = decltype(set_c)::value;
    constexpr int KIND = decltype(kind_c)::value;
#pragma unroll
    for (int ss = 0; ss < NS; ++ss) {
      const int s = s0 + ss;
      const uint32_t bufoff = static_cast<uint32_t>((s % kRing) * SLAB * 2);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((kRing - 2) * PPW) : "memory");
      request(s + kRing - 1);
      fread(fr[0], bufoff, 0);
      fread(fr[1], bufoff, 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < KST; ++i) {
        // the k-step of this slot: an old one of the slab before (i < 2) or k-step i - 2 of this slab
        const int ks = i < 2 ? KST - 2 + i : i - 2;
        const int sq = i < 2 ? (ss + NS - 1) % NS : ss;     // which slab of its tile the k-step belongs to
        constexpr int cur = SET;
        if (i < 2 && ss == 0) {
          acc[cur ^ 1][0] = mma16<DT>(fr[ks & 3][0], qf[sq * KST + ks], acc[cur ^ 1][0]);
          acc[cur ^ 1][1] = mma16<DT>(fr[ks & 3][1], qf[sq * KST + ks], acc[cur ^ 1][1]);
        } else {
          if (i == 2 && ss == 0) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[cur][j][e] = 0.f;
          }
          acc[cur][0] = mma16<DT>(fr[ks & 3][0], qf[sq * KST + ks], acc[cur][0]);
          acc[cur][1] = mma16<DT>(fr[ks & 3][1], qf[sq * KST + ks], acc[cur][1]);
        }
        // the piece of the other tile's pass that goes with this slot
        int jb = -1, part = 0, nparts = 1;
        if (NS == 2) {
          if (ss == 0 && i >= 2) jb = 0, part = i - 2, nparts = KST - 2;
          if (ss == 1) jb = 1, part = i, nparts = KST;
        } else if (i >= 2) {
          constexpr int half = (KST - 2) / 2;
          jb = (i - 2) / half, part = (i - 2) % half, nparts = half;
        }
        if (jb >= 0) {
          if constexpr (KIND == kStats) stats_part(acc[cur ^ 1][jb], 32 * jb, mask_c, limp, part, nparts);
          else write_part(acc[cur ^ 1][jb], 32 * jb, mask_c, limp, c0p, part, nparts);
        }
        if (i + 2 < KST) fread(fr[(i + 2) & 3], bufoff, i + 2);
        MEGA_SGB(0x008, 1);
        MEGA_SGB(0x402, 4);
        MEGA_SGB(0x008, 1);
        MEGA_SGB(0x402, 8);
        MEGA_SGB(0x100, 2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using std::integral_constant;
  const auto run = [&](auto set_c, int t) {
    const int tp = t - 1;
    const int c0p = tp < 0 ? 0 : tile_keys(tp);
    const int limp = tp < 0 ? -1 : lim_row - c0p - 4 * h;
    const bool mask = tp < 0 || !(rows_full && c0p + kKeys - 1 <= lim_wave);
    const bool stats = tp < nb;
    if (stats) {
      if (mask) tile(set_c, integral_constant<int, kStats>{}, std::true_type{}, t * NS, c0p, limp);
      else tile(set_c, integral_constant<int, kStats>{}, std::false_type{}, t * NS, c0p, limp);
    } else {
      if (mask) tile(set_c, integral_constant<int, kWrite>{}, std::true_type{}, t * NS, c0p, limp);
      else tile(set_c, integral_constant<int, kWrite>{}, std::false_type{}, t * NS, c0p, limp);
    }
    if (t == nb) {
      // pass 1 is complete (its last tile went through during tile nb): merge the two lanes of a row
      float ma = m, mb = m + 0.f, la = l, lb = l + 0.f;
      half_swap(ma, mb);
      half_swap(la, lb);
      const float mx = fmaxf(ma, mb);
      const float lt = la * __builtin_amdgcn_exp2f((ma - mx) * p.sl) + lb * __builtin_amdgcn_exp2f((mb - mx) * p.sl);
      nm = -mx * p.sl - __builtin_amdgcn_logf(lt);  // v_log_f32 is log2; a row always sees key 0, so lt >= 1
    }
  };

#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[1][j][i] = 0.f;
  // the first step's two old k-steps multiply these into set 1, which the first pass piece masks out
  fr[2][0] = fr[2][1] = fr[3][0] = fr[3][1] = u32x4{0u, 0u, 0u, 0u};
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // Q is in: from here on vmcnt counts slab requests
  for (int s = 0; s < kRing - 1; ++s) request(s);
  for (int t = 0; t < ntile; t += 2) {
    run(integral_constant<int, 0>{}, t);
    run(integral_constant<int, 1>{}, t + 1);
  }
  // the last tile of pass 2 (keys 0 .. 63, in set 1): its last two k-steps, then its pass
  {
#pragma unroll
    for (int ks = KST - 2; ks < KST; ++ks) {
      acc[1][0] = mma16<DT>(fr[ks & 3][0], qf[(NS - 1) * KST + ks], acc[1][0]);
      acc[1][1] = mma16<DT>(fr[ks & 3][1], qf[(NS - 1) * KST + ks], acc[1][1]);
    }
    const int limp = lim_row - 4 * h;
    write_part(acc[1][0], 0, std::true_type{}, limp, 0, 0, 1);
    write_part(acc[1][1], 32, std::true_type{}, limp, 0, 0, 1);
  }
  {
    // zeros behind the last tile: to the end of the row with `fill`, else as far as the products that
    // read P in 256-row tiles go (the last key the 256-row block of this row block can see)
    const int zend = (p.fill || !p.causal) ? p.L2 : min(p.L2, (m0 / 256 + 1) * 256 + p.off);
    const u32x4 zero = {0u, 0u, 0u, 0u};
    if (nb * kKeys < zend) {
      for (int rr = 0; rr < 32 && r0 + rr < p.L1; ++rr) {
        uint16_t* dst = p.w + (static_cast<int64_t>(z) * p.L1 + r0 + rr) * p.L2;
        // whole lines, not read by this kernel: non-temporal (forward with full rows 1.312 -> 1.291 ms)
        for (int c = nb * kKeys + lane * 8; c < zend; c += 64 * 8) __builtin_nontemporal_store(zero, reinterpret_cast<u32x4*>(dst + c));
      }
    }
  }
  // nothing may land in the LDS of a workgroup that has ended
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#undef MEGA_SGB
}

template <int DT, int H1>
int launch_probs(const ProbsParams& p, hipStream_t s) {
  constexpr int KW = H1 >= 128 ? 128 : 64;
  const size_t lds = sizeof(uint16_t) * kRing * kKeys * KW;
  MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_probs_kernel<DT, H1>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  attn_probs_kernel<DT, H1><<<dim3(static_cast<unsigned>(p.Z * p.MT)), 64 * kWaves, lds, s>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace

// w = causal softmax of scale q k^T for 16-bit q (B, L1, NH, H1), k (B, L2, NH, H1), w (B, NH, L1, L2).
// Returns MEGA_OK, an error, or -1 when the shape is outside this kernel (the caller then runs the
// product, softmax and zero fill as separate kernels): head widths other than 64, 128, 256, key
// counts that are not a multiple of 8, operands that are not 16-byte aligned, scale <= 0.
// With `causal`, row r is written up to the end of the 64-key tile that holds the last key of the
// row block (256 rows) it belongs to, with zeros behind its own last key; `fill` writes the zeros
// up to the end of the row as well (always done when L2 > L1, where the backward products of the
// operator read them).
int attention_probs_fused(int dtype, const uint16_t* q, const uint16_t* k, uint16_t* w, int64_t B, int64_t L1,
                          int64_t L2, int64_t NH, int64_t H1, float scale, int causal, int fill, hipStream_t s) {
  const auto a16 = [](const void* x) { return reinterpret_cast<uintptr_t>(x) % 16 == 0; };
  if (!(H1 == 64 || H1 == 128 || H1 == 256) || L2 % 8 != 0 || !a16(q) || !a16(k) || !a16(w)) return -1;
  if (!(scale > 0.f) || !(scale < 1e30f)) return -1;
  const int64_t MT = (L1 + kRows - 1) / kRows;
  if (L2 * NH * H1 >= (1ll << 30) || B * NH * MT >= (1ll << 31) || L1 < 1 || L2 < 1) return -1;
  ProbsParams p{};
  p.q = q; p.k = k; p.w = w;
  p.L1 = (int)L1; p.L2 = (int)L2; p.NH = (int)NH; p.Z = (int)(B * NH); p.MT = (int)MT;
  p.causal = causal ? 1 : 0;
  p.off = causal ? (int)(L2 - L1) : 0;
  p.fill = (causal && (fill || L2 > L1)) ? 1 : 0;
  p.sl = scale * 1.4426950408889634f;
#define MEGA_PROBS(DT)                                   \
  switch (H1) {                                          \
    case 64: return launch_probs<DT, 64>(p, s);          \
    case 128: return launch_probs<DT, 128>(p, s);        \
    default: return launch_probs<DT, 256>(p, s);         \
  }
  if (dtype == MEGA_BF16) { MEGA_PROBS(MEGA_BF16) }
  if (dtype == MEGA_F16) { MEGA_PROBS(MEGA_F16) }
#undef MEGA_PROBS
  return -1;
}

}  // namespace mega
