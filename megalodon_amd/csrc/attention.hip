// Chunk-causal attention for gfx950 (bf16 / fp16, fp32 accumulation on MFMA).
//
// Semantics follow the reference operator
//   megalodon/csrc/ops/attention_kernel.cu:40-133 (forward), :135-257 (backward)
//   megalodon/csrc/softmax.cuh:86-131,198-234 (causal softmax forward / backward):
//   S = scale * Q K^T rounded to the element type, P = softmax_fp32(S) over the
//   causal prefix (row r sees columns 0..L2-L1+r), P stored in the element type,
//   Y = P V;  dV = P^T dY, dP = dY V^T, dS = P o (dP - rowsum(P o dP)),
//   dQ = scale dS K, dK = scale dS^T Q.  Layout BLNH in and out; w = P is
//   returned (B, N, L1, L2) as the reference does.
//
// Differences in execution: the reference runs full-square cuBLAS GEMMs and a
// full-row softmax; here every product is one hand-written MFMA GEMM
// (v_mfma_f32_32x32x16, 256x256 workgroup tile, eight wavefronts of 128x64,
// double-buffered LDS staging of 32-wide k slabs) that skips the tiles above
// the causal diagonal and the k-ranges where P / dS are structurally zero, so
// causal attention costs half the flops and half the P traffic.  Operands whose
// reduction index is not the contiguous one (V, dY, K, Q, P, dS in the
// backward products) are staged k-major in LDS and read with the transposing
// LDS read, which hands each lane the 8 consecutive k an MFMA operand wants.
// A key/value prefix (L2 > L1, cached keys in front of the chunk) shifts the
// diagonal by L2 - L1 columns in every one of these rules.
#include "common.hpp"
#include "dropkey.hpp"

#include <algorithm>

namespace mega {

// float32 / float64 tensors: attention_f32.hip
template <typename T>
int attention_wide_fwd(const T* q, const T* k, const T* v, int64_t B, int64_t L1, int64_t L2,
                       int64_t NH, int64_t H1, int64_t H2, double scale, int causal, const DropKey* drop,
                       T* y, T* w, hipStream_t s);
template <typename T>
int attention_wide_bwd(const T* dy, const T* q, const T* k, const T* v, const T* w,
                       int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2, double scale,
                       int causal, T* dq, T* dk, T* dv, T* dp, hipStream_t s);
template <typename T>
int softmax_wide_fwd(T* x, int64_t Z, int64_t L1, int64_t L2, int causal, const DropKey* drop, hipStream_t s);
template <typename T>
int softmax_wide_bwd(const T* y, T* dy, int64_t Z, int64_t L1, int64_t L2, int causal, hipStream_t s);
// scores + softmax in one kernel (attention_scores.hip); -1: shape outside that kernel
int attention_probs_fused(int dtype, const uint16_t* q, const uint16_t* k, uint16_t* w, int64_t B, int64_t L1,
                          int64_t L2, int64_t NH, int64_t H1, float scale, int causal, int fill, hipStream_t s);

namespace {

constexpr int kTile = 256;     // workgroup tile (M and N)
constexpr int kSlab = 32;      // k elements staged per iteration
// LDS slab layout: 16-byte chunks (8 k values of one row), chunk (c, row) at
// index c * kChunkPitch + row.  A fragment read then has consecutive lanes on
// consecutive chunks.  16-byte LDS accesses go eight lanes at a time over 32
// banks (measured: a pitch of 260 chunks left a third of the LDS cycles as bank
// conflicts, 264 was worse, 258 leaves 3 %): the 4 (c) x 2 (row) chunks that
// eight neighbouring lanes write must differ mod 8, so the pitch is 2 mod 8.
constexpr int kChunkPitch = kTile + 2;
// k-major operands keep their rows of k: 256 + 32 elements per row, so that the
// four rows a transposing read touches start 16 banks apart.
constexpr int kPitchT = kTile + 32;
constexpr int kOperandElems = kSlab * kPitchT;  // elements per operand slab (either layout fits)
static_assert((kSlab / 8) * kChunkPitch * 8 <= kOperandElems, "chunk layout must fit");
constexpr int kThreads = 256;
constexpr int kXcds = 8;       // accelerator dies, each with a private L2
constexpr int kRing = 3;       // slabs in flight in registers (prefetch distance)
constexpr int kEpiPitch = 128 + 8;  // epilogue staging pitch (elements) of a wave's 128x128 tile (4-wave form)
constexpr size_t kGemmLds =
    sizeof(uint16_t) * (4 * 128 * kEpiPitch > 2 * 2 * kOperandElems ? 4 * 128 * kEpiPitch
                                                                     : 2 * 2 * kOperandElems);

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// native 16-byte vector: loads and stores of it are typed, so register arrays
// of it are promoted out of memory
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int DT> struct Mma;
template <> struct Mma<MEGA_BF16> {
  static __device__ __forceinline__ floatx16 run(u32x4 a, u32x4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<MEGA_F16> {
  static __device__ __forceinline__ floatx16 run(u32x4 a, u32x4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

// C[m][n] = alpha * sum_k A(m, k) B(n, k); element (m, k) of an operand sits at
// [m * ld + k], or at [k * ld + m] when the operand is flagged k-major
struct GemmParams {
  const uint16_t* A;
  const uint16_t* B;
  uint16_t* C;
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t sa0, sa1, sb0, sb1, sc0, sc1;  // batch z = z0 * nh + z1 -> offset z0*s0 + z1*s1
  int nh;
  float alpha;
  // Causal structure with rows = queries r, columns = keys c, c <= r + off
  // (off = L2 - L1 >= 0, the length of a key/value prefix):
  int tri_out;  // 1: tiles wholly above that diagonal are skipped (left unwritten)
  int k_mode;   // 0: all k; 1: m = queries, k = keys: k < (mt+1)*256 + off, rounded up to a slab;
                // 2: m = keys, k = queries: k >= mt*256 - off, rounded down to a slab
  int off;
  // persistent schedule (filled in by the launcher): work items of equal weight,
  // walked by gridDim.x workgroups
  int mt_count, nt_count;  // tiles along m and n
  int per_batch;           // work items per batch index
  int items;               // per_batch * batch
  int ta, tb;   // operand is k-major: element (m, k) at [k * ld + m]
  int n_group;  // plain schedule: tiles numbered n fastest inside bands of n_group column tiles, then m,
                // then band (0: one band) -- the 32 tiles an XCD works on at a time then share fewer
                // distinct operand blocks (4 x 8 instead of 2 x 16 of a 16-column problem)
};

template <bool ALIGNED>
__device__ __forceinline__ u32x4 load_chunk(const uint16_t* base, int64_t ld, int row, int rows,
                                            int k, int kend) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if (row < rows && k < kend) {
    const uint16_t* p = base + static_cast<int64_t>(row) * ld + k;
    if (ALIGNED && k + 8 <= kend) {
      v = *reinterpret_cast<const u32x4*>(p);
    } else {
      uint16_t t[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) t[e] = (k + e < kend) ? p[e] : static_cast<uint16_t>(0);
      v.x = t[0] | (static_cast<uint32_t>(t[1]) << 16);
      v.y = t[2] | (static_cast<uint32_t>(t[3]) << 16);
      v.z = t[4] | (static_cast<uint32_t>(t[5]) << 16);
      v.w = t[6] | (static_cast<uint32_t>(t[7]) << 16);
    }
  }
  return v;
}

// Workgroup barrier that waits for this wave's LDS traffic only, so global
// loads of later slabs stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Transposing LDS read (gfx950 ds_read_b64_tr_b16).  Inside each group of 16
// lanes, source lane 4a + b supplies 4 consecutive 16-bit elements s[4a+b][0..3]
// from its own address; destination lane 4b + c receives {s[4e + b][c]}, e =
// 0..3.  Pointing source lane 4a + b at row k0 + a, columns m0 + 4b .. + 3 of a
// k-major tile therefore hands lane t the column m0 + t at rows k0 .. k0 + 3:
// the k-contiguous quad an MFMA operand wants.
typedef short short4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_read_tr(const uint16_t* q) {
  const short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) short4v*)(q));
  return __builtin_bit_cast(uint2, v);
}

// C[m][n] = alpha * sum_k A(m, k) B(n, k).  An operand is either k-contiguous
// (rows m, `ld` between rows) or, with TA / TB, k-major (rows k, m contiguous).
// This is the form for operands of any alignment and extent: four waves of 128 x 128, slabs of
// 32 k through a ring of three register sets (bounds-checked element loads) and two LDS buffers.
// Aligned operands take the kernels below, whose slabs go from memory straight into LDS.
template <int DT, bool TA, bool TB>
__global__ __launch_bounds__(kThreads) void gemm_kernel(const GemmParams p) {
  extern __shared__ __align__(16) uint16_t smem[];
  // main loop: [buf][A|B] operand slabs; epilogue: [wave][128][pitch]
  constexpr int kOperand = kOperandElems;
  constexpr int T = kThreads;  // threads
  constexpr int JN = 4;        // 32-column blocks per wave
  constexpr int NL = 4;        // 16-byte chunks per thread, operand and slab
  constexpr int EP = kEpiPitch;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;

  // Persistent workgroups (one per CU) walk a list of work items of equal
  // weight, so nothing is launched for skipped tiles and no CU ends up with
  // the long tail of a triangular problem:
  //   tri_out: one item per tile on or below the (shifted) diagonal;
  //   k_mode:  one item = the tile pair (mt, mt_count - 1 - mt) of a column
  //            block, whose k ranges add up to the same length for every pair;
  //   else:    one item per tile.
  // Items are numbered n fastest, then m, then batch.  Workgroups are handed
  // to the 8 XCDs round-robin by index and each XCD has its own L2: an XCD
  // takes a contiguous eighth of the list and its workgroups interleave inside
  // it, so neighbours that share an A row block or the B matrix of a head hit
  // the same L2 at the same time.
  const int G = static_cast<int>(gridDim.x), lin = static_cast<int>(blockIdx.x);
  int it_lo, it_hi, it_step;
  if (G % kXcds == 0) {
    const int xcd = lin % kXcds;
    it_lo = static_cast<int>(static_cast<int64_t>(p.items) * xcd / kXcds) + lin / kXcds;
    it_hi = static_cast<int>(static_cast<int64_t>(p.items) * (xcd + 1) / kXcds);
    it_step = G / kXcds;
  } else {
    it_lo = lin;
    it_hi = p.items;
    it_step = G;
  }
  for (int item = it_lo; item < it_hi; item += it_step) {
  const int zz = item / p.per_batch;
  const int rem = item % p.per_batch;
  int nt, mt_first, mt_second = -1;
  if (p.tri_out) {
    // row mt holds the tiles nt <= (mt * 256 + 255 + off) / 256
    int t = rem, m = 0;
    while (true) {
      const int cnt = min(p.nt_count, (m * kTile + (kTile - 1) + p.off) / kTile + 1);
      if (t < cnt) break;
      t -= cnt;
      ++m;
    }
    mt_first = m;
    nt = t;
  } else if (p.k_mode) {
    nt = rem % p.nt_count;
    const int pr = rem / p.nt_count;
    mt_first = p.mt_count - 1 - pr;
    if (mt_first != pr) mt_second = pr;
  } else {
    nt = rem % p.nt_count;
    mt_first = rem / p.nt_count;
  }
  const int z0 = zz / p.nh, z1 = zz % p.nh;
  const uint16_t* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const uint16_t* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  uint16_t* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  for (int half = 0; half < 2; ++half) {
  const int mt = half == 0 ? mt_first : mt_second;
  if (mt < 0) break;
  const int m0 = mt * kTile, n0 = nt * kTile;
  int kb = 0, ke = p.K;
  if (p.k_mode == 1) ke = min(p.K, ((mt + 1) * kTile + p.off + kSlab - 1) / kSlab * kSlab);
  if (p.k_mode == 2) kb = min(p.K, max(0, mt * kTile - p.off) / kSlab * kSlab);
  const int nslab = (ke - kb + kSlab - 1) / kSlab;

  floatx16 acc[4][JN];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // register ring: slab s lives in ring slot s % 3 from its issue (three steps
  // before use) until it is written to LDS
  u32x4 ra0[NL], ra1[NL], ra2[NL], rb0[NL], rb1[NL], rb2[NL];

  // Global -> register chunk i of a thread (16 bytes), bounds-checked element loads:
  //   k-contiguous operand: row (tid >> 2) + T / 4 i, k chunk tid & 3
  //   k-major operand:      k row (tid >> 5) + T / 32 i, m chunk tid & 31
  auto gload = [&](u32x4* qa, u32x4* qb, int s) {
    const int k0 = kb + s * kSlab;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      if (TA) qa[i] = load_chunk<false>(A, p.lda, k0 + (tid >> 5) + (T / 32) * i, ke, m0 + (tid & 31) * 8, p.M);
      else qa[i] = load_chunk<false>(A, p.lda, m0 + (tid >> 2) + (T / 4) * i, p.M, k0 + (tid & 3) * 8, ke);
      if (TB) qb[i] = load_chunk<false>(B, p.ldb, k0 + (tid >> 5) + (T / 32) * i, ke, n0 + (tid & 31) * 8, p.N);
      else qb[i] = load_chunk<false>(B, p.ldb, n0 + (tid >> 2) + (T / 4) * i, p.N, k0 + (tid & 3) * 8, ke);
    }
  };
  // register -> LDS: chunk layout for k-contiguous operands, padded rows of k
  // for k-major ones
  const int st_a = TA ? (tid >> 5) * kPitchT + (tid & 31) * 8 : ((tid & 3) * kChunkPitch + (tid >> 2)) * 8;
  const int st_b = TB ? (tid >> 5) * kPitchT + (tid & 31) * 8 : ((tid & 3) * kChunkPitch + (tid >> 2)) * 8;
  auto sstore = [&](const u32x4* qa, const u32x4* qb, int s) {
    uint16_t* sa = smem + (s & 1) * 2 * kOperand + st_a;
    uint16_t* sb = smem + (s & 1) * 2 * kOperand + kOperand + st_b;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      *reinterpret_cast<u32x4*>(sa + i * (TA ? (T / 32) * kPitchT : (T / 4) * 8)) = qa[i];
      *reinterpret_cast<u32x4*>(sb + i * (TB ? (T / 32) * kPitchT : (T / 4) * 8)) = qb[i];
    }
  };

  // MFMA fragments: set ks holds the k-step ks (16 k values) of a slab; lane l
  // owns row l % 32 of a 32-row tile and k values 8 (l / 32) .. + 7
  static_assert(kSlab == 32, "the pipeline below is written for two k-steps per slab");
  u32x4 fa0[4], fb0[JN], fa1[4], fb1[JN];
  // Which k a fragment slot holds only has to agree between A and B: k-step
  // `set` of a slab takes k = 16 g + 8 set + e for lane half g = lane / 32, i.e.
  // chunk planes set and set + 2.
  const int tr_lane = (16 * (lane >> 5) + ((lane & 15) >> 2)) * kPitchT + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int frag_a = TA ? tr_lane + wm * 128 : ((lane >> 5) * 2 * kChunkPitch + wm * 128 + (lane & 31)) * 8;
  const int frag_b = kOperand + (TB ? tr_lane + wn * (32 * JN) : ((lane >> 5) * 2 * kChunkPitch + wn * (32 * JN) + (lane & 31)) * 8);
  auto fread = [&](u32x4* fa, u32x4* fb, int set, int buf) {
    const uint16_t* base = smem + buf * 2 * kOperand;
    const uint16_t* qa = base + frag_a + set * (TA ? 8 * kPitchT : kChunkPitch * 8);
    const uint16_t* qb = base + frag_b + set * (TB ? 8 * kPitchT : kChunkPitch * 8);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (TA) {
        const uint2 lo = lds_read_tr(qa + i * 32), hi = lds_read_tr(qa + i * 32 + 4 * kPitchT);
        fa[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
      } else {
        fa[i] = *reinterpret_cast<const u32x4*>(qa + i * 32 * 8);
      }
      if (TB) {
        const uint2 lo = lds_read_tr(qb + i * 32), hi = lds_read_tr(qb + i * 32 + 4 * kPitchT);
        fb[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
      } else {
        fb[i] = *reinterpret_cast<const u32x4*>(qb + i * 32 * 8);
      }
    }
  };
  auto mma = [&](const u32x4* fa, const u32x4* fb) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < JN; ++j) acc[i][j] = Mma<DT>::run(fb[j], fa[i], acc[i][j]);
  };

  // One step per slab, one barrier per step, placed between the two k-steps:
  //   first half:  read the second fragment set of slab cur, write slab cur+1
  //                to the other LDS buffer, 16 MFMAs on the first set,
  //   barrier,
  //   second half: read the first fragment set of slab cur+1, request slab
  //                cur+3, 16 MFMAs on the second set.
  // Loads and LDS stores are unconditional, so every path has the same number
  // of loads in flight and the waits can count.
#define MEGA_GEMM_STEP(R, CA, CB, NA, NB)                                  \
  {                                                                        \
    const int cur = it + (R);                                              \
    fread(fa1, fb1, 1, cur & 1);                                           \
    sstore(NA, NB, cur + 1);                                               \
    mma(fa0, fb0);                                                         \
    lds_barrier();                                                         \
    fread(fa0, fb0, 0, (cur + 1) & 1);                                     \
    gload(CA, CB, cur + kRing);                                            \
    mma(fa1, fb1);                                                         \
  }
  if (nslab > 0) {
    gload(ra0, rb0, 0);
    gload(ra1, rb1, 1);
    gload(ra2, rb2, 2);
    sstore(ra0, rb0, 0);
    lds_barrier();
    fread(fa0, fb0, 0, 0);
    // ring slot R held slab cur, already written to LDS, so it is free for
    // slab cur + kRing
    int it = 0;
    for (; it + kRing <= nslab; it += kRing) {
      MEGA_GEMM_STEP(0, ra0, rb0, ra1, rb1)
      MEGA_GEMM_STEP(1, ra1, rb1, ra2, rb2)
      MEGA_GEMM_STEP(2, ra2, rb2, ra0, rb0)
    }
    if (it < nslab) MEGA_GEMM_STEP(0, ra0, rb0, ra1, rb1)
    if (it + 1 < nslab) MEGA_GEMM_STEP(1, ra1, rb1, ra2, rb2)
    lds_barrier();  // every wave is done with the slab buffers before they are reused
  }
#undef MEGA_GEMM_STEP

  // epilogue: stage the wave's 128 x 128 tile in LDS ([row][col], element type),
  // then write it with 16-byte row segments.  The products are issued as
  // B-fragment x A-fragment, so a 32x32 MFMA tile holds C transposed: lane l has
  // row m = l % 32 and register r the column n = 8 (r / 4) + 4 (l / 32) + r % 4,
  // i.e. four consecutive columns per register quad -> one 8-byte LDS write.
  uint16_t* stage = smem + wave * 128 * EP;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      const int row = i * 32 + (lane & 31);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = j * 32 + 8 * g + 4 * (lane >> 5);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * acc[i][j][4 * g + e];
        uint2 w;
        if (DT == MEGA_BF16) {
          w.x = pack_bf16x2(v[0], v[1]);
          w.y = pack_bf16x2(v[2], v[3]);
        } else {
          w.x = static_cast<uint32_t>(float_to_f16_bits(v[0])) | (static_cast<uint32_t>(float_to_f16_bits(v[1])) << 16);
          w.y = static_cast<uint32_t>(float_to_f16_bits(v[2])) | (static_cast<uint32_t>(float_to_f16_bits(v[3])) << 16);
        }
        *reinterpret_cast<uint2*>(stage + row * EP + col) = w;
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave reads back only its own region
  const bool vec_ok = (p.ldc % 8 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
#pragma unroll 4
  for (int i = 0; i < 8 * JN; ++i) {
    const int c = lane + kWave * i;
    const int row = c / (4 * JN), kc = (c % (4 * JN)) * 8;
    const int grow = m0 + wm * 128 + row, gcol = n0 + wn * (32 * JN) + kc;
    if (grow < p.M && gcol < p.N) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * EP + kc);
      uint16_t* dst = C + static_cast<int64_t>(grow) * p.ldc + gcol;
      if (vec_ok && gcol + 8 <= p.N) {
        *reinterpret_cast<u32x4*>(dst) = v;
      } else {
        const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
        for (int q = 0; q < 8; ++q)
          if (gcol + q < p.N) dst[q] = e[q];
      }
    }
  }
  // the staging regions overlap the operand buffers of every wave: all reads
  // of this tile's epilogue retire before the next tile's first slab lands
  lds_barrier();
  }  // tile of the pair
  }  // work item
}

// ---- the same product with the operand slabs sent from memory straight into LDS ------
// Eight waves of 128 x 64 as above, aligned operands only.  `global_load_lds_dwordx4`
// writes the 64 lanes' 16-byte pieces to 1 KB of consecutive LDS (base in M0), so no slab
// passes through registers: no register ring, no LDS store instructions.  The LDS image
// is dense and the swizzle that keeps fragment reads off each other's banks is applied
// on the memory side -- which chunk a lane fetches:
//   k-contiguous operand: a slab is 256 rows of 64 bytes; 1 KB = 16 rows; the chunk at
//       position c of row r holds k chunk c ^ ((r >> 2) & 3) (16-byte reads go sixteen lanes at
//       a time over 64 banks: sixteen consecutive rows of one k chunk then cover sixteen different
//       16-byte bank groups; with (r >> 1) & 3, enough for eight lanes over 32 banks, half of the
//       LDS cycles were bank conflicts);
//   k-major operand: a slab is 32 rows of k, 512 bytes each; 1 KB = 2 rows; the chunk at
//       position c of row k holds m chunk c ^ ((k & 3) << 2) (the four rows of k that a
//       transposing read touches lie 64 bytes apart, as with the padded rows above).
// Four slab buffers: slab s + 4 is requested into the buffer of slab s right after the
// barrier that ends the reads of slab s; three slabs are in flight while one is read.
constexpr int kStages = 4;
constexpr int kDmaOperand = kTile * kSlab;   // elements of an operand slab (16 KB)
constexpr int kDmaStage = 2 * kDmaOperand;   // A, then B
constexpr size_t kDmaLds = sizeof(uint16_t) * (8 * 128 * (64 + 8) > kStages * kDmaStage ? 8 * 128 * (64 + 8)
                                                                                         : kStages * kDmaStage);

// One request: lane l's 16 bytes at base + offset go to LDS bytes lds_dst + 16 l .. + 15
// (lds_dst wave-uniform).  Written as assembly so that the compiler does not see a vector
// memory instruction that writes LDS: it would put a wait for every request in flight in
// front of the transposing LDS reads.  The waits for these requests are the explicit
// `s_waitcnt vmcnt` below.  M0 is reserved: the compiler keeps nothing in it across statements.
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t offset, uint32_t lds_dst) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(offset), "s"(base), "s"(lds_dst));
}

template <int DT, bool TA, bool TB>
__global__ __launch_bounds__(2 * kThreads) void gemm_dma_kernel(const GemmParams p) {
  extern __shared__ __align__(16) uint16_t smem[];
  constexpr int JN = 2, NL = 2, EP = 64 + 8;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 2, wn = wave & 3;
  // work items as in gemm_kernel
  const int G = static_cast<int>(gridDim.x), lin = static_cast<int>(blockIdx.x);
  int it_lo, it_hi, it_step;
  if (G % kXcds == 0) {
    const int xcd = lin % kXcds;
    it_lo = static_cast<int>(static_cast<int64_t>(p.items) * xcd / kXcds) + lin / kXcds;
    it_hi = static_cast<int>(static_cast<int64_t>(p.items) * (xcd + 1) / kXcds);
    it_step = G / kXcds;
  } else {
    it_lo = lin;
    it_hi = p.items;
    it_step = G;
  }
  for (int item = it_lo; item < it_hi; item += it_step) {
  const int zz = item / p.per_batch;
  const int rem = item % p.per_batch;
  int nt, mt_first, mt_second = -1;
  if (p.tri_out) {
    int t = rem, m = 0;
    while (true) {
      const int cnt = min(p.nt_count, (m * kTile + (kTile - 1) + p.off) / kTile + 1);
      if (t < cnt) break;
      t -= cnt;
      ++m;
    }
    mt_first = m;
    nt = t;
  } else if (p.k_mode) {
    nt = rem % p.nt_count;
    const int pr = rem / p.nt_count;
    mt_first = p.mt_count - 1 - pr;
    if (mt_first != pr) mt_second = pr;
  } else {
    if (p.n_group > 0) {
      const int band = p.n_group * p.mt_count;       // tiles of a full band
      const int b0 = rem / band, r2 = rem % band;
      const int w = min(p.n_group, p.nt_count - b0 * p.n_group);  // the last band may be narrower
      nt = b0 * p.n_group + r2 % w;
      mt_first = r2 / w;
    } else {
      nt = rem % p.nt_count;
      mt_first = rem / p.nt_count;
    }
  }
  const int z0 = zz / p.nh, z1 = zz % p.nh;
  const uint16_t* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const uint16_t* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  uint16_t* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  for (int half = 0; half < 2; ++half) {
  const int mt = half == 0 ? mt_first : mt_second;
  if (mt < 0) break;
  const int m0 = mt * kTile, n0 = nt * kTile;
  int kb = 0, ke = p.K;
  if (p.k_mode == 1) ke = min(p.K, ((mt + 1) * kTile + p.off + kSlab - 1) / kSlab * kSlab);
  if (p.k_mode == 2) kb = min(p.K, max(0, mt * kTile - p.off) / kSlab * kSlab);
  const int nslab = (ke - kb + kSlab - 1) / kSlab;

  floatx16 acc[4][JN];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // memory side: wave w sends the 1 KB pieces w and w + 8 of each operand slab; lane l
  // of piece pc fetches what belongs at position l of the piece (addresses clamped into
  // the matrix, so every lane always loads)
  uint32_t offa[NL], offb[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int pc = wave + 8 * i;
    const int krow = 2 * pc + (lane >> 5), cm = (lane & 31) ^ ((krow & 3) << 2);  // k-major piece
    const int row = 16 * pc + (lane >> 2), ck = (lane & 3) ^ ((lane >> 4) & 3);   // k-contiguous piece
    if (TA) offa[i] = static_cast<uint32_t>(((kb + krow) * p.lda + min(m0 + cm * 8, p.M - 8)) * 2);
    else offa[i] = static_cast<uint32_t>((static_cast<int64_t>(min(m0 + row, p.M - 1)) * p.lda + kb + ck * 8) * 2);
    if (TB) offb[i] = static_cast<uint32_t>(((kb + krow) * p.ldb + min(n0 + cm * 8, p.N - 8)) * 2);
    else offb[i] = static_cast<uint32_t>((static_cast<int64_t>(min(n0 + row, p.N - 1)) * p.ldb + kb + ck * 8) * 2);
  }
  const uint32_t stepa = static_cast<uint32_t>((TA ? p.lda : 1) * kSlab * 2);
  const uint32_t stepb = static_cast<uint32_t>((TB ? p.ldb : 1) * kSlab * 2);
  const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)(smem))) + wave * 1024);
  // request number n of a slab: n = 0, 2 the two pieces of A, n = 1, 3 those of B
  auto request_one = [&](int s, int stage, int n) {
    const uint32_t sc = static_cast<uint32_t>(min(s, nslab - 1));
    const uint32_t dst = lds_wave + static_cast<uint32_t>(stage * kDmaStage + (n >> 1) * 8 * 512 + (n & 1) * kDmaOperand) * 2;
    if (n & 1) load_to_lds16(B, offb[n >> 1] + sc * stepb, dst);
    else load_to_lds16(A, offa[n >> 1] + sc * stepa, dst);
  };
  auto request = [&](int s, int stage) {
#pragma unroll
    for (int n = 0; n < 2 * NL; ++n) request_one(s, stage, n);
  };

  // fragment side: k-step `set` of a slab takes k = 16 g + 8 set + e for lane half g
  const int g = lane >> 5, r = lane & 31;
  const int ta_a = (lane & 15) >> 2, ta_h = (lane >> 4) & 1, ta_b = lane & 3;
  int fra[4], frb[JN];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (TA) fra[i] = (16 * g + ta_a) * kTile + (((wm * 16 + 4 * i + 2 * ta_h + (ta_b >> 1)) ^ (ta_a << 2)) * 8) + 4 * (ta_b & 1);
    else fra[i] = (wm * 128 + 32 * i + r) * kSlab + (((2 * g) ^ ((r >> 2) & 3)) * 8);
  }
#pragma unroll
  for (int j = 0; j < JN; ++j) {
    if (TB) frb[j] = kDmaOperand + (16 * g + ta_a) * kTile + (((wn * 8 + 4 * j + 2 * ta_h + (ta_b >> 1)) ^ (ta_a << 2)) * 8) + 4 * (ta_b & 1);
    else frb[j] = kDmaOperand + (wn * 64 + 32 * j + r) * kSlab + (((2 * g) ^ ((r >> 2) & 3)) * 8);
  }
  u32x4 fa0[4], fb0[JN], fa1[4], fb1[JN];
  auto fread = [&](u32x4* fa, u32x4* fb, int set, int stage) {
    const uint16_t* base = smem + stage * kDmaStage;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (TA) {
        const uint16_t* q = base + fra[i] + set * 8 * kTile;
        const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * kTile);
        fa[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
      } else {
        // chunk 2 g + set sits at position (2 g + set) ^ swizzle = ((2 g) ^ swizzle) ^ set
        fa[i] = *reinterpret_cast<const u32x4*>(base + (fra[i] ^ (set * 8)));
      }
      if (i < JN) {
        if (TB) {
          const uint16_t* q = base + frb[i] + set * 8 * kTile;
          const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * kTile);
          fb[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
        } else {
          fb[i] = *reinterpret_cast<const u32x4*>(base + (frb[i] ^ (set * 8)));
        }
      }
    }
  };
  // products lo .. hi - 1 of a k-step, numbered 2 i + j
  auto mma = [&](const u32x4* fa, const u32x4* fb, int lo, int hi) {
#pragma unroll
    for (int n = 0; n < 4 * JN; ++n)
      if (n >= lo && n < hi) acc[n >> 1][n & 1] = Mma<DT>::run(fb[n & 1], fa[n >> 1], acc[n >> 1][n & 1]);
  };

  // One step per slab, one barrier per step, placed between the two k-steps:
  //   first half:  read the second fragment set of slab cur; 8 MFMAs on the first set;
  //   wait until this wave's pieces of slab cur + 1 have landed (at most the 8 requests of
  //   slabs cur + 2, cur + 3 still in flight) and its fragment reads have returned; barrier;
  //   second half: read the first fragment set of slab cur + 1, request slab cur + 4 into
  //                the buffer slab cur has just left, 8 MFMAs on the second set.
#define MEGA_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
  constexpr int kFragReads = (TA ? 2 : 1) + (TB ? JN / 2 : (JN + 3) / 4);
#define MEGA_DMA_STEP(R)                                                   \
  {                                                                        \
    const int cur = it + (R);                                              \
    fread(fa1, fb1, 1, (R));                                               \
    mma(fa0, fb0, 0, 8);                                                   \
    _Pragma("unroll") for (int sg = 0; sg < 4; ++sg) {                     \
      MEGA_SGB(0x008, 1);                                                  \
      MEGA_SGB(0x100, kFragReads);                                         \
    }                                                                      \
    MEGA_SGB(0x008, 4 * JN - 4);                                           \
    __builtin_amdgcn_sched_barrier(0);                                     \
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory"); \
    fread(fa0, fb0, 0, ((R) + 1) & 3);                                     \
    mma(fa1, fb1, 0, 4);                                                   \
    _Pragma("unroll") for (int sg = 0; sg < 4; ++sg) {                     \
      MEGA_SGB(0x008, 1);                                                  \
      MEGA_SGB(0x100, kFragReads);                                         \
    }                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                     \
    _Pragma("unroll") for (int n = 0; n < 2 * NL; ++n) {                   \
      request_one(cur + kStages, (R), n);                                  \
      mma(fa1, fb1, 4 + n, 5 + n);                                         \
      __builtin_amdgcn_sched_barrier(0);                                   \
    }                                                                      \
  }
  if (nslab > 0) {
    request(0, 0);
    request(1, 1);
    request(2, 2);
    request(3, 3);
    asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
    fread(fa0, fb0, 0, 0);
    int it = 0;
    for (; it + 4 <= nslab; it += 4) {
      MEGA_DMA_STEP(0)
      MEGA_DMA_STEP(1)
      MEGA_DMA_STEP(2)
      MEGA_DMA_STEP(3)
    }
    if (it < nslab) MEGA_DMA_STEP(0)
    if (it + 1 < nslab) MEGA_DMA_STEP(1)
    if (it + 2 < nslab) MEGA_DMA_STEP(2)
    // nothing may land in the buffers once they hold the output tiles
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
#undef MEGA_DMA_STEP
#undef MEGA_SGB

  // epilogue as in gemm_kernel: the wave's 128 x 64 tile through its own LDS region
  uint16_t* stage = smem + wave * 128 * EP;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      const int row = i * 32 + (lane & 31);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int col = j * 32 + 8 * q4 + 4 * (lane >> 5);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * acc[i][j][4 * q4 + e];
        uint2 w;
        if (DT == MEGA_BF16) {
          w.x = pack_bf16x2(v[0], v[1]);
          w.y = pack_bf16x2(v[2], v[3]);
        } else {
          w.x = static_cast<uint32_t>(float_to_f16_bits(v[0])) | (static_cast<uint32_t>(float_to_f16_bits(v[1])) << 16);
          w.y = static_cast<uint32_t>(float_to_f16_bits(v[2])) | (static_cast<uint32_t>(float_to_f16_bits(v[3])) << 16);
        }
        *reinterpret_cast<uint2*>(stage + row * EP + col) = w;
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave reads back only its own region
  const bool vec_ok = (p.ldc % 8 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
#pragma unroll 4
  for (int i = 0; i < 8 * JN; ++i) {
    const int c = lane + kWave * i;
    const int row = c / (4 * JN), kc = (c % (4 * JN)) * 8;
    const int grow = m0 + wm * 128 + row, gcol = n0 + wn * (32 * JN) + kc;
    if (grow < p.M && gcol < p.N) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * EP + kc);
      uint16_t* dst = C + static_cast<int64_t>(grow) * p.ldc + gcol;
      if (vec_ok && gcol + 8 <= p.N) {
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));  // whole lines, read by a later kernel
      } else {
        const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
        for (int q = 0; q < 8; ++q)
          if (gcol + q < p.N) dst[q] = e[q];
      }
    }
  }
  // the output regions overlap the slab buffers: every read of this tile's epilogue
  // retires before the next tile's first slab is requested
  lds_barrier();
  }  // tile of the pair
  }  // work item
}

// ---- the same with slabs of 64 k, for products of two k-contiguous operands ---------------
// With slabs of 32 k a k-contiguous operand arrives as 64-byte pieces of its rows, half a
// cache line each, sixteen lines per request; the products with such operands keep the matrix
// pipe 55-57 % busy where the one with two k-major operands (whole 512-byte rows) reaches 86 %.
// Here a slab is 64 k: k-contiguous rows come as whole 128-byte lines (1 KB = 8 rows, the chunk at
// position c of row r holds k chunk c ^ ((r >> 1) & 7)), k-major slabs would be 64 rows of k.
// Two slab buffers of 64 KB; slab s + 2 is requested into the buffer of slab s after the barrier
// that ends its reads, under the last of the slab's four k-steps.  Measured in one run at the
// attention benchmark shape: dP = dY V^T 1.15-1.27 -> 1.02-1.06 ms, forward / backward of the
// operator 1.436 / 2.59 -> 1.425 / 2.52 ms; with one k-major operand (PV, dQ) the forward was 1 %
// slower than with slabs of 32, so only the products of two k-contiguous operands come here (the
// template covers the other layouts; they are not instantiated).
constexpr int kSlab64 = 64;
constexpr int kDma64Operand = kTile * kSlab64;  // elements of an operand slab (32 KB)
constexpr int kDma64Stage = 2 * kDma64Operand;
static_assert(sizeof(uint16_t) * 2 * kDma64Stage <= kDmaLds, "two slab buffers fit");

template <int DT, bool TA, bool TB>
__global__ __launch_bounds__(2 * kThreads) void gemm_dma64_kernel(const GemmParams p) {
  extern __shared__ __align__(16) uint16_t smem[];
  constexpr int JN = 2, NL = 4, EP = 64 + 8;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 2, wn = wave & 3;
  const int G = static_cast<int>(gridDim.x), lin = static_cast<int>(blockIdx.x);
  int it_lo, it_hi, it_step;
  if (G % kXcds == 0) {
    const int xcd = lin % kXcds;
    it_lo = static_cast<int>(static_cast<int64_t>(p.items) * xcd / kXcds) + lin / kXcds;
    it_hi = static_cast<int>(static_cast<int64_t>(p.items) * (xcd + 1) / kXcds);
    it_step = G / kXcds;
  } else {
    it_lo = lin;
    it_hi = p.items;
    it_step = G;
  }
  for (int item = it_lo; item < it_hi; item += it_step) {
  const int zz = item / p.per_batch;
  const int rem = item % p.per_batch;
  int nt, mt_first, mt_second = -1;
  if (p.tri_out) {
    int t = rem, m = 0;
    while (true) {
      const int cnt = min(p.nt_count, (m * kTile + (kTile - 1) + p.off) / kTile + 1);
      if (t < cnt) break;
      t -= cnt;
      ++m;
    }
    mt_first = m;
    nt = t;
  } else if (p.k_mode) {
    nt = rem % p.nt_count;
    const int pr = rem / p.nt_count;
    mt_first = p.mt_count - 1 - pr;
    if (mt_first != pr) mt_second = pr;
  } else {
    nt = rem % p.nt_count;
    mt_first = rem / p.nt_count;
  }
  const int z0 = zz / p.nh, z1 = zz % p.nh;
  const uint16_t* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const uint16_t* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  uint16_t* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  for (int half = 0; half < 2; ++half) {
  const int mt = half == 0 ? mt_first : mt_second;
  if (mt < 0) break;
  const int m0 = mt * kTile, n0 = nt * kTile;
  // k range as in gemm_kernel, widened to whole slabs of 64 (K % 64 == 0): what the wider range
  // adds are probabilities the softmax has written as zeros
  int kb = 0, ke = p.K;
  if (p.k_mode == 1) ke = min(p.K, ((mt + 1) * kTile + p.off + kSlab64 - 1) / kSlab64 * kSlab64);
  if (p.k_mode == 2) kb = min(p.K, max(0, mt * kTile - p.off) / kSlab64 * kSlab64);
  const int nslab = (ke - kb + kSlab64 - 1) / kSlab64;

  floatx16 acc[4][JN];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // memory side: wave w sends the 1 KB pieces w, w + 8, w + 16, w + 24 of each operand slab
  uint32_t offa[NL], offb[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int pc = wave + 8 * i;
    const int krow = 2 * pc + (lane >> 5), cm = (lane & 31) ^ ((krow & 3) << 2);   // k-major piece: 2 rows of k
    const int row = 8 * pc + (lane >> 3), ck = (lane & 7) ^ ((row >> 1) & 7);      // k-contiguous piece: 8 rows
    if (TA) offa[i] = static_cast<uint32_t>(((kb + krow) * p.lda + min(m0 + cm * 8, p.M - 8)) * 2);
    else offa[i] = static_cast<uint32_t>((static_cast<int64_t>(min(m0 + row, p.M - 1)) * p.lda + kb + ck * 8) * 2);
    if (TB) offb[i] = static_cast<uint32_t>(((kb + krow) * p.ldb + min(n0 + cm * 8, p.N - 8)) * 2);
    else offb[i] = static_cast<uint32_t>((static_cast<int64_t>(min(n0 + row, p.N - 1)) * p.ldb + kb + ck * 8) * 2);
  }
  const uint32_t stepa = static_cast<uint32_t>((TA ? p.lda : 1) * kSlab64 * 2);
  const uint32_t stepb = static_cast<uint32_t>((TB ? p.ldb : 1) * kSlab64 * 2);
  const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)(smem))) + wave * 1024);
  // request number n of a slab: even n the pieces of A, odd n those of B
  auto request_one = [&](int s, int stage, int n) {
    const uint32_t sc = static_cast<uint32_t>(min(s, nslab - 1));
    const uint32_t dst = lds_wave + static_cast<uint32_t>(stage * kDma64Stage + (n >> 1) * 8 * 512 + (n & 1) * kDma64Operand) * 2;
    if (n & 1) load_to_lds16(B, offb[n >> 1] + sc * stepb, dst);
    else load_to_lds16(A, offa[n >> 1] + sc * stepa, dst);
  };
  auto request = [&](int s, int stage) {
#pragma unroll
    for (int n = 0; n < 2 * NL; ++n) request_one(s, stage, n);
  };

  // fragment side: k-step `set` (0 .. 3) of a slab takes k = 16 set + 8 g + e for lane half g
  const int g = lane >> 5, r = lane & 31;
  const int ta_a = (lane & 15) >> 2, ta_h = (lane >> 4) & 1, ta_b = lane & 3;
  int fra[4], frb[JN];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (TA) fra[i] = (8 * g + ta_a) * kTile + (((wm * 16 + 4 * i + 2 * ta_h + (ta_b >> 1)) ^ (ta_a << 2)) * 8) + 4 * (ta_b & 1);
    else fra[i] = (wm * 128 + 32 * i + r) * kSlab64 + ((g ^ ((r >> 1) & 7)) * 8);
  }
#pragma unroll
  for (int j = 0; j < JN; ++j) {
    if (TB) frb[j] = kDma64Operand + (8 * g + ta_a) * kTile + (((wn * 8 + 4 * j + 2 * ta_h + (ta_b >> 1)) ^ (ta_a << 2)) * 8) + 4 * (ta_b & 1);
    else frb[j] = kDma64Operand + (wn * 64 + 32 * j + r) * kSlab64 + ((g ^ ((r >> 1) & 7)) * 8);
  }
  u32x4 fa0[4], fb0[JN], fa1[4], fb1[JN];
  // fragments lo .. hi - 1 of a k-step: number i = row block i of A and, for i < JN, column block i of B
  auto fread = [&](u32x4* fa, u32x4* fb, int set, int stage, int lo = 0, int hi = 4) {
    const uint16_t* base = smem + stage * kDma64Stage;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < lo || i >= hi) continue;
      if (TA) {
        const uint16_t* q = base + fra[i] + set * 16 * kTile;
        const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * kTile);
        fa[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
      } else {
        // chunk 2 set + g sits at position (2 set + g) ^ swizzle = (g ^ swizzle) ^ (2 set)
        fa[i] = *reinterpret_cast<const u32x4*>(base + (fra[i] ^ (set * 16)));
      }
      if (i < JN) {
        if (TB) {
          const uint16_t* q = base + frb[i] + set * 16 * kTile;
          const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * kTile);
          fb[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
        } else {
          fb[i] = *reinterpret_cast<const u32x4*>(base + (frb[i] ^ (set * 16)));
        }
      }
    }
  };
  auto mma = [&](const u32x4* fa, const u32x4* fb, int lo, int hi) {
#pragma unroll
    for (int n = 0; n < 4 * JN; ++n)
      if (n >= lo && n < hi) acc[n >> 1][n & 1] = Mma<DT>::run(fb[n & 1], fa[n >> 1], acc[n >> 1][n & 1]);
  };

  // One step per slab of 64 k = four k-steps; the fragments of the next k-step are read under the
  // products of the current one.  Before the last k-step: this wave's pieces of the next slab have
  // landed (nothing else of its requests is in flight) and its reads of this slab have returned;
  // barrier; then the first fragments of the next slab, the requests for the slab after it into
  // the buffer just left (one per product), the last 8 products.
#define MEGA_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
  constexpr int kFragReads = (TA ? 2 : 1) + (TB ? JN / 2 : (JN + 3) / 4);
#define MEGA_DMA64_KSTEP(FA, FB, NFA, NFB, SET, STAGE)                     \
  {                                                                        \
    fread(NFA, NFB, (SET) + 1, (STAGE));                                   \
    mma(FA, FB, 0, 8);                                                     \
    _Pragma("unroll") for (int sg = 0; sg < 4; ++sg) {                     \
      MEGA_SGB(0x008, 1);                                                  \
      MEGA_SGB(0x100, kFragReads);                                         \
    }                                                                      \
    MEGA_SGB(0x008, 4);                                                    \
    __builtin_amdgcn_sched_barrier(0);                                     \
  }
#define MEGA_DMA64_STEP(R)                                                 \
  {                                                                        \
    const int cur = it + (R);                                              \
    MEGA_DMA64_KSTEP(fa0, fb0, fa1, fb1, 0, (R))                           \
    MEGA_DMA64_KSTEP(fa1, fb1, fa0, fb0, 1, (R))                           \
    MEGA_DMA64_KSTEP(fa0, fb0, fa1, fb1, 2, (R))                           \
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); \
    _Pragma("unroll") for (int n = 0; n < 2 * NL; ++n) {                   \
      if (n < 4) fread(fa0, fb0, 0, (R) ^ 1, n, n + 1);                    \
      request_one(cur + 2, (R), n);                                        \
      mma(fa1, fb1, n, n + 1);                                             \
      __builtin_amdgcn_sched_barrier(0);                                   \
    }                                                                      \
  }
  if (nslab > 0) {
    request(0, 0);
    request(1, 1);
    asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
    fread(fa0, fb0, 0, 0);
    int it = 0;
    for (; it + 2 <= nslab; it += 2) {
      MEGA_DMA64_STEP(0)
      MEGA_DMA64_STEP(1)
    }
    if (it < nslab) MEGA_DMA64_STEP(0)
    // nothing may land in the buffers once they hold the output tiles
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
#undef MEGA_DMA64_STEP
#undef MEGA_DMA64_KSTEP
#undef MEGA_SGB

  // epilogue as in gemm_kernel: the wave's 128 x 64 tile through its own LDS region
  uint16_t* stage = smem + wave * 128 * EP;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      const int row = i * 32 + (lane & 31);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int col = j * 32 + 8 * q4 + 4 * (lane >> 5);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * acc[i][j][4 * q4 + e];
        uint2 w;
        if (DT == MEGA_BF16) {
          w.x = pack_bf16x2(v[0], v[1]);
          w.y = pack_bf16x2(v[2], v[3]);
        } else {
          w.x = static_cast<uint32_t>(float_to_f16_bits(v[0])) | (static_cast<uint32_t>(float_to_f16_bits(v[1])) << 16);
          w.y = static_cast<uint32_t>(float_to_f16_bits(v[2])) | (static_cast<uint32_t>(float_to_f16_bits(v[3])) << 16);
        }
        *reinterpret_cast<uint2*>(stage + row * EP + col) = w;
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  const bool vec_ok = (p.ldc % 8 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
#pragma unroll 4
  for (int i = 0; i < 8 * JN; ++i) {
    const int c = lane + kWave * i;
    const int row = c / (4 * JN), kc = (c % (4 * JN)) * 8;
    const int grow = m0 + wm * 128 + row, gcol = n0 + wn * (32 * JN) + kc;
    if (grow < p.M && gcol < p.N) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * EP + kc);
      uint16_t* dst = C + static_cast<int64_t>(grow) * p.ldc + gcol;
      if (vec_ok && gcol + 8 <= p.N) {
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));  // whole lines, read by a later kernel
      } else {
        const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
        for (int q = 0; q < 8; ++q)
          if (gcol + q < p.N) dst[q] = e[q];
      }
    }
  }
  lds_barrier();
  }  // tile of the pair
  }  // work item
}

// ---- one k-contiguous and one k-major operand: A in slabs of 64 k, B in slabs of 32 k ------
// (PV and dQ: A = P or dS, rows of keys; B = V or K, rows of k.)  With slabs of 32 k the rows of A
// arrive as half cache lines, and the L2 answers a 64-byte request no faster than a 128-byte one:
// such a product sends 1.5 times the requests of one with two k-major operands and keeps the
// matrix pipe 55-68 % busy where that one reaches 86 %.  Slabs of 64 k for both operands leave
// room for two buffers only (gemm_dma64_kernel) and were 1 % slower here.  This form keeps the
// depth: three A buffers of 32 KB (256 rows x 64 k, whole lines) and four B buffers of 16 KB
// (32 rows of k), all 160 KB of the LDS; a step is 32 k as in gemm_dma_kernel.
constexpr int kA64Operand = kTile * kSlab64;        // elements of an A slab (32 KB)
constexpr int kA64BBase = 3 * kA64Operand;          // the B buffers start behind the three A buffers
constexpr size_t kA64Lds = sizeof(uint16_t) * (kA64BBase + kStages * kDmaOperand);
static_assert(kA64Lds <= 160 * 1024 && sizeof(uint16_t) * 8 * 128 * (64 + 8) <= kA64Lds, "fits the LDS, holds the output tiles");

template <int DT>
__global__ __launch_bounds__(2 * kThreads) void gemm_dma_a64_kernel(const GemmParams p) {
  extern __shared__ __align__(16) uint16_t smem[];
  constexpr int JN = 2, EP = 64 + 8;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 2, wn = wave & 3;
  // work items as in gemm_kernel
  const int G = static_cast<int>(gridDim.x), lin = static_cast<int>(blockIdx.x);
  int it_lo, it_hi, it_step;
  if (G % kXcds == 0) {
    const int xcd = lin % kXcds;
    it_lo = static_cast<int>(static_cast<int64_t>(p.items) * xcd / kXcds) + lin / kXcds;
    it_hi = static_cast<int>(static_cast<int64_t>(p.items) * (xcd + 1) / kXcds);
    it_step = G / kXcds;
  } else {
    it_lo = lin;
    it_hi = p.items;
    it_step = G;
  }
  for (int item = it_lo; item < it_hi; item += it_step) {
  const int zz = item / p.per_batch;
  const int rem = item % p.per_batch;
  int nt, mt_first, mt_second = -1;
  if (p.tri_out) {
    int t = rem, m = 0;
    while (true) {
      const int cnt = min(p.nt_count, (m * kTile + (kTile - 1) + p.off) / kTile + 1);
      if (t < cnt) break;
      t -= cnt;
      ++m;
    }
    mt_first = m;
    nt = t;
  } else if (p.k_mode) {
    nt = rem % p.nt_count;
    const int pr = rem / p.nt_count;
    mt_first = p.mt_count - 1 - pr;
    if (mt_first != pr) mt_second = pr;
  } else {
    if (p.n_group > 0) {
      const int band = p.n_group * p.mt_count;       // tiles of a full band
      const int b0 = rem / band, r2 = rem % band;
      const int w = min(p.n_group, p.nt_count - b0 * p.n_group);  // the last band may be narrower
      nt = b0 * p.n_group + r2 % w;
      mt_first = r2 / w;
    } else {
      nt = rem % p.nt_count;
      mt_first = rem / p.nt_count;
    }
  }
  const int z0 = zz / p.nh, z1 = zz % p.nh;
  const uint16_t* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const uint16_t* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  uint16_t* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  for (int half = 0; half < 2; ++half) {
  const int mt = half == 0 ? mt_first : mt_second;
  if (mt < 0) break;
  const int m0 = mt * kTile, n0 = nt * kTile;
  // k range as in gemm_kernel, widened to whole slabs of 64 (K % 64 == 0): what the wider range
  // adds are probabilities the softmax has written as zeros
  int kb = 0, ke = p.K;
  if (p.k_mode == 1) ke = min(p.K, ((mt + 1) * kTile + p.off + kSlab64 - 1) / kSlab64 * kSlab64);
  if (p.k_mode == 2) kb = min(p.K, max(0, mt * kTile - p.off) / kSlab64 * kSlab64);
  const int nslab = (ke - kb) / kSlab;   // steps of 32 k, an even number
  const int nslab_a = nslab / 2;         // slabs of A

  floatx16 acc[4][JN];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // memory side.  A: wave w sends the 1 KB pieces w, w + 8, w + 16, w + 24 of a slab (8 rows of
  // 128 bytes each, the chunk at position c of row r holds k chunk c ^ ((r >> 1) & 7)); B: the
  // pieces w, w + 8 (2 rows of k, 512 bytes each).  Addresses are clamped into the matrix.
  uint32_t offa[4], offb[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int pc = wave + 8 * i;
    const int row = 8 * pc + (lane >> 3), ck = (lane & 7) ^ ((row >> 1) & 7);
    offa[i] = static_cast<uint32_t>((static_cast<int64_t>(min(m0 + row, p.M - 1)) * p.lda + kb + ck * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int pc = wave + 8 * i;
    const int krow = 2 * pc + (lane >> 5), cm = (lane & 31) ^ ((krow & 3) << 2);
    offb[i] = static_cast<uint32_t>(((kb + krow) * p.ldb + min(n0 + cm * 8, p.N - 8)) * 2);
  }
  const uint32_t stepa = static_cast<uint32_t>(kSlab64 * 2);
  const uint32_t stepb = static_cast<uint32_t>(p.ldb * kSlab * 2);
  const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint16_t*)(smem))) + wave * 1024);
  // A slab ja into A buffer ab (4 requests), B slab s into B buffer bb (2 requests); slabs past the
  // end ask for the last one again, so that every step issues the same number of requests
  auto request_a = [&](int ja, int ab, int n) {
    const uint32_t sc = static_cast<uint32_t>(min(ja, nslab_a - 1));
    load_to_lds16(A, offa[n] + sc * stepa, lds_wave + static_cast<uint32_t>(ab * kA64Operand + n * 8 * 512) * 2);
  };
  auto request_b = [&](int sb, int bb, int n) {
    const uint32_t sc = static_cast<uint32_t>(min(sb, nslab - 1));
    load_to_lds16(B, offb[n] + sc * stepb, lds_wave + static_cast<uint32_t>(kA64BBase + bb * kDmaOperand + n * 8 * 512) * 2);
  };

  // fragment side: as in gemm_dma_kernel, k-step `set` of a 32-k step takes k = 16 g + 8 set + e
  // for lane half g; in the A slab that is chunk 4 h + 2 g + set of the row (h: which half of the
  // 64 k the step is), at position ((2 g) ^ swizzle) ^ (4 h + set)
  const int g = lane >> 5, r = lane & 31;
  const int ta_a = (lane & 15) >> 2, ta_h = (lane >> 4) & 1, ta_b = lane & 3;
  int fra[4], frb[JN];
#pragma unroll
  for (int i = 0; i < 4; ++i) fra[i] = (wm * 128 + 32 * i + r) * kSlab64 + (((2 * g) ^ ((r >> 1) & 7)) * 8);
#pragma unroll
  for (int j = 0; j < JN; ++j)
    frb[j] = kA64BBase + (16 * g + ta_a) * kTile + (((wn * 8 + 4 * j + 2 * ta_h + (ta_b >> 1)) ^ (ta_a << 2)) * 8) + 4 * (ta_b & 1);
  u32x4 fa0[4], fb0[JN], fa1[4], fb1[JN];
  // fragments of k-step `set` of a 32-k step: A buffer ab, chunk selector x = 4 h + set; B buffer bb
  auto fread = [&](u32x4* fa, u32x4* fb, int x, int ab, int set, int bb) {
    const uint16_t* abase = smem + ab * kA64Operand;
    const uint16_t* bbase = smem + bb * kDmaOperand;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      fa[i] = *reinterpret_cast<const u32x4*>(abase + (fra[i] ^ (x * 8)));
      if (i < JN) {
        const uint16_t* q = bbase + frb[i] + set * 8 * kTile;
        const uint2 lo = lds_read_tr(q), hi = lds_read_tr(q + 4 * kTile);
        fb[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
      }
    }
  };
  auto mma = [&](const u32x4* fa, const u32x4* fb, int lo, int hi) {
#pragma unroll
    for (int n = 0; n < 4 * JN; ++n)
      if (n >= lo && n < hi) acc[n >> 1][n & 1] = Mma<DT>::run(fb[n & 1], fa[n >> 1], acc[n >> 1][n & 1]);
  };

  // One step per 32 k as in gemm_dma_kernel.  An odd step also ends the reads of its A slab and
  // requests A slab (s >> 1) + 3 into that buffer, before the step's B requests.  In front of the
  // barrier of step s the requests of the two steps before it may still be in flight: two B slabs
  // and one A slab, 8 per wave; B slab s + 1 and, at odd s, A slab (s + 1) / 2 are older.
#define MEGA_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
  constexpr int kFragReads = 1 + JN / 2;
#define MEGA_A64_STEP(R)                                                   \
  {                                                                        \
    const int cur = it + (R);                                              \
    fread(fa1, fb1, 4 * ((R) & 1) + 1, ab, 1, (R));                        \
    mma(fa0, fb0, 0, 8);                                                   \
    _Pragma("unroll") for (int sg = 0; sg < 4; ++sg) {                     \
      MEGA_SGB(0x008, 1);                                                  \
      MEGA_SGB(0x100, kFragReads);                                         \
    }                                                                      \
    MEGA_SGB(0x008, 4 * JN - 4);                                           \
    __builtin_amdgcn_sched_barrier(0);                                     \
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory"); \
    const int ab_next = ((R) & 1) ? (ab == 2 ? 0 : ab + 1) : ab;           \
    fread(fa0, fb0, ((R) & 1) ? 0 : 4, ab_next, 0, ((R) + 1) & 3);         \
    mma(fa1, fb1, 0, 2);                                                   \
    _Pragma("unroll") for (int sg = 0; sg < 2; ++sg) {                     \
      MEGA_SGB(0x008, 1);                                                  \
      MEGA_SGB(0x100, 2 * kFragReads);                                     \
    }                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                     \
    _Pragma("unroll") for (int n = 0; n < 6; ++n) {                        \
      if ((R) & 1) {                                                       \
        if (n < 4) request_a((cur >> 1) + 3, ab, n);                       \
        else request_b(cur + kStages, (R), n - 4);                         \
      } else if (n < 2) {                                                  \
        request_b(cur + kStages, (R), n);                                  \
      }                                                                    \
      mma(fa1, fb1, 2 + n, 3 + n);                                         \
      __builtin_amdgcn_sched_barrier(0);                                   \
    }                                                                      \
    ab = ab_next;                                                          \
  }
  if (nslab > 0) {
    int ab = 0;
#pragma unroll
    for (int n = 0; n < 4; ++n) request_a(0, 0, n);
#pragma unroll
    for (int n = 0; n < 2; ++n) request_b(0, 0, n);
#pragma unroll
    for (int n = 0; n < 2; ++n) request_b(1, 1, n);
#pragma unroll
    for (int n = 0; n < 4; ++n) request_a(1, 1, n);
#pragma unroll
    for (int n = 0; n < 2; ++n) request_b(2, 2, n);
#pragma unroll
    for (int n = 0; n < 2; ++n) request_b(3, 3, n);
#pragma unroll
    for (int n = 0; n < 4; ++n) request_a(2, 2, n);
    asm volatile("s_waitcnt vmcnt(14)\n\ts_barrier" ::: "memory");
    fread(fa0, fb0, 0, 0, 0, 0);
    for (int it = 0; it < nslab; it += 4) {
      MEGA_A64_STEP(0)
      MEGA_A64_STEP(1)
      if (it + 2 < nslab) {
        MEGA_A64_STEP(2)
        MEGA_A64_STEP(3)
      }
    }
    // nothing may land in the buffers once they hold the output tiles
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
#undef MEGA_A64_STEP
#undef MEGA_SGB

  // epilogue as in gemm_kernel: the wave's 128 x 64 tile through its own LDS region
  uint16_t* stage = smem + wave * 128 * EP;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      const int row = i * 32 + (lane & 31);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int col = j * 32 + 8 * q4 + 4 * (lane >> 5);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = p.alpha * acc[i][j][4 * q4 + e];
        uint2 w;
        if (DT == MEGA_BF16) {
          w.x = pack_bf16x2(v[0], v[1]);
          w.y = pack_bf16x2(v[2], v[3]);
        } else {
          w.x = static_cast<uint32_t>(float_to_f16_bits(v[0])) | (static_cast<uint32_t>(float_to_f16_bits(v[1])) << 16);
          w.y = static_cast<uint32_t>(float_to_f16_bits(v[2])) | (static_cast<uint32_t>(float_to_f16_bits(v[3])) << 16);
        }
        *reinterpret_cast<uint2*>(stage + row * EP + col) = w;
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave reads back only its own region
  const bool vec_ok = (p.ldc % 8 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
#pragma unroll 4
  for (int i = 0; i < 8 * JN; ++i) {
    const int c = lane + kWave * i;
    const int row = c / (4 * JN), kc = (c % (4 * JN)) * 8;
    const int grow = m0 + wm * 128 + row, gcol = n0 + wn * (32 * JN) + kc;
    if (grow < p.M && gcol < p.N) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + row * EP + kc);
      uint16_t* dst = C + static_cast<int64_t>(grow) * p.ldc + gcol;
      if (vec_ok && gcol + 8 <= p.N) {
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));  // whole lines, read by a later kernel
      } else {
        const uint16_t* e = reinterpret_cast<const uint16_t*>(&v);
        for (int q = 0; q < 8; ++q)
          if (gcol + q < p.N) dst[q] = e[q];
      }
    }
  }
  // the output regions overlap the slab buffers: every read of this tile's epilogue
  // retires before the next tile's first slab is requested
  lds_barrier();
  }  // tile of the pair
  }  // work item
}

// ---- causal softmax over rows (in place), one wavefront per row ---------------
// `coff` < 0: every row keeps all L2 columns.  `coff` = L2 - L1 >= 0 (causal,
// bottom-right aligned, softmax.cuh:99-100): row r keeps columns [0, n) with
// n = r + 1 + coff.  The rest of the row is set to 0 -- with coff = 0 and
// `zfull` = 0 only up to the end of its 256-column tile, which is all the
// products of the fused attention read.
// softmax.cuh:86-131.
template <int DT, bool DROP>
__global__ __launch_bounds__(kThreads) void softmax_fwd_kernel(uint16_t* w, int L1, int L2,
                                                              int coff, int zfull, DropKey dk) {
  // grid.y carries the batch*heads index; grid.x covers the L1 rows
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const uint32_t row = blockIdx.y * static_cast<uint32_t>(L1) + r;
  uint16_t* x = w + (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  const int nz = (coff == 0 && !zfull) ? min(L2, (r / kTile + 1) * kTile) : L2;
  const auto score = [&](int j) {
    float v = Elem<DT>::load(x + j);
    if (DROP) {
      bool drops[4];
      dropkey_quad(dk, row, static_cast<uint32_t>(j) >> 2, drops);
      if (drops[j & 3]) v = -INFINITY;
    }
    return v;
  };
  float m = -INFINITY;
  for (int j = lane; j < n; j += kWave) m = fmaxf(m, score(j));
  m = wave_max(m);
  if (m == -INFINITY) m = 0.f;  // nothing kept: the row becomes 0 (softmax.cuh:113-116)
  float d = 0.f;
  for (int j = lane; j < n; j += kWave) d += __expf(score(j) - m);
  d = wave_sum(d);
  const float c = d == 0.f ? 0.f : 1.f / d;
  for (int j = lane; j < nz; j += kWave) {
    const float v = j < n ? __expf(score(j) - m) * c : 0.f;
    Elem<DT>::store(x + j, v);
  }
}


// Same contract with the row held in registers: needs L2 % 8 == 0, a 16-byte
// aligned base and L2 <= 64 * 8 * NCH; one read and one write of the row.
template <int DT, int NCH, bool DROP>
__global__ __launch_bounds__(kThreads) void softmax_fwd_vec_kernel(uint16_t* w, int L1, int L2,
                                                                  int coff, int zfull, DropKey dk) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const uint32_t row = blockIdx.y * static_cast<uint32_t>(L1) + r;
  uint16_t* x = w + (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  const int nz = (coff == 0 && !zfull) ? min(L2, (r / kTile + 1) * kTile) : L2;
  float v[NCH][8];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c8 = (lane + kWave * i) * 8;
    if (c8 < n) {
      unpack8<DT>(*reinterpret_cast<const uint4*>(x + c8), v[i]);
      if (DROP) {
        bool drops[8];
        dropkey_quad(dk, row, static_cast<uint32_t>(c8) >> 2, drops);
        dropkey_quad(dk, row, (static_cast<uint32_t>(c8) >> 2) + 1, drops + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (drops[e]) v[i][e] = -INFINITY;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (c8 + e >= n) v[i][e] = -INFINITY;
        m = fmaxf(m, v[i][e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] = -INFINITY;
    }
  }
  m = wave_max(m);
  if (m == -INFINITY) m = 0.f;  // nothing kept: the row becomes 0 (softmax.cuh:113-116)
  float d = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[i][e] = __expf(v[i][e] - m);  // exp(-inf) = 0 outside the kept prefix
      d += v[i][e];
    }
  d = wave_sum(d);
  const float c = d == 0.f ? 0.f : 1.f / d;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c8 = (lane + kWave * i) * 8;
    if (c8 < nz) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] *= c;
      *reinterpret_cast<uint4*>(x + c8) = pack8<DT>(v[i]);
    }
  }
}

// dS = P o (dP - sum_j P_j dP_j), written over dP.  softmax.cuh:198-234.
template <int DT>
__global__ __launch_bounds__(kThreads) void softmax_bwd_kernel(const uint16_t* w, uint16_t* dw,
                                                              int L1, int L2, int coff, int zfull) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const int64_t o = (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const uint16_t* pw = w + o;
  uint16_t* pd = dw + o;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  const int nz = (coff == 0 && !zfull) ? min(L2, (r / kTile + 1) * kTile) : L2;
  float s = 0.f;
  for (int j = lane; j < n; j += kWave) s += Elem<DT>::load(pw + j) * Elem<DT>::load(pd + j);
  s = wave_sum(s);
  for (int j = lane; j < nz; j += kWave) {
    const float v = j < n ? Elem<DT>::load(pw + j) * (Elem<DT>::load(pd + j) - s) : 0.f;
    Elem<DT>::store(pd + j, v);
  }
}

template <int DT, int NCH>
__global__ __launch_bounds__(kThreads) void softmax_bwd_vec_kernel(const uint16_t* w, uint16_t* dw,
                                                                  int L1, int L2, int coff, int zfull) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const int64_t o = (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const uint16_t* pw = w + o;
  uint16_t* pd = dw + o;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  const int nz = (coff == 0 && !zfull) ? min(L2, (r / kTile + 1) * kTile) : L2;
  float pv[NCH][8], dv[NCH][8];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c8 = (lane + kWave * i) * 8;
    if (c8 < n) {
      unpack8<DT>(*reinterpret_cast<const uint4*>(pw + c8), pv[i]);
      unpack8<DT>(*reinterpret_cast<const uint4*>(pd + c8), dv[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (c8 + e >= n) pv[i][e] = 0.f, dv[i][e] = 0.f;
        s += pv[i][e] * dv[i][e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) pv[i][e] = 0.f, dv[i][e] = 0.f;
    }
  }
  s = wave_sum(s);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c8 = (lane + kWave * i) * 8;
    if (c8 < nz) {
#pragma unroll
      for (int e = 0; e < 8; ++e) dv[i][e] = pv[i][e] * (dv[i][e] - s);
      *reinterpret_cast<uint4*>(pd + c8) = pack8<DT>(dv[i]);
    }
  }
}

template <int DT>
int launch_softmax(const uint16_t* p, uint16_t* x, int64_t Z, int64_t L1, int64_t L2, int causal,
                   hipStream_t s, int zfull = 0, const DropKey* drop = nullptr) {
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  // p == nullptr: forward over x in place; else backward with probabilities p
  if (Z == 0 || L1 == 0 || L2 == 0) return MEGA_OK;
  const dim3 grid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  const bool vec = L2 % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(p) % 16 == 0;
  const DropKey dk = drop ? *drop : DropKey{};
#define MEGA_SOFTMAX(NCH)                                                                        \
  if (p != nullptr)                                                                              \
    softmax_bwd_vec_kernel<DT, NCH><<<grid, kThreads, 0, s>>>(p, x, (int)L1, (int)L2, coff, zfull); \
  else if (drop)                                                                                 \
    softmax_fwd_vec_kernel<DT, NCH, true><<<grid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, zfull, dk); \
  else                                                                                           \
    softmax_fwd_vec_kernel<DT, NCH, false><<<grid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, zfull, dk);
  if (vec && L2 <= 512) {
    MEGA_SOFTMAX(1)
  } else if (vec && L2 <= 1024) {
    MEGA_SOFTMAX(2)
  } else if (vec && L2 <= 2048) {
    MEGA_SOFTMAX(4)
  } else if (vec && L2 <= 4096) {
    MEGA_SOFTMAX(8)
  } else if (p != nullptr) {
    softmax_bwd_kernel<DT><<<grid, kThreads, 0, s>>>(p, x, (int)L1, (int)L2, coff, zfull);
  } else if (drop) {
    softmax_fwd_kernel<DT, true><<<grid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, zfull, dk);
  } else {
    softmax_fwd_kernel<DT, false><<<grid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, zfull, dk);
  }
#undef MEGA_SOFTMAX
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

// ------------------------------ host side --------------------------------------
template <int DT, bool TA, bool TB>
int launch_gemm_t(const GemmParams& p, int batch, hipStream_t s) {
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const int64_t lim = 1ll << 30;  // elements: byte offsets stay below 2^31
  const bool fast_a = a16(p.A) && p.lda % 8 == 0 && p.sa0 % 8 == 0 && p.sa1 % 8 == 0 &&
                      (TA ? (p.M % 8 == 0 && p.M >= 8 && p.K * p.lda < lim) : p.M * p.lda < lim);
  const bool fast_b = a16(p.B) && p.ldb % 8 == 0 && p.sb0 % 8 == 0 && p.sb1 % 8 == 0 &&
                      (TB ? (p.N % 8 == 0 && p.N >= 8 && p.K * p.ldb < lim) : p.N * p.ldb < lim);
  const bool fast = fast_a && fast_b && p.K % kSlab == 0 && p.K >= kSlab;
  GemmParams q = p;
  q.mt_count = (p.M + kTile - 1) / kTile;
  q.nt_count = (p.N + kTile - 1) / kTile;
  int64_t per_batch;
  if (p.tri_out) {
    per_batch = 0;
    for (int m = 0; m < q.mt_count; ++m)
      per_batch += std::min<int64_t>(q.nt_count, (static_cast<int64_t>(m) * kTile + (kTile - 1) + p.off) / kTile + 1);
  } else if (p.k_mode) {
    per_batch = static_cast<int64_t>(q.nt_count) * ((q.mt_count + 1) / 2);
  } else {
    per_batch = static_cast<int64_t>(q.nt_count) * q.mt_count;
  }
  const int64_t items = per_batch * batch;
  MEGA_CHECK_ARG(items <= 0x7fffffff, "attention: too many tiles");
  q.per_batch = static_cast<int>(per_batch);
  q.items = static_cast<int>(items);
  int dev = 0, cus = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  // one workgroup per CU (its LDS and registers fill one); a multiple of the
  // XCD count whenever there are that many items
  int64_t g = std::min<int64_t>(items, cus);
  if (g >= kXcds) g -= g % kXcds;
  const dim3 grid(static_cast<unsigned>(g));
  const size_t lds = kGemmLds;
  // Aligned operands: slabs from memory straight into LDS, eight waves of 128 x 64.  Products of
  // two k-contiguous operands (S = Q K^T, dP = dY V^T) take slabs of 64 k; one k-contiguous and
  // one k-major operand (P V, dS K) take A in slabs of 64 k and B in slabs of 32 k; the rest
  // slabs of 32 k.
  bool done = false;
  if constexpr (!TA && !TB) {
    if (fast && p.K % kSlab64 == 0) {
      MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dma64_kernel<DT, TA, TB>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDmaLds));
      gemm_dma64_kernel<DT, TA, TB><<<grid, 2 * kThreads, kDmaLds, s>>>(q);
      done = true;
    }
  }
  if constexpr (!TA && TB) {
    if (fast && p.K % kSlab64 == 0) {
      MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dma_a64_kernel<DT>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kA64Lds));
      gemm_dma_a64_kernel<DT><<<grid, 2 * kThreads, kA64Lds, s>>>(q);
      done = true;
    }
  }
  if (!done && fast) {
    MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_dma_kernel<DT, TA, TB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDmaLds));
    gemm_dma_kernel<DT, TA, TB><<<grid, 2 * kThreads, kDmaLds, s>>>(q);
  } else if (!done) {
    MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<DT, TA, TB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    gemm_kernel<DT, TA, TB><<<grid, kThreads, lds, s>>>(q);
  }
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <int DT>
int launch_gemm(const GemmParams& p, int batch, hipStream_t s) {
  if (p.M == 0 || p.N == 0 || batch == 0) return MEGA_OK;
  if (p.ta) return p.tb ? launch_gemm_t<DT, true, true>(p, batch, s) : launch_gemm_t<DT, true, false>(p, batch, s);
  return p.tb ? launch_gemm_t<DT, false, true>(p, batch, s) : launch_gemm_t<DT, false, false>(p, batch, s);
}

struct AttnWs {
  int64_t dp, total;  // element offset of dP / dS, total bytes
};
AttnWs attn_ws(int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2, bool bwd) {
  AttnWs w;
  w.dp = 0;
  w.total = ((bwd ? B * NH * L1 * L2 : 0) + 8) * 2;
  return w;
}

int check_attn(const char* who, int dtype, int64_t B, int64_t L1, int64_t L2, int64_t NH,
               int64_t H1, int64_t H2, int causal) {
  MEGA_CHECK_ARG(valid_dtype(dtype) || dtype == MEGA_F64, "%s: unknown dtype %d", who, dtype);
  MEGA_CHECK_ARG(B >= 0 && L1 >= 0 && L2 >= 0 && NH >= 1 && H1 >= 1 && H2 >= 1, "%s: bad sizes", who);
  MEGA_CHECK_ARG(B * NH <= 65535, "%s: batch * heads exceeds 65535", who);
  MEGA_CHECK_ARG(L1 <= (1 << 24) && L2 <= (1 << 24), "%s: sequence too long", who);
  MEGA_CHECK_ARG(causal >= 0 && causal <= 2, "%s: causal must be 0, 1 or 2", who);
  MEGA_CHECK_ARG(!causal || L2 >= L1,
                 "%s: causal attention needs L2 >= L1 (row r sees keys 0 .. L2 - L1 + r)", who);
  return MEGA_OK;
}

template <int DT>
int attn_fwd_impl(const uint16_t* q, const uint16_t* k, const uint16_t* v, int64_t B, int64_t L1,
                  int64_t L2, int64_t NH, int64_t H1, int64_t H2, float scale, int causal,
                  uint16_t* y, uint16_t* w, uint16_t* ws, hipStream_t s, const DropKey* drop, int fill) {
  (void)ws;
  const int Z = static_cast<int>(B * NH);
  int rc = drop ? -1 : attention_probs_fused(DT, q, k, w, B, L1, L2, NH, H1, scale, causal, fill, s);
  if (rc > 0) return rc;
  if (rc < 0) {
  // S = scale Q K^T  -> w
  GemmParams g{};
  g.A = q; g.B = k; g.C = w; g.M = (int)L1; g.N = (int)L2; g.K = (int)H1;
  g.lda = NH * H1; g.ldb = NH * H1; g.ldc = L2;
  g.sa0 = L1 * NH * H1; g.sa1 = H1; g.sb0 = L2 * NH * H1; g.sb1 = H1;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = scale;
  g.tri_out = causal; g.k_mode = 0; g.off = causal ? (int)(L2 - L1) : 0;
  if ((rc = launch_gemm<DT>(g, Z, s)) != MEGA_OK) return rc;
  // P = softmax(S) in place
  if ((rc = launch_softmax<DT>(nullptr, w, Z, L1, L2, causal, s, fill, drop)) != MEGA_OK) return rc;
  }
  // Y = P V: V[key][c] is the k-major B operand
  GemmParams o{};
  o.A = w; o.B = v; o.C = y; o.M = (int)L1; o.N = (int)H2; o.K = (int)L2;
  o.lda = L2; o.ldb = NH * H2; o.ldc = NH * H2; o.tb = 1;
  o.sa0 = NH * L1 * L2; o.sa1 = L1 * L2; o.sb0 = L2 * NH * H2; o.sb1 = H2;
  o.sc0 = L1 * NH * H2; o.sc1 = H2; o.nh = (int)NH; o.alpha = 1.f;
  o.tri_out = 0; o.k_mode = causal ? 1 : 0; o.off = causal ? (int)(L2 - L1) : 0;
  return launch_gemm<DT>(o, Z, s);
}

template <int DT>
int attn_bwd_impl(const uint16_t* dy, const uint16_t* q, const uint16_t* k, const uint16_t* v,
                  const uint16_t* w, int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1,
                  int64_t H2, float scale, int causal, uint16_t* dq, uint16_t* dk, uint16_t* dv,
                  uint16_t* ws, hipStream_t s) {
  const AttnWs l = attn_ws(B, L1, L2, NH, H1, H2, true);
  const int Z = static_cast<int>(B * NH);
  uint16_t* dp = ws + l.dp;
  int rc;
  // dP = dY V^T
  GemmParams g{};
  g.A = dy; g.B = v; g.C = dp; g.M = (int)L1; g.N = (int)L2; g.K = (int)H2;
  g.lda = NH * H2; g.ldb = NH * H2; g.ldc = L2;
  g.sa0 = L1 * NH * H2; g.sa1 = H2; g.sb0 = L2 * NH * H2; g.sb1 = H2;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = 1.f;
  g.tri_out = causal; g.k_mode = 0; g.off = causal ? (int)(L2 - L1) : 0;
  if ((rc = launch_gemm<DT>(g, Z, s)) != MEGA_OK) return rc;
  // dS = P o (dP - rowsum(P o dP)) in place
  if ((rc = launch_softmax<DT>(w, dp, Z, L1, L2, causal, s)) != MEGA_OK) return rc;
  // dQ = scale dS K: K[key][h] is the k-major B operand
  GemmParams a{};
  a.A = dp; a.B = k; a.C = dq; a.M = (int)L1; a.N = (int)H1; a.K = (int)L2;
  a.lda = L2; a.ldb = NH * H1; a.ldc = NH * H1; a.tb = 1;
  a.sa0 = NH * L1 * L2; a.sa1 = L1 * L2; a.sb0 = L2 * NH * H1; a.sb1 = H1;
  a.sc0 = L1 * NH * H1; a.sc1 = H1; a.nh = (int)NH; a.alpha = scale; a.k_mode = causal ? 1 : 0; a.off = causal ? (int)(L2 - L1) : 0;
  if ((rc = launch_gemm<DT>(a, Z, s)) != MEGA_OK) return rc;
  // dK = scale dS^T Q: dS[q][key] and Q[q][h] are both k-major (k = q)
  GemmParams b{};
  b.A = dp; b.B = q; b.C = dk; b.M = (int)L2; b.N = (int)H1; b.K = (int)L1;
  b.lda = L2; b.ldb = NH * H1; b.ldc = NH * H1; b.ta = 1; b.tb = 1;
  b.sa0 = NH * L1 * L2; b.sa1 = L1 * L2; b.sb0 = L1 * NH * H1; b.sb1 = H1;
  b.sc0 = L2 * NH * H1; b.sc1 = H1; b.nh = (int)NH; b.alpha = scale; b.k_mode = causal ? 2 : 0; b.off = causal ? (int)(L2 - L1) : 0;
  if ((rc = launch_gemm<DT>(b, Z, s)) != MEGA_OK) return rc;
  // dV = P^T dY: P[q][key] and dY[q][c] are both k-major (k = q)
  GemmParams c{};
  c.A = w; c.B = dy; c.C = dv; c.M = (int)L2; c.N = (int)H2; c.K = (int)L1;
  c.lda = L2; c.ldb = NH * H2; c.ldc = NH * H2; c.ta = 1; c.tb = 1;
  c.sa0 = NH * L1 * L2; c.sa1 = L1 * L2; c.sb0 = L1 * NH * H2; c.sb1 = H2;
  c.sc0 = L2 * NH * H2; c.sc1 = H2; c.nh = (int)NH; c.alpha = 1.f; c.k_mode = causal ? 2 : 0; c.off = causal ? (int)(L2 - L1) : 0;
  return launch_gemm<DT>(c, Z, s);
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int64_t mega_attention_workspace_bytes(int64_t B, int64_t L1, int64_t L2, int64_t NH,
                                                  int64_t H1, int64_t H2, int backward) {
  if (B < 0 || L1 < 0 || L2 < 0 || NH < 1 || H1 < 1 || H2 < 1) return 16;
  return attn_ws(B, L1, L2, NH, H1, H2, backward != 0).total;
}

// p in [0, 1]; p == 0 means no DropKey
static int make_dropkey(const char* who, double dropout, uint64_t seed, uint64_t offset, int64_t rows,
                        DropKey* dk) {
  MEGA_CHECK_ARG(dropout >= 0.0 && dropout <= 1.0, "%s: dropout must lie in [0, 1]", who);
  MEGA_CHECK_ARG(rows < (1ll << 32), "%s: more than 2^32 rows", who);
  dk->p = static_cast<float>(dropout);
  dk->seed_lo = static_cast<uint32_t>(seed);
  dk->seed_hi = static_cast<uint32_t>(seed >> 32);
  dk->off_lo = static_cast<uint32_t>(offset);
  dk->off_hi = static_cast<uint32_t>(offset >> 32);
  return MEGA_OK;
}

static int attention_fwd_entry(const char* who, const void* q, const void* k, const void* v, int dtype,
                               int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2,
                               double scale, int causal, const DropKey* drop, void* y, void* w,
                               void* workspace, void* stream) {
  int rc = check_attn(who, dtype, B, L1, L2, NH, H1, H2, causal);
  if (rc != MEGA_OK) return rc;
  if (B == 0 || L1 == 0) return MEGA_OK;
  MEGA_CHECK_ARG(q && k && v && y && w && workspace, "%s: null pointer", who);
  MEGA_CHECK_ARG(L2 >= 1, "%s: no keys", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // causal == 2: as 1, but w need only hold what mega_attention_bwd reads
  const int fill = causal == 2 ? 0 : 1;
  causal = causal != 0;
  if (dtype == MEGA_F32)
    return attention_wide_fwd<float>(static_cast<const float*>(q), static_cast<const float*>(k),
                                     static_cast<const float*>(v), B, L1, L2, NH, H1, H2, scale, causal, drop,
                                     static_cast<float*>(y), static_cast<float*>(w), s);
  if (dtype == MEGA_F64)
    return attention_wide_fwd<double>(static_cast<const double*>(q), static_cast<const double*>(k),
                                      static_cast<const double*>(v), B, L1, L2, NH, H1, H2, scale, causal, drop,
                                      static_cast<double*>(y), static_cast<double*>(w), s);
  auto u = [](const void* p) { return static_cast<const uint16_t*>(p); };
  auto m = [](void* p) { return static_cast<uint16_t*>(p); };
  if (dtype == MEGA_BF16)
    return attn_fwd_impl<MEGA_BF16>(u(q), u(k), u(v), B, L1, L2, NH, H1, H2, (float)scale, causal,
                                    m(y), m(w), m(workspace), s, drop, fill);
  return attn_fwd_impl<MEGA_F16>(u(q), u(k), u(v), B, L1, L2, NH, H1, H2, (float)scale, causal,
                                 m(y), m(w), m(workspace), s, drop, fill);
}

extern "C" int mega_attention_fwd(const void* q, const void* k, const void* v, int dtype, int64_t B,
                                  int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2,
                                  double scale, int causal, void* y, void* w, void* workspace,
                                  void* stream) {
  return attention_fwd_entry("mega_attention_fwd", q, k, v, dtype, B, L1, L2, NH, H1, H2, scale,
                             causal, nullptr, y, w, workspace, stream);
}

extern "C" int mega_attention_dropkey_fwd(const void* q, const void* k, const void* v, int dtype,
                                          int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1,
                                          int64_t H2, double scale, int causal, double dropout,
                                          uint64_t seed, uint64_t offset, void* y, void* w,
                                          void* workspace, void* stream) {
  DropKey dk;
  int rc = make_dropkey("mega_attention_dropkey_fwd", dropout, seed, offset,
                        B >= 0 && NH >= 0 && L1 >= 0 ? B * NH * L1 : 0, &dk);
  if (rc != MEGA_OK) return rc;
  return attention_fwd_entry("mega_attention_dropkey_fwd", q, k, v, dtype, B, L1, L2, NH, H1, H2,
                             scale, causal, dropout > 0.0 ? &dk : nullptr, y, w, workspace, stream);
}

extern "C" int mega_attention_bwd(const void* dy, const void* q, const void* k, const void* v,
                                  const void* w, int dtype, int64_t B, int64_t L1, int64_t L2,
                                  int64_t NH, int64_t H1, int64_t H2, double scale, int causal,
                                  void* dq, void* dk, void* dv, void* workspace, void* stream) {
  int rc = check_attn("mega_attention_bwd", dtype, B, L1, L2, NH, H1, H2, causal);
  if (rc != MEGA_OK) return rc;
  if (B == 0) return MEGA_OK;
  MEGA_CHECK_ARG(dy && q && k && v && w && dq && dk && dv && workspace,
                 "mega_attention_bwd: null pointer");
  MEGA_CHECK_ARG(L1 >= 1 && L2 >= 1, "mega_attention_bwd: empty sequence");
  hipStream_t s = static_cast<hipStream_t>(stream);
  causal = causal != 0;  // the forward's 1 and 2 are the same mask
  if (dtype == MEGA_F32)
    return attention_wide_bwd<float>(static_cast<const float*>(dy), static_cast<const float*>(q),
                                     static_cast<const float*>(k), static_cast<const float*>(v),
                                     static_cast<const float*>(w), B, L1, L2, NH, H1, H2, scale, causal,
                                     static_cast<float*>(dq), static_cast<float*>(dk), static_cast<float*>(dv),
                                     static_cast<float*>(workspace), s);
  if (dtype == MEGA_F64)
    return attention_wide_bwd<double>(static_cast<const double*>(dy), static_cast<const double*>(q),
                                      static_cast<const double*>(k), static_cast<const double*>(v),
                                      static_cast<const double*>(w), B, L1, L2, NH, H1, H2, scale, causal,
                                      static_cast<double*>(dq), static_cast<double*>(dk), static_cast<double*>(dv),
                                      static_cast<double*>(workspace), s);
  auto u = [](const void* p) { return static_cast<const uint16_t*>(p); };
  auto m = [](void* p) { return static_cast<uint16_t*>(p); };
  if (dtype == MEGA_BF16)
    return attn_bwd_impl<MEGA_BF16>(u(dy), u(q), u(k), u(v), u(w), B, L1, L2, NH, H1, H2,
                                    (float)scale, causal, m(dq), m(dk), m(dv), m(workspace), s);
  return attn_bwd_impl<MEGA_F16>(u(dy), u(q), u(k), u(v), u(w), B, L1, L2, NH, H1, H2,
                                 (float)scale, causal, m(dq), m(dk), m(dv), m(workspace), s);
}

// ---- the weight gradient of a linear layer on the same product kernel ---------------
extern "C" int mega_linear_weight_grad(const void* dy, const void* x, int dtype, int64_t tokens, int64_t n_out,
                                       int64_t n_in, void* dw, void* stream) {
  MEGA_CHECK_ARG(dtype == MEGA_BF16 || dtype == MEGA_F16, "mega_linear_weight_grad: bfloat16 or float16 tensors");
  MEGA_CHECK_ARG(tokens >= 1 && n_out >= 1 && n_in >= 1 && tokens < (1ll << 31) && n_out < (1ll << 31) &&
                     n_in < (1ll << 31),
                 "mega_linear_weight_grad: bad sizes");
  MEGA_CHECK_ARG(dy && x && dw, "mega_linear_weight_grad: null pointer");
  // dw[o][i] = sum_t dy[t][o] x[t][i]: both operands k-major (k = tokens)
  GemmParams g{};
  g.A = static_cast<const uint16_t*>(dy);
  g.B = static_cast<const uint16_t*>(x);
  g.C = static_cast<uint16_t*>(dw);
  g.M = (int)n_out; g.N = (int)n_in; g.K = (int)tokens;
  g.lda = n_out; g.ldb = n_in; g.ldc = n_in; g.ta = 1; g.tb = 1;
  g.nh = 1; g.alpha = 1.f;
  g.n_group = 8;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == MEGA_BF16 ? launch_gemm<MEGA_BF16>(g, 1, s) : launch_gemm<MEGA_F16>(g, 1, s);
}

// ---- standalone causal softmax ---------------------------------------------------
static int check_softmax(const char* who, int dtype, int64_t Z, int64_t L1, int64_t L2, int causal) {
  MEGA_CHECK_ARG(valid_dtype(dtype) || dtype == MEGA_F64, "%s: unknown dtype %d", who, dtype);
  MEGA_CHECK_ARG(Z >= 0 && L1 >= 0 && L2 >= 0, "%s: bad sizes", who);
  MEGA_CHECK_ARG(Z <= 65535, "%s: more than 65535 matrices", who);
  MEGA_CHECK_ARG(L1 <= (1 << 24) && L2 <= (1 << 24), "%s: rows too long", who);
  MEGA_CHECK_ARG(!causal || L2 >= L1, "%s: causal softmax needs L2 >= L1", who);
  return MEGA_OK;
}

static int softmax_fwd_entry(const char* who, void* x, int dtype, int64_t Z, int64_t L1, int64_t L2,
                             int causal, const DropKey* drop, void* stream) {
  int rc = check_softmax(who, dtype, Z, L1, L2, causal);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG(x != nullptr || Z * L1 * L2 == 0, "%s: null pointer", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32) return softmax_wide_fwd<float>(static_cast<float*>(x), Z, L1, L2, causal, drop, s);
  if (dtype == MEGA_F64) return softmax_wide_fwd<double>(static_cast<double*>(x), Z, L1, L2, causal, drop, s);
  if (dtype == MEGA_BF16)
    return launch_softmax<MEGA_BF16>(nullptr, static_cast<uint16_t*>(x), Z, L1, L2, causal, s, 1, drop);
  return launch_softmax<MEGA_F16>(nullptr, static_cast<uint16_t*>(x), Z, L1, L2, causal, s, 1, drop);
}

extern "C" int mega_attention_softmax_fwd(void* x, int dtype, int64_t Z, int64_t L1, int64_t L2,
                                          int causal, void* stream) {
  return softmax_fwd_entry("mega_attention_softmax_fwd", x, dtype, Z, L1, L2, causal, nullptr, stream);
}

extern "C" int mega_attention_softmax_dropkey_fwd(void* x, int dtype, int64_t Z, int64_t L1,
                                                  int64_t L2, int causal, double dropout,
                                                  uint64_t seed, uint64_t offset, void* stream) {
  DropKey dk;
  int rc = make_dropkey("mega_attention_softmax_dropkey_fwd", dropout, seed, offset,
                        Z >= 0 && L1 >= 0 ? Z * L1 : 0, &dk);
  if (rc != MEGA_OK) return rc;
  return softmax_fwd_entry("mega_attention_softmax_dropkey_fwd", x, dtype, Z, L1, L2, causal,
                           dropout > 0.0 ? &dk : nullptr, stream);
}

extern "C" int mega_attention_softmax_bwd(const void* y, void* dy, int dtype, int64_t Z, int64_t L1,
                                          int64_t L2, int causal, void* stream) {
  int rc = check_softmax("mega_attention_softmax_bwd", dtype, Z, L1, L2, causal);
  if (rc != MEGA_OK) return rc;
  MEGA_CHECK_ARG((y != nullptr && dy != nullptr) || Z * L1 * L2 == 0,
                 "mega_attention_softmax_bwd: null pointer");
  if (Z * L1 * L2 == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MEGA_F32)
    return softmax_wide_bwd<float>(static_cast<const float*>(y), static_cast<float*>(dy), Z, L1, L2, causal, s);
  if (dtype == MEGA_F64)
    return softmax_wide_bwd<double>(static_cast<const double*>(y), static_cast<double*>(dy), Z, L1, L2, causal, s);
  if (dtype == MEGA_BF16)
    return launch_softmax<MEGA_BF16>(static_cast<const uint16_t*>(y), static_cast<uint16_t*>(dy), Z, L1,
                                     L2, causal, s, 1);
  return launch_softmax<MEGA_F16>(static_cast<const uint16_t*>(y), static_cast<uint16_t*>(dy), Z, L1, L2,
                                  causal, s, 1);
}
