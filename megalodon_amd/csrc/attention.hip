// Chunk-causal attention for gfx950 (bf16 / fp16, fp32 accumulation on MFMA).
//
// Semantics follow the reference operator
//   megalodon/csrc/ops/attention_kernel.cu:40-133 (forward), :135-257 (backward)
//   megalodon/csrc/softmax.cuh:86-131,198-234 (causal softmax forward / backward):
//   S = scale * Q K^T rounded to the element type, P = softmax_fp32(S) over the
//   causal prefix (row r sees columns 0..r), P stored in the element type,
//   Y = P V;  dV = P^T dY, dP = dY V^T, dS = P o (dP - rowsum(P o dP)),
//   dQ = scale dS K, dK = scale dS^T Q.  Layout BLNH in and out; w = P is
//   returned (B, N, L1, L2) as the reference does.
//
// Differences in execution: the reference runs full-square cuBLAS GEMMs and a
// full-row softmax; here every product is one hand-written MFMA GEMM
// (v_mfma_f32_32x32x16, 256x256 workgroup tile, 128x128 per wavefront,
// double-buffered LDS staging of 64-wide k slabs) that skips the tiles above
// the causal diagonal and the k-ranges where P / dS are structurally zero, so
// causal attention costs half the flops and half the P traffic.  Operands whose
// reduction index is not the contiguous one (V, dY, K, Q, P, dS in the
// backward products) are transposed first by a tiled copy kernel; the GEMM
// itself only ever sees k-contiguous rows, which is the form the MFMA operand
// registers want (8 consecutive k per lane).
#include "common.hpp"

namespace mega {
namespace {

constexpr int kTile = 256;     // workgroup tile (M and N)
constexpr int kSlab = 64;      // k elements staged per iteration
constexpr int kPitch = kSlab + 8;  // LDS row pitch in elements (144 B: conflict-free 16 B reads)
constexpr int kThreads = 256;

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <int DT> struct Mma;
template <> struct Mma<MEGA_BF16> {
  static __device__ __forceinline__ floatx16 run(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<MEGA_F16> {
  static __device__ __forceinline__ floatx16 run(uint4 a, uint4 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

// C[m][n] = alpha * sum_k A[m][k] B[n][k]   (both operands k-contiguous)
struct GemmParams {
  const uint16_t* A;
  const uint16_t* B;
  uint16_t* C;
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t sa0, sa1, sb0, sb1, sc0, sc1;  // batch z = z0 * nh + z1 -> offset z0*s0 + z1*s1
  int nh;
  float alpha;
  int tri_out;  // 1: tiles with nt > mt are skipped (left unwritten)
  int k_mode;   // 0: all k; 1: k < (mt+1)*256; 2: k >= mt*256
};

template <bool ALIGNED>
__device__ __forceinline__ uint4 load_chunk(const uint16_t* base, int64_t ld, int row, int rows,
                                            int k, int kend) {
  uint4 v = make_uint4(0, 0, 0, 0);
  if (row < rows && k < kend) {
    const uint16_t* p = base + static_cast<int64_t>(row) * ld + k;
    if (ALIGNED && k + 8 <= kend) {
      v = *reinterpret_cast<const uint4*>(p);
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

template <int DT, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void gemm_tn_kernel(const GemmParams p) {
  extern __shared__ __align__(16) uint16_t smem[];
  // [buf][A|B][256][kPitch]
  constexpr int kOperand = kTile * kPitch;
  const int mt = blockIdx.y, nt = blockIdx.x;
  if (p.tri_out && nt > mt) return;
  const int z0 = blockIdx.z / p.nh, z1 = blockIdx.z % p.nh;
  const uint16_t* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const uint16_t* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  uint16_t* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  const int m0 = mt * kTile, n0 = nt * kTile;
  int kb = 0, ke = p.K;
  if (p.k_mode == 1) ke = min(p.K, (mt + 1) * kTile);
  if (p.k_mode == 2) kb = min(p.K, mt * kTile);

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;

  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 ra[8], rb[8];
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = tid + kThreads * i;
      const int row = c >> 3, kc = (c & 7) * 8;
      ra[i] = load_chunk<ALIGNED>(A, p.lda, m0 + row, p.M, k0 + kc, ke);
      rb[i] = load_chunk<ALIGNED>(B, p.ldb, n0 + row, p.N, k0 + kc, ke);
    }
  };
  auto sstore = [&](int buf) {
    uint16_t* sa = smem + buf * 2 * kOperand;
    uint16_t* sb = sa + kOperand;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = tid + kThreads * i;
      const int row = c >> 3, kc = (c & 7) * 8;
      *reinterpret_cast<uint4*>(sa + row * kPitch + kc) = ra[i];
      *reinterpret_cast<uint4*>(sb + row * kPitch + kc) = rb[i];
    }
  };

  if (kb < ke) {
    gload(kb);
    sstore(0);
  }
  __syncthreads();
  int buf = 0;
  for (int k0 = kb; k0 < ke; k0 += kSlab) {
    const bool more = k0 + kSlab < ke;
    if (more) gload(k0 + kSlab);
    const uint16_t* sa = smem + buf * 2 * kOperand + (wm * 128 + (lane & 31)) * kPitch + 8 * (lane >> 5);
    const uint16_t* sb = smem + buf * 2 * kOperand + kOperand + (wn * 128 + (lane & 31)) * kPitch + 8 * (lane >> 5);
#pragma unroll
    for (int ks = 0; ks < kSlab / 16; ++ks) {
      uint4 fa[4], fb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        fa[i] = *reinterpret_cast<const uint4*>(sa + i * 32 * kPitch + ks * 16);
        fb[i] = *reinterpret_cast<const uint4*>(sb + i * 32 * kPitch + ks * 16);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = Mma<DT>::run(fa[i], fb[j], acc[i][j]);
    }
    if (more) sstore(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  // epilogue: D[i][j] of a 32x32 tile sits in lane (j = lane % 32), register
  // r -> i = 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + wn * 128 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row < p.M && col < p.N) {
          const float v = p.alpha * acc[i][j][r];
          C[static_cast<int64_t>(row) * p.ldc + col] =
              DT == MEGA_BF16 ? float_to_bf16_bits(v) : float_to_f16_bits(v);
        }
      }
    }
  }
}

// ---- causal softmax over rows (in place), one wavefront per row ---------------
// row r of matrix z keeps columns [0, n) with n = causal ? r + 1 : L2; the rest
// of the row up to the end of its 256-column tile is set to 0 (that is all the
// later products read).  softmax.cuh:86-131.
template <int DT>
__global__ __launch_bounds__(kThreads) void softmax_fwd_kernel(uint16_t* w, int L1, int L2,
                                                              int causal) {
  // grid.y carries the batch*heads index; grid.x covers the L1 rows
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  uint16_t* x = w + (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const int n = causal ? min(r + 1, L2) : L2;
  const int nz = causal ? min(L2, (r / kTile + 1) * kTile) : L2;
  float m = -INFINITY;
  for (int j = lane; j < n; j += kWave) m = fmaxf(m, Elem<DT>::load(x + j));
  m = wave_max(m);
  float d = 0.f;
  for (int j = lane; j < n; j += kWave) d += __expf(Elem<DT>::load(x + j) - m);
  d = wave_sum(d);
  const float c = d == 0.f ? 0.f : 1.f / d;
  for (int j = lane; j < nz; j += kWave) {
    const float v = j < n ? __expf(Elem<DT>::load(x + j) - m) * c : 0.f;
    Elem<DT>::store(x + j, v);
  }
}

// dS = P o (dP - sum_j P_j dP_j), written over dP.  softmax.cuh:198-234.
template <int DT>
__global__ __launch_bounds__(kThreads) void softmax_bwd_kernel(const uint16_t* w, uint16_t* dw,
                                                              int L1, int L2, int causal) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const int64_t o = (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const uint16_t* pw = w + o;
  uint16_t* pd = dw + o;
  const int n = causal ? min(r + 1, L2) : L2;
  const int nz = causal ? min(L2, (r / kTile + 1) * kTile) : L2;
  float s = 0.f;
  for (int j = lane; j < n; j += kWave) s += Elem<DT>::load(pw + j) * Elem<DT>::load(pd + j);
  s = wave_sum(s);
  for (int j = lane; j < nz; j += kWave) {
    const float v = j < n ? Elem<DT>::load(pw + j) * (Elem<DT>::load(pd + j) - s) : 0.f;
    Elem<DT>::store(pd + j, v);
  }
}

// ---- batched transpose of 16-bit matrices: out[z][c][r] = in[z][r][c] ----------
struct TransParams {
  const uint16_t* in;
  uint16_t* out;
  int R, Cc;
  int64_t ldi, ldo;
  int64_t si0, si1, so0, so1;
  int nh;
  int tri;  // 1: only 256-blocks with column block <= row block are copied
};
__global__ __launch_bounds__(256) void transpose_kernel(const TransParams p) {
  __shared__ uint16_t tile[64][66];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  if (p.tri && (c0 / kTile) > (r0 / kTile)) return;
  const int z0 = blockIdx.z / p.nh, z1 = blockIdx.z % p.nh;
  const uint16_t* in = p.in + z0 * p.si0 + z1 * p.si1;
  uint16_t* out = p.out + z0 * p.so0 + z1 * p.so1;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < p.R && c < p.Cc) ? in[static_cast<int64_t>(r) * p.ldi + c] : static_cast<uint16_t>(0);
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, r = r0 + tx;
    if (c < p.Cc && r < p.R) out[static_cast<int64_t>(c) * p.ldo + r] = tile[tx][i];
  }
}

// ------------------------------ host side --------------------------------------
template <int DT>
int launch_gemm(const GemmParams& p, int batch, hipStream_t s) {
  if (p.M == 0 || p.N == 0 || batch == 0) return MEGA_OK;
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool aligned = a16(p.A) && a16(p.B) && p.lda % 8 == 0 && p.ldb % 8 == 0 && p.sa0 % 8 == 0 &&
                       p.sa1 % 8 == 0 && p.sb0 % 8 == 0 && p.sb1 % 8 == 0;
  const dim3 grid((p.N + kTile - 1) / kTile, (p.M + kTile - 1) / kTile, batch);
  const size_t lds = sizeof(uint16_t) * 2 * 2 * kTile * kPitch;
  if (aligned) {
    MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tn_kernel<DT, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    gemm_tn_kernel<DT, true><<<grid, kThreads, lds, s>>>(p);
  } else {
    MEGA_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tn_kernel<DT, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    gemm_tn_kernel<DT, false><<<grid, kThreads, lds, s>>>(p);
  }
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

int launch_transpose(const TransParams& p, int batch, hipStream_t s) {
  if (p.R == 0 || p.Cc == 0 || batch == 0) return MEGA_OK;
  const dim3 grid((p.Cc + 63) / 64, (p.R + 63) / 64, batch);
  transpose_kernel<<<grid, 256, 0, s>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

inline int64_t up8(int64_t v) { return (v + 7) / 8 * 8; }

struct AttnWs {
  int64_t ld1, ld2;  // padded leading dimensions of transposed buffers (>= L1, L2)
  int64_t vt, dp, kt, qt, dot, pt, dst, total;  // element offsets
};
AttnWs attn_ws(int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2, bool bwd) {
  AttnWs w;
  w.ld1 = up8(L1);
  w.ld2 = up8(L2);
  int64_t o = 0;
  const int64_t Z = B * NH;
  w.vt = o; o += bwd ? 0 : Z * H2 * w.ld2;
  w.dp = o; o += bwd ? Z * L1 * L2 : 0;
  w.kt = o; o += bwd ? Z * H1 * w.ld2 : 0;
  w.qt = o; o += bwd ? Z * H1 * w.ld1 : 0;
  w.dot = o; o += bwd ? Z * H2 * w.ld1 : 0;
  w.pt = o; o += bwd ? Z * L2 * w.ld1 : 0;
  w.dst = o; o += bwd ? Z * L2 * w.ld1 : 0;
  w.total = (o + 8) * 2;
  return w;
}

int check_attn(const char* who, int dtype, int64_t B, int64_t L1, int64_t L2, int64_t NH,
               int64_t H1, int64_t H2, int causal) {
  if (dtype != MEGA_BF16 && dtype != MEGA_F16)
    return set_error(MEGA_ERR_UNSUPPORTED, "%s: only bfloat16 / float16 tensors are supported", who);
  MEGA_CHECK_ARG(B >= 0 && L1 >= 0 && L2 >= 0 && NH >= 1 && H1 >= 1 && H2 >= 1, "%s: bad sizes", who);
  MEGA_CHECK_ARG(B * NH <= 65535, "%s: batch * heads exceeds 65535", who);
  MEGA_CHECK_ARG(L1 <= (1 << 24) && L2 <= (1 << 24), "%s: sequence too long", who);
  if (causal && L1 != L2)
    return set_error(MEGA_ERR_UNSUPPORTED,
                     "%s: causal attention with L1 != L2 (key/value cache prefix) is not implemented", who);
  return MEGA_OK;
}

template <int DT>
int attn_fwd_impl(const uint16_t* q, const uint16_t* k, const uint16_t* v, int64_t B, int64_t L1,
                  int64_t L2, int64_t NH, int64_t H1, int64_t H2, float scale, int causal,
                  uint16_t* y, uint16_t* w, uint16_t* ws, hipStream_t s) {
  const AttnWs l = attn_ws(B, L1, L2, NH, H1, H2, false);
  const int Z = static_cast<int>(B * NH);
  // S = scale Q K^T  -> w
  GemmParams g{};
  g.A = q; g.B = k; g.C = w; g.M = (int)L1; g.N = (int)L2; g.K = (int)H1;
  g.lda = NH * H1; g.ldb = NH * H1; g.ldc = L2;
  g.sa0 = L1 * NH * H1; g.sa1 = H1; g.sb0 = L2 * NH * H1; g.sb1 = H1;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = scale;
  g.tri_out = causal; g.k_mode = 0;
  int rc = launch_gemm<DT>(g, Z, s);
  if (rc != MEGA_OK) return rc;
  // P = softmax(S) in place
  {
    const dim3 grid((unsigned)((L1 + 3) / 4), (unsigned)Z);
    softmax_fwd_kernel<DT><<<grid, kThreads, 0, s>>>(w, (int)L1, (int)L2, causal);
    MEGA_CHECK_LAUNCH();
  }
  // Vt[z][c][key]
  uint16_t* vt = ws + l.vt;
  TransParams t{};
  t.in = v; t.out = vt; t.R = (int)L2; t.Cc = (int)H2; t.ldi = NH * H2; t.ldo = l.ld2;
  t.si0 = L2 * NH * H2; t.si1 = H2; t.so0 = NH * H2 * l.ld2; t.so1 = H2 * l.ld2; t.nh = (int)NH;
  rc = launch_transpose(t, Z, s);
  if (rc != MEGA_OK) return rc;
  // Y = P Vt^T
  GemmParams o{};
  o.A = w; o.B = vt; o.C = y; o.M = (int)L1; o.N = (int)H2; o.K = (int)L2;
  o.lda = L2; o.ldb = l.ld2; o.ldc = NH * H2;
  o.sa0 = NH * L1 * L2; o.sa1 = L1 * L2; o.sb0 = NH * H2 * l.ld2; o.sb1 = H2 * l.ld2;
  o.sc0 = L1 * NH * H2; o.sc1 = H2; o.nh = (int)NH; o.alpha = 1.f;
  o.tri_out = 0; o.k_mode = causal ? 1 : 0;
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
  uint16_t* kt = ws + l.kt;
  uint16_t* qt = ws + l.qt;
  uint16_t* dot = ws + l.dot;
  uint16_t* pt = ws + l.pt;
  uint16_t* dst = ws + l.dst;
  int rc;
  // dP = dY V^T
  GemmParams g{};
  g.A = dy; g.B = v; g.C = dp; g.M = (int)L1; g.N = (int)L2; g.K = (int)H2;
  g.lda = NH * H2; g.ldb = NH * H2; g.ldc = L2;
  g.sa0 = L1 * NH * H2; g.sa1 = H2; g.sb0 = L2 * NH * H2; g.sb1 = H2;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = 1.f;
  g.tri_out = causal; g.k_mode = 0;
  if ((rc = launch_gemm<DT>(g, Z, s)) != MEGA_OK) return rc;
  // dS = P o (dP - rowsum(P o dP)) in place
  {
    const dim3 grid((unsigned)((L1 + 3) / 4), (unsigned)Z);
    softmax_bwd_kernel<DT><<<grid, kThreads, 0, s>>>(w, dp, (int)L1, (int)L2, causal);
    MEGA_CHECK_LAUNCH();
  }
  // transposes: Kt[z][h][key], Qt[z][h][q], dYt[z][c][q], Pt[z][key][q], dSt[z][key][q]
  TransParams t{};
  t.nh = (int)NH;
  t.in = k; t.out = kt; t.R = (int)L2; t.Cc = (int)H1; t.ldi = NH * H1; t.ldo = l.ld2;
  t.si0 = L2 * NH * H1; t.si1 = H1; t.so0 = NH * H1 * l.ld2; t.so1 = H1 * l.ld2; t.tri = 0;
  if ((rc = launch_transpose(t, Z, s)) != MEGA_OK) return rc;
  t.in = q; t.out = qt; t.R = (int)L1; t.Cc = (int)H1; t.ldi = NH * H1; t.ldo = l.ld1;
  t.si0 = L1 * NH * H1; t.si1 = H1; t.so0 = NH * H1 * l.ld1; t.so1 = H1 * l.ld1;
  if ((rc = launch_transpose(t, Z, s)) != MEGA_OK) return rc;
  t.in = dy; t.out = dot; t.R = (int)L1; t.Cc = (int)H2; t.ldi = NH * H2; t.ldo = l.ld1;
  t.si0 = L1 * NH * H2; t.si1 = H2; t.so0 = NH * H2 * l.ld1; t.so1 = H2 * l.ld1;
  if ((rc = launch_transpose(t, Z, s)) != MEGA_OK) return rc;
  t.in = w; t.out = pt; t.R = (int)L1; t.Cc = (int)L2; t.ldi = L2; t.ldo = l.ld1;
  t.si0 = NH * L1 * L2; t.si1 = L1 * L2; t.so0 = NH * L2 * l.ld1; t.so1 = L2 * l.ld1; t.tri = causal;
  if ((rc = launch_transpose(t, Z, s)) != MEGA_OK) return rc;
  t.in = dp; t.out = dst;
  if ((rc = launch_transpose(t, Z, s)) != MEGA_OK) return rc;
  // dQ = scale dS Kt^T
  GemmParams a{};
  a.A = dp; a.B = kt; a.C = dq; a.M = (int)L1; a.N = (int)H1; a.K = (int)L2;
  a.lda = L2; a.ldb = l.ld2; a.ldc = NH * H1;
  a.sa0 = NH * L1 * L2; a.sa1 = L1 * L2; a.sb0 = NH * H1 * l.ld2; a.sb1 = H1 * l.ld2;
  a.sc0 = L1 * NH * H1; a.sc1 = H1; a.nh = (int)NH; a.alpha = scale; a.k_mode = causal ? 1 : 0;
  if ((rc = launch_gemm<DT>(a, Z, s)) != MEGA_OK) return rc;
  // dK = scale dSt Qt^T
  GemmParams b{};
  b.A = dst; b.B = qt; b.C = dk; b.M = (int)L2; b.N = (int)H1; b.K = (int)L1;
  b.lda = l.ld1; b.ldb = l.ld1; b.ldc = NH * H1;
  b.sa0 = NH * L2 * l.ld1; b.sa1 = L2 * l.ld1; b.sb0 = NH * H1 * l.ld1; b.sb1 = H1 * l.ld1;
  b.sc0 = L2 * NH * H1; b.sc1 = H1; b.nh = (int)NH; b.alpha = scale; b.k_mode = causal ? 2 : 0;
  if ((rc = launch_gemm<DT>(b, Z, s)) != MEGA_OK) return rc;
  // dV = Pt dYt^T
  GemmParams c{};
  c.A = pt; c.B = dot; c.C = dv; c.M = (int)L2; c.N = (int)H2; c.K = (int)L1;
  c.lda = l.ld1; c.ldb = l.ld1; c.ldc = NH * H2;
  c.sa0 = NH * L2 * l.ld1; c.sa1 = L2 * l.ld1; c.sb0 = NH * H2 * l.ld1; c.sb1 = H2 * l.ld1;
  c.sc0 = L2 * NH * H2; c.sc1 = H2; c.nh = (int)NH; c.alpha = 1.f; c.k_mode = causal ? 2 : 0;
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

extern "C" int mega_attention_fwd(const void* q, const void* k, const void* v, int dtype, int64_t B,
                                  int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2,
                                  double scale, int causal, void* y, void* w, void* workspace,
                                  void* stream) {
  int rc = check_attn("mega_attention_fwd", dtype, B, L1, L2, NH, H1, H2, causal);
  if (rc != MEGA_OK) return rc;
  if (B == 0 || L1 == 0) return MEGA_OK;
  MEGA_CHECK_ARG(q && k && v && y && w && workspace, "mega_attention_fwd: null pointer");
  MEGA_CHECK_ARG(L2 >= 1, "mega_attention_fwd: no keys");
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto u = [](const void* p) { return static_cast<const uint16_t*>(p); };
  auto m = [](void* p) { return static_cast<uint16_t*>(p); };
  if (dtype == MEGA_BF16)
    return attn_fwd_impl<MEGA_BF16>(u(q), u(k), u(v), B, L1, L2, NH, H1, H2, (float)scale, causal,
                                    m(y), m(w), m(workspace), s);
  return attn_fwd_impl<MEGA_F16>(u(q), u(k), u(v), B, L1, L2, NH, H1, H2, (float)scale, causal,
                                 m(y), m(w), m(workspace), s);
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
  auto u = [](const void* p) { return static_cast<const uint16_t*>(p); };
  auto m = [](void* p) { return static_cast<uint16_t*>(p); };
  if (dtype == MEGA_BF16)
    return attn_bwd_impl<MEGA_BF16>(u(dy), u(q), u(k), u(v), u(w), B, L1, L2, NH, H1, H2,
                                    (float)scale, causal, m(dq), m(dk), m(dv), m(workspace), s);
  return attn_bwd_impl<MEGA_F16>(u(dy), u(q), u(k), u(v), u(w), B, L1, L2, NH, H1, H2,
                                 (float)scale, causal, m(dq), m(dk), m(dv), m(workspace), s);
}
