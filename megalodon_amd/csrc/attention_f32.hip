// Chunk-causal attention on float32 tensors.
//
// The reference dispatches its attention operator over float32 as well
// (megalodon/csrc/ops/attention_kernel.cu:269-281: cuBLAS sgemm, float32 w);
// the model itself runs it in bfloat16, which is what the matrix-core kernels
// of attention.hip are built for.  This file is the float32 flavour of the same
// operator: identical semantics (S = scale Q K^T, P = softmax over the causal
// prefix with an optional DropKey mask, Y = P V; dV = P^T dY, dP = dY V^T,
// dS = P o (dP - rowsum(P o dP)), dQ = scale dS K, dK = scale dS^T Q), float32
// storage and arithmetic throughout, on the vector ALUs: one generic LDS-tiled
// product kernel and row-per-wavefront softmax kernels.  It skips no tiles: the
// softmax writes exact zeros above the diagonal, so the full-range products
// are the causal ones.
#include "common.hpp"
#include "dropkey.hpp"

namespace mega {
namespace {

constexpr int kTM = 64, kTN = 64, kTK = 16;
constexpr int kThreads = 256;

// C[m][n] = alpha * sum_k A(m, k) B(n, k); element (m, k) of an operand at
// [m * ld + k], or at [k * ld + m] when the operand is k-major (ta / tb).
// Batch index z = z0 * nh + z1 selects the matrices by two strides each.
struct GemmF32 {
  const float* A;
  const float* B;
  float* C;
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t sa0, sa1, sb0, sb1, sc0, sc1;
  int nh, ta, tb;
  float alpha;
};

__global__ __launch_bounds__(kThreads) void gemm_f32_kernel(const GemmF32 p) {
  __shared__ float As[kTK][kTM + 4], Bs[kTK][kTN + 4];
  const int z = blockIdx.z, z0 = z / p.nh, z1 = z % p.nh;
  const float* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const float* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  float* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  const int m0 = blockIdx.y * kTM, n0 = blockIdx.x * kTN;
  const int tid = threadIdx.x, tm = tid / 16, tn = tid % 16;  // 4 x 4 outputs: rows 4 tm .., columns 4 tn ..
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < p.K; k0 += kTK) {
    // 64 x 16 elements per operand, four per thread; the index that is contiguous in memory
    // runs fastest over the threads
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + kThreads * i;
      {
        const int mm = p.ta ? e % kTM : e / kTK, kk = p.ta ? e / kTM : e % kTK;
        const int m = m0 + mm, k = k0 + kk;
        float v = 0.f;
        if (m < p.M && k < p.K) v = p.ta ? A[static_cast<int64_t>(k) * p.lda + m] : A[static_cast<int64_t>(m) * p.lda + k];
        As[kk][mm] = v;
      }
      {
        const int nn = p.tb ? e % kTN : e / kTK, kk = p.tb ? e / kTN : e % kTK;
        const int n = n0 + nn, k = k0 + kk;
        float v = 0.f;
        if (n < p.N && k < p.K) v = p.tb ? B[static_cast<int64_t>(k) * p.ldb + n] : B[static_cast<int64_t>(n) * p.ldb + k];
        Bs[kk][nn] = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][4 * tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][4 * tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + 4 * tm + i;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + 4 * tn + j;
      if (n < p.N) C[static_cast<int64_t>(m) * p.ldc + n] = p.alpha * acc[i][j];
    }
  }
}

int launch(const GemmF32& p, int batch, hipStream_t s) {
  if (p.M == 0 || p.N == 0 || batch == 0) return MEGA_OK;
  const dim3 grid((p.N + kTN - 1) / kTN, (p.M + kTM - 1) / kTM, batch);
  gemm_f32_kernel<<<grid, kThreads, 0, s>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

// Causal softmax over rows, in place, one wavefront per row (softmax.cuh:86-196): row r keeps
// columns [0, n), n = r + 1 + coff (coff = L2 - L1 >= 0) or all of them (coff < 0); the rest of
// the row becomes 0.  DropKey takes keys out of a row before the maximum is taken.
template <bool DROP>
__global__ __launch_bounds__(kThreads) void softmax_f32_fwd_kernel(float* w, int L1, int L2, int coff, DropKey dk) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const uint32_t row = blockIdx.y * static_cast<uint32_t>(L1) + r;
  float* x = w + (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  const auto score = [&](int j) {
    float v = x[j];
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
  for (int j = lane; j < n; j += kWave) d += expf(score(j) - m);
  d = wave_sum(d);
  const float c = d == 0.f ? 0.f : 1.f / d;
  for (int j = lane; j < L2; j += kWave) x[j] = j < n ? expf(score(j) - m) * c : 0.f;
}

// dS = P o (dP - sum_j P_j dP_j), written over dP (softmax.cuh:198-234); zero outside the kept prefix
__global__ __launch_bounds__(kThreads) void softmax_f32_bwd_kernel(const float* w, float* dw, int L1, int L2, int coff) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const int64_t o = (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const float* pw = w + o;
  float* pd = dw + o;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  float s = 0.f;
  for (int j = lane; j < n; j += kWave) s = fmaf(pw[j], pd[j], s);
  s = wave_sum(s);
  for (int j = lane; j < L2; j += kWave) pd[j] = j < n ? pw[j] * (pd[j] - s) : 0.f;
}

}  // namespace

int attention_f32_fwd(const float* q, const float* k, const float* v, int64_t B, int64_t L1, int64_t L2,
                      int64_t NH, int64_t H1, int64_t H2, float scale, int causal, const DropKey* drop,
                      float* y, float* w, hipStream_t s) {
  const int Z = static_cast<int>(B * NH);
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  GemmF32 g{};  // S = scale Q K^T -> w
  g.A = q; g.B = k; g.C = w; g.M = (int)L1; g.N = (int)L2; g.K = (int)H1;
  g.lda = NH * H1; g.ldb = NH * H1; g.ldc = L2;
  g.sa0 = L1 * NH * H1; g.sa1 = H1; g.sb0 = L2 * NH * H1; g.sb1 = H1;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = scale;
  int rc = launch(g, Z, s);
  if (rc != MEGA_OK) return rc;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  if (drop != nullptr) softmax_f32_fwd_kernel<true><<<sgrid, kThreads, 0, s>>>(w, (int)L1, (int)L2, coff, *drop);
  else softmax_f32_fwd_kernel<false><<<sgrid, kThreads, 0, s>>>(w, (int)L1, (int)L2, coff, DropKey{});
  MEGA_CHECK_LAUNCH();
  GemmF32 o{};  // Y = P V: V[key][c] is the k-major B operand
  o.A = w; o.B = v; o.C = y; o.M = (int)L1; o.N = (int)H2; o.K = (int)L2;
  o.lda = L2; o.ldb = NH * H2; o.ldc = NH * H2; o.tb = 1;
  o.sa0 = NH * L1 * L2; o.sa1 = L1 * L2; o.sb0 = L2 * NH * H2; o.sb1 = H2;
  o.sc0 = L1 * NH * H2; o.sc1 = H2; o.nh = (int)NH; o.alpha = 1.f;
  return launch(o, Z, s);
}

int attention_f32_bwd(const float* dy, const float* q, const float* k, const float* v, const float* w,
                      int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2, float scale,
                      int causal, float* dq, float* dk, float* dv, float* dp, hipStream_t s) {
  const int Z = static_cast<int>(B * NH);
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  int rc;
  GemmF32 g{};  // dP = dY V^T
  g.A = dy; g.B = v; g.C = dp; g.M = (int)L1; g.N = (int)L2; g.K = (int)H2;
  g.lda = NH * H2; g.ldb = NH * H2; g.ldc = L2;
  g.sa0 = L1 * NH * H2; g.sa1 = H2; g.sb0 = L2 * NH * H2; g.sb1 = H2;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = 1.f;
  if ((rc = launch(g, Z, s)) != MEGA_OK) return rc;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  softmax_f32_bwd_kernel<<<sgrid, kThreads, 0, s>>>(w, dp, (int)L1, (int)L2, coff);
  MEGA_CHECK_LAUNCH();
  GemmF32 a{};  // dQ = scale dS K: K[key][h] is the k-major B operand
  a.A = dp; a.B = k; a.C = dq; a.M = (int)L1; a.N = (int)H1; a.K = (int)L2;
  a.lda = L2; a.ldb = NH * H1; a.ldc = NH * H1; a.tb = 1;
  a.sa0 = NH * L1 * L2; a.sa1 = L1 * L2; a.sb0 = L2 * NH * H1; a.sb1 = H1;
  a.sc0 = L1 * NH * H1; a.sc1 = H1; a.nh = (int)NH; a.alpha = scale;
  if ((rc = launch(a, Z, s)) != MEGA_OK) return rc;
  GemmF32 b{};  // dK = scale dS^T Q: dS[q][key] and Q[q][h] are both k-major (k = q)
  b.A = dp; b.B = q; b.C = dk; b.M = (int)L2; b.N = (int)H1; b.K = (int)L1;
  b.lda = L2; b.ldb = NH * H1; b.ldc = NH * H1; b.ta = 1; b.tb = 1;
  b.sa0 = NH * L1 * L2; b.sa1 = L1 * L2; b.sb0 = L1 * NH * H1; b.sb1 = H1;
  b.sc0 = L2 * NH * H1; b.sc1 = H1; b.nh = (int)NH; b.alpha = scale;
  if ((rc = launch(b, Z, s)) != MEGA_OK) return rc;
  GemmF32 c{};  // dV = P^T dY: P[q][key] and dY[q][c] are both k-major (k = q)
  c.A = w; c.B = dy; c.C = dv; c.M = (int)L2; c.N = (int)H2; c.K = (int)L1;
  c.lda = L2; c.ldb = NH * H2; c.ldc = NH * H2; c.ta = 1; c.tb = 1;
  c.sa0 = NH * L1 * L2; c.sa1 = L1 * L2; c.sb0 = L1 * NH * H2; c.sb1 = H2;
  c.sc0 = L2 * NH * H2; c.sc1 = H2; c.nh = (int)NH; c.alpha = 1.f;
  return launch(c, Z, s);
}

int softmax_f32_fwd(float* x, int64_t Z, int64_t L1, int64_t L2, int causal, const DropKey* drop, hipStream_t s) {
  if (Z == 0 || L1 == 0 || L2 == 0) return MEGA_OK;
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  if (drop != nullptr) softmax_f32_fwd_kernel<true><<<sgrid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, *drop);
  else softmax_f32_fwd_kernel<false><<<sgrid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, DropKey{});
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

int softmax_f32_bwd(const float* y, float* dy, int64_t Z, int64_t L1, int64_t L2, int causal, hipStream_t s) {
  if (Z == 0 || L1 == 0 || L2 == 0) return MEGA_OK;
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  softmax_f32_bwd_kernel<<<sgrid, kThreads, 0, s>>>(y, dy, (int)L1, (int)L2, coff);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

}  // namespace mega
