// Chunk-causal attention on float32 and float64 tensors.
//
// The reference dispatches its attention operator over float32 and float64 as
// well (megalodon/csrc/ops/attention_kernel.cu:269-281: cuBLAS sgemm / dgemm, w
// of the tensors' type); the model itself runs it in bfloat16, which is what the
// matrix-core kernels of attention.hip are built for.  This file is the wide
// flavour of the same operator, templated over the element type T = float or
// double: identical semantics (S = scale Q K^T, P = softmax over the causal
// prefix with an optional DropKey mask, Y = P V; dV = P^T dY, dP = dY V^T,
// dS = P o (dP - rowsum(P o dP)), dQ = scale dS K, dK = scale dS^T Q), storage
// and arithmetic in T throughout, on the vector ALUs: one generic LDS-tiled
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
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ double wave_max(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmax(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float fma_t(float a, float b, float c) { return fmaf(a, b, c); }
__device__ __forceinline__ double fma_t(double a, double b, double c) { return fma(a, b, c); }
__device__ __forceinline__ float exp_t(float a) { return expf(a); }
__device__ __forceinline__ double exp_t(double a) { return exp(a); }
__device__ __forceinline__ float max_t(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double max_t(double a, double b) { return fmax(a, b); }

template <typename T>
struct GemmWide {
  const T* A;
  const T* B;
  T* C;
  int M, N, K;
  int64_t lda, ldb, ldc;
  int64_t sa0, sa1, sb0, sb1, sc0, sc1;
  int nh, ta, tb;
  T alpha;
};

template <typename T>
__global__ __launch_bounds__(kThreads) void gemm_wide_kernel(const GemmWide<T> p) {
  __shared__ T As[kTK][kTM + 4], Bs[kTK][kTN + 4];
  const int z = blockIdx.z, z0 = z / p.nh, z1 = z % p.nh;
  const T* A = p.A + z0 * p.sa0 + z1 * p.sa1;
  const T* B = p.B + z0 * p.sb0 + z1 * p.sb1;
  T* C = p.C + z0 * p.sc0 + z1 * p.sc1;
  const int m0 = blockIdx.y * kTM, n0 = blockIdx.x * kTN;
  const int tid = threadIdx.x, tm = tid / 16, tn = tid % 16;  // 4 x 4 outputs: rows 4 tm .., columns 4 tn ..
  T acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = T(0);
  for (int k0 = 0; k0 < p.K; k0 += kTK) {
    // 64 x 16 elements per operand, four per thread; the index that is contiguous in memory
    // runs fastest over the threads
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + kThreads * i;
      {
        const int mm = p.ta ? e % kTM : e / kTK, kk = p.ta ? e / kTM : e % kTK;
        const int m = m0 + mm, k = k0 + kk;
        T v = T(0);
        if (m < p.M && k < p.K) v = p.ta ? A[static_cast<int64_t>(k) * p.lda + m] : A[static_cast<int64_t>(m) * p.lda + k];
        As[kk][mm] = v;
      }
      {
        const int nn = p.tb ? e % kTN : e / kTK, kk = p.tb ? e / kTN : e % kTK;
        const int n = n0 + nn, k = k0 + kk;
        T v = T(0);
        if (n < p.N && k < p.K) v = p.tb ? B[static_cast<int64_t>(k) * p.ldb + n] : B[static_cast<int64_t>(n) * p.ldb + k];
        Bs[kk][nn] = v;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTK; ++kk) {
      T a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][4 * tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][4 * tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fma_t(a[i], b[j], acc[i][j]);
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

template <typename T>
int launch(const GemmWide<T>& p, int batch, hipStream_t s) {
  if (p.M == 0 || p.N == 0 || batch == 0) return MEGA_OK;
  const dim3 grid((p.N + kTN - 1) / kTN, (p.M + kTM - 1) / kTM, batch);
  gemm_wide_kernel<T><<<grid, kThreads, 0, s>>>(p);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

// Causal softmax over rows, in place, one wavefront per row (softmax.cuh:86-196): row r keeps
// columns [0, n), n = r + 1 + coff (coff = L2 - L1 >= 0) or all of them (coff < 0); the rest of
// the row becomes 0.  DropKey takes keys out of a row before the maximum is taken.
template <typename T, bool DROP>
__global__ __launch_bounds__(kThreads) void softmax_wide_fwd_kernel(T* w, int L1, int L2, int coff, DropKey dk) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const uint32_t row = blockIdx.y * static_cast<uint32_t>(L1) + r;
  T* x = w + (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  const auto score = [&](int j) {
    T v = x[j];
    if (DROP) {
      bool drops[4];
      dropkey_quad(dk, row, static_cast<uint32_t>(j) >> 2, drops);
      if (drops[j & 3]) v = -INFINITY;
    }
    return v;
  };
  T m = -INFINITY;
  for (int j = lane; j < n; j += kWave) m = max_t(m, score(j));
  m = wave_max(m);
  if (m == -INFINITY) m = T(0);  // nothing kept: the row becomes 0 (softmax.cuh:113-116)
  T d = T(0);
  for (int j = lane; j < n; j += kWave) d += exp_t(score(j) - m);
  d = wave_sum(d);
  const T c = d == T(0) ? T(0) : T(1) / d;
  for (int j = lane; j < L2; j += kWave) x[j] = j < n ? exp_t(score(j) - m) * c : T(0);
}

// dS = P o (dP - sum_j P_j dP_j), written over dP (softmax.cuh:198-234); zero outside the kept prefix
template <typename T>
__global__ __launch_bounds__(kThreads) void softmax_wide_bwd_kernel(const T* w, T* dw, int L1, int L2, int coff) {
  const int lane = threadIdx.x % kWave;
  const int r = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (r >= L1) return;
  const int64_t o = (static_cast<int64_t>(blockIdx.y) * L1 + r) * L2;
  const T* pw = w + o;
  T* pd = dw + o;
  const int n = coff >= 0 ? min(r + 1 + coff, L2) : L2;
  T s = T(0);
  for (int j = lane; j < n; j += kWave) s = fma_t(pw[j], pd[j], s);
  s = wave_sum(s);
  for (int j = lane; j < L2; j += kWave) pd[j] = j < n ? pw[j] * (pd[j] - s) : T(0);
}

}  // namespace

template <typename T>
int attention_wide_fwd(const T* q, const T* k, const T* v, int64_t B, int64_t L1, int64_t L2,
                       int64_t NH, int64_t H1, int64_t H2, double scale, int causal, const DropKey* drop,
                       T* y, T* w, hipStream_t s) {
  const int Z = static_cast<int>(B * NH);
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  GemmWide<T> g{};  // S = scale Q K^T -> w
  g.A = q; g.B = k; g.C = w; g.M = (int)L1; g.N = (int)L2; g.K = (int)H1;
  g.lda = NH * H1; g.ldb = NH * H1; g.ldc = L2;
  g.sa0 = L1 * NH * H1; g.sa1 = H1; g.sb0 = L2 * NH * H1; g.sb1 = H1;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = static_cast<T>(scale);
  int rc = launch(g, Z, s);
  if (rc != MEGA_OK) return rc;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  if (drop != nullptr) softmax_wide_fwd_kernel<T, true><<<sgrid, kThreads, 0, s>>>(w, (int)L1, (int)L2, coff, *drop);
  else softmax_wide_fwd_kernel<T, false><<<sgrid, kThreads, 0, s>>>(w, (int)L1, (int)L2, coff, DropKey{});
  MEGA_CHECK_LAUNCH();
  GemmWide<T> o{};  // Y = P V: V[key][c] is the k-major B operand
  o.A = w; o.B = v; o.C = y; o.M = (int)L1; o.N = (int)H2; o.K = (int)L2;
  o.lda = L2; o.ldb = NH * H2; o.ldc = NH * H2; o.tb = 1;
  o.sa0 = NH * L1 * L2; o.sa1 = L1 * L2; o.sb0 = L2 * NH * H2; o.sb1 = H2;
  o.sc0 = L1 * NH * H2; o.sc1 = H2; o.nh = (int)NH; o.alpha = T(1);
  return launch(o, Z, s);
}

template <typename T>
int attention_wide_bwd(const T* dy, const T* q, const T* k, const T* v, const T* w,
                       int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1, int64_t H2, double scale,
                       int causal, T* dq, T* dk, T* dv, T* dp, hipStream_t s) {
  const int Z = static_cast<int>(B * NH);
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  int rc;
  GemmWide<T> g{};  // dP = dY V^T
  g.A = dy; g.B = v; g.C = dp; g.M = (int)L1; g.N = (int)L2; g.K = (int)H2;
  g.lda = NH * H2; g.ldb = NH * H2; g.ldc = L2;
  g.sa0 = L1 * NH * H2; g.sa1 = H2; g.sb0 = L2 * NH * H2; g.sb1 = H2;
  g.sc0 = NH * L1 * L2; g.sc1 = L1 * L2; g.nh = (int)NH; g.alpha = T(1);
  if ((rc = launch(g, Z, s)) != MEGA_OK) return rc;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  softmax_wide_bwd_kernel<T><<<sgrid, kThreads, 0, s>>>(w, dp, (int)L1, (int)L2, coff);
  MEGA_CHECK_LAUNCH();
  GemmWide<T> a{};  // dQ = scale dS K: K[key][h] is the k-major B operand
  a.A = dp; a.B = k; a.C = dq; a.M = (int)L1; a.N = (int)H1; a.K = (int)L2;
  a.lda = L2; a.ldb = NH * H1; a.ldc = NH * H1; a.tb = 1;
  a.sa0 = NH * L1 * L2; a.sa1 = L1 * L2; a.sb0 = L2 * NH * H1; a.sb1 = H1;
  a.sc0 = L1 * NH * H1; a.sc1 = H1; a.nh = (int)NH; a.alpha = static_cast<T>(scale);
  if ((rc = launch(a, Z, s)) != MEGA_OK) return rc;
  GemmWide<T> b{};  // dK = scale dS^T Q: dS[q][key] and Q[q][h] are both k-major (k = q)
  b.A = dp; b.B = q; b.C = dk; b.M = (int)L2; b.N = (int)H1; b.K = (int)L1;
  b.lda = L2; b.ldb = NH * H1; b.ldc = NH * H1; b.ta = 1; b.tb = 1;
  b.sa0 = NH * L1 * L2; b.sa1 = L1 * L2; b.sb0 = L1 * NH * H1; b.sb1 = H1;
  b.sc0 = L2 * NH * H1; b.sc1 = H1; b.nh = (int)NH; b.alpha = static_cast<T>(scale);
  if ((rc = launch(b, Z, s)) != MEGA_OK) return rc;
  GemmWide<T> c{};  // dV = P^T dY: P[q][key] and dY[q][c] are both k-major (k = q)
  c.A = w; c.B = dy; c.C = dv; c.M = (int)L2; c.N = (int)H2; c.K = (int)L1;
  c.lda = L2; c.ldb = NH * H2; c.ldc = NH * H2; c.ta = 1; c.tb = 1;
  c.sa0 = NH * L1 * L2; c.sa1 = L1 * L2; c.sb0 = L1 * NH * H2; c.sb1 = H2;
  c.sc0 = L2 * NH * H2; c.sc1 = H2; c.nh = (int)NH; c.alpha = T(1);
  return launch(c, Z, s);
}

template <typename T>
int softmax_wide_fwd(T* x, int64_t Z, int64_t L1, int64_t L2, int causal, const DropKey* drop, hipStream_t s) {
  if (Z == 0 || L1 == 0 || L2 == 0) return MEGA_OK;
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  if (drop != nullptr) softmax_wide_fwd_kernel<T, true><<<sgrid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, *drop);
  else softmax_wide_fwd_kernel<T, false><<<sgrid, kThreads, 0, s>>>(x, (int)L1, (int)L2, coff, DropKey{});
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template <typename T>
int softmax_wide_bwd(const T* y, T* dy, int64_t Z, int64_t L1, int64_t L2, int causal, hipStream_t s) {
  if (Z == 0 || L1 == 0 || L2 == 0) return MEGA_OK;
  const int coff = causal ? static_cast<int>(L2 - L1) : -1;
  const dim3 sgrid((unsigned)((L1 + 3) / 4), (unsigned)Z);
  softmax_wide_bwd_kernel<T><<<sgrid, kThreads, 0, s>>>(y, dy, (int)L1, (int)L2, coff);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}

template int attention_wide_fwd<float>(const float*, const float*, const float*, int64_t, int64_t, int64_t, int64_t,
                                       int64_t, int64_t, double, int, const DropKey*, float*, float*, hipStream_t);
template int attention_wide_fwd<double>(const double*, const double*, const double*, int64_t, int64_t, int64_t,
                                        int64_t, int64_t, int64_t, double, int, const DropKey*, double*, double*,
                                        hipStream_t);
template int attention_wide_bwd<float>(const float*, const float*, const float*, const float*, const float*, int64_t,
                                       int64_t, int64_t, int64_t, int64_t, int64_t, double, int, float*, float*,
                                       float*, float*, hipStream_t);
template int attention_wide_bwd<double>(const double*, const double*, const double*, const double*, const double*,
                                        int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, double, int, double*,
                                        double*, double*, double*, hipStream_t);
template int softmax_wide_fwd<float>(float*, int64_t, int64_t, int64_t, int, const DropKey*, hipStream_t);
template int softmax_wide_fwd<double>(double*, int64_t, int64_t, int64_t, int, const DropKey*, hipStream_t);
template int softmax_wide_bwd<float>(const float*, float*, int64_t, int64_t, int64_t, int, hipStream_t);
template int softmax_wide_bwd<double>(const double*, double*, int64_t, int64_t, int64_t, int, hipStream_t);

}  // namespace mega
