// Causal FFT convolution for gfx950.
//
// Semantics follow megalodon/modules/fused_ops/fftconv.py:30-75:
//   forward   y  = irfft(rfft(x, 2N) * rfft(k, 2N))[:L]
//   backward  dx = flip(conv(flip(dy), k)),  dk = sum_b flip(conv(flip(dy_b), x_b))
// One workgroup convolves one (batch, channel) row entirely on chip: the row
// is read once per half (see fftconv_core.hpp), transformed with 32 complex
// points per lane in registers, multiplied with the parked spectrum of the
// other operand and transformed back; nothing but the rows themselves touches
// HBM (the reference's torch.fft path at L > 16384 makes ~7 full round trips
// and saves the 1 GiB spectra x_f / k_f for backward; here backward recomputes
// the spectra from x and k).
//
// Rows with L <= 2048 use a direct time-domain kernel (exact, O(L^2) per row).
#include "common.hpp"
#include "fftconv_core.hpp"
#include "fftconv_mfma.hpp"

#include <mutex>
#include <vector>

namespace mega {
namespace {

using namespace fftc;

// ------------------------------ tables --------------------------------------
constexpr int kMaxDevices = 16;
constexpr int kMaxScratch = 4;  // scratch blocks per device and size before streams start taking turns
struct StreamScratch {
  hipStream_t stream;  // the stream whose launches used the block last
  float* ptr;
  hipEvent_t done;     // recorded behind the last launch that used the block
  uint64_t tick;       // when that was
  bool pinned;         // used under stream capture: the graph's replays own the block from then on
};
struct TableCache {
  c32* ptr[kMaxDevices][4] = {};
  int slots[kMaxDevices][4] = {};
  // Launches on different streams of a device may overlap, and a workgroup's
  // slot is picked by its index alone, so a stream gets a block of its own --
  // up to kMaxScratch of them per device and size.  A further stream takes
  // over the block that has been idle longest and first waits (on the device,
  // through the block's event) for the last launch that used it.  Blocks used
  // under stream capture are never handed on.
  std::vector<StreamScratch> scratch[kMaxDevices][4];
  uint64_t tick = 0;
  std::mutex mu;
};
TableCache g_tables;

bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}

// Twiddle tables (one per device and transform size) and the per-workgroup
// scratch slots live for the life of the process.  They are made on first use,
// or ahead of time by mega_fftconv_prepare; making them allocates and, for the
// tables, synchronises the stream once, so that call cannot be captured into a
// graph.  Scratch is 2*M floats per resident workgroup (at most 2 workgroups
// per CU).
template <int LOGM>
int get_tables(hipStream_t stream, const c32** out, float** scratch, int* slots) {
  using C = Cfg<LOGM>;
  int dev = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  MEGA_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_tables.mu);
  c32*& slot = g_tables.ptr[dev][LOGM - 11];
  if (slot == nullptr) {
    hipDeviceProp_t prop;
    MEGA_CHECK_HIP(hipGetDeviceProperties(&prop, dev));
    const int per_cu = LOGM == 14 ? 1 : 2;
    g_tables.slots[dev][LOGM - 11] = prop.multiProcessorCount * per_cu;
    c32* p = nullptr;
    MEGA_CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&p), sizeof(c32) * C::TABLE));
    std::vector<c32> host(C::TABLE);
    fill_tables<LOGM>(host.data());
    hipError_t e = hipMemcpyAsync(p, host.data(), sizeof(c32) * C::TABLE, hipMemcpyHostToDevice, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
      (void)hipFree(p);
      return set_error(MEGA_ERR_HIP, "fftconv table init failed: %s", hipGetErrorString(e));
    }
    slot = p;
  }
  const int nslots = g_tables.slots[dev][LOGM - 11];
  std::vector<StreamScratch>& blocks = g_tables.scratch[dev][LOGM - 11];
  StreamScratch* mine = nullptr;
  int open_blocks = 0;
  for (StreamScratch& s : blocks) {
    if (s.stream == stream) mine = &s;
    open_blocks += s.pinned ? 0 : 1;
  }
  const bool capturing = stream_is_capturing(stream);
  if (mine == nullptr && open_blocks >= kMaxScratch && !capturing) {
    // take over the block that has been idle longest, behind its last launch
    for (StreamScratch& s : blocks)
      if (!s.pinned && (mine == nullptr || s.tick < mine->tick)) mine = &s;
    MEGA_CHECK_HIP(hipStreamWaitEvent(stream, mine->done, 0));
    mine->stream = stream;
  }
  if (mine == nullptr) {
    float* sc = nullptr;
    hipEvent_t ev = nullptr;
    MEGA_CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&sc), sizeof(float) * 2 * C::M * nslots));
    hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    if (e != hipSuccess) {
      (void)hipFree(sc);
      return set_error(MEGA_ERR_HIP, "fftconv scratch event: %s", hipGetErrorString(e));
    }
    blocks.push_back(StreamScratch{stream, sc, ev, 0, false});
    mine = &blocks.back();
  }
  mine->tick = ++g_tables.tick;
  if (capturing) mine->pinned = true;
  *out = slot;
  *scratch = mine->ptr;
  *slots = nslots;
  return MEGA_OK;
}

// Marks the end of the launches that used `stream`'s scratch block, so that a
// later take-over can order itself behind them.  Not recorded under capture
// (the block is pinned there).
template <int LOGM>
int scratch_used(hipStream_t stream) {
  int dev = 0;
  MEGA_CHECK_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_tables.mu);
  for (StreamScratch& s : g_tables.scratch[dev][LOGM - 11])
    if (s.stream == stream && !s.pinned) MEGA_CHECK_HIP(hipEventRecord(s.done, stream));
  return MEGA_OK;
}

// ------------------------------ row I/O --------------------------------------
template <int DT>
__device__ __forceinline__ float ld(const void* base, int64_t i) {
  return Elem<DT>::load(static_cast<const typename Elem<DT>::type*>(base) + i);
}
template <int DT>
__device__ __forceinline__ void st(void* base, int64_t i, float v) {
  Elem<DT>::store(static_cast<typename Elem<DT>::type*>(base) + i, v);
}

// uniform base + 32-bit unsigned byte offset (scalar-base addressing form)
template <typename V>
__device__ __forceinline__ V gld(const void* base, unsigned byte_off) {
  return *reinterpret_cast<const V*>(static_cast<const char*>(base) + byte_off);
}
template <typename V>
__device__ __forceinline__ void gst(void* base, unsigned byte_off, V v) {
  *reinterpret_cast<V*>(static_cast<char*>(base) + byte_off) = v;
}

// A pair of adjacent elements as one 32/64-bit access.
template <int DT> struct Pair;
template <> struct Pair<MEGA_F32> {
  using type = float2;
  static __device__ __forceinline__ void unpack(type v, float& lo, float& hi) { lo = v.x; hi = v.y; }
  static __device__ __forceinline__ type pack(float lo, float hi) { return make_float2(lo, hi); }
};
template <> struct Pair<MEGA_BF16> {
  using type = uint32_t;
  static __device__ __forceinline__ void unpack(type v, float& lo, float& hi) {
    lo = __uint_as_float(v << 16);
    hi = __uint_as_float(v & 0xffff0000u);
  }
  static __device__ __forceinline__ type pack(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <> struct Pair<MEGA_F16> {
  using type = uint32_t;
  static __device__ __forceinline__ void unpack(type v, float& lo, float& hi) {
    lo = f16_bits_to_float(static_cast<uint16_t>(v & 0xffffu));
    hi = f16_bits_to_float(static_cast<uint16_t>(v >> 16));
  }
  static __device__ __forceinline__ type pack(float lo, float hi) {
    return static_cast<uint32_t>(float_to_f16_bits(lo)) |
           (static_cast<uint32_t>(float_to_f16_bits(hi)) << 16);
  }
};

// z[n] = s[2n] + i s[2n+1] of the zero-padded (optionally reversed) row.
// VEC: L is even and the row is pair-aligned, so (s[2n], s[2n+1]) is one access
// addressed with a 32-bit offset from the wave-uniform row base.
template <int LOGM, int DT, bool VEC>
__device__ __forceinline__ void load_row(float* re, float* im, const void* row, int L, bool flip,
                                         int t) {
  using C = Cfg<LOGM>;
  if (VEC) {
    using P = typename Pair<DT>::type;
    const unsigned half = static_cast<unsigned>(L) >> 1;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const unsigned n = static_cast<unsigned>(t) + C::T * j;
      float lo = 0.f, hi = 0.f;
      if (n < half)
        Pair<DT>::unpack(gld<P>(row, (flip ? half - 1u - n : n) * static_cast<unsigned>(sizeof(P))), lo, hi);
      re[j] = flip ? hi : lo;
      im[j] = flip ? lo : hi;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const int m0 = 2 * (t + C::T * j), m1 = m0 + 1;
      float a = 0.f, b = 0.f;
      if (m0 < L) a = ld<DT>(row, flip ? L - 1 - m0 : m0);
      if (m1 < L) b = ld<DT>(row, flip ? L - 1 - m1 : m1);
      re[j] = a;
      im[j] = b;
    }
  }
}

// out[2n] = re[j], out[2n+1] = im[j] for n = t + T j (reversed when flip);
// ACC adds to what is there (fp32 rows only).  With `res` non-null the stored
// value is out[m] + w * res[m] (res has the dtype and layout of the output row).
template <int LOGM, int DT, bool VEC, bool ACC>
__device__ __forceinline__ void store_row(const float* re, const float* im, void* row, int L,
                                          bool flip, int t, const void* res = nullptr,
                                          float w = 0.f) {
  using C = Cfg<LOGM>;
  if (VEC) {
    using P = typename Pair<DT>::type;
    const unsigned half = static_cast<unsigned>(L) >> 1;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const unsigned n = static_cast<unsigned>(t) + C::T * j;
      if (n < half) {
        float lo = flip ? im[j] : re[j], hi = flip ? re[j] : im[j];
        const unsigned off = (flip ? half - 1u - n : n) * static_cast<unsigned>(sizeof(P));
        if (ACC) {
          float plo, phi;
          Pair<DT>::unpack(gld<P>(row, off), plo, phi);
          lo += plo;
          hi += phi;
        }
        if (res != nullptr) {
          float rlo, rhi;
          Pair<DT>::unpack(gld<P>(res, off), rlo, rhi);
          lo = fmaf(w, rlo, lo);
          hi = fmaf(w, rhi, hi);
        }
        gst<P>(row, off, Pair<DT>::pack(lo, hi));
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const int m0 = 2 * (t + C::T * j), m1 = m0 + 1;
      if (m0 < L) {
        const int o = flip ? L - 1 - m0 : m0;
        const float r = res != nullptr ? w * ld<DT>(res, o) : 0.f;
        st<DT>(row, o, (ACC ? ld<DT>(row, o) + re[j] : re[j]) + r);
      }
      if (m1 < L) {
        const int o = flip ? L - 1 - m1 : m1;
        const float r = res != nullptr ? w * ld<DT>(res, o) : 0.f;
        st<DT>(row, o, (ACC ? ld<DT>(row, o) + im[j] : im[j]) + r);
      }
    }
  }
}

// Hides the table base from common-subexpression elimination / loop hoisting:
// twiddles are re-read from L1/L2 at each use instead of being kept live in
// registers across transforms (which would spill).
__device__ __forceinline__ Tables launder(Tables tb) {
  asm volatile("" : "+s"(tb.kr), "+s"(tb.kbo), "+s"(tb.kbe), "+s"(tb.kbo2));
  asm volatile("" : "+s"(tb.kp2), "+s"(tb.ki3), "+s"(tb.kre), "+s"(tb.kro), "+s"(tb.pw));
  return tb;
}

template <int LOGM, int H>
__device__ __forceinline__ void forward_half(float* re, float* im, int t, const Tables& tb0,
                                             float* lre, float* lim) {
  const Tables tb = launder(tb0);
  fwd_pass1<LOGM, H>(re, im, t, tb);
  __syncthreads();
  x1_write<LOGM>(re, im, t, lre, lim);
  __syncthreads();
  x1_read<LOGM>(re, im, t, lre, lim);
  fwd_pass2<LOGM>(re, im, t, tb);
  __syncthreads();
  x2_write<LOGM>(re, im, t, lre, lim);
  __syncthreads();
  x2_read<LOGM, H>(re, im, t, lre, lim);
  fwd_pass3<LOGM>(re, im);
}

template <int LOGM, int H>
__device__ __forceinline__ void inverse_half(float* re, float* im, int t, const Tables& tb0,
                                             float* lre, float* lim) {
  const Tables tb = launder(tb0);
  inv_pass3<LOGM, H>(re, im, t, tb);
  __syncthreads();
  ix2_write<LOGM, H>(re, im, t, lre, lim);
  __syncthreads();
  ix2_read<LOGM>(re, im, t, lre, lim);
  inv_pass2<LOGM, H>(re, im, t, tb);
  __syncthreads();
  ix1_write<LOGM>(re, im, t, lre, lim);
  __syncthreads();
  ix1_read<LOGM>(re, im, t, lre, lim);
  inv_pass1<H>(re, im);
}

// conv half H of rows a (in flight) and b (parked).  Half 0 leaves its M
// outputs zy[t + T j] in the workgroup's scratch slot (float index j*T + t,
// re plane then im plane); half 1 adds them back and returns the sum in
// (ore, oim) with zy[t + T j] at register j.
template <int LOGM, int DTA, int DTB, bool VEC, int H>
__device__ __forceinline__ void conv_half(const void* arow, bool flip_a, const void* brow, int L,
                                          int t, const Tables& tb, float* lre, float* lim,
                                          float* __restrict__ scratch, float* ore, float* oim) {
  using C = Cfg<LOGM>;
  float re[32], im[32], pre[32], pim[32];
  load_row<LOGM, DTB, VEC>(pre, pim, brow, L, false, t);
  forward_half<LOGM, H>(pre, pim, t, tb, lre, lim);
  constexpr float scale = 1.0f / (8.0f * C::M);  // 1/(4N): E, O halves and the inverse
#pragma unroll
  for (int j = 0; j < 32; ++j) {
    pre[j] *= scale;
    pim[j] *= scale;
  }
  load_row<LOGM, DTA, VEC>(re, im, arow, L, flip_a, t);
  forward_half<LOGM, H>(re, im, t, tb, lre, lim);
  pointwise<LOGM, H>(re, im, pre, pim, t, launder(tb));
  inverse_half<LOGM, H>(re, im, t, tb, lre, lim);
  if (H == 0) {
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      gst<float>(scratch, (j * C::T + t) * 4u, re[out_pos<H>(j)]);
      gst<float>(scratch, (C::M + j * C::T + t) * 4u, im[out_pos<H>(j)]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      ore[j] = re[out_pos<H>(j)] + gld<float>(scratch, (j * C::T + t) * 4u);
      oim[j] = im[out_pos<H>(j)] + gld<float>(scratch, (C::M + j * C::T + t) * 4u);
    }
  }
}

// MODE 0: out[b,d,:] = conv(a[b,d,:], k[d,:]) (+ omega[d] a[b,d,:] when omega is
//         given); `flip` reverses a on load and the result on store (backward
//         dx).  a, out have dtype DT; k is fp32.
// MODE 1: out[d,:] (+)= reverse(conv(reverse(a[b0,d,:]), x[b0,d,:])), fp32
//         (backward dk, one batch index per launch; `flip` != 0 accumulates).
// Persistent: workgroup g handles rows g, g + gridDim.x, ... and owns scratch
// slot g (2*M floats).
template <int LOGM, int DT, int MODE, bool VEC>
__global__ __launch_bounds__(Cfg<LOGM>::T) void fftconv_kernel(
    const void* __restrict__ a, const void* __restrict__ b, void* __restrict__ out, int rows,
    int D, int L, int flip, const c32* __restrict__ tab, float* __restrict__ scratch_all,
    const float* __restrict__ omega) {
  using C = Cfg<LOGM>;
  extern __shared__ float lds[];
  float* lre = lds;
  float* lim = lds + C::PLANE;
  const Tables tb = make_tables<LOGM>(tab);
  const int64_t esz = DT == MEGA_F32 ? 4 : 2;
  float* scratch = scratch_all + static_cast<int64_t>(blockIdx.x) * 2 * C::M;

  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    // the lane id is re-materialised per row so that address arithmetic is not
    // hoisted out of the row loop (it would pin hundreds of registers)
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    t &= C::T - 1;  // restores the range so offsets stay 32-bit
    float ore[32], oim[32];
    if (MODE == 0) {
      const int64_t d = row % D;
      const char* arow = static_cast<const char*>(a) + row * L * esz;
      const float* krow = static_cast<const float*>(b) + d * L;
      char* orow = static_cast<char*>(out) + row * L * esz;
      conv_half<LOGM, DT, MEGA_F32, VEC, 0>(arow, flip != 0, krow, L, t, tb, lre, lim, scratch, ore, oim);
      conv_half<LOGM, DT, MEGA_F32, VEC, 1>(arow, flip != 0, krow, L, t, tb, lre, lim, scratch, ore, oim);
      // optional residual: out += omega[d] * a (MODE 0 only)
      store_row<LOGM, DT, VEC, false>(ore, oim, orow, L, flip != 0, t,
                                      omega != nullptr ? arow : nullptr,
                                      omega != nullptr ? omega[d] : 0.f);
    } else {
      const char* arow = static_cast<const char*>(a) + row * L * esz;
      const char* xrow = static_cast<const char*>(b) + row * L * esz;
      float* orow = static_cast<float*>(out) + row * L;
      conv_half<LOGM, DT, DT, VEC, 0>(arow, true, xrow, L, t, tb, lre, lim, scratch, ore, oim);
      conv_half<LOGM, DT, DT, VEC, 1>(arow, true, xrow, L, t, tb, lre, lim, scratch, ore, oim);
      if (flip)
        store_row<LOGM, MEGA_F32, VEC, true>(ore, oim, orow, L, true, t);
      else
        store_row<LOGM, MEGA_F32, VEC, false>(ore, oim, orow, L, true, t);
    }
  }
}

template <int LOGM, int DT, int MODE, bool VEC>
int launch_fft_v(const void* a, const void* b, void* out, int64_t B, int64_t D, int64_t L,
                 int flip, const float* omega, hipStream_t stream) {
  using C = Cfg<LOGM>;
  const c32* tab = nullptr;
  float* scratch = nullptr;
  int slots = 0;
  const int rc = get_tables<LOGM>(stream, &tab, &scratch, &slots);
  if (rc != MEGA_OK) return rc;
  const size_t lds_bytes = sizeof(float) * 2 * C::PLANE;
  MEGA_CHECK_HIP(hipFuncSetAttribute(
      reinterpret_cast<const void*>(&fftconv_kernel<LOGM, DT, MODE, VEC>),
      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
  const int64_t esz = DT == MEGA_F32 ? 4 : 2;
  if (MODE == 0) {
    const int64_t rows = B * D;
    MEGA_CHECK_ARG(rows <= 0x7fffffff, "fftconv: too many rows");
    const unsigned grid = static_cast<unsigned>(rows < slots ? rows : slots);
    fftconv_kernel<LOGM, DT, MODE, VEC><<<dim3(grid), C::T, lds_bytes, stream>>>(
        a, b, out, static_cast<int>(rows), static_cast<int>(D), static_cast<int>(L), flip, tab,
        scratch, omega);
    MEGA_CHECK_LAUNCH();
  } else {
    const unsigned grid = static_cast<unsigned>(D < slots ? D : slots);
    for (int64_t bb = 0; bb < B; ++bb) {
      const char* ab = static_cast<const char*>(a) + bb * D * L * esz;
      const char* xb = static_cast<const char*>(b) + bb * D * L * esz;
      fftconv_kernel<LOGM, DT, MODE, VEC><<<dim3(grid), C::T, lds_bytes, stream>>>(
          ab, xb, out, static_cast<int>(D), static_cast<int>(D), static_cast<int>(L),
          bb > 0 ? 1 : 0, tab, scratch, nullptr);
      MEGA_CHECK_LAUNCH();
    }
  }
  return scratch_used<LOGM>(stream);
}

template <int LOGM, int DT, int MODE>
int launch_fft(const void* a, const void* b, void* out, int64_t B, int64_t D, int64_t L, int flip,
               const float* omega, hipStream_t stream) {
  const auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 8 == 0; };
  const bool vec = (L % 2 == 0) && al(a) && al(b) && al(out);
  if (vec) return launch_fft_v<LOGM, DT, MODE, true>(a, b, out, B, D, L, flip, omega, stream);
#ifdef MEGA_FFTCONV_SINGLE
  return MEGA_ERR_UNSUPPORTED;
#else
  return launch_fft_v<LOGM, DT, MODE, false>(a, b, out, B, D, L, flip, omega, stream);
#endif
}

// ------------------------------ direct kernel --------------------------------
// L <= 2048: time-domain sums with both rows staged in LDS.
constexpr int kDirectMaxL = 2048;
constexpr int kDirectThreads = 256;

template <int DT, int MODE>
__global__ __launch_bounds__(kDirectThreads) void direct_conv_kernel(
    const void* __restrict__ a, const void* __restrict__ b, void* __restrict__ out, int B, int D,
    int L, int flip, const float* __restrict__ omega) {
  __shared__ float sa[kDirectMaxL];
  __shared__ float sb[kDirectMaxL];
  const int64_t esz = DT == MEGA_F32 ? 4 : 2;
  const int nb = MODE == 0 ? 1 : B;
  const int64_t d = MODE == 0 ? blockIdx.x % D : blockIdx.x;
  for (int bb = 0; bb < nb; ++bb) {
    const int64_t row = MODE == 0 ? blockIdx.x : static_cast<int64_t>(bb) * D + d;
    const char* arow = static_cast<const char*>(a) + row * L * esz;
    const bool fl = MODE == 1 || flip != 0;
    __syncthreads();
    for (int i = threadIdx.x; i < L; i += kDirectThreads) {
      sa[i] = ld<DT>(arow, fl ? L - 1 - i : i);
      if (MODE == 0)
        sb[i] = static_cast<const float*>(b)[d * L + i];
      else
        sb[i] = ld<DT>(static_cast<const char*>(b) + row * L * esz, i);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < L; i += kDirectThreads) {
      float acc = 0.f;
      for (int s = 0; s <= i; ++s) acc = fmaf(sb[i - s], sa[s], acc);
      const int o = fl ? L - 1 - i : i;
      if (MODE == 0) {
        if (omega != nullptr) acc = fmaf(omega[d], sa[i], acc);  // sa[i] is a[o]
        st<DT>(static_cast<char*>(out) + row * L * esz, o, acc);
      } else {
        float* orow = static_cast<float*>(out) + d * L;
        orow[o] = bb == 0 ? acc : orow[o] + acc;
      }
    }
  }
}

// The transforms are float32 unless MEGA_FFTCONV_F16_STAGES is set (to anything
// but "0") in the environment: then 16-bit rows the matrix-core engine can take
// run its fp16-operand DFT stages (3x faster, error ~1e-3 of the largest
// output instead of ~1e-6).  Read per call.
bool f16_stages_enabled() {
  const char* v = getenv("MEGA_FFTCONV_F16_STAGES");
  return v != nullptr && !(v[0] == '0' && v[1] == 0);
}

template <int DT, int MODE>
int launch_conv(const void* a, const void* b, void* out, int64_t B, int64_t D, int64_t L, int flip,
                const float* omega, hipStream_t stream) {
#ifdef MEGA_FFTCONV_SINGLE  // development switch: one instantiation, fast compile
  if (DT == MEGA_BF16 && MODE == 0) return launch_fft<14, MEGA_BF16, 0>(a, b, out, B, D, L, flip, omega, stream);
  return MEGA_ERR_UNSUPPORTED;
#else
  if (L <= kDirectMaxL) {
    const int64_t rows = MODE == 0 ? B * D : D;
    MEGA_CHECK_ARG(rows <= 0x7fffffff, "fftconv: too many rows");
    direct_conv_kernel<DT, MODE><<<dim3(static_cast<unsigned>(rows)), kDirectThreads, 0, stream>>>(
        a, b, out, static_cast<int>(B), static_cast<int>(D), static_cast<int>(L), flip, omega);
    MEGA_CHECK_LAUNCH();
    return MEGA_OK;
  }
  // opt-in: 16-bit rows run their DFT stages on the matrix cores with fp16 operands
  if (f16_stages_enabled() && fftm::applicable(DT, L, a, b, out))
    return fftm::launch_conv(DT, MODE, a, b, out, B, D, L, flip, omega, stream);
  if (L <= 4096) return launch_fft<11, DT, MODE>(a, b, out, B, D, L, flip, omega, stream);
  if (L <= 8192) return launch_fft<12, DT, MODE>(a, b, out, B, D, L, flip, omega, stream);
  if (L <= 16384) return launch_fft<13, DT, MODE>(a, b, out, B, D, L, flip, omega, stream);
  return launch_fft<14, DT, MODE>(a, b, out, B, D, L, flip, omega, stream);
#endif
}

template <int MODE>
int dispatch_conv(int dtype, const void* a, const void* b, void* out, int64_t B, int64_t D,
                  int64_t L, int flip, const float* omega, hipStream_t stream) {
  switch (dtype) {
    case MEGA_F32: return launch_conv<MEGA_F32, MODE>(a, b, out, B, D, L, flip, omega, stream);
    case MEGA_BF16: return launch_conv<MEGA_BF16, MODE>(a, b, out, B, D, L, flip, omega, stream);
    case MEGA_F16: return launch_conv<MEGA_F16, MODE>(a, b, out, B, D, L, flip, omega, stream);
  }
  return set_error(MEGA_ERR_INVALID_ARG, "fftconv: bad dtype %d", dtype);
}

constexpr int64_t kMaxL = 32768;

__global__ void zero_fill_kernel(float* p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_fftconv_max_length(void) { return static_cast<int>(kMaxL); }

extern "C" int mega_fftconv_prepare(int64_t L, void* stream) {
  MEGA_CHECK_ARG(L >= 0, "mega_fftconv_prepare: negative size");
  if (L > kMaxL)
    return set_error(MEGA_ERR_UNSUPPORTED, "mega_fftconv_prepare: L=%lld exceeds the supported %lld",
                     (long long)L, (long long)kMaxL);
  if (L <= kDirectMaxL) return MEGA_OK;  // the time-domain kernel needs neither tables nor scratch
  hipStream_t s = static_cast<hipStream_t>(stream);
  const c32* tab = nullptr;
  float* scratch = nullptr;
  int slots = 0;
  if (L <= 4096) return get_tables<11>(s, &tab, &scratch, &slots);
  if (L <= 8192) return get_tables<12>(s, &tab, &scratch, &slots);
  if (L <= 16384) return get_tables<13>(s, &tab, &scratch, &slots);
  return get_tables<14>(s, &tab, &scratch, &slots);
}

// Scratch blocks held on the current device for the transform size that rows
// of L samples take (0 for rows the time-domain kernel takes).
extern "C" int mega_fftconv_scratch_blocks(int64_t L) {
  if (L <= kDirectMaxL || L > kMaxL) return 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  const int size = L <= 4096 ? 0 : L <= 8192 ? 1 : L <= 16384 ? 2 : 3;
  std::lock_guard<std::mutex> lock(g_tables.mu);
  return static_cast<int>(g_tables.scratch[dev][size].size());
}

namespace {
int fftconv_fwd_impl(const char* who, const void* x, int dtype, const float* k, const float* omega,
                     int64_t B, int64_t D, int64_t L, void* y, void* stream) {
  MEGA_CHECK_ARG(x && k && y, "%s: null pointer", who);
  MEGA_CHECK_ARG(valid_dtype(dtype), "%s: bad dtype %d", who, dtype);
  MEGA_CHECK_ARG(B >= 0 && D >= 0 && L >= 0, "%s: negative size", who);
  if (L > kMaxL)
    return set_error(MEGA_ERR_UNSUPPORTED, "%s: L=%lld exceeds the supported %lld", who,
                     (long long)L, (long long)kMaxL);
  if (B == 0 || D == 0 || L == 0) return MEGA_OK;
  return dispatch_conv<0>(dtype, x, k, y, B, D, L, 0, omega, static_cast<hipStream_t>(stream));
}

int fftconv_bwd_impl(const char* who, const void* dy, const void* x, int dtype, const float* k,
                     const float* omega, int64_t B, int64_t D, int64_t L, void* dx, float* dk,
                     void* stream) {
  MEGA_CHECK_ARG(dy && x && k && dx && dk, "%s: null pointer", who);
  MEGA_CHECK_ARG(valid_dtype(dtype), "%s: bad dtype %d", who, dtype);
  MEGA_CHECK_ARG(B >= 0 && D >= 0 && L >= 0, "%s: negative size", who);
  if (L > kMaxL)
    return set_error(MEGA_ERR_UNSUPPORTED, "%s: L=%lld exceeds the supported %lld", who,
                     (long long)L, (long long)kMaxL);
  if (D == 0 || L == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0) {
    const int64_t n = D * L;
    zero_fill_kernel<<<dim3(static_cast<unsigned>((n + 255) / 256)), 256, 0, s>>>(dk, n);
    MEGA_CHECK_LAUNCH();
    return MEGA_OK;
  }
  if (fftm::applicable(dtype, L, dy, x, dx) && reinterpret_cast<uintptr_t>(k) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(dk) % 16 == 0 && f16_stages_enabled())
    return fftm::launch_backward(dtype, dy, x, k, dx, dk, B, D, L, omega, s);
  int rc = dispatch_conv<0>(dtype, dy, k, dx, B, D, L, 1, omega, s);
  if (rc != MEGA_OK) return rc;
  return dispatch_conv<1>(dtype, dy, x, dk, B, D, L, 1, nullptr, s);
}
}  // namespace

extern "C" int mega_fftconv_fwd(const void* x, int dtype, const float* k, int64_t B, int64_t D,
                                int64_t L, void* y, void* stream) {
  return fftconv_fwd_impl("mega_fftconv_fwd", x, dtype, k, nullptr, B, D, L, y, stream);
}

extern "C" int mega_fftconv_bwd(const void* dy, const void* x, int dtype, const float* k,
                                int64_t B, int64_t D, int64_t L, void* dx, float* dk,
                                void* stream) {
  return fftconv_bwd_impl("mega_fftconv_bwd", dy, x, dtype, k, nullptr, B, D, L, dx, dk, stream);
}

extern "C" int mega_fftconv_residual_fwd(const void* x, int dtype, const float* k,
                                         const float* omega, int64_t B, int64_t D, int64_t L,
                                         void* y, void* stream) {
  MEGA_CHECK_ARG(omega, "mega_fftconv_residual_fwd: null omega");
  return fftconv_fwd_impl("mega_fftconv_residual_fwd", x, dtype, k, omega, B, D, L, y, stream);
}

extern "C" int mega_fftconv_residual_bwd(const void* dy, const void* x, int dtype, const float* k,
                                         const float* omega, int64_t B, int64_t D, int64_t L,
                                         void* dx, float* dk, void* stream) {
  MEGA_CHECK_ARG(omega, "mega_fftconv_residual_bwd: null omega");
  return fftconv_bwd_impl("mega_fftconv_residual_bwd", dy, x, dtype, k, omega, B, D, L, dx, dk,
                          stream);
}

// ---- forward that keeps the spectra of x and k, backward that uses them ----------
extern "C" int64_t mega_fftconv_spectrum_bytes(int dtype, int64_t B, int64_t D, int64_t L) {
  if (B <= 0 || D <= 0 || L <= 0 || !f16_stages_enabled()) return 0;
  return fftm::spectrum_bytes(dtype, B, D, L);
}

extern "C" int mega_fftconv_residual_fwd_saving(const void* x, int dtype, const float* k,
                                                const float* omega, int64_t B, int64_t D,
                                                int64_t L, void* y, void* spec_x, void* spec_k,
                                                void* stream) {
  const char* who = "mega_fftconv_residual_fwd_saving";
  MEGA_CHECK_ARG(x && k && y && spec_x && spec_k, "%s: null pointer", who);
  MEGA_CHECK_ARG(fftm::spectrum_bytes(dtype, B, D, L) > 0 && fftm::applicable(dtype, L, x, k, y) &&
                     reinterpret_cast<uintptr_t>(spec_x) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(spec_k) % 16 == 0,
                 "%s: shape, dtype or alignment outside the saved-spectrum path "
                 "(mega_fftconv_spectrum_bytes returns 0 for it)", who);
  return fftm::launch_forward_saving(dtype, x, k, y, B, D, L, omega, spec_x, spec_k,
                                     static_cast<hipStream_t>(stream));
}

extern "C" int mega_fftconv_residual_bwd_saved(const void* dy, int dtype, const void* spec_x,
                                               const void* spec_k, const float* omega, int64_t B,
                                               int64_t D, int64_t L, void* dx, float* dk,
                                               void* stream) {
  const char* who = "mega_fftconv_residual_bwd_saved";
  MEGA_CHECK_ARG(dy && spec_x && spec_k && dx && dk, "%s: null pointer", who);
  MEGA_CHECK_ARG(fftm::spectrum_bytes(dtype, B, D, L) > 0 && fftm::applicable(dtype, L, dy, dx, dk) &&
                     reinterpret_cast<uintptr_t>(spec_x) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(spec_k) % 16 == 0,
                 "%s: shape, dtype or alignment outside the saved-spectrum path", who);
  return fftm::launch_backward_saved(dtype, dy, spec_x, spec_k, dx, dk, B, D, L, omega,
                                     static_cast<hipStream_t>(stream));
}
