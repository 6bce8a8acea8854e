// Streaming reference kernels: what this part's memory system delivers to a
// kernel that only moves the bytes of an HBM-bound operator, measured beside
// that operator.  out = a (one read stream, one write stream: the shape of the
// TimestepNorm and CEMA forward passes) or out = a ^ b (two read streams, one
// write stream: their backward passes).  Grid-stride over 16-byte vectors,
// eight loads per lane in flight before the first store.
#include "common.hpp"

namespace mega {
namespace {

constexpr int kInFlight = 8;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <bool TWO, bool NT>
__global__ __launch_bounds__(256) void stream_copy_kernel(const u32x4* __restrict__ a, const u32x4* __restrict__ b,
                                                          u32x4* __restrict__ out, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  constexpr int U = TWO ? kInFlight / 2 : kInFlight;
  for (; i + (U - 1) * stride < n; i += U * stride) {
    u32x4 va[U], vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      va[u] = NT ? __builtin_nontemporal_load(a + i + u * stride) : a[i + u * stride];
      if (TWO) vb[u] = NT ? __builtin_nontemporal_load(b + i + u * stride) : b[i + u * stride];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      u32x4 v = va[u];
      if (TWO) v ^= vb[u];
      if (NT) __builtin_nontemporal_store(v, out + i + u * stride);
      else out[i + u * stride] = v;
    }
  }
  for (; i < n; i += stride) {
    u32x4 v = a[i];
    if (TWO) v ^= b[i];
    out[i] = v;
  }
}

}  // namespace
}  // namespace mega

using namespace mega;

extern "C" int mega_bench_stream_copy(const void* a, const void* b, void* out, int64_t bytes, int workgroups,
                                      int nontemporal, void* stream) {
  MEGA_CHECK_ARG(a != nullptr && out != nullptr && bytes >= 0 && bytes % 16 == 0,
                 "mega_bench_stream_copy: null pointer or size not a multiple of 16 bytes");
  const auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  MEGA_CHECK_ARG(al(a) && al(out) && (b == nullptr || al(b)), "mega_bench_stream_copy: operands must be 16-byte aligned");
  MEGA_CHECK_ARG(workgroups >= 1 && workgroups <= (1 << 20), "mega_bench_stream_copy: bad workgroup count");
  if (bytes == 0) return MEGA_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = bytes / 16;
  const u32x4* pa = static_cast<const u32x4*>(a);
  const u32x4* pb = static_cast<const u32x4*>(b);
  u32x4* po = static_cast<u32x4*>(out);
  if (b == nullptr && nontemporal) stream_copy_kernel<false, true><<<workgroups, 256, 0, s>>>(pa, pb, po, n);
  else if (b == nullptr) stream_copy_kernel<false, false><<<workgroups, 256, 0, s>>>(pa, pb, po, n);
  else if (nontemporal) stream_copy_kernel<true, true><<<workgroups, 256, 0, s>>>(pa, pb, po, n);
  else stream_copy_kernel<true, false><<<workgroups, 256, 0, s>>>(pa, pb, po, n);
  MEGA_CHECK_LAUNCH();
  return MEGA_OK;
}
