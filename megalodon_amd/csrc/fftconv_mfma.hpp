// Matrix-core convolution engine for 16-bit rows (fftconv_mfma.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mega {
namespace fftm {

// bf16 / fp16 rows, 2048 < L <= 32768, L % 8 == 0, 16-byte aligned operands
bool applicable(int dtype, int64_t L, const void* a, const void* b, const void* out);

// mode 0: out[b,d,:] = conv(a[b,d,:], k[d,:]) (+ omega[d] a), k fp32, `flip` = backward dx form;
// mode 1: out[d,:] = sum_b reverse(conv(reverse(a[b,d,:]), x[b,d,:])), fp32 out.
int launch_conv(int dtype, int mode, const void* a, const void* b, void* out, int64_t B, int64_t D,
                int64_t L, int flip, const float* omega, hipStream_t stream);

// dx (+ omega dy) and dk of the convolution in one launch (dy is transformed once);
// dk (D, L) fp32 is overwritten.  Same applicability as launch_conv; B >= 1.
int launch_backward(int dtype, const void* dy, const void* x, const float* k, void* dx, float* dk,
                    int64_t B, int64_t D, int64_t L, const float* omega, hipStream_t stream);

}  // namespace fftm
}  // namespace mega
