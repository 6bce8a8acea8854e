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

// Saved spectra.  spectrum_bytes: size of the spectrum buffer of x for the shape
// (that of k, kept once per channel, has the size for B = 1), 0 when the shape cannot take this path (16-bit rows, 2048 < L
// <= 32768, L % 8 == 0, D a multiple of the rows per pass).  launch_forward_saving
// is launch_conv mode 0 that also fills both buffers; launch_backward_saved
// computes dx (+ omega dy) and dk from dy and the two buffers alone.
int64_t spectrum_bytes(int dtype, int64_t B, int64_t D, int64_t L);
int launch_forward_saving(int dtype, const void* x, const float* k, void* y, int64_t B, int64_t D,
                          int64_t L, const float* omega, void* spec_x, void* spec_k,
                          hipStream_t stream);
int launch_backward_saved(int dtype, const void* dy, const void* spec_x, const void* spec_k, void* dx,
                          float* dk, int64_t B, int64_t D, int64_t L, const float* omega,
                          hipStream_t stream);

}  // namespace fftm
}  // namespace mega
