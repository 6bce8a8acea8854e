/*
 * megalodon_hip.h -- C ABI of libmegalodon_hip.so (gfx950 / MI355X).
 *
 * Drop-in boundary for the fused-op hot path of XuezheMax/megalodon.  Each
 * entry point replaces one function of the reference's pybind module
 * `megalodon_extension.ops` (registered in megalodon/csrc/megalodon_extension.cc:14-24).
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer to contiguous memory unless stated;
 *   - the caller owns and allocates inputs AND outputs (the reference's
 *     callee-allocates `torch::empty` moves to the Python wrapper);
 *   - `stream` is a hipStream_t passed as void*; kernels are enqueued on it and
 *     the call returns without synchronising (the reference enqueues on the
 *     current CUDA stream the same way, e.g. ema_parameters_kernel.cu:1033);
 *   - return value 0 = MEGA_OK; otherwise an error code, with a message kept
 *     in a thread-local buffer readable through mega_last_error() (the
 *     reference raises c10::Error through TORCH_CHECK);
 *   - complex tensors are interleaved (re, im) float pairs = torch.complex64;
 *   - no entry point allocates device memory except where a `workspace`
 *     argument is documented.
 */
#ifndef MEGALODON_HIP_H_
#define MEGALODON_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MEGA_OK 0
#define MEGA_ERR_INVALID_ARG 1
#define MEGA_ERR_UNSUPPORTED 2
#define MEGA_ERR_HIP 3
#define MEGA_ERR_TIMEOUT 4   /* a bounded device-side wait ran out (mega_group_timestep_norm_status) */

/* element types of activation tensors (x, y, dy, dx, q, k, v ...) */
#define MEGA_F32 0
#define MEGA_BF16 1
#define MEGA_F16 2
/* float64: taken by the operators that say so (the double-precision flavours) */
#define MEGA_F64 3

/* Library version (major*10000 + minor*100 + patch). */
int mega_version(void);

/* Message of the last error raised on the calling thread ("" if none). */
const char* mega_last_error(void);

/* ------------------------------------------------------------------------
 * CEMA convolution-kernel generation (weight path).
 *
 * Replaces ema_parameters_fwd(p, log_q, gamma, h=None, L) -> (w, None, None)
 *   reference: megalodon/csrc/ops/ema_parameters.cc:17-52 (CPU),
 *              ema_parameters_kernel.cu:74-121 (CUDA), binding ema_parameters.cc:289.
 *   w[d, j] = sum_n Re(p[d,n] * gamma[d,n] * exp(log_q[d,n] * j)),  j = 0..L-1
 *   p      (D, N)  float32
 *   log_q  (D, N)  complex64
 *   gamma  (D, N)  complex64
 *   w      (D, L)  float32 (output)
 *   1 <= N <= 32 (reference limit, ema_parameters_kernel.cu:1026).
 * ---------------------------------------------------------------------- */
int mega_ema_weight_fwd(const float* p, const float* log_q, const float* gamma,
                        int64_t D, int64_t N, int64_t L, float* w,
                        void* stream);

/* Replaces ema_parameters_bwd(dw, None, p, log_q, gamma, None, None)
 *   -> (dp, dq, dgamma, None)
 *   reference: ema_parameters.cc:80-98,141-156 (CPU),
 *              ema_parameters_kernel.cu:396-472 (CUDA), binding ema_parameters.cc:290.
 *   S1 = sum_j dw[j] * j * q^(j-1),  S2 = sum_j dw[j] * q^j
 *   dp = Re(S2 * gamma), dq = conj(S1 * p * gamma), dgamma = conj(S2 * p)
 *   (gradients w.r.t. q, not log q; PyTorch conjugate convention)
 *   dw (D, L) float32; dp (D, N) float32; dq, dgamma (D, N) complex64. */
int mega_ema_weight_bwd(const float* dw, const float* p, const float* log_q,
                        const float* gamma, int64_t D, int64_t N, int64_t L,
                        float* dp, float* dq, float* dgamma, void* stream);

/* The double-precision flavours of the two operators above and of the causal
 * convolution (ema_parameters_kernel.cu:1227 dispatches p over float64 with
 * complex128 log_q / gamma; fftconv_kernel.cu:468-476,487-499 takes float64 x
 * with complex128 spectra): the defining sums evaluated directly in double --
 * every power from its own exp / sincos, the convolution as the triangular sum
 * out[r, t] = sum_{s <= t} a[r % rows_a, s] * b[r, t - s] (rows of L doubles;
 * a = the kernel rows (D, L), b = x (B*D, L) gives fftconv's y; the two
 * backward sums are the same convolution of time-reversed rows).  For checking
 * results, not for speed.  Sizes and layouts as above with double / complex128. */
int mega_ema_weight_fwd_f64(const double* p, const double* log_q, const double* gamma,
                            int64_t D, int64_t N, int64_t L, double* w, void* stream);
int mega_ema_weight_bwd_f64(const double* dw, const double* p, const double* log_q,
                            const double* gamma, int64_t D, int64_t N, int64_t L,
                            double* dp, double* dq, double* dgamma, void* stream);
int mega_causal_conv_f64(const double* a, const double* b, int64_t rows_a, int64_t rows,
                         int64_t L, double* out, void* stream);

/* ------------------------------------------------------------------------
 * CEMA coefficients from the raw parameters, and their gradients.
 *
 * Replaces MultiHeadComplexEMA._calc_coeffs and its autograd graph
 *   reference: megalodon/modules/complex_exponential_moving_average.py:100-117
 *   (about thirty elementwise PyTorch kernels per training step there).
 *   alpha, delta (D, N), theta (D), gamma (D, N, 2) float32 ->
 *   p = sigmoid(alpha) (D, N) float32;
 *   log_q = (ln(1 - sigmoid(alpha) sigmoid(delta)), n sigmoid(theta) 2 pi / N),
 *   n = 1 .. N, (D, N) complex64 -- the logarithm of the reference's q, which is
 *   what mega_ema_weight_fwd takes;
 *   gamma_hat = (gamma_0 + i gamma_1) sqrt(1 / N) (D, N) complex64.  N <= 64.
 * Backward: dp (D, N) float32, dq and dgamma_hat (D, N) complex64 as
 *   mega_ema_weight_bwd returns them (gradient w.r.t. q, PyTorch's complex
 *   convention) -> dalpha, ddelta (D, N), dtheta (D), dgamma (D, N, 2).
 * ---------------------------------------------------------------------- */
int mega_cema_coeffs_fwd(const float* alpha, const float* delta, const float* theta,
                         const float* gamma, int64_t D, int64_t N, float* p, float* log_q,
                         float* gamma_hat, void* stream);
int mega_cema_coeffs_bwd(const float* dp, const float* dq, const float* dgamma_hat,
                         const float* alpha, const float* delta, const float* theta, int64_t D,
                         int64_t N, float* dalpha, float* ddelta, float* dtheta, float* dgamma,
                         void* stream);

/* ------------------------------------------------------------------------
 * Causal FFT convolution.
 *
 * Replaces fftconv_fwd(x, k_f) -> (y, x_f) and the torch.fft branch used for
 * L > 16384, i.e. `_fftconv_fwd` / `fused_fftconv_fwd`
 *   reference: megalodon/modules/fused_ops/fftconv.py:30-50,79-93,
 *              megalodon/csrc/ops/fftconv_kernel.cu:34-78,480-501, binding fftconv.cc:22-33.
 *   y[b,d,t] = sum_{s<=t} k[d,t-s] x[b,d,s]
 *            = irfft(rfft(x, 2N) * rfft(k, 2N))[:L],  N = 2^ceil(log2 L)
 *   x, y (B, D, L) of `dtype` (MEGA_F32 / MEGA_BF16 / MEGA_F16);
 *   k (D, L) float32 in the TIME domain (the reference passes rfft(k); here
 *   the transform of k happens inside the kernel and nothing is saved).
 *   Arithmetic is float32 throughout for every dtype (16-bit rows are
 *   widened on load as the reference does, fftconv.py:37-44; y is rounded
 *   once on store): error against a float64 convolution ~1e-6 of the largest
 *   output before that rounding.
 *   Opt-in: with MEGA_FFTCONV_F16_STAGES set in the environment (to anything
 *   but "0"; read per call), bfloat16 / float16 rows with 2048 < L,
 *   L % 8 == 0 and 16-byte aligned x, k, y run their DFT stages on the matrix
 *   cores (fp16 operands, fp32 accumulation, fp16 between stages, rows
 *   pre-scaled by a power of two; twiddles, the spectral product and all sums
 *   in float32): about 3x faster, measured error <= 4e-3 of the largest output
 *   (y, dx) and 1.1e-3 (dk), i.e. inside the 16-bit bar but not the float32
 *   one.
 *   L <= mega_fftconv_max_length() (32768); longer rows return
 *   MEGA_ERR_UNSUPPORTED.
 *   The float32 engine needs twiddle tables (one per device and transform
 *   size) and per-workgroup scratch blocks (per device and transform size:
 *   a stream gets a block of its own, so launches on different streams never
 *   share slots, up to four blocks; a fifth stream takes over the block that
 *   has been idle longest and waits on the device for the last launch that
 *   used it); they are kept until process exit (64 MiB per block at the
 *   largest size on 256 compute units).  mega_fftconv_prepare(L, stream) makes
 *   them ahead of time (it allocates and synchronises `stream` once; not
 *   capturable); after it, the convolution entry points on that stream only
 *   enqueue.  Without it the first call for a size / stream does the same
 *   work itself.  To capture a convolution into a graph, prepare the stream
 *   the capture runs on; a block used under capture belongs to that graph's
 *   replays and is never handed to another stream.
 *   mega_fftconv_scratch_blocks(L): blocks held on the current device for the
 *   transform size of rows of L samples.
 * ---------------------------------------------------------------------- */
int mega_fftconv_prepare(int64_t L, void* stream);
int mega_fftconv_scratch_blocks(int64_t L);
int mega_fftconv_max_length(void);
int mega_fftconv_fwd(const void* x, int dtype, const float* k, int64_t B,
                     int64_t D, int64_t L, void* y, void* stream);

/* Replaces fftconv_bwd(dy, x_f, k_f, k_dtype) -> (dx, dk) / `_fftconv_bwd`
 *   reference: fftconv.py:53-75,96-106, fftconv_kernel.cu:80-164,503-520.
 *   dx[b,d,t] = sum_{s>=t} dy[b,d,s] k[d,s-t]
 *   dk[d,j]   = sum_b sum_{t>=j} dy[b,d,t] x[b,d,t-j]
 *   Takes x and k themselves (the spectra are recomputed, not saved).
 *   dy, x, dx (B, D, L) of `dtype`; k, dk (D, L) float32. */
int mega_fftconv_bwd(const void* dy, const void* x, int dtype, const float* k,
                     int64_t B, int64_t D, int64_t L, void* dx, float* dk,
                     void* stream);

/* The convolution and the per-channel skip term of MultiHeadComplexEMA in one
 * pass: y = fftconv(x, k) + omega[d] * x.
 *   Replaces the pair `fftconv(x, k) + x * self.omega` of
 *   megalodon/modules/complex_exponential_moving_average.py:129-141 (forward of
 *   MultiHeadComplexEMA); omega (D) float32, the rest as mega_fftconv_fwd/bwd.
 *   Backward: dx = (dx of the convolution) + omega[d] * dy; dk as in
 *   mega_fftconv_bwd.  The gradient of omega is dk[:, 0]
 *   (sum_b sum_t dy[b,d,t] x[b,d,t], the lag-0 correlation), so it has no
 *   output of its own. */
int mega_fftconv_residual_fwd(const void* x, int dtype, const float* k,
                              const float* omega, int64_t B, int64_t D,
                              int64_t L, void* y, void* stream);
int mega_fftconv_residual_bwd(const void* dy, const void* x, int dtype,
                              const float* k, const float* omega, int64_t B,
                              int64_t D, int64_t L, void* dx, float* dk,
                              void* stream);

/* ------------------------------------------------------------------------
 * Group TimestepNorm (cumulative group mean / variance over time).
 *
 * Replaces group_timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma,
 *   beta, padding_mask?, num_groups, eps)
 *   -> (y, count, mean, var, cummean, cumrstd)
 *   reference: megalodon/csrc/ops/timestep_norm.cc:218-316 (CPU),
 *              timestep_norm_kernel.cu:453-681,1252-1326 (CUDA), binding timestep_norm.cc:702.
 *   x, y (B, L, D) of `dtype`; gamma, beta (D); prev_mean, prev_var, mean, var
 *   (B, G), all of `dtype`; prev_count, count (B) int64; padding_mask (B, L)
 *   bytes (non-zero = padding) or NULL; cummean, cumrstd (B, L, G) float32.
 *   Masked steps leave the running statistics unchanged and give y = 0; the
 *   stored cummean / cumrstd at a masked step are those of the unchanged state.
 *   `workspace`: mega_group_timestep_norm_workspace_bytes(B, L, D, G, 0) bytes
 *   of device memory, contents irrelevant on entry (cleared by the call).
 * ---------------------------------------------------------------------- */
int64_t mega_group_timestep_norm_workspace_bytes(int64_t B, int64_t L, int64_t D,
                                                 int64_t G, int backward);
int mega_group_timestep_norm_fwd(const void* x, int dtype, const int64_t* prev_count,
                                 const void* prev_mean, const void* prev_var,
                                 const void* gamma, const void* beta,
                                 const uint8_t* padding_mask, int64_t B, int64_t L,
                                 int64_t D, int64_t G, double eps, void* y,
                                 int64_t* count, void* mean, void* var,
                                 float* cummean, float* cumrstd, void* workspace,
                                 void* stream);

/* mega_group_timestep_norm_fwd / _bwd with the saved statistics time-last:
 * cummean, cumrstd (B, G, L) instead of the reference's (B, L, G)
 * (timestep_norm_kernel.cu:1553-1565 allocates them as {B, L, G}).  For a caller
 * that hands them from the forward to the backward and nowhere else: a
 * wavefront owns 64 steps of one group, so time-last it writes and reads 256
 * contiguous bytes per array where the reference layout has it touch 64 lines
 * for 4 bytes each.  Everything else as the two entry points without _tl
 * (declared here for the forward, below for the backward). */
int mega_group_timestep_norm_fwd_tl(const void* x, int dtype, const int64_t* prev_count,
                                    const void* prev_mean, const void* prev_var,
                                    const void* gamma, const void* beta,
                                    const uint8_t* padding_mask, int64_t B, int64_t L,
                                    int64_t D, int64_t G, double eps, void* y,
                                    int64_t* count, void* mean, void* var,
                                    float* cummean, float* cumrstd, void* workspace,
                                    void* stream);

/* The forward above for callers that cannot allocate (code under graph
 * capture, serving loops, harnesses that forbid it).  No counterpart in the
 * reference, whose operators allocate their own scratch (torch::empty in
 * timestep_norm_kernel.cu:1542-1565).  Same arguments without `workspace`: the
 * tickets, per-tile counts and look-back records live in a static device
 * array of mega_group_timestep_norm_static_scratch_bytes() (2 MiB) per GPU,
 * held until the process ends.  Shapes whose
 * mega_group_timestep_norm_workspace_bytes(B, L, D, G, 0) exceeds it return
 * MEGA_ERR_UNSUPPORTED.  The call allocates and frees nothing and clears what
 * it needs itself with a kernel; all calls on one GPU share the one array, so
 * two calls that overlap on a GPU (different streams, different threads) race
 * -- serialise them. */
int64_t mega_group_timestep_norm_static_scratch_bytes(void);
int mega_group_timestep_norm_fwd_static(const void* x, int dtype, const int64_t* prev_count,
                                        const void* prev_mean, const void* prev_var,
                                        const void* gamma, const void* beta,
                                        const uint8_t* padding_mask, int64_t B, int64_t L,
                                        int64_t D, int64_t G, double eps, void* y, int64_t* count,
                                        void* mean, void* var, float* cummean, float* cumrstd,
                                        void* stream);

/* Replaces group_timestep_norm_bwd(dy, dmean, dvar, x, prev_mean, count,
 *   cummean, cumrstd, gamma, padding_mask?, num_groups)
 *   -> (dx, dprev_mean, dprev_var, dgamma, dbeta)
 *   reference: timestep_norm.cc:318-450 (CPU), timestep_norm_kernel.cu:683-1086,
 *              1328-1439 (CUDA), binding timestep_norm.cc:704.
 *   `count` is the forward's output count; dgamma, dbeta (D) of `dtype`.
 *   `workspace`: mega_group_timestep_norm_workspace_bytes(B, L, D, G, 1) bytes. */
int mega_group_timestep_norm_bwd(const void* dy, const void* dmean, const void* dvar,
                                 const void* x, int dtype, const void* prev_mean,
                                 const int64_t* count, const float* cummean,
                                 const float* cumrstd, const void* gamma,
                                 const uint8_t* padding_mask, int64_t B, int64_t L,
                                 int64_t D, int64_t G, void* dx, void* dprev_mean,
                                 void* dprev_var, void* dgamma, void* dbeta,
                                 void* workspace, void* stream);
/* the same with cummean, cumrstd (B, G, L), as mega_group_timestep_norm_fwd_tl writes them */
int mega_group_timestep_norm_bwd_tl(const void* dy, const void* dmean, const void* dvar,
                                    const void* x, int dtype, const void* prev_mean,
                                    const int64_t* count, const float* cummean,
                                    const float* cumrstd, const void* gamma,
                                    const uint8_t* padding_mask, int64_t B, int64_t L,
                                    int64_t D, int64_t G, void* dx, void* dprev_mean,
                                    void* dprev_var, void* dgamma, void* dbeta,
                                    void* workspace, void* stream);

/* The double-precision flavour of the two operators above
 * (timestep_norm_kernel.cu:1567-1576 instantiates the reference's kernels for
 * double, with float64 cummean / cumrstd, :1553-1565): every tensor float64
 * except prev_count / count (int64) and the mask; one wavefront per (batch,
 * group) chain walks the sequence, so there are no look-back records and the
 * forward needs no workspace.  The backward's `workspace`: 2 * B * D doubles. */
int mega_group_timestep_norm_fwd_f64(const double* x, const int64_t* prev_count,
                                     const double* prev_mean, const double* prev_var,
                                     const double* gamma, const double* beta,
                                     const uint8_t* padding_mask, int64_t B, int64_t L,
                                     int64_t D, int64_t G, double eps, double* y,
                                     int64_t* count, double* mean, double* var,
                                     double* cummean, double* cumrstd, void* stream);
int mega_group_timestep_norm_bwd_f64(const double* dy, const double* dmean, const double* dvar,
                                     const double* x, const double* prev_mean,
                                     const int64_t* count, const double* cummean,
                                     const double* cumrstd, const double* gamma,
                                     const uint8_t* padding_mask, int64_t B, int64_t L,
                                     int64_t D, int64_t G, double* dx, double* dprev_mean,
                                     double* dprev_var, double* dgamma, double* dbeta,
                                     double* workspace, void* stream);

/* The tiled kernels above hand running statistics from tile to tile through
 * records in `workspace`; a tile polls for its predecessors' records at most a
 * fixed number of times (a couple of seconds), then sets a status word in the
 * workspace, continues with NaN in place of the missing value and exits, so a
 * launch always drains.  No counterpart in the reference, whose kernels scan a
 * sequence inside one thread block (timestep_norm_kernel.cu:1288-1325).
 * mega_group_timestep_norm_status waits for `stream`, reads the status word of
 * the last forward or backward launch that used `workspace` (NULL: the static
 * buffer of mega_group_timestep_norm_fwd_static on the current device) and
 * returns MEGA_OK or MEGA_ERR_TIMEOUT.
 * mega_test_timestep_norm_lookback is a test hook for the launches that
 * follow it: `spin_limit` polls per wait (<= 0: the default) and a tile index
 * that publishes no record (-1: none), which makes its successors run into
 * the limit without any kernel hanging. */
int mega_group_timestep_norm_status(const void* workspace, void* stream);
void mega_test_timestep_norm_lookback(long long spin_limit, int mute_tile);

/* ------------------------------------------------------------------------
 * Chunk attention (causal inside each chunk), fused fp32 softmax.
 *
 * Replaces attention_fwd(q, k, v, scale, dropout=0, use_causal_mask) -> (y, w)
 *   reference: megalodon/csrc/ops/attention_kernel.cu:40-133,261-281,
 *              megalodon/csrc/softmax.cuh:86-131, binding attention.cc:28.
 *   q (B, L1, NH, H1), k (B, L2, NH, H1), v (B, L2, NH, H2), y (B, L1, NH, H2),
 *   w (B, NH, L1, L2), all of `dtype`, contiguous; B counts chunks (the
 *   module views (batch, L) as (batch*L/chunk, chunk)).  MEGA_BF16 / MEGA_F16
 *   run on the matrix cores and are what follows describes; MEGA_F32 and
 *   MEGA_F64 (attention_kernel.cu:269-281 dispatches over them too) keep
 *   storage and arithmetic of that type on the vector ALUs, write every row of
 *   w to its end, and need two / four times the workspace bytes the size query
 *   returns.
 *   S = scale * q k^T (rounded to `dtype` as in the reference where S passes
 *   through w; the one-kernel path below feeds it to the softmax in float32);
 *   with `causal` row r keeps columns
 *   0 .. L2 - L1 + r (L2 >= L1 required: cached keys / values in front of the
 *   chunk, softmax.cuh:99-100), all columns otherwise; P = softmax in fp32,
 *   stored in `dtype` into w; y = P v.
 *   `causal`: 0 = every key; 1 = the causal mask, every row of w written to
 *   its end as the reference's softmax does (masked columns are exp(-inf) = 0,
 *   softmax.cuh:99-105,127-129); 2 = the same mask and the same y, but with
 *   L1 == L2 a row of w is written only up to the end of the 256-column block
 *   that holds its diagonal (zeros above the diagonal inside that block) and
 *   the blocks to the right are left untouched -- for a caller that hands w
 *   to mega_attention_bwd and nowhere else (the backward never reads them;
 *   the zero fill is 0.1 ms of 1.3 at 32 x 4096 x 4096).  With L2 > L1 both
 *   values write every row to its end.
 *   For head widths H1 of 64, 128 or 256 (16-byte aligned tensors, L2 % 8 == 0,
 *   no dropout) scores and softmax are one kernel and S never reaches memory;
 *   other shapes form S in w and run the softmax over it in place.
 *   Without dropout use mega_attention_fwd; with DropKey dropout
 *   (softmax.cuh:135-196, attention_kernel.cu:99-116)
 *   mega_attention_dropkey_fwd, below.
 *   `workspace`: mega_attention_workspace_bytes(B, L1, L2, NH, H1, H2, 0) bytes.
 * ---------------------------------------------------------------------- */
int64_t mega_attention_workspace_bytes(int64_t B, int64_t L1, int64_t L2, int64_t NH,
                                       int64_t H1, int64_t H2, int backward);
int mega_attention_fwd(const void* q, const void* k, const void* v, int dtype,
                       int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1,
                       int64_t H2, double scale, int causal, void* y, void* w,
                       void* workspace, void* stream);

/* attention_fwd with dropout > 0 (attention_kernel.cu:99-116, softmax.cuh:135-196):
 *   before the softmax every kept key of every row is taken out (score -> -inf)
 *   with probability `dropout`; the survivors are not rescaled; a row that
 *   loses all its keys becomes 0.  The backward is mega_attention_bwd unchanged
 *   (a dropped key has probability 0 in w).  The draw for (row i, column j),
 *   i = (b * NH + head) * L1 + r, is word j % 4 of Philox4x32-10 with counter
 *   (j / 4, i, offset & 0xffffffff, offset >> 32) and key (seed & 0xffffffff,
 *   seed >> 32): dropped iff (word >> 8) * 2^-24 < (float)dropout.  The reference
 *   takes (seed, offset) from PyTorch's CUDA generator and walks curand's
 *   per-thread streams, so the two masks differ for the same seed while their
 *   distribution is the same; a caller that wants fresh masks advances `offset`
 *   by any amount between calls.  dropout == 0 is mega_attention_fwd. */
int mega_attention_dropkey_fwd(const void* q, const void* k, const void* v, int dtype,
                               int64_t B, int64_t L1, int64_t L2, int64_t NH, int64_t H1,
                               int64_t H2, double scale, int causal, double dropout,
                               uint64_t seed, uint64_t offset, void* y, void* w,
                               void* workspace, void* stream);

/* Replaces attention_bwd(dy, q, k, v, w, scale, use_causal_mask) -> (dq, dk, dv)
 *   reference: attention_kernel.cu:135-257,283-303, softmax.cuh:198-234,
 *              binding attention.cc:29.
 *   dv = P^T dy; dP = dy v^T; dS = P o (dP - rowsum(P o dP)); dq = scale dS k;
 *   dk = scale dS^T q.  `w` is the forward's output.
 *   `workspace`: mega_attention_workspace_bytes(B, L1, L2, NH, H1, H2, 1) bytes. */
int mega_attention_bwd(const void* dy, const void* q, const void* k, const void* v,
                       const void* w, int dtype, int64_t B, int64_t L1, int64_t L2,
                       int64_t NH, int64_t H1, int64_t H2, double scale, int causal,
                       void* dq, void* dk, void* dv, void* workspace, void* stream);

/* dw[o][i] = sum_t dy[t][o] * x[t][i]: the weight gradient of y = x W^T for dy
 * (tokens, n_out) and x (tokens, n_in), dw (n_out, n_in), all of `dtype`
 * (MEGA_BF16 / MEGA_F16, float32 accumulation), contiguous, on the attention
 * operator's product kernel (both operands run across the reduction axis, as in
 * dV = P^T dY).  Replaces the `grad_output.t().matmul(input)` of the linear layers'
 * autograd (megalodon/modules/model_parallel/layers.py:222-235,321-341 are
 * F.linear at model-parallel world size 1). */
int mega_linear_weight_grad(const void* dy, const void* x, int dtype, int64_t tokens,
                            int64_t n_out, int64_t n_in, void* dw, void* stream);

/* ------------------------------------------------------------------------
 * Convolution with spectra kept between forward and backward.
 *
 * The reference's fused operator returns the spectrum of x for the backward
 * pass and takes the spectrum of k (fftconv_fwd(x, k_f) -> (y, x_f),
 * fftconv_bwd(dy, x_f, k_f, k_dtype), megalodon/modules/fused_ops/fftconv.py:
 * 21-28,62-75, csrc/ops/fftconv_kernel.cu:34-164).  This pair does the same for
 * the matrix-core path (the fp16-stage engine, opt-in through
 * MEGA_FFTCONV_F16_STAGES as described at mega_fftconv_fwd; without it
 * mega_fftconv_spectrum_bytes returns 0): the forward also writes the spectra of x and of k (an
 * opaque fp16 layout with the rows' scales, 16-byte aligned: spec_x takes
 * mega_fftconv_spectrum_bytes(dtype, B, D, L) bytes, spec_k, which depends on
 * the channel only, mega_fftconv_spectrum_bytes(dtype, 1, D, L)), the backward
 * needs only dy and the two buffers: dx = corr(dy, k) + omega dy, dk = sum_b corr(dy, x) from three
 * transforms per row instead of five.  mega_fftconv_spectrum_bytes returns 0
 * for shapes outside this path (float32 rows, L <= 2048, L % 8 != 0, D not a
 * multiple of the rows per pass: 32768 / 2^ceil(log2 L) for L > 2048); use
 * mega_fftconv_residual_fwd / _bwd then.  omega may be null (no skip term).
 * ---------------------------------------------------------------------- */
int64_t mega_fftconv_spectrum_bytes(int dtype, int64_t B, int64_t D, int64_t L);
int mega_fftconv_residual_fwd_saving(const void* x, int dtype, const float* k, const float* omega,
                                     int64_t B, int64_t D, int64_t L, void* y, void* spec_x,
                                     void* spec_k, void* stream);
int mega_fftconv_residual_bwd_saved(const void* dy, int dtype, const void* spec_x,
                                    const void* spec_k, const float* omega, int64_t B, int64_t D,
                                    int64_t L, void* dx, float* dk, void* stream);

/* ------------------------------------------------------------------------
 * Standalone softmax of attention scores, in place.
 *
 * Replaces attention_softmax_fwd(x, dropout=0, use_causal_mask) -> y
 *   reference: megalodon/csrc/ops/attention_softmax_kernel.cu:22-66,96-108,
 *              megalodon/csrc/softmax.cuh:86-131, binding attention_softmax.cc:6-10,20-22.
 *   x: Z matrices (L1, L2) of `dtype` (MEGA_BF16 or MEGA_F16), contiguous,
 *   overwritten by y = softmax over the last axis in float32; with `causal`
 *   row r keeps columns 0 .. L2 - L1 + r (L2 >= L1) and the rest of the row
 *   becomes 0.  The caller copies x first if it must survive (the reference
 *   returns a new tensor).  mega_attention_softmax_dropkey_fwd is the same with
 *   DropKey dropout (attention_softmax_kernel.cu:50-65); rows are numbered
 *   i = matrix * L1 + r and drawn as described at mega_attention_dropkey_fwd.
 * Replaces attention_softmax_bwd(y_grad, y, use_causal_mask) -> x_grad
 *   reference: attention_softmax_kernel.cu:68-94,110-123, softmax.cuh:198-234,
 *              binding attention_softmax.cc:12-18.
 *   dy is overwritten by dx = y o (dy - rowsum(y o dy)) (0 where masked).
 * ---------------------------------------------------------------------- */
int mega_attention_softmax_fwd(void* x, int dtype, int64_t Z, int64_t L1, int64_t L2,
                               int causal, void* stream);
int mega_attention_softmax_dropkey_fwd(void* x, int dtype, int64_t Z, int64_t L1, int64_t L2,
                                       int causal, double dropout, uint64_t seed,
                                       uint64_t offset, void* stream);
int mega_attention_softmax_bwd(const void* y, void* dy, int dtype, int64_t Z, int64_t L1,
                               int64_t L2, int causal, void* stream);

/* ------------------------------------------------------------------------
 * Dropout that keeps no mask and no generator state.
 *
 * Replaces memory_efficient_dropout_fwd / _bwd
 *   reference: megalodon/modules/fused_ops/memory_efficient_dropout.py:39-96
 *   (bernoulli(1 - p) / (1 - p) noise, rebuilt in the backward by replaying the
 *   CUDA generator from its saved state).
 *   out[e] = in[e] / (1 - p) if element e is kept, else 0; e is kept iff word
 *   e % 4 of Philox4x32-10 with counter (e / 4 as two 32-bit words, offset as
 *   two 32-bit words) and key seed gives (word >> 8) * 2^-24 >= (float)p.  The
 *   backward is the same call on the gradient with the same (p, seed, offset).
 *   `in` and `out` (n elements of `dtype`: float32, bfloat16 or float16) may be
 *   the same buffer.  p == 1 gives zeros (the reference's 0 / 0 gives NaN).
 * ---------------------------------------------------------------------- */
int mega_dropout(const void* in, int dtype, int64_t n, double p, uint64_t seed, uint64_t offset,
                 void* out, void* stream);

/* ------------------------------------------------------------------------
 * Block glue: the transposes around the EMA convolution and the SiLU gates.
 *
 * mega_transpose: in (Z, R, C) -> out (Z, C, R), contiguous, `in` != `out`.
 *   Replaces the strided copies behind `out_tsn.transpose(1, 2)` and
 *   `out_cema.transpose(1, 2)` (megalodon/modules/moving_average_gated_attention.py:
 *   299-300,314, and their gradients).  16-bit elements with R % 8 == 0,
 *   C % 8 == 0 and 16-byte aligned buffers move in 128 x 128 tiles with 16-byte
 *   accesses on both sides; everything else takes a 32 x 32 element-wise path.
 * mega_silu_mul_fwd: out = silu(a) * b, n elements of `dtype`, float32 inside
 *   with one rounding (PyTorch's `F.silu(a) * b` rounds twice).
 *   Replaces `F.silu(self.fc1(x)) * self.fc3(x)`
 *   (normalized_feedforward_network.py:82) and `attn * F.silu(self.wr(mx))`
 *   (moving_average_gated_attention.py:333-336).
 * mega_silu_mul_bwd: da = dout * b * s * (1 + a (1 - s)), db = dout * a * s,
 *   s = sigmoid(a); the forward's result is not needed.
 * ---------------------------------------------------------------------- */
int mega_transpose(const void* in, int dtype, int64_t Z, int64_t R, int64_t C, void* out,
                   void* stream);
int mega_silu_mul_fwd(const void* a, const void* b, int dtype, int64_t n, void* out, void* stream);
int mega_silu_mul_bwd(const void* dout, const void* a, const void* b, int dtype, int64_t n,
                      void* da, void* db, void* stream);

/* ------------------------------------------------------------------------
 * LayerNorm / RMSNorm over the last axis, stored weight = gamma - 1.
 *
 * Replaces FusedLayerNorm / FusedRMSNorm (megalodon/modules/layer_norm.py:14-66:
 *   `weight + 1` handed to apex's fused_layer_norm_cuda, which is not in the
 *   reference tree; apex's definition is the usual one restated here).
 *   x, y (rows, D) of `dtype`; weight, bias (D) of the same dtype or null
 *   (no affine parameters); mean, rstd (rows) float32 are saved for the
 *   backward.  rms == 0: mean = E[x], var = E[(x - mean)^2],
 *   y = (x - mean) rstd (weight + 1) + bias.  rms != 0: rstd = 1/sqrt(E[x^2] + eps),
 *   y = x rstd (weight + 1); `bias` and `mean` are ignored.  float32 inside.
 *   16-bit rows of 128, 256, 512, 1024, 2048 or 4096 elements stay in
 *   registers (x read once); other shapes re-read the row from cache.
 * Backward: dx, and (when `dweight` is not null) dweight, dbias (null for rms
 *   or no bias) in `dtype`, summed over rows in a fixed order.
 *   `workspace`: mega_layer_norm_workspace_bytes(rows, D) bytes, needed when
 *   dweight is not null.
 * ---------------------------------------------------------------------- */
int64_t mega_layer_norm_workspace_bytes(int64_t rows, int64_t D);
int mega_layer_norm_fwd(const void* x, const void* weight, const void* bias, int dtype,
                        int64_t rows, int64_t D, double eps, int rms, void* y, float* mean,
                        float* rstd, void* stream);
int mega_layer_norm_bwd(const void* dy, const void* x, const void* weight, const float* mean,
                        const float* rstd, int dtype, int64_t rows, int64_t D, int rms, void* dx,
                        void* dweight, void* dbias, void* workspace, void* stream);

/* ------------------------------------------------------------------------
 * z -> (q, k): per-head RMSNorm, the two affine maps and the rotary product.
 *
 * Replaces, in one pass over z, megalodon/modules/moving_average_gated_attention.py:
 *   319-330 (`self.znorm(z.view(B, L, heads, Dh))`, `z.unsqueeze(2) * (gamma + 1)
 *   / sqrt(Dh) + beta`, `torch.unbind`) and the rotary product of
 *   megalodon/modules/rotary_positional_embedding.py:53-77 that
 *   _InnerAttention applies to q and k (moving_average_gated_attention.py:
 *   88-90,113-114).
 *   z, q, k (rows, S) of `dtype` (bfloat16 / float16), rows = batch * L; gamma,
 *   beta (2, S) of `dtype` as the module stores them; heads of Dh elements,
 *   Dh in {64, 128, 256, 512}, S in {512, 1024, 2048, 4096}.  `freqs`: (P, Dh/2)
 *   complex numbers as float32 pairs (cos, sin), or null for no rotary; row r
 *   uses position (r % L) % P (P = chunk length, or L for a shorter piece).
 *   rstd (rows, S / Dh) float32 is saved for the backward.  All buffers 16-byte
 *   aligned.  Other shapes return MEGA_ERR_UNSUPPORTED (the module then keeps
 *   the PyTorch expressions).
 * Backward: dz, dgamma (2, S), dbeta (2, S) in `dtype`;
 *   `workspace`: mega_qk_norm_rotary_workspace_bytes(S) bytes.
 * ---------------------------------------------------------------------- */
int64_t mega_qk_norm_rotary_workspace_bytes(int64_t S);
int mega_qk_norm_rotary_fwd(const void* z, const void* gamma, const void* beta, const float* freqs,
                            int dtype, int64_t rows, int64_t L, int64_t P, int64_t S, int64_t Dh,
                            double eps, void* q, void* k, float* rstd, void* stream);
int mega_qk_norm_rotary_bwd(const void* dq, const void* dk, const void* z, const void* gamma,
                            const float* rstd, const float* freqs, int dtype, int64_t rows,
                            int64_t L, int64_t P, int64_t S, int64_t Dh, void* dz, void* dgamma,
                            void* dbeta, void* workspace, void* stream);

/* ------------------------------------------------------------------------
 * Real FFT of zero-padded rows.
 *
 * Replaces rfft(x, flip) -> y (megalodon/csrc/ops/fftconv.cc:6-8,22,
 *   fftconv_kernel.cu:23-32,170-215; called for a 16-bit convolution kernel in
 *   fused_ops/fftconv.py:88-91).
 *   x (rows, L) of `dtype`, L <= 16384; y (rows, M + 1) complex64 as float32
 *   pairs, M = max(2^ceil(log2 L), 32) = mega_rfft_bins(L) - 1:
 *   y = rfft(x, n = 2 M), with x reversed in time first when `flip` is set.
 *   The convolution entry points above take k in the time domain and do not
 *   need this operator.
 * ---------------------------------------------------------------------- */
int64_t mega_rfft_bins(int64_t L);
int mega_rfft(const void* x, int dtype, int64_t rows, int64_t L, int flip, void* y, void* stream);

/* ------------------------------------------------------------------------
 * Whole-sequence (non-causal) group normalisation.
 *
 * Replaces group_sequence_norm_fwd(X, gamma, beta, padding_mask, num_groups,
 *   eps, length_last) -> (Y, count, mean, rstd) and group_sequence_norm_bwd(
 *   Y_grad, X, count, mean, rstd, gamma, padding_mask, num_groups,
 *   length_last) -> (X_grad, gamma_grad, beta_grad)
 *   (megalodon/csrc/ops/sequence_norm.cc:531-842,953-1063, binding :1068-1071),
 *   and with num_groups = H the per-feature pair sequence_norm_fwd/bwd
 *   (:258-529,844-951, binding :1066-1067).
 *   x, y, dy, dx: (B, L, H) when length_last = 0, (B, H, L) when 1, of
 *   `dtype`; gamma, beta, dgamma, dbeta (H) of `dtype`; padding_mask (B, L)
 *   bytes, nonzero = step left out (may be null); count (B) int64 = unmasked
 *   steps; mean, rstd (B, num_groups) float32 over the unmasked steps and the
 *   H / num_groups features of a group (biased variance);
 *   y = (x - mean) rstd gamma + beta, 0 at masked steps.
 *   workspace: mega_group_sequence_norm_workspace_bytes(...) bytes, contents
 *   not kept between calls.
 * ---------------------------------------------------------------------- */
int64_t mega_group_sequence_norm_workspace_bytes(int64_t B, int64_t L, int64_t H, int64_t num_groups,
                                                 int length_last);
int mega_group_sequence_norm_fwd(const void* x, const void* gamma, const void* beta,
                                 const uint8_t* padding_mask, int dtype, int64_t B, int64_t L,
                                 int64_t H, int64_t num_groups, double eps, int length_last, void* y,
                                 int64_t* count, float* mean, float* rstd, void* workspace,
                                 void* stream);
int mega_group_sequence_norm_bwd(const void* dy, const void* x, const int64_t* count,
                                 const float* mean, const float* rstd, const void* gamma,
                                 const uint8_t* padding_mask, int dtype, int64_t B, int64_t L,
                                 int64_t H, int64_t num_groups, int length_last, void* dx,
                                 void* dgamma, void* dbeta, void* workspace, void* stream);

/* ------------------------------------------------------------------------
 * The CEMA layer as a chunked recurrence (no kernel row, no spectra).
 *
 * Replaces, for one call of MultiHeadComplexEMA.forward
 *   (megalodon/modules/complex_exponential_moving_average.py:127-147), the chain
 *   k, b = ema_parameters(p, q, gamma, hx, L)      (fused_ops/ema_parameters.py:8-35,
 *                                                    csrc/ops/ema_parameters.cc:17-77)
 *   out  = fftconv(x, k) + x * omega (+ b)          (fused_ops/fftconv.py:9-50)
 *   h    = ema_hidden(x, p, q, hx)                  (csrc/ops/ema_hidden.cc:16-62)
 * which is the recurrence h[t] = q h[t-1] + p x[t], out[t] = Re sum_n gamma_n
 * h_n[t] + omega x[t] with h[-1] = hx.  The row is processed in chunks of 64
 * steps as matrix products on the matrix cores (bf16 operand pieces carrying
 * 16 significant bits, float32 states and accumulation); x is read once and
 * out written once.
 *   x, y (B, D, L) of `dtype` (MEGA_BF16, MEGA_F16 or MEGA_F32; float32 rows
 *   enter the products with their 16 leading bits, y is written in float32),
 *   16-byte aligned, any L % 8 == 0 (no upper limit); p (D, N) float32; log_q, gamma (D, N)
 *   complex64 as mega_ema_weight_fwd takes them, N <= 16; omega (D) float32 or
 *   null; h0 (B, D, N) complex64 or null (zero state); h_last (B, D, N)
 *   complex64 or null (not wanted).
 *   mega_cema_scan_supported(dtype, N, L) tells whether a shape is taken;
 *   others return MEGA_ERR_UNSUPPORTED (use the kernel-row path then).
 * ---------------------------------------------------------------------- */
int mega_cema_scan_supported(int dtype, int64_t N, int64_t L);
int mega_cema_scan_fwd(const void* x, int dtype, const float* p, const float* log_q,
                       const float* gamma, const float* omega, const float* h0, int64_t B,
                       int64_t D, int64_t N, int64_t L, void* y, float* h_last, void* stream);

/* Backward of mega_cema_scan_fwd without a carried state (the training path):
 * replaces the chain fftconv_bwd -> (dx, dk), ema_parameters_bwd(dk, ...) ->
 * (dp, dq, dgamma) and the two elementwise passes of the skip term
 *   (fused_ops/fftconv.py:53-75, csrc/ops/ema_parameters.cc:80-98,141-156);
 * dk is never formed.  dy, x, dx (B, D, L) bfloat16, 16-byte aligned,
 * L % 8 == 0; the parameter gradients come PER ROW, (B, D, N) -- dp float32,
 * dq and dgamma complex64 in PyTorch's conjugate convention, as
 * mega_ema_weight_bwd returns them -- and domega (B, D) float32; the caller
 * sums over B.  mega_cema_scan_bwd_supported(dtype, N, L) tells whether a
 * shape is taken. */
int mega_cema_scan_bwd_supported(int dtype, int64_t N, int64_t L);
int mega_cema_scan_bwd(const void* dy, const void* x, int dtype, const float* p,
                       const float* log_q, const float* gamma, const float* omega, int64_t B,
                       int64_t D, int64_t N, int64_t L, void* dx, float* dp, float* dq,
                       float* dgamma, float* domega, void* stream);

/* The same backward for a forward that had a carried state h0 (B, D, N)
 * complex64: the state adds b[t] = Re sum_n gamma_n q_n^(t+1) h0_n to the output
 * (csrc/ops/ema_parameters.cc:56-77), and its backward
 * (ema_parameters.cc:100-117,158-188) adds conj(q h0 R0) to dgamma and
 * conj(gamma h0 (R0 + q R0')) to dq, with R0 = sum_t dy[t] q^t, R0' = dR0/dq --
 * what the kernel's reverse scan has carried to the start of the row -- and
 * returns dh0 = conj(gamma q R0), (B, D, N) complex64 (NULL: not wanted).
 * h0 == NULL is mega_cema_scan_bwd.  The gradient of a last state taken from
 * the forward is a separate operator (ema_hidden_bwd, csrc/ops/ema_hidden.cc:63-159). */
int mega_cema_scan_bwd_state(const void* dy, const void* x, int dtype, const float* p,
                             const float* log_q, const float* gamma, const float* omega,
                             const float* h0, int64_t B, int64_t D, int64_t N, int64_t L, void* dx,
                             float* dp, float* dq, float* dgamma, float* domega, float* dh0,
                             void* stream);

/* mega_cema_scan_bwd on bfloat16 dy and x with dx written in float32, or not at
 * all when `dx` is NULL; with `accumulate_dx` the launch adds to what dx holds.  The backward is linear in dy and, for the parameter
 * gradients, in x: a caller with float16 or float32 tensors (the reference's
 * operators take them, fused_ops/fftconv.py:37-44 upcasts to float32) runs
 * this on the bfloat16 pieces of dy and x and adds the results up
 * (extension.py:cema_scan_bwd does); h0 / dh0 as in mega_cema_scan_bwd_state, to be
 * passed with the pieces of dy and the leading piece of x only (the state's terms
 * do not depend on x). */
int mega_cema_scan_bwd_wide(const void* dy, const void* x, const float* p, const float* log_q,
                            const float* gamma, const float* omega, const float* h0, int64_t B,
                            int64_t D, int64_t N, int64_t L, float* dx, int accumulate_dx, float* dp,
                            float* dq, float* dgamma, float* domega, float* dh0, void* stream);

/* src (n elements, MEGA_F32 or MEGA_F16, n % 8 == 0, 16-byte aligned) as the sum of two
 * bfloat16 tensors: hi = bf16(src), lo = bf16(src - hi) -- 16 significant bits of a float32
 * value, every bit of a float16 one.  The pieces mega_cema_scan_bwd_wide runs on. */
int mega_split_bf16(const void* src, int dtype, int64_t n, void* hi, void* lo, void* stream);

/* ------------------------------------------------------------------------
 * Streaming reference kernel for measurements (no counterpart in the
 * reference): out = a (b == NULL) or out = a XOR b over `bytes` bytes
 * (multiple of 16, operands 16-byte aligned), grid-stride with `workgroups`
 * workgroups of 256 lanes, 16-byte accesses, eight loads per lane in flight,
 * with nontemporal accesses if `nontemporal` is non-zero.
 * Its rate is the practical ceiling the HBM-bound operators are compared with
 * next to the published peak.
 * ---------------------------------------------------------------------- */
int mega_bench_stream_copy(const void* a, const void* b, void* out, int64_t bytes,
                           int workgroups, int nontemporal, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* MEGALODON_HIP_H_ */
