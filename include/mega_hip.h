/* mega_hip.h -- C ABI of libmega_hip.so: the Mega/Mega2 sequence-mixing hot path
 * (EMA kernel generation, long causal / bidirectional convolution, TimestepNorm,
 * chunked attention softmax, SwiGLU gate) as hand-written HIP kernels for gfx950.
 *
 * Conventions (every entry point):
 *  - plain pointers and sizes only; every data pointer is DEVICE memory of the
 *    current HIP device unless the comment says "host";
 *  - outputs are caller-allocated, inputs are never written;
 *  - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *    default stream) and the call returns without synchronising;
 *  - the library never allocates device memory: scratch comes in through
 *    `workspace` (size from the matching *_workspace_bytes query).  A workspace
 *    that is handed to mega_*_timestep_norm_fwd must be zero-filled once when it
 *    is created and then belongs to these calls (they keep a launch epoch in
 *    it), so it can be reused by later calls on the same stream.  Calls that
 *    share one workspace must not overlap in time;
 *  - return value 0 = launched; a negative value = rejected before anything was
 *    launched (MEGA_ERR_*), with a human-readable reason in mega_last_error()
 *    (thread-local).  This mirrors the TORCH_CHECK -> RuntimeError behaviour of
 *    the reference ops; the Python host raises RuntimeError from it.
 *
 * The reference has no C ABI: its boundary is C++ functions over torch::Tensor
 * exported by pybind11 as fairseq.mega2_extension.ops
 * (fairseq/csrc/mega2_extension.cc:14-24).  Each entry point below cites the
 * reference function it stands in for.
 */
#ifndef MEGA_HIP_H_
#define MEGA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of activations */
enum { MEGA_F32 = 0, MEGA_BF16 = 1, MEGA_F16 = 2 };

/* error codes */
enum {
  MEGA_OK = 0,
  MEGA_ERR_ARG = -1,       /* bad shape / pointer / flag                     */
  MEGA_ERR_UNSUPPORTED = -2, /* valid request outside the implemented envelope */
  MEGA_ERR_WORKSPACE = -3, /* workspace missing or too small                 */
  MEGA_ERR_LAUNCH = -4     /* hipLaunchKernel reported an error, or an earlier launch gave up a bounded wait */
};

/* reason for the last negative return on this thread (never NULL) */
const char* mega_last_error(void);

/* library version, bumped when a signature or a contract changes.
 *   3: mega_norm_ema_step / mega_norm_ema_steps reject count == prev_count and mega_group_timestep_norm_fwd /
 *      mega_norm_ema_fwd reject outputs that overlap the prior statistics (version 2 allowed the outputs to alias the
 *      inputs); MEGA_ERR_LAUNCH may also report an earlier launch's give-up (below); mega_timestep_norm_fwd returns
 *      MEGA_ERR_WORKSPACE for rows of more than 128 tokens without a workspace (version 2 ran a serial kernel);
 *      mega_group_timestep_norm_fwd_noalloc requires mega_lookback_init(); the workspace of mega_norm_ema_fwd holds
 *      one more record per (row, group)                                                                      */
int mega_abi_version(void);

/* Bounded waits between workgroups.  The group TimestepNorm kernel and the one-kernel TimestepNorm -> moving
 * average block let a time tile wait for the words of the earlier tiles of its row; they count on the
 * hardware starting workgroups in id order, and the wait is bounded.  A tile that gives up writes NaN into
 * every output and statistic that depended on the missing words (count becomes -1), sets the error word of
 * its workspace and a host-mapped status word of its device.  The entry points that launch these kernels
 * (mega_group_timestep_norm_fwd, mega_norm_ema_fwd) look at that word before anything else: if it is set they
 * clear it and return MEGA_ERR_LAUNCH without launching, so a give-up surfaces on the next call the way a
 * sticky launch error does (C10_CUDA_KERNEL_LAUNCH_CHECK(), fairseq/csrc/ops/timestep_norm_kernel.cu:641).
 * mega_lookback_status reads the word of the current device without synchronising (a launch still running
 * may set it later; after a synchronisation it is final); clear != 0 resets it.
 * The word is pinned, device-mapped host memory, created per device by the first regular call that needs it or by
 * mega_lookback_init (MEGA_OK, or MEGA_ERR_LAUNCH when the runtime refuses the allocation).  Callers that must not
 * allocate inside a region (HIP graph capture) call mega_lookback_init once per device before it;
 * mega_group_timestep_norm_fwd_noalloc, which may not create the word itself, returns MEGA_ERR_UNSUPPORTED until
 * it exists (no counterpart in the reference).                                                        */
int mega_lookback_init(void);
int mega_lookback_status(int clear);
/* Checked mode, off by default (on: mega_lookback_checked(1), or MEGA_LOOKBACK_CHECKED=1 in the environment when the
 * library is first asked): mega_group_timestep_norm_fwd and mega_norm_ema_fwd(_train) wait for their stream after
 * the launch and return MEGA_ERR_LAUNCH for a give-up of that very call instead of leaving it to the next one.  For
 * debugging and for callers that prefer a synchronous error to throughput; not usable under stream capture.   */
void mega_lookback_checked(int on);

/* Test hook for the failure path, so that it can be exercised with every kernel exiting normally:
 * spin_limit = polls before a wait gives up (0 = the default, 2^22); withhold_first != 0 makes the first
 * tile of every row publish nothing, so the later tiles of the row run into the limit; raise != 0 sets the
 * status word of the current device from the host.  Not for production use.                         */
void mega_test_lookback(unsigned spin_limit, int withhold_first, int raise);

/* Test hook: on == 0 keeps mega_(group_)timestep_norm_bwd on its three-pass form (tile maps, carry, dx) also where
 * the one-launch form with its look-back over the later tiles would run (16-bit activations in 16-byte vectors, at
 * most 16 groups); on != 0 (the default) restores the choice.  For tests that compare the two forms; no counterpart
 * in the reference.                                                                                   */
void mega_test_timestep_norm_bwd_onepass(int on);

/* Address audit (host only, nothing is launched, no GPU needed; no counterpart in the reference).  Between
 * mega_audit_begin() and mega_audit_end() the calling thread's calls to mega_attention_bwd, mega_gate_qk_bwd,
 * mega_ema_param_grad and mega_(group_)timestep_norm_bwd launch nothing: for every launch they would make they
 * compute, from the sizes and strides the kernel would get, the last byte every operand is addressed at and check
 * that it lies inside one of the byte ranges registered with mega_audit_add (the tensors and the workspace of the
 * call, at any made-up addresses that satisfy the alignment rules).  mega_audit_end returns the number of
 * violations (the first one in mega_last_error()) and, through `checks`, how many ranges were checked.    */
void mega_audit_begin(void);
int mega_audit_add(const void* base, size_t bytes);
int mega_audit_end(int* checks);

/* ------------------------------------------------------------------------ */
/* EMA coefficients -> convolution kernel and carried-state bias            */
/* stands in for ema_parameters_fwd (fairseq/csrc/ops/ema_parameters.cc:211-286,
 * CUDA side ops/ema_parameters_kernel.cu:446-525; Python caller
 * fairseq/modules/fused_ops/ema_parameters.py:13-20).
 *   p      [K,N]      real
 *   log_q  [K,N,2]    complex (re,im) -- principal log of q, as the reference passes it
 *   gamma  [K,N,2]    complex
 *   h      [B,K,N,2]  complex carried state, or NULL
 *   w      [K,L]      out: w[d,l] = Re sum_n p gamma exp(l log q)
 *   b      [B,K,L]    out (only if h != NULL): Re sum_n gamma h exp((l+1) log q)
 * N <= 32 (the limit of the reference, ema_parameters_kernel.cu:455).            */
int mega_ema_parameters_fwd(const float* p, const float* log_q, const float* gamma,
                            const float* h, int64_t B, int64_t K, int64_t N, int64_t L,
                            float* w, float* b, void* stream);

/* ------------------------------------------------------------------------ */
/* EMA hidden state after a chunk                                            */
/* stands in for ema_hidden_fwd (fairseq/csrc/ops/ema_hidden.cc:163-194, CUDA
 * side ops/ema_hidden_kernel.cu:472-536; caller fused_ops/ema_hidden.py:13-17).
 *   x      [B,D,L] activations of type `dtype`, element strides (sxb,sxd,sxl)
 *   p      [D,N]; log_q [D,N,2]; h [B,D,N,2] or NULL
 *   h_out  [B,D,N,2]: p sum_j q^{L-1-j} x_j + q^L h                              */
size_t mega_ema_hidden_workspace_bytes(int64_t B, int64_t D, int64_t N, int64_t L);
int mega_ema_hidden_fwd(const void* x, int dtype, int64_t sxb, int64_t sxd, int64_t sxl,
                        const float* p, const float* log_q, const float* h, int64_t B,
                        int64_t D, int64_t N, int64_t L, float* h_out, void* workspace,
                        size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Fused moving-average layer forward                                        */
/* stands in for BaseMovingLayer.forward as a whole
 * (fairseq/modules/base_moving_average.py:120-172): mask, kernel generation
 * (ema_parameters), long convolution (fftconv / bidirectional_fftconv,
 * fairseq/modules/fused_ops/fftconv.py:11-27, 85-100), carried-state bias,
 * ema_hidden and the omega residual in one pass over x.  The D x L kernel is
 * never materialised.
 *   x, y    [B,D,L] of `dtype` with element strides (sxb,sxd,sxl) / (syb,syd,syl);
 *           x and y may each use either contiguous layout, [B,D,L] or [B,L,D], independently
 *           (the reference's convolution returns [B,D,L] rows for a transposed [B,L,D] input)
 *   p       [K,N] real, q [K,N,2] complex (q itself, not its log), gamma [K,N,2]
 *           complex already scaled by sqrt(1/N); K = D, or 2D when bidirectional
 *   is_complex   0: imaginary parts are ignored / assumed zero (real EMA)
 *   omega   [D]
 *   mask    [B,L] bytes, non-zero = padding, or NULL
 *   h_in    [B,D,N,2] carried state or NULL; h_out [B,D,N,2] or NULL
 *           (both must be NULL when bidirectional)
 *   truncation  <= 0: kernel length L; otherwise min(truncation, L)
 *   shift   bidirectional only: 1 = the backward half starts at lag 1
 *   image   operand images from mega_ema_prepare for the same coefficients, or NULL: then
 *           kernel generation runs inside this call (into the workspace)
 * All three activation types run on the matrix cores for ndim <= 16 without truncation, as the
 * reference's convolution serves them alike (ops/fftconv_kernel.cu:214-269): bf16 in either
 * layout; fp32 / fp16 on [B,D,L] rows (sxl = syl = 1) of up to 16384 tokens, where fp32 values
 * and operands travel as two fp16 terms (error ~ 2^-22 of the largest term, accumulation in
 * fp32).  Other cases take the chunked scan on the vector ALUs.                            */
size_t mega_ema_fwd_workspace_bytes(int64_t B, int64_t D, int64_t N, int64_t L,
                                    int bidirectional, int64_t truncation);
int mega_ema_fwd(const void* x, void* y, int dtype, int64_t sxb, int64_t sxd, int64_t sxl,
                 int64_t syb, int64_t syd, int64_t syl, const float* p, const float* q,
                 const float* gamma, int is_complex, const float* omega,
                 const uint8_t* mask, const float* h_in, float* h_out, int64_t B,
                 int64_t D, int64_t N, int64_t L, int bidirectional, int64_t truncation,
                 int shift, const void* image, void* workspace, size_t workspace_bytes,
                 void* stream);

/* EMA kernel generation for the matrix-core path: from the coefficients to per-channel
 * operand images (the 32-tap Toeplitz block of k[l] = Re sum_n p gamma q^l, the state
 * input / output blocks p q^{31-i} and gamma q^{i+1} as bf16 and as fp16 terms, and the
 * powers of q that join tiles, segments and blocks), 36 KB per coefficient row whatever L is.  Stands in for what the reference recomputes or caches per call:
 * _compute_kernel / ema_parameters (fairseq/modules/complex_exponential_moving_average.py:
 * 98-109, fairseq/csrc/ops/ema_parameters_kernel.cu:40-66) and the eval-mode `_coeffs`
 * cache (fairseq/modules/base_moving_average.py:52-58).  The image is valid while p, q,
 * gamma, omega, bidirectional and shift are unchanged; it only exists for ndim <= 16
 * (mega_ema_image_bytes returns 0 otherwise).                                            */
size_t mega_ema_image_bytes(int64_t D, int64_t N, int bidirectional);
int mega_ema_prepare(const float* p, const float* q, const float* gamma, int is_complex,
                     const float* omega, int64_t D, int64_t N, int bidirectional, int shift,
                     void* image, size_t image_bytes, void* stream);

/* One decode step of the same layer: h' = q h + p x, y = Re sum gamma h' + omega x
 * (BaseMovingLayer.one_step, fairseq/modules/base_moving_average.py:105-118, and the
 * L = 1 case of forward with incremental_state).
 *   x, y [B,D] of `dtype` (contiguous); h_in may be NULL (zero state); h_out [B,D,N,2];
 *   h_out may alias h_in.                                                         */
int mega_ema_step(const void* x, void* y, int dtype, const float* p, const float* q,
                  const float* gamma, int is_complex, const float* omega, const float* h_in,
                  float* h_out, int64_t B, int64_t D, int64_t N, void* stream);

/* One decode step of the norm -> moving-average pair in one launch: streaming group
 * TimestepNorm of a single token (TimestepNorm.forward with L = 1 and incremental state,
 * fairseq/modules/norm_layer/timestep_norm.py:100-139) followed by mega_ema_step on the
 * normalised token (BaseMovingLayer.forward with L = 1 and incremental state,
 * fairseq/modules/base_moving_average.py:144-160).  The reference runs these as two modules
 * and >= 6 kernels per step.
 *   x, xn, y [B,D] of `dtype`; norm state in (prev_*) and out (count, mean, var);
 *   norm_gamma (= weight + 1), norm_beta [D]; EMA coefficients as mega_ema_step;
 *   h_in may be NULL (zero state).
 *   In-place update: mean / var may be the prev_mean / prev_var buffers and h_out may be h_in
 *   (one workgroup owns each of those words: it reads, then writes).  count must NOT overlap
 *   prev_count (MEGA_ERR_ARG): all G workgroups of a stream read prev_count[b] while one of
 *   them writes count[b]; a streaming caller alternates between two count buffers.         */
int mega_norm_ema_step(const void* x, void* xn, void* y, int dtype, const int64_t* prev_count,
                       const float* prev_mean, const float* prev_var, int64_t* count,
                       float* mean, float* var, const float* norm_gamma, const float* norm_beta,
                       double eps, const float* p, const float* q, const float* gamma,
                       int is_complex, const float* omega, const float* h_in, float* h_out,
                       int64_t B, int64_t D, int64_t G, int64_t N, void* stream);

/* K consecutive tokens of every stream in one launch: the same result as K calls of
 * mega_norm_ema_step on x[:, k] (the reference's chunk-wise streaming, fairseq_cli/train.py:406-417,
 * with chunks of K tokens through TimestepNorm.forward and BaseMovingLayer.forward with incremental
 * state, timestep_norm.py:100-139 and base_moving_average.py:144-160), but the state h is read and
 * written once per launch, not once per token, and the host enqueues one kernel instead of K.
 *   x, xn, y [B,K,D] of `dtype` (contiguous); everything else as mega_norm_ema_step, the same
 *   in-place rules (count must not overlap prev_count; count advances by K).
 *   Covered: complex coefficient storage (is_complex != 0), ndim in {4, 8, 16, 32}, 16-byte aligned
 *   p, q, gamma, h; MEGA_ERR_UNSUPPORTED otherwise (call mega_norm_ema_step per token).        */
int mega_norm_ema_steps(const void* x, void* xn, void* y, int dtype, int64_t K,
                        const int64_t* prev_count, const float* prev_mean, const float* prev_var,
                        int64_t* count, float* mean, float* var, const float* norm_gamma,
                        const float* norm_beta, double eps, const float* p, const float* q,
                        const float* gamma, int is_complex, const float* omega, const float* h_in,
                        float* h_out, int64_t B, int64_t D, int64_t G, int64_t N, void* stream);

/* TimestepNorm followed by the moving-average layer in one call: what
 * MovingAverageGatedAttention.forward does with x at
 * fairseq/modules/moving_average_gated_attention.py:304-315 (x = norm(x), then
 * mx = move(x^T)), i.e. mega_group_timestep_norm_fwd (x -> xn, [B,L,D]) followed by
 * mega_ema_fwd on the transposed view of xn (-> y).  xn is an output too: the layer also
 * feeds it to v_proj.
 *   x, xn      [B,L,D] contiguous of `dtype`; y of `dtype` with element strides
 *              (syb, syd, syl) over (batch, channel, time): [B,D,L] rows, which is what the
 *              reference's convolution returns, or [B,L,D]
 *   norm state / parameters / mask as mega_group_timestep_norm_fwd (norm_gamma = weight + 1);
 *   moving-average coefficients, h_in / h_out and `image` as mega_ema_fwd (unidirectional,
 *   no truncation); h_out must not overlap h_in.
 * bf16 activations with 64 or 128 channels per norm group (D = 64 G or 128 G), ndim <= 16, with or
 * without a mask, ceil(L / 1024) (+ 1 with h_in) <= 16 run as ONE kernel that reads x once and writes xn
 * and y once.  L need not be a multiple of 1024 (the blocks are aligned to the end of the row, so h_out is
 * the state after the last token), but such a row takes no h_in, and [B,D,L] rows then need L % 8 == 0.
 * Everything else runs the two operators one after the other.
 * `workspace` (launch epoch, block / tile records) must be zero-filled once and then belongs to
 * these calls, exactly like the TimestepNorm workspace (the two may be the same buffer);
 * `scratch` needs no initialisation and is used only when the two operators run one after the
 * other or when image == NULL (kernel generation inside the call).                          */
size_t mega_norm_ema_fwd_workspace_bytes(int64_t B, int64_t L, int64_t D, int64_t G, int64_t N);
size_t mega_norm_ema_fwd_scratch_bytes(int64_t B, int64_t L, int64_t D, int64_t G, int64_t N);
int mega_norm_ema_fwd(const void* x, void* xn, void* y, int dtype, int64_t syb, int64_t syd,
                      int64_t syl, const int64_t* prev_count, const float* prev_mean,
                      const float* prev_var, const float* norm_gamma, const float* norm_beta,
                      const uint8_t* mask, double eps, int64_t* count, float* mean, float* var,
                      const float* p, const float* q, const float* gamma, int is_complex,
                      const float* omega, const float* h_in, float* h_out, int64_t B, int64_t L,
                      int64_t D, int64_t G, int64_t N, const void* image, void* workspace,
                      size_t workspace_bytes, void* scratch, size_t scratch_bytes, void* stream);
/* The same call for a training forward: additionally writes cummean, cumrstd [B,L,G] fp32, the
 * running statistics of every token that group_timestep_norm_fwd hands to its backward pass
 * (fairseq/modules/norm_layer/timestep_norm.py:35-43; at a padded token the carried statistics), so
 * that mega_group_timestep_norm_bwd (group_mean = NULL) and the moving-average backward can follow
 * a forward that ran as one kernel.  Both pointers NULL: exactly mega_norm_ema_fwd.            */
int mega_norm_ema_fwd_train(const void* x, void* xn, void* y, int dtype, int64_t syb, int64_t syd,
                            int64_t syl, const int64_t* prev_count, const float* prev_mean,
                            const float* prev_var, const float* norm_gamma, const float* norm_beta,
                            const uint8_t* mask, double eps, int64_t* count, float* mean, float* var,
                            float* cummean, float* cumrstd, const float* p, const float* q,
                            const float* gamma, int is_complex, const float* omega,
                            const float* h_in, float* h_out, int64_t B, int64_t L, int64_t D,
                            int64_t G, int64_t N, const void* image, void* workspace,
                            size_t workspace_bytes, void* scratch, size_t scratch_bytes,
                            void* stream);

/* ------------------------------------------------------------------------ */
/* Moving-average backward (unidirectional, no carried state)                  */
/* The input gradient is the same layer run backwards in time: call mega_ema_fwd with
 * x = y_grad, pointers at the last token and negated token strides (the kernel is
 * k[l] for l >= 0, so dx[t] = sum_{s>=t} k[s-t] dy[s] + omega dy[t]).
 * mega_ema_param_grad stands in for the kernel-gradient half of fftconv_bwd
 * (fairseq/modules/fused_ops/fftconv.py:66-88) followed by ema_parameters_bwd
 * (fairseq/csrc/ops/ema_parameters.cc:80-97) for a layer without carried state, without
 * forming dk:
 *   S2[d,n] = sum_{b,t} dy[t] s[t],  S1[d,n] = sum_{b,t} dy[t] g[t],
 *   s[t] = q s[t-1] + x[t] (masked x enters as 0), g[t] = q g[t-1] + s[t-1];
 *   dp = Re(S2 gamma), dq = conj(S1 p gamma), dgamma = conj(S2 p) (ema_parameters.cc:95-96),
 *   domega[d] = sum_{b,t} dy[t] x[t].
 *   dy, x [B,D,L] of `dtype` with element strides; p [D,N], q, gamma [D,N,2] fp32 (imaginary
 *   parts 0 for the real layer); mask [B,L] or NULL; outputs dp [D,N], dq, dgamma [D,N,2],
 *   domega [D] fp32; N <= 16 per call (the sums of one state do not involve the others: a layer
 *   with more states passes slices of 16 columns of p, q, gamma); workspace of
 *   mega_ema_param_grad_workspace_bytes(B, D, N).
 *   A two-sided layer takes two calls: its first D coefficient rows as above; its second D rows
 *   with reverse_time = 1 (the tokens are walked from the last to the first) and lag_one = shift
 *   (dy[t] is paired with the state before token t: kernel lags start at 1).               */
size_t mega_ema_param_grad_workspace_bytes(int64_t B, int64_t D, int64_t N);
int mega_ema_param_grad(const void* dy, const void* x, int dtype, int64_t sgb, int64_t sgd,
                        int64_t sgl, int64_t sxb, int64_t sxd, int64_t sxl, const float* p,
                        const float* q, const float* gamma, const uint8_t* mask, int64_t B,
                        int64_t D, int64_t N, int64_t L, int reverse_time, int lag_one, float* dp,
                        float* dq, float* dgamma, float* domega, void* workspace,
                        size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Parameter formulas in front of the kernels, one launch each way                            */
/* mega_ema_coeffs_fwd / _bwd: the coefficients of the moving average from the stored parameters, in the
 * reference a chain of torch operations per call (complex layer:
 * fairseq/modules/complex_exponential_moving_average.py:79-96, p = sigmoid(alpha),
 * q = (1 - sigmoid(alpha) sigmoid(delta)) exp(i (n + 1) sigmoid(theta) 2 pi / N), gamma complex times sqrt(1 / N);
 * real layer: exponential_moving_average.py:71-80, p = sigmoid(alpha) beta, q = 1 - sigmoid(alpha) sigmoid(delta),
 * gamma times sqrt(1 / N)).  alpha, delta [K, N]; theta [K] (complex) or beta [K, N] (real); gamma [K, N, 2]
 * (complex) or [K, N] (real); omega [D]; all of `dtype` (the parameters' storage type), K = D or 2 D.
 * Results in the layout every other entry point takes: p [K, N], q, gamma_out [K, N, 2], omega_out [D], fp32.
 * The backward takes the gradients of those four (fp32; for the complex layer q_grad, gamma_out_grad [K, N, 2] as
 * (d/dRe, d/dIm) pairs, which is torch's convention for a real loss; for the real layer [K, N]) and writes the
 * parameters' gradients in `dtype`.                                                                       */
int mega_ema_coeffs_fwd(const void* alpha, const void* delta, const void* theta_or_beta,
                        const void* gamma, const void* omega, int dtype, int is_complex, int64_t K,
                        int64_t N, int64_t D, float* p, float* q, float* gamma_out, float* omega_out,
                        void* stream);
int mega_ema_coeffs_bwd(const float* p_grad, const float* q_grad, const float* gamma_out_grad,
                        const float* omega_out_grad, const void* alpha, const void* delta,
                        const void* theta_or_beta, int dtype, int is_complex, int64_t K, int64_t N,
                        int64_t D, void* alpha_grad, void* delta_grad, void* theta_or_beta_grad,
                        void* gamma_grad, void* omega_grad, void* stream);
/* mega_norm_params_fwd / _bwd: the operands TimestepNorm.forward derives from its parameters on every call
 * (fairseq/modules/norm_layer/timestep_norm.py:118-131): gamma = weight + 1, beta = bias [H] fp32, and the
 * prior expanded over the batch, prev_mean = prior_mean, prev_var = exp(prior_logv) [B, G] fp32.  weight, bias
 * of `dtype`, prior_mean, prior_logv [G] of `prior_dtype`.  The backward writes the four parameter gradients in
 * their storage types (the prior's are sums over the batch; both NULL when the prior is a buffer).       */
int mega_norm_params_fwd(const void* weight, const void* bias, int dtype, const void* prior_mean,
                         const void* prior_logv, int prior_dtype, int64_t H, int64_t G, int64_t B,
                         float* gamma, float* beta, float* prev_mean, float* prev_var, void* stream);
int mega_norm_params_bwd(const float* gamma_grad, const float* beta_grad, const float* prev_mean_grad,
                         const float* prev_var_grad, const void* prior_logv, int dtype,
                         int prior_dtype, int64_t H, int64_t G, int64_t B, void* weight_grad,
                         void* bias_grad, void* prior_mean_grad, void* prior_logv_grad, void* stream);

/* ------------------------------------------------------------------------ */
/* Long convolution with an explicit time-domain kernel                      */
/* stands in for fftconv(x, k) (fairseq/modules/fused_ops/fftconv.py:11-27, 45-61;
 * fused CUDA op fftconv_fwd, ops/fftconv_kernel.cu:431-470) and
 * bidirectional_fftconv (fused_ops/fftconv.py:85-100).
 *   x, y [B,D,L] contiguous of `dtype`; k [K,Lk] fp32, K = D (causal) or 2D
 *   (bidirectional), Lk <= L.  Kernels of 512 lags and more with L + Lk <= 16384
 *   go through a Fourier transform held in LDS (fp32, two batch rows per complex
 *   transform, as fftconv_kernel.cu does with registers and shared memory); shorter
 *   kernels and longer rows take the direct sum.                                  */
int mega_long_conv_fwd(const void* x, void* y, int dtype, const float* k, int64_t B,
                       int64_t D, int64_t L, int64_t Lk, int bidirectional, int shift,
                       void* stream);

/* ------------------------------------------------------------------------ */
/* TimestepNorm                                                               */
/* group variant: stands in for group_timestep_norm_fwd
 * (fairseq/csrc/ops/timestep_norm.cc:568-636, CUDA side
 * ops/timestep_norm_kernel.cu:712-784; caller norm_layer/timestep_norm.py:35).
 *   x, y         [B,L,H] contiguous of `dtype`
 *   prev_count   [B] int64; prev_mean, prev_var [B,G] fp32
 *   gamma, beta  [H] fp32 (gamma is weight + 1, as the module passes it)
 *   mask         [B,L] bytes, non-zero = padding, or NULL
 *   count [B] int64, mean, var [B,G] fp32: state after the last token; they must not overlap
 *   prev_count / prev_mean / prev_var (MEGA_ERR_ARG): every time tile of a row reads the prior
 *   state while the row's last tile writes the new one (per-feature variant: count must not
 *   overlap prev_count; mean / var may be updated in place there)
 *   group_mean, cummean, cumrstd: [B,L,G] fp32 each, or NULL to skip (they exist for
 *   the backward pass only)
 * per-feature variant (G == H): stands in for timestep_norm_fwd
 * (timestep_norm.cc:452-510; timestep_norm_kernel.cu:602-654); here prev_mean,
 * prev_var, mean, var, cummean, cumrstd have H in place of G and group_mean is unused.  Rows of more
 * than 128 tokens need the workspace (mega_timestep_norm_workspace_bytes with G = H); without it the
 * call returns MEGA_ERR_WORKSPACE (shorter rows run a one-thread-per-feature kernel and need none). */
size_t mega_timestep_norm_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G);
int mega_group_timestep_norm_fwd(const void* x, void* y, int dtype, const int64_t* prev_count,
                                 const float* prev_mean, const float* prev_var,
                                 const float* gamma, const float* beta, const uint8_t* mask,
                                 int64_t B, int64_t L, int64_t H, int64_t G, double eps,
                                 int64_t* count, float* mean, float* var, float* group_mean,
                                 float* cummean, float* cumrstd, void* workspace,
                                 size_t workspace_bytes, void* stream);
int mega_timestep_norm_fwd(const void* x, void* y, int dtype, const int64_t* prev_count,
                           const float* prev_mean, const float* prev_var, const float* gamma,
                           const float* beta, const uint8_t* mask, int64_t B, int64_t L,
                           int64_t H, double eps, int64_t* count, float* mean, float* var,
                           float* cummean, float* cumrstd, void* workspace,
                           size_t workspace_bytes, void* stream);

/* mega_group_timestep_norm_fwd without the workspace arguments.  No counterpart in the
 * reference: it exists for callers that cannot allocate device memory or hand one over --
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The
 * launch epoch, retire counters and tile records live in a 1 MiB device array inside the
 * library (each GPU the library runs on holds its own copy until the process ends); the call
 * itself allocates and frees nothing.  Same arguments, results and errors as
 * mega_group_timestep_norm_fwd, plus:
 *   - MEGA_ERR_UNSUPPORTED until mega_lookback_init() has created the device's status word (the word
 *     a failed wait is reported through; creating it allocates pinned host memory, which this entry
 *     point must not do);
 *   - MEGA_ERR_UNSUPPORTED when the tile records do not fit:
 *     256 + B * (T + ceil(T / 32)) * (2 G + 1) * 8 bytes <= 1 MiB with T = ceil(L / TT) tiles,
 *     TT = tokens per tile (<= 64; one more record per 32 tiles holds their aggregate;
 *     mega_timestep_norm_workspace_bytes returns the exact figure for a shape);
 *   - the first call on a device looks the array's address up (hipGetSymbolAddress): make
 *     that call outside stream capture;
 *   - all calls on one GPU share the array and it keeps the previous call's contents (the
 *     records carry launch tags, so nothing needs clearing, also when the shape changes):
 *     calls that can overlap in time on one GPU -- two streams, two host threads -- race.   */
int mega_group_timestep_norm_fwd_noalloc(const void* x, void* y, int dtype,
                                         const int64_t* prev_count, const float* prev_mean,
                                         const float* prev_var, const float* gamma,
                                         const float* beta, const uint8_t* mask, int64_t B,
                                         int64_t L, int64_t H, int64_t G, double eps,
                                         int64_t* count, float* mean, float* var,
                                         float* group_mean, float* cummean, float* cumrstd,
                                         void* stream);

/* backward: stands in for group_timestep_norm_bwd and timestep_norm_bwd
 * (fairseq/csrc/ops/timestep_norm.cc:318-450 and :104-217, CUDA side
 * ops/timestep_norm_kernel.cu; caller norm_layer/timestep_norm.py:45-66).
 *   y_grad, x, x_grad [B,L,H] contiguous of `dtype`; mean_grad, var_grad [B,G] fp32 or NULL
 *   (zeros); prev_mean [B,G]; count [B] = the forward's count output; group_mean (NULL:
 *   recomputed from x), cummean, cumrstd [B,L,G] fp32 as the forward wrote them (at a masked
 *   token cummean must hold the carried mean, which is what this library's forward stores);
 *   gamma [H] fp32 (weight + 1).  Outputs: x_grad, prev_mean_grad, prev_var_grad [B,G],
 *   gamma_grad, beta_grad [H] fp32.  The per-feature form has H in place of G.
 *   bf16 / fp16 activations whose groups are whole 16-byte vectors (one vector per lane), with at
 *   most 16 groups, run as ONE launch that reads y_grad and x once: every tile of 32 (or 16)
 *   tokens publishes its map of the carried pair (u_grad, v_grad) and composes the maps of the
 *   tiles behind it with bounded waits, like the forward's look-back.  A wait that gives up leaves
 *   NaN in x_grad / prev_mean_grad / prev_var_grad and is reported like the forward's: the next
 *   call returns MEGA_ERR_LAUNCH (mega_lookback_status, checked mode: the same call).  Everything
 *   else takes three passes (tile maps, carry, x_grad) without waits; the per-feature form with an even
 *   number of channels runs them with the channels across the lanes (a thread walks its tile's tokens).  The workspace needs no
 *   initialisation and nothing in it survives the call (the records are cleared by the call). */
size_t mega_timestep_norm_bwd_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G);
int mega_group_timestep_norm_bwd(const void* y_grad, const float* mean_grad, const float* var_grad,
                                 const void* x, int dtype, const float* prev_mean,
                                 const int64_t* count, const float* group_mean,
                                 const float* cummean, const float* cumrstd, const float* gamma,
                                 const uint8_t* mask, int64_t B, int64_t L, int64_t H, int64_t G,
                                 void* x_grad, float* prev_mean_grad, float* prev_var_grad,
                                 float* gamma_grad, float* beta_grad, void* workspace,
                                 size_t workspace_bytes, void* stream);
int mega_timestep_norm_bwd(const void* y_grad, const float* mean_grad, const float* var_grad,
                           const void* x, int dtype, const float* prev_mean, const int64_t* count,
                           const float* cummean, const float* cumrstd, const float* gamma,
                           const uint8_t* mask, int64_t B, int64_t L, int64_t H, void* x_grad,
                           float* prev_mean_grad, float* prev_var_grad, float* gamma_grad,
                           float* beta_grad, void* workspace, size_t workspace_bytes,
                           void* stream);

/* ------------------------------------------------------------------------ */
/* SequenceNorm (the whole-sequence twin of TimestepNorm, used by bidirectional layers)      */
/* stands in for group_sequence_norm_fwd and sequence_norm_fwd
 * (fairseq/csrc/ops/sequence_norm.cc:953-1010 and :844-900; loops at :531-656, :258-372;
 * caller norm_layer/sequence_norm.py:14-33).
 *   x, y   [B,L,H] (length_last = 0) or [B,H,L] (length_last = 1) contiguous of `dtype`
 *   gamma, beta [H] fp32 (gamma is weight + 1); mask [B,L] bytes, non-zero = padding, or NULL
 *   count [B] int64 = unmasked tokens; mean, rstd [B,G] fp32: statistics over the unmasked
 *   tokens and the group's channels (biased variance); masked tokens of y are 0.
 * The per-feature form has H in place of G.                                                 */
size_t mega_sequence_norm_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t H, int64_t G,
                                          int length_last);
int mega_group_sequence_norm_fwd(const void* x, void* y, int dtype, const float* gamma,
                                 const float* beta, const uint8_t* mask, int64_t B, int64_t L,
                                 int64_t H, int64_t G, double eps, int length_last,
                                 int64_t* count, float* mean, float* rstd, void* workspace,
                                 size_t workspace_bytes, void* stream);
int mega_sequence_norm_fwd(const void* x, void* y, int dtype, const float* gamma, const float* beta,
                           const uint8_t* mask, int64_t B, int64_t L, int64_t H, double eps,
                           int length_last, int64_t* count, float* mean, float* rstd,
                           void* workspace, size_t workspace_bytes, void* stream);
/* backward for the [B,H,L] layout (the one the reference module uses): stands in for
 * group_sequence_norm_bwd / sequence_norm_bwd with length_last = true
 * (fairseq/csrc/ops/sequence_norm.cc:756-842, :459-529; pass G = H for the per-feature form).
 *   y_grad, x, x_grad [B,H,L] contiguous of `dtype`; count, mean, rstd as the forward wrote
 *   them; outputs x_grad, gamma_grad, beta_grad [H] fp32.                                 */
size_t mega_sequence_norm_bwd_workspace_bytes(int64_t B, int64_t H, int64_t G);
int mega_group_sequence_norm_bwd(const void* y_grad, const void* x, int dtype, const int64_t* count,
                                 const float* mean, const float* rstd, const float* gamma,
                                 const uint8_t* mask, int64_t B, int64_t L, int64_t H, int64_t G,
                                 void* x_grad, float* gamma_grad, float* beta_grad,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Attention softmax and the fused attention op                              */
/* stands in for attention_softmax_fwd (fairseq/csrc/ops/attention_softmax.cc:6-18,
 * ops/attention_softmax_kernel.cu:22-64, softmax.cuh:90-185).
 *   x, y [batch, outer, inner] contiguous of `dtype`; causal: row r keeps the first
 *   inner - outer + r + 1 columns; a fully masked row becomes zeros.
 *   dropout in [0, 1] is DropKey (softmax.cuh:157-185): each score is replaced by -inf with
 *   that probability before the softmax.  The reference draws from the Philox stream of its
 *   CUDA generator; here the draw for element e of the flattened input is a counter-based hash
 *   of (seed, e), so one seed names one mask, for this op and for mega_attention_fwd alike.
 *   dropout = 0 ignores the seed.                                                       */
int mega_attention_softmax_fwd(const void* x, void* y, int dtype, int64_t batch, int64_t outer,
                               int64_t inner, int causal, float dropout, uint64_t seed,
                               void* stream);
/* stands in for attention_softmax_bwd (fairseq/csrc/ops/attention_softmax.cc:20-26,
 * softmax.cuh AttentionSoftmaxBwdKernel; also the middle step of attention_bwd,
 * ops/attention_kernel.cu:195-203):
 *   x_grad = scale * y * (y_grad - rowsum(y * y_grad)); columns behind the causal limit are 0.
 *   x_grad may be the same buffer as y_grad.                                            */
int mega_attention_softmax_bwd(const void* y_grad, const void* y, void* x_grad, int dtype,
                               int64_t batch, int64_t outer, int64_t inner, int causal,
                               float scale, void* stream);

/* stands in for attention_fwd (fairseq/csrc/ops/attention_kernel.cu:40-131, 257-276):
 *   q, k [B,L,Nh,H1]; v, y [B,L,Nh,H2] contiguous of `dtype`;
 *   y[b,:,n,:] = softmax_causal(scale q k^T) v per (b, n).  The L x L weights are
 *   not returned unless w != NULL (w [B,Nh,L,L] of `dtype`).  y = NULL with w != NULL forms the weights
 *   alone (matrix-core path only, MEGA_ERR_UNSUPPORTED otherwise): for a backward that did not keep them.
 *   dropout, seed: DropKey on the scaled scores, as in mega_attention_softmax_fwd; element
 *   e is the score's place in the [B,Nh,L,L] weights.
 *   16-bit activations with H1 % 8 == 0 run on the matrix cores and need the workspace
 *   (scores in fp32, probabilities and v^T in the activation type); other requests need
 *   none (mega_attention_workspace_bytes returns 0).                                   */
size_t mega_attention_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1,
                                      int64_t H2);
int mega_attention_fwd(const void* q, const void* k, const void* v, void* y, void* w, int dtype,
                       int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2, float scale,
                       int causal, float dropout, uint64_t seed, void* workspace,
                       size_t workspace_bytes, void* stream);
/* stands in for attention_bwd (fairseq/csrc/ops/attention_kernel.cu:133-255, 278-296): the gradients of
 * mega_attention_fwd with respect to q, k and v from y_grad [B,L,Nh,H2] and the forward's weights
 * w [B,Nh,L,L] (the reference keeps them for the backward as well):
 *   w_grad = y_grad v^T;  s_grad = scale w (w_grad - rowsum(w w_grad));
 *   v_grad = w^T y_grad;  q_grad = s_grad k;  k_grad = s_grad^T q           per (b, n),
 * with the causal half of every product skipped when causal != 0.  Weights that DropKey zeroed in
 * the forward give zero gradients by the same formulas.  16-bit activations with H1 % 8 == 0 and
 * H2 % 8 == 0, 16-byte aligned tensors, B * Nh <= 65535, L < 32768 (MEGA_ERR_UNSUPPORTED otherwise;
 * mega_attention_bwd_workspace_bytes returns 0 for such a request).
 *   y: the forward's output [B,L,Nh,H2], or NULL (the reference's backward does not take it).  With
 *   y, rowsum(w w_grad) = rowsum(y_grad y) is known before the first product, and when L % 8 == 0
 *   s_grad leaves that product's epilogue directly: no L x L fp32 weight gradient in memory.  y must
 *   be what mega_attention_fwd wrote for this very w (y = w v); nothing checks it, and a y from
 *   elsewhere gives a wrong s_grad.
 * The workspace holds the fp32 weight gradient, s_grad, the row sums and, for rows of w that are
 * not whole 16-byte pieces (L % 8 != 0), transposed copies of w, s_grad, y_grad, q and k.   */
size_t mega_attention_bwd_workspace_bytes(int dtype, int64_t B, int64_t L, int64_t Nh, int64_t H1,
                                          int64_t H2);
int mega_attention_bwd(const void* y_grad, const void* q, const void* k, const void* v,
                       const void* w, const void* y, void* q_grad, void* k_grad, void* v_grad, int dtype,
                       int64_t B, int64_t L, int64_t Nh, int64_t H1, int64_t H2, float scale,
                       int causal, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* SwiGLU gate: y = silu(a) * b, elementwise over n elements of `dtype`.
 * No counterpart in the reference (its FFN is SiLU-MLP,
 * fairseq/modules/normalized_feedforward_network.py:77-93); the activation itself is
 * the reference's F.silu.                                                         */
int mega_swiglu_fwd(const void* a, const void* b, void* y, int dtype, int64_t n, void* stream);

/* The activation alone: y = silu(a) = a / (1 + exp(-a)), elementwise over n elements of `dtype`
 * (arithmetic in fp32); y may be a itself.  Stands in for the F.silu calls of the layer on the
 * value projection and the moving-average output
 * (fairseq/modules/moving_average_gated_attention.py:303, 308, 316 with moving_act = silu) and of
 * the feed-forward block (fairseq/modules/normalized_feedforward_network.py:82).                              */
int mega_silu_fwd(const void* a, void* y, int dtype, int64_t n, void* stream);

/* ------------------------------------------------------------------------ */
/* Per-token glue of the gated-attention layer.  Inputs are [T, *] row-major with an
 * element stride per row (so a slice of a wider projection output is passed in place);
 * outputs are contiguous [T, *] of the same `dtype`; arithmetic in fp32.
 *
 * mega_rms_norm_fwd stands in for FusedRMSNorm.forward
 *   (fairseq/modules/norm_layer/layer_norm.py:51-59): y = x * rsqrt(mean(x^2) + eps) * weight,
 *   weight [D] fp32 or NULL.
 * mega_gate_qk_fwd stands in for moving_average_gated_attention.py:324-328 followed by
 *   RotaryEmbedding.forward (relative_positional_bias.py:86-97) with qidx = 0:
 *   zn = z / max(|z|_2, eps); q = rot(zn * gamma[0] + beta[0]); k = rot(zn * gamma[1] + beta[1]);
 *   gamma, beta [2, S] fp32 (gamma already holds the "+ 1"); rot turns features (2i, 2i+1) of
 *   each of the `heads` slices of S/heads features by (pos0 + t % chunk) * freqs[i],
 *   freqs [S/heads/2] fp32 (the module's buffer).
 * mega_gate_mul_fwd: y = a * silu(r)                      (lines 330 and 407)
 * mega_gate_out_fwd: y = residual + sigmoid(u) * (silu(hx + hp) - residual)
 *                                                          (lines 322, 409 and 412)        */
int mega_rms_norm_fwd(const void* x, int64_t x_stride, const float* weight, void* y, int dtype,
                      int64_t T, int64_t D, double eps, void* stream);
int mega_gate_qk_fwd(const void* z, int64_t z_stride, const float* gamma, const float* beta,
                     const float* freqs, void* q, void* k, int dtype, int64_t T, int64_t S,
                     int64_t heads, int64_t chunk, int64_t pos0, double eps, void* stream);
int mega_gate_mul_fwd(const void* a, int64_t a_stride, const void* r, int64_t r_stride, void* y,
                      int dtype, int64_t T, int64_t E, void* stream);
int mega_gate_out_fwd(const void* residual, int64_t residual_stride, const void* u,
                      int64_t u_stride, const void* hx, int64_t hx_stride, const void* hp,
                      int64_t hp_stride, void* y, int dtype, int64_t T, int64_t D, void* stream);
/* Backward of the element-wise gates (in the reference these are autograd graphs of torch
 * element-wise operations over the same lines); gradients are contiguous [T, *] of `dtype`:
 *   mega_gate_mul_bwd: a_grad = y_grad silu(r), r_grad = y_grad a silu'(r)
 *   mega_gate_out_bwd: residual_grad = y_grad (1 - s), u_grad = y_grad (h - residual) s (1 - s),
 *                      h_grad = y_grad s silu'(hx + hp) (the gradient of hx and of hp),
 *                      s = sigmoid(u), h = silu(hx + hp)
 *   mega_swiglu_bwd:   a_grad = y_grad b silu'(a), b_grad = y_grad silu(a)                 */
/* Backward of mega_gate_qk_fwd (the autograd graph of moving_average_gated_attention.py:324-328
 * and of the rotation, relative_positional_bias.py:86-97): q_grad, k_grad, z_grad contiguous [T, S]
 * of `dtype`, z as in the forward call; gamma [2, S] (holding the "+ 1"); gamma_grad, beta_grad
 * [2, S] fp32.  S a multiple of 16 bytes' worth of elements, at most 1024 (bf16, fp16) or 512 (fp32)
 * features.  The workspace holds one row of partial parameter sums per workgroup.          */
size_t mega_gate_qk_bwd_workspace_bytes(int64_t T, int64_t S);
int mega_gate_qk_bwd(const void* q_grad, const void* k_grad, const void* z, int64_t z_stride,
                     const float* gamma, const float* freqs, void* z_grad, float* gamma_grad,
                     float* beta_grad, int dtype, int64_t T, int64_t S, int64_t heads,
                     int64_t chunk, int64_t pos0, double eps, void* workspace,
                     size_t workspace_bytes, void* stream);
int mega_gate_mul_bwd(const void* y_grad, const void* a, int64_t a_stride, const void* r,
                      int64_t r_stride, void* a_grad, void* r_grad, int dtype, int64_t T, int64_t E,
                      void* stream);
int mega_gate_out_bwd(const void* y_grad, const void* residual, int64_t residual_stride,
                      const void* u, int64_t u_stride, const void* hx, int64_t hx_stride,
                      const void* hp, int64_t hp_stride, void* residual_grad, void* u_grad,
                      void* h_grad, int dtype, int64_t T, int64_t D, void* stream);
int mega_swiglu_bwd(const void* y_grad, const void* a, const void* b, void* a_grad, void* b_grad,
                    int dtype, int64_t n, void* stream);
/* Backward of mega_silu_fwd (F.silu under autograd): a_grad = y_grad silu'(a), contiguous, n elements.   */
int mega_silu_bwd(const void* y_grad, const void* a, void* a_grad, int dtype, int64_t n, void* stream);
/* out[b][c][r] = in[b][r'][c'] for `batch` matrices of rows x cols elements of 2 or 4 bytes (any values: the
 * elements are moved, not interpreted), with r' = rows - 1 - r when reverse_rows and c' = cols - 1 - c when
 * reverse_cols; in and out are contiguous and must not overlap.  No counterpart in the reference, which calls
 * Tensor::transpose(...).contiguous() and flip(): the Python host uses it to hand fp32 / fp16 activations that lie
 * time-major in memory ([B, L, D]) to the moving average's rows kernels ([B, D, L]) and back, reversed in time for
 * the input gradient.                                                                                         */
int mega_transpose_2d(const void* in, void* out, int elem_bytes, int64_t batch, int64_t rows, int64_t cols,
                      int reverse_rows, int reverse_cols, void* stream);

/* Column sums of x [T, W] (row stride in elements) into out [W] of `out_dtype`: the bias gradient of a projection
 * (in the reference torch's sum over the tokens inside the backward of F.linear).  Rows of whole 16-byte pieces;
 * slabs of 256 rows are added in a fixed order (the same bits on every run); workspace of
 * mega_colsum_workspace_bytes(T, W), no initialisation.                                              */
size_t mega_colsum_workspace_bytes(int64_t T, int64_t W);
int mega_colsum(const void* x, int64_t row_stride, int dtype, int64_t T, int64_t W, void* out,
                int out_dtype, void* workspace, size_t workspace_bytes, void* stream);
/* The same three with row strides (in elements) on the gradients of u, z, r, hx: these four are slices of
 * the mx_proj output (torch.split, moving_average_gated_attention.py:319), whose backward in the reference is
 * a concatenation of the four gradients; a caller that owns one [T, D + S + E + D] gradient buffer lets each
 * kernel write its slice in place (row stride = the buffer's width) and skips that copy.  h_grad is read by
 * the output projection's backward as well: a row-strided matrix operand.                               */
int mega_gate_qk_bwd_strided(const void* q_grad, const void* k_grad, const void* z, int64_t z_stride,
                             const float* gamma, const float* freqs, void* z_grad,
                             int64_t z_grad_stride, float* gamma_grad, float* beta_grad, int dtype,
                             int64_t T, int64_t S, int64_t heads, int64_t chunk, int64_t pos0,
                             double eps, void* workspace, size_t workspace_bytes, void* stream);
int mega_gate_mul_bwd_strided(const void* y_grad, const void* a, int64_t a_stride, const void* r,
                              int64_t r_stride, void* a_grad, void* r_grad, int64_t r_grad_stride,
                              int dtype, int64_t T, int64_t E, void* stream);
int mega_gate_out_bwd_strided(const void* y_grad, const void* residual, int64_t residual_stride,
                              const void* u, int64_t u_stride, const void* hx, int64_t hx_stride,
                              const void* hp, int64_t hp_stride, void* residual_grad, void* u_grad,
                              int64_t u_grad_stride, void* h_grad, int64_t h_grad_stride, int dtype,
                              int64_t T, int64_t D, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MEGA_HIP_H_ */
