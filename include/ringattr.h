/*
 * ringattr.h -- C ABI of the MI355X (gfx950) leaky ring-attractor time loop.
 *
 * One shared library (libringattr.so) exports the forward recurrence and its
 * reverse-time BPTT.  All tensors are fp32, contiguous, row-major DEVICE
 * pointers owned by the caller; the library allocates nothing inside the
 * ringattr_* entry points (the caller brings the workspace).  Work is enqueued
 * on the HIP stream passed as `stream` (a hipStream_t, NULL = the null stream)
 * and the calls return without synchronising.
 *
 * Shapes (B = batch_size, T = seq_len, k = a_dim, N = neurons):
 *   A            [B,T,k]   action signal
 *   Wa           [k,N,N]   action-modulated weight bank
 *   Wo           [N,N]     recurrent weights
 *   r_init       [B,N]     initial state (never modified)
 *   bump_history [T,B,N]   state after every step (forward output)
 *   grad_output  [T,B,N]   dL/d bump_history
 *   grad_Wa [k,N,N], grad_Wo [N,N]   accumulate = 1: added to (the reference's contract, cpp/ring_rnn_cuda.py:98-99:
 *                                    the caller zeroes them); accumulate = 0: overwritten (may be uninitialised)
 *
 * Math per sample b and step t (r_prev = r_init at t = 0):
 *   re  = J0*sum_j r_prev[j] + J1*(Wo r_prev) + sum_c A[b,t,c]*(Wa[c] r_prev)
 *   r_t = (1-alpha)*r_prev + alpha*F(re),   F in {relu, gelu(erf), tanh, silu}
 *
 * activation_type: 0 relu, 1 gelu, 2 tanh, 3 silu
 * (reference: cpp/ring_rnn_cuda.py:63, cpp/cuda_common.cuh:56).
 *
 * Every int-returning entry point returns RINGATTR_OK or an error code;
 * ringattr_last_error() gives the message.  Nothing here ever exits the process
 * (the reference's CHECK_CUDA_ERROR does, cpp/cuda_common.cuh:30-39).
 */
#ifndef RINGATTR_H
#define RINGATTR_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RINGATTR_API __attribute__((visibility("default")))

#define RINGATTR_OK 0
#define RINGATTR_ERR_INVALID 1   /* bad shape, null pointer, unknown activation */
#define RINGATTR_ERR_WORKSPACE 2 /* workspace pointer null or too small */
#define RINGATTR_ERR_HIP 3       /* a HIP runtime call or kernel launch failed */

/* Library version (major*1000 + minor). */
RINGATTR_API int ringattr_version(void);

/* Message of the last failing call made on the calling thread ("" if none). */
RINGATTR_API const char* ringattr_last_error(void);

/* Bytes of the "saved activations" buffer the forward pass fills for training:
 * alpha*F'(re) as fp16 and the bf16 operand copy of r_prev, both in the kernels'
 * private tile order, and the transposed bf16 weight fragments the backward
 * multiplies with (so a backward that is handed `saved` differentiates at the
 * weights its forward saw and needs no packing launch of its own).  Opaque to
 * the caller: allocate, pass to ringattr_fwd, keep until ringattr_bwd.  Replaces the reference's re_history slot
 * (cpp/ring_rnn_cuda.py:106, cpp/bwd.cu:12). */
RINGATTR_API size_t ringattr_saved_bytes(int N, int a_dim, int seq_len, int batch_size);

/* Scratch bytes needed by ringattr_fwd / ringattr_bwd.  have_saved = 1 when the
 * forward's saved buffer will be handed to the backward, 0 when the backward
 * must rebuild it from bump_history (then the workspace also holds it).
 * At N = 512 with two action channels the forward's figure includes the exchange area of the
 * kernel that spreads the weights over four compute units; a forward handed less than that (but at
 * least the packed weights) runs the weight-streaming kernel instead.
 * The backward's figure at that width includes the scratch area of the BPTT on the same clusters
 * (switched on by RINGATTR_CLUSTER_BPTT=1), whether it is on or not.
 * Replaces the fixed workspace list of cpp/ring_rnn_cuda.py:108-114. */
RINGATTR_API size_t ringattr_fwd_workspace_bytes(int N, int a_dim, int seq_len, int batch_size);
RINGATTR_API size_t ringattr_bwd_workspace_bytes(int N, int a_dim, int seq_len, int batch_size, int have_saved);

/* Forward recurrence over all T steps in one persistent launch.
 * Replaces fwd_cuda (cpp/fwd.cu:21-50) and the pybind shim cpp/fwd.cpp:20-47.
 * `saved` may be NULL (inference: nothing but bump_history is written). */
RINGATTR_API int ringattr_fwd(const void* A, const void* Wa, float J0, float J1, const void* Wo,
                 const void* r_init, void* bump_history, float alpha,
                 int N, int a_dim, int seq_len, int batch_size, int activation_type,
                 void* saved, void* workspace, size_t workspace_bytes, void* stream);

/* ringattr_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * ringattr_fwd without the workspace pair: the packed bf16 weights go into a fixed array of
 * RINGATTR_NOALLOC_SCRATCH_BYTES that lives inside the library's code object on every GPU it runs on (held until
 * the process ends).  The call allocates and frees nothing.  Shapes whose packed weights
 * ((1 + a_dim) * NPAD^2 * 2 bytes, NPAD = N rounded up to the kernel's tiling) exceed the array are rejected with
 * RINGATTR_ERR_WORKSPACE.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (different streams, different threads) race on it; calls on one stream are ordered and safe.  The device that
 * owns the tensors must be current.  `saved` may be NULL or a caller buffer of ringattr_saved_bytes. */
#define RINGATTR_NOALLOC_SCRATCH_BYTES (4u << 20)
RINGATTR_API int ringattr_fwd_noalloc(const void* A, const void* Wa, float J0, float J1, const void* Wo,
                 const void* r_init, void* bump_history, float alpha,
                 int N, int a_dim, int seq_len, int batch_size, int activation_type,
                 void* saved, void* stream);

/* Reverse-time BPTT + weight gradients.
 * Replaces bwd_cuda (cpp/bwd.cu:4-52) and cpp/bwd.cpp:34-99.
 * `saved` may be NULL: the saved record is then recomputed, from bump_history
 * or (weight-resident geometry: a_dim == 2, 128 < N <= 256) by running the
 * recurrence again from r_init, which reproduces the forward's own numbers.
 * grad_A [B,T,k] and grad_r_init [B,N] are optional outputs (NULL = skip), written
 * rather than accumulated; the reference returns None for both
 * (cpp/ring_rnn_cuda.py:144).  grad_A comes out of the BPTT kernel itself up to N = 512 (the
 * weight-resident kernel reads the bf16 operand copy of r_prev with the step's other inputs; the persistent
 * streaming kernel stages its per-channel shares in LDS, which limits it to a_dim <= 48) and from a pass of its own
 * after the BPTT steps on the step-per-launch kernels (wide rings and small batches; any a_dim, seq_len <= 65535).
 * With a saved buffer, the buffer must be the one the forward filled, at the address it filled it, and the
 * weights must be unchanged since (the forward's transposed weight copy inside it is reused on an exact match of
 * shape, J0, J1 and weight addresses; anything else is repacked).
 * accumulate != 0: grad_Wa / grad_Wo are added to, as in the reference, whose caller zeroes them first
 * (cpp/ring_rnn_cuda.py:98-99); accumulate == 0: they are overwritten and need no zeroing. */
RINGATTR_API int ringattr_bwd(const void* grad_output, const void* A, const void* Wa, float J0, float J1,
                 const void* Wo, const void* bump_history, const void* r_init,
                 void* grad_Wa, void* grad_Wo, float alpha,
                 int N, int a_dim, int seq_len, int batch_size, int activation_type, int accumulate,
                 const void* saved, void* grad_A, void* grad_r_init,
                 void* workspace, size_t workspace_bytes, void* stream);

/* Fused decode + loss head over bump_history [T,B,N]: the cosine-similarity head-direction loss of the
 * max-normalised cosine read-out plus bump_weight times the bump-amplitude loss.  No counterpart in the
 * reference's extension: it replaces the chain of torch tensor ops in the training script (root
 * train_general_ring_no_gain.py:113-116, 324-330; train/train_ring_attractor.py:190-220, 275-298), whose
 * W_delta7 read-out has rank two, so a row contributes through three sums over its N values.
 *   target_angle      [B,T] true angles (radians)
 *   target_amplitude  [B] or NULL (NULL: the amplitude of the first step, which then also receives gradient)
 *   loss_out          3 floats on the device: total, cos-sim loss, amplitude loss
 *   upstream          one float on the device (d objective / d total) or NULL for 1
 *   grad_history      [T,B,N], overwritten with d total / d bump_history * upstream
 * ringattr_loss_bwd needs the workspace ringattr_loss_fwd filled for the same inputs.  N <= 2048. */
RINGATTR_API size_t ringattr_loss_workspace_bytes(int N, int seq_len, int batch_size);
RINGATTR_API int ringattr_loss_fwd(const void* bump_history, const void* target_angle, const void* target_amplitude,
                      float bump_weight, void* loss_out, int N, int seq_len, int batch_size,
                      void* workspace, size_t workspace_bytes, void* stream);
RINGATTR_API int ringattr_loss_bwd(const void* bump_history, const void* target_angle, const void* target_amplitude,
                      float bump_weight, const void* upstream, void* grad_history, int N, int seq_len,
                      int batch_size, const void* workspace, size_t workspace_bytes, void* stream);

/* ringattr_fwd followed by ringattr_loss_fwd in one call (same arguments, the time loop's first): the forward of
 *   total = loss_pair(bump_history),  bump_history = forward(...)
 * The persistent forward kernels (N <= 512, except small-batch forwards that are split over workgroups) form the loss
 * head's three sums per history row themselves, right after the activation, and the loss needs no pass of its own
 * over the history (-4N bytes read per sample-step); other shapes run the two stages back to back.  Either way loss_workspace ends up
 * as ringattr_loss_fwd leaves it (for ringattr_loss_bwd / ringattr_bwd_loss).  No counterpart in the reference. */
RINGATTR_API int ringattr_fwd_loss(const void* A, const void* Wa, float J0, float J1, const void* Wo, const void* r_init,
                      void* bump_history, float alpha, int N, int a_dim, int seq_len, int batch_size,
                      int activation_type, void* saved, void* workspace, size_t workspace_bytes,
                      const void* target_angle, const void* target_amplitude, float bump_weight, void* loss_out,
                      void* loss_workspace, size_t loss_workspace_bytes, void* stream);

/* ringattr_bwd with the loss head's gradient in place of grad_output: the backward of
 *   total = loss_pair(bump_history),  bump_history = forward(...)
 * in one call.  No counterpart in the reference (its training script lets autograd chain the torch loss ops into
 * RingRnnCudaFunc.backward, cpp/ring_rnn_cuda.py:81-144).  loss_workspace is the workspace ringattr_loss_fwd
 * filled for this bump_history; upstream is one device float (d objective / d total) or NULL for 1; every other
 * argument is ringattr_bwd's, the workspace included (ringattr_bwd_workspace_bytes).  The BPTT kernels form
 * grad_output in registers from the bump_history rows they load in its place and the loss head's per-row
 * coefficients, so the [T,B,N] gradient is neither written nor read. */
RINGATTR_API int ringattr_bwd_loss(const void* loss_workspace, const void* upstream, const void* A, const void* Wa,
                      float J0, float J1, const void* Wo, const void* bump_history, const void* r_init,
                      void* grad_Wa, void* grad_Wo, float alpha,
                      int N, int a_dim, int seq_len, int batch_size, int activation_type, int accumulate,
                      const void* saved, void* grad_A, void* grad_r_init,
                      void* workspace, size_t workspace_bytes, void* stream);

/* 1 when ringattr_bwd_loss can serve this shape: every shape the time loop itself accepts (all kernel families form
 * the loss gradient themselves); 0 only for shapes ringattr_bwd rejects as well.  A caller that finds 0 runs
 * ringattr_loss_bwd and hands its [T,B,N] result to ringattr_bwd.  No counterpart in the reference. */
RINGATTR_API int ringattr_bwd_loss_available(int N, int a_dim, int seq_len, int batch_size);

/* Gain networks of the action signal, forward and backward.  Replaces the per-channel nn.Sequential(Linear(1,h), GELU,
 * Linear(h,1), Softplus) evaluation and its autograd in the reference models (train/train_ring_attractor.py:70-79,
 * 136-146; train/train_general_ring_attractor.py:38-46, 99-109): per sample, step and channel c
 *   A[b,t,c] = x * softplus(sum_j w2[c][j] * gelu(w1[c][j] * |x| + b1[c][j]) + b2[c]),   x = base_signal[b,t,c].
 * The networks depend only on the input signal, so they run once for all (b, t) in front of the time loop.
 *   base_signal, action_signal, grad_action_signal, grad_base_signal  [B,T,k] fp32
 *   params, grad_params  [k][3*hidden + 1] fp32, per channel [w1 | b1 | w2 | b2]
 * ringattr_gain_bwd overwrites grad_params with the sums over all B*T samples (fixed summation order: repeatable
 * bit for bit) and, when grad_base_signal is not NULL, writes dL/d base_signal.  hidden <= 32, a_dim <= 64. */
RINGATTR_API size_t ringattr_gain_workspace_bytes(int a_dim, int hidden, int seq_len, int batch_size);
RINGATTR_API int ringattr_gain_fwd(const void* base_signal, const void* params, void* action_signal,
                      int a_dim, int hidden, int seq_len, int batch_size, void* stream);
RINGATTR_API int ringattr_gain_bwd(const void* base_signal, const void* params, const void* grad_action_signal,
                      void* grad_params, void* grad_base_signal, int a_dim, int hidden, int seq_len, int batch_size,
                      void* workspace, size_t workspace_bytes, void* stream);

/* Synthetic inputs generated on the device: angular-velocity trials, integrated angles, the action signal and the
 * initial bump, written where the time loop reads them.  Replaces generate_av_integration_data_ultra_fast
 * (utils/generate_av_integration_data.py:11-58), av_to_action_signal / av_to_action_signal_ND (root
 * train_general_ring_no_gain.py:176-229) and create_initial_bump (train/train_ring_attractor.py:21-52).  Same
 * distributions; the random stream is the library's own counter-based generator, a function of `seed` only
 * (repeatable bit for bit, independent of launch geometry).
 *   zero_padding_start_ratio   the first int(seq_len * ratio) steps of every trial are zero; a double, and the
 *                     product is formed in double precision, so the count is the one Python's int() gives
 *   zero_ratios       HOST array of 1..8 floats (per trial one is picked uniformly)
 *   spread_action     0: channels 0 / 1 = relu(-av) / relu(av), others zero; 1: relu(av * linspace(-1, 1, a_dim))
 *   bump_kind, bump_param   0: Gaussian on the circular distance, width N / bump_param (the reference, 10);
 *                           1: von Mises exp(kappa cos(phi_i - angle)), kappa = bump_param; both L2-normalised
 *   av, angle [B,T]; action_signal [B,T,a_dim]; r_init [B,N] or NULL (all fp32 device pointers, outputs) */
/* Number of leading zero steps the generator gives every trial: int(seq_len * zero_padding_start_ratio) as the
 * reference's Python evaluates it (utils/generate_av_integration_data.py:21); -1 for arguments out of range.
 * Host arithmetic only (callable without a GPU). */
RINGATTR_API int ringattr_generator_initial_zeros(int seq_len, double zero_padding_start_ratio);
RINGATTR_API int ringattr_generate_inputs(unsigned long long seed, int N, int a_dim, int seq_len, int batch_size,
                      double zero_padding_start_ratio, const float* zero_ratios, int n_zero_ratios, float max_av,
                      int spread_action, int bump_kind, float bump_param,
                      void* av, void* angle, void* action_signal, void* r_init, void* stream);

/* Optimizer tail of a training step: torch.nn.utils.clip_grad_norm_(parameters, max_norm) followed by
 * torch.optim.Adam.step() (root train_general_ring_no_gain.py:333-336), for up to 16 fp32 tensors in three launches.
 * The gradient norm is summed in a fixed order (repeatable).  params / grads / exp_avg / exp_avg_sq are HOST arrays of
 * n_tensors device pointers, numel a host array; grads are scaled in place by min(1, max_norm / (norm + 1e-6))
 * (max_norm <= 0: no clipping), then m, v and the parameters are updated in place; `step` counts from 1.
 * The gradient norm before clipping is left in the workspace as float number sum_i ceil(numel[i] / 4096) (behind the
 * per-chunk partial sums). */
RINGATTR_API size_t ringattr_clip_adam_workspace_bytes(int n_tensors, const size_t* numel);
RINGATTR_API int ringattr_clip_adam(int n_tensors, void* const* params, void* const* grads, void* const* exp_avg,
                      void* const* exp_avg_sq, const size_t* numel, float lr, float beta1, float beta2, float eps,
                      float max_norm, int step, void* workspace, size_t workspace_bytes, void* stream);
/* The same step with Adam's step number kept on the device: step_counter is a device int32 (zero before the first
 * step) that the call advances by one and derives the bias corrections from, so a training step recorded into a HIP
 * graph keeps counting on every replay (torch.optim.Adam(capturable=True) keeps its step on the device likewise;
 * the reference's eager loop, root train_general_ring_no_gain.py:333-336, has no counterpart). */
RINGATTR_API int ringattr_clip_adam_counted(int n_tensors, void* const* params, void* const* grads, void* const* exp_avg,
                      void* const* exp_avg_sq, const size_t* numel, float lr, float beta1, float beta2, float eps,
                      float max_norm, void* step_counter, void* workspace, size_t workspace_bytes, void* stream);

/* Per-kernel timing for benchmarks; no counterpart in the reference.  ringattr_profile_enable(n): n = 0 switches it
 * off; n >= 1 brackets every n-th launch of each kernel (counted per kernel from this call on) by two HIP events
 * recorded on the launch stream.  The two records cost about 4-5 us of stream time per bracketed launch (23 us per
 * forward + backward at n = 1 on an MI355X), which is why a benchmark that also reports wall time samples with
 * n > 1.  ringattr_profile_read waits
 * for the recorded events, adds their durations into ms[RINGATTR_NUM_KERNELS] and the launch counts
 * into launches[RINGATTR_NUM_KERNELS] (both caller arrays, not cleared first) and forgets them. */
#define RINGATTR_NUM_KERNELS 6
#define RINGATTR_K_PACK 0
#define RINGATTR_K_FWD 1
#define RINGATTR_K_REBUILD 2
#define RINGATTR_K_BPTT 3
#define RINGATTR_K_DW 4
#define RINGATTR_K_DW_REDUCE 5
RINGATTR_API int ringattr_profile_enable(int on);
/* Time segments the weight-gradient kernel of a backward at this shape is launched in (1: one launch per group of three
 * matrices; long sequences are cut so that the workgroups that share operand streams stay aligned in L2; the
 * environment variable RINGATTR_DW_SEGMENT, K chunks of 32 samples per workgroup and launch, default 640, 0 = never
 * cut, is read at every call).  Host arithmetic only; -1 for an unsupported shape. */
RINGATTR_API int ringattr_dw_segments(int N, int a_dim, int seq_len, int batch_size);
/* Name of the kernel this process launched last in slot `kernel` (RINGATTR_K_*), e.g.
 * "ring_fwd_res256_kernel<1,true,true,false>" (demangled, no return type, parameter list or blanks), or the empty
 * string if the slot has not launched yet.  For benchmarks that pair a timing with a stored counter profile. */
RINGATTR_API int ringattr_last_kernel_name(int kernel, char* buf, size_t buf_bytes);
RINGATTR_API int ringattr_profile_read(double* ms, long long* launches);

/* Reference-signature entry points, argument for argument (cpp/fwd.cu:21-35,
 * cpp/bwd.cu:4-30).  They run on the null stream, obtain their scratch with
 * hipMalloc/hipFree around the call, ignore the reference's workspace pointers
 * and cublas_handle, and report failures on stderr without exiting. */
RINGATTR_API void fwd_cuda(void* A, void* Wa, float J0, float J1, void* Wo, void* r_init, void* bump_history,
              float alpha, int N, int a_dim, int seq_len, int batch_size, int activation_type);
RINGATTR_API void bwd_cuda(void* grad_output, void* A, void* Wa, float J0, float J1, void* Wo,
              void* bump_history, void* re_history, void* r_init, void* grad_Wa, void* grad_Wo,
              float alpha, int N, int a_dim, int seq_len, int batch_size, int activation_type,
              void* grad_r, void* W_eff_temp, void* grad_re_temp, void* grad_W_eff_temp_bf16,
              void* A_t_temp_bf16, void* grad_re_temp_T, void* cublas_handle);

#ifdef __cplusplus
}
#endif
#endif /* RINGATTR_H */
