// Host-visible argument blocks and launchers of the ring-attractor kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

typedef float ring_f32x4 __attribute__((ext_vector_type(4)));

struct RingFwdArgs {
  const float* A;        // [B,T,k]
  const void* Wpack;     // packed bf16 forward fragments
  const float* r_init;   // [B,N]
  float* hist;           // [T,B,N] (forward: output; rebuild: input)
  _Float16* dfrag;       // F'(re) in tile order, or null
  __bf16* rfrag;         // bf16 r_prev in tile order, or null
  float J0, J1, alpha;
  int N, k, T, B, nbt, act;
  // Loss head's per-row sums (sum_i r_i cos(phi_i), sum_i r_i sin(phi_i), sum_i |r_i|, -) of every history row
  // [T*B], written by the weight-resident forward kernel itself when non-null (other kernels ignore it).
  ring_f32x4* loss_stats = nullptr;
  // Non-null: run the four-compute-unit cluster kernel (ring_cluster.hip) with this scratch area of
  // ring_cluster_workspace_bytes(nbt) bytes; Wpack is then in that kernel's column order with J1 * Wo + J0 as matrix 0.
  void* cluster_ws = nullptr;
};

struct RingBpttArgs {
  const float* A;
  const void* Wpack;     // packed bf16 transposed fragments
  const float* grad_out; // [T,B,N]
  const _Float16* dfrag;
  __bf16* gfrag;         // bf16 g in tile order (output)
  const __bf16* rfrag;   // bf16 r_prev in tile order (the forward's operand copy); read for grad_A by the weight-resident kernel
  float* grad_r_init;    // [B,N] or null
  float* grad_A;         // [B,T,k] or null (written, not accumulated); needs hist and r_init (streaming kernel) or rfrag
  const float* hist;     // [T,B,N] state history (r_prev of step t is hist[t-1]); read for grad_A and by the fused loss head
  const float* r_init;   // [B,N]
  // Loss head fused into the weight-resident BPTT kernel (null: grad_out is read).  loss_coef[t*B + b] holds the
  // row's (kc, ks, beta, -) as ring_loss_stats/rows/decode left them; the kernel then reads hist, not grad_out.
  const ring_f32x4* loss_coef;
  const float* loss_upstream;   // one float on the device, or null for 1
  float loss_inv_rows;          // 1 / (T * B)
  const float* loss_trig = nullptr;   // step-per-launch kernels with loss_coef: (cos, sin)(2 pi j / N) pairs, j < NPAD
  float* wide_carry;     // N > 512 only: 2 x [16*nbt][NPAD] fp32 scratch for the carried gradient between step launches
  float J0, J1, alpha;
  int N, k, T, B, nbt;
  void* cluster_ws = nullptr;   // non-null: the cluster kernel (ring_cluster.hip), ring_cluster_bptt_workspace_bytes(nbt) bytes
};

struct RingDwArgs {
  const float* A;
  const __bf16* gfrag;
  const __bf16* rfrag;
  ring_f32x4* partial;   // [nz][1+k][NT][NT][64] fp32x4
  float* grad_Wo;        // [N,N], accumulated into
  float* grad_Wa;        // [k,N,N], accumulated into
  float J1;
  int accumulate;        // non-zero: += into grad_Wo / grad_Wa (the caller zeroed them); zero: overwrite
  int N, k, T, B, nbt, nz;
};

// matrix 0 is packed as scale0 * Wo + shift0 (see ring_pack_weights_kernel)
hipError_t ring_launch_pack(const float* Wo, const float* Wa, void* out, int N, int k, int NC, int transposed,
                            int split_k, float scale0, float shift0, hipStream_t st);
// two packed copies in one launch (out2 may be null)
hipError_t ring_launch_pack2(const float* Wo, const float* Wa, int N, int k, int NC, void* out, int transposed,
                             int split_k, float scale0, float shift0, void* out2, int transposed2, int split_k2,
                             float scale2, float shift2, hipStream_t st);
hipError_t ring_launch_fwd(const RingFwdArgs& a, int NC, hipStream_t st);
bool ring_fwd_forms_loss_sums(const RingFwdArgs& a, int NC);   // will that launch fill a.loss_stats?
hipError_t ring_launch_rebuild(const RingFwdArgs& a, int NC, hipStream_t st);
hipError_t ring_launch_bptt(const RingBpttArgs& a, int NC, hipStream_t st);
hipError_t ring_launch_dw(const RingDwArgs& a, int NC, hipStream_t st);

// Weight-resident variants for 128 < N <= 256, a_dim == 2 (ring_res256.hip).
bool ring_res256_applicable(int N, int k);
bool ring_uses_resident(int N, int k);   // applicable and not disabled by RINGATTR_STREAMING=1
hipError_t ring_launch_fwd_res256(const RingFwdArgs& a, hipStream_t st);
hipError_t ring_launch_bptt_res256(const RingBpttArgs& a, hipStream_t st);

// Weight-resident forward over clusters of four compute units for N == 512, a_dim == 2 (ring_cluster.hip).
struct RingClusterArgs {
  void* xchg;        // [2][2 * npairs][16 K chunks][4][16 rows] x 16 bytes: the state in MFMA A-operand order
  int* flags;        // [nclusters][ppc][32]: last state number published per (pair, member, wave)
  int* hello;        // [nclusters][4]: XCC_ID + 1 of each member
  int* host_err;     // word in pinned host memory, RING_CLUSTER_ERR_* when a wait ran out
  void* ghalf;       // BPTT: the same order x 16 bytes, the first 8: bf16 g of the last odd step
  float* carry;      // BPTT: [2 * npairs][4 members][8 waves][64 lanes] x 16 bytes, (1 - alpha) G of the lane's four rows
  int npairs, nclusters, ppc, spin_max;
};
enum { RING_CLUSTER_ERR_XCD = 1, RING_CLUSTER_ERR_START = 2, RING_CLUSTER_ERR_WAIT = 3 };
bool ring_cluster_applicable(int N, int k);               // the shape alone
size_t ring_cluster_workspace_bytes(int nbt);
bool ring_uses_cluster(int N, int k, int B, int T);       // applicable, switched on, whole pairs of batch tiles, and the device has the compute units
bool ring_uses_cluster_bptt(int N, int k, int B, int T);  // the BPTT on clusters: the same conditions, and only when asked for (RINGATTR_CLUSTER_BPTT=1)
int ring_cluster_error();                                 // the host word: non-zero once a cluster kernel gave up waiting
int ring_cluster_take_error();                            // the same, the first time it is found set; 0 afterwards
int ring_cluster_pack_order(int N, int B, int T);        // the column order (ring_pack_weights_kernel's split_k) its kernel for that shape reads
hipError_t ring_launch_fwd_cluster(const RingFwdArgs& a, hipStream_t st);
size_t ring_cluster_bptt_workspace_bytes(int nbt);
hipError_t ring_launch_bptt_cluster(const RingBpttArgs& a, hipStream_t st);   // a.cluster_ws; Wpack transposed, in ring_cluster_pack_order, J1 * Wo^T + J0 as matrix 0

// Step-per-launch kernels for 512 < N <= 2048, NC in {16, 24, 32} (ring_bign.hip).
bool ring_wide_applicable(int NC);
size_t ring_wide_carry_bytes(int NC, int nbt);
hipError_t ring_launch_wide_fwd(const RingFwdArgs& a, int NC, bool rebuild, int tiles_per_wave, hipStream_t st);
hipError_t ring_launch_wide_bptt(const RingBpttArgs& a, int NC, float* carry, hipStream_t st);

// Step-per-launch kernels with several batch tiles per workgroup (ring_block.hip); same saved-record layout and
// carry buffer as the wide-ring kernels.
hipError_t ring_launch_block_fwd(const RingFwdArgs& a, int NC, bool rebuild, hipStream_t st);
hipError_t ring_launch_block_bptt(const RingBpttArgs& a, int NC, float* carry, hipStream_t st);
bool ring_block_many_matrices(int k);   // the weight stream dominates a step: the block kernels lead at any batch size
// dL/dA of the step-per-launch families: a separate pass after the BPTT steps (Wf: forward-orientation packed weights)
// (cos, sin)(2 pi j / N) for j < N, zero up to NPAD: what the step-per-launch BPTT kernels read with the fused loss head
hipError_t ring_launch_trig_table(float* out, int N, int NPAD, hipStream_t st);
hipError_t ring_launch_block_grad_A(const RingBpttArgs& a, const void* Wf, int NC, hipStream_t st);
// which kernel family runs a problem with a saved record: 0 persistent, 1 step-per-launch (wide or block)
bool ring_uses_step_kernels(int N, int k, int NC, int nbt);

// LDS-tiled weight-gradient contraction for NC in {4, 8, 16, 24, 32} (ring_dw.hip).
bool ring_dw_tiled_applicable(int NC);
int ring_dw_tiled_nz(int NC, int k, long nchunk);
hipError_t ring_launch_dw_tiled(const RingDwArgs& a, int NC, hipStream_t st);

// Fused decode + loss head over the state history (ring_loss.hip).
size_t ring_loss_workspace_bytes(int T, int B);
hipError_t ring_launch_loss_fwd(const float* hist, const float* angle, const float* target_amp, float bump_weight,
                                float* loss_out, int N, int T, int B, void* workspace, bool have_row_sums,
                                hipStream_t st);
// where the forward kernel leaves the per-row sums for ring_launch_loss_fwd(..., have_row_sums = true)
ring_f32x4* ring_loss_row_sums(void* workspace);
hipError_t ring_launch_loss_bwd(const float* hist, const float* angle, const float* target_amp, float bump_weight,
                                const float* upstream, float* grad_hist, int N, int T, int B, const void* workspace,
                                hipStream_t st);
// the per-row coefficients (kc, ks, beta, -) inside a workspace that ring_launch_loss_fwd filled
const ring_f32x4* ring_loss_row_coefficients(const void* workspace);

// Gain networks of the action signal (ring_gain.hip): params / grad_params are [k][3h+1] = [w1 | b1 | w2 | b2] per channel.
size_t ring_gain_workspace_bytes(int k, int h, long samples);
hipError_t ring_launch_gain_fwd(const float* x, const float* params, float* out, int k, int h, long samples, hipStream_t st);
hipError_t ring_launch_gain_bwd(const float* x, const float* params, const float* grad_A, float* grad_params, float* grad_x,
                                int k, int h, long samples, void* workspace, hipStream_t st);

// Synthetic input generator and optimizer tail (ring_aux.hip).
struct RingGenArgs {
  unsigned long long seed;
  float* av;             // [B,T]
  float* angle;          // [B,T]
  float* action;         // [B,T,k]
  float* r_init;         // [B,N] or null
  float ratios[8];       // zero ratios to pick from
  int n_ratios;
  int n_initial_zeros;   // leading zero steps of every trial
  float max_av, bump_param;
  int spread;            // 0: (L, R) in channels 0, 1, zeros elsewhere; 1: relu(av * linspace(-1, 1, k))
  int bump_kind;         // 0: Gaussian of width N / bump_param on the circular distance; 1: von Mises, kappa = bump_param
  int N, k, T, B;
};
hipError_t ring_launch_generate(const RingGenArgs& a, hipStream_t st);

constexpr int RING_OPT_MAX_TENSORS = 16;
struct RingOptArgs {
  float* param[RING_OPT_MAX_TENSORS];
  float* grad[RING_OPT_MAX_TENSORS];
  float* exp_avg[RING_OPT_MAX_TENSORS];
  float* exp_avg_sq[RING_OPT_MAX_TENSORS];
  size_t numel[RING_OPT_MAX_TENSORS];
  int chunks[RING_OPT_MAX_TENSORS];
  int n;
  float beta1, beta2, eps, max_norm;
  float step_size;       // lr / (1 - beta1^t)
  float inv_sqrt_bc2;    // 1 / sqrt(1 - beta2^t)
  int* step_counter;     // non-null: t lives on the device; the call advances it and derives the two factors itself
  float lr;              // (used with step_counter)
};
int ring_opt_chunks(size_t numel);
hipError_t ring_launch_clip_adam(const RingOptArgs& a, float* workspace, hipStream_t st);

// Which kernel ran.  The dispatch functions open a scope that names the slot (RINGATTR_K_*) their launches belong
// to; RING_LAUNCH remembers the kernel it launches under the innermost open slot of the calling thread, and
// ring_last_kernel_name gives that kernel's name ("ring_fwd_res256_kernel<1,true,true,false>": demangled, without
// return type, parameter list and blanks), so that a benchmark can tell whether a stored counter summary is of the
// kernel it has just timed.
void ring_note_kernel(const void* host_function);
int ring_last_kernel_name(int id, char* buf, size_t n);
#define RING_LAUNCH(kern, grid, block, lds, st, ...)                       \
  do {                                                                     \
    ring_note_kernel(reinterpret_cast<const void*>(kern));                 \
    hipLaunchKernelGGL(kern, grid, block, lds, st, __VA_ARGS__);           \
  } while (0)

bool ring_dw_tiled_applicable(int NC);
int ring_dw_tiled_segments(int nbt, int T, int nz);   // launches per matrix group of the tiled weight-gradient kernel

// Optional event bracketing of launches (benchmark support).
void ring_profile_set(int stride);
bool ring_profile_on();
hipError_t ring_profile_collect(double* ms, long long* launches);
