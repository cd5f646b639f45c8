// C ABI of libringattr.so: argument validation, workspace carving and kernel sequencing.
// Entry points and the reference interfaces they replace are documented in include/ringattr.h.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <math.h>

#include <mutex>

#include "ring_kernels.hpp"
#include "ringattr.h"

// Fixed device-side scratch of ringattr_fwd_noalloc: every GPU the library runs on holds its own copy of this array
// until the process ends.  In host code the name below is only a handle for hipGetSymbolAddress; the address the
// kernels receive is the per-device pointer that call returns (noalloc_scratch()).
static __device__ __align__(256) unsigned char scratch[RINGATTR_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

constexpr size_t kAlign = 256;
size_t align_up(size_t x) { return (x + kAlign - 1) / kAlign * kAlign; }

struct Geo {
  int N, k, T, B, NC, NPAD, nbt, nz;
  size_t wpack_bytes;    // one packed copy of [Wo|Wa] in bf16
  size_t side_bytes;     // saved F' (fp16), [T,16*nbt,NPAD] in lane order
  size_t pair_bytes;     // one bf16 operand copy, time steps paired: [ceil(T/2)*2,16*nbt,NPAD]
  size_t partial_bytes;  // split-K partials of the weight gradient
  size_t carry_bytes;    // N > 512: the carried gradient between the per-step BPTT launches
  size_t trig_bytes;     // step-per-launch kernels with the fused loss head: (cos, sin) of every neuron's angle
};

// Smallest supported neuron tiling with 64*NC >= N: the persistent kernels up to N = 512, the step-per-launch
// kernels (NPAD a multiple of 512) up to N = 2048.
int pick_nc(int N) {
  for (int nc = 1; nc <= 8; nc *= 2)
    if (64 * nc >= N) return nc;
  for (int nc = 16; nc <= 32; nc += 8)
    if (64 * nc >= N) return nc;
  return 0;
}

int make_geo(int N, int k, int T, int B, Geo& g) {
  if (N <= 0 || k <= 0 || T <= 0 || B <= 0)
    return fail(RINGATTR_ERR_INVALID, "N, a_dim, seq_len, batch_size must be positive (got %d, %d, %d, %d)", N, k, T, B);
  const int nc = pick_nc(N);
  if (nc == 0) return fail(RINGATTR_ERR_INVALID, "N = %d exceeds the supported maximum of 2048 neurons", N);
  g.N = N;
  g.k = k;
  g.T = T;
  g.B = B;
  g.NC = nc;
  g.NPAD = 64 * nc;
  g.nbt = (B + 15) / 16;
  g.wpack_bytes = align_up((size_t)(1 + k) * g.NPAD * g.NPAD * 2);
  g.side_bytes = align_up((size_t)T * g.nbt * 16 * g.NPAD * 2);
  g.pair_bytes = align_up((size_t)((T + 1) / 2) * 2 * g.nbt * 16 * g.NPAD * 2);
  const int NT = 4 * nc, TJ = nc == 1 ? 4 : 8;
  const long per_z = (long)(NT / 2) * (NT / TJ) * ((k + 3) / 3);  // wave work items per K split
  const long nchunk = (long)g.nbt * ((T + 1) / 2);
  if (nchunk > 0x7fffffffL) return fail(RINGATTR_ERR_INVALID, "batch_size * seq_len is too large");
  long nz = (2048 + per_z - 1) / per_z;
  if (nz > 128) nz = 128;
  if (nz > nchunk) nz = nchunk;
  if (nz < 1) nz = 1;
  g.nz = ring_dw_tiled_applicable(nc) ? ring_dw_tiled_nz(nc, k, nchunk) : (int)nz;
  g.partial_bytes = align_up((size_t)g.nz * (1 + k) * g.NPAD * g.NPAD * 4);
  g.carry_bytes = nc >= 4 ? align_up(ring_wide_carry_bytes(nc, g.nbt)) : 0;   // (small; sized whichever family runs)
  g.trig_bytes = nc >= 4 ? align_up((size_t)g.NPAD * 2 * sizeof(float)) : 0;
  return RINGATTR_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_act(int a) {
  if (a < 0 || a > 3) return fail(RINGATTR_ERR_INVALID, "activation_type %d is not one of 0 relu, 1 gelu, 2 tanh, 3 silu", a);
  return RINGATTR_OK;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(RINGATTR_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

// What a forward left in a saved buffer.  The transposed weight copy behind the saved activations has J0 and J1
// folded into Wo for the weight-resident BPTT kernel and is plain for the streaming one, and the derivative record of
// the step-per-launch family has its own layout.  The forward notes, under the buffer's address, the family, the
// shape, J0, J1 and the weight tensors' addresses it packed; a backward trusts the transposed copy in the buffer only
// if every one of them matches its own arguments, and packs its own copy otherwise (no note: another process state
// or a copied buffer; a stale note: the address was reused; RINGATTR_STREAMING / RINGATTR_BLOCK changed in between;
// other J0, J1 or weights).  A buffer must not be copied or moved between the forward and the backward that
// consumes it, and the weights must not change in between (pass saved = NULL to recompute instead).
constexpr int kSavedNotes = 256;
struct SavedNote {
  const void* ptr;
  int family;   // 1 streaming, 2 weight-resident, 3 step-per-launch
  int N, k, T, B;
  float J0, J1;
  const void *Wo, *Wa;
};
std::mutex g_saved_mu;
SavedNote g_saved_notes[kSavedNotes] = {};
int g_saved_next = 0;

void saved_note_put(const SavedNote& note) {
  std::lock_guard<std::mutex> lk(g_saved_mu);
  for (auto& n : g_saved_notes)
    if (n.ptr == note.ptr) { n = note; return; }
  g_saved_notes[g_saved_next] = note;
  g_saved_next = (g_saved_next + 1) % kSavedNotes;
}

// The note under ptr (family 0 if there is none).
SavedNote saved_note_get(const void* ptr) {
  std::lock_guard<std::mutex> lk(g_saved_mu);
  for (const auto& n : g_saved_notes)
    if (n.ptr == ptr) return n;
  return SavedNote{};
}

bool saved_note_matches(const SavedNote& n, int family, int N, int k, int T, int B, float J0, float J1, const void* Wo,
                        const void* Wa) {
  return n.family == family && n.N == N && n.k == k && n.T == T && n.B == B && n.J0 == J0 && n.J1 == J1 && n.Wo == Wo &&
         n.Wa == Wa;
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

int noalloc_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(RINGATTR_ERR_INVALID, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!p) return fail(RINGATTR_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return RINGATTR_OK;
}

}  // namespace

extern "C" {

int ringattr_version(void) { return 1001; }

const char* ringattr_last_error(void) { return g_err; }

size_t ringattr_saved_bytes(int N, int a_dim, int seq_len, int batch_size) {
  Geo g;
  if (make_geo(N, a_dim, seq_len, batch_size, g) != RINGATTR_OK) return 0;
  return g.side_bytes + g.pair_bytes + g.wpack_bytes;
}

size_t ringattr_fwd_workspace_bytes(int N, int a_dim, int seq_len, int batch_size) {
  Geo g;
  if (make_geo(N, a_dim, seq_len, batch_size, g) != RINGATTR_OK) return 0;
  // (the cluster forward's exchange area is asked for wherever its shape applies, switched on or not)
  return g.wpack_bytes + (ring_cluster_applicable(N, a_dim) ? ring_cluster_workspace_bytes(g.nbt) : 0);
}

size_t ringattr_bwd_workspace_bytes(int N, int a_dim, int seq_len, int batch_size, int have_saved) {
  Geo g;
  if (make_geo(N, a_dim, seq_len, batch_size, g) != RINGATTR_OK) return 0;
  size_t s = g.wpack_bytes + g.pair_bytes + g.partial_bytes + g.carry_bytes + g.trig_bytes;
  if (!have_saved) s += g.wpack_bytes + g.side_bytes + g.pair_bytes;
  // (the cluster BPTT's scratch area is asked for wherever its shape applies, switched on or not)
  if (ring_cluster_applicable(N, a_dim)) s += ring_cluster_bptt_workspace_bytes(g.nbt);
  return s;
}

// loss_stats != null: the forward kernel that can do so also leaves the loss head's per-row sums there; *stats_done
// says whether it did.
static int fwd_impl(const void* A, const void* Wa, float J0, float J1, const void* Wo, const void* r_init,
                    void* bump_history, float alpha, int N, int a_dim, int seq_len, int batch_size, int activation_type,
                    void* saved, void* workspace, size_t workspace_bytes, ring_f32x4* loss_stats, bool* stats_done,
                    void* stream);

int ringattr_fwd(const void* A, const void* Wa, float J0, float J1, const void* Wo, const void* r_init,
                 void* bump_history, float alpha, int N, int a_dim, int seq_len, int batch_size,
                 int activation_type, void* saved, void* workspace, size_t workspace_bytes, void* stream) {
  return fwd_impl(A, Wa, J0, J1, Wo, r_init, bump_history, alpha, N, a_dim, seq_len, batch_size, activation_type, saved,
                  workspace, workspace_bytes, nullptr, nullptr, stream);
}

int ringattr_fwd_loss(const void* A, const void* Wa, float J0, float J1, const void* Wo, const void* r_init,
                      void* bump_history, float alpha, int N, int a_dim, int seq_len, int batch_size, int activation_type,
                      void* saved, void* workspace, size_t workspace_bytes, const void* target_angle,
                      const void* target_amplitude, float bump_weight, void* loss_out, void* loss_workspace,
                      size_t loss_workspace_bytes, void* stream) {
  const size_t need = ringattr_loss_workspace_bytes(N, seq_len, batch_size);
  if (need == 0) return RINGATTR_ERR_INVALID;
  if (!target_angle || !loss_out) return fail(RINGATTR_ERR_INVALID, "ringattr_fwd_loss: null tensor pointer");
  if (!aligned16(loss_workspace)) return fail(RINGATTR_ERR_INVALID, "ringattr_fwd_loss: every pointer must be 16-byte aligned");
  if (!loss_workspace || loss_workspace_bytes < need)
    return fail(RINGATTR_ERR_WORKSPACE, "ringattr_fwd_loss: loss workspace of %zu bytes needed, %zu given", need,
                loss_workspace ? loss_workspace_bytes : (size_t)0);
  bool stats_done = false;
  const int rc = fwd_impl(A, Wa, J0, J1, Wo, r_init, bump_history, alpha, N, a_dim, seq_len, batch_size, activation_type,
                          saved, workspace, workspace_bytes, ring_loss_row_sums(loss_workspace), &stats_done, stream);
  if (rc) return rc;
  hipError_t e = ring_launch_loss_fwd((const float*)bump_history, (const float*)target_angle, (const float*)target_amplitude,
                                      bump_weight, (float*)loss_out, N, seq_len, batch_size, loss_workspace, stats_done,
                                      static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "loss head forward launch");
  return RINGATTR_OK;
}

static int fwd_impl(const void* A, const void* Wa, float J0, float J1, const void* Wo, const void* r_init,
                    void* bump_history, float alpha, int N, int a_dim, int seq_len, int batch_size, int activation_type,
                    void* saved, void* workspace, size_t workspace_bytes, ring_f32x4* loss_stats, bool* stats_done,
                    void* stream) {
  Geo g;
  int rc = make_geo(N, a_dim, seq_len, batch_size, g);
  if (rc) return rc;
  if ((rc = check_act(activation_type))) return rc;
  if (!A || !Wa || !Wo || !r_init || !bump_history) return fail(RINGATTR_ERR_INVALID, "ringattr_fwd: null tensor pointer");
  if (!aligned16(A) || !aligned16(Wa) || !aligned16(Wo) || !aligned16(r_init) || !aligned16(bump_history) ||
      !aligned16(saved) || !aligned16(workspace))
    return fail(RINGATTR_ERR_INVALID, "ringattr_fwd: every pointer must be 16-byte aligned");
  if (!workspace || workspace_bytes < g.wpack_bytes)
    return fail(RINGATTR_ERR_WORKSPACE, "ringattr_fwd: workspace of %zu bytes needed, %zu given", g.wpack_bytes,
                workspace ? workspace_bytes : (size_t)0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const int ce = ring_cluster_take_error())
    return fail(RINGATTR_ERR_HIP,
                "an earlier cluster forward gave up waiting for a sibling workgroup (code %d: 1 members on different "
                "XCDs, 2 members not resident together, 3 a published state never arrived) and its results are "
                "invalid; this is reported once, and the streaming kernels run N = 512 from here on",
                ce);

  // With a saved buffer the same launch also writes the transposed copy the backward will need behind the saved
  // activations.  The weight-resident kernels take Wo as J1 * Wo + J0 in both copies; the cluster forward takes it so
  // in its own copy and leaves the plain transposed one the streaming BPTT expects.
  const int resident = ring_uses_resident(N, a_dim) ? 1 : 0;
  const size_t cluster_bytes = ring_cluster_applicable(N, a_dim) ? ring_cluster_workspace_bytes(g.nbt) : 0;
  const bool cluster = !resident && ring_uses_cluster(N, a_dim, batch_size, seq_len) && !ring_uses_step_kernels(N, a_dim, g.NC, g.nbt) &&
                       workspace_bytes >= g.wpack_bytes + cluster_bytes;
  void* wpack_t = saved ? (char*)saved + g.side_bytes + g.pair_bytes : nullptr;
  const float s0 = (resident || cluster) ? J1 : 1.f, h0 = (resident || cluster) ? J0 : 0.f;
  const float s2 = resident ? J1 : 1.f, h2 = resident ? J0 : 0.f;
  hipError_t e = ring_launch_pack2((const float*)Wo, (const float*)Wa, N, a_dim, g.NC, workspace, 0,
                                   cluster ? ring_cluster_pack_order(N, batch_size, seq_len) : resident,
                                   s0, h0, wpack_t, 1, 0, s2, h2, st);
  if (e != hipSuccess) return hip_fail(e, "pack weights");
  if (saved)
    saved_note_put(SavedNote{saved, ring_uses_step_kernels(N, a_dim, g.NC, g.nbt) ? 3 : (resident ? 2 : 1), N, a_dim,
                             seq_len, batch_size, J0, J1, Wo, Wa});

  RingFwdArgs a;
  a.A = (const float*)A;
  a.Wpack = workspace;
  a.r_init = (const float*)r_init;
  a.hist = (float*)bump_history;
  a.dfrag = saved ? (_Float16*)saved : nullptr;
  a.rfrag = saved ? (__bf16*)((char*)saved + g.side_bytes) : nullptr;
  a.J0 = J0;
  a.J1 = J1;
  a.alpha = alpha;
  a.N = N;
  a.k = a_dim;
  a.T = seq_len;
  a.B = batch_size;
  a.nbt = g.nbt;
  a.act = activation_type;
  a.cluster_ws = cluster ? (char*)workspace + g.wpack_bytes : nullptr;
  // the persistent forward kernels form the loss head's row sums themselves
  a.loss_stats = ring_fwd_forms_loss_sums(a, g.NC) ? loss_stats : nullptr;
  if (stats_done) *stats_done = a.loss_stats != nullptr;
  e = ring_launch_fwd(a, g.NC, st);
  if (e != hipSuccess) return hip_fail(e, "forward launch");
  return RINGATTR_OK;
}

int ringattr_fwd_noalloc(const void* A, const void* Wa, float J0, float J1, const void* Wo, const void* r_init,
                         void* bump_history, float alpha, int N, int a_dim, int seq_len, int batch_size,
                         int activation_type, void* saved, void* stream) {
  Geo g;
  int rc = make_geo(N, a_dim, seq_len, batch_size, g);
  if (rc) return rc;
  if (g.wpack_bytes > (size_t)RINGATTR_NOALLOC_SCRATCH_BYTES)
    return fail(RINGATTR_ERR_WORKSPACE,
                "ringattr_fwd_noalloc: N = %d with a_dim = %d needs %zu bytes of packed weights, the built-in scratch "
                "holds %zu; use ringattr_fwd with a caller workspace",
                N, a_dim, g.wpack_bytes, (size_t)RINGATTR_NOALLOC_SCRATCH_BYTES);
  if ((rc = check_act(activation_type))) return rc;
  if (!A || !Wa || !Wo || !r_init || !bump_history)
    return fail(RINGATTR_ERR_INVALID, "ringattr_fwd_noalloc: null tensor pointer");
  void* ws = nullptr;
  if ((rc = noalloc_scratch(&ws))) return rc;
  // Every byte of the packed-weight area this call reads is rewritten by its own packing launch, so nothing of an
  // earlier call's contents survives into the result; calls that overlap on one GPU would race on the array.
  return ringattr_fwd(A, Wa, J0, J1, Wo, r_init, bump_history, alpha, N, a_dim, seq_len, batch_size, activation_type,
                      saved, ws, (size_t)RINGATTR_NOALLOC_SCRATCH_BYTES, stream);
}

// grad_output != null: plain backward.  Otherwise loss_workspace (filled by ringattr_loss_fwd) describes grad_output.
static int bwd_impl(const char* who, const void* grad_output, const void* loss_workspace, const void* upstream, const void* A,
                    const void* Wa, float J0, float J1, const void* Wo, const void* bump_history, const void* r_init,
                    void* grad_Wa, void* grad_Wo, float alpha, int N, int a_dim, int seq_len, int batch_size,
                    int activation_type, int accumulate, const void* saved, void* grad_A, void* grad_r_init,
                    void* workspace, size_t workspace_bytes, void* stream);

int ringattr_bwd(const void* grad_output, const void* A, const void* Wa, float J0, float J1, const void* Wo,
                 const void* bump_history, const void* r_init, void* grad_Wa, void* grad_Wo, float alpha, int N,
                 int a_dim, int seq_len, int batch_size, int activation_type, int accumulate, const void* saved,
                 void* grad_A, void* grad_r_init, void* workspace, size_t workspace_bytes, void* stream) {
  if (!grad_output) return fail(RINGATTR_ERR_INVALID, "ringattr_bwd: null tensor pointer");
  return bwd_impl("ringattr_bwd", grad_output, nullptr, nullptr, A, Wa, J0, J1, Wo, bump_history, r_init, grad_Wa, grad_Wo,
                  alpha, N, a_dim, seq_len, batch_size, activation_type, accumulate, saved, grad_A, grad_r_init, workspace,
                  workspace_bytes, stream);
}

int ringattr_bwd_loss(const void* loss_workspace, const void* upstream, const void* A, const void* Wa, float J0, float J1,
                      const void* Wo, const void* bump_history, const void* r_init, void* grad_Wa, void* grad_Wo,
                      float alpha, int N, int a_dim, int seq_len, int batch_size, int activation_type, int accumulate,
                      const void* saved, void* grad_A, void* grad_r_init, void* workspace, size_t workspace_bytes,
                      void* stream) {
  if (!loss_workspace) return fail(RINGATTR_ERR_INVALID, "ringattr_bwd_loss: null loss workspace");
  if (!aligned16(loss_workspace)) return fail(RINGATTR_ERR_INVALID, "ringattr_bwd_loss: every pointer must be 16-byte aligned");
  if (N > 2048) return fail(RINGATTR_ERR_INVALID, "the loss head supports N <= 2048 (got %d)", N);
  return bwd_impl("ringattr_bwd_loss", nullptr, loss_workspace, upstream, A, Wa, J0, J1, Wo, bump_history, r_init, grad_Wa,
                  grad_Wo, alpha, N, a_dim, seq_len, batch_size, activation_type, accumulate, saved, grad_A, grad_r_init,
                  workspace, workspace_bytes, stream);
}

int ringattr_bwd_loss_available(int N, int a_dim, int seq_len, int batch_size) {
  Geo g;
  return make_geo(N, a_dim, seq_len, batch_size, g) == RINGATTR_OK ? 1 : 0;
}

static int bwd_impl(const char* who, const void* grad_output, const void* loss_workspace, const void* upstream, const void* A,
                    const void* Wa, float J0, float J1, const void* Wo, const void* bump_history, const void* r_init,
                    void* grad_Wa, void* grad_Wo, float alpha, int N, int a_dim, int seq_len, int batch_size,
                    int activation_type, int accumulate, const void* saved, void* grad_A, void* grad_r_init,
                    void* workspace, size_t workspace_bytes, void* stream) {
  Geo g;
  int rc = make_geo(N, a_dim, seq_len, batch_size, g);
  if (rc) return rc;
  if ((rc = check_act(activation_type))) return rc;
  if (!A || !Wa || !Wo || !bump_history || !r_init || !grad_Wa || !grad_Wo)
    return fail(RINGATTR_ERR_INVALID, "%s: null tensor pointer", who);
  const bool step_family = ring_uses_step_kernels(N, a_dim, g.NC, g.nbt);
  // the persistent streaming BPTT kernel stages the per-channel shares of dL/dA in 24 KiB of LDS; the
  // step-per-launch families form dL/dA in a pass of their own that has no such stage
  if (grad_A && !step_family && !ring_uses_resident(N, a_dim) && (size_t)2 * a_dim * 64 * sizeof(float) > 24 * 1024)
    return fail(RINGATTR_ERR_INVALID, "%s: grad_A on the persistent streaming kernels (N <= 512 at this batch) is "
                "supported for a_dim <= 48 (got %d)", who, a_dim);
  if (step_family && grad_A && seq_len > 65535)
    return fail(RINGATTR_ERR_INVALID, "%s: grad_A on the step-per-launch kernels supports seq_len <= 65535", who);
  if (!aligned16(grad_output) || !aligned16(A) || !aligned16(Wa) || !aligned16(Wo) || !aligned16(bump_history) ||
      !aligned16(r_init) || !aligned16(grad_Wa) || !aligned16(grad_Wo) || !aligned16(saved) ||
      !aligned16(grad_r_init) || !aligned16(grad_A) || !aligned16(workspace))
    return fail(RINGATTR_ERR_INVALID, "%s: every pointer must be 16-byte aligned", who);
  const size_t need = ringattr_bwd_workspace_bytes(N, a_dim, seq_len, batch_size, saved != nullptr);
  if (!workspace || workspace_bytes < need)
    return fail(RINGATTR_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", who, need,
                workspace ? workspace_bytes : (size_t)0);
  hipStream_t st = static_cast<hipStream_t>(stream);

  char* ws = (char*)workspace;
  void* wb = ws;
  ws += g.wpack_bytes;
  __bf16* gfrag = (__bf16*)ws;
  ws += g.pair_bytes;
  ring_f32x4* partial = (ring_f32x4*)ws;
  ws += g.partial_bytes;
  float* carry = g.carry_bytes ? (float*)ws : nullptr;
  ws += g.carry_bytes;
  float* trig = g.trig_bytes ? (float*)ws : nullptr;
  ws += g.trig_bytes;

  const _Float16* dfrag;
  const __bf16* rfrag;
  if (saved) {
    dfrag = (const _Float16*)saved;
    rfrag = (const __bf16*)((const char*)saved + g.side_bytes);
  } else {
    void* wf = ws;
    ws += g.wpack_bytes;
    _Float16* d = (_Float16*)ws;
    ws += g.side_bytes;
    __bf16* r = (__bf16*)ws;
    const bool res = ring_uses_resident(N, a_dim);
    hipError_t e = ring_launch_pack((const float*)Wo, (const float*)Wa, wf, N, a_dim, g.NC, 0, res ? 1 : 0, res ? J1 : 1.f,
                                    res ? J0 : 0.f, st);
    if (e != hipSuccess) return hip_fail(e, "pack weights");
    RingFwdArgs f;
    f.A = (const float*)A;
    f.Wpack = wf;
    f.r_init = (const float*)r_init;
    f.hist = (float*)const_cast<void*>(bump_history);  // read only in the rebuild kernel
    f.dfrag = d;
    f.rfrag = r;
    f.J0 = J0;
    f.J1 = J1;
    f.alpha = alpha;
    f.N = N;
    f.k = a_dim;
    f.T = seq_len;
    f.B = batch_size;
    f.nbt = g.nbt;
    f.act = activation_type;
    e = ring_launch_rebuild(f, g.NC, st);
    if (e != hipSuccess) return hip_fail(e, "rebuild launch");
    dfrag = d;
    rfrag = r;
  }

  // The cluster BPTT (N = 512, where ring_uses_cluster_bptt says so; no dL/dA, no fused loss head) packs its own
  // transposed copy, in its column order with J1 * Wo^T + J0 as matrix 0; its scratch area is the workspace's tail.
  const bool bptt_cluster = !step_family && !grad_A && !loss_workspace && ring_uses_cluster_bptt(N, a_dim, batch_size, seq_len) &&
                            !ring_uses_resident(N, a_dim);
  void* const cluster_ws = bptt_cluster ? (char*)workspace + need - ring_cluster_bptt_workspace_bytes(g.nbt) : nullptr;
  // the weight-resident BPTT kernel takes J1 * Wo + J0 in the transposed Wo fragments
  const bool resident = ring_uses_resident(N, a_dim);
  const bool bptt_resident = resident;
  hipError_t e = hipSuccess;
  const int family = step_family ? 3 : (bptt_resident ? 2 : 1);
  const SavedNote note = saved ? saved_note_get(saved) : SavedNote{};
  const int noted = note.family;
  if (noted != 0 && (noted == 3) != (family == 3))
    return fail(RINGATTR_ERR_INVALID, "%s: the saved buffer was filled by the other kernel family (its derivative record "
                "has a different layout); run forward and backward under the same RINGATTR_BLOCK setting", who);
  if (bptt_cluster) {
    e = ring_launch_pack((const float*)Wo, (const float*)Wa, wb, N, a_dim, g.NC, 1,
                         ring_cluster_pack_order(N, batch_size, seq_len), J1, J0, st);
    if (e != hipSuccess) return hip_fail(e, "pack transposed weights");
  } else if (saved && saved_note_matches(note, family, N, a_dim, seq_len, batch_size, J0, J1, Wo, Wa)) {
    // the forward left the transposed copy, in the form this BPTT kernel expects, behind the saved activations
    wb = (char*)const_cast<void*>(saved) + g.side_bytes + g.pair_bytes;
  } else {
    e = ring_launch_pack((const float*)Wo, (const float*)Wa, wb, N, a_dim, g.NC, 1, 0, bptt_resident ? J1 : 1.f,
                         bptt_resident ? J0 : 0.f, st);
    if (e != hipSuccess) return hip_fail(e, "pack transposed weights");
  }

  RingBpttArgs b;
  b.A = (const float*)A;
  b.Wpack = wb;
  b.grad_out = (const float*)grad_output;
  b.dfrag = dfrag;
  b.gfrag = gfrag;
  b.rfrag = rfrag;
  b.grad_r_init = (float*)grad_r_init;
  b.grad_A = step_family ? nullptr : (float*)grad_A;   // the step-per-launch families take dL/dA in a pass of its own
  b.hist = (const float*)bump_history;
  b.r_init = (const float*)r_init;
  b.wide_carry = carry;
  b.loss_coef = loss_workspace ? ring_loss_row_coefficients(loss_workspace) : nullptr;
  b.loss_upstream = (const float*)upstream;
  b.loss_inv_rows = 1.f / ((float)seq_len * (float)batch_size);
  if (step_family && loss_workspace) {
    if (!trig) return fail(RINGATTR_ERR_INVALID, "%s: no room for the angle table in this geometry", who);
    e = ring_launch_trig_table(trig, N, g.NPAD, st);
    if (e != hipSuccess) return hip_fail(e, "angle table launch");
    b.loss_trig = trig;
  }
  b.J0 = J0;
  b.J1 = J1;
  b.alpha = alpha;
  b.N = N;
  b.k = a_dim;
  b.T = seq_len;
  b.B = batch_size;
  b.nbt = g.nbt;
  b.cluster_ws = cluster_ws;
  e = ring_launch_bptt(b, g.NC, st);
  if (e != hipSuccess) return hip_fail(e, "BPTT launch");
  if (step_family && grad_A) {
    // forward-orientation fragments, packed into the split-K partial area (not yet in use, and never smaller)
    e = ring_launch_pack((const float*)Wo, (const float*)Wa, partial, N, a_dim, g.NC, 0, 0, 1.f, 0.f, st);
    if (e != hipSuccess) return hip_fail(e, "pack weights");
    b.grad_A = (float*)grad_A;
    e = ring_launch_block_grad_A(b, partial, g.NC, st);
    if (e != hipSuccess) return hip_fail(e, "grad_A launch");
  }

  RingDwArgs d;
  d.A = (const float*)A;
  d.gfrag = gfrag;
  d.rfrag = rfrag;
  d.partial = partial;
  d.grad_Wo = (float*)grad_Wo;
  d.grad_Wa = (float*)grad_Wa;
  d.J1 = J1;
  d.accumulate = accumulate;
  d.N = N;
  d.k = a_dim;
  d.T = seq_len;
  d.B = batch_size;
  d.nbt = g.nbt;
  d.nz = g.nz;
  e = ring_launch_dw(d, g.NC, st);
  if (e != hipSuccess) return hip_fail(e, "weight-gradient launch");
  return RINGATTR_OK;
}

size_t ringattr_loss_workspace_bytes(int N, int seq_len, int batch_size) {
  if (N <= 0 || seq_len <= 0 || batch_size <= 0) {
    fail(RINGATTR_ERR_INVALID, "N, seq_len, batch_size must be positive (got %d, %d, %d)", N, seq_len, batch_size);
    return 0;
  }
  if (N > 2048) {
    fail(RINGATTR_ERR_INVALID, "the loss head supports N <= 2048 (got %d)", N);
    return 0;
  }
  return align_up(ring_loss_workspace_bytes(seq_len, batch_size));
}

int ringattr_loss_fwd(const void* bump_history, const void* target_angle, const void* target_amplitude, float bump_weight,
                      void* loss_out, int N, int seq_len, int batch_size, void* workspace, size_t workspace_bytes,
                      void* stream) {
  const size_t need = ringattr_loss_workspace_bytes(N, seq_len, batch_size);
  if (need == 0) return RINGATTR_ERR_INVALID;
  if (!bump_history || !target_angle || !loss_out) return fail(RINGATTR_ERR_INVALID, "ringattr_loss_fwd: null tensor pointer");
  if (!aligned16(bump_history) || !aligned16(workspace))
    return fail(RINGATTR_ERR_INVALID, "ringattr_loss_fwd: bump_history and workspace must be 16-byte aligned");
  if (!workspace || workspace_bytes < need)
    return fail(RINGATTR_ERR_WORKSPACE, "ringattr_loss_fwd: workspace of %zu bytes needed, %zu given", need,
                workspace ? workspace_bytes : (size_t)0);
  hipError_t e = ring_launch_loss_fwd((const float*)bump_history, (const float*)target_angle, (const float*)target_amplitude,
                                      bump_weight, (float*)loss_out, N, seq_len, batch_size, workspace, false,
                                      static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "loss head forward launch");
  return RINGATTR_OK;
}

int ringattr_loss_bwd(const void* bump_history, const void* target_angle, const void* target_amplitude, float bump_weight,
                      const void* upstream, void* grad_history, int N, int seq_len, int batch_size, const void* workspace,
                      size_t workspace_bytes, void* stream) {
  const size_t need = ringattr_loss_workspace_bytes(N, seq_len, batch_size);
  if (need == 0) return RINGATTR_ERR_INVALID;
  if (!bump_history || !target_angle || !grad_history)
    return fail(RINGATTR_ERR_INVALID, "ringattr_loss_bwd: null tensor pointer");
  if (!aligned16(bump_history) || !aligned16(grad_history) || !aligned16(workspace))
    return fail(RINGATTR_ERR_INVALID, "ringattr_loss_bwd: bump_history, grad_history and workspace must be 16-byte aligned");
  if (!workspace || workspace_bytes < need)
    return fail(RINGATTR_ERR_WORKSPACE, "ringattr_loss_bwd: workspace of %zu bytes needed, %zu given", need,
                workspace ? workspace_bytes : (size_t)0);
  hipError_t e = ring_launch_loss_bwd((const float*)bump_history, (const float*)target_angle, (const float*)target_amplitude,
                                      bump_weight, (const float*)upstream, (float*)grad_history, N, seq_len, batch_size,
                                      workspace, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "loss head backward launch");
  return RINGATTR_OK;
}

size_t ringattr_gain_workspace_bytes(int a_dim, int hidden, int seq_len, int batch_size) {
  if (a_dim <= 0 || hidden <= 0 || seq_len <= 0 || batch_size <= 0) {
    fail(RINGATTR_ERR_INVALID, "a_dim, hidden, seq_len, batch_size must be positive (got %d, %d, %d, %d)", a_dim, hidden,
         seq_len, batch_size);
    return 0;
  }
  if (hidden > 32 || a_dim > 64) {
    fail(RINGATTR_ERR_INVALID, "the gain networks support hidden <= 32 and a_dim <= 64 (got %d, %d)", hidden, a_dim);
    return 0;
  }
  return align_up(ring_gain_workspace_bytes(a_dim, hidden, (long)seq_len * batch_size));
}

int ringattr_gain_fwd(const void* base_signal, const void* params, void* action_signal, int a_dim, int hidden, int seq_len,
                      int batch_size, void* stream) {
  if (ringattr_gain_workspace_bytes(a_dim, hidden, seq_len, batch_size) == 0) return RINGATTR_ERR_INVALID;
  if (!base_signal || !params || !action_signal) return fail(RINGATTR_ERR_INVALID, "ringattr_gain_fwd: null tensor pointer");
  hipError_t e = ring_launch_gain_fwd((const float*)base_signal, (const float*)params, (float*)action_signal, a_dim, hidden,
                                      (long)seq_len * batch_size, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "gain network forward launch");
  return RINGATTR_OK;
}

int ringattr_gain_bwd(const void* base_signal, const void* params, const void* grad_action_signal, void* grad_params,
                      void* grad_base_signal, int a_dim, int hidden, int seq_len, int batch_size, void* workspace,
                      size_t workspace_bytes, void* stream) {
  const size_t need = ringattr_gain_workspace_bytes(a_dim, hidden, seq_len, batch_size);
  if (need == 0) return RINGATTR_ERR_INVALID;
  if (!base_signal || !params || !grad_action_signal || !grad_params)
    return fail(RINGATTR_ERR_INVALID, "ringattr_gain_bwd: null tensor pointer");
  if (!workspace || workspace_bytes < need)
    return fail(RINGATTR_ERR_WORKSPACE, "ringattr_gain_bwd: workspace of %zu bytes needed, %zu given", need,
                workspace ? workspace_bytes : (size_t)0);
  hipError_t e = ring_launch_gain_bwd((const float*)base_signal, (const float*)params, (const float*)grad_action_signal,
                                      (float*)grad_params, (float*)grad_base_signal, a_dim, hidden,
                                      (long)seq_len * batch_size, workspace, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "gain network backward launch");
  return RINGATTR_OK;
}

int ringattr_generator_initial_zeros(int seq_len, double zero_padding_start_ratio) {
  // int(seq_len * ratio) with the product in double precision, as Python evaluates it
  // (utils/generate_av_integration_data.py:21); a float product differs by one for some (length, ratio) pairs
  if (seq_len <= 0 || !(zero_padding_start_ratio >= 0.0 && zero_padding_start_ratio <= 1.0)) return -1;
  return (int)((double)seq_len * zero_padding_start_ratio);
}

int ringattr_generate_inputs(unsigned long long seed, int N, int a_dim, int seq_len, int batch_size,
                             double zero_padding_start_ratio, const float* zero_ratios, int n_zero_ratios, float max_av,
                             int spread_action, int bump_kind, float bump_param, void* av, void* angle,
                             void* action_signal, void* r_init, void* stream) {
  if (N <= 0 || a_dim <= 0 || seq_len <= 0 || batch_size <= 0)
    return fail(RINGATTR_ERR_INVALID, "N, a_dim, seq_len, batch_size must be positive (got %d, %d, %d, %d)", N, a_dim,
                seq_len, batch_size);
  if (!zero_ratios || n_zero_ratios < 1 || n_zero_ratios > 8)
    return fail(RINGATTR_ERR_INVALID, "ringattr_generate_inputs: between 1 and 8 zero ratios (host array) are needed");
  if (!(zero_padding_start_ratio >= 0.0 && zero_padding_start_ratio <= 1.0))
    return fail(RINGATTR_ERR_INVALID, "ringattr_generate_inputs: zero_padding_start_ratio must lie in [0, 1]");
  if ((bump_kind != 0 && bump_kind != 1) || !(bump_param > 0.f))
    return fail(RINGATTR_ERR_INVALID, "ringattr_generate_inputs: bump_kind is 0 (Gaussian) or 1 (von Mises), bump_param > 0");
  if (!av || !angle || !action_signal) return fail(RINGATTR_ERR_INVALID, "ringattr_generate_inputs: null tensor pointer");
  RingGenArgs a;
  a.seed = seed;
  a.av = (float*)av;
  a.angle = (float*)angle;
  a.action = (float*)action_signal;
  a.r_init = (float*)r_init;
  for (int i = 0; i < 8; ++i) a.ratios[i] = i < n_zero_ratios ? zero_ratios[i] : 0.f;
  a.n_ratios = n_zero_ratios;
  a.n_initial_zeros = ringattr_generator_initial_zeros(seq_len, zero_padding_start_ratio);
  a.max_av = max_av;
  a.bump_param = bump_param;
  a.spread = spread_action ? 1 : 0;
  a.bump_kind = bump_kind;
  a.N = N;
  a.k = a_dim;
  a.T = seq_len;
  a.B = batch_size;
  hipError_t e = ring_launch_generate(a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "input generator launch");
  return RINGATTR_OK;
}

size_t ringattr_clip_adam_workspace_bytes(int n_tensors, const size_t* numel) {
  if (n_tensors < 1 || n_tensors > RING_OPT_MAX_TENSORS || !numel) {
    fail(RINGATTR_ERR_INVALID, "between 1 and %d tensors are supported (got %d)", RING_OPT_MAX_TENSORS, n_tensors);
    return 0;
  }
  size_t chunks = 0;
  for (int i = 0; i < n_tensors; ++i) chunks += (size_t)ring_opt_chunks(numel[i]);
  return align_up((chunks + 3) * sizeof(float));
}

// step_counter != null: the step number lives on the device (ringattr_clip_adam_counted); otherwise `step` is it.
static int clip_adam_impl(int n_tensors, void* const* params, void* const* grads, void* const* exp_avg,
                          void* const* exp_avg_sq, const size_t* numel, float lr, float beta1, float beta2, float eps,
                          float max_norm, int step, void* step_counter, void* workspace, size_t workspace_bytes,
                          void* stream);

int ringattr_clip_adam(int n_tensors, void* const* params, void* const* grads, void* const* exp_avg,
                       void* const* exp_avg_sq, const size_t* numel, float lr, float beta1, float beta2, float eps,
                       float max_norm, int step, void* workspace, size_t workspace_bytes, void* stream) {
  if (step < 1) return fail(RINGATTR_ERR_INVALID, "ringattr_clip_adam: step counts from 1 (got %d)", step);
  return clip_adam_impl(n_tensors, params, grads, exp_avg, exp_avg_sq, numel, lr, beta1, beta2, eps, max_norm, step,
                        nullptr, workspace, workspace_bytes, stream);
}

int ringattr_clip_adam_counted(int n_tensors, void* const* params, void* const* grads, void* const* exp_avg,
                               void* const* exp_avg_sq, const size_t* numel, float lr, float beta1, float beta2,
                               float eps, float max_norm, void* step_counter, void* workspace, size_t workspace_bytes,
                               void* stream) {
  if (!step_counter || (reinterpret_cast<uintptr_t>(step_counter) & 3))
    return fail(RINGATTR_ERR_INVALID, "ringattr_clip_adam_counted: the step counter must be a 4-byte aligned device pointer");
  return clip_adam_impl(n_tensors, params, grads, exp_avg, exp_avg_sq, numel, lr, beta1, beta2, eps, max_norm, 1,
                        step_counter, workspace, workspace_bytes, stream);
}

static int clip_adam_impl(int n_tensors, void* const* params, void* const* grads, void* const* exp_avg,
                          void* const* exp_avg_sq, const size_t* numel, float lr, float beta1, float beta2, float eps,
                          float max_norm, int step, void* step_counter, void* workspace, size_t workspace_bytes,
                          void* stream) {
  const size_t need = ringattr_clip_adam_workspace_bytes(n_tensors, numel);
  if (need == 0) return RINGATTR_ERR_INVALID;
  if (!params || !grads || !exp_avg || !exp_avg_sq) return fail(RINGATTR_ERR_INVALID, "ringattr_clip_adam: null pointer list");
  if (!workspace || workspace_bytes < need)
    return fail(RINGATTR_ERR_WORKSPACE, "ringattr_clip_adam: workspace of %zu bytes needed, %zu given", need,
                workspace ? workspace_bytes : (size_t)0);
  RingOptArgs a;
  memset(&a, 0, sizeof(a));
  for (int i = 0; i < n_tensors; ++i) {
    if (!params[i] || !grads[i] || !exp_avg[i] || !exp_avg_sq[i] || numel[i] == 0)
      return fail(RINGATTR_ERR_INVALID, "ringattr_clip_adam: tensor %d has a null pointer or no elements", i);
    a.param[i] = (float*)params[i];
    a.grad[i] = (float*)grads[i];
    a.exp_avg[i] = (float*)exp_avg[i];
    a.exp_avg_sq[i] = (float*)exp_avg_sq[i];
    a.numel[i] = numel[i];
    a.chunks[i] = ring_opt_chunks(numel[i]);
  }
  a.n = n_tensors;
  a.beta1 = beta1;
  a.beta2 = beta2;
  a.eps = eps;
  a.max_norm = max_norm;
  a.step_size = (float)((double)lr / (1.0 - pow((double)beta1, (double)step)));
  a.inv_sqrt_bc2 = (float)(1.0 / sqrt(1.0 - pow((double)beta2, (double)step)));
  a.step_counter = (int*)step_counter;
  a.lr = lr;
  hipError_t e = ring_launch_clip_adam(a, (float*)workspace, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "clip + Adam launch");
  return RINGATTR_OK;
}

int ringattr_profile_enable(int on) {
  ring_profile_set(on);
  return RINGATTR_OK;
}

int ringattr_dw_segments(int N, int a_dim, int seq_len, int batch_size) {
  Geo g;
  if (make_geo(N, a_dim, seq_len, batch_size, g) != RINGATTR_OK) return -1;
  return ring_dw_tiled_applicable(g.NC) ? ring_dw_tiled_segments(g.nbt, seq_len, g.nz) : 1;
}

int ringattr_last_kernel_name(int kernel, char* buf, size_t buf_bytes) {
  if (!buf || buf_bytes == 0) return fail(RINGATTR_ERR_INVALID, "ringattr_last_kernel_name: null buffer");
  if (kernel < 0 || kernel >= RINGATTR_NUM_KERNELS) return fail(RINGATTR_ERR_INVALID, "ringattr_last_kernel_name: no such kernel slot");
  if (ring_last_kernel_name(kernel, buf, buf_bytes) < 0) return fail(RINGATTR_ERR_HIP, "ringattr_last_kernel_name: the runtime does not know the kernel");
  return RINGATTR_OK;
}

int ringattr_profile_read(double* ms, long long* launches) {
  if (!ms || !launches) return fail(RINGATTR_ERR_INVALID, "ringattr_profile_read: null output array");
  hipError_t e = ring_profile_collect(ms, launches);
  if (e != hipSuccess) return hip_fail(e, "profile events");
  return RINGATTR_OK;
}

void fwd_cuda(void* A, void* Wa, float J0, float J1, void* Wo, void* r_init, void* bump_history, float alpha, int N,
              int a_dim, int seq_len, int batch_size, int activation_type) {
  const size_t need = ringattr_fwd_workspace_bytes(N, a_dim, seq_len, batch_size);
  void* ws = nullptr;
  if (need == 0 || hipMalloc(&ws, need) != hipSuccess) {
    fprintf(stderr, "fwd_cuda: %s\n", need ? "workspace allocation failed" : ringattr_last_error());
    return;
  }
  if (ringattr_fwd(A, Wa, J0, J1, Wo, r_init, bump_history, alpha, N, a_dim, seq_len, batch_size, activation_type,
                   nullptr, ws, need, nullptr) != RINGATTR_OK)
    fprintf(stderr, "fwd_cuda: %s\n", ringattr_last_error());
  (void)hipStreamSynchronize(nullptr);
  (void)hipFree(ws);
}

void bwd_cuda(void* grad_output, void* A, void* Wa, float J0, float J1, void* Wo, void* bump_history,
              void* re_history, void* r_init, void* grad_Wa, void* grad_Wo, float alpha, int N, int a_dim,
              int seq_len, int batch_size, int activation_type, void* grad_r, void* W_eff_temp, void* grad_re_temp,
              void* grad_W_eff_temp_bf16, void* A_t_temp_bf16, void* grad_re_temp_T, void* cublas_handle) {
  (void)re_history;
  (void)grad_r;
  (void)W_eff_temp;
  (void)grad_re_temp;
  (void)grad_W_eff_temp_bf16;
  (void)A_t_temp_bf16;
  (void)grad_re_temp_T;
  (void)cublas_handle;
  const size_t need = ringattr_bwd_workspace_bytes(N, a_dim, seq_len, batch_size, 0);
  void* ws = nullptr;
  if (need == 0 || hipMalloc(&ws, need) != hipSuccess) {
    fprintf(stderr, "bwd_cuda: %s\n", need ? "workspace allocation failed" : ringattr_last_error());
    return;
  }
  if (ringattr_bwd(grad_output, A, Wa, J0, J1, Wo, bump_history, r_init, grad_Wa, grad_Wo, alpha, N, a_dim, seq_len,
                   batch_size, activation_type, /*accumulate=*/1, nullptr, nullptr, nullptr, ws, need, nullptr) != RINGATTR_OK)
    fprintf(stderr, "bwd_cuda: %s\n", ringattr_last_error());
  (void)hipStreamSynchronize(nullptr);
  (void)hipFree(ws);
}

}  // extern "C"
