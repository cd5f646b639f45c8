// Kernels for wide rings: 512 < N <= 2048 (NC = NPAD / 64 in {16, 24, 32}).
//
// The persistent kernels keep a batch tile's whole state and all (1 + a_dim) products of a step in one workgroup's
// registers and LDS; past N = 512 neither fits.  Here a time step is one launch (the host loops over t, as the
// reference does for every N: cpp/kernels/fwd_1loop_tc_idx.cuh:265-277, bwd_mixed_precision_aggressive.cuh:563-672)
// and the output neurons of a batch tile are split over workgroups: workgroup (bt, cb) owns batch rows 16*bt..+15
// and the 16 column tiles 16*cb..16*cb+15 (256 neurons), wave v of it tiles 16*cb + 4*v .. +3.  Every workgroup
// stages the tile's full operand row block (r_prev or g, all NPAD neurons, bf16) in LDS, streams its 256-column
// slice of each packed weight matrix from L2 once, and contracts over the whole ring with MFMA.  At these widths a
// step is 20 us and more, so the launch per step is noise, and the state travels between steps through the history
// tensor (forward) or a small fp32 carry buffer (BPTT), both L2 resident.
//
// Layouts are the common ones with NC as a run-time number: weights [mm][tile][kc][lane][8] (ring_pack_weights_kernel),
// operand copies for the weight-gradient kernel in paired tile order (pair_offset).  The saved derivative record is
// private to this family: row-major fp16 [t][16*nbt][NPAD].
#include "ring_step_common.hpp"

namespace {

constexpr int BN_KG = 4;   // K chunks per weight prefetch group

// acc[cl][e] += sum_mm coef_mm[e] * (X @ W_mm)[row 4q+e][tile tg0 + cl], X from the LDS operand buffer (all KCH chunks),
// W_mm streamed from the packed global copy.  coef_0 = J1, coef_{1+c} = gate of channel c; channels whose gate is
// zero in all 16 rows are skipped when the gates are staged (a_dim <= BN_GATE_KMAX).
// TPW: column tiles per wave (a workgroup owns 4 * TPW tiles).
template <int TPW>
__device__ __forceinline__ void wide_products(const bf16x8* xb, const bf16x8* __restrict__ Wp, const float* __restrict__ A,
                                              const float* gl, bool staged, int k, int T, int B, int t, int b0, float J1,
                                              int NC, int tg0, int lane, f32x4 (&acc)[TPW]) {
  const int KCH = 2 * NC, q = lane >> 4, n = lane & 15;
  const unsigned long long active = staged ? active_channels(gl, k, lane) : ~0ull;
  // next matrix worth multiplying after mm (matrix 1 + c is gated by channel c), or -1
  auto next_matrix = [&](int mm) {
    if (!staged) return mm < k ? mm + 1 : -1;
    const unsigned long long rest = mm >= 64 ? 0ull : (active >> mm);
    const int nx = rest ? mm + 1 + (int)__builtin_ctzll(rest) : -1;
    return nx <= k ? nx : -1;
  };
  // tile tg0 + cl, chunk kc of matrix mm: fragment ((mm * 4NC + tile) * KCH + kc) * 64 + lane
  auto matrix_ptr = [&](int mm) { return Wp + ((size_t)mm * 4 * NC + tg0) * KCH * 64 + lane; };
  // The weights of a step are one stream: the prefetch runs one group of BN_KG chunks ahead and straight across
  // matrix boundaries, so the pipeline fills once per step, not once per matrix.  (KCH / BN_KG is even, so every
  // matrix starts in register buffer 0.)
  bf16x8 wf[2][BN_KG][TPW];
  {
    const bf16x8* w0 = matrix_ptr(0);
#pragma unroll
    for (int u = 0; u < BN_KG; ++u)
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) wf[0][u][cl] = w0[((size_t)cl * KCH + u) * 64];
  }
  const int ngroups = KCH / BN_KG;         // KCH = 2 NC is a multiple of 8
  for (int mm = 0; mm >= 0;) {
    const int nxt = next_matrix(mm);
    float coef[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (mm == 0) coef[e] = J1;
      else if (staged) coef[e] = gl[(4 * q + e) * BN_GATE_KMAX + (mm - 1)];
      else coef[e] = (b0 + e < B) ? A[((size_t)(b0 + e) * T + t) * k + (mm - 1)] : 0.f;
    }
    f32x4 p[TPW];
#pragma unroll
    for (int cl = 0; cl < TPW; ++cl) p[cl] = f32x4{0.f, 0.f, 0.f, 0.f};
    const bf16x8* wm = matrix_ptr(mm);
    const bf16x8* wn = matrix_ptr(nxt >= 0 ? nxt : mm);   // past the last matrix: a re-read, unused
    for (int g2 = 0; g2 < ngroups; g2 += 2) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int g = g2 + half;
        const bf16x8* src = g + 1 < ngroups ? wm + (size_t)(g + 1) * BN_KG * 64 : wn;
#pragma unroll
        for (int u = 0; u < BN_KG; ++u)
#pragma unroll
          for (int cl = 0; cl < TPW; ++cl) wf[half ^ 1][u][cl] = src[((size_t)cl * KCH + u) * 64];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < BN_KG; ++u) {
          const bf16x8 af = xb[((g * BN_KG + u) * 4 + q) * XG + n];
#pragma unroll
          for (int cl = 0; cl < TPW; ++cl) p[cl] = mfma16(af, wf[half][u][cl], p[cl]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int cl = 0; cl < TPW; ++cl)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[cl][e] = fmaf(coef[e], p[cl][e], acc[cl][e]);
    mm = nxt;
  }
}

}  // namespace

// One forward step (REBUILD = false: r_prev from r_init / hist[t-1], writes hist[t]) or the recomputation of the saved
// record of every step at once from an existing history (REBUILD = true: grid.z = T, hist is only read).
// TPW column tiles per wave: a workgroup owns 64 * TPW neurons.  Wide rings use 4; narrower rings with few batch
// tiles use fewer so that the step still spreads over the device (forward without saved record only).
template <int ACT, bool REBUILD, int TPW>
__global__ __launch_bounds__(256) void ring_wide_fwd_kernel(RingFwdArgs p, int NC, int t_arg, int xcd_map) {
  extern __shared__ __attribute__((aligned(16))) char wide_lds[];
  bf16x8* xb = reinterpret_cast<bf16x8*>(wide_lds);
  __shared__ float rs[16];
  __shared__ float gl[16 * BN_GATE_KMAX];
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  int bt, cb;
  step_block_coords(xcd_map, bt, cb);
  const int t = REBUILD ? (int)blockIdx.z : t_arg;
  const int N = p.N, B = p.B, T = p.T, NPAD = 64 * NC;
  const bool staged = p.k <= BN_GATE_KMAX;
  const float* prev = (t == 0) ? p.r_init : p.hist + (size_t)(t - 1) * B * N;

  stage_rows(xb, rs, NPAD, tid, [&](int row, int j) { return load4_masked(prev, N, B, 16 * bt + row, j); });
  if (staged) stage_gates(gl, p.A, p.k, T, B, t, bt, tid);
  lds_barrier();

  const int tg0 = 4 * TPW * cb + TPW * wv;                // this wave's first column tile
  const int wg = tg0 / NC, c0 = tg0 % NC;                 // common tile order: tile = wg * NC + c
  const int j0 = 16 * NC * wg + NC * n + c0;              // the lane's TPW consecutive neurons
  const int b0 = 16 * bt + 4 * q;
  f32x4 acc[TPW];
#pragma unroll
  for (int cl = 0; cl < TPW; ++cl) acc[cl] = f32x4{0.f, 0.f, 0.f, 0.f};
  wide_products<TPW>(xb, (const bf16x8*)p.Wpack, p.A, gl, staged, p.k, T, B, t, b0, p.J1, NC, tg0, lane, acc);

  const float oma = 1.f - p.alpha;
  const size_t rows_pad = (size_t)16 * p.nbt;
  bf16x4 rcopy[TPW], ncopy[TPW];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int b = b0 + e;
    const f32x4 rp = loadv_masked<TPW>(prev, N, B, b, j0);
    const float js = p.J0 * rs[4 * q + e];
    f32x4 rn = {0.f, 0.f, 0.f, 0.f}, dd = rn;
#pragma unroll
    for (int cl = 0; cl < TPW; ++cl) {
      float F, D;
      act_fast<ACT>(acc[cl][e] + js, F, D);
      const bool ok = b < B && j0 + cl < N;
      rn[cl] = ok ? fmaf(p.alpha, F, oma * rp[cl]) : 0.f;
      dd[cl] = ok ? p.alpha * D : 0.f;
      rcopy[cl][e] = (__bf16)rp[cl];
      ncopy[cl][e] = (__bf16)rn[cl];
    }
    if constexpr (REBUILD) {   // the copy is of the history as given, not of the state recomputed here
      const f32x4 rh = loadv_masked<TPW>(p.hist + (size_t)t * B * N, N, B, b, j0);
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) ncopy[cl][e] = (__bf16)rh[cl];
    }
    if (!REBUILD) storev_masked<TPW>(p.hist + (size_t)t * B * N, N, B, b, j0, rn);
    if (p.dfrag) {
      _Float16* dst = p.dfrag + ((size_t)t * rows_pad + 16 * bt + 4 * q + e) * NPAD + j0;
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) dst[cl] = (_Float16)dd[cl];
    }
  }
  if (p.rfrag && (t & 1) == 0) {
    // bf16 copies of the operands of this step and the next (r_prev and the new r) for the weight-gradient kernel:
    // the paired buffer holds steps 2j and 2j+1 in one 16-byte slot, and an even step has both halves in registers,
    // so they leave as one store (odd steps write none); past an odd sequence's last step the second half is zero
    const bool tail = t + 1 == T;
#pragma unroll
    for (int cl = 0; cl < TPW; ++cl) {
      const bf16x4 hi = tail ? bf16x4{(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f} : ncopy[cl];
      *reinterpret_cast<bf16x8*>(p.rfrag + pair_off_rt(NC, t, p.nbt, bt, tg0 + cl, lane)) =
          __builtin_shufflevector(rcopy[cl], hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }
}

// One BPTT step t: G = grad_output[t] + carry_in, g = (alpha F') * G (operand, all neurons, every workgroup of the batch
// tile), carry_out = (1-alpha) G + J0 sum(g) + J1 (g Wo) + sum_c A_c (g Wa_c) for the workgroup's own 256 neurons.
// carry_in == nullptr at the last time step (zero carry); at t == 0 the host points carry_out at grad_r_init or scratch.
template <bool LOSS>
__global__ __launch_bounds__(256) void ring_wide_bptt_kernel(RingBpttArgs p, int NC, int t, const float* carry_in,
                                                             float* carry_out, int xcd_map) {
  extern __shared__ __attribute__((aligned(16))) char wide_lds[];
  bf16x8* xb = reinterpret_cast<bf16x8*>(wide_lds);
  __shared__ float rs[16];
  __shared__ float gl[16 * BN_GATE_KMAX];
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  int bt, cb;
  step_block_coords(xcd_map, bt, cb);
  const int N = p.N, B = p.B, T = p.T, NPAD = 64 * NC;
  const bool staged = p.k <= BN_GATE_KMAX;
  const size_t rows_pad = (size_t)16 * p.nbt;
  const float* gout = LOSS ? nullptr : p.grad_out + (size_t)t * B * N;
  const _Float16* drow = p.dfrag + (size_t)t * rows_pad * NPAD;
  // LOSS: grad_output is not read; it is formed from the state history and the loss head's row coefficients
  const float up = LOSS ? (p.loss_upstream ? p.loss_upstream[0] : 1.f) * p.loss_inv_rows : 0.f;

  // g of (row, j..j+3): carry rows live in a padded [16*nbt][NPAD] buffer
  auto g4 = [&](int row, int j, f32x4& G) {
    const int b = 16 * bt + row;
    if constexpr (LOSS) G = loss_grad4(p, t, b, j, up);
    else G = load4_masked(gout, N, B, b, j);
    if (carry_in) {
      const f32x4 cin = *reinterpret_cast<const f32x4*>(carry_in + ((size_t)16 * bt + row) * NPAD + j);
      G += cin;
    }
    const f16x4 d = *reinterpret_cast<const f16x4*>(drow + ((size_t)16 * bt + row) * NPAD + j);
    // products rounded on their own (never contracted into the row sum that follows), so that both step-per-launch
    // families form bit-identical g and row sums whatever the compiler does with the surrounding code
    f32x4 g;
    {
#pragma clang fp contract(off)
      g = f32x4{(float)d[0] * G[0], (float)d[1] * G[1], (float)d[2] * G[2], (float)d[3] * G[3]};
    }
    return g;
  };
  stage_rows(xb, rs, NPAD, tid, [&](int row, int j) { f32x4 G; return g4(row, j, G); });
  if (staged) stage_gates(gl, p.A, p.k, T, B, t, bt, tid);
  lds_barrier();

  const int tg0 = 16 * cb + 4 * wv;
  const int wg = tg0 / NC, c0 = tg0 % NC;
  const int j0 = 16 * NC * wg + NC * n + c0;
  const int b0 = 16 * bt + 4 * q;
  const float oma = 1.f - p.alpha;
  f32x4 acc[4];
  bf16x4 gcopy[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f32x4 G;
    const f32x4 g = g4(4 * q + e, j0, G);
    const float js = p.J0 * rs[4 * q + e];
#pragma unroll
    for (int cl = 0; cl < 4; ++cl) {
      acc[cl][e] = fmaf(oma, G[cl], js);
      gcopy[cl][e] = (__bf16)g[cl];
    }
  }
#pragma unroll
  for (int cl = 0; cl < 4; ++cl)
    *reinterpret_cast<bf16x4*>(p.gfrag + pair_off_rt(NC, t, p.nbt, bt, tg0 + cl, lane)) = gcopy[cl];
  if (t == T - 1 && (T & 1)) {
    const bf16x4 z = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
#pragma unroll
    for (int cl = 0; cl < 4; ++cl) *reinterpret_cast<bf16x4*>(p.gfrag + pair_off_rt(NC, T, p.nbt, bt, tg0 + cl, lane)) = z;
  }
  wide_products<4>(xb, (const bf16x8*)p.Wpack, p.A, gl, staged, p.k, T, B, t, b0, p.J1, NC, tg0, lane, acc);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int b = b0 + e;
    f32x4 out;
#pragma unroll
    for (int cl = 0; cl < 4; ++cl) out[cl] = (b < B && j0 + cl < N) ? acc[cl][e] : 0.f;
    *reinterpret_cast<f32x4*>(carry_out + ((size_t)16 * bt + 4 * q + e) * NPAD + j0) = out;
    if (t == 0 && p.grad_r_init) store4_masked(p.grad_r_init, N, B, b, j0, out);
  }
}

// ------------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------------
bool ring_wide_applicable(int NC) { return NC == 16 || NC == 24 || NC == 32; }

size_t ring_wide_carry_bytes(int NC, int nbt) { return (size_t)2 * 16 * nbt * 64 * NC * sizeof(float); }

static size_t wide_lds_bytes(int NC) { return (size_t)2 * NC * 4 * XG * sizeof(bf16x8); }

template <typename K>
static hipError_t wide_attr(K kern, size_t dyn) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
}

template <int ACT, int TPW>
static hipError_t wide_fwd_tpw(const RingFwdArgs& a, int NC, bool rebuild, hipStream_t st) {
  const size_t dyn = wide_lds_bytes(NC);
  const unsigned ncb = (unsigned)(NC / TPW);              // 4 NC tiles / (4 TPW per workgroup)
  if (rebuild) {
    hipError_t e = wide_attr(ring_wide_fwd_kernel<ACT, true, TPW>, dyn);
    if (e != hipSuccess) return e;
    RING_LAUNCH((ring_wide_fwd_kernel<ACT, true, TPW>), dim3(a.nbt, ncb, a.T), dim3(256), dyn, st, a, NC, 0, step_xcd_map());
    return hipGetLastError();
  }
  hipError_t e = wide_attr(ring_wide_fwd_kernel<ACT, false, TPW>, dyn);
  if (e != hipSuccess) return e;
  for (int t = 0; t < a.T; ++t) {
    RING_LAUNCH((ring_wide_fwd_kernel<ACT, false, TPW>), dim3(a.nbt, ncb), dim3(256), dyn, st, a, NC, t, step_xcd_map());
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int ACT>
static hipError_t wide_fwd_act(const RingFwdArgs& a, int NC, bool rebuild, int tpw, hipStream_t st) {
  if (tpw == 1) return wide_fwd_tpw<ACT, 1>(a, NC, rebuild, st);
  if (tpw == 2) return wide_fwd_tpw<ACT, 2>(a, NC, rebuild, st);
  return wide_fwd_tpw<ACT, 4>(a, NC, rebuild, st);
}

// tpw = 4 whenever a saved record is written (the layout the BPTT and weight-gradient kernels of this family read)
hipError_t ring_launch_wide_fwd(const RingFwdArgs& a, int NC, bool rebuild, int tpw, hipStream_t st) {
  if (NC % 4 != 0 || (tpw != 1 && tpw != 2 && tpw != 4)) return hipErrorInvalidValue;
  switch (a.act) {
    case ACT_RELU: return wide_fwd_act<ACT_RELU>(a, NC, rebuild, tpw, st);
    case ACT_GELU: return wide_fwd_act<ACT_GELU>(a, NC, rebuild, tpw, st);
    case ACT_TANH: return wide_fwd_act<ACT_TANH>(a, NC, rebuild, tpw, st);
    case ACT_SILU: return wide_fwd_act<ACT_SILU>(a, NC, rebuild, tpw, st);
    default: return hipErrorInvalidValue;
  }
}

// carry: 2 * 16 * nbt * NPAD floats of scratch (ring_wide_carry_bytes), used as two alternating buffers
__global__ __launch_bounds__(256) void ring_trig_table_kernel(float* out, int N, int NPAD) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= NPAD) return;
  float s = 0.f, c = 0.f;
  if (j < N) sincosf(6.283185307179586f * (float)j / (float)N, &s, &c);
  out[2 * j] = c;
  out[2 * j + 1] = s;
}

hipError_t ring_launch_trig_table(float* out, int N, int NPAD, hipStream_t st) {
  RING_LAUNCH(ring_trig_table_kernel, dim3((NPAD + 255) / 256), dim3(256), 0, st, out, N, NPAD);
  return hipGetLastError();
}

hipError_t ring_launch_wide_bptt(const RingBpttArgs& a, int NC, float* carry, hipStream_t st) {
  const size_t dyn = wide_lds_bytes(NC);
  const bool loss = a.loss_coef != nullptr;
  if (loss && (!a.loss_trig || !a.hist)) return hipErrorInvalidValue;
  if (!loss && !a.grad_out) return hipErrorInvalidValue;
  hipError_t e = loss ? wide_attr(ring_wide_bptt_kernel<true>, dyn) : wide_attr(ring_wide_bptt_kernel<false>, dyn);
  if (e != hipSuccess) return e;
  const size_t half = (size_t)16 * a.nbt * 64 * NC;
  const unsigned ncb = (unsigned)(NC / 4);
  for (int t = a.T - 1, u = 0; t >= 0; --t, ++u) {
    const float* cin = (u == 0) ? nullptr : carry + (size_t)((u - 1) & 1) * half;
    float* cout = carry + (size_t)(u & 1) * half;
    if (loss) RING_LAUNCH(ring_wide_bptt_kernel<true>, dim3(a.nbt, ncb), dim3(256), dyn, st, a, NC, t, cin, cout, step_xcd_map());
    else RING_LAUNCH(ring_wide_bptt_kernel<false>, dim3(a.nbt, ncb), dim3(256), dyn, st, a, NC, t, cin, cout, step_xcd_map());
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}
