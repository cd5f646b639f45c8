// gfx950 kernels of the leaky ring-attractor time loop: weight packing, the persistent forward
// recurrence, the reverse-time BPTT recurrence, the rebuild of saved activations from the state
// history, and the split-K weight-gradient contraction with its fixed-order reduction.
//
// The per-step product r @ [Wo|Wa_0|..]^T is a dense bf16 MFMA contraction with fp32 accumulation;
// the reference instead rebuilds W_eff per sample (cpp/kernels/fwd_1loop_tc_idx.cuh:50-232,
// cpp/kernels/bwd_mixed_precision_aggressive.cuh:53-318).
#include "ring_common.hpp"
#include "ring_kernels.hpp"

// ------------------------------------------------------------------------------------------------
// Weight packing: fp32 [N][N] matrices -> bf16 MFMA B-operand fragments, zero padded to NPAD.
//   out[mm][w][c][kc][lane][8]; lane (q,n) owns output column 16*NC*w + NC*n + c and the eight
//   contraction indices 32kc+8q .. +7.  transposed = 0: value = W[col][contr] (forward, re = W r);
//   transposed = 1: value = W[contr][col] (backward, g @ W).
//   Matrix 0 (Wo) is stored as scale0 * Wo + shift0 (rounded once, after the fp32 sum): the weight-resident kernels
//   pass (J1, J0), which turns  J0 * sum_j x_j + J1 * (x Wo^T)  into one product; the others pass (1, 0).  Padding
//   stays zero.
//   split_k = 1 (NC = 4 only): contraction position kappa stands for neuron split_k_neuron(kappa) and output
//   column n of tile c for neuron 64*w + 32*(c/2) + 2*n + c%2: the pipelined weight-resident forward's order.
//   split_k = 2 (NC = 8 only): the same column order (neuron 128*w + 32*(c/2) + 2*n + c%2) with the contraction in
//   neuron order: the cluster forward's (four waves).
//   split_k = 3 (NC = 8 only): tile c of wave group w holds the 16 consecutive neurons 128*w + 16*c + n, contraction
//   in neuron order: the eight-wave cluster forward's.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ bf16x8 pack_fragment(const float* __restrict__ Wo, const float* __restrict__ Wa, size_t u,
                                                int N, int NC, int transposed, int split_k, float scale0, float shift0) {
  const int KCH = 2 * NC;
  const int lane = (int)(u & 63);
  size_t v = u >> 6;
  const int kc = (int)(v % KCH);
  v /= KCH;
  const int c = (int)(v % NC);
  v /= NC;
  const int w = (int)(v & 3);
  const int mm = (int)(v >> 2);
  const int q = lane >> 4, n = lane & 15;
  // split_k: the output columns follow the pipelined forward's ownership as well (tile c = 2*h + cc of wave w)
  const int col = split_k == 3 ? 16 * NC * w + 16 * c + n
                               : (split_k ? 16 * NC * w + 32 * (c >> 1) + 2 * n + (c & 1) : 16 * NC * w + NC * n + c);
  const int k0 = 32 * kc + 8 * q;
  const float* W = (mm == 0) ? Wo : Wa + (size_t)(mm - 1) * N * N;
  bf16x8 pk;
  if (!transposed && !split_k && (N & 3) == 0 && col < N && k0 + 8 <= N) {
    // forward orientation away from the padding: the fragment's eight values lie side by side in one row
    const f32x4* src = reinterpret_cast<const f32x4*>(W + (size_t)col * N + k0);
    const f32x4 a = src[0], b = src[1];
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      float val = x < 4 ? a[x] : b[x - 4];
      if (mm == 0) val = fmaf(val, scale0, shift0);
      pk[x] = (__bf16)val;
    }
    return pk;
  }
#pragma unroll
  for (int x = 0; x < 8; ++x) {
    const int kk = split_k == 1 ? split_k_neuron(k0 + x) : k0 + x;
    float val = 0.f;
    if (col < N && kk < N) {
      val = transposed ? W[(size_t)kk * N + col] : W[(size_t)col * N + kk];
      if (mm == 0) val = fmaf(val, scale0, shift0);
    }
    pk[x] = (__bf16)val;
  }
  return pk;
}

// One launch can write two packed copies (the forward's own and the transposed one its backward will
// need): fragments [0, total) go to out, [total, 2*total) to out2 when out2 is not null.
__global__ __launch_bounds__(256) void ring_pack_weights_kernel(const float* __restrict__ Wo,
                                                                const float* __restrict__ Wa,
                                                                bf16x8* __restrict__ out, bf16x8* __restrict__ out2, int N,
                                                                int k, int NC, int transposed, int split_k, float scale0,
                                                                float shift0, int transposed2, int split_k2, float scale2,
                                                                float shift2) {
  const size_t total = (size_t)(1 + k) * 4 * NC * 2 * NC * 64;
  const size_t all = out2 ? 2 * total : total;
  for (size_t u = (size_t)blockIdx.x * blockDim.x + threadIdx.x; u < all; u += (size_t)gridDim.x * blockDim.x) {
    if (u < total) out[u] = pack_fragment(Wo, Wa, u, N, NC, transposed, split_k, scale0, shift0);
    else out2[u - total] = pack_fragment(Wo, Wa, u - total, N, NC, transposed2, split_k2, scale2, shift2);
  }
}

// ------------------------------------------------------------------------------------------------
// Gated products for one step:  acc[c][e] = sum_mm coef_mm[e] * (X @ W_mm)[row 4q+e][tile c]
// X is read as MFMA A-operand fragments from the LDS operand buffer, W_mm streams from the packed
// global copy (L2 resident).  coef_0 = J1, coef_{1+j}[e] = A[b_e, t, j].
// ------------------------------------------------------------------------------------------------
// Action gates of one step for the workgroup's 16 rows, staged through LDS one step ahead (a_dim <= GATE_KMAX):
// a coalesced tile load instead of scattered per-lane loads, and the place where all-zero channels are
// found.  A channel whose gate is zero for all 16 rows at this step contributes nothing to the
// pre-activation (forward) or to the carried gradient (BPTT), so its matrix is neither fetched nor
// multiplied: zero-padded action signals (16 channels of which two are driven) cost what two cost.
constexpr int GATE_KMAX = 64;

__device__ __forceinline__ void gates_stage(float* gl, const float* __restrict__ A, int k, int T, int B, int t, int bt,
                                            int tid) {
  for (int idx = tid; idx < 16 * k; idx += 256) {
    const int row = idx / k, c = idx - row * k, b = 16 * bt + row;
    gl[row * GATE_KMAX + c] = b < B ? A[((size_t)b * T + t) * k + c] : 0.f;
  }
}

// The same in two halves, for the time loops: the loads go into registers a step ahead (GATE_KMAX * 16 / 256
// values per thread) and are written to LDS later in the step, when they have landed; a load followed at once
// by its LDS store would wait for the load and, the memory counter being in order, for the acknowledgement of
// every history store issued before it.
constexpr int GATE_REGS = GATE_KMAX * 16 / 256;

__device__ __forceinline__ void gates_fetch_regs(float (&gv)[GATE_REGS], const float* __restrict__ A, int k, int T, int B, int t,
                                                 int bt, int tid) {
#pragma unroll
  for (int j = 0; j < GATE_REGS; ++j) {
    const int idx = tid + 256 * j;
    const int row = idx / k, c = idx - row * k, b = 16 * bt + row;
    gv[j] = (idx < 16 * k && b < B) ? A[((size_t)b * T + t) * k + c] : 0.f;
  }
}

__device__ __forceinline__ void gates_publish_regs(float* gl, const float (&gv)[GATE_REGS], int k, int tid) {
#pragma unroll
  for (int j = 0; j < GATE_REGS; ++j) {
    const int idx = tid + 256 * j;
    const int row = idx / k, c = idx - row * k;
    if (idx < 16 * k) gl[row * GATE_KMAX + c] = gv[j];
  }
}

// bit c set <=> channel c has a non-zero gate in some row; every wave computes the same mask
// (over the rt gate tiles that follow each other at gl)
__device__ __forceinline__ unsigned long long gates_active(const float* gl, int k, int lane, int rt = 1) {
  unsigned long long m = 0;
  for (int c0 = 0; c0 < k; c0 += 4) {
    const int c = c0 + (lane >> 4);
    bool nz = false;
    for (int i = 0; i < rt; ++i) nz |= c < k && gl[(i * 16 + (lane & 15)) * GATE_KMAX + c] != 0.f;
    const unsigned long long bal = __ballot(nz);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if ((bal >> (16 * j)) & 0xffffull) m |= 1ull << (c0 + j);
  }
  // the mask is the same in every lane; say so, so that the matrix loop it drives is scalar control flow
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)m), hi = __builtin_amdgcn_readfirstlane((unsigned)(m >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// Weight pipeline geometry: a unit is one column tile x KG K chunks; PD register buffers, PD - 1 units in
// flight ahead of the MFMAs.  With more than one batch tile the units are halved and twice as many are
// kept in flight: the same bytes on their way, half the A-operand registers per tile.
template <int NC, int RT>
struct StreamCfg {
  using TL = Tile<NC>;
  static constexpr int KG = (RT > 1 && TL::KG == 8) ? 4 : TL::KG, NKG = TL::KCH / KG;
  static constexpr int UPM = NKG * NC;                 // units per matrix
  // (four tiles: every fetched fragment feeds four MFMAs, so half as many units in flight cover the same time)
  static constexpr int PDMAX = (RT >= 4) ? 4 : ((RT > 1 && TL::KG == 8) ? 8 : 4);
  static constexpr int PD = UPM >= PDMAX ? PDMAX : UPM;
  static_assert(UPM % PD == 0, "static register-buffer indices need whole rounds per matrix");
};

// With GA, rp holds r_prev[row 4q+e][neuron tile c] and ga_part (k x 4 waves x 16 rows) receives, per action
// matrix and batch row, this wave's share of  sum_j (X @ W_mm)[row][j] * r_prev[row][j]  (= dL/dA[b,t,mm-1]).
// gl: this step's staged gates (null: read A from global); active: channels worth multiplying.
// RT: batch tiles of 16 rows that share every weight fragment a wave fetches (one L2 read feeds RT MFMAs).
// Tile rt reads the operand buffer xb + rt * SLOTS and the gate tile gl + rt * 16 * GATE_KMAX, and its
// rows start at b0 + 16 * rt.
// wf: the caller's weight register buffers.  primed: they already hold the first PD - 1 units of matrix 0
// (a previous call ran with carry_over, which points the prefetch of the last matrix at matrix 0 again:
// the weights do not change between steps, so the next step's first units load during this step's epilogue).
template <int NC, bool GA = false, int RT = 1>
__device__ __forceinline__ void gated_products(const bf16x8* __restrict__ xb, const bf16x8* __restrict__ Wp,
                                               const float* __restrict__ A, const float* gl, unsigned long long active,
                                               int k, int T, int B, int t, int b0, float J1, int w, int lane,
                                               f32x4 (&acc)[RT][NC],
                                               bf16x8 (&wf)[StreamCfg<NC, RT>::PD][StreamCfg<NC, RT>::KG],
                                               bool primed, bool carry_over, const float (*rp)[NC] = nullptr,
                                               float* ga_part = nullptr, bool acc_preset = false) {
  static_assert(!GA || RT == 1, "dL/dA is produced one batch tile at a time");
  using TL = Tile<NC>;
  using SC = StreamCfg<NC, RT>;
  constexpr int KG = SC::KG, NKG = SC::NKG, UPM = SC::UPM, PD = SC::PD;
  const int q = lane >> 4, n = lane & 15;
  if (!acc_preset) {                            // otherwise the caller's values are what the products add to
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int c = 0; c < NC; ++c) acc[rt][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // The weights of a step stream from L2 as one linear sequence of units, active matrix after active
  // matrix; what bounds the step is how many bytes are in flight, so the prefetch runs PD - 1 units
  // ahead and straight across matrix boundaries (past the last matrix: into matrix 0 for the next step,
  // or a re-read of that one, unused).
  // Matrix 0 (Wo) is always active; matrix mm >= 1 is gated by channel mm - 1.
  const bool skipping = gl != nullptr && !GA;   // dL/dA needs every product, also where the gate is zero
  auto next_matrix = [&](int mm) {               // next active matrix after mm, or -1
    if (!skipping) return mm < k ? mm + 1 : -1;
    const unsigned long long rest = mm >= 64 ? 0ull : (active >> mm);   // channels mm, mm+1, ... <-> matrices mm+1, ...
    return rest ? mm + 1 + (int)__builtin_ctzll(rest) : -1;
  };
  // A unit's address is a wave-uniform base (scalar registers) plus the lane's 16-byte slot: no vector
  // registers are spent on addresses.
  const int ws = __builtin_amdgcn_readfirstlane(w);
  const unsigned lane_off = (unsigned)lane * 16u;
  auto unit_ptr = [&](int mm, int ul) {
    const int kg = ul / NC, c = ul % NC;
    return reinterpret_cast<const char*>(Wp) + ((size_t)((mm * 4 + ws) * NC + c) * TL::KCH + kg * KG) * 1024;
  };
  auto unit_load = [&](const char* base, int u) {
    return *reinterpret_cast<const bf16x8*>(base + u * 1024 + lane_off);
  };
  if (!primed) {
#pragma unroll
    for (int d = 0; d < PD - 1; ++d) {          // PD - 1 < UPM: the first units all belong to matrix 0
      const char* src = unit_ptr(0, d);
#pragma unroll
      for (int u = 0; u < KG; ++u) wf[d][u] = unit_load(src, u);
    }
  }

  for (int mm = 0; mm >= 0;) {
    const int nxt = next_matrix(mm);
    const int pre = nxt >= 0 ? nxt : (carry_over ? 0 : mm);   // matrix the prefetch runs into
    float coef[RT][4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int b = b0 + 16 * rt + e;
        if (mm == 0) coef[rt][e] = J1;
        else if (gl) coef[rt][e] = gl[(rt * 16 + 4 * q + e) * GATE_KMAX + (mm - 1)];
        else coef[rt][e] = (b < B) ? A[((size_t)b * T + t) * k + (mm - 1)] : 0.f;
      }
    f32x4 p[RT][NC];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int c = 0; c < NC; ++c) p[rt][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    // The A operands do not depend on the matrix.  With one batch tile they are read from LDS once per
    // step and kept; with more, that would take the registers the weight pipeline needs, so they are read
    // again for every matrix (xo is opaque to the compiler so that it does not hoist the reads).
    int xo = q * XG + n;
    if constexpr (RT > 1) asm volatile("" : "+v"(xo));
#pragma unroll
    for (int kg = 0; kg < NKG; ++kg) {
      bf16x8 af[RT][KG];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int u = 0; u < KG; ++u) af[rt][u] = xb[rt * TL::SLOTS + (kg * KG + u) * 4 * XG + xo];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int ul = kg * NC + c;             // unit within the matrix; UPM % PD == 0 keeps buffer indices static
        {
          const int ahead = ul + PD - 1;
          const char* src = ahead < UPM ? unit_ptr(mm, ahead) : unit_ptr(pre, ahead - UPM);
#pragma unroll
          for (int u = 0; u < KG; ++u) wf[ahead % PD][u] = unit_load(src, u);
        }
        // Pin the order "loads of unit ul + PD - 1, then MFMAs of unit ul": left to itself the scheduler
        // sinks the loads towards their use (to save registers) and the prefetch distance is gone.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < KG; ++u)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) p[rt][c] = mfma16(af[rt][u], wf[ul % PD][u], p[rt][c]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[rt][c][e] += coef[rt][e] * p[rt][c][e];
    if constexpr (GA) {
      if (mm > 0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float d = 0.f;
#pragma unroll
          for (int c = 0; c < NC; ++c) d = fmaf(p[0][c][e], rp[e][c], d);
          d = row16_sum(d);
          if (n == 0) ga_part[((mm - 1) * 4 + w) * 16 + 4 * q + e] = d;
        }
      }
    }
    mm = nxt;
  }
}

// Row sums over neurons: per-wave partials go to psum[w][16]; readers add the four in wave order.
template <int NC>
__device__ __forceinline__ void publish_rowsum(float* psum, const float (&v)[4][NC], int w, int q, int n) {
  float s[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float a = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) a += v[e][c];
    s[e] = row16_sum(a);
  }
  if (n == 0) {
#pragma unroll
    for (int e = 0; e < 4; ++e) psum[w * 16 + 4 * q + e] = s[e];
  }
}

__device__ __forceinline__ void read_rowsum(const float* psum, int q, float (&s)[4]) {
#pragma unroll
  for (int e = 0; e < 4; ++e)
    s[e] = ((psum[0 * 16 + 4 * q + e] + psum[1 * 16 + 4 * q + e]) + psum[2 * 16 + 4 * q + e]) + psum[3 * 16 + 4 * q + e];
}

// The loss head's three sums per row (sum_i v_i cos(phi_i), sum_i v_i sin(phi_i), sum_i |v_i|, phi_i = 2 pi i / N)
// over the wave's neurons: per-wave partials to lsum[kind][w * 16 + row].  The lane's NC consecutive angles come from
// its first one by the angle-addition recurrence (c0, s0 = cos, sin of phi_{i0}; cd, sd = cos, sin of 2 pi / N).
template <int NC>
__device__ __forceinline__ void publish_loss_sums(float* lsum, const float (&v)[4][NC], float c0, float s0, float cd,
                                                  float sd, int w, int q, int n) {
  float C[4] = {0.f, 0.f, 0.f, 0.f}, S[4] = {0.f, 0.f, 0.f, 0.f}, A[4] = {0.f, 0.f, 0.f, 0.f};
  float cc = c0, ss = s0;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      C[e] = fmaf(v[e][c], cc, C[e]);
      S[e] = fmaf(v[e][c], ss, S[e]);
      A[e] += fabsf(v[e][c]);
    }
    const float cn = fmaf(cc, cd, -ss * sd);
    ss = fmaf(ss, cd, cc * sd);
    cc = cn;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    C[e] = row16_sum(C[e]);
    S[e] = row16_sum(S[e]);
    A[e] = row16_sum(A[e]);
  }
  if (n == 0) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lsum[0 * 64 + w * 16 + 4 * q + e] = C[e];
      lsum[1 * 64 + w * 16 + 4 * q + e] = S[e];
      lsum[2 * 64 + w * 16 + 4 * q + e] = A[e];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Forward: one workgroup = RT tiles of 16 batch rows for all T steps.  r lives in fp32 registers; its
// bf16 copy is exchanged between the four waves through a double-buffered LDS operand buffer (one
// barrier per step).  Writes bump_history [T,B,N] fp32 and, when training, F'(re) (fp16) and the bf16
// operand copy of r_prev in tile order.  The operand buffers [2][RT][SLOTS] are dynamic shared memory.
// ------------------------------------------------------------------------------------------------
template <int NC, int RT>
constexpr size_t stream_lds_bytes() { return (size_t)2 * RT * Tile<NC>::SLOTS * sizeof(bf16x8); }

// Bytes of the packed weights (all matrices), and the copy of them into LDS by the whole workgroup.
template <int NC>
__host__ __device__ constexpr size_t packed_weight_bytes(int k) { return (size_t)(1 + k) * 4 * NC * Tile<NC>::KCH * 64 * sizeof(bf16x8); }

template <int NC>
__device__ __forceinline__ void weights_to_lds(bf16x8* wl, const bf16x8* __restrict__ Wp, int k, int tid) {
  const int frags = (1 + k) * 4 * NC * Tile<NC>::KCH * 64;
  for (int i = tid; i < frags; i += 256) wl[i] = Wp[i];
}

// With more than one batch tile per workgroup the forward keeps its fp32 state in LDS between steps
// (one read and one write per lane and step) instead of in registers the weight pipeline needs.
template <int NC, int RT>
constexpr size_t fwd_state_lds_bytes() { return RT > 1 ? (size_t)RT * 4 * NC * 256 * sizeof(float) : 0; }

// WL: the packed weights of all 1 + a_dim matrices fit in LDS next to the operand buffers (small N): the workgroup
// copies them there once and the per-step "stream" reads LDS instead of L2.
// STATS: also leave the loss head's three sums of every history row in p.loss_stats[t * B + b] (the waves' shares
// meet in LDS by step parity and are added in wave order behind the step's barrier), so that the loss needs no pass
// of its own over the history.
template <int NC, int ACT, int RT, bool WL, bool STATS>
__global__ __launch_bounds__(256) void ring_fwd_kernel(RingFwdArgs p) {
  using TL = Tile<NC>;
  extern __shared__ __attribute__((aligned(16))) char stream_lds[];
  bf16x8* const xbuf = reinterpret_cast<bf16x8*>(stream_lds);   // [2][RT][SLOTS]
  static_assert(!WL || RT == 1, "LDS-resident weights go with one batch tile per workgroup");
  const bf16x8* wsrc = (const bf16x8*)p.Wpack;
  if constexpr (WL) {
    bf16x8* wl = reinterpret_cast<bf16x8*>(stream_lds + stream_lds_bytes<NC, RT>());
    weights_to_lds<NC>(wl, (const bf16x8*)p.Wpack, p.k, threadIdx.x);   // published by the barrier before the loop
    wsrc = wl;
  }
  __shared__ float psum[2][RT][64];
  __shared__ float gl[2][RT * 16 * GATE_KMAX];
  __shared__ float lsum[STATS ? 2 : 1][RT][3 * 64];

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt0 = blockIdx.x * RT;             // tile rt is batch tile bt0 + rt (past the last one: all rows masked)
  const int b0 = 16 * bt0 + 4 * q;
  const int i0 = 16 * NC * w + NC * n;
  const int N = p.N, B = p.B, T = p.T;
  const float oma = 1.f - p.alpha;
  const bool staged = p.k <= GATE_KMAX;
  float lc0 = 0.f, ls0 = 0.f, lcd = 0.f, lsd = 0.f;
  if constexpr (STATS) {
    sincosf(6.283185307179586f * (float)i0 / (float)N, &ls0, &lc0);
    sincosf(6.283185307179586f / (float)N, &lsd, &lcd);
  }
  // row sums of history row `row_t` from the shares in lsum[buf] (complete behind a barrier): threads 0 .. 64 RT - 1
  auto flush_loss_sums = [&](int row_t, int buf) {
    if (tid < 64 * RT) {
      const int rt = tid >> 6, kind = (tid >> 4) & 3, row = tid & 15, b = 16 * (bt0 + rt) + row;
      float v = 0.f;
      if (kind < 3) {
        const float* src = lsum[buf][rt] + kind * 64 + row;
        v = ((src[0] + src[16]) + src[32]) + src[48];
      }
      if (b < B) reinterpret_cast<float*>(p.loss_stats + (size_t)row_t * B + b)[kind] = v;
    }
  };
  auto xb = [&](int buf, int rt) { return xbuf + (size_t)(buf * RT + rt) * TL::SLOTS; };

  constexpr bool LDS_STATE = RT > 1;
  float* const state = reinterpret_cast<float*>(stream_lds + stream_lds_bytes<NC, RT>());   // [RT][4][NC][256 lanes]
  float rkeep[4][NC];
  auto state_get = [&](int rt, float (&v)[4][NC]) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < NC; ++c) v[e][c] = LDS_STATE ? state[((rt * 4 + e) * NC + c) * 256 + tid] : rkeep[e][c];
  };
  auto state_put = [&](int rt, const float (&v)[4][NC]) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        if constexpr (LDS_STATE) state[((rt * 4 + e) * NC + c) * 256 + tid] = v[e][c];
        else rkeep[e][c] = v[e][c];
      }
  };

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float r[4][NC];
    rows_load<NC>(p.r_init, N, B, b0 + 16 * rt, i0, r);
    state_put(rt, r);
    write_operand<NC>(xb(0, rt), r, w, q, n);
    publish_rowsum<NC>(psum[0][rt], r, w, q, n);
    if (staged) gates_stage(gl[0] + rt * 16 * GATE_KMAX, p.A, p.k, T, B, 0, bt0 + rt, tid);
  }
  lds_barrier();

  bf16x8 wf[StreamCfg<NC, RT>::PD][StreamCfg<NC, RT>::KG];
  for (int t = 0; t < T; ++t) {
    const int cur = t & 1;
    if constexpr (STATS) {
      if (t > 0) flush_loss_sums(t - 1, cur);    // row t-1's shares were left in lsum[(t-1)&1 ^ 1] = lsum[cur]
    }
    f32x4 acc[RT][NC];
    // next step's gates: loaded now, written to LDS after the products (nothing waits for them before that).
    // Two paired tiles at the widest tiling have no registers to hold them and stage them in one go.
    constexpr bool GATE_PIPE = !(NC == 8 && RT > 1);
    float gv[RT][GATE_REGS];
    const bool stage_next = staged && t + 1 < T;
    if (stage_next) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if constexpr (GATE_PIPE) gates_fetch_regs(gv[rt], p.A, p.k, T, B, t + 1, bt0 + rt, tid);
        else gates_stage(gl[cur ^ 1] + rt * 16 * GATE_KMAX, p.A, p.k, T, B, t + 1, bt0 + rt, tid);
      }
    }
    gated_products<NC, false, RT>(xb(cur, 0), wsrc, p.A, staged ? gl[cur] : nullptr,
                                  staged ? gates_active(gl[cur], p.k, lane, RT) : ~0ull, p.k, T, B, t, b0, p.J1, w, lane,
                                  acc, wf, t > 0, t + 1 < T);
    if (GATE_PIPE && stage_next) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) gates_publish_regs(gl[cur ^ 1] + rt * 16 * GATE_KMAX, gv[rt], p.k, tid);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int bq = b0 + 16 * rt;
      float s[4];
      read_rowsum(psum[cur][rt], q, s);
      float r[4][NC], d[4][NC];
      state_get(rt, r);
      const bool live = bt0 + rt < p.nbt;
      // The bf16 operand copy pairs steps 2j and 2j+1 in one 16-byte slot per lane and tile.  At an even step both
      // halves are in registers, this step's operand (r before the update) and the next one's (r after it): they
      // leave as one 16-byte store, whole 32-byte sectors per lane pair, where two 8-byte stores a time step apart
      // reach memory as two partial writes once a step outlasts the line's stay in L2 (wide tilings).
      const bool pair_now = p.rfrag && live && (t & 1) == 0;
      const bool tail = t + 1 == T;                // odd length: the last slot's second half has no step and reads as zero
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        bf16x4 lo = {(__bf16)r[0][c], (__bf16)r[1][c], (__bf16)r[2][c], (__bf16)r[3][c]};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = acc[rt][c][e] + p.J0 * s[e];
          float F, D;
          act_fast<ACT>(x, F, D);
          const bool ok = (bq + e < B) && (i0 + c < N);
          r[e][c] = ok ? (oma * r[e][c] + p.alpha * F) : 0.f;
          d[e][c] = ok ? p.alpha * D : 0.f;   // the saved record is alpha * F'(re)
        }
        if (pair_now) {
          bf16x4 hi = {(__bf16)r[0][c], (__bf16)r[1][c], (__bf16)r[2][c], (__bf16)r[3][c]};
          if (tail) hi = bf16x4{(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
          *reinterpret_cast<bf16x8*>(p.rfrag + pair_offset<NC>(t, p.nbt, bt0 + rt, w * NC + c, lane)) =
              __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
      }
      rows_store<NC>(p.hist + (size_t)t * B * N, N, B, bq, i0, r);
      if (p.dfrag && live) side_store<NC, f16x4, _Float16>(p.dfrag + side_offset<NC>(t, p.nbt, bt0 + rt, w, lane), d);
      if constexpr (STATS) publish_loss_sums<NC>(lsum[cur ^ 1][rt], r, lc0, ls0, lcd, lsd, w, q, n);
      if (t + 1 < T) {
        state_put(rt, r);
        write_operand<NC>(xb(cur ^ 1, rt), r, w, q, n);
        publish_rowsum<NC>(psum[cur ^ 1][rt], r, w, q, n);
      }
    }
    lds_barrier();
  }
  if constexpr (STATS) flush_loss_sums(T - 1, T & 1);   // the last row's shares: lsum[((T-1)&1) ^ 1]
}

// ------------------------------------------------------------------------------------------------
// Rebuild of the saved activations from the state history (used when the forward's buffer was not
// kept): one workgroup per (batch tile, step); no recurrence.
// ------------------------------------------------------------------------------------------------
template <int NC, int ACT, int RT>
__global__ __launch_bounds__(256) void ring_rebuild_saved_kernel(RingFwdArgs p) {
  using TL = Tile<NC>;
  __shared__ bf16x8 xbuf[RT * TL::SLOTS];
  __shared__ float psum[RT][64];
  __shared__ float gl[RT * 16 * GATE_KMAX];

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt0 = blockIdx.x * RT, t = blockIdx.y;
  const int b0 = 16 * bt0 + 4 * q;
  const int i0 = 16 * NC * w + NC * n;
  const int N = p.N, B = p.B, T = p.T;
  const bool staged = p.k <= GATE_KMAX;

  const float* prev = (t == 0) ? p.r_init : p.hist + (size_t)(t - 1) * B * N;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float r[4][NC];
    rows_load<NC>(prev, N, B, b0 + 16 * rt, i0, r);
    write_operand<NC>(xbuf + rt * TL::SLOTS, r, w, q, n);
    publish_rowsum<NC>(psum[rt], r, w, q, n);
    if (bt0 + rt < p.nbt) {
      pair_store<NC>(p.rfrag, t, p.nbt, bt0 + rt, w, lane, r);
      if (t == T - 1) pair_zero_tail<NC>(p.rfrag, T, p.nbt, bt0 + rt, w, lane);
    }
    if (staged) gates_stage(gl + rt * 16 * GATE_KMAX, p.A, p.k, T, B, t, bt0 + rt, tid);
  }
  lds_barrier();

  f32x4 acc[RT][NC];
  bf16x8 wf[StreamCfg<NC, RT>::PD][StreamCfg<NC, RT>::KG];
  gated_products<NC, false, RT>(xbuf, (const bf16x8*)p.Wpack, p.A, staged ? gl : nullptr,
                                staged ? gates_active(gl, p.k, lane, RT) : ~0ull, p.k, T, B, t, b0, p.J1, w, lane, acc,
                                wf, false, false);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (bt0 + rt >= p.nbt) continue;
    float s[4];
    read_rowsum(psum[rt], q, s);
    float d[4][NC];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        float F, D;
        act_fast<ACT>(acc[rt][c][e] + p.J0 * s[e], F, D);
        d[e][c] = ((b0 + 16 * rt + e < B) && (i0 + c < N)) ? p.alpha * D : 0.f;
      }
    }
    side_store<NC, f16x4, _Float16>(p.dfrag + side_offset<NC>(t, p.nbt, bt0 + rt, w, lane), d);
  }
}

// The same rebuild with four row tiles per workgroup: two batch tiles x two consecutive time steps.  Nothing here
// depends on an earlier step (every step's r_prev is a row of the history), so rows of different steps can share a
// fetched weight fragment just as rows of different samples do: each fragment feeds four MFMAs and the workgroups
// together stream the weights from L2 half as often as with two tiles.  Tile rt is (batch tile bt0 + rt % 2, step
// 2 * blockIdx.y + rt / 2); the operand tiles live in dynamic shared memory (4 * SLOTS fragments).
template <int NC, int ACT>
__global__ __launch_bounds__(256) void ring_rebuild_saved4_kernel(RingFwdArgs p) {
  using TL = Tile<NC>;
  constexpr int RT = 4;
  extern __shared__ __attribute__((aligned(16))) char rebuild_lds[];
  bf16x8* const xbuf = reinterpret_cast<bf16x8*>(rebuild_lds);
  __shared__ float psum[RT][64];
  __shared__ float gl[RT * 16 * GATE_KMAX];

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt0 = blockIdx.x * 2, t0 = blockIdx.y * 2;
  const int i0 = 16 * NC * w + NC * n;
  const int N = p.N, B = p.B, T = p.T;

  bool live[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int bt = bt0 + (rt & 1), t = t0 + (rt >> 1);
    live[rt] = bt < p.nbt && t < T;
    const int tc = t < T ? t : T - 1;                      // a step past the end re-reads the last one, unused
    const float* prev = (tc == 0) ? p.r_init : p.hist + (size_t)(tc - 1) * B * N;
    float r[4][NC];
    rows_load<NC>(prev, N, B, 16 * bt + 4 * q, i0, r);
    write_operand<NC>(xbuf + rt * TL::SLOTS, r, w, q, n);
    publish_rowsum<NC>(psum[rt], r, w, q, n);
    if (live[rt]) {
      pair_store<NC>(p.rfrag, t, p.nbt, bt, w, lane, r);
      if (t == T - 1) pair_zero_tail<NC>(p.rfrag, T, p.nbt, bt, w, lane);
    }
    gates_stage(gl + rt * 16 * GATE_KMAX, p.A, p.k, T, B, tc, bt, tid);
  }
  lds_barrier();

  f32x4 acc[RT][NC];
  bf16x8 wf[StreamCfg<NC, RT>::PD][StreamCfg<NC, RT>::KG];
  gated_products<NC, false, RT>(xbuf, (const bf16x8*)p.Wpack, p.A, gl, gates_active(gl, p.k, lane, RT), p.k, T, B, t0,
                                16 * bt0 + 4 * q, p.J1, w, lane, acc, wf, false, false);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (!live[rt]) continue;
    const int bt = bt0 + (rt & 1), t = t0 + (rt >> 1);
    float s[4];
    read_rowsum(psum[rt], q, s);
    float d[4][NC];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        float F, D;
        act_fast<ACT>(acc[rt][c][e] + p.J0 * s[e], F, D);
        d[e][c] = ((16 * bt + 4 * q + e < B) && (i0 + c < N)) ? p.alpha * D : 0.f;
      }
    }
    side_store<NC, f16x4, _Float16>(p.dfrag + side_offset<NC>(t, p.nbt, bt, w, lane), d);
  }
}

// ------------------------------------------------------------------------------------------------
// BPTT recurrence, reverse time.  carry = dL/dr_t flowing in from later steps (fp32 registers).
//   G = carry + grad_output[t];  g = (alpha * F'(re_t)) * G  (saved record; bf16 copy -> LDS operand + gfrag)
//   carry' = (1-alpha) G + J0 * sum_i g + J1 (g @ Wo) + sum_j A_j (g @ Wa_j)
// legacy/bwd_fp32.py:86-109.  One barrier per step.
// ------------------------------------------------------------------------------------------------
// Sum the four waves' shares of one step in wave order and write grad_A[b, t, c] for the tile's 16 rows.
__device__ __forceinline__ void bptt_flush_grad_A(const RingBpttArgs& p, const float* part, int t, int bt, int tid) {
  for (int idx = tid; idx < 16 * p.k; idx += 256) {
    const int c = idx >> 4, row = idx & 15, b = 16 * bt + row;
    const float* s = part + c * 64 + row;
    if (b < p.B) p.grad_A[((size_t)b * p.T + t) * p.k + c] = ((s[0] + s[16]) + s[32]) + s[48];
  }
}

// GA: also produce grad_A[b,t,c] = sum_j (g Wa[c])[j] * r_prev[j] (one batch tile per workgroup).  The
// per-wave shares of a step go to a double-buffered LDS array (2*k*64 floats behind the operand buffers
// in dynamic shared memory) and are summed in wave order and written out after the next step's barrier.
// LOSS: grad_output is not read; it is formed per element from the state history and the loss head's row
// coefficients,  up * (kc cos(phi_i) + ks sin(phi_i) + beta sign(r_i)),  phi_i = 2 pi i / N,  up = upstream / (T * B).
template <int NC, bool GA, int RT, bool LOSS, bool WL>
__global__ __launch_bounds__(256) void ring_bptt_kernel(RingBpttArgs p) {
  static_assert(!GA || RT == 1, "dL/dA is produced one batch tile at a time");
  static_assert(!WL || RT == 1, "LDS-resident weights go with one batch tile per workgroup");
  using TL = Tile<NC>;
  extern __shared__ __attribute__((aligned(16))) char stream_lds[];
  bf16x8* const xbuf = reinterpret_cast<bf16x8*>(stream_lds);                              // [2][RT][SLOTS]
  float* const ga_buf = reinterpret_cast<float*>(stream_lds + stream_lds_bytes<NC, RT>());  // [2][k][4 waves][16 rows] when GA
  const bf16x8* wsrc = (const bf16x8*)p.Wpack;
  if constexpr (WL) {   // behind the operand buffers and the dL/dA shares
    bf16x8* wl = reinterpret_cast<bf16x8*>(stream_lds + stream_lds_bytes<NC, RT>() + (GA ? (size_t)2 * p.k * 64 * sizeof(float) : 0));
    weights_to_lds<NC>(wl, (const bf16x8*)p.Wpack, p.k, threadIdx.x);   // published by the first step's barrier
    wsrc = wl;
  }
  __shared__ float psum[2][RT][64];
  __shared__ float gl[2][RT * 16 * GATE_KMAX];

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt0 = blockIdx.x * RT;
  const int b0 = 16 * bt0 + 4 * q;
  const int i0 = 16 * NC * w + NC * n;
  const int N = p.N, B = p.B, T = p.T;
  const float oma = 1.f - p.alpha;
  auto xb = [&](int buf, int rt) { return xbuf + (size_t)(buf * RT + rt) * TL::SLOTS; };

  const bool staged = p.k <= GATE_KMAX;
  float carry[RT][4][NC];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < NC; ++c) carry[rt][e][c] = 0.f;
  }
  // the lane's cos(phi_i), sin(phi_i): in registers, or (paired tiles, where registers are short) in LDS
  constexpr bool CS_LDS = LOSS && RT > 1;
  __shared__ float cs_lds[CS_LDS ? 2 * NC * 256 : 1];
  float cs[NC], sn[NC], up = 0.f;
  if constexpr (LOSS) {
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const float phi = 6.2831853071795864769f * (float)(i0 + c) / (float)N;
      cs[c] = cosf(phi);
      sn[c] = sinf(phi);
      if constexpr (CS_LDS) {
        cs_lds[(2 * c) * 256 + tid] = cs[c];
        cs_lds[(2 * c + 1) * 256 + tid] = sn[c];
      }
    }
    up = (p.loss_upstream ? p.loss_upstream[0] : 1.f) * p.loss_inv_rows;
  }

  // A step's inputs -- grad_output (or, with the loss head fused in, the state rows and their coefficient
  // records) and the saved F' record -- are loaded one step ahead into registers, right after the previous
  // step consumed them, so that their HBM latency runs under that step's products.  (The variants of the widest
  // tiling that have no registers left for that load at the top of the step.)
  constexpr bool PREFETCH = NC <= 4 || (RT == 1 && !GA && !LOSS);
  constexpr bool GATE_PIPE = PREFETCH;
  struct StepIn {
    float G[4][NC];
    f16x4 d[NC];
    ring_f32x4 cf[LOSS ? 4 : 1];
  };
  auto fetch_in = [&](int t, int rt, StepIn& in) {
    rows_load<NC>((LOSS ? p.hist : p.grad_out) + (size_t)t * B * N, N, B, b0 + 16 * rt, i0, in.G);
    if (bt0 + rt < p.nbt) {
      const _Float16* src = p.dfrag + side_offset<NC>(t, p.nbt, bt0 + rt, w, lane);
#pragma unroll
      for (int c = 0; c < NC; ++c) in.d[c] = *reinterpret_cast<const f16x4*>(src + 4 * c);
    } else {
#pragma unroll
      for (int c = 0; c < NC; ++c) in.d[c] = f16x4{(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
    }
    if constexpr (LOSS) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int b = b0 + 16 * rt + e;
        in.cf[e] = p.loss_coef[(size_t)t * B + (b < B ? b : B - 1)];
      }
    }
  };
  StepIn in[RT];
  float gv[RT][GATE_REGS];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if constexpr (PREFETCH) fetch_in(T - 1, rt, in[rt]);
    if (GATE_PIPE && staged) {
      gates_fetch_regs(gv[rt], p.A, p.k, T, B, T - 1, bt0 + rt, tid);
      gates_publish_regs(gl[0] + rt * 16 * GATE_KMAX, gv[rt], p.k, tid);   // published by the first step's barrier
    }
  }

  // The weight pipeline restarts every step here; carrying its buffers over would cost registers.
  bf16x8 wf[StreamCfg<NC, RT>::PD][StreamCfg<NC, RT>::KG];
  // The bf16 operand copy of g pairs steps 2j and 2j+1 in one 16-byte slot per lane and tile: the odd step's half
  // waits in registers for the even step that follows it here, and the two leave as one 16-byte store (whole
  // 32-byte sectors per lane pair instead of two partial writes a time step apart).  An odd sequence length starts
  // on an even step, whose slot's second half has no step and is written as zero.
  // (paired tiles at the widest tiling have no registers left for it and park it in LDS, each thread its own words)
  constexpr bool HOLD_LDS = NC == 8 && RT > 1;
  __shared__ bf16x4 held_lds[HOLD_LDS ? RT * NC * 256 : 1];
  bf16x4 held[HOLD_LDS ? 1 : RT][HOLD_LDS ? 1 : NC];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const bf16x4 z = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
      if constexpr (HOLD_LDS) held_lds[(rt * NC + c) * 256 + tid] = z;
      else held[rt][c] = z;
    }
  for (int t = T - 1; t >= 0; --t) {
    const int cur = (T - 1 - t) & 1;
    // The accumulators start at (1-alpha) G, so that G itself is dead before the products begin.
    f32x4 acc[RT][NC];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const bool live = bt0 + rt < p.nbt;
      if constexpr (!PREFETCH) fetch_in(t, rt, in[rt]);
      float G[4][NC], g[4][NC];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float kc = 0.f, ks = 0.f, beta = 0.f;
        if constexpr (LOSS) {
          kc = in[rt].cf[e][0] * up;
          ks = in[rt].cf[e][1] * up;
          beta = in[rt].cf[e][2] * up;
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          float go = in[rt].G[e][c];
          if constexpr (LOSS) {   // the rows are the state; columns past N get a finite value that meets F' = 0
            const float r = go;
            const float sb = r > 0.f ? beta : (r < 0.f ? -beta : 0.f);          // beta * sign(r), sign(0) = 0
            const float co = CS_LDS ? cs_lds[(2 * c) * 256 + tid] : cs[c];
            const float si = CS_LDS ? cs_lds[(2 * c + 1) * 256 + tid] : sn[c];
            go = fmaf(kc, co, fmaf(ks, si, sb));
          }
          G[e][c] = go + carry[rt][e][c];
          g[e][c] = (float)in[rt].d[c][e] * G[e][c];   // the saved record already carries alpha
          acc[rt][c][e] = oma * G[e][c];
        }
      }
      if constexpr (PREFETCH) {
        if (t > 0) fetch_in(t - 1, rt, in[rt]);
      }
      // the gates of the next step (t - 1): loaded now, written to LDS after the products
      if constexpr (GATE_PIPE) {
        if (staged && t > 0) gates_fetch_regs(gv[rt], p.A, p.k, T, B, t - 1, bt0 + rt, tid);
      } else {
        if (staged) gates_stage(gl[cur] + rt * 16 * GATE_KMAX, p.A, p.k, T, B, t, bt0 + rt, tid);
      }
      write_operand<NC>(xb(cur, rt), g, w, q, n);
      publish_rowsum<NC>(psum[cur][rt], g, w, q, n);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const bf16x4 pk = {(__bf16)g[0][c], (__bf16)g[1][c], (__bf16)g[2][c], (__bf16)g[3][c]};
        if (t & 1) {
          if constexpr (HOLD_LDS) held_lds[(rt * NC + c) * 256 + tid] = pk;
          else held[rt][c] = pk;
        } else if (live) {
          bf16x4 hi;
          if constexpr (HOLD_LDS) hi = held_lds[(rt * NC + c) * 256 + tid];
          else hi = held[rt][c];
          *reinterpret_cast<bf16x8*>(p.gfrag + pair_offset<NC>(t, p.nbt, bt0 + rt, w * NC + c, lane)) =
              __builtin_shufflevector(pk, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
      }
    }
    lds_barrier();
    const float* glt = staged ? gl[cur] : nullptr;
    const unsigned long long active = staged ? gates_active(gl[cur], p.k, lane, RT) : ~0ull;

    if constexpr (GA) {
      // the shares of step t+1 are complete (every wave passed the barrier above after writing them)
      if (t + 1 < T) bptt_flush_grad_A(p, ga_buf + (cur ^ 1) * p.k * 64, t + 1, bt0, tid);
      float rp[4][NC];
      rows_load<NC>(t == 0 ? p.r_init : p.hist + (size_t)(t - 1) * B * N, N, B, b0, i0, rp);
      gated_products<NC, true, 1>(xb(cur, 0), wsrc, p.A, glt, active, p.k, T, B, t, b0, p.J1, w, lane,
                                  acc, wf, false, false, rp, ga_buf + cur * p.k * 64, true);
    } else {
      gated_products<NC, false, RT>(xb(cur, 0), wsrc, p.A, glt, active, p.k, T, B, t, b0, p.J1, w,
                                    lane, acc, wf, false, false, nullptr, nullptr, true);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      // the other gate buffer was last read during the previous step's products, before this step's barrier
      if (GATE_PIPE && staged && t > 0) gates_publish_regs(gl[cur ^ 1] + rt * 16 * GATE_KMAX, gv[rt], p.k, tid);
      float s[4];
      read_rowsum(psum[cur][rt], q, s);
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const bool ok = (b0 + 16 * rt + e < B) && (i0 + c < N);
          carry[rt][e][c] = ok ? (acc[rt][c][e] + p.J0 * s[e]) : 0.f;
        }
    }
  }
  if constexpr (GA) {
    lds_barrier();
    bptt_flush_grad_A(p, ga_buf + ((T - 1) & 1) * p.k * 64, 0, bt0, tid);
  }
  if (p.grad_r_init) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) rows_store<NC>(p.grad_r_init, N, B, b0 + 16 * rt, i0, carry[rt]);
  }
}

// ------------------------------------------------------------------------------------------------
// Weight gradients: dW_mm[i][j] = sum over samples (b,t) of coef_mm(b,t) * g[t,b,i] * r_prev[t,b,j]
// (coef_0 = 1 here, J1 is applied in the reduction; coef_{1+c} = A[b,t,c]).
// A K chunk is 16 batch rows x 2 time steps = 32 samples; MFMA fragments come straight from the
// tile-ordered gfrag / rfrag buffers.  Each wave owns 2 row tiles x TJ column tiles x 3 matrices
// over one K split and writes its fp32 partial; no atomics, fixed reduction order afterwards.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ bf16x8 join8(bf16x4 lo, bf16x4 hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ bf16x8 gate8(bf16x8 x, const float (&cf)[8]) {
  bf16x8 o;
#pragma unroll
  for (int u = 0; u < 8; ++u) o[u] = (__bf16)((float)x[u] * cf[u]);
  return o;
}

template <int NC, int TJ>
__global__ __launch_bounds__(256) void ring_dw_kernel(RingDwArgs p) {
  constexpr int NT = 4 * NC;       // 16-wide tiles per matrix side
  constexpr int NIP = NT / 2;      // row-tile pairs
  constexpr int NJO = NT / TJ;     // column-tile groups
  const int lane = threadIdx.x & 63, q = lane >> 4;
  const int nmg = (p.k + 3) / 3;   // groups of 3 matrices
  long wid = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int ip = (int)(wid % NIP);
  wid /= NIP;
  const int jo = (int)(wid % NJO);
  wid /= NJO;
  const int mg = (int)(wid % nmg);
  const int z = (int)(wid / nmg);
  if (z >= p.nz) return;

  const int T = p.T, B = p.B, k = p.k, nbt = p.nbt;
  const int TP = (T + 1) / 2;
  const long nchunk = (long)nbt * TP;
  const long ch0 = nchunk * z / p.nz, ch1 = nchunk * (z + 1) / p.nz;

  f32x4 acc[3][2][TJ];
#pragma unroll
  for (int a = 0; a < 3; ++a)
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
      for (int u = 0; u < TJ; ++u) acc[a][ii][u] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bf16x4 zero4 = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
  for (long ch = ch0; ch < ch1; ++ch) {
    const int bt = (int)(ch % nbt);
    const int t0 = 2 * (int)(ch / nbt), t1 = t0 + 1;
    const bool has1 = t1 < T;
    bf16x8 ga[2], rb[TJ];
#pragma unroll
    for (int ii = 0; ii < 2; ++ii) {
      ga[ii] = *reinterpret_cast<const bf16x8*>(p.gfrag + pair_offset<NC>(t0, nbt, bt, 2 * ip + ii, lane));
      if (!has1) ga[ii] = join8(__builtin_shufflevector(ga[ii], ga[ii], 0, 1, 2, 3), zero4);
    }
#pragma unroll
    for (int u = 0; u < TJ; ++u) {
      rb[u] = *reinterpret_cast<const bf16x8*>(p.rfrag + pair_offset<NC>(t0, nbt, bt, jo * TJ + u, lane));
      if (!has1) rb[u] = join8(__builtin_shufflevector(rb[u], rb[u], 0, 1, 2, 3), zero4);
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int mm = 3 * mg + a;
      if (mm > k) break;
      bf16x8 gg[2];
      if (mm == 0) {
        gg[0] = ga[0];
        gg[1] = ga[1];
      } else {
        float cf[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int b = 16 * bt + 4 * q + e;
          cf[e] = (b < B) ? p.A[((size_t)b * T + t0) * k + (mm - 1)] : 0.f;
          cf[4 + e] = (b < B && has1) ? p.A[((size_t)b * T + t1) * k + (mm - 1)] : 0.f;
        }
        gg[0] = gate8(ga[0], cf);
        gg[1] = gate8(ga[1], cf);
      }
#pragma unroll
      for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int u = 0; u < TJ; ++u) acc[a][ii][u] = mfma16(gg[ii], rb[u], acc[a][ii][u]);
    }
  }

#pragma unroll
  for (int a = 0; a < 3; ++a) {
    const int mm = 3 * mg + a;
    if (mm > k) break;
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
      for (int u = 0; u < TJ; ++u) {
        const int it = 2 * ip + ii, jt = jo * TJ + u;
        p.partial[((((size_t)z * (k + 1) + mm) * NT + it) * NT + jt) * 64 + lane] = acc[a][ii][u];
      }
  }
}

// Fixed-order sum of the K-split partials, undoing the tile permutation, accumulated into the
// caller's grad_Wo / grad_Wa (which the caller zeroed, cpp/ring_rnn_cuda.py:98-99) or written over them.
__global__ __launch_bounds__(256) void ring_dw_reduce_kernel(RingDwArgs p, int NC) {
  const int NT = 4 * NC;
  const size_t per_z = (size_t)(p.k + 1) * NT * NT * 64;
  const size_t u = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (u >= per_z) return;
  // fixed summation order z = 0, 1, 2, ...; the loads of sixteen slices are issued together
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  int z = 0;
  for (; z + 16 <= p.nz; z += 16) {
    f32x4 v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = __builtin_nontemporal_load(&p.partial[(size_t)(z + i) * per_z + u]);
#pragma unroll
    for (int i = 0; i < 16; ++i) s += v[i];
  }
  for (; z < p.nz; ++z) s += p.partial[(size_t)z * per_z + u];
  const int lane = (int)(u & 63);
  size_t v = u >> 6;
  const int jt = (int)(v % NT);
  v /= NT;
  const int it = (int)(v % NT);
  const int mm = (int)(v / NT);
  const int q = lane >> 4, n = lane & 15;
  const int j = 16 * NC * (jt / NC) + NC * n + (jt % NC);
  if (j >= p.N) return;
  float* out = (mm == 0) ? p.grad_Wo : p.grad_Wa + (size_t)(mm - 1) * p.N * p.N;
  const float scale = (mm == 0) ? p.J1 : 1.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int i = 16 * NC * (it / NC) + NC * (4 * q + e) + (it % NC);
    if (i < p.N) {
      float* o = out + (size_t)i * p.N + j;
      *o = p.accumulate ? *o + scale * s[e] : scale * s[e];
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Optional per-launch HIP event bracketing (benchmarks only).
// ------------------------------------------------------------------------------------------------
#include <cxxabi.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <mutex>
#include <string>
#include <vector>
namespace {
constexpr int PROF_SLOTS = 8;
thread_local int t_kernel_slot = -1;                     // innermost open ProfScope of this thread
std::atomic<const void*> g_last_kernel[PROF_SLOTS];      // host function of the last launch per slot
struct ProfRec { hipEvent_t a, b; int id; };
std::mutex g_prof_mu;
std::vector<ProfRec> g_prof;
int g_prof_stride = 0;                       // 0: off; n: every n-th launch of each kernel is bracketed
long g_prof_seen[PROF_SLOTS] = {0, 0, 0, 0, 0, 0, 0, 0};

struct ProfScope {
  hipStream_t st;
  ProfRec rec;
  bool active;
  int outer;
  ProfScope(int id, hipStream_t s) : st(s), active(false), outer(t_kernel_slot) {
    t_kernel_slot = id;
    if (g_prof_stride <= 0) return;
    {
      std::lock_guard<std::mutex> lk(g_prof_mu);
      if (g_prof_seen[id]++ % g_prof_stride != 0) return;
    }
    if (hipEventCreate(&rec.a) != hipSuccess) return;
    if (hipEventCreate(&rec.b) != hipSuccess) { (void)hipEventDestroy(rec.a); return; }
    rec.id = id;
    active = true;
    (void)hipEventRecord(rec.a, st);
  }
  ~ProfScope() {
    t_kernel_slot = outer;
    if (!active) return;
    (void)hipEventRecord(rec.b, st);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof.push_back(rec);
  }
};
}  // namespace

void ring_note_kernel(const void* host_function) {
  const int slot = t_kernel_slot;
  if (slot >= 0 && slot < PROF_SLOTS) g_last_kernel[slot].store(host_function, std::memory_order_relaxed);
}

int ring_last_kernel_name(int id, char* buf, size_t n) {
  if (!buf || n == 0) return -1;
  buf[0] = 0;
  if (id < 0 || id >= PROF_SLOTS) return -1;
  const void* fn = g_last_kernel[id].load(std::memory_order_relaxed);
  if (!fn) return 0;
  const char* mangled = hipKernelNameRefByPtr(fn, nullptr);
  if (!mangled) return -1;
  int status = 0;
  char* dem = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
  std::string name = (status == 0 && dem) ? dem : mangled;
  free(dem);
  if (name.rfind("void ", 0) == 0) name.erase(0, 5);
  // cut the parameter list: the first '(' outside the template argument list
  int depth = 0;
  for (size_t i = 0; i < name.size(); ++i) {
    if (name[i] == '<') ++depth;
    else if (name[i] == '>') --depth;
    else if (name[i] == '(' && depth == 0) { name.erase(i); break; }
  }
  std::string out;
  for (char c : name) if (c != ' ') out.push_back(c);
  strncpy(buf, out.c_str(), n - 1);
  buf[n - 1] = 0;
  return (int)out.size();
}

void ring_profile_set(int stride) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof_stride = stride > 0 ? stride : 0;
  for (long& c : g_prof_seen) c = 0;
}
bool ring_profile_on() { return g_prof_stride > 0; }

hipError_t ring_profile_collect(double* ms, long long* launches) {
  std::vector<ProfRec> recs;
  {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    recs.swap(g_prof);
  }
  hipError_t first = hipSuccess;
  for (auto& r : recs) {
    float t = 0.f;
    hipError_t e = hipEventSynchronize(r.b);
    if (e == hipSuccess) e = hipEventElapsedTime(&t, r.a, r.b);
    if (e == hipSuccess) {
      ms[r.id] += t;
      launches[r.id] += 1;
    } else if (first == hipSuccess) {
      first = e;
    }
    (void)hipEventDestroy(r.a);
    (void)hipEventDestroy(r.b);
  }
  return first;
}

// ------------------------------------------------------------------------------------------------
// Launchers (host).  NC is chosen by the caller as the smallest of {1,2,4,8} with 64*NC >= N.
// ------------------------------------------------------------------------------------------------
#define RING_DISPATCH_ACT(ACTv, CALL)                          \
  switch (ACTv) {                                              \
    case ACT_RELU: { constexpr int ACT = ACT_RELU; CALL; } break; \
    case ACT_GELU: { constexpr int ACT = ACT_GELU; CALL; } break; \
    case ACT_TANH: { constexpr int ACT = ACT_TANH; CALL; } break; \
    case ACT_SILU: { constexpr int ACT = ACT_SILU; CALL; } break; \
    default: return hipErrorInvalidValue;                      \
  }

#define RING_DISPATCH_NC(NCv, CALL)                 \
  switch (NCv) {                                    \
    case 1: { constexpr int NC = 1; CALL; } break;  \
    case 2: { constexpr int NC = 2; CALL; } break;  \
    case 4: { constexpr int NC = 4; CALL; } break;  \
    case 8: { constexpr int NC = 8; CALL; } break;  \
    default: return hipErrorInvalidValue;           \
  }

hipError_t ring_launch_pack2(const float* Wo, const float* Wa, int N, int k, int NC, void* out, int transposed,
                             int split_k, float scale0, float shift0, void* out2, int transposed2, int split_k2,
                             float scale2, float shift2, hipStream_t st) {
  auto order_ok = [&](int sk) { return sk == 0 || (sk == 1 && NC == 4) || ((sk == 2 || sk == 3) && NC == 8); };
  if (!order_ok(split_k) || (out2 && !order_ok(split_k2))) return hipErrorInvalidValue;
  const size_t total = (size_t)(1 + k) * 4 * NC * 2 * NC * 64 * (out2 ? 2 : 1);
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  ProfScope prof(0, st);
  RING_LAUNCH(ring_pack_weights_kernel, dim3(blocks), dim3(256), 0, st, Wo, Wa, (bf16x8*)out, (bf16x8*)out2, N, k,
                     NC, transposed, split_k, scale0, shift0, transposed2, split_k2, scale2, shift2);
  return hipGetLastError();
}

hipError_t ring_launch_pack(const float* Wo, const float* Wa, void* out, int N, int k, int NC, int transposed,
                            int split_k, float scale0, float shift0, hipStream_t st) {
  return ring_launch_pack2(Wo, Wa, N, k, NC, out, transposed, split_k, scale0, shift0, nullptr, 0, 0, 1.f, 0.f, st);
}

// RINGATTR_STREAMING=1 forces the generic weight-streaming kernels (used by tests to cross-check).
bool ring_uses_resident(int N, int k) {
  if (!ring_res256_applicable(N, k)) return false;
  const char* v = getenv("RINGATTR_STREAMING");
  return !(v && v[0] == '1');
}

// Batch tiles per workgroup of the streaming kernels.  A step of these kernels is bound by the weight
// bytes a compute unit can pull from L2, and two tiles share every fetched fragment; pairing pays when
// the workgroups would otherwise run in more rounds than the paired ones (more tiles than compute units).
// RINGATTR_ROW_TILES=1|2 overrides the choice (tests cross-check the two forms).
static int stream_row_tiles(int NCv, int nbt, bool one_workgroup_per_step) {
  if (NCv < 4 || nbt < 2) return 1;
  const char* v = getenv("RINGATTR_ROW_TILES");
  if (v && (v[0] == '1' || v[0] == '2')) return v[0] - '0';
  if (one_workgroup_per_step) return NCv >= 8 ? 2 : 1;   // a grid of tiles x steps fills the device; pairing pays at the widest tiling
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus = n;
  }
  const long rounds1 = (nbt + cus - 1) / cus, rounds2 = ((nbt + 1) / 2 + cus - 1) / cus;
  return 4 * rounds2 < 3 * rounds1 ? 2 : 1;    // a paired step takes about 1.4 times a single one
}

template <typename K, typename Args>
static hipError_t launch_stream(K kern, dim3 grid, size_t dyn, hipStream_t st, const Args& a) {
  if (dyn > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
    if (e != hipSuccess) return e;
  }
  RING_LAUNCH(kern, grid, dim3(256), dyn, st, a);
  return hipGetLastError();
}

#define RING_DISPATCH_RT(RTv, CALL)                                         \
  if ((RTv) == 2) { constexpr int RT = 2; if constexpr (NC >= 4) { CALL; } } \
  else { constexpr int RT = 1; CALL; }

// LDS-resident weights for the streaming kernels: everything must fit next to the operand buffers, the gate
// stage and (BPTT with dL/dA) the per-wave shares.  RINGATTR_LDS_WEIGHTS=0 keeps the weights in L2 (tests).
static bool weights_fit_lds(int NCv, int k, size_t other_dynamic) {
  if (NCv > 2) return false;
  const char* v = getenv("RINGATTR_LDS_WEIGHTS");
  if (v && v[0] == '0') return false;
  const size_t wb = NCv == 1 ? packed_weight_bytes<1>(k) : packed_weight_bytes<2>(k);
  return wb + other_dynamic + 20 * 1024 <= 128 * 1024;   // 20 KiB: static LDS of these kernels, rounded up
}

// Which time loop runs a problem that keeps a saved record (forward and backward must agree: the record's layout
// differs between the persistent and the step-per-launch families).  Wide rings have only the step-per-launch
// kernels; RINGATTR_BLOCK=1 / 0 forces / forbids them where the persistent streaming kernels also apply.
bool ring_uses_step_kernels(int N, int k, int NCv, int nbt) {
  if (NCv > 8) return true;
  if (NCv < 4 || ring_uses_resident(N, k)) return false;
  const char* v = getenv("RINGATTR_BLOCK");
  if (v && (v[0] == '0' || v[0] == '1')) return v[0] == '1';
  (void)nbt;
  return false;
}

// Which step-per-launch family.  With few matrices the block kernels (K-outer, three matrices' products at a time)
// are ahead on few batch tiles and the one-tile-per-workgroup kernels of ring_bign.hip (up to 1.6 times) on many;
// measured crossover about nbt * NC = 512 (N = 1024: 512 rows, N = 2048: 256 rows).  With many matrices (16 action
// channels) the block kernels lead at every measured batch size (1.3 to 2 times).  RINGATTR_WIDE=1 / 0 forces one or
// the other (cross-checks); the two share the record layout, so forward and backward may choose independently.
static bool step_prefers_wide(int NCv, int nbt, int k) {
  if (NCv % 4 != 0) return false;
  const char* v = getenv("RINGATTR_WIDE");
  if (v && (v[0] == '0' || v[0] == '1')) return v[0] == '1';
  if (ring_block_many_matrices(k)) return false;
  return (long)nbt * NCv > 512;
}

// Does ring_launch_fwd fill a.loss_stats for this problem?  The persistent kernels do; the step-per-launch ones
// (wide rings, and the split forward of small batches) do not.
bool ring_fwd_forms_loss_sums(const RingFwdArgs& a, int NCv) {
  if (ring_uses_step_kernels(a.N, a.k, NCv, a.nbt)) return false;
  if (a.cluster_ws) return false;
  if (!a.dfrag && !a.rfrag && NCv >= 4 && a.nbt <= 64 && !ring_uses_resident(a.N, a.k)) {
    const char* v = getenv("RINGATTR_SPLIT_FORWARD");
    if (!(v && v[0] == '0')) return false;
  }
  return true;
}

hipError_t ring_launch_fwd(const RingFwdArgs& a, int NCv, hipStream_t st) {
  // the kernels write the derivative record and the operand copy together: both or neither
  if ((a.dfrag != nullptr) != (a.rfrag != nullptr)) return hipErrorInvalidValue;
  ProfScope prof(1, st);
  if (ring_uses_step_kernels(a.N, a.k, NCv, a.nbt))
    return step_prefers_wide(NCv, a.nbt, a.k) ? ring_launch_wide_fwd(a, NCv, false, 4, st) : ring_launch_block_fwd(a, NCv, false, st);
  if (a.cluster_ws) return ring_launch_fwd_cluster(a, st);   // (the caller's choice: ring_uses_cluster)
  // A forward that keeps nothing for a backward, on few batch tiles, with weights too large to stay on chip: the
  // persistent kernels would pull every weight byte through a handful of compute units once per step.  One launch per
  // step with the output columns split over workgroups spreads that over the device (a launch costs a few
  // microseconds, the step it replaces tens).  RINGATTR_SPLIT_FORWARD=0 keeps the persistent kernel (tests).
  if (!a.dfrag && !a.rfrag && NCv >= 4 && a.nbt <= 64 && !ring_uses_resident(a.N, a.k)) {
    const char* v = getenv("RINGATTR_SPLIT_FORWARD");
    if (!(v && v[0] == '0')) {
      const int tpw = a.nbt * NCv >= 512 ? 4 : (a.nbt * NCv >= 256 ? 2 : 1);   // aim at >= 128 workgroups
      return ring_launch_wide_fwd(a, NCv, false, tpw, st);
    }
  }
  if (ring_uses_resident(a.N, a.k)) return ring_launch_fwd_res256(a, st);
  const int rt = stream_row_tiles(NCv, a.nbt, false);
  hipError_t e = hipErrorInvalidValue;
  if (weights_fit_lds(NCv, a.k, 8 * 1024)) {
    if (a.loss_stats) {
      RING_DISPATCH_NC(NCv, RING_DISPATCH_ACT(a.act, if constexpr (NC <= 2)
          e = launch_stream(ring_fwd_kernel<NC, ACT, 1, true, true>, dim3(a.nbt), stream_lds_bytes<NC, 1>() + packed_weight_bytes<NC>(a.k), st, a)));
      return e;
    }
    RING_DISPATCH_NC(NCv, RING_DISPATCH_ACT(a.act, if constexpr (NC <= 2)
        e = launch_stream(ring_fwd_kernel<NC, ACT, 1, true, false>, dim3(a.nbt), stream_lds_bytes<NC, 1>() + packed_weight_bytes<NC>(a.k), st, a)));
    return e;
  }
  if (a.loss_stats) {
    RING_DISPATCH_NC(NCv, RING_DISPATCH_ACT(a.act, RING_DISPATCH_RT(rt,
        e = launch_stream(ring_fwd_kernel<NC, ACT, RT, false, true>, dim3((a.nbt + RT - 1) / RT),
                          stream_lds_bytes<NC, RT>() + fwd_state_lds_bytes<NC, RT>(), st, a))));
    return e;
  }
  RING_DISPATCH_NC(NCv, RING_DISPATCH_ACT(a.act, RING_DISPATCH_RT(rt,
      e = launch_stream(ring_fwd_kernel<NC, ACT, RT, false, false>, dim3((a.nbt + RT - 1) / RT),
                        stream_lds_bytes<NC, RT>() + fwd_state_lds_bytes<NC, RT>(), st, a))));
  return e;
}

// For the weight-resident geometry the saved record is rebuilt by running the forward recurrence again
// from r_init with its history stores switched off (a.hist is not read): the same kernel, the same
// numbers the forward would have saved, and no pass over the weights per (batch tile, step).
hipError_t ring_launch_rebuild(const RingFwdArgs& a, int NCv, hipStream_t st) {
  if (!a.dfrag || !a.rfrag) return hipErrorInvalidValue;
  ProfScope prof(2, st);
  if (ring_uses_step_kernels(a.N, a.k, NCv, a.nbt))
    return step_prefers_wide(NCv, a.nbt, a.k) ? ring_launch_wide_fwd(a, NCv, true, 4, st) : ring_launch_block_fwd(a, NCv, true, st);
  if (ring_uses_resident(a.N, a.k)) {
    RingFwdArgs f = a;
    f.hist = nullptr;
    return ring_launch_fwd_res256(f, st);
  }
  const int rt = stream_row_tiles(NCv, a.nbt, true);
  hipError_t e = hipErrorInvalidValue;
  // widest tiling, staged gates, more than one step and batch tile: four row tiles (two batch tiles x two steps)
  // share every fetched weight fragment.  RINGATTR_REBUILD_TILES=2 keeps the two-tile kernel (cross-checks).
  static const bool four = [] { const char* v = getenv("RINGATTR_REBUILD_TILES"); return !(v && v[0] == '2'); }();
  if (four && NCv == 8 && rt == 2 && a.k <= GATE_KMAX && a.T >= 2) {
    constexpr int NC = 8;
    RING_DISPATCH_ACT(a.act, e = launch_stream(ring_rebuild_saved4_kernel<NC, ACT>, dim3((a.nbt + 1) / 2, (a.T + 1) / 2),
                                               4 * Tile<NC>::SLOTS * sizeof(bf16x8), st, a));
    return e;
  }
  RING_DISPATCH_NC(NCv, RING_DISPATCH_ACT(a.act, RING_DISPATCH_RT(rt,
      e = launch_stream(ring_rebuild_saved_kernel<NC, ACT, RT>, dim3((a.nbt + RT - 1) / RT, a.T), 0, st, a))));
  return e;
}

template <int NC, bool GA, int RT, bool WL>
static hipError_t launch_bptt_stream(const RingBpttArgs& a, dim3 grid, size_t dyn, hipStream_t st) {
  return a.loss_coef ? launch_stream(ring_bptt_kernel<NC, GA, RT, true, WL>, grid, dyn, st, a)
                     : launch_stream(ring_bptt_kernel<NC, GA, RT, false, WL>, grid, dyn, st, a);
}

hipError_t ring_launch_bptt(const RingBpttArgs& a, int NCv, hipStream_t st) {
  ProfScope prof(3, st);
  hipError_t e = hipErrorInvalidValue;
  if (a.cluster_ws) return ring_launch_bptt_cluster(a, st);   // (the caller's choice: ring_uses_cluster_bptt)
  if (ring_uses_step_kernels(a.N, a.k, NCv, a.nbt)) {
    if (a.grad_A || !a.wide_carry) return hipErrorInvalidValue;   // (dL/dA comes from a pass of its own, see the C ABI)
    return step_prefers_wide(NCv, a.nbt, a.k) ? ring_launch_wide_bptt(a, NCv, a.wide_carry, st)
                                  : ring_launch_block_bptt(a, NCv, a.wide_carry, st);
  }
  // (the parentheses keep the commas of the template argument lists away from the dispatch macros)
  if (a.grad_A && !ring_uses_resident(a.N, a.k)) {   // the streaming kernel's dL/dA variant
    const size_t ga = (size_t)2 * a.k * 64 * sizeof(float);
    if (weights_fit_lds(NCv, a.k, 8 * 1024 + ga)) {
      RING_DISPATCH_NC(NCv, if constexpr (NC <= 2) (e = launch_bptt_stream<NC, true, 1, true>(
          a, dim3(a.nbt), stream_lds_bytes<NC, 1>() + ga + packed_weight_bytes<NC>(a.k), st)));
    } else {
      RING_DISPATCH_NC(NCv, (e = launch_bptt_stream<NC, true, 1, false>(a, dim3(a.nbt), stream_lds_bytes<NC, 1>() + ga, st)));
    }
    return e;
  }
  if (ring_uses_resident(a.N, a.k)) return ring_launch_bptt_res256(a, st);
  if (weights_fit_lds(NCv, a.k, 8 * 1024)) {
    RING_DISPATCH_NC(NCv, if constexpr (NC <= 2) (e = launch_bptt_stream<NC, false, 1, true>(
        a, dim3(a.nbt), stream_lds_bytes<NC, 1>() + packed_weight_bytes<NC>(a.k), st)));
    return e;
  }
  const int rt = stream_row_tiles(NCv, a.nbt, false);
  RING_DISPATCH_NC(NCv, RING_DISPATCH_RT(rt, (e = launch_bptt_stream<NC, false, RT, false>(
      a, dim3((a.nbt + RT - 1) / RT), stream_lds_bytes<NC, RT>(), st))));
  return e;
}

hipError_t ring_launch_dw(const RingDwArgs& a, int NCv, hipStream_t st) {
  const int NT = 4 * NCv;
  const int TJ = NCv == 1 ? 4 : 8;
  const long waves = (long)(NT / 2) * (NT / TJ) * ((a.k + 3) / 3) * a.nz;
  const int blocks = (int)((waves + 3) / 4);
  hipError_t e;
  {
  ProfScope prof(4, st);
  if (ring_dw_tiled_applicable(NCv)) {
    e = ring_launch_dw_tiled(a, NCv, st);   // every group's launch status, first failure wins
  } else {
    if (NCv == 1) {
      RING_LAUNCH((ring_dw_kernel<1, 4>), dim3(blocks), dim3(256), 0, st, a);
    } else {
      RING_DISPATCH_NC(NCv, if constexpr (NC >= 2) RING_LAUNCH((ring_dw_kernel<NC, 8>), dim3(blocks), dim3(256), 0, st, a));
    }
    e = hipGetLastError();
  }
  }
  if (e != hipSuccess) return e;   // the reduction must not sum partials that were never written
  const size_t per_z = (size_t)(a.k + 1) * NT * NT * 64;
  ProfScope prof(5, st);
  RING_LAUNCH(ring_dw_reduce_kernel, dim3((unsigned)((per_z + 255) / 256)), dim3(256), 0, st, a, NCv);
  return hipGetLastError();
}
