// Weight-resident kernels for the headline geometry: 128 < N <= 256 (NPAD = 256, NC = 4), a_dim = 2.
//
// [Wo|Wl|Wr] in bf16 is 384 KiB -- more than one CU's LDS (160 KiB) but less than its register
// file (512 KiB).  A workgroup keeps the slices of the two gated matrices in registers for the whole
// sequence (accumulation VGPRs, which MFMA reads as B operands) and the Wo slices in LDS (128 KiB per
// workgroup, each read back by the lane that wrote it), so no weight byte is fetched from L2/HBM inside
// the time loop.  One workgroup per CU and 16 batch rows per workgroup; the forward runs eight waves
// (two per SIMD, in two roles half a step apart), BPTT four (one per SIMD).
#include "ring_common.hpp"
#include "ring_kernels.hpp"

#include <type_traits>

namespace {

constexpr int R_NC = 4;
constexpr int R_KCH = 8;
constexpr int R_WLDS_SLOTS = 4 * R_NC * R_KCH * 64;   // 16-byte slots of the LDS-resident matrix
constexpr int R_XSLOTS = R_KCH * 4 * XG;
constexpr int R_GCH = 32;                             // time steps of action gates staged per LDS chunk
constexpr int R_BPTT_DEPTH_MAX = 4;                   // BPTT steps whose grad_output / F' loads are in flight (template DEPTH <= this)
constexpr size_t R_GA_BYTES = 2 * 2 * 4 * 16 * sizeof(float);   // dL/dA shares: [step parity][channel][wave][row]
constexpr size_t R_LDS_BYTES = (size_t)(R_WLDS_SLOTS + 2 * R_XSLOTS) * 16 + 2 * R_GCH * 16 * 8 + R_GA_BYTES;   // BPTT layout

// Action gates (A[b,t,0], A[b,t,1]) reach the lanes through LDS in chunks of R_GCH steps, so the
// time loop issues no vector-memory load whose wait would also drain the history stores.
// Chunk ci holds loop iterations u = ci*R_GCH + l; iteration u is time step u (dir > 0, forward)
// or T-1-u (dir < 0, BPTT).  Thread (row = tid/16, j = tid%16) moves l = j and l = j + 16.
struct GateStage {
  f32x2 a, b;
};

__device__ __forceinline__ void gates_fetch(const float* A, int T, int B, int bt, int ci, int dir, int tid, GateStage& g) {
  const int row = tid >> 4, j = tid & 15;
  const int b = 16 * bt + row;
  const int bc = b < B ? b : B - 1;
  int u1 = ci * R_GCH + j, u2 = u1 + 16;
  u1 = u1 < T ? u1 : T - 1;
  u2 = u2 < T ? u2 : T - 1;
  const int t1 = dir > 0 ? u1 : T - 1 - u1, t2 = dir > 0 ? u2 : T - 1 - u2;
  const f32x2 va = *reinterpret_cast<const f32x2*>(A + ((size_t)bc * T + t1) * 2);
  const f32x2 vb = *reinterpret_cast<const f32x2*>(A + ((size_t)bc * T + t2) * 2);
  g.a = va;
  g.b = vb;
}

// Rows past the batch get zero gates.  The mask is applied here, not in gates_fetch, so that nothing
// touches the loaded values (and waits for them) until the chunk is actually needed.
__device__ __forceinline__ void gates_publish(f32x2* gb, int tid, int B, int bt, const GateStage& g) {
  const int row = tid >> 4, j = tid & 15;
  const float m = 16 * bt + row < B ? 1.f : 0.f;
  gb[j * 16 + row] = g.a * m;
  gb[(j + 16) * 16 + row] = g.b * m;
}

// Load this wave's resident weight slices: matrix 0 into the lane's own LDS slots, matrices 1 and 2
// into accumulation VGPRs (MFMA reads B operands there directly, which leaves the 256 architectural
// VGPRs to operands, accumulators and the epilogue).
__device__ __forceinline__ void load_resident(const bf16x8* Wp, bf16x8* wl, bf16x8 (&wreg)[2][R_NC][R_KCH], int w, int lane) {
#pragma unroll
  for (int c = 0; c < R_NC; ++c)
#pragma unroll
    for (int kc = 0; kc < R_KCH; ++kc) {
      wl[(c * R_KCH + kc) * 64] = Wp[((size_t)((0 * 4 + w) * R_NC + c) * R_KCH + kc) * 64 + lane];
      wreg[0][c][kc] = Wp[((size_t)((1 * 4 + w) * R_NC + c) * R_KCH + kc) * 64 + lane];
      wreg[1][c][kc] = Wp[((size_t)((2 * 4 + w) * R_NC + c) * R_KCH + kc) * 64 + lane];
      asm volatile("" : "+a"(wreg[0][c][kc]));
      asm volatile("" : "+a"(wreg[1][c][kc]));
    }
}

}  // namespace

// ------------------------------------------------------------------------------------------------
// Forward, weights resident.  Same contract as ring_fwd_kernel<4> with k == 2.
// FULL: N == 256 and B % 16 == 0, no masking anywhere.
//
// One wave issues at most one instruction every four cycles and hides only about two vector-ALU
// instructions under each MFMA, while the epilogue of a step (gating, activation, leak, conversions)
// is several hundred of them.  So the workgroup runs EIGHT waves, two per SIMD, in two roles that
// are half a step out of phase: while one wave of a SIMD is in its vector-ALU epilogue the other one
// feeds the matrix pipe.  Wave (w, h), w = 0..3, h = 0/1, owns column tiles 2h and 2h+1 of neuron
// group w (neurons 64w + 32h + 2n + {0,1}: a row group's 16 lanes cover 32 consecutive neurons, so a history
// store fills whole cache lines); h = 0 is the "early" role E, h = 1 the "late" role L.  The
// contraction index is ordered so that K chunks 0..3 hold the E neurons and 4..7 the L neurons
// (split_k_neuron), and the step t (r_t -> r_{t+1}) is
//      barrier A_t   (r^E_t visible)
//   E: tiles x K chunks 0..3                         L: activation of step t-1 -> r^L_t, stores of t-1
//      barrier B_t   (r^L_t visible)
//   E: tiles x K chunks 4..7, epilogue -> r^E_{t+1}   L: tiles x K chunks 0..7 -> pre-activations of step t
// The E half of the operand tile is double-buffered by step parity (L still reads r^E_t while E
// writes r^E_{t+1}); the L half is written and read in different intervals and needs one buffer.
// The packed Wo slice holds J1 * Wo + J0 (ring_pack_weights_kernel), so the global-inhibition term J0 * sum_j r_j
// and the J1 scale are part of the one product and cost neither row sums nor epilogue arithmetic.
// Registers: 128 AGPRs hold the wave's slices of the two gated matrices, the slice of Wo sits in LDS.
// ------------------------------------------------------------------------------------------------
namespace {

constexpr int R8_HALF_SLOTS = 4 * 4 * XG;   // 16-byte slots of one operand half (4 K chunks)
constexpr size_t R8_STAT_FLOATS = 2 * 8 * 3 * 16;   // loss-head row sums per wave: [step parity][wave][C, S, |r|][row]
constexpr size_t R8_LDS_BYTES = (size_t)(R_WLDS_SLOTS + 3 * R8_HALF_SLOTS) * 16 + 2 * R_GCH * 16 * 8 + R8_STAT_FLOATS * 4;

__device__ __forceinline__ void load_resident8(const bf16x8* Wp, bf16x8* wl, bf16x8 (&wreg)[2][2][R_KCH], int w, int h,
                                               int lane) {
#pragma unroll
  for (int cc = 0; cc < 2; ++cc)
#pragma unroll
    for (int kc = 0; kc < R_KCH; ++kc) {
      const int c = 2 * h + cc;
      wl[(cc * R_KCH + kc) * 64] = Wp[((size_t)((0 * 4 + w) * R_NC + c) * R_KCH + kc) * 64 + lane];
      wreg[0][cc][kc] = Wp[((size_t)((1 * 4 + w) * R_NC + c) * R_KCH + kc) * 64 + lane];
      wreg[1][cc][kc] = Wp[((size_t)((2 * 4 + w) * R_NC + c) * R_KCH + kc) * 64 + lane];
      asm volatile("" : "+a"(wreg[0][cc][kc]));
      asm volatile("" : "+a"(wreg[1][cc][kc]));
    }
}

// bf16 write-back of the wave's tile pair into K chunk w of one operand half.
__device__ __forceinline__ void write_half(bf16x8* half, const float (&v)[4][2], int w, int q, int n) {
  char* base = reinterpret_cast<char*>(half) + (size_t)((w * 4 + (n >> 2)) * XG + 4 * q) * 16 + (n & 3) * 4;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    bf16x2 pk = {(__bf16)v[e][0], (__bf16)v[e][1]};
    *reinterpret_cast<bf16x2*>(base + e * 16) = pk;
  }
}

}  // namespace

// STATS: also leave the loss head's three sums of every history row (sum_i r_i cos(phi_i), sum_i r_i sin(phi_i),
// sum_i |r_i|, phi_i = 2 pi i / N) in p.loss_stats[t * B + b], so that the loss needs no pass of its own over the
// history.  Each wave reduces its 32 neurons' share over the row group's 16 lanes right after the activation, the
// eight shares meet in LDS (buffer by step parity) and wave 0 adds them in wave order behind the next barrier.
template <int ACT, bool SAVE, bool FULL, bool STATS>
__global__ __launch_bounds__(512) void ring_fwd_res256_kernel(RingFwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xE = wlds + R_WLDS_SLOTS;               // two buffers, step parity
  bf16x8* xL = xE + 2 * R8_HALF_SLOTS;
  f32x2* gbuf = reinterpret_cast<f32x2*>(xL + R8_HALF_SLOTS);
  float* statp = reinterpret_cast<float*>(gbuf + 2 * R_GCH * 16);

  const int tid = threadIdx.x, w8 = tid >> 6, h = w8 >> 2, w = w8 & 3, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt = blockIdx.x;
  const int b0 = 16 * bt + 4 * q;
  const int i0 = 64 * w + 32 * h + 2 * n;         // this lane's two neurons: i0, i0 + 1 (one per tile)
  // their slots in the common tile order of the saved buffers: tile ct0 + cc, lane lc (same row group q)
  const int ct0 = 2 * (n & 1), lc = (lane & 48) | (8 * h + (n >> 1));
  const int N = p.N, B = p.B, T = p.T;
  const float oma = 1.f - p.alpha;
  const ActScale asc = act_scale_make(p.alpha);
  constexpr int HK = R_KCH / 2;
  // wave-uniform indices as scalars: store addresses then split into a scalar base and a per-lane constant
  const int wu = __builtin_amdgcn_readfirstlane(w), hu = __builtin_amdgcn_readfirstlane(h);

  bf16x8 wreg[2][2][R_KCH];
  bf16x8* wl = wlds + (size_t)(w8 * 2 * R_KCH) * 64 + lane;
  load_resident8(reinterpret_cast<const bf16x8*>(p.Wpack), wl, wreg, w, h, lane);

  float r[4][2], okf[4][2], d[4][2];
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      const bool ok = (b0 + e < B) && (i0 + cc < N);
      okf[e][cc] = ok ? 1.f : 0.f;
      r[e][cc] = ok ? p.r_init[(size_t)(b0 + e) * N + i0 + cc] : 0.f;
    }
  auto save_r = [&](int t) {   // bf16 copy of r_t (operand of step t) for the weight-gradient GEMM
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      bf16x4 pk = {(__bf16)r[0][cc], (__bf16)r[1][cc], (__bf16)r[2][cc], (__bf16)r[3][cc]};
      *reinterpret_cast<bf16x4*>(p.rfrag + pair_offset<R_NC>(t, p.nbt, bt, w * R_NC + ct0 + cc, lc)) = pk;
    }
  };
  float scs[2] = {0.f, 0.f}, ssn[2] = {0.f, 0.f};
  if constexpr (STATS) {
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) sincosf(6.283185307179586f * (float)(i0 + cc) / (float)N, &ssn[cc], &scs[cc]);
  }
  // r[][] holds this wave's part of history row `row_t` (masked entries are zero): its share of the three sums
  auto stat_share = [&](int row_t) {
    float* dst = statp + (size_t)(((row_t & 1) * 8 + w8) * 3) * 16 + 4 * q;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float c = fmaf(r[e][1], scs[1], r[e][0] * scs[0]);
      float sn = fmaf(r[e][1], ssn[1], r[e][0] * ssn[0]);
      float ab = fabsf(r[e][0]) + fabsf(r[e][1]);
      c = row16_sum_dpp(c);
      sn = row16_sum_dpp(sn);
      ab = row16_sum_dpp(ab);
      if (n == 0) {
        dst[e] = c;
        dst[16 + e] = sn;
        dst[32 + e] = ab;
      }
    }
  };
  // the eight shares of row `row_t` are complete behind a barrier: wave 0 adds them in wave order and stores the row sums
  auto stat_flush = [&](int row_t) {
    if (w8 == 0) {
      const int kind = lane >> 4, row = lane & 15, b = 16 * bt + row;
      float v = 0.f;
      if (kind < 3) {
        const float* src = statp + (size_t)((row_t & 1) * 8 * 3 + kind) * 16 + row;
#pragma unroll
        for (int wv = 0; wv < 8; ++wv) v += src[wv * 3 * 16];
      }
      if (b < B) reinterpret_cast<float*>(p.loss_stats + (size_t)row_t * B + b)[kind] = v;
    }
  };
  write_half(h ? xL : xE, r, w, q, n);
  if (SAVE) {
    save_r(0);
    if (T & 1) {
      const bf16x4 z = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
        *reinterpret_cast<bf16x4*>(p.rfrag + pair_offset<R_NC>(T, p.nbt, bt, w * R_NC + ct0 + cc, lc)) = z;
    }
  }
  GateStage gs;
  if (h == 0) {
    gates_fetch(p.A, T, B, bt, 0, +1, tid, gs);
    gates_publish(gbuf, tid, B, bt, gs);
  }

  // The LDS-resident slice is consumed in units f = 4*ph + 2*cc + j of two fragments (tile cc, chunks
  // 4*ph + 2*j + {0,1}), eight units per step; fragment g = 2*f + u.  An LDS read takes about 130 cycles to land
  // and a fragment's three MFMAs 48.  The unmasked variants (which have the registers to pin the reads early)
  // run the fragments through a ring of four registers filled three fragments ahead of the MFMAs -- across
  // tiles, halves and time steps alike, since the slice never changes; the masked ones fetch unit f + 1 while
  // unit f is multiplied and leave the placement of the reads to the compiler.
  constexpr int UF = 2;
  auto frag_slot = [&](int g) {
    const int f = g >> 1, u = g & 1;
    return ((((f >> 1) & 1) * R_KCH) + (f >> 2) * HK + (f & 1) * UF + u) * 64;
  };
  bf16x8 w0[4];
#pragma unroll
  for (int g = 0; g < (FULL ? 3 : UF); ++g) w0[g] = wl[frag_slot(g)];
  lds_barrier();   // A_0

  // History / F' / operand-copy stores of a finished step are not issued in one burst behind its
  // epilogue (the write path would throttle the wave for the whole burst while the matrix pipe
  // idles) but one at a time between the MFMA groups of the following contraction.  The values stay
  // in r[] and d[] until the next activation.  slot 0..3: history rows, 4..5: F', 6..7: operand copy.
  // Lane-constant byte offsets of the three kinds of store; what varies with the step is wave-uniform and is
  // added on the scalar unit (the unmasked variant addresses every store as scalar base + lane offset + immediate).
  const unsigned hist_lane = (unsigned)((4 * q * 256 + 2 * n) * sizeof(float));           // + row e * 1 KiB
  const unsigned d_lane = (unsigned)((lc * 4 * R_NC + 4 * ct0) * sizeof(_Float16));        // + tile cc * 8 B
  const unsigned r_lane = (unsigned)((ct0 * 64 + lc) * 16);                                // + tile cc * 1 KiB
  auto emit_store = [&](int t, int slot) {
    __builtin_amdgcn_sched_barrier(0);
    if (slot < 4) {
      if (p.hist == nullptr) return;   // recompute of the saved record only: the history already exists
      const int e = slot;
      if constexpr (FULL) {
        char* base = reinterpret_cast<char*>(p.hist + ((size_t)t * B + 16 * bt) * 256 + 64 * wu + 32 * hu);
        *reinterpret_cast<f32x2*>(base + hist_lane + e * 1024) = f32x2{r[e][0], r[e][1]};
      } else {
        float* dst = p.hist + ((size_t)t * B + b0 + e) * N + i0;
        if (okf[e][0] != 0.f) dst[0] = r[e][0];
        if (okf[e][1] != 0.f) dst[1] = r[e][1];
      }
    } else if (slot < 6) {
      // the lane's two tiles lie side by side in the record: one 16-byte store (slot 4), whole 32-byte sectors per
      // lane pair; two 8-byte stores would each write every other 8 bytes, and a store of partial sectors costs the
      // wave several times what a whole one costs
      if (SAVE && slot == 4) {
        typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
        char* base = reinterpret_cast<char*>(p.dfrag + side_offset<R_NC>(t, p.nbt, bt, wu, 0));
        const f16x8 pk = {(_Float16)d[0][0], (_Float16)d[1][0], (_Float16)d[2][0], (_Float16)d[3][0],
                          (_Float16)d[0][1], (_Float16)d[1][1], (_Float16)d[2][1], (_Float16)d[3][1]};
        *reinterpret_cast<f16x8*>(base + d_lane) = pk;
      }
    } else if (SAVE) {
      const int cc = slot - 6;   // r after step t is the operand of step t+1
      char* base = reinterpret_cast<char*>(p.rfrag + pair_offset<R_NC>(t + 1, p.nbt, bt, wu * R_NC, 0));
      bf16x4 pk = {(__bf16)r[0][cc], (__bf16)r[1][cc], (__bf16)r[2][cc], (__bf16)r[3][cc]};
      *reinterpret_cast<bf16x4*>(base + r_lane + cc * 1024) = pk;
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  f32x4 P[2][3];
  auto mfma_unit = [&](int f, const bf16x8 (&af)[HK]) {
    const int cc = (f >> 1) & 1, ph = f >> 2, j = f & 1;
    if constexpr (!FULL) {
#pragma unroll
      for (int u = 0; u < UF; ++u) w0[((f + 1) & 1) * UF + u] = wl[frag_slot((2 * (f + 1) + u) & 15)];
    }
#pragma unroll
    for (int u = 0; u < UF; ++u) {
      const int g = 2 * f + u, kl = j * UF + u, kc = ph * HK + kl;
      if constexpr (FULL) {
        w0[(g + 3) & 3] = wl[frag_slot((g + 3) & 15)];
        // keep the read where it is: left alone it sinks towards its use and the distance is gone
        __builtin_amdgcn_sched_barrier(0);
      }
      P[cc][1] = mfma16(af[kl], wreg[0][cc][kc], P[cc][1]);
      P[cc][2] = mfma16(af[kl], wreg[1][cc][kc], P[cc][2]);
      P[cc][0] = mfma16(af[kl], w0[g & 3], P[cc][0]);
      if constexpr (FULL) __builtin_amdgcn_sched_barrier(0);
    }
  };
  // K chunks 0..3 (ph = 0, from the E buffer of this step's parity) or 4..7 (ph = 1, from the L half);
  // with emit, four of the eight pending stores of step ts go out between the MFMA groups.
  auto contract_half = [&](int ph, const bf16x8* half, int ts, auto emit) {
    bf16x8 af[HK];
    const bf16x8* xrow = half + q * XG + n;
#pragma unroll
    for (int u = 0; u < HK; ++u) af[u] = xrow[u * 4 * XG];
    if (ph == 0) {
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) P[cc][0] = P[cc][1] = P[cc][2] = z;
    }
    // The two waves of a SIMD share one issue port for vector-ALU and MFMA instructions, and the arbiter serves
    // the older wave first: without a hint a wave in its (long, dense) activation starves the other one's MFMAs
    // and the matrix pipe idles until the activation is over.  A wave that is contracting asks for priority.
    __builtin_amdgcn_s_setprio(3);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (decltype(emit)::value) emit_store(ts, 4 * ph + j);
      mfma_unit(4 * ph + j, af);
    }
    __builtin_amdgcn_s_setprio(0);
  };
  // x[e][cc] = P0 + a0*P1 + a1*P2 with the gates of step t (P0 already holds J0*rowsum + J1*(Wo r))
  auto preactivation = [&](int t, float (&x)[4][2]) {
    const f32x2* gb = gbuf + (((t / R_GCH) & 1) * R_GCH + t % R_GCH) * 16 + 4 * q;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const f32x2 gate = gb[e];
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        const float v = fmaf(gate[0], P[cc][1][e], P[cc][0][e]);
        x[e][cc] = fmaf(gate[1], P[cc][2][e], v);
      }
    }
  };
  auto activate = [&](const float (&x)[4][2]) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        float aF, aD;
        act_scaled<ACT>(x[e][cc], asc, aF, aD);
        float rn = fmaf(oma, r[e][cc], aF);
        if constexpr (!FULL) {
          rn *= okf[e][cc];
          aD *= okf[e][cc];
        }
        r[e][cc] = rn;
        d[e][cc] = aD;          // the saved record is alpha * F'(re)
      }
  };
  constexpr std::true_type with_stores{};
  constexpr std::false_type no_stores{};
  if (h == 0) {
    // ---------------- role E ----------------
    auto e_step = [&](int t, auto emit) {
      const int ci = t / R_GCH, l = t % R_GCH;
      if (l == 0 && (ci + 1) * R_GCH < T) gates_fetch(p.A, T, B, bt, ci + 1, +1, tid, gs);
      contract_half(0, xE + (t & 1) * R8_HALF_SLOTS, t - 1, emit);
      lds_barrier();   // B_t
      if constexpr (STATS) {
        if (t > 0) stat_flush(t - 1);            // both roles' shares of row t-1 are in
      }
      contract_half(1, xL, t - 1, emit);
      float x[4][2];
      preactivation(t, x);
      activate(x);
      if constexpr (STATS) stat_share(t);
      if (t + 1 < T) write_half(xE + ((t + 1) & 1) * R8_HALF_SLOTS, r, w, q, n);
      // the next chunk's gates are first read after barrier B of its first step
      if (l == R_GCH - 1 && t + 1 < T) gates_publish(gbuf + ((ci + 1) & 1) * R_GCH * 16, tid, B, bt, gs);
      lds_barrier();   // A_{t+1}
    };
    e_step(0, no_stores);
    for (int t = 1; t < T; ++t) e_step(t, with_stores);
  } else {
    // ---------------- role L ----------------
    float x[4][2];
    lds_barrier();   // B_0 (r^L_0 was written before A_0)
    contract_half(0, xE, -1, no_stores);
    contract_half(1, xL, -1, no_stores);
    preactivation(0, x);
    lds_barrier();   // A_1
    for (int t = 1; t < T; ++t) {
      activate(x);   // step t-1 -> r^L_t
      if constexpr (STATS) stat_share(t - 1);
      write_half(xL, r, w, q, n);
      lds_barrier();   // B_t
      contract_half(0, xE + (t & 1) * R8_HALF_SLOTS, t - 1, with_stores);
      contract_half(1, xL, t - 1, with_stores);
      preactivation(t, x);
      lds_barrier();   // A_{t+1}
    }
    activate(x);
    if constexpr (STATS) stat_share(T - 1);
  }
  if constexpr (STATS) {
    lds_barrier();                                 // the late role's share of the last row
    stat_flush(T - 1);
  }
  // stores of the last step (its state is not an operand of any further step)
#pragma unroll
  for (int slot = 0; slot < 6; ++slot) emit_store(T - 1, slot);
}

// ------------------------------------------------------------------------------------------------
// BPTT recurrence, transposed weights resident.  Same contract as ring_bptt_kernel<4> with k == 2.
// grad_output and F' are prefetched DEPTH steps ahead into register stages (loop unrolled to match).
// ------------------------------------------------------------------------------------------------
namespace {

// One step's inputs in flight: grad_output rows (4 x 16 B) and the saved F' record (2 x 16 B, fp16).  With the
// loss head fused in (LOSS) the rows are those of the state history instead and C holds the four rows' loss
// coefficients (kc, ks, beta, -), from which the kernel forms grad_output itself.
// With dL/dA requested (GA), R holds the bf16 operand copy of r_prev for the lane's four neurons (4 rows each).
struct BpttStage {
  f32x4 G[4];
  f32x4 D[2];
  f32x4 C[4];
  f32x2 R[4];
};

// In the unmasked variant the loads of a stage are issued with inline assembly and waited for
// with an explicit vmcnt.  The compiler, seeing loads and stores share that counter, would otherwise
// drain it completely (vmcnt(0)) before every use and expose a full HBM round trip per time step.
// Safety of bptt_stage_wait<K>: vector-memory operations leave the counter in issue order, so once at
// most K are outstanding and at least K were issued after this stage's loads, the stage has landed.  The "+v" operands order every use after the wait.
__device__ __forceinline__ f32x4 async_load16(const void* ptr) {
  f32x4 v;
  // (the local labels cost nothing at run time; the build check uses them to find these loads and
  // their waits in the emitted code)
  asm volatile(".Lring_async_load_%=:\n\tglobal_load_dwordx4 %0, %1, off" : "=&v"(v) : "v"(ptr) : "memory");
  return v;
}

// The same load addressed as a wave-uniform base (scalar registers) plus a 32-bit per-lane byte offset plus an
// immediate: the per-step address arithmetic then runs on the scalar unit and costs the vector ALU nothing.
// Non-temporal: grad_output and the saved record are read exactly once, and what should stay in the caches
// is the operand copy this kernel writes for the weight-gradient kernel that follows.
template <int IMM>
__device__ __forceinline__ f32x4 async_load16_s(const void* uniform_base, unsigned lane_off) {
  f32x4 v;
  asm volatile(".Lring_async_load_%=:\n\tglobal_load_dwordx4 %0, %1, %2 offset:%3 nt"
               : "=&v"(v)
               : "v"(lane_off), "s"(uniform_base), "n"(IMM)
               : "memory");
  return v;
}

template <int IMM>
__device__ __forceinline__ f32x2 async_load8_s(const void* uniform_base, unsigned lane_off) {
  f32x2 v;
  asm volatile(".Lring_async_load_%=:\n\tglobal_load_dwordx2 %0, %1, %2 offset:%3 nt"
               : "=&v"(v)
               : "v"(lane_off), "s"(uniform_base), "n"(IMM)
               : "memory");
  return v;
}

template <int K, bool LOSS, bool GA>
__device__ __forceinline__ void bptt_stage_wait(BpttStage& s) {
  if constexpr (LOSS && GA) {
    asm volatile(".Lring_async_wait_%=:\n\ts_waitcnt vmcnt(%14)"
                 : "+v"(s.G[0]), "+v"(s.G[1]), "+v"(s.G[2]), "+v"(s.G[3]), "+v"(s.D[0]), "+v"(s.D[1]), "+v"(s.C[0]),
                   "+v"(s.C[1]), "+v"(s.C[2]), "+v"(s.C[3]), "+v"(s.R[0]), "+v"(s.R[1]), "+v"(s.R[2]), "+v"(s.R[3])
                 : "n"(K)
                 : "memory");
  } else if constexpr (GA) {
    asm volatile(".Lring_async_wait_%=:\n\ts_waitcnt vmcnt(%10)"
                 : "+v"(s.G[0]), "+v"(s.G[1]), "+v"(s.G[2]), "+v"(s.G[3]), "+v"(s.D[0]), "+v"(s.D[1]), "+v"(s.R[0]),
                   "+v"(s.R[1]), "+v"(s.R[2]), "+v"(s.R[3])
                 : "n"(K)
                 : "memory");
  } else if constexpr (LOSS) {
    asm volatile(".Lring_async_wait_%=:\n\ts_waitcnt vmcnt(%10)"
                 : "+v"(s.G[0]), "+v"(s.G[1]), "+v"(s.G[2]), "+v"(s.G[3]), "+v"(s.D[0]), "+v"(s.D[1]), "+v"(s.C[0]),
                   "+v"(s.C[1]), "+v"(s.C[2]), "+v"(s.C[3])
                 : "n"(K)
                 : "memory");
  } else {
    asm volatile(".Lring_async_wait_%=:\n\ts_waitcnt vmcnt(%6)"
                 : "+v"(s.G[0]), "+v"(s.G[1]), "+v"(s.G[2]), "+v"(s.G[3]), "+v"(s.D[0]), "+v"(s.D[1])
                 : "n"(K)
                 : "memory");
  }
}

template <bool FULL, bool LOSS, bool GA>
__device__ __forceinline__ void bptt_stage_load(const RingBpttArgs& p, int t, int bt, int w, int lane, int b0, int i0,
                                                BpttStage& s) {
  if (t < 0) t = 0;   // redundant reload past the start of the sequence; never consumed
  const _Float16* drec = p.dfrag + side_offset<R_NC>(t, p.nbt, bt, w, lane);
  const float* rows = LOSS ? p.hist : p.grad_out;
  if constexpr (FULL) {
    // FULL: N == 256 and whole batch tiles, so row e of the lane's four sits e KiB after row 0
    const int q = lane >> 4, n = lane & 15;
    const int ws = __builtin_amdgcn_readfirstlane(w);
    const float* gtile = rows + ((size_t)t * p.B + 16 * bt) * 256;                      // uniform: the tile's 16 rows
    const unsigned goff = (unsigned)((4 * q * 256 + 16 * R_NC * ws + R_NC * n) * sizeof(float));
    s.G[0] = async_load16_s<0>(gtile, goff);
    s.G[1] = async_load16_s<1024>(gtile, goff);
    s.G[2] = async_load16_s<2048>(gtile, goff);
    s.G[3] = async_load16_s<3072>(gtile, goff);
    const _Float16* dtile = p.dfrag + side_offset<R_NC>(t, p.nbt, bt, ws, 0);           // uniform: the wave's record block
    const unsigned doff = (unsigned)lane * (4 * R_NC * sizeof(_Float16));
    s.D[0] = async_load16_s<0>(dtile, doff);
    s.D[1] = async_load16_s<16>(dtile, doff);
    if constexpr (LOSS) {
      const ring_f32x4* ctile = p.loss_coef + (size_t)t * p.B + 16 * bt;                  // uniform: the tile's 16 records
      const unsigned coff = (unsigned)(4 * q) * sizeof(ring_f32x4);
      s.C[0] = async_load16_s<0>(ctile, coff);
      s.C[1] = async_load16_s<16>(ctile, coff);
      s.C[2] = async_load16_s<32>(ctile, coff);
      s.C[3] = async_load16_s<48>(ctile, coff);
    }
    (void)drec;
    (void)b0;
    (void)i0;
  } else {
    float G[4][R_NC];
    rows_load<R_NC>(rows + (size_t)t * p.B * p.N, p.N, p.B, b0, i0, G);
#pragma unroll
    for (int e = 0; e < 4; ++e) s.G[e] = f32x4{G[e][0], G[e][1], G[e][2], G[e][3]};
    s.D[0] = *reinterpret_cast<const f32x4*>(drec);
    s.D[1] = *reinterpret_cast<const f32x4*>(drec + 8);
    if constexpr (LOSS) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int b = b0 + e < p.B ? b0 + e : p.B - 1;   // rows past the batch meet a zero F' record
        s.C[e] = p.loss_coef[(size_t)t * p.B + b];
      }
    }
  }
}

// The r_prev part of a stage (dL/dA only).  It is consumed during the step's products, after the refill of the
// rest of the stage has been issued, so it is refilled separately at the end of the step: a refill before its
// last use would need a register copy of values that are still in flight.
template <bool FULL>
__device__ __forceinline__ void bptt_stage_load_r(const RingBpttArgs& p, int t, int bt, int w, int lane, BpttStage& s) {
  if (t < 0) t = 0;
  if constexpr (FULL) {
    // the half (t % 2) of the pair slots of the wave's four tiles, 1 KiB apart
    const int ws = __builtin_amdgcn_readfirstlane(w);
    const __bf16* rtile = p.rfrag + pair_offset<R_NC>(t, p.nbt, bt, ws * R_NC, 0);       // uniform
    const unsigned roff = (unsigned)lane * 16u;
    s.R[0] = async_load8_s<0>(rtile, roff);
    s.R[1] = async_load8_s<1024>(rtile, roff);
    s.R[2] = async_load8_s<2048>(rtile, roff);
    s.R[3] = async_load8_s<3072>(rtile, roff);
  } else {
#pragma unroll
    for (int c = 0; c < R_NC; ++c)
      s.R[c] = *reinterpret_cast<const f32x2*>(p.rfrag + pair_offset<R_NC>(t, p.nbt, bt, w * R_NC + c, lane));
  }
}

// F' of neuron c, rows e = 0..3: the record is [c][e] in fp16.
__device__ __forceinline__ float stage_dact(const BpttStage& s, int e, int c) {
  const f16x4 h = __builtin_bit_cast(f16x4, f32x2{s.D[c >> 1][2 * (c & 1)], s.D[c >> 1][2 * (c & 1) + 1]});
  return (float)h[e];
}

}  // namespace

// LOSS: grad_output is not read; it is formed per element from the state history and the loss head's row
// coefficients,  up * (kc cos(phi_i) + ks sin(phi_i) + beta sign(r_i)),  phi_i = 2 pi i / N,
// up = upstream / (T * B)  (what ring_loss_grad_kernel would have written to HBM for this kernel to read back).
// MERGE (needs FULL and an even T): the operand copy of g pairs time steps 2j and 2j+1 in one 16-byte slot per
// lane; the kernel walks down through 2j+1 and 2j in one trip of its unrolled loop, keeps the first in registers
// and writes both with one 16-byte store per tile (whole cache lines, half as many store instructions).
// DEPTH: steps whose inputs are in flight (register stages); even, so that a trip of the unrolled loop holds whole pairs.
// GA: also write grad_A[b,t,c] = sum_j (g Wa[c])[j] * r_prev[j], c = 0, 1: the per-matrix products of the step are
// dotted with the bf16 operand copy of r_prev (the forward's, read with the step's other inputs), summed over the
// row group's 16 lanes with data-parallel adds, over the four waves through LDS in wave order, and written out
// after the next step's barrier.
template <bool FULL, bool LOSS, bool MERGE, int DEPTH, bool GA>
__global__ __launch_bounds__(256) void ring_bptt_res256_kernel(RingBpttArgs p) {
  static_assert(DEPTH % 2 == 0 && DEPTH <= R_BPTT_DEPTH_MAX, "the unrolled loop walks whole step pairs");
  static_assert(!MERGE || FULL, "merged pair stores need the unmasked loop");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xbuf = wlds + R_WLDS_SLOTS;
  f32x2* gbuf = reinterpret_cast<f32x2*>(xbuf + 2 * R_XSLOTS);
  float* gabuf = reinterpret_cast<float*>(gbuf + 2 * R_GCH * 16);   // [step parity][channel][wave][row]

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt = blockIdx.x;
  const int b0 = 16 * bt + 4 * q;
  const int i0 = 16 * R_NC * w + R_NC * n;
  const int N = p.N, B = p.B, T = p.T;
  // dL/dA of step t from the shares the four waves left in buffer `par` (call after a barrier that follows them)
  auto flush_grad_A = [&](int t, int par) {
    if (tid < 32) {
      const int ch = tid >> 4, row = tid & 15, b = 16 * bt + row;
      const float* sh = gabuf + (par * 2 + ch) * 64 + row;
      if (b < B) p.grad_A[((size_t)b * T + t) * 2 + ch] = ((sh[0] + sh[16]) + sh[32]) + sh[48];
    }
  };
  const float oma = 1.f - p.alpha;   // alpha rides in the saved F' record, J0 and J1 in the packed Wo fragments
  const int wu = __builtin_amdgcn_readfirstlane(w);   // the wave index as a scalar, for address arithmetic

  bf16x8 wreg[2][R_NC][R_KCH];
  bf16x8* wl = wlds + (size_t)w * R_NC * R_KCH * 64 + lane;
  load_resident(reinterpret_cast<const bf16x8*>(p.Wpack), wl, wreg, w, lane);

  float carry[4][R_NC];
  float okf[4][R_NC];
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int c = 0; c < R_NC; ++c) {
      carry[e][c] = 0.f;
      okf[e][c] = ((b0 + e < B) && (i0 + c < N)) ? 1.f : 0.f;
    }

  float cs[R_NC], sn[R_NC], up = 0.f;
  if constexpr (LOSS) {
#pragma unroll
    for (int c = 0; c < R_NC; ++c) {
      const float phi = 6.2831853071795864769f * (float)(i0 + c) / (float)N;
      cs[c] = cosf(phi);
      sn[c] = sinf(phi);
    }
    up = (p.loss_upstream ? p.loss_upstream[0] : 1.f) * p.loss_inv_rows;
  }

  pair_zero_tail<R_NC>(p.gfrag, T, p.nbt, bt, w, lane);
  BpttStage st[DEPTH];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    bptt_stage_load<FULL, LOSS, GA>(p, T - 1 - d, bt, w, lane, b0, i0, st[d]);
    if constexpr (GA) bptt_stage_load_r<FULL>(p, T - 1 - d, bt, w, lane, st[d]);
  }
  GateStage gs;
  gates_fetch(p.A, T, B, bt, 0, -1, tid, gs);
  gates_publish(gbuf, tid, B, bt, gs);
  // The LDS-resident slice is consumed one fragment at a time.  PAIR (the variants with registers to spare): two
  // tiles are contracted together, fragment g of a step = tile pair g/16, K chunk (g/2)%8, tile g%2 of the pair,
  // through a ring of eight registers filled seven fragments ahead across tiles and steps; otherwise tile by tile
  // in half-tile units of four fragments, one unit ahead.
  constexpr bool PAIR = FULL && !(LOSS && GA);
  auto frag_slot = [&](int g) { return ((2 * (g >> 4) + (g & 1)) * R_KCH + ((g >> 1) & 7)) * 64; };
  bf16x8 w0[8];
  if constexpr (PAIR) {
#pragma unroll
    for (int g = 0; g < 7; ++g) w0[g] = wl[frag_slot(g)];
  } else {
#pragma unroll
    for (int u = 0; u < R_KCH / 2; ++u) w0[u] = wl[u * 64];
  }
  // (the first lds_barrier inside the loop also publishes the gates)

  bf16x4 held[R_NC];   // MERGE: the odd step's bf16 g, waiting for its even partner
  for (int u0 = 0; u0 < T; u0 += DEPTH) {
#pragma unroll
    for (int half = 0; half < DEPTH; ++half) {
      const int u = u0 + half;
      if (u >= T) break;
      const int t = T - 1 - u;
      const int cur = u & 1, ci = u / R_GCH, l = u % R_GCH;
      if (l == 0 && (ci + 1) * R_GCH < T) gates_fetch(p.A, T, B, bt, ci + 1, -1, tid, gs);
      BpttStage& S = st[half];
      // Issued after this stage's loads (six; ten with the loss head fused in), in order: per later step its
      // operand-copy stores and then another stage's loads.  The counter is in order, so once no more than that
      // many operations are outstanding this stage has landed; a smaller number would also wait for later loads
      // and for store acknowledgements.  Unmerged, every step issues four stores.  With merged pair stores the
      // four stores sit in the second step of each pair (odd `half`): the steps since this stage was loaded are
      // half - DEPTH + 1 .. half - 1, of which DEPTH / 2 are odd when `half` is even and DEPTH / 2 - 1 otherwise.
      // (with dL/dA: four more loads per stage, and the one store of the previous step's dL/dA, issued by some waves
      // only, which makes the bound conservative for the others: it can only wait for more)
      constexpr int LOADS = 6 + (LOSS ? 4 : 0) + (GA ? 4 : 0);
      if constexpr (MERGE) {
        if ((half & 1) == 0) bptt_stage_wait<LOADS * (DEPTH - 1) + 4 * (DEPTH / 2), LOSS, GA>(S);
        else bptt_stage_wait<LOADS * (DEPTH - 1) + 4 * (DEPTH / 2 - 1), LOSS, GA>(S);
      } else if constexpr (FULL) {
        bptt_stage_wait<(LOADS + 4) * (DEPTH - 1), LOSS, GA>(S);
      }
      // (the stage's r_prev part is issued last in a step, behind everything counted above, and used in place)

      float G[4][R_NC], g[4][R_NC];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float kc = 0.f, ks = 0.f, beta = 0.f;
        if constexpr (LOSS) {
          kc = S.C[e][0] * up;
          ks = S.C[e][1] * up;
          beta = S.C[e][2] * up;
        }
#pragma unroll
        for (int c = 0; c < R_NC; ++c) {
          float go = S.G[e][c];
          if constexpr (LOSS) {
            const float r = go;                                      // the stage holds the state, not a gradient
            const float sb = r > 0.f ? beta : (r < 0.f ? -beta : 0.f);          // beta * sign(r), sign(0) = 0
            go = fmaf(kc, cs[c], fmaf(ks, sn[c], sb));
          }
          G[e][c] = go + carry[e][c];
          g[e][c] = __builtin_fmaf(stage_dact(S, e, c), G[e][c], 0.f);   // one mixed-precision FMA: the fp16 record is an operand as it is
        }
      }
      bf16x8* xb = xbuf + cur * R_XSLOTS;
      write_operand<R_NC>(xb, g, w, q, n);
      {
        // pair_store with the address split into a wave-uniform base and the lane's slot: tile w*NC + c is c KiB on
        char* gt = reinterpret_cast<char*>(p.gfrag + pair_offset<R_NC>(t, p.nbt, bt, wu * R_NC, 0));
        const unsigned goff = (unsigned)lane * 16u;
#pragma unroll
        for (int c = 0; c < R_NC; ++c) {
          const bf16x4 pk = {(__bf16)g[0][c], (__bf16)g[1][c], (__bf16)g[2][c], (__bf16)g[3][c]};
          if constexpr (MERGE) {
            if ((half & 1) == 0) {
              held[c] = pk;            // t is odd here (T even): the slot's second half, written with the first
            } else {
              const bf16x8 both = __builtin_shufflevector(pk, held[c], 0, 1, 2, 3, 4, 5, 6, 7);
              *reinterpret_cast<bf16x8*>(gt + c * 1024 + goff) = both;
            }
          } else {
            *reinterpret_cast<bf16x4*>(gt + c * 1024 + goff) = pk;
          }
        }
      }
      bptt_stage_load<FULL, LOSS, GA>(p, t - DEPTH, bt, w, lane, b0, i0, S);
      lds_barrier();
      if constexpr (GA) {
        if (u > 0) flush_grad_A(t + 1, cur ^ 1);   // the previous step's shares are complete behind this barrier
      }
      float ga[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};

      bf16x8 af[R_KCH];
#pragma unroll
      for (int kc = 0; kc < R_KCH; ++kc) af[kc] = xb[(kc * 4 + q) * XG + n];
      f32x2 gate[4];
      {
        const f32x2* gb = gbuf + ((ci & 1) * R_GCH + l) * 16 + 4 * q;
#pragma unroll
        for (int e = 0; e < 4; ++e) gate[e] = gb[e];
      }
      // the ungated chain starts from the term that needs no product, (1 - alpha) * G; J0 * sum(g) comes with
      // the product itself (the packed fragments hold J1 * Wo^T + J0)
      auto tile_epilogue = [&](int c, const f32x4& P0, const f32x4& P1, const f32x4& P2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float x = fmaf(gate[e][0], P1[e], P0[e]);
          x = fmaf(gate[e][1], P2[e], x);
          if constexpr (!FULL) x *= okf[e][c];
          carry[e][c] = x;
        }
        if constexpr (GA) {
          const bf16x4 rp = __builtin_bit_cast(bf16x4, S.R[c]);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float rv = (float)rp[e];
            ga[0][e] = fmaf(P1[e], rv, ga[0][e]);
            ga[1][e] = fmaf(P2[e], rv, ga[1][e]);
          }
        }
      };
      if constexpr (PAIR) {
#pragma unroll
        for (int cp = 0; cp < R_NC / 2; ++cp) {
          f32x4 P[2][3];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int c = 2 * cp + j;
            P[j][0] = f32x4{oma * G[0][c], oma * G[1][c], oma * G[2][c], oma * G[3][c]};
            P[j][1] = f32x4{0.f, 0.f, 0.f, 0.f};
            P[j][2] = P[j][1];
          }
#pragma unroll
          for (int kc = 0; kc < R_KCH; ++kc)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const int c = 2 * cp + j, g = (cp * R_KCH + kc) * 2 + j;
              w0[(g + 7) & 7] = wl[frag_slot((g + 7) & 31)];
              __builtin_amdgcn_sched_barrier(0);   // the read stays seven fragments ahead of its use
              P[j][1] = mfma16(af[kc], wreg[0][c][kc], P[j][1]);
              P[j][2] = mfma16(af[kc], wreg[1][c][kc], P[j][2]);
              P[j][0] = mfma16(af[kc], w0[g & 7], P[j][0]);
            }
#pragma unroll
          for (int j = 0; j < 2; ++j) tile_epilogue(2 * cp + j, P[j][0], P[j][1], P[j][2]);
        }
      } else {
#pragma unroll
        for (int c = 0; c < R_NC; ++c) {
          f32x4 P0 = {oma * G[0][c], oma * G[1][c], oma * G[2][c], oma * G[3][c]};
          f32x4 P1 = {0.f, 0.f, 0.f, 0.f}, P2 = P1;
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            // stage the next half tile of the LDS-resident matrix (wraps to tile 0 of the next step)
            constexpr int HK = R_KCH / 2;
            const int f = 2 * c + h, fn = (f + 1) & 7;
#pragma unroll
            for (int u = 0; u < HK; ++u) w0[((f + 1) & 1) * HK + u] = wl[(fn * HK + u) * 64];
#pragma unroll
            for (int u = 0; u < HK; ++u) {
              const int kc = h * HK + u;
              P0 = mfma16(af[kc], w0[(f & 1) * HK + u], P0);
              P1 = mfma16(af[kc], wreg[0][c][kc], P1);
              P2 = mfma16(af[kc], wreg[1][c][kc], P2);
            }
          }
          tile_epilogue(c, P0, P1, P2);
        }
      }
      if constexpr (GA) {
        // the other parity's buffer is being read by this step's flush; this one was read one step ago, before
        // the barrier above
#pragma unroll
        for (int ch = 0; ch < 2; ++ch)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float tot = row16_sum_dpp(ga[ch][e]);
            if (n == 0) gabuf[((cur * 2 + ch) * 4 + w) * 16 + 4 * q + e] = tot;
          }
        bptt_stage_load_r<FULL>(p, t - DEPTH, bt, w, lane, S);
      }
      // the next iteration overwrites the other operand buffer and, every R_GCH steps, the other
      // gate chunk; both were last read before the barrier above, so no second barrier is needed
      if (l == R_GCH - 1 && u + 1 < T) gates_publish(gbuf + ((ci + 1) & 1) * R_GCH * 16, tid, B, bt, gs);
    }
  }
  // the last iterations prefetched (clamped) steps that are never consumed: let those loads land
  // while their destination registers are still reserved, before anything below reuses them
  if constexpr (FULL) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) bptt_stage_wait<0, LOSS, GA>(st[d]);
  }
  if constexpr (GA) {
    lds_barrier();
    flush_grad_A(0, (T - 1) & 1);
  }
  if (p.grad_r_init) rows_store<R_NC>(p.grad_r_init, N, B, b0, i0, carry);
}

// ------------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------------
bool ring_res256_applicable(int N, int k) { return k == 2 && N > 128 && N <= 256; }

template <int ACT, bool SAVE, bool FULL, bool STATS>
static hipError_t launch_fwd_variant(const RingFwdArgs& a, hipStream_t st) {
  auto kern = ring_fwd_res256_kernel<ACT, SAVE, FULL, STATS>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)R8_LDS_BYTES);
  if (e != hipSuccess) return e;
  RING_LAUNCH(kern, dim3(a.nbt), dim3(512), R8_LDS_BYTES, st, a);
  return hipGetLastError();
}

template <int ACT>
static hipError_t launch_fwd_act(const RingFwdArgs& a, hipStream_t st) {
  const bool full = (a.N == 256) && (a.B % 16 == 0);
  if (a.loss_stats) {
    if (a.dfrag) return full ? launch_fwd_variant<ACT, true, true, true>(a, st) : launch_fwd_variant<ACT, true, false, true>(a, st);
    return full ? launch_fwd_variant<ACT, false, true, true>(a, st) : launch_fwd_variant<ACT, false, false, true>(a, st);
  }
  if (a.dfrag) return full ? launch_fwd_variant<ACT, true, true, false>(a, st) : launch_fwd_variant<ACT, true, false, false>(a, st);
  return full ? launch_fwd_variant<ACT, false, true, false>(a, st) : launch_fwd_variant<ACT, false, false, false>(a, st);
}

hipError_t ring_launch_fwd_res256(const RingFwdArgs& a, hipStream_t st) {
  switch (a.act) {
    case ACT_RELU: return launch_fwd_act<ACT_RELU>(a, st);
    case ACT_GELU: return launch_fwd_act<ACT_GELU>(a, st);
    case ACT_TANH: return launch_fwd_act<ACT_TANH>(a, st);
    case ACT_SILU: return launch_fwd_act<ACT_SILU>(a, st);
    default: return hipErrorInvalidValue;
  }
}

template <bool FULL, bool LOSS, bool MERGE, int DEPTH, bool GA>
static hipError_t launch_bptt_variant(const RingBpttArgs& a, hipStream_t st) {
  auto kern = ring_bptt_res256_kernel<FULL, LOSS, MERGE, DEPTH, GA>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)R_LDS_BYTES);
  if (e != hipSuccess) return e;
  RING_LAUNCH(kern, dim3(a.nbt), dim3(256), R_LDS_BYTES, st, a);
  return hipGetLastError();
}

// Two steps of inputs in flight.  (Four, which the unmasked kernel that reads grad_output has the registers for,
// measured the same: the kernel does not wait for its loads.)
template <bool GA>
static hipError_t launch_bptt_ga(const RingBpttArgs& a, hipStream_t st) {
  const bool full = (a.N == 256) && (a.B % 16 == 0);
  const bool merge = full && (a.T % 2 == 0);
  if (a.loss_coef) {
    if (merge) return launch_bptt_variant<true, true, true, 2, GA>(a, st);
    return full ? launch_bptt_variant<true, true, false, 2, GA>(a, st) : launch_bptt_variant<false, true, false, 2, GA>(a, st);
  }
  if (merge) return launch_bptt_variant<true, false, true, 2, GA>(a, st);
  return full ? launch_bptt_variant<true, false, false, 2, GA>(a, st) : launch_bptt_variant<false, false, false, 2, GA>(a, st);
}

hipError_t ring_launch_bptt_res256(const RingBpttArgs& a, hipStream_t st) {
  if (a.grad_A) {
    if (!a.rfrag) return hipErrorInvalidValue;
    return launch_bptt_ga<true>(a, st);
  }
  return launch_bptt_ga<false>(a, st);
}
