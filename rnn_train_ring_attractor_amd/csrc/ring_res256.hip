// Weight-resident kernels for the headline geometry: 192 < N <= 256 (NPAD = 256, NC = 4), a_dim = 2.
//
// [Wo|Wl|Wr] in bf16 is 384 KiB -- more than one CU's LDS (160 KiB) but less than its register
// file (512 KiB).  Each of the 4 waves keeps its 64-neuron slice of two matrices (64 fragments,
// 256 VGPRs) in registers for the whole sequence and the slice of the third in LDS (128 KiB per
// workgroup, read back by the lane that wrote it), so no weight byte is fetched from L2/HBM inside
// the time loop.  One workgroup per CU, one wave per SIMD, 16 batch rows per workgroup.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

namespace {

constexpr int R_NC = 4;
constexpr int R_KCH = 8;
constexpr int R_WLDS_SLOTS = 4 * R_NC * R_KCH * 64;   // 16-byte slots of the LDS-resident matrix
constexpr int R_XSLOTS = R_KCH * 4 * XG;
constexpr int R_GCH = 32;                             // time steps of action gates staged per LDS chunk
constexpr size_t R_LDS_BYTES = (size_t)(R_WLDS_SLOTS + 2 * R_XSLOTS) * 16 + 2 * 64 * 4 + 2 * R_GCH * 16 * 8;

// Cheap activation pairs (F, F') for the per-step critical path.
//  gelu: Phi via the Abramowitz-Stegun 7.1.26 erfc polynomial (|err| < 1.5e-7), sharing exp(-x^2/2)
//  with the density term of F'.   tanh/silu: one v_exp + one v_rcp.
template <int ACT>
__device__ __forceinline__ void act_fast(float x, float& F, float& D) {
  if constexpr (ACT == ACT_RELU) {
    F = fmaxf(x, 0.f);
    D = x > 0.f ? 1.f : 0.f;
  } else if constexpr (ACT == ACT_GELU) {
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(fmaf(ax, 0.3275911f * 0.70710678f, 1.f));
    const float e = __builtin_amdgcn_exp2f(x * x * -0.72134752f);   // exp(-x^2/2)
    float poly = fmaf(t, 0.5f * 1.061405429f, 0.5f * -1.453152027f);
    poly = fmaf(t, poly, 0.5f * 1.421413741f);
    poly = fmaf(t, poly, 0.5f * -0.284496736f);
    poly = fmaf(t, poly, 0.5f * 0.254829592f);
    const float h = poly * t * e;                 // 0.5*erfc(|x|/sqrt2) = Phi(-|x|)
    const float cdf = x >= 0.f ? 1.f - h : h;
    F = x * cdf;
    D = fmaf(x * e, 0.39894228f, cdf);
  } else if constexpr (ACT == ACT_TANH) {
    const float xc = fminf(fmaxf(x, -15.f), 15.f);
    const float e2 = __builtin_amdgcn_exp2f(xc * 2.88539008f);      // exp(2x)
    const float th = 1.f - 2.f * __builtin_amdgcn_rcpf(e2 + 1.f);
    F = th;
    D = 1.f - th * th;
  } else {
    const float xc = fmaxf(x, -87.f);
    const float s = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(xc * -1.44269504f));
    F = x * s;
    D = s * fmaf(x, 1.f - s, 1.f);
  }
}

__device__ __forceinline__ float dpp_row_sum(float v) {
  // butterfly over the 16 lanes of a DPP row: quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror, row_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));
  return v;
}

__device__ __forceinline__ void publish_rowsum4(float* psum, const float (&v)[4][R_NC], int w, int q, int n) {
  f32x4 s;
#pragma unroll
  for (int e = 0; e < 4; ++e) s[e] = dpp_row_sum((v[e][0] + v[e][1]) + (v[e][2] + v[e][3]));
  if (n == 0) *reinterpret_cast<f32x4*>(psum + w * 16 + 4 * q) = s;
}

__device__ __forceinline__ f32x4 read_rowsum4(const float* psum, int q) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(psum + 0 * 16 + 4 * q);
  const f32x4 b = *reinterpret_cast<const f32x4*>(psum + 1 * 16 + 4 * q);
  const f32x4 c = *reinterpret_cast<const f32x4*>(psum + 2 * 16 + 4 * q);
  const f32x4 d = *reinterpret_cast<const f32x4*>(psum + 3 * 16 + 4 * q);
  return ((a + b) + c) + d;
}

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
  const float m = b < B ? 1.f : 0.f;
  g.a = va * m;
  g.b = vb * m;
}

__device__ __forceinline__ void gates_publish(f32x2* gb, int tid, const GateStage& g) {
  const int row = tid >> 4, j = tid & 15;
  gb[j * 16 + row] = g.a;
  gb[(j + 16) * 16 + row] = g.b;
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
// ------------------------------------------------------------------------------------------------
template <int ACT, bool SAVE, bool FULL>
__global__ __launch_bounds__(256) void ring_fwd_res256_kernel(RingFwdArgs p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xbuf = wlds + R_WLDS_SLOTS;
  float* psum = reinterpret_cast<float*>(xbuf + 2 * R_XSLOTS);
  f32x2* gbuf = reinterpret_cast<f32x2*>(psum + 2 * 64);

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt = blockIdx.x;
  const int b0 = 16 * bt + 4 * q;
  const int i0 = 16 * R_NC * w + R_NC * n;
  const int N = p.N, B = p.B, T = p.T;
  const float oma = 1.f - p.alpha, alpha = p.alpha, J0 = p.J0, J1 = p.J1;

  bf16x8 wreg[2][R_NC][R_KCH];
  bf16x8* wl = wlds + (size_t)w * R_NC * R_KCH * 64 + lane;
  load_resident(reinterpret_cast<const bf16x8*>(p.Wpack), wl, wreg, w, lane);

  float r[4][R_NC];
  float okf[4][R_NC];
  rows_load<R_NC>(p.r_init, N, B, b0, i0, r);
  if constexpr (!FULL) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < R_NC; ++c) okf[e][c] = ((b0 + e < B) && (i0 + c < N)) ? 1.f : 0.f;
  }
  write_operand<R_NC>(xbuf, r, w, q, n);
  publish_rowsum4(psum, r, w, q, n);
  if (SAVE) {
    pair_store<R_NC>(p.rfrag, 0, p.nbt, bt, w, lane, r);
    pair_zero_tail<R_NC>(p.rfrag, T, p.nbt, bt, w, lane);
  }
  GateStage gs;
  gates_fetch(p.A, T, B, bt, 0, +1, tid, gs);
  gates_publish(gbuf, tid, gs);

  bf16x8 w0[2][R_KCH / 2];
#pragma unroll
  for (int u = 0; u < R_KCH / 2; ++u) w0[0][u] = wl[u * 64];
  lds_barrier();

  for (int t = 0; t < T; ++t) {
    const int cur = t & 1, ci = t / R_GCH, l = t % R_GCH;
    if (l == 0 && (ci + 1) * R_GCH < T) gates_fetch(p.A, T, B, bt, ci + 1, +1, tid, gs);

    const bf16x8* xb = xbuf + cur * R_XSLOTS;
    bf16x8 af[R_KCH];
#pragma unroll
    for (int kc = 0; kc < R_KCH; ++kc) af[kc] = xb[(kc * 4 + q) * XG + n];
    const f32x4 s = read_rowsum4(psum + cur * 64, q);
    f32x2 gate[4];
    {
      const f32x2* gb = gbuf + ((ci & 1) * R_GCH + l) * 16 + 4 * q;
#pragma unroll
      for (int e = 0; e < 4; ++e) gate[e] = gb[e];
    }

    float d[4][R_NC];
    // Software pipeline over the four column tiles: the 24 MFMAs of tile c+1 are issued while the
    // vector ALU runs the epilogue (gating, activation, leak) of tile c, so the matrix pipe works in
    // the shadow of the epilogue instead of before it.
    f32x4 P[2][3];
    const f32x4 js = s * J0;
    auto mfma_tile = [&](int c, f32x4 (&Pc)[3]) {
      Pc[0] = Pc[1] = Pc[2] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // stage the next half tile of the LDS-resident matrix (wraps to tile 0 of the next step)
        constexpr int HK = R_KCH / 2;
        const int f = 2 * c + h, fn = (f + 1) & 7;
#pragma unroll
        for (int u = 0; u < HK; ++u) w0[(f + 1) & 1][u] = wl[(fn * HK + u) * 64];
#pragma unroll
        for (int u = 0; u < HK; ++u) {
          const int kc = h * HK + u;
          Pc[0] = mfma16(af[kc], w0[f & 1][u], Pc[0]);
          Pc[1] = mfma16(af[kc], wreg[0][c][kc], Pc[1]);
          Pc[2] = mfma16(af[kc], wreg[1][c][kc], Pc[2]);
        }
      }
    };
    auto epilogue_tile = [&](int c, const f32x4 (&Pc)[3]) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float x = fmaf(J1, Pc[0][e], js[e]);
        x = fmaf(gate[e][0], Pc[1][e], x);
        x = fmaf(gate[e][1], Pc[2][e], x);
        float F, D;
        act_fast<ACT>(x, F, D);
        float rn = fmaf(alpha, F, oma * r[e][c]);
        if constexpr (!FULL) {
          rn *= okf[e][c];
          D *= okf[e][c];
        }
        r[e][c] = rn;
        d[e][c] = D;
      }
    };
    mfma_tile(0, P[0]);
#pragma unroll
    for (int c = 0; c < R_NC; ++c) {
      if (c + 1 < R_NC) mfma_tile(c + 1, P[(c + 1) & 1]);
      epilogue_tile(c, P[c & 1]);
    }
    if constexpr (FULL) {
      float* hrow = p.hist + ((size_t)t * B + b0) * N + i0;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        *reinterpret_cast<f32x4*>(hrow + (size_t)e * N) = f32x4{r[e][0], r[e][1], r[e][2], r[e][3]};
    } else {
      rows_store<R_NC>(p.hist + (size_t)t * B * N, N, B, b0, i0, r);
    }
    if (SAVE) side_store<R_NC, f16x4, _Float16>(p.dfrag + side_offset<R_NC>(t, p.nbt, bt, w, lane), d);
    if (t + 1 < T) {
      write_operand<R_NC>(xbuf + (cur ^ 1) * R_XSLOTS, r, w, q, n);
      publish_rowsum4(psum + (cur ^ 1) * 64, r, w, q, n);
      if (SAVE) pair_store<R_NC>(p.rfrag, t + 1, p.nbt, bt, w, lane, r);
    }
    if (l == R_GCH - 1 && t + 1 < T) gates_publish(gbuf + ((ci + 1) & 1) * R_GCH * 16, tid, gs);
    lds_barrier();
  }
}

// ------------------------------------------------------------------------------------------------
// BPTT recurrence, transposed weights resident.  Same contract as ring_bptt_kernel<4> with k == 2.
// grad_output and F' are prefetched two steps ahead into two register stages (loop unrolled by 2).
// ------------------------------------------------------------------------------------------------
namespace {

// One step's inputs in flight: grad_output rows (4 x 16 B) and the saved F' record (2 x 16 B, fp16).
struct BpttStage {
  f32x4 G[4];
  f32x4 D[2];
};

// In the unmasked variant the six loads of a stage are issued with inline assembly and waited for
// with an explicit vmcnt.  The compiler, seeing loads and stores share that counter, would otherwise
// drain it completely (vmcnt(0)) before every use and expose a full HBM round trip per time step.
// Safety of bptt_stage_wait<K>: loads return in issue order, so once at most K vector-memory
// operations are outstanding and K later loads were issued after this stage, the stage has landed;
// later stores can only make the wait longer.  The "+v" operands order every use after the wait.
__device__ __forceinline__ f32x4 async_load16(const void* ptr) {
  f32x4 v;
  // (the local labels cost nothing at run time; the build check uses them to find these loads and
  // their waits in the emitted code)
  asm volatile(".Lring_async_load_%=:\n\tglobal_load_dwordx4 %0, %1, off" : "=&v"(v) : "v"(ptr) : "memory");
  return v;
}

template <int K>
__device__ __forceinline__ void bptt_stage_wait(BpttStage& s) {
  asm volatile(".Lring_async_wait_%=:\n\ts_waitcnt vmcnt(%6)"
               : "+v"(s.G[0]), "+v"(s.G[1]), "+v"(s.G[2]), "+v"(s.G[3]), "+v"(s.D[0]), "+v"(s.D[1])
               : "n"(K)
               : "memory");
}

template <bool FULL>
__device__ __forceinline__ void bptt_stage_load(const RingBpttArgs& p, int t, int bt, int w, int lane, int b0, int i0,
                                                BpttStage& s) {
  if (t < 0) t = 0;   // redundant reload past the start of the sequence; never consumed
  const _Float16* drec = p.dfrag + side_offset<R_NC>(t, p.nbt, bt, w, lane);
  if constexpr (FULL) {
    const float* grow = p.grad_out + ((size_t)t * p.B + b0) * p.N + i0;
#pragma unroll
    for (int e = 0; e < 4; ++e) s.G[e] = async_load16(grow + (size_t)e * p.N);
    s.D[0] = async_load16(drec);
    s.D[1] = async_load16(drec + 8);
  } else {
    float G[4][R_NC];
    rows_load<R_NC>(p.grad_out + (size_t)t * p.B * p.N, p.N, p.B, b0, i0, G);
#pragma unroll
    for (int e = 0; e < 4; ++e) s.G[e] = f32x4{G[e][0], G[e][1], G[e][2], G[e][3]};
    s.D[0] = *reinterpret_cast<const f32x4*>(drec);
    s.D[1] = *reinterpret_cast<const f32x4*>(drec + 8);
  }
}

// F' of neuron c, rows e = 0..3: the record is [c][e] in fp16.
__device__ __forceinline__ float stage_dact(const BpttStage& s, int e, int c) {
  const f16x4 h = __builtin_bit_cast(f16x4, f32x2{s.D[c >> 1][2 * (c & 1)], s.D[c >> 1][2 * (c & 1) + 1]});
  return (float)h[e];
}

}  // namespace

template <bool FULL>
__global__ __launch_bounds__(256) void ring_bptt_res256_kernel(RingBpttArgs p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xbuf = wlds + R_WLDS_SLOTS;
  float* psum = reinterpret_cast<float*>(xbuf + 2 * R_XSLOTS);
  f32x2* gbuf = reinterpret_cast<f32x2*>(psum + 2 * 64);

  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt = blockIdx.x;
  const int b0 = 16 * bt + 4 * q;
  const int i0 = 16 * R_NC * w + R_NC * n;
  const int N = p.N, B = p.B, T = p.T;
  const float oma = 1.f - p.alpha, alpha = p.alpha, J0 = p.J0, J1 = p.J1;

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

  pair_zero_tail<R_NC>(p.gfrag, T, p.nbt, bt, w, lane);
  BpttStage st[2];
  bptt_stage_load<FULL>(p, T - 1, bt, w, lane, b0, i0, st[0]);
  bptt_stage_load<FULL>(p, T - 2, bt, w, lane, b0, i0, st[1]);
  GateStage gs;
  gates_fetch(p.A, T, B, bt, 0, -1, tid, gs);
  gates_publish(gbuf, tid, gs);
  bf16x8 w0[2][R_KCH / 2];
#pragma unroll
  for (int u = 0; u < R_KCH / 2; ++u) w0[0][u] = wl[u * 64];
  // (the first lds_barrier inside the loop also publishes the gates)

  for (int u0 = 0; u0 < T; u0 += 2) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int u = u0 + half;
      if (u >= T) break;
      const int t = T - 1 - u;
      const int cur = u & 1, ci = u / R_GCH, l = u % R_GCH;
      if (l == 0 && (ci + 1) * R_GCH < T) gates_fetch(p.A, T, B, bt, ci + 1, -1, tid, gs);
      BpttStage& S = st[half];
      // the other stage's six loads are the only loads issued after this stage's
      if constexpr (FULL) bptt_stage_wait<6>(S);

      float G[4][R_NC], g[4][R_NC];
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int c = 0; c < R_NC; ++c) {
          G[e][c] = S.G[e][c] + carry[e][c];
          g[e][c] = alpha * stage_dact(S, e, c) * G[e][c];
        }
      bf16x8* xb = xbuf + cur * R_XSLOTS;
      write_operand<R_NC>(xb, g, w, q, n);
      publish_rowsum4(psum + cur * 64, g, w, q, n);
      pair_store<R_NC>(p.gfrag, t, p.nbt, bt, w, lane, g);
      bptt_stage_load<FULL>(p, t - 2, bt, w, lane, b0, i0, S);
      lds_barrier();

      bf16x8 af[R_KCH];
#pragma unroll
      for (int kc = 0; kc < R_KCH; ++kc) af[kc] = xb[(kc * 4 + q) * XG + n];
      const f32x4 s = read_rowsum4(psum + cur * 64, q);
      f32x2 gate[4];
      {
        const f32x2* gb = gbuf + ((ci & 1) * R_GCH + l) * 16 + 4 * q;
#pragma unroll
        for (int e = 0; e < 4; ++e) gate[e] = gb[e];
      }
#pragma unroll
      for (int c = 0; c < R_NC; ++c) {
        f32x4 P0 = {0.f, 0.f, 0.f, 0.f}, P1 = P0, P2 = P0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          // stage the next half tile of the LDS-resident matrix (wraps to tile 0 of the next step)
          constexpr int HK = R_KCH / 2;
          const int f = 2 * c + h, fn = (f + 1) & 7;
#pragma unroll
          for (int u = 0; u < HK; ++u) w0[(f + 1) & 1][u] = wl[(fn * HK + u) * 64];
#pragma unroll
          for (int u = 0; u < HK; ++u) {
            const int kc = h * HK + u;
            P0 = mfma16(af[kc], w0[f & 1][u], P0);
            P1 = mfma16(af[kc], wreg[0][c][kc], P1);
            P2 = mfma16(af[kc], wreg[1][c][kc], P2);
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float x = fmaf(oma, G[e][c], J0 * s[e]);
          x = fmaf(J1, P0[e], x);
          x = fmaf(gate[e][0], P1[e], x);
          x = fmaf(gate[e][1], P2[e], x);
          if constexpr (!FULL) x *= okf[e][c];
          carry[e][c] = x;
        }
      }
      // the next iteration overwrites the other operand buffer and, every R_GCH steps, the other
      // gate chunk; both were last read before the barrier above, so no second barrier is needed
      if (l == R_GCH - 1 && u + 1 < T) gates_publish(gbuf + ((ci + 1) & 1) * R_GCH * 16, tid, gs);
    }
  }
  // the last two iterations prefetched (clamped) steps that are never consumed: let those loads land
  // while their destination registers are still reserved, before anything below reuses them
  if constexpr (FULL) {
    bptt_stage_wait<0>(st[0]);
    bptt_stage_wait<0>(st[1]);
  }
  if (p.grad_r_init) rows_store<R_NC>(p.grad_r_init, N, B, b0, i0, carry);
}

// ------------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------------
bool ring_res256_applicable(int N, int k) { return k == 2 && N > 128 && N <= 256; }

template <int ACT, bool SAVE, bool FULL>
static hipError_t launch_fwd_variant(const RingFwdArgs& a, hipStream_t st) {
  auto kern = ring_fwd_res256_kernel<ACT, SAVE, FULL>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)R_LDS_BYTES);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(a.nbt), dim3(256), R_LDS_BYTES, st, a);
  return hipGetLastError();
}

template <int ACT>
static hipError_t launch_fwd_act(const RingFwdArgs& a, hipStream_t st) {
  const bool full = (a.N == 256) && (a.B % 16 == 0);
  if (a.dfrag) return full ? launch_fwd_variant<ACT, true, true>(a, st) : launch_fwd_variant<ACT, true, false>(a, st);
  return full ? launch_fwd_variant<ACT, false, true>(a, st) : launch_fwd_variant<ACT, false, false>(a, st);
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

template <bool FULL>
static hipError_t launch_bptt_variant(const RingBpttArgs& a, hipStream_t st) {
  auto kern = ring_bptt_res256_kernel<FULL>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)R_LDS_BYTES);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(a.nbt), dim3(256), R_LDS_BYTES, st, a);
  return hipGetLastError();
}

hipError_t ring_launch_bptt_res256(const RingBpttArgs& a, hipStream_t st) {
  const bool full = (a.N == 256) && (a.B % 16 == 0);
  return full ? launch_bptt_variant<true>(a, st) : launch_bptt_variant<false>(a, st);
}
