// Step-per-launch kernels for wide rings on few batch tiles ("block" kernels).
//
// A workgroup owns RT batch tiles (16 * RT rows) and 64 * TPW output neurons for one time step: it stages the rows'
// operand (r_prev or g, all NPAD neurons, bf16) in LDS, streams its column slice of each matrix straight from L2
// into registers, K-outer, with the products of three matrices at a time in accumulation registers (one pass over
// the operand in LDS per group of three matrices, each weight fragment fetched once per step and workgroup), and
// applies gates, activation and leak in the epilogue.  One launch per time step; the state travels between
// launches through bump_history (forward) or a small fp32 carry buffer (BPTT), which is what makes any split of
// rows and columns over workgroups legal without a barrier.
//
// Measured against the one-tile-per-workgroup kernels of ring_bign.hip (same layouts): 10-25 % faster while the
// batch is small (N = 1024 up to 512 rows, N = 2048 up to 256 rows, e.g. 1.47 against 1.91 ms for 20 steps of
// N = 1024, B = 256, 16 channels), up to 1.6 times slower on large batches, where the launcher picks the others.
// More than one batch tile per workgroup (RT = 2) does not pay at the sizes the launcher sends here and exists for
// the forced path (RINGATTR_WIDE=0, RINGATTR_BLOCK=1); four or more need more accumulators than the register
// file holds next to a useful prefetch depth and were slower still.
//
// Layouts: weights [mm][tile][kc][lane][8] (ring_pack_weights_kernel, common tile order with run-time NC), operand
// copies for the weight-gradient kernel in paired tile order, the saved derivative record row-major fp16
// [t][16*nbt][NPAD] (the layout of the step-per-launch families).
#include "ring_step_common.hpp"

namespace {

// Stage RT batch tiles' operand rows (bf16, tile i at xb + i * slots) and their fp32 row sums (rs[16*i + row]).
template <int RT, typename F>
__device__ __forceinline__ void stage_tiles(bf16x8* xb, int slots, float* rs, int NPAD, int tid, F&& value4) {
  const int row = tid >> 4, sub = tid & 15;
#pragma unroll 1
  for (int i = 0; i < RT; ++i) {
    float sum = 0.f;
    char* base = reinterpret_cast<char*>(xb + (size_t)i * slots);
    for (int j = 4 * sub; j < NPAD; j += 64) {
      const f32x4 v = value4(16 * i + row, j);
      sum += (v[0] + v[1]) + (v[2] + v[3]);
      const bf16x4 pk = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
      *reinterpret_cast<bf16x4*>(base + (size_t)op_slot(j, row) * 16 + (j & 7) * 2) = pk;
    }
    sum = row16_sum_dpp(sum);
    if (sub == 0) rs[16 * i + row] = sum;
  }
}

// gates of the workgroup's RT*16 rows at step t, row-major with stride k (dynamic LDS behind the operand tiles)
template <int RT>
__device__ __forceinline__ void stage_gates_rt(float* gl, const float* __restrict__ A, int k, int T, int B, int t, int bt0,
                                               int tid) {
  for (int idx = tid; idx < RT * 16 * k; idx += 256) {
    const int row = idx / k, c = idx - row * k, b = 16 * bt0 + row;
    gl[idx] = b < B ? A[((size_t)b * T + t) * k + c] : 0.f;
  }
}

// bit c set <=> channel c has a non-zero gate in some of the workgroup's RT*16 rows
template <int RT>
__device__ __forceinline__ unsigned long long active_channels_rt(const float* gl, int k, int lane) {
  unsigned long long m = 0;
  for (int c0 = 0; c0 < k; c0 += 4) {
    const int c = c0 + (lane >> 4);
    bool nz = false;
    for (int i = 0; i < RT; ++i) nz |= c < k && gl[(16 * i + (lane & 15)) * k + c] != 0.f;
    const unsigned long long bal = __ballot(nz);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if ((bal >> (16 * j)) & 0xffffull) m |= 1ull << (c0 + j);
  }
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)m), hi = __builtin_amdgcn_readfirstlane((unsigned)(m >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// acc[i][cl][e] += sum_mm coef_mm[i][e] * (X_i @ W_mm)[row 4q+e][tile tg0 + cl] for the RT staged tiles X_i.
// Matrices are taken three at a time: one pass over the K chunks per group, the three products of every (i, cl) in
// accumulation registers, each A fragment read from LDS once per group and each weight fragment from global memory
// once per step.  coef_0 = J1, coef_{1+c} = gate of channel c; matrices whose channel is zero in all rows are skipped.
template <int RT, int TPW>
__device__ __forceinline__ void block_products(const bf16x8* xb, int slots, const bf16x8* __restrict__ Wp,
                                               const float* __restrict__ A, const float* gl, bool staged, int k, int T, int B,
                                               int t, int b0, float J1, int NC, int tg0, int lane,
                                               f32x4 (&acc)[RT][TPW]) {
  const int KCH = 2 * NC, q = lane >> 4, n = lane & 15;
  const unsigned long long active = staged ? active_channels_rt<RT>(gl, k, lane) : ~0ull;
  constexpr int PD = 8 / TPW;                              // K chunks of weight fragments in flight (24 KiB per wave)
  for (int m0 = 0; m0 <= k; m0 += 3) {
    bool use[3];
    const bf16x8* wm[3];
    bool any = false;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int mm = m0 + a;
      use[a] = mm <= k && (mm == 0 || !staged || ((active >> (mm - 1)) & 1ull));
      any |= use[a];
      // an unused slot points at matrix 0 (valid memory); its loads are issued and ignored
      wm[a] = Wp + ((size_t)(use[a] ? mm : 0) * 4 * NC + tg0) * KCH * 64 + lane;
    }
    if (!any) continue;
    f32x4 p[3][RT][TPW];
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
      for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int cl = 0; cl < TPW; ++cl) {
          p[a][i][cl] = f32x4{0.f, 0.f, 0.f, 0.f};
          asm volatile("" : "+a"(p[a][i][cl]));            // products live in the accumulation-register half
        }
    bf16x8 wf[PD][3][TPW];
#pragma unroll
    for (int d = 0; d < PD; ++d)
#pragma unroll
      for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int cl = 0; cl < TPW; ++cl) wf[d][a][cl] = wm[a][((size_t)cl * KCH + d) * 64];
    bf16x8 af[2][RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) af[0][i] = xb[(size_t)i * slots + (0 * 4 + q) * XG + n];
    for (int kc0 = 0; kc0 < KCH; kc0 += PD) {
#pragma unroll
      for (int d = 0; d < PD; ++d) {
        const int kc = kc0 + d;
        const int kn = kc + 1 < KCH ? kc + 1 : kc;         // next chunk's A fragments (past the end: a re-read)
#pragma unroll
        for (int i = 0; i < RT; ++i) af[(d + 1) & 1][i] = xb[(size_t)i * slots + (kn * 4 + q) * XG + n];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int a = 0; a < 3; ++a) {
          if (!use[a]) continue;
#pragma unroll
          for (int cl = 0; cl < TPW; ++cl)
#pragma unroll
            for (int i = 0; i < RT; ++i) p[a][i][cl] = mfma16(af[d & 1][i], wf[d][a][cl], p[a][i][cl]);
        }
        // refill this slot with the chunk PD ahead (past the end: a re-read of the last chunk, unused)
        const int kp = kc + PD < KCH ? kc + PD : KCH - 1;
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
          for (int cl = 0; cl < TPW; ++cl) wf[d][a][cl] = wm[a][((size_t)cl * KCH + kp) * 64];
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      if (!use[a]) continue;
      const int mm = m0 + a;
#pragma unroll
      for (int i = 0; i < RT; ++i) {
        float coef[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (mm == 0) coef[e] = J1;
          else if (staged) coef[e] = gl[(16 * i + 4 * q + e) * k + (mm - 1)];
          else coef[e] = (b0 + 16 * i + e < B) ? A[((size_t)(b0 + 16 * i + e) * T + t) * k + (mm - 1)] : 0.f;
        }
#pragma unroll
        for (int cl = 0; cl < TPW; ++cl)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][cl][e] = fmaf(coef[e], p[a][i][cl][e], acc[i][cl][e]);
      }
    }
  }
}

}  // namespace

// One forward step for RT batch tiles x 64*TPW neurons per workgroup (REBUILD: the saved record of every step at
// once from an existing history, grid.z = T).
template <int ACT, bool REBUILD, int RT, int TPW>
__global__ __launch_bounds__(256) void ring_block_fwd_kernel(RingFwdArgs p, int NC, int t_arg, int xcd_map) {
  extern __shared__ __attribute__((aligned(16))) char block_lds[];
  bf16x8* xb = reinterpret_cast<bf16x8*>(block_lds);
  __shared__ float rs[16 * RT];
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  int rgi, cb;
  step_block_coords(xcd_map, rgi, cb);
  const int bt0 = rgi * RT, t = REBUILD ? (int)blockIdx.z : t_arg;
  const int N = p.N, B = p.B, T = p.T, NPAD = 64 * NC, slots = 2 * NC * 4 * XG;
  const bool staged = p.k <= BN_GATE_KMAX;
  float* gl = reinterpret_cast<float*>(xb + (size_t)RT * slots);
  const float* prev = (t == 0) ? p.r_init : p.hist + (size_t)(t - 1) * B * N;

  stage_tiles<RT>(xb, slots, rs, NPAD, tid, [&](int row, int j) { return load4_masked(prev, N, B, 16 * bt0 + row, j); });
  if (staged) stage_gates_rt<RT>(gl, p.A, p.k, T, B, t, bt0, tid);
  lds_barrier();

  const int tg0 = 4 * TPW * cb + TPW * wv;                // this wave's first column tile
  const int wg = tg0 / NC, c0 = tg0 % NC;                 // common tile order: tile = wg * NC + c
  const int j0 = 16 * NC * wg + NC * n + c0;              // the lane's TPW consecutive neurons
  const int b0 = 16 * bt0 + 4 * q;
  f32x4 acc[RT][TPW];
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int cl = 0; cl < TPW; ++cl) acc[i][cl] = f32x4{0.f, 0.f, 0.f, 0.f};
  block_products<RT, TPW>(xb, slots, (const bf16x8*)p.Wpack, p.A, gl, staged, p.k, T, B, t, b0, p.J1, NC, tg0, lane, acc);

  const float oma = 1.f - p.alpha;
  const size_t rows_pad = (size_t)16 * p.nbt;
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    if (bt0 + i >= p.nbt) break;                           // a partial last block of batch tiles
    bf16x4 rcopy[TPW], ncopy[TPW];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int b = b0 + 16 * i + e;
      const f32x4 rp = loadv_masked<TPW>(prev, N, B, b, j0);
      const float js = p.J0 * rs[16 * i + 4 * q + e];
      f32x4 rn = {0.f, 0.f, 0.f, 0.f}, dd = rn;
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) {
        float F, D;
        act_fast<ACT>(acc[i][cl][e] + js, F, D);
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
        _Float16* dst = p.dfrag + ((size_t)t * rows_pad + 16 * (bt0 + i) + 4 * q + e) * NPAD + j0;
#pragma unroll
        for (int cl = 0; cl < TPW; ++cl) dst[cl] = (_Float16)dd[cl];
      }
    }
    if (p.rfrag && (t & 1) == 0) {
      // both halves of the pair slot (this step's operand and the next one's) as one 16-byte store, as in
      // ring_wide_fwd_kernel; odd steps write none
      const bool tail = t + 1 == T;
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) {
        const bf16x4 hi = tail ? bf16x4{(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f} : ncopy[cl];
        *reinterpret_cast<bf16x8*>(p.rfrag + pair_off_rt(NC, t, p.nbt, bt0 + i, tg0 + cl, lane)) =
            __builtin_shufflevector(rcopy[cl], hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    }
  }
}

// One BPTT step t for RT batch tiles x 64*TPW neurons per workgroup (see ring_wide_bptt_kernel for the recurrence).
template <int RT, int TPW, bool LOSS>
__global__ __launch_bounds__(256) void ring_block_bptt_kernel(RingBpttArgs p, int NC, int t, const float* carry_in,
                                                              float* carry_out, int xcd_map) {
  extern __shared__ __attribute__((aligned(16))) char block_lds[];
  bf16x8* xb = reinterpret_cast<bf16x8*>(block_lds);
  __shared__ float rs[16 * RT];
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  int rgi, cb;
  step_block_coords(xcd_map, rgi, cb);
  const int bt0 = rgi * RT;
  const int N = p.N, B = p.B, T = p.T, NPAD = 64 * NC, slots = 2 * NC * 4 * XG;
  const bool staged = p.k <= BN_GATE_KMAX;
  float* gl = reinterpret_cast<float*>(xb + (size_t)RT * slots);
  const size_t rows_pad = (size_t)16 * p.nbt;
  const float* gout = LOSS ? nullptr : p.grad_out + (size_t)t * B * N;
  const _Float16* drow = p.dfrag + (size_t)t * rows_pad * NPAD;
  // LOSS: grad_output is not read; it is formed from the state history and the loss head's row coefficients
  const float up = LOSS ? (p.loss_upstream ? p.loss_upstream[0] : 1.f) * p.loss_inv_rows : 0.f;

  // g of (row within the block, j..j+V-1); carry rows live in a padded [16*nbt][NPAD] buffer.  Rows of batch tiles
  // past the last one (a partial last block) read as zero.
  auto g4 = [&](int row, int j, f32x4& G) {
    const size_t prow = (size_t)16 * bt0 + row;
    G = f32x4{0.f, 0.f, 0.f, 0.f};
    if (prow >= rows_pad) return G;
    if constexpr (LOSS) G = loss_grad4(p, t, (int)prow, j, up);
    else G = load4_masked(gout, N, B, (int)prow, j);
    if (carry_in) G += *reinterpret_cast<const f32x4*>(carry_in + prow * NPAD + j);
    const f16x4 d = *reinterpret_cast<const f16x4*>(drow + prow * NPAD + j);
    // products rounded on their own (never contracted into the row sum that follows), so that both step-per-launch
    // families form bit-identical g and row sums whatever the compiler does with the surrounding code
    f32x4 g;
    {
#pragma clang fp contract(off)
      g = f32x4{(float)d[0] * G[0], (float)d[1] * G[1], (float)d[2] * G[2], (float)d[3] * G[3]};
    }
    return g;
  };
  stage_tiles<RT>(xb, slots, rs, NPAD, tid, [&](int row, int j) { f32x4 G; return g4(row, j, G); });
  if (staged) stage_gates_rt<RT>(gl, p.A, p.k, T, B, t, bt0, tid);
  lds_barrier();

  const int tg0 = 4 * TPW * cb + TPW * wv;
  const int wg = tg0 / NC, c0 = tg0 % NC;
  const int j0 = 16 * NC * wg + NC * n + c0;
  const int j4 = j0 & ~3, jo = j0 & 3;                    // the 16-byte group holding the lane's TPW neurons
  const int b0 = 16 * bt0 + 4 * q;
  const float oma = 1.f - p.alpha;
  f32x4 acc[RT][TPW];
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    bf16x4 gcopy[TPW];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f32x4 G;
      const f32x4 g = g4(16 * i + 4 * q + e, j4, G);
      const float js = p.J0 * rs[16 * i + 4 * q + e];
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) {
        acc[i][cl][e] = fmaf(oma, G[jo + cl], js);
        gcopy[cl][e] = (__bf16)g[jo + cl];
      }
    }
    if (bt0 + i < p.nbt) {
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl)
        *reinterpret_cast<bf16x4*>(p.gfrag + pair_off_rt(NC, t, p.nbt, bt0 + i, tg0 + cl, lane)) = gcopy[cl];
      if (t == T - 1 && (T & 1)) {
        const bf16x4 z = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
#pragma unroll
        for (int cl = 0; cl < TPW; ++cl)
          *reinterpret_cast<bf16x4*>(p.gfrag + pair_off_rt(NC, T, p.nbt, bt0 + i, tg0 + cl, lane)) = z;
      }
    }
  }
  block_products<RT, TPW>(xb, slots, (const bf16x8*)p.Wpack, p.A, gl, staged, p.k, T, B, t, b0, p.J1, NC, tg0, lane, acc);
#pragma unroll
  for (int i = 0; i < RT; ++i) {
    if (bt0 + i >= p.nbt) break;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int b = b0 + 16 * i + e;
      f32x4 out = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) out[cl] = (b < B && j0 + cl < N) ? acc[i][cl][e] : 0.f;
      float* dst = carry_out + ((size_t)16 * (bt0 + i) + 4 * q + e) * NPAD + j0;
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) dst[cl] = out[cl];
      if (t == 0 && p.grad_r_init) storev_masked<TPW>(p.grad_r_init, N, B, b, j0, out);
    }
  }
}

// dL/dA for the step-per-launch families, after the BPTT steps have left g (bf16, paired tile order) for every step:
//   grad_A[b, t, c] = sum_i g[t, b, i] * (Wa[c] @ r_prev[t, b])_i
// No recurrence: one workgroup per (batch tile, step) stages the tile's r_prev rows as the forward does, walks all
// column blocks with the forward fragments of three channels at a time, multiplies each product by the lane's g
// (the paired layout is exactly the MFMA result layout) and reduces over neurons -- lanes by DPP, waves through LDS
// in wave order, so the result does not depend on scheduling.  Wf: forward-orientation packed weights.
template <int TPW>
__global__ __launch_bounds__(256) void ring_block_grad_A_kernel(RingBpttArgs p, const bf16x8* __restrict__ Wf, int NC) {
  extern __shared__ __attribute__((aligned(16))) char block_lds[];
  bf16x8* xb = reinterpret_cast<bf16x8*>(block_lds);
  __shared__ float rs[16];
  __shared__ float part[3][4][16];
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int bt = blockIdx.x, t = blockIdx.y;
  const int N = p.N, B = p.B, T = p.T, k = p.k, NPAD = 64 * NC, slots = 2 * NC * 4 * XG, KCH = 2 * NC;
  const float* prev = (t == 0) ? p.r_init : p.hist + (size_t)(t - 1) * B * N;
  stage_tiles<1>(xb, slots, rs, NPAD, tid, [&](int row, int j) { return load4_masked(prev, N, B, 16 * bt + row, j); });
  lds_barrier();

  for (int m0 = 1; m0 <= k; m0 += 3) {
    float ga[3][4];
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
      for (int e = 0; e < 4; ++e) ga[a][e] = 0.f;
    for (int cb = 0; cb < NC / TPW; ++cb) {
      const int tg0 = 4 * TPW * cb + TPW * wv;
      const bf16x8* wm[3];
#pragma unroll
      for (int a = 0; a < 3; ++a)   // a slot past the last channel reads channel k again (valid memory), result unused
        wm[a] = Wf + ((size_t)(m0 + a <= k ? m0 + a : k) * 4 * NC + tg0) * KCH * 64 + lane;
      f32x4 pr[3][TPW];
#pragma unroll
      for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int cl = 0; cl < TPW; ++cl) pr[a][cl] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int kc0 = 0; kc0 < KCH; kc0 += 4) {          // NC is even, so KCH is a multiple of four
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int kc = kc0 + u;
          const bf16x8 af = xb[(kc * 4 + q) * XG + n];
#pragma unroll
          for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int cl = 0; cl < TPW; ++cl) pr[a][cl] = mfma16(af, wm[a][((size_t)cl * KCH + kc) * 64], pr[a][cl]);
        }
      }
#pragma unroll
      for (int cl = 0; cl < TPW; ++cl) {
        const bf16x4 gv = *reinterpret_cast<const bf16x4*>(p.gfrag + pair_off_rt(NC, t, p.nbt, bt, tg0 + cl, lane));
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
          for (int e = 0; e < 4; ++e) ga[a][e] = fmaf(pr[a][cl][e], (float)gv[e], ga[a][e]);
      }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sum = row16_sum_dpp(ga[a][e]);
        if (n == 0) part[a][wv][4 * q + e] = sum;
      }
    lds_barrier();
    if (tid < 48) {
      const int a = tid >> 4, row = tid & 15, c = m0 - 1 + a, b = 16 * bt + row;
      if (c < k && b < B)
        p.grad_A[((size_t)b * T + t) * k + c] = ((part[a][0][row] + part[a][1][row]) + part[a][2][row]) + part[a][3][row];
    }
    lds_barrier();
  }
}

// ------------------------------------------------------------------------------------------------
// Launchers
// ------------------------------------------------------------------------------------------------
// operand tiles + the staged gates (a_dim <= BN_GATE_KMAX; wider action signals read their gates from global memory)
static size_t block_lds_bytes(int NC, int RT, int k) {
  return (size_t)RT * 2 * NC * 4 * XG * sizeof(bf16x8) + (k <= BN_GATE_KMAX ? (size_t)RT * 16 * k * sizeof(float) : 0);
}

// Tiles per wave (a workgroup owns 64 * tpw neurons) and row tiles per workgroup, from measurements on 16 to 256
// batch tiles at N = 1024 and 2048:
//  * many matrices (more than two groups of three, e.g. 16 action channels): the weight stream dominates.  Two row
//    tiles per workgroup (every fetched fragment feeds two MFMAs) and one tile per wave while all workgroups are
//    resident at once (twice the streams in flight), two tiles per wave beyond that;
//  * few matrices: staging the operand rows is what a workgroup waits for, so one row tile and two tiles per wave
//    (fewest workgroups re-staging the same rows) until the grid covers the device also with two row tiles.
// RINGATTR_BLOCK_SHAPE=<rt><tpw> (e.g. 21) forces a shape (cross-checks).
bool ring_block_many_matrices(int k) { return 1 + k > 6; }

void ring_block_geometry(int NC, int nbt, int k, int* rt_out, int* tpw_out) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
  const size_t lds_cap = 160 * 1024 - 2 * 1024;
  int rt, tpw;
  if (ring_block_many_matrices(k)) {
    rt = (nbt >= 2 && block_lds_bytes(NC, 2, k) <= lds_cap) ? 2 : 1;
    const long per_cu = (long)(lds_cap / block_lds_bytes(NC, rt, k));
    tpw = (long)((nbt + rt - 1) / rt) * NC <= (long)cus * (per_cu > 0 ? per_cu : 1) ? 1 : 2;
  } else {
    tpw = 2;
    rt = (block_lds_bytes(NC, 2, k) <= lds_cap && (long)((nbt + 1) / 2) * (NC / 2) >= cus) ? 2 : 1;
  }
  if (const char* v = getenv("RINGATTR_BLOCK_SHAPE")) {
    if ((v[0] == '1' || v[0] == '2') && (v[1] == '1' || v[1] == '2') && v[2] == 0) {
      const int frt = v[0] - '0';
      if (block_lds_bytes(NC, frt, k) <= lds_cap) rt = frt;
      tpw = v[1] - '0';
    }
  }
  *rt_out = rt;
  *tpw_out = tpw;
}

template <typename K>
static hipError_t block_attr(K kern, size_t dyn) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
}

template <int ACT, int RT, int TPW>
static hipError_t block_fwd_shape(const RingFwdArgs& a, int NC, bool rebuild, hipStream_t st) {
  const size_t dyn = block_lds_bytes(NC, RT, a.k);
  const dim3 grid((a.nbt + RT - 1) / RT, NC / TPW, rebuild ? a.T : 1);
  const int xm = step_xcd_map();
  if (rebuild) {
    hipError_t e = block_attr(ring_block_fwd_kernel<ACT, true, RT, TPW>, dyn);
    if (e != hipSuccess) return e;
    RING_LAUNCH((ring_block_fwd_kernel<ACT, true, RT, TPW>), grid, dim3(256), dyn, st, a, NC, 0, xm);
    return hipGetLastError();
  }
  hipError_t e = block_attr(ring_block_fwd_kernel<ACT, false, RT, TPW>, dyn);
  if (e != hipSuccess) return e;
  for (int t = 0; t < a.T; ++t) {
    RING_LAUNCH((ring_block_fwd_kernel<ACT, false, RT, TPW>), grid, dim3(256), dyn, st, a, NC, t, xm);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int ACT>
static hipError_t block_fwd_act(const RingFwdArgs& a, int NC, bool rebuild, int rt, int tpw, hipStream_t st) {
  if (rt == 2) return tpw == 2 ? block_fwd_shape<ACT, 2, 2>(a, NC, rebuild, st) : block_fwd_shape<ACT, 2, 1>(a, NC, rebuild, st);
  return tpw == 2 ? block_fwd_shape<ACT, 1, 2>(a, NC, rebuild, st) : block_fwd_shape<ACT, 1, 1>(a, NC, rebuild, st);
}

hipError_t ring_launch_block_fwd(const RingFwdArgs& a, int NC, bool rebuild, hipStream_t st) {
  if (NC % 2 != 0) return hipErrorInvalidValue;
  int rt, tpw;
  ring_block_geometry(NC, a.nbt, a.k, &rt, &tpw);
  switch (a.act) {
    case ACT_RELU: return block_fwd_act<ACT_RELU>(a, NC, rebuild, rt, tpw, st);
    case ACT_GELU: return block_fwd_act<ACT_GELU>(a, NC, rebuild, rt, tpw, st);
    case ACT_TANH: return block_fwd_act<ACT_TANH>(a, NC, rebuild, rt, tpw, st);
    case ACT_SILU: return block_fwd_act<ACT_SILU>(a, NC, rebuild, rt, tpw, st);
    default: return hipErrorInvalidValue;
  }
}

template <int RT, int TPW, bool LOSS>
static hipError_t block_bptt_shape(const RingBpttArgs& a, int NC, float* carry, hipStream_t st) {
  const size_t dyn = block_lds_bytes(NC, RT, a.k);
  hipError_t e = block_attr(ring_block_bptt_kernel<RT, TPW, LOSS>, dyn);
  if (e != hipSuccess) return e;
  const size_t half = (size_t)16 * a.nbt * 64 * NC;
  const dim3 grid((a.nbt + RT - 1) / RT, NC / TPW);
  const int xm = step_xcd_map();
  for (int t = a.T - 1, u = 0; t >= 0; --t, ++u) {
    const float* cin = (u == 0) ? nullptr : carry + (size_t)((u - 1) & 1) * half;
    float* cout = carry + (size_t)(u & 1) * half;
    RING_LAUNCH((ring_block_bptt_kernel<RT, TPW, LOSS>), grid, dim3(256), dyn, st, a, NC, t, cin, cout, xm);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// carry: 2 * 16 * nbt * NPAD floats of scratch (ring_wide_carry_bytes), used as two alternating buffers
hipError_t ring_launch_block_bptt(const RingBpttArgs& a, int NC, float* carry, hipStream_t st) {
  if (NC % 2 != 0) return hipErrorInvalidValue;
  int rt, tpw;
  ring_block_geometry(NC, a.nbt, a.k, &rt, &tpw);
  if (a.loss_coef) {
    if (!a.loss_trig || !a.hist) return hipErrorInvalidValue;
    if (rt == 2) return tpw == 2 ? block_bptt_shape<2, 2, true>(a, NC, carry, st) : block_bptt_shape<2, 1, true>(a, NC, carry, st);
    return tpw == 2 ? block_bptt_shape<1, 2, true>(a, NC, carry, st) : block_bptt_shape<1, 1, true>(a, NC, carry, st);
  }
  if (!a.grad_out) return hipErrorInvalidValue;
  if (rt == 2) return tpw == 2 ? block_bptt_shape<2, 2, false>(a, NC, carry, st) : block_bptt_shape<2, 1, false>(a, NC, carry, st);
  return tpw == 2 ? block_bptt_shape<1, 2, false>(a, NC, carry, st) : block_bptt_shape<1, 1, false>(a, NC, carry, st);
}

// a.grad_A, a.gfrag (complete), a.hist, a.r_init; Wf: forward-orientation packed weights (matrix 0 is not read)
hipError_t ring_launch_block_grad_A(const RingBpttArgs& a, const void* Wf, int NC, hipStream_t st) {
  if (NC % 2 != 0 || !a.grad_A || !a.gfrag || !a.hist || !a.r_init || !Wf) return hipErrorInvalidValue;
  if (a.T > 65535) return hipErrorInvalidValue;   // grid.y
  const size_t dyn = (size_t)2 * NC * 4 * XG * sizeof(bf16x8);
  hipError_t e = block_attr(ring_block_grad_A_kernel<2>, dyn);
  if (e != hipSuccess) return e;
  RING_LAUNCH((ring_block_grad_A_kernel<2>), dim3(a.nbt, a.T), dim3(256), dyn, st, a, (const bf16x8*)Wf, NC);
  return hipGetLastError();
}
