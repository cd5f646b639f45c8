// Helpers shared by the step-per-launch kernel families (ring_bign.hip, ring_block.hip): run-time-NC layout
// offsets, masked row loads and stores, staging of operand rows and action gates into LDS.
#pragma once
#include "ring_common.hpp"
#include "ring_kernels.hpp"

#include <stdlib.h>

namespace {

constexpr int BN_GATE_KMAX = 64;

// Which (row group, column block) a workgroup takes.  Workgroups go to the eight XCDs round-robin by linear index,
// and every XCD has its own L2.  With the plain (x = row group, y = column block) order each XCD sees every column
// block, i.e. pulls the whole packed weight set out of HBM for itself -- eight fetches of every weight byte per
// step, which is what bounds small batches of wide rings.  When the column blocks divide by eight, XCD x instead
// owns column blocks x * cpx .. (x+1) * cpx - 1 for all row groups: each weight byte leaves HBM once per step and is
// shared through that XCD's L2 by the row groups running side by side.  With fewer than eight column blocks the
// packed weights are small enough for every XCD's L2, and letting several XCDs share a block was measured to cost a
// little, so those grids keep the plain order.  Any placement gives correct results; the mapping only decides what
// the caches see.  xcd_map = 0 keeps the plain order.
__device__ __forceinline__ void step_block_coords(int xcd_map, int& rg, int& cb) {
  const int nrg = gridDim.x, ncb = gridDim.y;
  rg = blockIdx.x;
  cb = blockIdx.y;
  if (xcd_map && (ncb & 7) == 0) {
    const int L = blockIdx.x + nrg * blockIdx.y, xcd = L & 7, w = L >> 3, cpx = ncb >> 3;
    rg = w % nrg;
    cb = xcd * cpx + w / nrg;
  }
}

// RINGATTR_XCD_MAP=0: plain workgroup order (see step_block_coords)
inline int step_xcd_map() {
  const char* v = getenv("RINGATTR_XCD_MAP");
  return (v && v[0] == '0') ? 0 : 1;
}


__device__ __forceinline__ size_t pair_off_rt(int NC, int t, int nbt, int bt, int tile, int lane) {
  return (((((size_t)(t >> 1) * nbt + bt) * (size_t)(4 * NC) + tile) * 64 + lane) * 2 + (t & 1)) * 4;
}

// slot of K position j (neuron), row b in the LDS operand buffer (see write_operand): 16-byte slots, groups padded to XG
__device__ __forceinline__ int op_slot(int j, int b) { return ((j >> 5) * 4 + ((j >> 3) & 3)) * XG + b; }

// Stage the batch tile's operand rows: v(row, j) for all j < NPAD as bf16 into xb, and the fp32 row sums into rs[16].
// Thread (row = tid / 16, sub = tid % 16) walks its row in float4 groups 64 neurons apart.  F(b, j4, ok4) returns the
// four fp32 values of neurons j4..j4+3 of batch row b (zero where masked).
template <typename F>
__device__ __forceinline__ void stage_rows(bf16x8* xb, float* rs, int NPAD, int tid, F&& value4) {
  const int row = tid >> 4, sub = tid & 15;
  float sum = 0.f;
  char* base = reinterpret_cast<char*>(xb);
  for (int j = 4 * sub; j < NPAD; j += 64) {
    const f32x4 v = value4(row, j);
    sum += (v[0] + v[1]) + (v[2] + v[3]);
    const bf16x4 pk = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
    *reinterpret_cast<bf16x4*>(base + (size_t)op_slot(j, row) * 16 + (j & 7) * 2) = pk;
  }
  sum = row16_sum_dpp(sum);
  if (sub == 0) rs[row] = sum;
}

// fp32 [rows][N] row-major, four consecutive neurons, masked
__device__ __forceinline__ f32x4 load4_masked(const float* slab, int N, int B, int b, int j) {
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  if (b >= B || j >= N) return v;
  const float* src = slab + (size_t)b * N + j;
  if ((N & 3) == 0) return *reinterpret_cast<const f32x4*>(src);   // j is a multiple of 4, so j + 3 < N
#pragma unroll
  for (int x = 0; x < 4; ++x)
    if (j + x < N) v[x] = src[x];
  return v;
}

// The loss head's gradient in place of grad_output (step-per-launch BPTT kernels): four neurons j..j+3 of history row
// (t, b),  up * (kc cos(phi_j) + ks sin(phi_j) + beta sign(r_j)),  (kc, ks, beta) = loss_coef[t * B + b], the state r
// read where grad_output would have been (same bytes), (cos, sin) from the table of ring_launch_trig_table.
__device__ __forceinline__ f32x4 loss_grad4(const RingBpttArgs& p, int t, int b, int j, float up) {
  f32x4 g = {0.f, 0.f, 0.f, 0.f};
  if (b >= p.B || j >= p.N) return g;
  const f32x4 c = p.loss_coef[(size_t)t * p.B + b];
  const f32x4 r = load4_masked(p.hist + (size_t)t * p.B * p.N, p.N, p.B, b, j);
  const float kc = c[0] * up, ks = c[1] * up, beta = c[2] * up;
  const f32x4 t0 = *reinterpret_cast<const f32x4*>(p.loss_trig + 2 * j);        // j is a multiple of 4
  const f32x4 t1 = *reinterpret_cast<const f32x4*>(p.loss_trig + 2 * j + 4);
  const float cs[4] = {t0[0], t0[2], t1[0], t1[2]}, sn[4] = {t0[1], t0[3], t1[1], t1[3]};
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const float sb = r[x] > 0.f ? beta : (r[x] < 0.f ? -beta : 0.f);              // beta * sign(r), sign(0) = 0
    g[x] = j + x < p.N ? fmaf(kc, cs[x], fmaf(ks, sn[x], sb)) : 0.f;
  }
  return g;
}

__device__ __forceinline__ void store4_masked(float* slab, int N, int B, int b, int j, f32x4 v) {
  if (b >= B || j >= N) return;
  float* dst = slab + (size_t)b * N + j;
  if ((N & 3) == 0) {
    *reinterpret_cast<f32x4*>(dst) = v;
    return;
  }
#pragma unroll
  for (int x = 0; x < 4; ++x)
    if (j + x < N) dst[x] = v[x];
}

// V consecutive neurons (V in {1, 2, 4}) of one batch row as a zero-padded f32x4
template <int V>
__device__ __forceinline__ f32x4 loadv_masked(const float* slab, int N, int B, int b, int j) {
  if constexpr (V == 4) return load4_masked(slab, N, B, b, j);
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  if (b >= B) return v;
  const float* src = slab + (size_t)b * N + j;
#pragma unroll
  for (int x = 0; x < V; ++x)
    if (j + x < N) v[x] = src[x];
  return v;
}

template <int V>
__device__ __forceinline__ void storev_masked(float* slab, int N, int B, int b, int j, f32x4 v) {
  if constexpr (V == 4) {
    store4_masked(slab, N, B, b, j, v);
    return;
  }
  if (b >= B) return;
  float* dst = slab + (size_t)b * N + j;
#pragma unroll
  for (int x = 0; x < V; ++x)
    if (j + x < N) dst[x] = v[x];
}

__device__ __forceinline__ void stage_gates(float* gl, const float* __restrict__ A, int k, int T, int B, int t, int bt, int tid) {
  for (int idx = tid; idx < 16 * k; idx += 256) {
    const int row = idx / k, c = idx - row * k, b = 16 * bt + row;
    gl[row * BN_GATE_KMAX + c] = b < B ? A[((size_t)b * T + t) * k + c] : 0.f;
  }
}

// bit c set <=> channel c has a non-zero gate in some of the 16 rows (same value in every lane)
__device__ __forceinline__ unsigned long long active_channels(const float* gl, int k, int lane) {
  unsigned long long m = 0;
  for (int c0 = 0; c0 < k; c0 += 4) {
    const int c = c0 + (lane >> 4);
    const bool nz = c < k && gl[(lane & 15) * BN_GATE_KMAX + c] != 0.f;
    const unsigned long long bal = __ballot(nz);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if ((bal >> (16 * j)) & 0xffffull) m |= 1ull << (c0 + j);
  }
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)m), hi = __builtin_amdgcn_readfirstlane((unsigned)(m >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

}  // namespace
