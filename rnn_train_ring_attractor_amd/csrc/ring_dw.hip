// Weight-gradient contraction, LDS-tiled variant for NPAD >= 256 (NC = 4 or 8).
//
//   dW_mm[i][j] = sum over samples (b,t) of coef_mm(b,t) * g[t,b,i] * r_prev[t,b,j]
//
// Work decomposition: a workgroup (8 waves, 2 per SIMD) owns a 128 (i) x 128 (j) output tile of up to
// three matrices over one K split; wave v owns row tiles 2*(v/2), 2*(v/2)+1 against column tiles
// 4*(v%2) .. +3 (24 MFMAs per 6 operand reads: the LDS pipe, shared by the CU, stays under the MFMA
// time).  A K chunk is 16 batch rows x 2 time steps (32 samples, one MFMA K).  The paired
// tile-major operand buffers hold every tile of a chunk as 1 KiB of ready-made MFMA fragments, so
// the stage is a verbatim copy: global -> registers (DW_DEPTH chunks in flight) -> double-buffered
// LDS -> one conflict-free ds_read_b128 per operand.  The action gates of the chunk ride along.
// Partials are written once per workgroup; a fixed-order reduction follows.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

namespace {

constexpr int DW_TI = 8;      // row tiles per workgroup (128 neurons)
constexpr int DW_TJ = 8;      // column tiles per workgroup (128 neurons)
constexpr int DW_DEPTH = 4;   // K chunks in flight in registers

constexpr int DW_THREADS = 512;
constexpr int DW_WI = 2, DW_WJ = 4;   // row / column tiles per wave

struct DwStage {
  f32x4 a;      // one 16-byte fragment of the g block (8 tiles x 64 lanes = 512 fragments)
  f32x4 b;      // one of the r_prev block
  float cf;     // one gate value (meaningful in threads 0..95)
};

// Branch-free on purpose: with no control flow around the loads the compiler can count the chunks in
// flight and wait for exactly the oldest one (s_waitcnt vmcnt(n)) instead of draining all of them.
// The chunk (bt, t0) is valid by construction of the caller's cursor; gate indices that fall outside the problem are clamped and zeroed.
template <int NC>
__device__ __forceinline__ void dw_fetch(const RingDwArgs& p, int bt, int t0, int it0, int jt0, int mg, int tid, DwStage& s) {
  const int nbt = p.nbt, T = p.T;
  const f32x4* ga = reinterpret_cast<const f32x4*>(p.gfrag + pair_offset<NC>(t0, nbt, bt, it0, 0));
  const f32x4* rb = reinterpret_cast<const f32x4*>(p.rfrag + pair_offset<NC>(t0, nbt, bt, jt0, 0));
  s.a = ga[tid];
  s.b = rb[tid];
  // gates: thread = (a, tau, row); threads past 96 load a clamped duplicate that is zeroed
  const int a = tid >> 5, tau = (tid >> 4) & 1, row = tid & 15;
  const int mm = 3 * mg + a, b = 16 * bt + row, t = t0 + tau;
  const bool ok = (a < 3) && (mm >= 1) && (mm <= p.k) && (b < p.B) && (t < T);
  const int mmc = mm < 1 ? 1 : (mm > p.k ? p.k : mm);
  const int bc = b < p.B ? b : p.B - 1, tc = t < T ? t : T - 1;
  const float v = p.A[((size_t)bc * T + tc) * p.k + (mmc - 1)];
  s.cf = ok ? v : 0.f;
}

__device__ __forceinline__ void dw_publish(f32x4* la, f32x4* lb, float* lc, int tid, const DwStage& s) {
  la[tid] = s.a;
  lb[tid] = s.b;
  lc[tid] = s.cf;
}

__device__ __forceinline__ bf16x8 gate_frag(bf16x8 x, f32x4 c0, f32x4 c1) {
  bf16x8 o;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    o[u] = (__bf16)((float)x[u] * c0[u]);
    o[4 + u] = (__bf16)((float)x[4 + u] * c1[u]);
  }
  return o;
}

}  // namespace

// NMAT = matrices of this workgroup's group (1..3); FIRST = the group starts with Wo (ungated).
template <int NC, int NMAT, bool FIRST>
__global__ __launch_bounds__(DW_THREADS) void ring_dw_tiled_kernel(RingDwArgs p, int mg) {
  constexpr int NT = 4 * NC;
  constexpr int NIB = NT / DW_TI, NJB = NT / DW_TJ;
  __shared__ __attribute__((aligned(16))) f32x4 lds_a[2][DW_TI * 64];
  __shared__ __attribute__((aligned(16))) f32x4 lds_b[2][DW_TJ * 64];
  __shared__ __attribute__((aligned(16))) float lds_c[2][DW_THREADS];

  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4;
  const int wi = wv >> 1, wj = wv & 1;
  const int tiles = NIB * NJB;
  // keep the workgroups that share a K split on one XCD (workgroup ids are dealt round-robin to
  // the 8 XCDs) so the operand bytes they all read come out of that XCD's L2
  int z, tile;
  {
    const int bid = blockIdx.x;
    if ((p.nz & 7) == 0) {
      const int xcd = bid & 7, slot = bid >> 3;
      z = xcd * (p.nz >> 3) + slot / tiles;
      tile = slot % tiles;
    } else {
      z = bid / tiles;
      tile = bid % tiles;
    }
  }
  const int ib = tile % NIB, jb = tile / NIB;
  const int it0 = ib * DW_TI, jt0 = jb * DW_TJ;

  const int nchunk = p.nbt * ((p.T + 1) / 2);   // the host checked that this fits an int
  const int ch0 = (int)((long)nchunk * z / p.nz), ch1 = (int)((long)nchunk * (z + 1) / p.nz);

  f32x4 acc[NMAT][DW_WI][DW_WJ];
#pragma unroll
  for (int a = 0; a < NMAT; ++a)
#pragma unroll
    for (int ii = 0; ii < DW_WI; ++ii)
#pragma unroll
      for (int u = 0; u < DW_WJ; ++u) acc[a][ii][u] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Fetch cursor: chunk = (batch tile fb, time-step pair ft), batch tile fastest.  It advances one
  // chunk per fetch with compare-and-wrap (no division in the loop) and parks on the last chunk of
  // the split, so fetches past the end re-read valid data that is never consumed.
  int fc = ch0, fb = ch0 % p.nbt, ft = ch0 / p.nbt;
  auto fetch_next = [&](DwStage& s) {
    dw_fetch<NC>(p, fb, 2 * ft, it0, jt0, mg, tid, s);
    // branch-free advance (scalar selects): a trip of the main loop must stay one basic block so
    // that the compiler keeps an exact count of the loads in flight
    const int adv = (fc + 1 < ch1) ? 1 : 0;
    fc += adv;
    fb += adv;
    const int wrap = (fb == p.nbt) ? 1 : 0;
    fb = wrap ? 0 : fb;
    ft += wrap;
  };
  auto compute = [&](int cur) {
    bf16x8 ga[DW_WI], rb[DW_WJ];
#pragma unroll
    for (int ii = 0; ii < DW_WI; ++ii)
      ga[ii] = *reinterpret_cast<const bf16x8*>(&lds_a[cur][(DW_WI * wi + ii) * 64 + lane]);
    f32x4 cf[NMAT][2];
#pragma unroll
    for (int a = 0; a < NMAT; ++a) {
      cf[a][0] = *reinterpret_cast<const f32x4*>(&lds_c[cur][a * 32 + 4 * q]);
      cf[a][1] = *reinterpret_cast<const f32x4*>(&lds_c[cur][a * 32 + 16 + 4 * q]);
    }
#pragma unroll
    for (int u = 0; u < DW_WJ; ++u) rb[u] = *reinterpret_cast<const bf16x8*>(&lds_b[cur][(DW_WJ * wj + u) * 64 + lane]);
#pragma unroll
    for (int a = 0; a < NMAT; ++a) {
#pragma unroll
      for (int ii = 0; ii < DW_WI; ++ii) {
        const bf16x8 gg = (FIRST && a == 0) ? ga[ii] : gate_frag(ga[ii], cf[a][0], cf[a][1]);
#pragma unroll
        for (int u = 0; u < DW_WJ; ++u) acc[a][ii][u] = mfma16(gg, rb[u], acc[a][ii][u]);
      }
    }
  };

  if (ch0 < ch1) {
    DwStage st[DW_DEPTH];
#pragma unroll
    for (int d = 0; d < DW_DEPTH; ++d) fetch_next(st[d]);
    dw_publish(lds_a[0], lds_b[0], lds_c[0], tid, st[0]);
    __syncthreads();

    // main loop: DW_DEPTH chunks per trip, no control flow inside a trip
    int base = ch0;
    for (; base + DW_DEPTH <= ch1; base += DW_DEPTH) {
#pragma unroll
      for (int d = 0; d < DW_DEPTH; ++d) {
        const int cur = d & 1;   // DW_DEPTH is even, so chunk parity == d parity
        // stage d was published one step ago; refill it DW_DEPTH chunks ahead
        fetch_next(st[d]);
        compute(cur);
        dw_publish(lds_a[cur ^ 1], lds_b[cur ^ 1], lds_c[cur ^ 1], tid, st[(d + 1) % DW_DEPTH]);
        __syncthreads();
      }
    }
    // tail (< DW_DEPTH chunks): stages 0.. hold chunks base.., LDS buffer 0 holds chunk `base`
#pragma unroll
    for (int d = 0; d < DW_DEPTH - 1; ++d) {
      if (base + d >= ch1) break;
      compute(d & 1);
      dw_publish(lds_a[(d & 1) ^ 1], lds_b[(d & 1) ^ 1], lds_c[(d & 1) ^ 1], tid, st[d + 1]);
      __syncthreads();
    }
  }

#pragma unroll
  for (int a = 0; a < NMAT; ++a) {
    const int mm = 3 * mg + a;
#pragma unroll
    for (int ii = 0; ii < DW_WI; ++ii)
#pragma unroll
      for (int u = 0; u < DW_WJ; ++u) {
        const int it = it0 + DW_WI * wi + ii, jt = jt0 + DW_WJ * wj + u;
        p.partial[((((size_t)z * (p.k + 1) + mm) * NT + it) * NT + jt) * 64 + lane] = acc[a][ii][u];
      }
  }
}

bool ring_dw_tiled_applicable(int NC) { return NC == 4 || NC == 8; }

// K splits for the tiled kernel: about two workgroups per CU, a multiple of 8 when possible.
int ring_dw_tiled_nz(int NC, int k, long nchunk) {
  const int NT = 4 * NC;
  (void)k;   // one launch per matrix group: the grid of a launch does not depend on a_dim
  const long tiles = (long)(NT / DW_TI) * (NT / DW_TJ);
  long nz = (256 + tiles - 1) / tiles;   // one workgroup per CU
  if (nz >= 8) nz = (nz + 7) / 8 * 8;
  if (nz > 128) nz = 128;
  if (nz > nchunk) nz = nchunk;
  if (nz < 1) nz = 1;
  return (int)nz;
}

template <int NC>
static hipError_t launch_group(const RingDwArgs& a, int mg, unsigned blocks, hipStream_t st) {
  const int nmat = (a.k + 1 - 3 * mg) < 3 ? (a.k + 1 - 3 * mg) : 3;
  if (mg == 0) {
    if (nmat == 3) hipLaunchKernelGGL((ring_dw_tiled_kernel<NC, 3, true>), dim3(blocks), dim3(DW_THREADS), 0, st, a, mg);
    else if (nmat == 2) hipLaunchKernelGGL((ring_dw_tiled_kernel<NC, 2, true>), dim3(blocks), dim3(DW_THREADS), 0, st, a, mg);
    else hipLaunchKernelGGL((ring_dw_tiled_kernel<NC, 1, true>), dim3(blocks), dim3(DW_THREADS), 0, st, a, mg);
  } else {
    if (nmat == 3) hipLaunchKernelGGL((ring_dw_tiled_kernel<NC, 3, false>), dim3(blocks), dim3(DW_THREADS), 0, st, a, mg);
    else if (nmat == 2) hipLaunchKernelGGL((ring_dw_tiled_kernel<NC, 2, false>), dim3(blocks), dim3(DW_THREADS), 0, st, a, mg);
    else hipLaunchKernelGGL((ring_dw_tiled_kernel<NC, 1, false>), dim3(blocks), dim3(DW_THREADS), 0, st, a, mg);
  }
  return hipGetLastError();
}

// One launch per group of three matrices (a_dim = 2 needs exactly one).
hipError_t ring_launch_dw_tiled(const RingDwArgs& a, int NC, hipStream_t st) {
  const int NT = 4 * NC;
  const unsigned blocks = (unsigned)((NT / DW_TI) * (NT / DW_TJ) * a.nz);
  const int nmg = (a.k + 3) / 3;
  for (int mg = 0; mg < nmg; ++mg) {
    hipError_t e = NC == 4 ? launch_group<4>(a, mg, blocks, st) : (NC == 8 ? launch_group<8>(a, mg, blocks, st) : hipErrorInvalidValue);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}
