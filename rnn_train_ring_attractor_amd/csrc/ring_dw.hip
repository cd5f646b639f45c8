// Weight-gradient contraction, LDS-tiled variant for NPAD >= 256 (NC = 4 or 8).
//
//   dW_mm[i][j] = sum over samples (b,t) of coef_mm(b,t) * g[t,b,i] * r_prev[t,b,j]
//
// Work decomposition: a workgroup (4 waves) owns a 64 (i) x 128 (j) output tile of up to three
// matrices over one K split; wave v owns row tile v of the block (16 neurons) against all eight
// column tiles.  A K chunk is 16 batch rows x 2 time steps (32 samples, one MFMA K).  The bf16
// operands stream from the tile-ordered side buffers through a double-buffered LDS stage laid out
// fragment-major, so every MFMA operand is one conflict-free ds_read_b128; the action gates of the
// chunk are staged next to them.  Two workgroups fit a CU (2 waves per SIMD) and hide each other's
// load latency.  Partials are written once per workgroup; a fixed-order reduction follows.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

namespace {

constexpr int DW_TI = 4;   // row tiles per workgroup (64 neurons)
constexpr int DW_TJ = 8;   // column tiles per workgroup (128 neurons)

struct DwStage {           // one K chunk in flight in registers (global -> regs -> LDS)
  f32x2 a[2];              // 2 x 8 bytes of g
  f32x2 b[4];              // 4 x 8 bytes of r_prev
  float cf;                // one gate value (threads 0..95)
};

// Unit x of an operand block: tau = time step within the chunk, then (record group, lane, c).
template <int NC, int TT>
__device__ __forceinline__ void unit_decode(int x, int it0, int& tau, int& tl, int& lane, int& w, int& c) {
  constexpr int CB = NC < TT ? NC : TT;         // consecutive column tiles held in one lane record
  tau = x / (TT * 64);
  const int y = x % (TT * 64);
  const int cl = y % CB;
  lane = (y / CB) % 64;
  const int wl = y / (CB * 64);
  tl = wl * CB + cl;
  const int it = it0 + tl;
  w = it / NC;
  c = it % NC;
}

template <int NC>
__device__ __forceinline__ void dw_fetch(const RingDwArgs& p, long ch, int it0, int jt0, int mg, int tid, DwStage& s) {
  const int nbt = p.nbt, T = p.T;
  const int bt = (int)(ch % nbt);
  const int t0 = 2 * (int)(ch / nbt);
  const f32x2 zero = {0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    int tau, tl, lane, w, c;
    unit_decode<NC, DW_TI>(tid + 256 * u, it0, tau, tl, lane, w, c);
    const int t = t0 + tau;
    s.a[u] = (t < T) ? *reinterpret_cast<const f32x2*>(p.gfrag + side_offset<NC>(t, nbt, bt, w, lane) + 4 * c) : zero;
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int tau, tl, lane, w, c;
    unit_decode<NC, DW_TJ>(tid + 256 * u, jt0, tau, tl, lane, w, c);
    const int t = t0 + tau;
    s.b[u] = (t < T) ? *reinterpret_cast<const f32x2*>(p.rfrag + side_offset<NC>(t, nbt, bt, w, lane) + 4 * c) : zero;
  }
  // gates: thread = (a, tau, row) for a < 3, tau < 2, row < 16
  s.cf = 0.f;
  if (tid < 96) {
    const int a = tid / 32, tau = (tid / 16) & 1, row = tid & 15;
    const int mm = 3 * mg + a, b = 16 * bt + row, t = t0 + tau;
    if (mm >= 1 && mm <= p.k && b < p.B && t < T) s.cf = p.A[((size_t)b * T + t) * p.k + (mm - 1)];
  }
}

template <int NC>
__device__ __forceinline__ void dw_publish(f32x2* la, f32x2* lb, float* lc, int tid, const DwStage& s) {
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    int tau, tl, lane, w, c;
    unit_decode<NC, DW_TI>(tid + 256 * u, 0, tau, tl, lane, w, c);
    la[(tl * 64 + lane) * 2 + tau] = s.a[u];
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int tau, tl, lane, w, c;
    unit_decode<NC, DW_TJ>(tid + 256 * u, 0, tau, tl, lane, w, c);
    lb[(tl * 64 + lane) * 2 + tau] = s.b[u];
  }
  if (tid < 96) lc[tid] = s.cf;
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

template <int NC>
__global__ __launch_bounds__(256, 2) void ring_dw_tiled_kernel(RingDwArgs p) {
  constexpr int NT = 4 * NC;
  constexpr int NIB = NT / DW_TI, NJB = NT / DW_TJ;
  __shared__ __attribute__((aligned(16))) f32x2 lds_a[2][DW_TI * 64 * 2];
  __shared__ __attribute__((aligned(16))) f32x2 lds_b[2][DW_TJ * 64 * 2];
  __shared__ __attribute__((aligned(16))) float lds_c[2][96];

  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, q = lane >> 4;
  const int nmg = (p.k + 3) / 3;
  const int tiles = NIB * NJB * nmg;
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
  const int ib = tile % NIB, jb = (tile / NIB) % NJB, mg = tile / (NIB * NJB);
  const int it0 = ib * DW_TI, jt0 = jb * DW_TJ;

  const long nchunk = (long)p.nbt * ((p.T + 1) / 2);
  const long ch0 = nchunk * z / p.nz, ch1 = nchunk * (z + 1) / p.nz;

  f32x4 acc[3][DW_TJ];
#pragma unroll
  for (int a = 0; a < 3; ++a)
#pragma unroll
    for (int u = 0; u < DW_TJ; ++u) acc[a][u] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int nmat = (p.k + 1 - 3 * mg) < 3 ? (p.k + 1 - 3 * mg) : 3;   // matrices of this group

  DwStage st;
  if (ch0 < ch1) {
    dw_fetch<NC>(p, ch0, it0, jt0, mg, tid, st);
    dw_publish<NC>(lds_a[0], lds_b[0], lds_c[0], tid, st);
  }
  __syncthreads();

  for (long ch = ch0; ch < ch1; ++ch) {
    const int cur = (int)((ch - ch0) & 1);
    const bool more = ch + 1 < ch1;
    if (more) dw_fetch<NC>(p, ch + 1, it0, jt0, mg, tid, st);

    const bf16x8 ga = *reinterpret_cast<const bf16x8*>(&lds_a[cur][(wv * 64 + lane) * 2]);
    bf16x8 rb[DW_TJ];
#pragma unroll
    for (int u = 0; u < DW_TJ; ++u) rb[u] = *reinterpret_cast<const bf16x8*>(&lds_b[cur][(u * 64 + lane) * 2]);
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      if (a >= nmat) break;
      bf16x8 gg = ga;
      if (3 * mg + a != 0) {
        const f32x4 c0 = *reinterpret_cast<const f32x4*>(&lds_c[cur][a * 32 + 4 * q]);
        const f32x4 c1 = *reinterpret_cast<const f32x4*>(&lds_c[cur][a * 32 + 16 + 4 * q]);
        gg = gate_frag(ga, c0, c1);
      }
#pragma unroll
      for (int u = 0; u < DW_TJ; ++u) acc[a][u] = mfma16(gg, rb[u], acc[a][u]);
    }
    if (more) dw_publish<NC>(lds_a[cur ^ 1], lds_b[cur ^ 1], lds_c[cur ^ 1], tid, st);
    __syncthreads();
  }

#pragma unroll
  for (int a = 0; a < 3; ++a) {
    if (a >= nmat) break;
    const int mm = 3 * mg + a;
#pragma unroll
    for (int u = 0; u < DW_TJ; ++u) {
      const int it = it0 + wv, jt = jt0 + u;
      p.partial[((((size_t)z * (p.k + 1) + mm) * NT + it) * NT + jt) * 64 + lane] = acc[a][u];
    }
  }
}

bool ring_dw_tiled_applicable(int NC) { return NC == 4 || NC == 8; }

// K splits for the tiled kernel: about two workgroups per CU, a multiple of 8 when possible.
int ring_dw_tiled_nz(int NC, int k, long nchunk) {
  const int NT = 4 * NC;
  const long tiles = (long)(NT / DW_TI) * (NT / DW_TJ) * ((k + 3) / 3);
  long nz = (512 + tiles - 1) / tiles;
  if (nz >= 8) nz = (nz + 7) / 8 * 8;
  if (nz > 128) nz = 128;
  if (nz > nchunk) nz = nchunk;
  if (nz < 1) nz = 1;
  return (int)nz;
}

hipError_t ring_launch_dw_tiled(const RingDwArgs& a, int NC, hipStream_t st) {
  const int NT = 4 * NC;
  const long tiles = (long)(NT / DW_TI) * (NT / DW_TJ) * ((a.k + 3) / 3);
  const unsigned blocks = (unsigned)(tiles * a.nz);
  if (NC == 4)
    hipLaunchKernelGGL(ring_dw_tiled_kernel<4>, dim3(blocks), dim3(256), 0, st, a);
  else if (NC == 8)
    hipLaunchKernelGGL(ring_dw_tiled_kernel<8>, dim3(blocks), dim3(256), 0, st, a);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
