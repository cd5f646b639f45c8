// Weight-gradient contraction, register-tiled variant for NPAD >= 256 (NC = 4 or 8).
//
//   dW_mm[i][j] = sum over samples (b,t) of coef_mm(b,t) * g[t,b,i] * r_prev[t,b,j]
//
// A workgroup (4 waves, one per SIMD) owns a 128 (i) x 128 (j) block of up to three matrices over one
// K split; wave v owns rows 32v..32v+31 against all 128 columns: 2 x 8 MFMA tiles x 3 matrices = 48
// accumulators (192 accumulation VGPRs).  A K chunk is 16 batch rows x 2 time steps (32 samples, one
// MFMA K).  The paired tile-major operand buffers hold every tile of a chunk as 1 KiB of ready-made
// MFMA fragments, so nothing is ever transposed or repacked:
//   * the wave's own two g fragments load straight into registers;
//   * the action gates of a chunk (16 rows x 2 steps x up to 3 matrices) are fetched one value per
//     thread and handed round through a small LDS stage next to the r_prev one: per-lane gate loads
//     (eight scattered 4-byte loads per wave and chunk) cost more than the whole gating arithmetic;
//   * the eight r_prev fragments every wave needs are copied verbatim into an LDS stage of DW_LDS
//     buffers once per workgroup (8 KiB per chunk) and read back with conflict-free ds_read_b128, one
//     chunk ahead of the MFMAs that use them -- L2 -> CU traffic stays at 16 KiB per chunk and the LDS
//     pipe at 40 KiB, both under the MFMA time.
// DW_DEPTH chunks are in flight in registers; a trip of the main loop is one basic block containing
// loads only, so the compiler waits for exactly the oldest chunk (s_waitcnt vmcnt(n), n > 0).
// Partials are written once per wave; a fixed-order reduction follows.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

#include <stdlib.h>

namespace {

constexpr int DW_WI = 2;      // MFMA row tiles per wave (32 neurons of g)
constexpr int DW_WJ = 8;      // MFMA column tiles per wave (128 neurons of r_prev)
constexpr int DW_DEPTH = 4;   // K chunks in flight per wave
constexpr int DW_LDS = 4;     // LDS stage buffers (chunk c lives in buffer c % DW_LDS)

template <int NG>
struct DwStage {
  bf16x8 a[DW_WI];                    // g fragments of the wave's row tiles
  f32x4 bpart[2];                     // this thread's two fragments of the chunk's r_prev block (LDS stage)
  float gate;                         // one action gate of the chunk: matrix tid/32 % 4, row (tid/2) % 16, step tid % 2
};

// NMAT matrices in this launch's group, the first of them ungated (Wo) when FIRST.
// ga points at this lane's fragment of the wave's first row tile, rb at fragment `tid` of the block's
// eight column tiles (512 fragments, two per thread); chunks are laid out back to back (pair-major,
// batch tile fastest), 4*NC KiB apart.
template <int NC, int NMAT, bool FIRST>
__device__ __forceinline__ void dw_fetch(const RingDwArgs& p, const bf16x8* ga, const f32x4* rb, int bt, int t0, int mg,
                                         int tid, DwStage<NMAT - (FIRST ? 1 : 0)>& s) {
  const int T = p.T, k = p.k;
#pragma unroll
  for (int u = 0; u < DW_WI; ++u) s.a[u] = ga[u * 64];
  s.bpart[0] = rb[0];
  s.bpart[1] = rb[256];
  // gate of (gated matrix ga, sample row, step t0 + tt) for thread tid = 32*ga + 2*row + tt (mod 128).
  // The address is clamped into the tensor and the value used as loaded: rows past B and the missing
  // second step of an odd-length sequence meet zero g fragments.
  {
    const int gi = tid & 127, gm = gi >> 5, row = (gi >> 1) & 15, tt = gi & 1;
    constexpr int NG = NMAT - (FIRST ? 1 : 0);
    const int ch = 3 * mg + (gm < NG ? gm : 0) - (FIRST ? 0 : 1);   // matrix 3*mg + a gates with channel 3*mg + a - 1
    const int b = 16 * bt + row, bc = b < p.B ? b : p.B - 1;
    const int tg = t0 + tt < T ? t0 + tt : t0;
    s.gate = p.A[((size_t)bc * T + tg) * k + ch];
  }
}

// g8 = gates of rows 4q..4q+3 as (t0, t0+1) pairs: K slot e of the fragment is row e at t0, slot 4+e row e at t0+1
__device__ __forceinline__ bf16x8 gate_frag(bf16x8 x, const f32x4 (&g8)[2]) {
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o[e] = (__bf16)((float)x[e] * g8[e >> 1][2 * (e & 1)]);
    o[4 + e] = (__bf16)((float)x[4 + e] * g8[e >> 1][2 * (e & 1) + 1]);
  }
  return o;
}

}  // namespace

// seg_begin / seg_end: the launch covers K chunks [seg_begin, seg_end) of the sequence (chunk = time-step pair *
// batch tiles + batch tile, so a range of chunks is a range of time steps); add != 0: the wave adds its result
// to the partial sums an earlier launch left.
template <int NC, int NMAT, bool FIRST>
__global__ __launch_bounds__(256) void ring_dw_direct_kernel(RingDwArgs p, int mg, int seg_begin, int seg_end, int add) {
  constexpr int NT = 4 * NC;
  constexpr int NB = NT / 8;             // 128-neuron blocks per side
  constexpr int NG = NMAT - (FIRST ? 1 : 0);
  __shared__ __attribute__((aligned(16))) f32x4 lds_b[DW_LDS][DW_WJ * 64];
  __shared__ __attribute__((aligned(16))) float lds_g[DW_LDS][4][16][2];   // [buffer][gated matrix][row][step]
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
  const int tiles = NB * NB;
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
  const int it0 = (tile % NB) * 8 + wv * DW_WI;
  const int jt0 = (tile / NB) * 8;

  const int nchunk = seg_end - seg_begin;       // (the host checked that the sequence's chunk count fits an int)
  const int ch0 = seg_begin + (int)((long)nchunk * z / p.nz), ch1 = seg_begin + (int)((long)nchunk * (z + 1) / p.nz);

  f32x4 acc[NMAT][DW_WI][DW_WJ];
#pragma unroll
  for (int a = 0; a < NMAT; ++a)
#pragma unroll
    for (int ii = 0; ii < DW_WI; ++ii)
#pragma unroll
      for (int u = 0; u < DW_WJ; ++u) {
        acc[a][ii][u] = f32x4{0.f, 0.f, 0.f, 0.f};
        // accumulate in the accumulation-VGPR half of the register file; the architectural half
        // then holds nothing but the operand stages in flight
        asm volatile("" : "+a"(acc[a][ii][u]));
      }

  // Fetch cursor: chunk = (batch tile fb, time-step pair ft), batch tile fastest.  It advances with
  // scalar selects (no branch, no division) and parks on the last chunk of the split, so fetches
  // past the end re-read valid data that is never consumed.
  int fc = ch0, fb = ch0 % p.nbt, ft = ch0 / p.nbt;
  constexpr size_t CHUNK_FRAGS = (size_t)NT * 64;   // 16-byte fragments per chunk
  const bf16x8* ga = reinterpret_cast<const bf16x8*>(p.gfrag) + (size_t)ch0 * CHUNK_FRAGS + (size_t)it0 * 64 + lane;
  const f32x4* rb = reinterpret_cast<const f32x4*>(p.rfrag) + (size_t)ch0 * CHUNK_FRAGS + (size_t)jt0 * 64 + tid;
  auto fetch_next = [&](DwStage<NG>& s) {
    dw_fetch<NC, NMAT, FIRST>(p, ga, rb, fb, 2 * ft, mg, tid, s);
    const int adv = (fc + 1 < ch1) ? 1 : 0;
    ga += adv * CHUNK_FRAGS;
    rb += adv * CHUNK_FRAGS;
    fc += adv;
    fb += adv;
    const int wrap = (fb == p.nbt) ? 1 : 0;
    fb = wrap ? 0 : fb;
    ft += wrap;
  };
  // The LDS stage has DW_LDS buffers and is read one chunk ahead of the MFMAs that use it: the reads of
  // chunk i+1 are issued before the MFMAs of chunk i and land while those run.  A chunk is therefore
  // published two chunks before it is used, with a barrier between the publication and the read.
  struct DwOperands {
    bf16x8 b[DW_WJ];
    f32x4 g8[NG > 0 ? NG : 1][2];
  };
  auto lds_read = [&](DwOperands& o, int buf) {
#pragma unroll
    for (int u = 0; u < DW_WJ; ++u) o.b[u] = *reinterpret_cast<const bf16x8*>(&lds_b[buf][u * 64 + lane]);
#pragma unroll
    for (int a = 0; a < NG; ++a) {
      const f32x4* gp = reinterpret_cast<const f32x4*>(&lds_g[buf][a][4 * (lane >> 4)][0]);
      o.g8[a][0] = gp[0];
      o.g8[a][1] = gp[1];
    }
  };
  auto compute = [&](const DwStage<NG>& s, const DwOperands& o) {
#pragma unroll
    for (int a = 0; a < NMAT; ++a) {
#pragma unroll
      for (int ii = 0; ii < DW_WI; ++ii) {
        const bf16x8 gg = (FIRST && a == 0) ? s.a[ii] : gate_frag(s.a[ii], o.g8[a - (FIRST ? 1 : 0)]);
#pragma unroll
        for (int u = 0; u < DW_WJ; ++u) acc[a][ii][u] = mfma16(gg, o.b[u], acc[a][ii][u]);
      }
    }
  };
  auto publish = [&](const DwStage<NG>& s, int buf) {
    lds_b[buf][tid] = s.bpart[0];
    lds_b[buf][tid + 256] = s.bpart[1];
    if (tid < 128) (&lds_g[buf][0][0][0])[tid] = s.gate;
  };

  if (ch0 < ch1) {
    static_assert(DW_DEPTH == DW_LDS, "stage d of the register pipeline and LDS buffer d hold the same chunk");
    DwStage<NG> st[DW_DEPTH];
    DwOperands op[2];
#pragma unroll
    for (int d = 0; d < DW_DEPTH; ++d) fetch_next(st[d]);
    publish(st[0], 0);
    publish(st[1], 1);
    lds_barrier();
    lds_read(op[0], 0);
    // Invariant at the top of step d (chunk base + d): op[d & 1] holds (or is about to receive) that chunk's
    // operands, buffer d + 1 holds the next chunk behind a barrier, stage d + 2 is the next to publish.
    int base = ch0;
    for (; base + DW_DEPTH <= ch1; base += DW_DEPTH) {
#pragma unroll
      for (int d = 0; d < DW_DEPTH; ++d) {
        lds_read(op[(d + 1) & 1], (d + 1) % DW_LDS);
        __builtin_amdgcn_sched_barrier(0);          // issue the reads first: left alone they sink below the MFMAs
        compute(st[d], op[d & 1]);
        fetch_next(st[d]);                          // refill DW_DEPTH chunks ahead
        publish(st[(d + 2) % DW_DEPTH], (d + 2) % DW_LDS);
        lds_barrier();
        // keep the refill of stage d where it is: the scheduler would otherwise sink all refills of
        // a trip to its end and drain the whole queue once per trip
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // tail (< DW_DEPTH chunks): stage d holds chunk base + d (past the split's end: copies of its last chunk)
#pragma unroll
    for (int d = 0; d < DW_DEPTH - 1; ++d) {
      if (base + d >= ch1) break;
      lds_read(op[(d + 1) & 1], (d + 1) % DW_LDS);
      compute(st[d], op[d & 1]);
      publish(st[(d + 2) % DW_DEPTH], (d + 2) % DW_LDS);
      lds_barrier();
    }
  }

#pragma unroll
  for (int a = 0; a < NMAT; ++a) {
    const int mm = 3 * mg + a;
#pragma unroll
    for (int ii = 0; ii < DW_WI; ++ii)
#pragma unroll
      for (int u = 0; u < DW_WJ; ++u) {
        ring_f32x4* dst = p.partial + ((((size_t)z * (p.k + 1) + mm) * NT + it0 + ii) * NT + jt0 + u) * 64 + lane;
        *dst = add ? *dst + acc[a][ii][u] : acc[a][ii][u];
      }
  }
}

bool ring_dw_tiled_applicable(int NC) { return NC == 4 || NC == 8 || NC == 16 || NC == 24 || NC == 32; }

// K splits: one workgroup per CU, a multiple of 8 when possible (XCD grouping).  One launch per
// group of three matrices, so the grid of a launch does not depend on a_dim.
int ring_dw_tiled_nz(int NC, int k, long nchunk) {
  (void)k;
  const int NB = 4 * NC / 8;
  const long tiles = (long)NB * NB;
  long nz = (256 + tiles - 1) / tiles;
  if (nz >= 8) nz = (nz + 7) / 8 * 8;
  if (nz > 128) nz = 128;
  if (nz > nchunk) nz = nchunk;
  if (nz < 1) nz = 1;
  return (int)nz;
}

template <int NC>
static hipError_t launch_group(const RingDwArgs& a, int mg, unsigned blocks, int seg_begin, int seg_end, int add,
                               hipStream_t st) {
  const int nmat = (a.k + 1 - 3 * mg) < 3 ? (a.k + 1 - 3 * mg) : 3;
  if (mg == 0) {
    if (nmat == 3) RING_LAUNCH((ring_dw_direct_kernel<NC, 3, true>), dim3(blocks), dim3(256), 0, st, a, mg, seg_begin, seg_end, add);
    else if (nmat == 2) RING_LAUNCH((ring_dw_direct_kernel<NC, 2, true>), dim3(blocks), dim3(256), 0, st, a, mg, seg_begin, seg_end, add);
    else RING_LAUNCH((ring_dw_direct_kernel<NC, 1, true>), dim3(blocks), dim3(256), 0, st, a, mg, seg_begin, seg_end, add);
  } else {
    if (nmat == 3) RING_LAUNCH((ring_dw_direct_kernel<NC, 3, false>), dim3(blocks), dim3(256), 0, st, a, mg, seg_begin, seg_end, add);
    else if (nmat == 2) RING_LAUNCH((ring_dw_direct_kernel<NC, 2, false>), dim3(blocks), dim3(256), 0, st, a, mg, seg_begin, seg_end, add);
    else RING_LAUNCH((ring_dw_direct_kernel<NC, 1, false>), dim3(blocks), dim3(256), 0, st, a, mg, seg_begin, seg_end, add);
  }
  return hipGetLastError();
}

// K chunks a workgroup walks per launch, at most.  The workgroups of a K split read the same two operand streams
// and find each other's fragments in their XCD's L2 only while they stay within about 32 chunks of one another
// (4 MiB of L2 against 128 KiB of new operand bytes per chunk step and XCD).  Nothing synchronises them, so over a
// long walk they drift apart and every one fetches its operands from memory for itself: at N = 512, B = 8192 the
// kernel reads 1.02 x its operands over 512 chunks per workgroup, 1.45 x over 2048 and 2.47 x over 8192.  A long
// sequence is therefore cut into segments in time, one launch each (a launch boundary re-aligns the workgroups);
// the launches after the first add to the partial sums.  RINGATTR_DW_SEGMENT overrides the length (0: no cut).
static int dw_segment_chunks() {
  const char* e = getenv("RINGATTR_DW_SEGMENT");   // read at every call: tests switch it between calls
  return e ? atoi(e) : 640;
}

// Time-step pairs per segment (whole pairs, so that a segment is a contiguous range of chunks).
static long dw_pairs_per_segment(int nbt, int T, int nz) {
  const int npairs = (T + 1) / 2;
  const long nchunk = (long)nbt * npairs;
  const int seg = dw_segment_chunks();
  long pairs_per_seg = npairs;
  if (seg > 0 && nz > 0 && nchunk / nz > seg) {
    pairs_per_seg = ((long)seg * nz) / nbt;
    if (pairs_per_seg < 1) pairs_per_seg = 1;
  }
  return pairs_per_seg;
}

int ring_dw_tiled_segments(int nbt, int T, int nz) {
  const long per = dw_pairs_per_segment(nbt, T, nz);
  return (int)(((T + 1) / 2 + per - 1) / per);
}

// One launch per group of three matrices (a_dim = 2 needs exactly one) and segment.
hipError_t ring_launch_dw_tiled(const RingDwArgs& a, int NC, hipStream_t st) {
  const int NB = 4 * NC / 8;
  const unsigned blocks = (unsigned)(NB * NB * a.nz);
  const int nmg = (a.k + 3) / 3;
  const int npairs = (a.T + 1) / 2;
  const long pairs_per_seg = dw_pairs_per_segment(a.nbt, a.T, a.nz);
  for (int mg = 0; mg < nmg; ++mg) {
    for (long p0 = 0; p0 < npairs; p0 += pairs_per_seg) {
      const long p1 = p0 + pairs_per_seg < npairs ? p0 + pairs_per_seg : npairs;
      const int b = (int)(p0 * a.nbt), e_ = (int)(p1 * a.nbt), add = p0 > 0 ? 1 : 0;
      hipError_t e = hipErrorInvalidValue;
      switch (NC) {
        case 4: e = launch_group<4>(a, mg, blocks, b, e_, add, st); break;
        case 8: e = launch_group<8>(a, mg, blocks, b, e_, add, st); break;
        case 16: e = launch_group<16>(a, mg, blocks, b, e_, add, st); break;
        case 24: e = launch_group<24>(a, mg, blocks, b, e_, add, st); break;
        case 32: e = launch_group<32>(a, mg, blocks, b, e_, add, st); break;
        default: break;
      }
      if (e != hipSuccess) return e;
    }
  }
  return hipSuccess;
}
