// Weight-resident forward (and, further down, BPTT) for N = 512 (NC = 8), a_dim = 2: the weights stay on chip, spread
// over a cluster of four compute units.
//
// [Wo|Wl|Wr] in bf16 is 1.5 MiB at N = 512, four times what one compute unit can hold (the streaming kernels
// therefore pull all of it from L2 once per step and batch-tile pair, and a step is bound by that stream).  Here
// four workgroups on four compute units of ONE XCD (one L2) form a cluster: member m keeps the slices for output
// neurons 128 m .. 128 m + 127 for the whole sequence -- the two gated matrices in accumulation VGPRs, Wo in LDS,
// the split of the N <= 256 weight-resident kernels -- and computes those neurons for all the cluster's batch rows.
// What the members exchange per step is the new state in bf16, in the layout the next step's MFMA A operand is
// read in:
//   xchg[t & 1][batch tile][K chunk kc][q][row] x 16 bytes  =  r_t[row][32 kc + 8 q .. + 7],
// written with ordinary stores (they reach the XCD's L2; vmcnt tells when) and read with device-scope loads (which
// miss the vector L1).  A flag per (batch-tile pair, member, wave) carries the number of the last state written; a
// reader looks at the 32 flags of a pair before it loads the pair's operand.  The buffer has two halves by step
// parity: nobody can write state t+1 of a pair before every member has published state t of it, i.e. has finished
// reading state t-1, which is what lives in the half being overwritten.
//
// Workgroups are dispatched to XCDs round robin by workgroup index; the four members of a cluster are taken 8 apart
// and check at start (by the hardware's XCC_ID) that they did land on one XCD, since the L2 caches of different XCDs
// are not coherent inside a kernel.  That handshake also proves that all four are resident, after which a member can
// only wait for a sibling that is running.  Every wait is bounded all the same: on a time-out the member sets the
// workgroup's abort word and a word in host memory and all its waves leave at the next common point; the siblings
// then run into their own time-outs.  The host finds the word set on its next call into the library.
//
// A cluster works on its batch-tile pairs (32 rows) round robin inside a step -- pair-steps -- so that the state a
// pair-step needs was produced a whole round earlier and its flags are normally up when a wave looks; two batch tiles
// share every LDS fetch of a Wo fragment.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

#include <type_traits>

namespace {

constexpr int C_NC = 8;
constexpr int C_KCH = 16;
constexpr int C_TILE_UNITS = C_KCH * 4 * 16;      // 16-byte units of one batch tile's operand
constexpr int C_XSLOTS = 2 * C_TILE_UNITS;
constexpr size_t C_BIN_BYTES = 128 * 1024;        // where stores go that have nothing to store (see the kernel)

__device__ __forceinline__ int flag_load(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void flag_store(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

}  // namespace

namespace {

// lane j's a[i] <-> lane i's a[j] among the four lanes of a quad (j = lane & 3)
__device__ __forceinline__ void quad_transpose(unsigned (&a)[4], int j) {
  auto xchg_dpp = [](unsigned x, auto ctrl) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, decltype(ctrl)::value, 0xF, 0xF, false);
  };
  const bool odd = j & 1, hi = j & 2;
  {
    const unsigned s0 = odd ? a[0] : a[1], s1 = odd ? a[2] : a[3];
    const unsigned r0 = xchg_dpp(s0, std::integral_constant<int, 0xB1>{}), r1 = xchg_dpp(s1, std::integral_constant<int, 0xB1>{});
    a[0] = odd ? r0 : a[0];
    a[1] = odd ? a[1] : r0;
    a[2] = odd ? r1 : a[2];
    a[3] = odd ? a[3] : r1;
  }
  {
    const unsigned s0 = hi ? a[0] : a[2], s1 = hi ? a[1] : a[3];
    const unsigned r0 = xchg_dpp(s0, std::integral_constant<int, 0x4E>{}), r1 = xchg_dpp(s1, std::integral_constant<int, 0x4E>{});
    a[0] = hi ? r0 : a[0];
    a[2] = hi ? a[2] : r0;
    a[1] = hi ? r1 : a[1];
    a[3] = hi ? a[3] : r1;
  }
}

// scalar base + 32-bit lane offset + immediate
// (A store of more than 8 bytes per lane reads its data registers over the cycles after it issues; a vector-ALU write
// to one of them in the next two wait states changes what is stored.  The compiler keeps that distance for the stores
// it knows, not for one inside an asm statement, hence the s_nop.)
template <int IMM>
__device__ __forceinline__ void sstore16(const void* sbase, unsigned voff, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, %2 offset:%3\n\ts_nop 1" ::"v"(voff), "v"(v), "s"(sbase), "n"(IMM) : "memory");
}
template <int IMM>
__device__ __forceinline__ void sstore8(const void* sbase, unsigned voff, f32x2 v) {
  asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3" ::"v"(voff), "v"(v), "s"(sbase), "n"(IMM) : "memory");
}
// (A base the compiler cannot prove wave-uniform would be handed over in vector registers, which the instruction does
// not take: the two halves go through readfirstlane, which costs nothing where the value is scalar already.)
__device__ __forceinline__ const void* uniform_ptr(const void* ptr) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(ptr);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
  return reinterpret_cast<const void*>(((unsigned long long)hi << 32) | lo);
}
__device__ __forceinline__ void sstore4_dev(const void* sbase, unsigned voff, int v) {
  asm volatile("global_store_dword %0, %1, %2 sc1" ::"v"(voff), "v"(v), "s"(uniform_ptr(sbase)) : "memory");
}
template <int IMM>
__device__ __forceinline__ f32x4 sload16(const void* sbase, unsigned voff) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=&v"(v) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
  return v;
}
template <int IMM>
__device__ __forceinline__ f32x4 sload16_dev(const void* sbase, unsigned voff) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 sc1" : "=&v"(v) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
  return v;
}
template <int IMM>
__device__ __forceinline__ f32x2 sload8(const void* sbase, unsigned voff) {
  f32x2 v;
  asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=&v"(v) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
  return v;
}
__device__ __forceinline__ int sload4_dev(const void* sbase, unsigned voff) {
  int v;
  asm volatile("global_load_dword %0, %1, %2 sc1" : "=&v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}
__device__ __forceinline__ float sload4(const void* sbase, unsigned voff) {
  float v;
  asm volatile("global_load_dword %0, %1, %2" : "=&v"(v) : "v"(voff), "s"(sbase) : "memory");
  return v;
}

template <int K>
__device__ __forceinline__ void vm_wait_plain() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K) : "memory");
}

}  // namespace

// ------------------------------------------------------------------------------------------------
// The kernel: two waves per SIMD.
//
// A wave that issues a store stands still until the store's data has left the register file (some 150 cycles for
// 16 bytes per lane, with four waves going through the compute unit's one store path), and a wave in the vector-ALU
// epilogue feeds the matrix pipe nothing: with one wave per SIMD a pair-step is the SUM of its products, its
// epilogue and its stores.  Here the workgroup has eight waves.  Wave (v, h) owns ONE column tile, the 16 neurons
// 128 m + 16 (2 v + h) .. + 15 (its slices of the gated matrices fill its 128 accumulation registers), and the two
// halves h = 0 / 1 run half a pair-step apart:
//        half 0:   products(s)     epilogue(s)   | staging(s+1) |  products(s+1)   epilogue(s+1)
//        half 1:   epilogue(s-1)   products(s)   |              |  epilogue(s)     products(s+1)
// so each SIMD always has one wave on the matrix pipe and one in the epilogue or its stores.  The staged operand of
// pair-step s serves both halves and is replaced between two workgroup barriers.  (A cluster with a single pair has
// nothing to run ahead of: the next pair-step needs this one's state, and both halves run in phase.)
// ------------------------------------------------------------------------------------------------
namespace {
#ifndef C8_PRIO
#define C8_PRIO 2
#endif
constexpr int C8_WFR = C_KCH - 1;                 // Wo fragments of a wave kept in LDS
constexpr int C8_WSLOTS = 8 * C8_WFR * 64;
constexpr size_t C8_LDS_BYTES = (size_t)(C8_WSLOTS + C_XSLOTS) * 16 + 2 * 256 + 64;
}  // namespace

template <int ACT, bool SAVE>
__global__ __launch_bounds__(512) void ring_fwd_cluster8_kernel(RingFwdArgs p, RingClusterArgs c) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xs = wlds + C8_WSLOTS;
  float* gl = reinterpret_cast<float*>(xs + C_XSLOTS);   // [2][32 rows][2] action gates, by pair-step parity
  int* misc = reinterpret_cast<int*>(gl + 128);          // [0]: abort
  char* const xchg = reinterpret_cast<char*>(c.xchg);
  constexpr int NSTE = SAVE ? 6 : 4;                     // stores of every epilogue: 2 exchange, 2 history, 2 record (+ 2 at even steps)

  const int tid = threadIdx.x, w8 = tid >> 6, v = w8 & 3, h = w8 >> 2, lane = tid & 63, q = lane >> 4, n = lane & 15,
            g4 = n >> 2, j4 = n & 3;
  const int ct = 2 * v + h;
  const int blk = blockIdx.x, xcd = blk & 7, gi = blk >> 3, m = gi & 3, cl = (gi >> 2) * 8 + xcd;
  if (cl >= c.nclusters) return;
  const int B = p.B, T = p.T, nbt = p.nbt;
  constexpr int N = 512;
  const int my_ppc = (c.npairs - cl + c.nclusters - 1) / c.nclusters;
  const int w8u = __builtin_amdgcn_readfirstlane(w8);
  const bool skew = __builtin_amdgcn_readfirstlane(h) == 1 && my_ppc >= 2;   // this wave's epilogue runs a phase late

  if (tid == 0) misc[0] = 0;
  if (w8 == 0) {
    const int mine = (__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15) + 1;   // XCC_ID + 1
    if (lane == 0) flag_store(c.hello + cl * 4 + m, mine);
    int bad = c.spin_max < 0 ? 2 : 0;   // (a negative limit gives up at once: the host's way to exercise this exit)
    for (int spins = 0; !bad; ++spins) {
      const int hh = lane < 4 ? flag_load(c.hello + cl * 4 + lane) : mine;
      if (__ballot(hh == 0) == 0) {
        bad = __ballot(hh != mine) != 0 ? 1 : 0;
        break;
      }
      if (spins > c.spin_max) {
        bad = 2;
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    if (bad && lane == 0) {
      misc[0] = 1;
      *c.host_err = bad == 1 ? RING_CLUSTER_ERR_XCD : RING_CLUSTER_ERR_START;
    }
  }

  bf16x8 wreg[2][C_KCH];
  bf16x8 wo_last;
  bf16x8* wl = wlds + (size_t)(w8 * C8_WFR) * 64 + lane;
  {
    const bf16x8* Wp = reinterpret_cast<const bf16x8*>(p.Wpack);
#pragma unroll
    for (int kc = 0; kc < C_KCH; ++kc) {
      wreg[0][kc] = Wp[((size_t)((1 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
      wreg[1][kc] = Wp[((size_t)((2 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
    }
#pragma unroll
    for (int k8 = 0; k8 < C_KCH; k8 += 8) {
      bf16x8 f[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) f[x] = Wp[((size_t)((0 * 4 + m) * C_NC + ct) * C_KCH + k8 + x) * 64 + lane];
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        if (k8 + x < C8_WFR) wl[(k8 + x) * 64] = f[x];
        else wo_last = f[x];
      }
    }
#pragma unroll
    for (int kc = 0; kc < C_KCH; ++kc) {
      asm volatile("" : "+a"(wreg[0][kc]));
      asm volatile("" : "+a"(wreg[1][kc]));
    }
  }

  const float oma = 1.f - p.alpha;
  const ActScale asc = act_scale_make(p.alpha);
  const size_t xhalf_bytes = (size_t)2 * c.npairs * C_TILE_UNITS * 16;
  char* const bin = xchg + 2 * xhalf_bytes;
  // lane-constant byte offsets
  const unsigned row_lane = (unsigned)(((4 * q + j4) * N + 128 * m + 16 * ct + 4 * g4) * 4);   // fp32 [16 rows][N]: row 4q+j4, four neurons
  const unsigned xq_lane = (unsigned)(((((4 * m + (ct >> 1)) * 4 + 2 * (ct & 1) + (g4 >> 1)) * 16) + 4 * q + j4) * 16 + 8 * (g4 & 1));
  const int lane_c = (lane & 48) | (2 * ct + (n >> 3)), cp = n & 7;   // the neuron's place in the common tile order
  const unsigned d_lane = (unsigned)(lane_c * 64 + 8 * cp);
  const unsigned r_lane = (unsigned)((cp * 64 + lane_c) * 16);
  const unsigned x_lane = (unsigned)(lane * 16);
  const unsigned g_lane = (unsigned)(((lane >> 1) * T * 2 + (lane & 1)) * 4);
  const unsigned f_lane = (unsigned)((lane & 31) * 4);

  auto hist_base = [&](int t, int bt) { return reinterpret_cast<const char*>(p.hist) + ((size_t)t * B + 16 * bt) * N * 4; };
  auto flag_base = [&](int pl) { return reinterpret_cast<const char*>(c.flags) + ((size_t)cl * c.ppc + pl) * 32 * 4; };
  auto x_base = [&](int t, int pr) {
    return xchg + (size_t)(t & 1) * xhalf_bytes + ((size_t)(2 * pr) * C_TILE_UNITS + w8u * 256) * 16;
  };
  auto gate_base = [&](int t, int pr) { return reinterpret_cast<const char*>(p.A) + ((size_t)(32 * pr) * T + t) * 8; };
  auto stage_from_r_init = [&](int pr) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int u = w8 * 256 + jj * 64 + lane;
      const int tl = u >> 10, kc = (u >> 6) & 15, qq = (u >> 4) & 3, row = u & 15;
      const f32x4* src = reinterpret_cast<const f32x4*>(p.r_init + (size_t)(32 * pr + 16 * tl + row) * N + 32 * kc + 8 * qq);
      const f32x4 lo = src[0], hi = src[1];
      bf16x8 pk;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        pk[x] = (__bf16)lo[x];
        pk[4 + x] = (__bf16)hi[x];
      }
      xs[u] = pk;
    }
  };

  int pf_pl = -1, pf_val = 0;   // exchange stores issued, flag not yet up: pair (local) and state number
  f32x4 P[2][3];           // products of the pair-step in hand: [tile][matrix]
  f32x4 Lr[2];             // previous state of its rows (row 4q+j4, four neurons), per tile
  // the pair-step whose products are in P and whose epilogue is still to run (skewed half)
  int et = 0, epr = 0, epl = 0, eit = 0;
  bool epending = false;

  // Epilogue of pair-step (t, pr, pl), number `it` in this cluster's order, in two parts: the arithmetic on P and Lr
  // (its products and previous state) leaves everything in the form it is stored in; the stores follow.
  struct EpiOut {
    unsigned xe[2][2];
    f32x4 hv[2];
    f32x2 dk[2], rk[2], r0k[2];
  };
  auto epi_math = [&](int it, const f32x4 (&Lp)[2], EpiOut& o) {
    const float* gb = gl + (it & 1) * 64;
#pragma unroll
    for (int tl = 0; tl < 2; ++tl) {
      unsigned ro[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e0 = Lp[tl][i];
        ro[i] = __builtin_bit_cast(unsigned, e0);
      }
      quad_transpose(ro, j4);   // -> rows 4q+e of the lane's own neuron
      const f32x4 ga = *reinterpret_cast<const f32x4*>(gb + (16 * tl + 4 * q) * 2);
      const f32x4 gc = *reinterpret_cast<const f32x4*>(gb + (16 * tl + 4 * q + 2) * 2);
      float rn[4], dv[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float g0 = e < 2 ? ga[2 * e] : gc[2 * (e - 2)], g1 = e < 2 ? ga[2 * e + 1] : gc[2 * (e - 2) + 1];
        const float p0 = P[tl][0][e], p1 = P[tl][1][e], p2 = P[tl][2][e];
        const float x = fmaf(g1, p2, fmaf(g0, p1, p0));
        float aF, aD;
        act_scaled<ACT>(x, asc, aF, aD);
        rn[e] = fmaf(oma, __builtin_bit_cast(float, ro[e]), aF);
        dv[e] = aD;
      }
      if constexpr (SAVE) {
        const f16x4 d4 = {(_Float16)dv[0], (_Float16)dv[1], (_Float16)dv[2], (_Float16)dv[3]};
        o.dk[tl] = __builtin_bit_cast(f32x2, d4);
        const bf16x4 r4 = {(__bf16)rn[0], (__bf16)rn[1], (__bf16)rn[2], (__bf16)rn[3]};
        o.rk[tl] = __builtin_bit_cast(f32x2, r4);
        const bf16x4 o4 = {(__bf16)__builtin_bit_cast(float, ro[0]), (__bf16)__builtin_bit_cast(float, ro[1]),
                           (__bf16)__builtin_bit_cast(float, ro[2]), (__bf16)__builtin_bit_cast(float, ro[3])};
        o.r0k[tl] = __builtin_bit_cast(f32x2, o4);
      }
      unsigned hh[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) hh[e] = __builtin_bit_cast(unsigned, rn[e]);
      quad_transpose(hh, j4);   // -> row 4q+j4, neurons 4 g4 + i
      o.hv[tl] = f32x4{__builtin_bit_cast(float, hh[0]), __builtin_bit_cast(float, hh[1]), __builtin_bit_cast(float, hh[2]),
                     __builtin_bit_cast(float, hh[3])};
      const float h0 = o.hv[tl][0], h1 = o.hv[tl][1], h2 = o.hv[tl][2], h3 = o.hv[tl][3];
      const bf16x2 b01 = {(__bf16)h0, (__bf16)h1}, b23 = {(__bf16)h2, (__bf16)h3};
      o.xe[tl][0] = __builtin_bit_cast(unsigned, b01);
      o.xe[tl][1] = __builtin_bit_cast(unsigned, b23);
    }
  };
  auto epi_stores = [&](int t, int pr, int pl, const EpiOut& o) {
    const bool more = t + 1 < T;
    // the exchange first: its flag goes up as soon as the two stores have landed
    {
      const char* xb = xchg + (size_t)((t + 1) & 1) * xhalf_bytes + (size_t)(2 * pr) * C_TILE_UNITS * 16;
      const f32x2 x0 = {__builtin_bit_cast(float, o.xe[0][0]), __builtin_bit_cast(float, o.xe[0][1])};
      const f32x2 x1 = {__builtin_bit_cast(float, o.xe[1][0]), __builtin_bit_cast(float, o.xe[1][1])};
      sstore8<0>(more ? xb : bin, xq_lane, x0);
      sstore8<0>(more ? xb + C_TILE_UNITS * 16 : bin, xq_lane, x1);
    }
    sstore16<0>(hist_base(t, 2 * pr), row_lane, o.hv[0]);
    sstore16<0>(hist_base(t, 2 * pr + 1), row_lane, o.hv[1]);
    if constexpr (SAVE) {
      const char* db = reinterpret_cast<const char*>(p.dfrag) + ((((size_t)t * nbt + 2 * pr) * 4 + m) * 64) * 64;
      sstore8<0>(db, d_lane, o.dk[0]);
      sstore8<0>(db + 4 * 64 * 64, d_lane, o.dk[1]);
      // The operand copy keeps steps 2j and 2j+1 side by side in one 16-byte slot per lane.  An even step has both
      // halves at hand -- the state before it (slot t) and after it (slot t+1; past an odd length's end: the zero
      // tail) -- and stores the slot whole; an odd step stores nothing.  (Eight bytes at a time would be partial
      // 32-byte sectors, which cost a store five times what a whole one costs.)
      if ((t & 1) == 0) {
        const char* rb = reinterpret_cast<const char*>(p.rfrag) + (((size_t)(t >> 1) * nbt + 2 * pr) * 32 + 8 * m) * 64 * 16;
        const f32x2 z = {0.f, 0.f};
        const f32x2 n0 = more ? o.rk[0] : z, n1 = more ? o.rk[1] : z;
        sstore16<0>(rb, r_lane, f32x4{o.r0k[0][0], o.r0k[0][1], n0[0], n0[1]});
        sstore16<0>(rb + 32 * 64 * 16, r_lane, f32x4{o.r0k[1][0], o.r0k[1][1], n1[0], n1[1]});
      }
    }
    // the flag of these two exchange stores goes up behind this wave's next full wait (fetch_decide, or the slow
    // path of the staging): by then they have long landed, and nothing stands still for their acknowledgement
    pf_pl = more ? pl : -1;
    pf_val = t + 1;
  };

  // the first pair-step's operand and gates
  stage_from_r_init(cl);
  if (w8 == 0) gl[lane] = *reinterpret_cast<const float*>(gate_base(0, cl) + g_lane);
  lds_barrier();
  if (misc[0]) return;

  int t = 0, pl = 0, it = 0;
  for (;;) {
    const int pr = cl + c.nclusters * pl;
    int nt = t, npl = pl + 1;
    if (npl == my_ppc) {
      npl = 0;
      nt = t + 1;
    }
    const bool have_next = nt < T;
    const bool look = have_next && nt >= 1;
    const int npr = cl + c.nclusters * npl;

    f32x4 sreg[4];      // this wave's eighth of the next pair-step's operand
    int nflag;
    float gnext;
    bool up = false;
    auto fetch_issue = [&]() {
      gnext = sload4(have_next ? gate_base(nt, npr) : gate_base(t, pr), g_lane);
      nflag = sload4_dev(flag_base(look ? npl : pl), f_lane);
    };
    auto fetch_decide = [&]() {
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(nflag), "+v"(gnext)::"memory");
      up = look && __ballot(nflag < nt) == 0;
      sstore4_dev(pf_pl >= 0 ? flag_base(pf_pl) : bin, (unsigned)((8 * m + w8u) * 4), pf_val);   // (every lane the same word)
      pf_pl = -1;
    };
    auto fetch_x = [&](auto iv) {
      constexpr int i = decltype(iv)::value;
      const char* xb = look ? x_base(nt, npr) : x_base(t, pr);
      sreg[i] = sload16_dev<1024 * i>(xb, x_lane);
    };

    const bool thin = skew && !epending;   // no epilogue (and none of its stores) behind this pair-step's fetches
    if (skew) {
      // the late half: the previous pair-step's epilogue comes first, and the fetches for the next pair-step go out
      // around it (its products follow at once, and the operand must have landed when they end)
      EpiOut o = {};
      fetch_issue();
      if (epending) epi_math(eit, Lr, o);
      fetch_decide();
      fetch_x(std::integral_constant<int, 0>{});
      fetch_x(std::integral_constant<int, 1>{});
      fetch_x(std::integral_constant<int, 2>{});
      fetch_x(std::integral_constant<int, 3>{});
      if (epending) epi_stores(et, epr, epl, o);
    }

    // ---- products ----
    {
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int tl = 0; tl < 2; ++tl) P[tl][0] = P[tl][1] = P[tl][2] = z;
    }
    // previous state of this pair-step's rows
    const char* const pb = t == 0 ? reinterpret_cast<const char*>(p.r_init) + (size_t)(32 * pr) * N * 4 : hist_base(t - 1, 2 * pr);
    bf16x8 af[2][2], wf[2];
    auto frag_fetch = [&](auto kcv, int stg) {
      constexpr int kc = decltype(kcv)::value;
      af[stg][0] = xs[(0 * C_KCH + kc) * 64 + lane];
      af[stg][1] = xs[(1 * C_KCH + kc) * 64 + lane];
      if constexpr (kc < C8_WFR) wf[stg] = wl[kc * 64];
      else wf[stg] = wo_last;
    };
    auto body = [&](auto kcv, auto slotsv) {
      constexpr int kc = decltype(kcv)::value, stg = kc & 1;
      if constexpr (kc + 1 < C_KCH) frag_fetch(std::integral_constant<int, kc + 1>{}, stg ^ 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (decltype(slotsv)::value) {
        if constexpr (kc == 0) fetch_issue();
        if constexpr (kc == 12) fetch_decide();
        if constexpr (kc >= 12) fetch_x(std::integral_constant<int, kc - 12>{});
        __builtin_amdgcn_sched_barrier(0);
      }
      P[0][1] = mfma16(af[stg][0], wreg[0][kc], P[0][1]);
      P[1][1] = mfma16(af[stg][1], wreg[0][kc], P[1][1]);
      P[0][2] = mfma16(af[stg][0], wreg[1][kc], P[0][2]);
      P[1][2] = mfma16(af[stg][1], wreg[1][kc], P[1][2]);
      P[0][0] = mfma16(af[stg][0], wf[stg], P[0][0]);
      P[1][0] = mfma16(af[stg][1], wf[stg], P[1][0]);
      __builtin_amdgcn_sched_barrier(0);
    };
    auto products = [&](auto slotsv) {
      frag_fetch(std::integral_constant<int, 0>{}, 0);
      __builtin_amdgcn_s_setprio(C8_PRIO);
      body(std::integral_constant<int, 0>{}, slotsv);
      body(std::integral_constant<int, 1>{}, slotsv);
      body(std::integral_constant<int, 2>{}, slotsv);
      body(std::integral_constant<int, 3>{}, slotsv);
      body(std::integral_constant<int, 4>{}, slotsv);
      body(std::integral_constant<int, 5>{}, slotsv);
      body(std::integral_constant<int, 6>{}, slotsv);
      body(std::integral_constant<int, 7>{}, slotsv);
      body(std::integral_constant<int, 8>{}, slotsv);
      body(std::integral_constant<int, 9>{}, slotsv);
      body(std::integral_constant<int, 10>{}, slotsv);
      body(std::integral_constant<int, 11>{}, slotsv);
      body(std::integral_constant<int, 12>{}, slotsv);
      body(std::integral_constant<int, 13>{}, slotsv);
      body(std::integral_constant<int, 14>{}, slotsv);
      body(std::integral_constant<int, 15>{}, slotsv);
      __builtin_amdgcn_s_setprio(0);
    };
    if (skew) {
      // (ordinary loads: they are read in the next pair-step's first phase, and the compiler waits for them there)
      Lr[0] = *reinterpret_cast<const f32x4*>(pb + row_lane);
      Lr[1] = *reinterpret_cast<const f32x4*>(pb + 16 * N * 4 + row_lane);
      products(std::false_type{});
      et = t;
      epr = pr;
      epl = pl;
      eit = it;
      epending = true;
    } else {
      // the early half reads them right behind its products: seven operations younger (gates, flags, the flag
      // store, four operand loads) are still allowed to be out when it does
      f32x4 La[2];
      La[0] = sload16<0>(pb, row_lane);
      La[1] = sload16<0>(pb + 16 * N * 4, row_lane);
      products(std::true_type{});
      asm volatile("s_waitcnt vmcnt(7)" : "+v"(La[0]), "+v"(La[1])::"memory");
      EpiOut o;
      epi_math(it, La, o);
      epi_stores(t, pr, pl, o);
    }

    // ---- the next pair-step's operand and gates into LDS ----
    lds_barrier();   // every wave has finished with this pair-step's operand (and the late half with the gates before it)
    // the four operand loads are older than the epilogue's stores, which every wave has issued since; the late
    // half's first pair-step has no epilogue in front of it, and a plain vmcnt(0) covers that one time
    if (thin) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NSTE) : "memory");
    if (!have_next) break;
    if (nt == 0) {
      stage_from_r_init(npr);
    } else {
      if (up) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) xs[w8 * 256 + jj * 64 + lane] = __builtin_bit_cast(bf16x8, sreg[jj]);
      } else {
        // nothing valid was fetched ahead: put up the flag still held back (the producers of what is waited for may
        // be waiting for it in turn), wait for the flags, then ordinary loads behind a device-scope acquire
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (pf_pl >= 0) sstore4_dev(flag_base(pf_pl), (unsigned)((8 * m + w8u) * 4), pf_val);
        pf_pl = -1;
        bool ok = false;
        for (int spins = 0; spins <= c.spin_max; ++spins) {
          const int f = flag_load(c.flags + ((size_t)cl * c.ppc + npl) * 32 + (lane & 31));
          if ((ok = (__ballot(f < nt) == 0))) break;
          __builtin_amdgcn_s_sleep(2);
        }
        if (!ok && lane == 0) {
          misc[0] = 1;
          *c.host_err = RING_CLUSTER_ERR_WAIT;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const bf16x8* xb = reinterpret_cast<const bf16x8*>(x_base(nt, npr));
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) xs[w8 * 256 + jj * 64 + lane] = xb[jj * 64 + lane];
      }
    }
    if (w8 == 0) gl[((it + 1) & 1) * 64 + lane] = gnext;
    lds_barrier();
    if (misc[0]) return;
    t = nt;
    pl = npl;
    ++it;
  }
  if (skew && epending) {
    EpiOut o;
    epi_math(eit, Lr, o);
    epi_stores(et, epr, epl, o);
  }
}

// ------------------------------------------------------------------------------------------------
// BPTT on the same clusters.  Visit s = 0 .. T-1 of a pair produces g of step t = T-1-s:
//     carry_t = (1 - alpha) G_{t+1} + [g_{t+1} (J1 Wo + J0)] + sum_c A_c(t+1) [g_{t+1} Wa_c]     (0 at t = T-1)
//     G_t = grad_output_t + carry_t,      g_t = (alpha F'(re_t)) G_t                              (the record carries alpha)
// with the products in brackets taken over all N neurons of g_{t+1}: that is what the members exchange, by the
// forward's protocol with s in the place of its t (state s = g_{t+1}; a pair's first visit has no products).  Wpack
// holds the transposed matrices in this kernel's column order, J1 Wo^T + J0 as matrix 0.  What a pair carries from
// one visit to the next besides the exchanged g lives in a private scratch record per lane (registers and LDS are
// full of weights): (1 - alpha) G_t for its four rows (fp32) and, behind odd steps, the bf16 g of those rows -- the
// copy of g for the weight-gradient kernel keeps steps 2j and 2j+1 side by side in one 16-byte slot, and the even
// step that follows stores the slot whole.
// One more visit (t = -1) forms dL/dr_init when it is asked for.  No dL/dA and no fused loss head here: the caller
// runs those on the streaming kernel.
// ------------------------------------------------------------------------------------------------
template <bool GRI>
__global__ __launch_bounds__(512) void ring_bptt_cluster8_kernel(RingBpttArgs p, RingClusterArgs c) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xs = wlds + C8_WSLOTS;
  float* gl = reinterpret_cast<float*>(xs + C_XSLOTS);   // [2][32 rows][2] action gates, by pair-step parity
  int* misc = reinterpret_cast<int*>(gl + 128);          // [0]: abort
  char* const xchg = reinterpret_cast<char*>(c.xchg);
  constexpr int NSTE = 6;                                // stores of every epilogue: per tile exchange, carry record, g

  const int tid = threadIdx.x, w8 = tid >> 6, v = w8 & 3, h = w8 >> 2, lane = tid & 63, q = lane >> 4, n = lane & 15,
            g4 = n >> 2, j4 = n & 3;
  const int ct = 2 * v + h;
  const int blk = blockIdx.x, xcd = blk & 7, gi = blk >> 3, m = gi & 3, cl = (gi >> 2) * 8 + xcd;
  if (cl >= c.nclusters) return;
  const int B = p.B, T = p.T, nbt = p.nbt;
  constexpr int N = 512;
  const int S = T + (GRI ? 1 : 0);   // visits per pair
  const int my_ppc = (c.npairs - cl + c.nclusters - 1) / c.nclusters;
  const int w8u = __builtin_amdgcn_readfirstlane(w8);
  const bool skew = __builtin_amdgcn_readfirstlane(h) == 1 && my_ppc >= 2;

  if (tid == 0) misc[0] = 0;
  if (w8 == 0) {
    const int mine = (__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15) + 1;   // XCC_ID + 1
    if (lane == 0) flag_store(c.hello + cl * 4 + m, mine);
    int bad = c.spin_max < 0 ? 2 : 0;
    for (int spins = 0; !bad; ++spins) {
      const int hh = lane < 4 ? flag_load(c.hello + cl * 4 + lane) : mine;
      if (__ballot(hh == 0) == 0) {
        bad = __ballot(hh != mine) != 0 ? 1 : 0;
        break;
      }
      if (spins > c.spin_max) {
        bad = 2;
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    if (bad && lane == 0) {
      misc[0] = 1;
      *c.host_err = bad == 1 ? RING_CLUSTER_ERR_XCD : RING_CLUSTER_ERR_START;
    }
  }

  bf16x8 wreg[2][C_KCH];
  bf16x8 wo_last;
  bf16x8* wl = wlds + (size_t)(w8 * C8_WFR) * 64 + lane;
  {
    const bf16x8* Wp = reinterpret_cast<const bf16x8*>(p.Wpack);
#pragma unroll
    for (int kc = 0; kc < C_KCH; ++kc) {
      wreg[0][kc] = Wp[((size_t)((1 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
      wreg[1][kc] = Wp[((size_t)((2 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
    }
#pragma unroll
    for (int k8 = 0; k8 < C_KCH; k8 += 8) {
      bf16x8 f[8];
#pragma unroll
      for (int x = 0; x < 8; ++x) f[x] = Wp[((size_t)((0 * 4 + m) * C_NC + ct) * C_KCH + k8 + x) * 64 + lane];
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        if (k8 + x < C8_WFR) wl[(k8 + x) * 64] = f[x];
        else wo_last = f[x];
      }
    }
#pragma unroll
    for (int kc = 0; kc < C_KCH; ++kc) {
      asm volatile("" : "+a"(wreg[0][kc]));
      asm volatile("" : "+a"(wreg[1][kc]));
    }
  }

  const float oma = 1.f - p.alpha;
  const size_t xhalf_bytes = (size_t)2 * c.npairs * C_TILE_UNITS * 16;
  char* const bin = xchg + 2 * xhalf_bytes;
  char* const carry = reinterpret_cast<char*>(c.carry);     // [batch tile][member][wave][lane] x 16 bytes
  char* const ghalf = reinterpret_cast<char*>(c.ghalf);     // the same, first 8 bytes: bf16 g of the last odd step
  // lane-constant byte offsets
  const unsigned row_lane = (unsigned)(((4 * q + j4) * N + 128 * m + 16 * ct + 4 * g4) * 4);   // fp32 [16 rows][N]: row 4q+j4, four neurons
  const unsigned xq_lane = (unsigned)(((((4 * m + (ct >> 1)) * 4 + 2 * (ct & 1) + (g4 >> 1)) * 16) + 4 * q + j4) * 16 + 8 * (g4 & 1));
  const int lane_c = (lane & 48) | (2 * ct + (n >> 3)), cp = n & 7;   // the neuron's place in the common tile order
  const unsigned d_lane = (unsigned)(lane_c * 64 + 8 * cp);
  const unsigned r_lane = (unsigned)((cp * 64 + lane_c) * 16);
  const unsigned x_lane = (unsigned)(lane * 16);
  const unsigned g_lane = (unsigned)(((lane >> 1) * T * 2 + (lane & 1)) * 4);
  const unsigned f_lane = (unsigned)((lane & 31) * 4);
  const unsigned c_lane = (unsigned)(((m * 8 + w8) * 64 + lane) * 16);

  auto rows_base = [&](const float* base, int t, int bt) { return reinterpret_cast<const char*>(base) + ((size_t)t * B + 16 * bt) * N * 4; };
  auto flag_base = [&](int pl) { return reinterpret_cast<const char*>(c.flags) + ((size_t)cl * c.ppc + pl) * 32 * 4; };
  auto x_base = [&](int s, int pr) {
    return xchg + (size_t)(s & 1) * xhalf_bytes + ((size_t)(2 * pr) * C_TILE_UNITS + w8u * 256) * 16;
  };
  // gates of visit s: those of step t+1 = T - s, the step whose g is multiplied (the first visit multiplies zeros)
  auto gate_base = [&](int s, int pr) {
    const int tg = s == 0 ? T - 1 : T - s;
    return reinterpret_cast<const char*>(p.A) + ((size_t)(32 * pr) * T + tg) * 8;
  };

  int pf_pl = -1, pf_val = 0;   // exchange stores issued, flag not yet up: pair (local) and state number
  f32x4 P[2][3];                // products of the visit in hand: [tile][matrix]
  // what the epilogue of a visit reads besides P: grad_output rows (row 4q+j4, four neurons), the carry record, F', the held g half
  struct EpiIn {
    f32x4 go[2], cp[2];
    f32x2 fd[2], gh[2];
  };
  EpiIn Lr;
  int es = 0, epr = 0, epl = 0, eit = 0;   // the visit whose products are in P and whose epilogue is still to run (late half)
  bool epending = false;

  // Epilogue of visit (s, pr, pl), number `it` in this cluster's order, one batch tile at a time: the arithmetic on P
  // and the loaded inputs, then the tile's three stores (exchange, carry record, g copy).  The count of stores is the
  // same on every path -- the staging of the next operand counts on it -- so what has no place to go goes to the bin.
  struct EpiT {
    f32x2 xe;
    f32x4 cv, gvv;
  };
  auto epi_tile_math = [&](auto tlv, int s, int it, const EpiIn& in, EpiT& o) {
    constexpr int tl = decltype(tlv)::value;
    const float* gb = gl + (it & 1) * 64;
    const int t = T - 1 - s;
    const bool last = GRI && t < 0;       // the visit that forms dL/dr_init
    unsigned gr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float e0 = in.go[tl][i];
      gr[i] = __builtin_bit_cast(unsigned, e0);
    }
    quad_transpose(gr, j4);   // -> rows 4q+e of the lane's own neuron
    const f32x4 ga = *reinterpret_cast<const f32x4*>(gb + (16 * tl + 4 * q) * 2);
    const f32x4 gc = *reinterpret_cast<const f32x4*>(gb + (16 * tl + 4 * q + 2) * 2);
    const f16x4 d4 = __builtin_bit_cast(f16x4, in.fd[tl]);
    float gv[4], cn[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float g0 = e < 2 ? ga[2 * e] : gc[2 * (e - 2)], g1 = e < 2 ? ga[2 * e + 1] : gc[2 * (e - 2) + 1];
      const float p0 = P[tl][0][e], p1 = P[tl][1][e], p2 = P[tl][2][e];
      const float cprev = in.cp[tl][e];
      // (a pair's first visit has no step behind it: whatever operand was staged for it, its products are dropped)
      const float carry_t = s > 0 ? cprev + fmaf(g1, p2, fmaf(g0, p1, p0)) : 0.f;
      const float G = last ? carry_t : __builtin_bit_cast(float, gr[e]) + carry_t;
      const float dF = (float)d4[e];
      gv[e] = last ? G : dF * G;          // (last: the rows of dL/dr_init travel in gv)
      cn[e] = oma * G;
    }
    const bf16x4 g4b = {(__bf16)gv[0], (__bf16)gv[1], (__bf16)gv[2], (__bf16)gv[3]};
    const f32x2 gk = __builtin_bit_cast(f32x2, g4b);
    unsigned hh[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) hh[e] = __builtin_bit_cast(unsigned, gv[e]);
    quad_transpose(hh, j4);   // -> row 4q+j4, neurons 4 g4 + i
    const float h0 = __builtin_bit_cast(float, hh[0]), h1 = __builtin_bit_cast(float, hh[1]), h2 = __builtin_bit_cast(float, hh[2]),
                h3 = __builtin_bit_cast(float, hh[3]);
    const bf16x2 b01 = {(__bf16)h0, (__bf16)h1}, b23 = {(__bf16)h2, (__bf16)h3};
    o.xe = f32x2{__builtin_bit_cast(float, b01), __builtin_bit_cast(float, b23)};
    // (the dL/dr_init visit stores its fp32 rows where the others store the carry record)
    o.cv = f32x4{last ? h0 : cn[0], last ? h1 : cn[1], last ? h2 : cn[2], last ? h3 : cn[3]};
    const bool tail = t + 1 < T;
    o.gvv = f32x4{gk[0], gk[1], tail ? in.gh[tl][0] : 0.f, tail ? in.gh[tl][1] : 0.f};   // (an odd length's last slot: zero tail)
  };
  auto epi_tile_stores = [&](auto tlv, int s, int pr, const EpiT& o) {
    constexpr int tl = decltype(tlv)::value;
    const int t = T - 1 - s;
    const bool last = GRI && t < 0;
    const bool more = s + 1 < S;
    // 1: the exchange (a pair's last visit: nobody reads it)
    {
      const char* xb = xchg + (size_t)((s + 1) & 1) * xhalf_bytes + (size_t)(2 * pr + tl) * C_TILE_UNITS * 16;
      sstore8<0>(more ? xb : bin, xq_lane, o.xe);
    }
    // 2: the carry record, or the rows of dL/dr_init
    {
      const char* cb = carry + (size_t)(2 * pr + tl) * 32768;
      const char* ib = reinterpret_cast<const char*>(p.grad_r_init) + (size_t)(32 * pr + 16 * tl) * N * 4;
      sstore16<0>(last ? ib : cb, last ? row_lane : c_lane, o.cv);
    }
    // 3: the copy of g for the weight gradient: an odd step's half is held in the private record until the even step
    // that follows stores the slot whole
    {
      const char* hb = ghalf + (size_t)(2 * pr + tl) * 32768;
      const int tt = t < 0 ? 0 : t;
      const char* rb = reinterpret_cast<const char*>(p.gfrag) + (((size_t)(tt >> 1) * nbt + 2 * pr + tl) * 32 + 8 * m) * 64 * 16;
      const bool whole = !last && (t & 1) == 0;
      // (the half goes out as a whole 16-byte record too: one form of store on both paths)
      sstore16<0>(last ? bin : whole ? rb : hb, whole ? r_lane : c_lane, o.gvv);
    }
  };
  auto epi_done = [&](int s, int pl) {
    pf_pl = s + 1 < S ? pl : -1;
    pf_val = s + 1;
  };

  // the first visit has nothing to multiply (its products are dropped); zeros keep the matrix pipe's inputs tame
  {
    const bf16x8 z8 = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) xs[w8 * 256 + jj * 64 + lane] = z8;
  }
  if (w8 == 0) gl[lane] = *reinterpret_cast<const float*>(gate_base(0, cl) + g_lane);
  lds_barrier();
  if (misc[0]) return;

  // The two halves run different loops (one body, compiled twice): what the late half carries from one visit to the
  // next -- its products and the loaded inputs of the epilogue still to run -- would otherwise occupy registers on the
  // early half's path as well.
  auto run = [&](auto skv) {
    constexpr bool SK = decltype(skv)::value;
    int s = 0, pl = 0, it = 0;
    for (;;) {
      const int pr = cl + c.nclusters * pl;
      int ns = s, npl = pl + 1;
      if (npl == my_ppc) {
        npl = 0;
        ns = s + 1;
      }
      const bool have_next = ns < S;
      const bool look = have_next && ns >= 1;
      const int npr = cl + c.nclusters * npl;
      const int tc = T - 1 - s < 0 ? 0 : T - 1 - s;   // the step whose inputs this visit's epilogue reads (the last visit: none)

      f32x4 sreg[4];      // this wave's eighth of the next visit's operand
      int nflag;
      float gnext;
      bool up = false;
      auto fetch_issue = [&]() {
        gnext = sload4(have_next ? gate_base(ns, npr) : gate_base(s, pr), g_lane);
        nflag = sload4_dev(flag_base(look ? npl : pl), f_lane);
      };
      auto fetch_decide = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(nflag), "+v"(gnext)::"memory");
        up = look && __ballot(nflag < ns) == 0;
        sstore4_dev(pf_pl >= 0 ? flag_base(pf_pl) : bin, (unsigned)((8 * m + w8u) * 4), pf_val);   // (every lane the same word)
        pf_pl = -1;
      };
      auto fetch_x = [&](auto iv) {
        constexpr int i = decltype(iv)::value;
        const char* xb = look ? x_base(ns, npr) : x_base(s, pr);
        sreg[i] = sload16_dev<1024 * i>(xb, x_lane);
      };

      const bool thin = SK && !epending;
      if constexpr (SK) {
        EpiT o = {};
        fetch_issue();
        if (epending) epi_tile_math(std::integral_constant<int, 0>{}, es, eit, Lr, o);
        fetch_decide();
        fetch_x(std::integral_constant<int, 0>{});
        fetch_x(std::integral_constant<int, 1>{});
        fetch_x(std::integral_constant<int, 2>{});
        fetch_x(std::integral_constant<int, 3>{});
        if (epending) {
          epi_tile_stores(std::integral_constant<int, 0>{}, es, epr, o);
          epi_tile_math(std::integral_constant<int, 1>{}, es, eit, Lr, o);
          epi_tile_stores(std::integral_constant<int, 1>{}, es, epr, o);
          epi_done(es, epl);
        }
      }

      // ---- products ----
      {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
  #pragma unroll
        for (int tl = 0; tl < 2; ++tl) P[tl][0] = P[tl][1] = P[tl][2] = z;
      }
      const char* const gob = rows_base(p.grad_out, tc, 2 * pr);
      const char* const fdb = reinterpret_cast<const char*>(p.dfrag) + ((((size_t)tc * nbt + 2 * pr) * 4 + m) * 64) * 64;
      const char* const cpb = carry + (size_t)(2 * pr) * 32768;
      const char* const ghb = ghalf + (size_t)(2 * pr) * 32768;
      bf16x8 af[2][2], wf[2];
      auto frag_fetch = [&](auto kcv, int stg) {
        constexpr int kc = decltype(kcv)::value;
        af[stg][0] = xs[(0 * C_KCH + kc) * 64 + lane];
        af[stg][1] = xs[(1 * C_KCH + kc) * 64 + lane];
        if constexpr (kc < C8_WFR) wf[stg] = wl[kc * 64];
        else wf[stg] = wo_last;
      };
      auto body = [&](auto kcv, auto slotsv) {
        constexpr int kc = decltype(kcv)::value, stg = kc & 1;
        if constexpr (kc + 1 < C_KCH) frag_fetch(std::integral_constant<int, kc + 1>{}, stg ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (decltype(slotsv)::value) {
          if constexpr (kc == 0) fetch_issue();
          if constexpr (kc == 12) fetch_decide();
          if constexpr (kc >= 12) fetch_x(std::integral_constant<int, kc - 12>{});
          __builtin_amdgcn_sched_barrier(0);
        }
        P[0][1] = mfma16(af[stg][0], wreg[0][kc], P[0][1]);
        P[1][1] = mfma16(af[stg][1], wreg[0][kc], P[1][1]);
        P[0][2] = mfma16(af[stg][0], wreg[1][kc], P[0][2]);
        P[1][2] = mfma16(af[stg][1], wreg[1][kc], P[1][2]);
        P[0][0] = mfma16(af[stg][0], wf[stg], P[0][0]);
        P[1][0] = mfma16(af[stg][1], wf[stg], P[1][0]);
        __builtin_amdgcn_sched_barrier(0);
      };
      auto products = [&](auto slotsv) {
        frag_fetch(std::integral_constant<int, 0>{}, 0);
        __builtin_amdgcn_s_setprio(C8_PRIO);
        body(std::integral_constant<int, 0>{}, slotsv);
        body(std::integral_constant<int, 1>{}, slotsv);
        body(std::integral_constant<int, 2>{}, slotsv);
        body(std::integral_constant<int, 3>{}, slotsv);
        body(std::integral_constant<int, 4>{}, slotsv);
        body(std::integral_constant<int, 5>{}, slotsv);
        body(std::integral_constant<int, 6>{}, slotsv);
        body(std::integral_constant<int, 7>{}, slotsv);
        body(std::integral_constant<int, 8>{}, slotsv);
        body(std::integral_constant<int, 9>{}, slotsv);
        body(std::integral_constant<int, 10>{}, slotsv);
        body(std::integral_constant<int, 11>{}, slotsv);
        body(std::integral_constant<int, 12>{}, slotsv);
        body(std::integral_constant<int, 13>{}, slotsv);
        body(std::integral_constant<int, 14>{}, slotsv);
        body(std::integral_constant<int, 15>{}, slotsv);
        __builtin_amdgcn_s_setprio(0);
      };
      if constexpr (SK) {
        // (ordinary loads: they are read in the next visit's first phase, and the compiler waits for them there)
        Lr.go[0] = *reinterpret_cast<const f32x4*>(gob + row_lane);
        Lr.go[1] = *reinterpret_cast<const f32x4*>(gob + 16 * N * 4 + row_lane);
        Lr.cp[0] = *reinterpret_cast<const f32x4*>(cpb + c_lane);
        Lr.cp[1] = *reinterpret_cast<const f32x4*>(cpb + 32768 + c_lane);
        Lr.fd[0] = *reinterpret_cast<const f32x2*>(fdb + d_lane);
        Lr.fd[1] = *reinterpret_cast<const f32x2*>(fdb + 4 * 64 * 64 + d_lane);
        Lr.gh[0] = *reinterpret_cast<const f32x2*>(ghb + c_lane);
        Lr.gh[1] = *reinterpret_cast<const f32x2*>(ghb + 32768 + c_lane);
        products(std::false_type{});
        es = s;
        epr = pr;
        epl = pl;
        eit = it;
        epending = true;
      } else {
        // the early half reads them right behind its products: seven operations younger (gates, flags, the flag
        // store, four operand loads) are still allowed to be out when it does
        EpiIn La;
        La.go[0] = sload16<0>(gob, row_lane);
        La.go[1] = sload16<0>(gob + 16 * N * 4, row_lane);
        La.cp[0] = sload16<0>(cpb, c_lane);
        La.cp[1] = sload16<0>(cpb + 32768, c_lane);
        La.fd[0] = sload8<0>(fdb, d_lane);
        La.fd[1] = sload8<0>(fdb + 4 * 64 * 64, d_lane);
        La.gh[0] = sload8<0>(ghb, c_lane);
        La.gh[1] = sload8<0>(ghb + 32768, c_lane);
        products(std::true_type{});
        asm volatile("s_waitcnt vmcnt(7)"
                     : "+v"(La.go[0]), "+v"(La.go[1]), "+v"(La.cp[0]), "+v"(La.cp[1]), "+v"(La.fd[0]), "+v"(La.fd[1]), "+v"(La.gh[0]),
                       "+v"(La.gh[1])::"memory");
        EpiT o;
        epi_tile_math(std::integral_constant<int, 0>{}, s, it, La, o);
        epi_tile_stores(std::integral_constant<int, 0>{}, s, pr, o);
        epi_tile_math(std::integral_constant<int, 1>{}, s, it, La, o);
        epi_tile_stores(std::integral_constant<int, 1>{}, s, pr, o);
        epi_done(s, pl);
      }

      // ---- the next visit's operand and gates into LDS ----
      lds_barrier();
      if (thin) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NSTE) : "memory");
      if (!have_next) break;
      if (up) {
  #pragma unroll
        for (int jj = 0; jj < 4; ++jj) xs[w8 * 256 + jj * 64 + lane] = __builtin_bit_cast(bf16x8, sreg[jj]);
      } else {
        // nothing valid was fetched ahead: put up the flag still held back (the producers of what is waited for may
        // be waiting for it in turn), wait for the flags, then ordinary loads behind a device-scope acquire
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (pf_pl >= 0) sstore4_dev(flag_base(pf_pl), (unsigned)((8 * m + w8u) * 4), pf_val);
        pf_pl = -1;
        bool ok = false;
        for (int spins = 0; spins <= c.spin_max; ++spins) {
          const int f = flag_load(c.flags + ((size_t)cl * c.ppc + npl) * 32 + (lane & 31));
          if ((ok = (__ballot(f < ns) == 0))) break;
          __builtin_amdgcn_s_sleep(2);
        }
        if (!ok && lane == 0) {
          misc[0] = 1;
          *c.host_err = RING_CLUSTER_ERR_WAIT;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const bf16x8* xb = reinterpret_cast<const bf16x8*>(x_base(ns, npr));
  #pragma unroll
        for (int jj = 0; jj < 4; ++jj) xs[w8 * 256 + jj * 64 + lane] = xb[jj * 64 + lane];
      }
      if (w8 == 0) gl[((it + 1) & 1) * 64 + lane] = gnext;
      lds_barrier();
      if (misc[0]) return;
      s = ns;
      pl = npl;
      ++it;
    }
    if (SK && epending) {
      EpiT o;
      epi_tile_math(std::integral_constant<int, 0>{}, es, eit, Lr, o);
      epi_tile_stores(std::integral_constant<int, 0>{}, es, epr, o);
      epi_tile_math(std::integral_constant<int, 1>{}, es, eit, Lr, o);
      epi_tile_stores(std::integral_constant<int, 1>{}, es, epr, o);
    }

  };
  if (skew) run(std::true_type{});
  else run(std::false_type{});
}

// ------------------------------------------------------------------------------------------------
// Host side.
// ------------------------------------------------------------------------------------------------
namespace {

struct ClusterGeo {
  int npairs, ppc, nclusters, grid;
  size_t xchg_bytes, flag_bytes, hello_bytes;
};

constexpr size_t c_align(size_t n) { return (n + 255) & ~(size_t)255; }

ClusterGeo cluster_geo(int nbt) {
  ClusterGeo g;
  g.npairs = (nbt + 1) / 2;
  g.ppc = (g.npairs + 63) / 64;
  g.nclusters = (g.npairs + g.ppc - 1) / g.ppc;
  g.grid = 32 * ((g.nclusters + 7) / 8);
  g.xchg_bytes = c_align((size_t)2 * 2 * g.npairs * C_TILE_UNITS * 16 + C_BIN_BYTES);
  g.flag_bytes = c_align((size_t)g.nclusters * g.ppc * 32 * sizeof(int));   // (the eight-wave kernel: 32 per pair)
  g.hello_bytes = c_align((size_t)g.nclusters * 4 * sizeof(int));
  return g;
}

__global__ void ring_cluster_clear_kernel(int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// One word of pinned host memory for the whole process: a kernel that gives up a wait writes its reason there, and
// the host can look at it without synchronizing with the device.
int* g_host_err = nullptr;
int* g_host_err_dev = nullptr;

hipError_t host_err_word(int** dev) {
  static hipError_t status = [] {
    hipError_t e = hipHostMalloc((void**)&g_host_err, 64, hipHostMallocMapped | hipHostMallocPortable);
    if (e != hipSuccess) return e;
    *g_host_err = 0;
    return hipHostGetDevicePointer((void**)&g_host_err_dev, g_host_err, 0);
  }();
  *dev = g_host_err_dev;
  return status;
}

}  // namespace

bool ring_cluster_applicable(int N, int k) { return N == 512 && k == 2; }

size_t ring_cluster_workspace_bytes(int nbt) {
  const ClusterGeo g = cluster_geo(nbt);
  return g.xchg_bytes + g.flag_bytes + g.hello_bytes;
}

int ring_cluster_error() { return g_host_err ? *(volatile int*)g_host_err : 0; }

// The error word, the first time it is found set (0 afterwards): the caller reports it once; from then on the cluster
// kernel stays switched off (ring_uses_cluster) and the streaming kernels do the work.
int ring_cluster_take_error() {
  static bool reported = false;
  const int e = ring_cluster_error();
  if (e == 0 || reported) return 0;
  reported = true;
  return e;
}

// Where the cluster kernel runs.  It wins where every cluster has at least four batch-tile pairs to rotate through
// (B >= 6176 or so: 17 to 25 % at B = 8192 and 16384); with fewer, a pair-step waits for the state its siblings are
// still computing and the streaming kernels are several times faster.  RINGATTR_CLUSTER=0 switches it off, =1 on
// wherever the shape allows (tests of the short rotations).  Unasked, it also wants the device it was measured on
// (256 compute units in 8 XCDs); the placement check in the kernel is what it relies on elsewhere.
// (1: the cluster kernels can run this shape here; 0: not; ppc: batch-tile pairs per cluster)
static bool cluster_can_run(int N, int k, int B, int T, int* ppc, int* cus_out) {
  if (!ring_cluster_applicable(N, k) || B % 32 != 0 || T > (1 << 20)) return false;   // whole pairs of batch tiles
  const char* v = getenv("RINGATTR_CLUSTER");
  if (v && v[0] == '0') return false;
  if (ring_cluster_error()) return false;
  int dev = 0, cus = 0;   // (of the current device: asked every time, a process may hold several kinds)
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return false;
  const ClusterGeo g = cluster_geo(B / 16);
  if (g.grid > cus) return false;   // every workgroup needs a compute unit of its own, all at once
  *ppc = g.ppc;
  *cus_out = cus;
  return true;
}

bool ring_uses_cluster(int N, int k, int B, int T) {
  int ppc = 0, cus = 0;
  if (!cluster_can_run(N, k, B, T, &ppc, &cus)) return false;
  const char* v = getenv("RINGATTR_CLUSTER");
  const bool forced = v && v[0] == '1';
  return forced || (cus == 256 && ppc >= 4 && T >= 16);
}

// The cluster BPTT runs only where it is asked for (RINGATTR_CLUSTER_BPTT=1): at N = 512, B = 8192, T = 512 it takes
// 10.5 to 10.9 ms against the streaming kernel's 10.6, and the weight-gradient kernel behind it runs 0.5 ms slower.
// Unlike the forward, a visit has per-lane state to carry (fp32, 32 bytes per lane and pair) that fits neither the
// registers nor LDS beside the weights; its loads and stores, and the misses they cause in an L2 that also holds the
// exchange buffer, cost what keeping the weights on chip gains.
bool ring_uses_cluster_bptt(int N, int k, int B, int T) {
  const char* v = getenv("RINGATTR_CLUSTER_BPTT");
  if (!v || v[0] != '1') return false;
  int ppc = 0, cus = 0;
  return cluster_can_run(N, k, B, T, &ppc, &cus);
}

int ring_cluster_pack_order(int, int, int) { return 3; }

size_t ring_cluster_bptt_workspace_bytes(int nbt) {
  const ClusterGeo g = cluster_geo(nbt);
  return ring_cluster_workspace_bytes(nbt) + (size_t)2 * g.npairs * (32768 + 32768);   // + carry records, held g halves
}

template <int ACT>
static hipError_t launch_fwd_cluster_act(const RingFwdArgs& a, const RingClusterArgs& c, int grid, hipStream_t st) {
  auto go = [&](auto kern) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)C8_LDS_BYTES);
    if (e != hipSuccess) return e;
    RING_LAUNCH(kern, dim3(grid), dim3(512), C8_LDS_BYTES, st, a, c);
    return hipGetLastError();
  };
  return a.dfrag ? go(ring_fwd_cluster8_kernel<ACT, true>) : go(ring_fwd_cluster8_kernel<ACT, false>);
}

// The scratch area's parts, the flags cleared (on the stream, by a small kernel: the launch may be under graph capture).
static hipError_t cluster_args(void* cluster_ws, int nbt, RingClusterArgs& c, int& grid, hipStream_t st) {
  const ClusterGeo g = cluster_geo(nbt);
  char* ws = static_cast<char*>(cluster_ws);
  c.xchg = ws;
  c.flags = reinterpret_cast<int*>(ws + g.xchg_bytes);
  c.hello = reinterpret_cast<int*>(ws + g.xchg_bytes + g.flag_bytes);
  c.carry = reinterpret_cast<float*>(ws + g.xchg_bytes + g.flag_bytes + g.hello_bytes);
  c.ghalf = ws + g.xchg_bytes + g.flag_bytes + g.hello_bytes + (size_t)2 * g.npairs * 32768;
  hipError_t e = host_err_word(&c.host_err);
  if (e != hipSuccess) return e;
  c.npairs = g.npairs;
  c.nclusters = g.nclusters;
  c.ppc = g.ppc;
  c.spin_max = 4000000;
  if (const char* v = getenv("RINGATTR_CLUSTER_SPIN")) {
    const long s = atol(v);
    if (s >= -1 && s <= 100000000L) c.spin_max = (int)s;
  }
  grid = g.grid;
  const int nclear = (int)((g.flag_bytes + g.hello_bytes) / sizeof(int));
  hipLaunchKernelGGL(ring_cluster_clear_kernel, dim3((nclear + 255) / 256), dim3(256), 0, st, c.flags, nclear);
  return hipGetLastError();
}

hipError_t ring_launch_bptt_cluster(const RingBpttArgs& a, hipStream_t st) {
  if (!a.cluster_ws || !ring_cluster_applicable(a.N, a.k) || a.B % 32 != 0 || a.grad_A || a.loss_coef || !a.grad_out ||
      !a.dfrag || !a.gfrag)
    return hipErrorInvalidValue;
  RingClusterArgs c;
  int grid = 0;
  hipError_t e = cluster_args(a.cluster_ws, a.nbt, c, grid, st);
  if (e != hipSuccess) return e;
  auto go = [&](auto kern) {
    hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)C8_LDS_BYTES);
    if (e2 != hipSuccess) return e2;
    RING_LAUNCH(kern, dim3(grid), dim3(512), C8_LDS_BYTES, st, a, c);
    return hipGetLastError();
  };
  return a.grad_r_init ? go(ring_bptt_cluster8_kernel<true>) : go(ring_bptt_cluster8_kernel<false>);
}

hipError_t ring_launch_fwd_cluster(const RingFwdArgs& a, hipStream_t st) {
  if (!a.cluster_ws || !ring_cluster_applicable(a.N, a.k) || a.B % 32 != 0 || !a.hist) return hipErrorInvalidValue;
  RingClusterArgs c;
  int grid = 0;
  hipError_t e = cluster_args(a.cluster_ws, a.nbt, c, grid, st);
  if (e != hipSuccess) return e;
  switch (a.act) {
    case ACT_RELU: return launch_fwd_cluster_act<ACT_RELU>(a, c, grid, st);
    case ACT_GELU: return launch_fwd_cluster_act<ACT_GELU>(a, c, grid, st);
    case ACT_TANH: return launch_fwd_cluster_act<ACT_TANH>(a, c, grid, st);
    case ACT_SILU: return launch_fwd_cluster_act<ACT_SILU>(a, c, grid, st);
    default: return hipErrorInvalidValue;
  }
}
