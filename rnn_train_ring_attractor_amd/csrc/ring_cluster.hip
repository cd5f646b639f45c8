// Weight-resident forward for 256 < N <= 512 (NPAD = 512, NC = 8), a_dim = 2: the weights stay on chip, spread
// over a cluster of four compute units.
//
// [Wo|Wl|Wr] in bf16 is 1.5 MiB at NPAD = 512, four times what one compute unit can hold (the streaming kernels
// therefore pull all of it from L2 once per step and batch-tile pair, and a step is bound by that stream).  Here
// four workgroups on four compute units of ONE XCD (one L2) form a cluster: member m keeps the slices for output
// neurons 128 m .. 128 m + 127 for the whole sequence -- the two gated matrices in accumulation VGPRs, Wo in LDS,
// exactly the split of the N <= 256 weight-resident kernels -- and computes those neurons for all the cluster's
// batch rows.  What the members exchange per step is the new state in bf16, in the layout the next step's MFMA
// A operand is read in:
//   xchg[(t) & 1][batch tile][K chunk kc][q][row] x 16 bytes  =  r_t[row][32 kc + 8 q .. + 7],
// written with ordinary stores (they reach the XCD's L2, vmcnt tells when) and read with device-scope loads (which
// miss the vector L1).  A flag per (batch-tile pair, member, wave) carries the number of the last state written;
// a reader polls the sixteen flags of a pair before it loads the pair's operand.  The buffer has two halves by step
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
// A cluster works on its batch-tile pairs round robin inside a step (pair-steps), so that the state a pair-step
// needs was produced a whole round earlier and its flags are normally up when it looks; two batch tiles share every
// LDS fetch of a Wo fragment.  Per pair-step a wave (one per SIMD, two column tiles = 32 neurons = one K chunk of the
// next step's operand) issues 192 MFMAs.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

#include <type_traits>

namespace {

constexpr int C_NC = 8;
constexpr int C_KCH = 16;
constexpr int C_WFR = 2 * C_KCH - 1;              // Wo fragments of a wave kept in LDS (its last one stays in registers)
constexpr int C_WSLOTS = 4 * C_WFR * 64;
constexpr int C_TILE_UNITS = C_KCH * 4 * 16;      // 16-byte units of one batch tile's operand
constexpr int C_XSLOTS = 2 * C_TILE_UNITS;
constexpr size_t C_BIN_BYTES = 128 * 1024;        // target of the pipelined kernel's stores that have nothing to store
constexpr size_t C_LDS_BYTES = (size_t)(C_WSLOTS + C_XSLOTS) * 16 + 256 + 64;   // + gates, abort word

__device__ __forceinline__ f32x4 xchg_load16(const void* ptr) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=&v"(v) : "v"(ptr) : "memory");
  return v;
}
// Stores whose instruction count the waits below rely on (one instruction each, by construction).
__device__ __forceinline__ void store4(void* ptr, unsigned v) {
  asm volatile("global_store_dword %0, %1, off" ::"v"(ptr), "v"(v) : "memory");
}
__device__ __forceinline__ void store8(void* ptr, f32x2 v) {
  asm volatile("global_store_dwordx2 %0, %1, off" ::"v"(ptr), "v"(v) : "memory");
}
__device__ __forceinline__ void store16(void* ptr, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off" ::"v"(ptr), "v"(v) : "memory");
}

template <int K>
__device__ __forceinline__ void wait_staged(f32x4 (&s)[8]) {
  asm volatile("s_waitcnt vmcnt(%8)"
               : "+v"(s[0]), "+v"(s[1]), "+v"(s[2]), "+v"(s[3]), "+v"(s[4]), "+v"(s[5]), "+v"(s[6]), "+v"(s[7])
               : "n"(K)
               : "memory");
}

__device__ __forceinline__ int flag_load(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void flag_store(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

#ifdef CL_PROF
#define CL2_DECL() long long stamp_[10]; int item_ = 0
#define CL2_STAMP(i) stamp_[i] = clock64()
#define CL2_FLUSH() do { if (blk == 0 && tid == 0 && item_ >= 16 && item_ < 80) { for (int i_ = 0; i_ < 10; ++i_) g_cl_prof[(item_ - 16) * 16 + i_] = stamp_[i_]; g_cl_prof[(item_ - 16) * 16 + 10] = up; } ++item_; } while (0)
#else
#define CL2_DECL() do { } while (0)
#define CL2_STAMP(i) do { } while (0)
#define CL2_FLUSH() do { } while (0)
#endif
#ifdef CL_PROF
__device__ long long g_cl_prof[64 * 16];
#define CL_STAMP(i) do { if (blk == 0 && tid == 0 && prof_row >= 0 && prof_row < 64) g_cl_prof[prof_row * 16 + (i)] = clock64(); } while (0)
#else
#define CL_STAMP(i) do { } while (0)
#endif

}  // namespace

#ifdef CL_PROF
extern "C" __attribute__((visibility("default"))) int ringattr_exp_cl_prof(long long* out) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_cl_prof), sizeof(long long) * 64 * 16);
}
#endif

// FULL: N == 512 and B % 32 == 0 (no masking, counted waits).
template <int ACT, bool SAVE, bool FULL>
__global__ __launch_bounds__(256) void ring_fwd_cluster_kernel(RingFwdArgs p, RingClusterArgs c) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xs = wlds + C_WSLOTS;
  int* misc = reinterpret_cast<int*>(xs + C_XSLOTS);   // [0]: abort
  bf16x8* const xchg = reinterpret_cast<bf16x8*>(c.xchg);

  const int tid = threadIdx.x, v = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15;
  const int blk = blockIdx.x, xcd = blk & 7, gi = blk >> 3, m = gi & 3, cl = (gi >> 2) * 8 + xcd;
  if (cl >= c.nclusters) return;
  const int N = p.N, B = p.B, T = p.T, nbt = p.nbt;
  const int my_ppc = (c.npairs - cl + c.nclusters - 1) / c.nclusters;   // pairs cl, cl + nclusters, ...
  const int vu = __builtin_amdgcn_readfirstlane(v);

  // ---- handshake: all four members resident, on one XCD ----
  if (tid == 0) misc[0] = 0;
  if (v == 0) {
    const int mine = (__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15) + 1;   // XCC_ID + 1
    if (lane == 0) flag_store(c.hello + cl * 4 + m, mine);
    int bad = 0;
    for (int spins = 0;; ++spins) {
      const int h = lane < 4 ? flag_load(c.hello + cl * 4 + lane) : mine;
      if (__ballot(h == 0) == 0) {
        bad = __ballot(h != mine) != 0 ? 1 : 0;
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

  // ---- resident weights ----
  bf16x8 wreg[2][2][C_KCH];
  bf16x8 wo_last;
  bf16x8* wl = wlds + (size_t)(v * C_WFR) * 64 + lane;
  {
    const bf16x8* Wp = reinterpret_cast<const bf16x8*>(p.Wpack);
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int kc = 0; kc < C_KCH; ++kc) {
        const int ct = 2 * v + cc;
        const bf16x8 f0 = Wp[((size_t)((0 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
        if (cc * C_KCH + kc < C_WFR) wl[(cc * C_KCH + kc) * 64] = f0;
        else wo_last = f0;
        wreg[0][cc][kc] = Wp[((size_t)((1 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
        wreg[1][cc][kc] = Wp[((size_t)((2 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
        asm volatile("" : "+a"(wreg[0][cc][kc]));
        asm volatile("" : "+a"(wreg[1][cc][kc]));
      }
  }
  lds_barrier();
  if (misc[0]) return;

  const float oma = 1.f - p.alpha;
  const ActScale asc = act_scale_make(p.alpha);
  const int i0 = 128 * m + 32 * v + 2 * n;            // this lane's two neurons (one per column tile)
  // their place in the common tile order of the saved buffers (tile c, column n' <-> neuron 128 m + 8 n' + c)
  const int lane_c = (lane & 48) | (4 * v + (n >> 2)), c0 = 2 * (n & 3);
  const size_t xhalf = (size_t)2 * c.npairs * C_TILE_UNITS;   // units per parity half of the exchange buffer

  f32x4 sreg[8];              // this wave's quarter of the next pair's operand, in flight
  bool prefetched = false;
  int pend_idx = -1, pend_val = 0;   // flag of the last pair-step whose exchange stores are not yet published
  int nst = 0;                       // stores the last pair-step's epilogue issued (unmasked variant: exact)

  auto signal_pending = [&]() {   // only behind a wait that covers the exchange stores
    if (pend_idx >= 0 && lane == 0) flag_store(c.flags + pend_idx, pend_val);
    pend_idx = -1;
  };
  auto flags_up = [&](int pl, int need) {
    const int f = lane < 16 ? flag_load(c.flags + ((size_t)cl * c.ppc + pl) * 16 + lane) : need;
    return __ballot(f < need) == 0;
  };
  auto issue_xchg_loads = [&](int t, int pr) {
    const bf16x8* src = xchg + (size_t)(t & 1) * xhalf + (size_t)(2 * pr) * C_TILE_UNITS + v * 512 + lane;
#pragma unroll
    for (int j = 0; j < 8; ++j) sreg[j] = xchg_load16(src + j * 64);
  };

  for (int t = 0; t < T; ++t) {
    for (int pl = 0; pl < my_ppc; ++pl) {
      const int pr = cl + c.nclusters * pl;
#ifdef CL_PROF
      const int prof_row = (t - 4) * my_ppc + pl;   // rows 0.. from step 4 on
      const bool was_prefetched = prefetched;
#endif
      CL_STAMP(0);
      lds_barrier();   // every wave has finished reading the operand of the previous pair-step
      CL_STAMP(1);
      if (t == 0) {
        // the first operand comes from r_init
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int u = v * 512 + j * 64 + lane;
          const int tl = u >> 10, kc = (u >> 6) & 15, qq = (u >> 4) & 3, row = u & 15;
          const int b = 32 * pr + 16 * tl + row, k0 = 32 * kc + 8 * qq;
          bf16x8 pk;
          if (FULL || (b < B && k0 + 8 <= N && (N & 3) == 0)) {
            const f32x4* src = reinterpret_cast<const f32x4*>(p.r_init + (size_t)b * N + k0);
            const f32x4 lo = src[0], hi = src[1];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
              pk[x] = (__bf16)lo[x];
              pk[4 + x] = (__bf16)hi[x];
            }
          } else {
#pragma unroll
            for (int x = 0; x < 8; ++x) pk[x] = (__bf16)((b < B && k0 + x < N) ? p.r_init[(size_t)b * N + k0 + x] : 0.f);
          }
          xs[u] = pk;
        }
      } else {
        if (!prefetched) {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          signal_pending();
          bool up = false;
          for (int spins = 0; spins <= c.spin_max; ++spins) {
            if ((up = flags_up(pl, t))) break;
            __builtin_amdgcn_s_sleep(2);
          }
          if (up) {
            issue_xchg_loads(t, pr);
          } else if (lane == 0) {
            misc[0] = 1;
            *c.host_err = RING_CLUSTER_ERR_WAIT;
          }
          wait_staged<0>(sreg);
        } else if constexpr (FULL) {
          // the prefetch is older than the nst stores of the pair-step in between, and nothing else was issued since
          switch (nst) {
            case 8: wait_staged<8>(sreg); break;
            case 10: wait_staged<10>(sreg); break;
            case 14: wait_staged<14>(sreg); break;
            case 16: wait_staged<16>(sreg); break;
            case 18: wait_staged<18>(sreg); break;
            case 22: wait_staged<22>(sreg); break;
            case 26: wait_staged<26>(sreg); break;
            default: wait_staged<0>(sreg); break;
          }
        } else {
          wait_staged<0>(sreg);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) xs[v * 512 + j * 64 + lane] = __builtin_bit_cast(bf16x8, sreg[j]);
        prefetched = false;
      }
      CL_STAMP(2);
      lds_barrier();
      if (misc[0]) return;
      CL_STAMP(3);

      // inputs of this pair-step's epilogue: previous state (fp32) and action gates of the lane's rows
      f32x2 rold[2][4], gate[2][4];
#pragma unroll
      for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int b = 32 * pr + 16 * tl + 4 * q + e;
          const int bc = FULL ? b : (b < B ? b : B - 1);
          gate[tl][e] = *reinterpret_cast<const f32x2*>(p.A + ((size_t)bc * T + t) * 2);
          const float* prev = (t == 0 ? p.r_init : p.hist + (size_t)(t - 1) * B * N) + (size_t)bc * N + i0;
          if (FULL) {
            rold[tl][e] = *reinterpret_cast<const f32x2*>(prev);
          } else {
            rold[tl][e][0] = (b < B && i0 < N) ? prev[0] : 0.f;
            rold[tl][e][1] = (b < B && i0 + 1 < N) ? prev[1] : 0.f;
          }
        }
      // the next pair-step and whether its operand can be fetched under this one's products
      int nt = t, npl = pl + 1;
      if (npl == my_ppc) {
        npl = 0;
        nt = t + 1;
      }
      const bool look = nt < T && nt >= 1;
      // (always issued: its arrival is also what tells that the previous pair-step's stores have landed)
      const int nflag = flag_load(c.flags + ((size_t)cl * c.ppc + (look ? npl : pl)) * 16 + n);

      // ---- products: P[tile][cc][matrix] ----
      f32x4 P[2][2][3];
      {
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int tl = 0; tl < 2; ++tl)
#pragma unroll
          for (int cc = 0; cc < 2; ++cc) P[tl][cc][0] = P[tl][cc][1] = P[tl][cc][2] = z;
      }
      bf16x8 af[2][2], wf[2][2];
      auto frag_fetch = [&](auto kcv, int stg) {
        constexpr int kc = decltype(kcv)::value;
        af[stg][0] = xs[(0 * C_KCH + kc) * 64 + lane];
        af[stg][1] = xs[(1 * C_KCH + kc) * 64 + lane];
        wf[stg][0] = wl[(0 * C_KCH + kc) * 64];
        if constexpr (C_KCH + kc < C_WFR) wf[stg][1] = wl[(1 * C_KCH + kc) * 64];
        else wf[stg][1] = wo_last;
      };
      auto mfma_half = [&](auto halfv) {
        constexpr int half = decltype(halfv)::value;
        auto body = [&](auto jv) {
          constexpr int kc = 8 * half + decltype(jv)::value, stg = kc & 1;
          if constexpr (kc + 1 < C_KCH) {
            frag_fetch(std::integral_constant<int, kc + 1>{}, stg ^ 1);
            __builtin_amdgcn_sched_barrier(0);
          }
#pragma unroll
          for (int cc = 0; cc < 2; ++cc) {
            P[0][cc][1] = mfma16(af[stg][0], wreg[0][cc][kc], P[0][cc][1]);
            P[1][cc][1] = mfma16(af[stg][1], wreg[0][cc][kc], P[1][cc][1]);
            P[0][cc][2] = mfma16(af[stg][0], wreg[1][cc][kc], P[0][cc][2]);
            P[1][cc][2] = mfma16(af[stg][1], wreg[1][cc][kc], P[1][cc][2]);
            P[0][cc][0] = mfma16(af[stg][0], wf[stg][cc], P[0][cc][0]);
            P[1][cc][0] = mfma16(af[stg][1], wf[stg][cc], P[1][cc][0]);
          }
          __builtin_amdgcn_sched_barrier(0);
        };
        body(std::integral_constant<int, 0>{});
        body(std::integral_constant<int, 1>{});
        body(std::integral_constant<int, 2>{});
        body(std::integral_constant<int, 3>{});
        body(std::integral_constant<int, 4>{});
        body(std::integral_constant<int, 5>{});
        body(std::integral_constant<int, 6>{});
        body(std::integral_constant<int, 7>{});
      };
      frag_fetch(std::integral_constant<int, 0>{}, 0);
      __builtin_amdgcn_s_setprio(1);
      CL_STAMP(4);
      mfma_half(std::integral_constant<int, 0>{});
      CL_STAMP(5);
      // The flag load above is younger than every store of the previous pair-step, and vector-memory operations
      // leave the counter in issue order: once its value is here, those stores have reached L2.
      asm volatile("" ::"v"(nflag) : "memory");
      signal_pending();
      if (look && __ballot(nflag < nt) == 0) {
        issue_xchg_loads(nt, cl + c.nclusters * npl);
        prefetched = true;
      }
      CL_STAMP(6);
      mfma_half(std::integral_constant<int, 1>{});
      __builtin_amdgcn_s_setprio(0);
      CL_STAMP(7);

      // ---- epilogue ----
      const bool more = t + 1 < T;
      float rn[2][4][2], dd[2][4][2];
#pragma unroll
      for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int b = 32 * pr + 16 * tl + 4 * q + e;
#pragma unroll
          for (int cc = 0; cc < 2; ++cc) {
            const float x = fmaf(gate[tl][e][1], P[tl][cc][2][e], fmaf(gate[tl][e][0], P[tl][cc][1][e], P[tl][cc][0][e]));
            float aF, aD;
            act_scaled<ACT>(x, asc, aF, aD);
            float r1 = fmaf(oma, rold[tl][e][cc], aF);
            if constexpr (!FULL) {
              const bool ok = b < B && i0 + cc < N;
              r1 = ok ? r1 : 0.f;
              aD = ok ? aD : 0.f;
            }
            rn[tl][e][cc] = r1;
            dd[tl][e][cc] = aD;
          }
        }
      nst = 0;
      CL_STAMP(8);
#pragma unroll
      for (int tl = 0; tl < 2; ++tl) {
        const int bt = 2 * pr + tl;
        const bool live = FULL || bt < nbt;
        // history rows
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int b = 16 * bt + 4 * q + e;
          float* dst = p.hist + ((size_t)t * B + b) * N + i0;
          if constexpr (FULL) {
            store8(dst, f32x2{rn[tl][e][0], rn[tl][e][1]});
          } else if (b < B) {
            if (i0 < N) dst[0] = rn[tl][e][0];
            if (i0 + 1 < N) dst[1] = rn[tl][e][1];
          }
        }
        nst += 4;
        if (SAVE && live) {
          // alpha F'(re): the lane's two tiles lie side by side in the record
          typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
          const f16x8 dk = {(_Float16)dd[tl][0][0], (_Float16)dd[tl][1][0], (_Float16)dd[tl][2][0], (_Float16)dd[tl][3][0],
                            (_Float16)dd[tl][0][1], (_Float16)dd[tl][1][1], (_Float16)dd[tl][2][1], (_Float16)dd[tl][3][1]};
          store16(p.dfrag + side_offset<C_NC>(t, nbt, bt, m, lane_c) + 4 * c0, __builtin_bit_cast(f32x4, dk));
          nst += 1;
          // bf16 operand copies for the weight gradient: slot t' holds the state before step t'; an odd length's
          // last pair has a zero second half
          if (t == 0) {
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) {
              const bf16x4 pk = {(__bf16)rold[tl][0][cc], (__bf16)rold[tl][1][cc], (__bf16)rold[tl][2][cc], (__bf16)rold[tl][3][cc]};
              store8(p.rfrag + pair_offset<C_NC>(0, nbt, bt, m * C_NC + c0 + cc, lane_c), __builtin_bit_cast(f32x2, pk));
            }
            nst += 2;
          }
          if (more || (T & 1)) {
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) {
              const bf16x4 pk = {(__bf16)rn[tl][0][cc], (__bf16)rn[tl][1][cc], (__bf16)rn[tl][2][cc], (__bf16)rn[tl][3][cc]};
              store8(p.rfrag + pair_offset<C_NC>(t + 1, nbt, bt, m * C_NC + c0 + cc, lane_c),
                     more ? __builtin_bit_cast(f32x2, pk) : f32x2{0.f, 0.f});
            }
            nst += 2;
          }
        }
        if (more) {
          // the next step's operand, for all four members
          char* dst = reinterpret_cast<char*>(xchg + (size_t)((t + 1) & 1) * xhalf + (size_t)bt * C_TILE_UNITS +
                                              ((4 * m + vu) * 4 + (n >> 2)) * 16 + 4 * q) + (n & 3) * 4;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bf16x2 pk = {(__bf16)rn[tl][e][0], (__bf16)rn[tl][e][1]};
            store4(dst + e * 16, __builtin_bit_cast(unsigned, pk));
          }
          nst += 4;
        }
      }
      if (more) {
        pend_idx = (int)(((size_t)cl * c.ppc + pl) * 16 + 4 * m + v);
        pend_val = t + 1;
      }
      CL_STAMP(9);
#ifdef CL_PROF
      if (blk == 0 && tid == 0 && prof_row >= 0 && prof_row < 64) g_cl_prof[prof_row * 16 + 10] = was_prefetched;
#endif
    }
  }
  // (the last step publishes nothing: pend_idx is unset here)
}

// ------------------------------------------------------------------------------------------------
// The unmasked forward (N == 512, B % 32 == 0), pipelined.
//
// One compute unit has one address path for vector memory, shared by its four waves, and every load or store
// instruction of a wave occupies it for tens of cycles: issued in bursts between the products (as above) the ~190
// memory instructions of a pair-step cost more time than its 768 MFMAs.  This variant
//  * issues every vector-memory instruction of the time loop between MFMA groups: the stores of pair-step s-1 and the
//    loads for s and s+1 ride in the product loop of pair-step s (all through inline assembly, so that their number
//    is known and the waits can count: vector-memory operations leave the counter in issue order);
//  * moves whole 16-byte pieces: a quad of lanes holds [4 rows][8 neurons] of a tile as 4 x 2 per lane, and a 4x4
//    transpose inside the quad (DPP) turns that into one row's eight neurons per lane, for the history rows, the
//    previous state and the exchanged operand alike;
//  * fetches the action gates of a pair-step once per workgroup (one load by wave 0, through LDS).
// ------------------------------------------------------------------------------------------------
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
template <int IMM>
__device__ __forceinline__ void sstore16(const void* sbase, unsigned voff, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, %2 offset:%3" ::"v"(voff), "v"(v), "s"(sbase), "n"(IMM) : "memory");
}
template <int IMM>
__device__ __forceinline__ void sstore8(const void* sbase, unsigned voff, f32x2 v) {
  asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3" ::"v"(voff), "v"(v), "s"(sbase), "n"(IMM) : "memory");
}
__device__ __forceinline__ void sstore4_dev(const void* sbase, unsigned voff, int v) {
  asm volatile("global_store_dword %0, %1, %2 sc1" ::"v"(voff), "v"(v), "s"(sbase) : "memory");
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
__device__ __forceinline__ void vm_wait_x(f32x4 (&s)[8]) {
  asm volatile("s_waitcnt vmcnt(%8)"
               : "+v"(s[0]), "+v"(s[1]), "+v"(s[2]), "+v"(s[3]), "+v"(s[4]), "+v"(s[5]), "+v"(s[6]), "+v"(s[7])
               : "n"(K)
               : "memory");
}
template <int K>
__device__ __forceinline__ void vm_wait_in(f32x4 (&l)[2][2], int& flag, float& gate) {
  asm volatile("s_waitcnt vmcnt(%6)"
               : "+v"(l[0][0]), "+v"(l[0][1]), "+v"(l[1][0]), "+v"(l[1][1]), "+v"(flag), "+v"(gate)
               : "n"(K)
               : "memory");
}
template <int K>
__device__ __forceinline__ void vm_wait_plain() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(K) : "memory");
}

}  // namespace

// The instruction stream of a pair-step is the same every time -- where there is nothing to store or to fetch, the
// instruction goes to a scratch bin of the workspace or reads what is at hand -- so every wait below counts against a
// fixed number of younger operations (anything the compiler adds on top only makes a wait stricter).  Per pair-step,
// in issue order:
//   slot 0        4 loads of the previous state, 1 of the next pair-step's gates, 1 of its flags          (6 loads)
//   slots 1..6    the stores of the previous pair-step: 2 exchange, 4 history, [2 record, 4 operand copy] (NST)
//   slot 8        wait for the six loads: vmcnt(NST); slots 8..11: the next pair-step's operand          (8 loads)
//   after the products: wait for the two exchange stores: vmcnt(NST - 2 + 8), then the flag store         (1 store)
//   [first step only: 4 stores of the operand copy's slot 0]
//   staging of the next operand: wait for the 8 loads: vmcnt(1)
template <int ACT, bool SAVE>
__global__ __launch_bounds__(256) void ring_fwd_cluster_full_kernel(RingFwdArgs p, RingClusterArgs c) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  bf16x8* wlds = reinterpret_cast<bf16x8*>(smem);
  bf16x8* xs = wlds + C_WSLOTS;
  float* gl = reinterpret_cast<float*>(xs + C_XSLOTS);   // [32 rows][2] action gates of the current pair-step
  int* misc = reinterpret_cast<int*>(gl + 64);           // [0]: abort
  char* const xchg = reinterpret_cast<char*>(c.xchg);
  constexpr int NST = SAVE ? 12 : 6;

  const int tid = threadIdx.x, v = tid >> 6, lane = tid & 63, q = lane >> 4, n = lane & 15, g4 = n >> 2, j4 = n & 3;
  const int blk = blockIdx.x, xcd = blk & 7, gi = blk >> 3, m = gi & 3, cl = (gi >> 2) * 8 + xcd;
  if (cl >= c.nclusters) return;
  const int B = p.B, T = p.T, nbt = p.nbt;
  constexpr int N = 512;
  const int my_ppc = (c.npairs - cl + c.nclusters - 1) / c.nclusters;
  const int vu = __builtin_amdgcn_readfirstlane(v);

  if (tid == 0) misc[0] = 0;
  if (v == 0) {
    const int mine = (__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 15) + 1;   // XCC_ID + 1
    if (lane == 0) flag_store(c.hello + cl * 4 + m, mine);
    int bad = 0;
    for (int spins = 0;; ++spins) {
      const int h = lane < 4 ? flag_load(c.hello + cl * 4 + lane) : mine;
      if (__ballot(h == 0) == 0) {
        bad = __ballot(h != mine) != 0 ? 1 : 0;
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

  bf16x8 wreg[2][2][C_KCH];
  bf16x8 wo_last;
  bf16x8* wl = wlds + (size_t)(v * C_WFR) * 64 + lane;
  {
    const bf16x8* Wp = reinterpret_cast<const bf16x8*>(p.Wpack);
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int kc = 0; kc < C_KCH; ++kc) {
        const int ct = 2 * v + cc;
        wreg[0][cc][kc] = Wp[((size_t)((1 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
        wreg[1][cc][kc] = Wp[((size_t)((2 * 4 + m) * C_NC + ct) * C_KCH + kc) * 64 + lane];
      }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int k8 = 0; k8 < C_KCH; k8 += 8) {
        bf16x8 f[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) f[x] = Wp[((size_t)((0 * 4 + m) * C_NC + 2 * v + cc) * C_KCH + k8 + x) * 64 + lane];
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          if (cc * C_KCH + k8 + x < C_WFR) wl[(cc * C_KCH + k8 + x) * 64] = f[x];
          else wo_last = f[x];
        }
      }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc)
#pragma unroll
      for (int kc = 0; kc < C_KCH; ++kc) {
        asm volatile("" : "+a"(wreg[0][cc][kc]));
        asm volatile("" : "+a"(wreg[1][cc][kc]));
      }
  }

  const float oma = 1.f - p.alpha;
  const ActScale asc = act_scale_make(p.alpha);
  const int lane_c = (lane & 48) | (4 * v + g4), c0 = 2 * j4;
  const size_t xhalf_bytes = (size_t)2 * c.npairs * C_TILE_UNITS * 16;
  char* const bin = xchg + 2 * xhalf_bytes;   // where stores go that have nothing to store (C_BIN_BYTES)
  // lane-constant byte offsets (what varies with step and tile is wave-uniform and goes into the scalar base)
  const unsigned row_lane = (unsigned)(((4 * q + j4) * N + 128 * m + 32 * v + 8 * g4) * 4);   // fp32 [16 rows][N]: row 4q+j4, eight neurons
  const unsigned xq_lane = (unsigned)(((((4 * m + v) * 4 + g4) * 16) + 4 * q + j4) * 16);     // exchange unit (own K chunk, g4, row 4q+j4)
  const unsigned d_lane = (unsigned)(lane_c * 64 + 8 * c0);
  const unsigned r_lane = (unsigned)((c0 * 64 + lane_c) * 16);
  const unsigned x_lane = (unsigned)(lane * 16), x_lane_hi = x_lane + 4096;
  const unsigned g_lane = (unsigned)(((lane >> 1) * T * 2 + (lane & 1)) * 4);
  const unsigned f_lane = (unsigned)(n * 4);

  // deferred stores of the last finished pair-step
  f32x4 dh[2][2], dd16[2], dx[2];
  f32x2 dr[2][2];
  {
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    dh[0][0] = dh[0][1] = dh[1][0] = dh[1][1] = dd16[0] = dd16[1] = dx[0] = dx[1] = z;
    dr[0][0] = dr[0][1] = dr[1][0] = dr[1][1] = f32x2{0.f, 0.f};
  }
  bool dreal = false, dmore = false;
  int dt = 0, dpr = 0, dpl = 0;

  auto hist_base = [&](int t, int bt) { return reinterpret_cast<const char*>(p.hist) + ((size_t)t * B + 16 * bt) * N * 4; };
  auto emit = [&](auto iv) {
    constexpr int i = decltype(iv)::value;
    if constexpr (i < 2) {
      const char* base = xchg + (size_t)((dt + 1) & 1) * xhalf_bytes + (size_t)(2 * dpr + i) * C_TILE_UNITS * 16;
      sstore16<0>(dreal ? base : bin, xq_lane, dx[i]);
    } else if constexpr (i < 6) {
      constexpr int tl = (i - 2) >> 1, hf = (i - 2) & 1;
      const char* base = hist_base(dt, 2 * dpr + tl);
#ifdef CL_KNOCK_BIN
      sstore16<16 * hf>(bin, row_lane, dh[tl][hf]);
#else
      sstore16<16 * hf>(dreal ? base : bin, row_lane, dh[tl][hf]);
#endif
    } else if constexpr (i < 8) {
      if constexpr (SAVE) {
        constexpr int tl = i - 6;
        const char* base = reinterpret_cast<const char*>(p.dfrag) + ((((size_t)dt * nbt + 2 * dpr + tl) * 4 + m) * 64) * 64;
#ifdef CL_KNOCK_BIN
        sstore16<0>(bin, d_lane, dd16[tl]);
#else
        sstore16<0>(dreal ? base : bin, d_lane, dd16[tl]);
#endif
      }
    } else {
      if constexpr (SAVE) {
        constexpr int tl = (i - 8) >> 1, cc = (i - 8) & 1;
        // slot t+1 of the operand copy; past the last step there is none (an odd length's is the zero tail)
        const char* base = reinterpret_cast<const char*>(p.rfrag) +
                           (((size_t)((dt + 1) >> 1) * nbt + 2 * dpr + tl) * 32 + 8 * m) * 64 * 16 + ((dt + 1) & 1) * 8;
        const bool there = dreal && (dmore || (T & 1));
#ifdef CL_KNOCK_BIN
        sstore8<1024 * cc>(there ? bin : bin, r_lane, dmore ? dr[tl][cc] : f32x2{0.f, 0.f});
#else
        sstore8<1024 * cc>(there ? base : bin, r_lane, dmore ? dr[tl][cc] : f32x2{0.f, 0.f});
#endif
      }
    }
  };
  auto emit_all = [&]() {
    emit(std::integral_constant<int, 0>{});
    emit(std::integral_constant<int, 1>{});
    emit(std::integral_constant<int, 2>{});
    emit(std::integral_constant<int, 3>{});
    emit(std::integral_constant<int, 4>{});
    emit(std::integral_constant<int, 5>{});
    emit(std::integral_constant<int, 6>{});
    emit(std::integral_constant<int, 7>{});
    emit(std::integral_constant<int, 8>{});
    emit(std::integral_constant<int, 9>{});
    emit(std::integral_constant<int, 10>{});
    emit(std::integral_constant<int, 11>{});
  };
  auto flag_base = [&](int pl) { return reinterpret_cast<const char*>(c.flags) + ((size_t)cl * c.ppc + pl) * 16 * 4; };
  auto x_base = [&](int t, int pr) {
    return xchg + (size_t)(t & 1) * xhalf_bytes + ((size_t)(2 * pr) * C_TILE_UNITS + vu * 512) * 16;
  };
  auto gate_base = [&](int t, int pr) { return reinterpret_cast<const char*>(p.A) + ((size_t)(32 * pr) * T + t) * 8; };
  auto stage_from_r_init = [&](int pr) {
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      const int u = v * 512 + jj * 64 + lane;
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

  // the first pair-step's operand and gates
  stage_from_r_init(cl);
  if (v == 0) gl[lane] = *reinterpret_cast<const float*>(gate_base(0, cl) + g_lane);
  lds_barrier();
  if (misc[0]) return;

  int t = 0, pl = 0;
  CL2_DECL();
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

    f32x4 P[2][2][3];
    {
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int tl = 0; tl < 2; ++tl)
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) P[tl][cc][0] = P[tl][cc][1] = P[tl][cc][2] = z;
    }
    f32x4 L[2][2];      // previous state: eight neurons of the lane's row 4q+j4, per tile
    f32x4 sreg[8];      // this wave's quarter of the next pair-step's operand
    int nflag;
    float gnext;
    bool up = false;
    // what goes out between the MFMA groups of K chunk kc
    auto slot = [&](auto kcv) {
      constexpr int kc = decltype(kcv)::value;
      if constexpr (kc == 0) {
        const char* pb = t == 0 ? reinterpret_cast<const char*>(p.r_init) + (size_t)(32 * pr) * N * 4 : hist_base(t - 1, 2 * pr);
        L[0][0] = sload16<0>(pb, row_lane);
        L[0][1] = sload16<16>(pb, row_lane);
        L[1][0] = sload16<0>(pb + 16 * N * 4, row_lane);
        L[1][1] = sload16<16>(pb + 16 * N * 4, row_lane);
        gnext = sload4(have_next ? gate_base(nt, npr) : gate_base(t, pr), g_lane);
        nflag = sload4_dev(flag_base(look ? npl : pl), f_lane);
      } else if constexpr (kc >= 1 && kc <= 6) {
        emit(std::integral_constant<int, 2 * (kc - 1)>{});
        emit(std::integral_constant<int, 2 * (kc - 1) + 1>{});
      } else if constexpr (kc == 8) {
        vm_wait_in<NST>(L, nflag, gnext);
        up = look && __ballot(nflag < nt) == 0;
      }
      if constexpr (kc >= 8 && kc <= 11) {
        const char* xb = look ? x_base(nt, npr) : x_base(t, pr);
        constexpr int jj = 2 * (kc - 8);
        sreg[jj] = sload16_dev<1024 * (jj & 3)>(xb, jj < 4 ? x_lane : x_lane_hi);
        sreg[jj + 1] = sload16_dev<1024 * ((jj + 1) & 3)>(xb, jj < 4 ? x_lane : x_lane_hi);
      }
    };
    bf16x8 af[2][2], wf[2][2];
    auto frag_fetch = [&](auto kcv, int stg) {
      constexpr int kc = decltype(kcv)::value;
      af[stg][0] = xs[(0 * C_KCH + kc) * 64 + lane];
      af[stg][1] = xs[(1 * C_KCH + kc) * 64 + lane];
      wf[stg][0] = wl[(0 * C_KCH + kc) * 64];
      if constexpr (C_KCH + kc < C_WFR) wf[stg][1] = wl[(1 * C_KCH + kc) * 64];
      else wf[stg][1] = wo_last;
    };
    auto body = [&](auto kcv) {
      constexpr int kc = decltype(kcv)::value, stg = kc & 1;
      if constexpr (kc + 1 < C_KCH) frag_fetch(std::integral_constant<int, kc + 1>{}, stg ^ 1);
      __builtin_amdgcn_sched_barrier(0);
      slot(kcv);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        P[0][cc][1] = mfma16(af[stg][0], wreg[0][cc][kc], P[0][cc][1]);
        P[1][cc][1] = mfma16(af[stg][1], wreg[0][cc][kc], P[1][cc][1]);
        P[0][cc][2] = mfma16(af[stg][0], wreg[1][cc][kc], P[0][cc][2]);
        P[1][cc][2] = mfma16(af[stg][1], wreg[1][cc][kc], P[1][cc][2]);
        P[0][cc][0] = mfma16(af[stg][0], wf[stg][cc], P[0][cc][0]);
        P[1][cc][0] = mfma16(af[stg][1], wf[stg][cc], P[1][cc][0]);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    CL2_STAMP(0);
    frag_fetch(std::integral_constant<int, 0>{}, 0);
    __builtin_amdgcn_s_setprio(1);
    body(std::integral_constant<int, 0>{});
    body(std::integral_constant<int, 1>{});
    body(std::integral_constant<int, 2>{});
    body(std::integral_constant<int, 3>{});
    body(std::integral_constant<int, 4>{});
    body(std::integral_constant<int, 5>{});
    body(std::integral_constant<int, 6>{});
    body(std::integral_constant<int, 7>{});
    CL2_STAMP(1);
    body(std::integral_constant<int, 8>{});
    CL2_STAMP(2);
    body(std::integral_constant<int, 9>{});
    body(std::integral_constant<int, 10>{});
    body(std::integral_constant<int, 11>{});
    body(std::integral_constant<int, 12>{});
    body(std::integral_constant<int, 13>{});
    body(std::integral_constant<int, 14>{});
    body(std::integral_constant<int, 15>{});
    __builtin_amdgcn_s_setprio(0);
    CL2_STAMP(3);
    // the exchange stores of the previous pair-step went out in slot 1: once they have landed, publish them
    vm_wait_plain<NST - 2 + 8>();
    sstore4_dev((dreal && dmore) ? flag_base(dpl) : bin, (unsigned)((4 * m + vu) * 4), dt + 1);   // (every lane the same word)

    CL2_STAMP(4);
    // ---- epilogue ----
    const bool more = t + 1 < T;
#pragma unroll
    for (int tl = 0; tl < 2; ++tl) {
      // previous state: the lane loaded eight neurons of row 4q+j4; the quad turns that into rows 4q+e of its own two
      unsigned pl0[4], pl1[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // (through named floats: a bit cast applied directly to a vector element reads the wrong lanes)
        const float e0 = L[tl][i >> 1][(i & 1) * 2 + 0], e1 = L[tl][i >> 1][(i & 1) * 2 + 1];
        pl0[i] = __builtin_bit_cast(unsigned, e0);
        pl1[i] = __builtin_bit_cast(unsigned, e1);
      }
      quad_transpose(pl0, j4);
      quad_transpose(pl1, j4);
      float rn[4][2], dv[4][2];
      const f32x4 ga = *reinterpret_cast<const f32x4*>(gl + (16 * tl + 4 * q) * 2);       // rows 4q, 4q+1
      const f32x4 gb = *reinterpret_cast<const f32x4*>(gl + (16 * tl + 4 * q + 2) * 2);   // rows 4q+2, 4q+3
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float g0 = e < 2 ? ga[2 * e] : gb[2 * (e - 2)], g1 = e < 2 ? ga[2 * e + 1] : gb[2 * (e - 2) + 1];
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
          const float x = fmaf(g1, P[tl][cc][2][e], fmaf(g0, P[tl][cc][1][e], P[tl][cc][0][e]));
          float aF, aD;
          act_scaled<ACT>(x, asc, aF, aD);
          const float ro = __builtin_bit_cast(float, cc ? pl1[e] : pl0[e]);
          rn[e][cc] = fmaf(oma, ro, aF);
          dv[e][cc] = aD;
        }
      }
      if (SAVE && t == 0) {
        // slot 0 of the operand copy is the initial state
        const char* base = reinterpret_cast<const char*>(p.rfrag) + (((size_t)0 * nbt + 2 * pr + tl) * 32 + 8 * m) * 64 * 16;
        const bf16x4 k0 = {(__bf16)__builtin_bit_cast(float, pl0[0]), (__bf16)__builtin_bit_cast(float, pl0[1]),
                           (__bf16)__builtin_bit_cast(float, pl0[2]), (__bf16)__builtin_bit_cast(float, pl0[3])};
        const bf16x4 k1 = {(__bf16)__builtin_bit_cast(float, pl1[0]), (__bf16)__builtin_bit_cast(float, pl1[1]),
                           (__bf16)__builtin_bit_cast(float, pl1[2]), (__bf16)__builtin_bit_cast(float, pl1[3])};
        sstore8<0>(base, r_lane, __builtin_bit_cast(f32x2, k0));
        sstore8<1024>(base, r_lane, __builtin_bit_cast(f32x2, k1));
      }
      // hold the results back in the form they are stored in
      {
        unsigned h0[4], h1[4], xe[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          h0[e] = __builtin_bit_cast(unsigned, rn[e][0]);
          h1[e] = __builtin_bit_cast(unsigned, rn[e][1]);
          const bf16x2 pk = {(__bf16)rn[e][0], (__bf16)rn[e][1]};
          xe[e] = __builtin_bit_cast(unsigned, pk);
        }
        quad_transpose(h0, j4);
        quad_transpose(h1, j4);
        quad_transpose(xe, j4);
        dh[tl][0] = f32x4{__builtin_bit_cast(float, h0[0]), __builtin_bit_cast(float, h1[0]), __builtin_bit_cast(float, h0[1]),
                          __builtin_bit_cast(float, h1[1])};
        dh[tl][1] = f32x4{__builtin_bit_cast(float, h0[2]), __builtin_bit_cast(float, h1[2]), __builtin_bit_cast(float, h0[3]),
                          __builtin_bit_cast(float, h1[3])};
        dx[tl] = f32x4{__builtin_bit_cast(float, xe[0]), __builtin_bit_cast(float, xe[1]), __builtin_bit_cast(float, xe[2]),
                       __builtin_bit_cast(float, xe[3])};
      }
      if constexpr (SAVE) {
        typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
        const f16x8 dk = {(_Float16)dv[0][0], (_Float16)dv[1][0], (_Float16)dv[2][0], (_Float16)dv[3][0],
                          (_Float16)dv[0][1], (_Float16)dv[1][1], (_Float16)dv[2][1], (_Float16)dv[3][1]};
        dd16[tl] = __builtin_bit_cast(f32x4, dk);
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
          const bf16x4 pk = {(__bf16)rn[0][cc], (__bf16)rn[1][cc], (__bf16)rn[2][cc], (__bf16)rn[3][cc]};
          dr[tl][cc] = __builtin_bit_cast(f32x2, pk);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    dreal = true;
    dmore = more;
    dt = t;
    dpr = pr;
    dpl = pl;

    CL2_STAMP(5);
    // ---- the next pair-step's operand and gates into LDS ----
    lds_barrier();
    CL2_STAMP(6);   // every wave has finished with the operand and the gates of this pair-step
    // Whatever the slots fetched has landed after this wait, wanted or not.  (One wait, in straight-line code: a wait
    // inside the branches below would have the compiler copy the registers into place in front of it, in flight.)
    vm_wait_x<1>(sreg);
    CL2_STAMP(7);
    if (!have_next) break;
    if (nt == 0) {
      stage_from_r_init(npr);
    } else {
      if (up) {
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) xs[v * 512 + jj * 64 + lane] = __builtin_bit_cast(bf16x8, sreg[jj]);
      } else {
        // nothing valid was fetched ahead (the producers of this operand were not done when slot 8 looked, or
        // this is the cluster's only pair): publish what is still held back, then wait for the flags
        emit_all();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (dmore) sstore4_dev(flag_base(dpl), (unsigned)((4 * m + vu) * 4), dt + 1);
        dreal = false;
        bool ok = false;
        for (int spins = 0; spins <= c.spin_max; ++spins) {
          const int f = flag_load(c.flags + ((size_t)cl * c.ppc + npl) * 16 + n);
          if ((ok = (__ballot(f < nt) == 0))) break;
          __builtin_amdgcn_s_sleep(2);
        }
        if (!ok && lane == 0) {
          misc[0] = 1;
          *c.host_err = RING_CLUSTER_ERR_WAIT;
        }
        // ordinary loads behind a device-scope acquire (which drops the vector L1's lines): the compiler waits for them
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const bf16x8* xb = reinterpret_cast<const bf16x8*>(x_base(nt, npr));
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) xs[v * 512 + jj * 64 + lane] = xb[jj * 64 + lane];
      }
    }
    if (v == 0) gl[lane] = gnext;
    CL2_STAMP(8);
    lds_barrier();
    CL2_STAMP(9);
    CL2_FLUSH();
    if (misc[0]) return;
    t = nt;
    pl = npl;
  }
  emit_all();   // the last pair-step's results (its state is nobody's operand)
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
  g.flag_bytes = c_align((size_t)g.nclusters * g.ppc * 16 * sizeof(int));
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

bool ring_cluster_applicable(int N, int k) { return N > 256 && N <= 512 && k == 2; }

size_t ring_cluster_workspace_bytes(int nbt) {
  const ClusterGeo g = cluster_geo(nbt);
  return g.xchg_bytes + g.flag_bytes + g.hello_bytes;
}

int ring_cluster_error() { return g_host_err ? *(volatile int*)g_host_err : 0; }

// RINGATTR_CLUSTER=1 / 0 switches the cluster kernel on / off where it applies.
bool ring_uses_cluster(int N, int k, int nbt) {
  if (!ring_cluster_applicable(N, k)) return false;
  const char* v = getenv("RINGATTR_CLUSTER");
  if (!(v && v[0] == '1')) return false;
  if (ring_cluster_error()) return false;
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = -1;
    cus = n;
  }
  return cluster_geo(nbt).grid <= cus;   // every workgroup needs a compute unit of its own, all at once
}

template <int ACT>
static hipError_t launch_fwd_cluster_act(const RingFwdArgs& a, const RingClusterArgs& c, int grid, hipStream_t st) {
  const bool full = a.N == 512 && a.B % 32 == 0;
  auto go = [&](auto kern) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)C_LDS_BYTES);
    if (e != hipSuccess) return e;
    RING_LAUNCH(kern, dim3(grid), dim3(256), C_LDS_BYTES, st, a, c);
    return hipGetLastError();
  };
  static const bool burst = [] { const char* v = getenv("RINGATTR_CLUSTER_BURST"); return v && v[0] == '1'; }();
  if (full && !burst && a.T <= (1 << 20))
    return a.dfrag ? go(ring_fwd_cluster_full_kernel<ACT, true>) : go(ring_fwd_cluster_full_kernel<ACT, false>);
  if (a.dfrag) return full ? go(ring_fwd_cluster_kernel<ACT, true, true>) : go(ring_fwd_cluster_kernel<ACT, true, false>);
  return full ? go(ring_fwd_cluster_kernel<ACT, false, true>) : go(ring_fwd_cluster_kernel<ACT, false, false>);
}

hipError_t ring_launch_fwd_cluster(const RingFwdArgs& a, hipStream_t st) {
  if (!a.cluster_ws || !ring_cluster_applicable(a.N, a.k) || !a.hist) return hipErrorInvalidValue;
  const ClusterGeo g = cluster_geo(a.nbt);
  RingClusterArgs c;
  char* ws = static_cast<char*>(a.cluster_ws);
  c.xchg = ws;
  c.flags = reinterpret_cast<int*>(ws + g.xchg_bytes);
  c.hello = reinterpret_cast<int*>(ws + g.xchg_bytes + g.flag_bytes);
  hipError_t e = host_err_word(&c.host_err);
  if (e != hipSuccess) return e;
  c.npairs = g.npairs;
  c.nclusters = g.nclusters;
  c.ppc = g.ppc;
  c.spin_max = 4000000;
  if (const char* v = getenv("RINGATTR_CLUSTER_SPIN")) {
    const long s = atol(v);
    if (s >= 0 && s <= 100000000L) c.spin_max = (int)s;
  }
  const int nclear = (int)((g.flag_bytes + g.hello_bytes) / sizeof(int));
  hipLaunchKernelGGL(ring_cluster_clear_kernel, dim3((nclear + 255) / 256), dim3(256), 0, st, c.flags, nclear);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  switch (a.act) {
    case ACT_RELU: return launch_fwd_cluster_act<ACT_RELU>(a, c, g.grid, st);
    case ACT_GELU: return launch_fwd_cluster_act<ACT_GELU>(a, c, g.grid, st);
    case ACT_TANH: return launch_fwd_cluster_act<ACT_TANH>(a, c, g.grid, st);
    case ACT_SILU: return launch_fwd_cluster_act<ACT_SILU>(a, c, g.grid, st);
    default: return hipErrorInvalidValue;
  }
}
