// Shared device helpers for the gfx950 ring-attractor kernels: vector types, tile geometry,
// activation math, LDS operand exchange, and the private "tile order" used for side buffers.
//
// Tile geometry (all kernels).  A workgroup is 4 wavefronts (256 lanes) and owns 16 batch rows.
// Neurons are padded to NPAD = 64*NC; wave w owns the 16*NC contiguous neurons starting at
// 16*NC*w and splits them into NC MFMA column tiles of 16: tile c, column n <-> neuron
// 16*NC*w + NC*n + c.  A lane (q = lane/16, n = lane%16) therefore holds, after a 16x16 MFMA,
// batch rows 4q..4q+3 of NC CONSECUTIVE neurons -- which makes the fp32 history stores, the bf16
// operand write-back and the side-buffer stores all contiguous per lane.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

enum : int { ACT_RELU = 0, ACT_GELU = 1, ACT_TANH = 2, ACT_SILU = 3 };  // cpp/cuda_common.cuh:56

template <int NC_>
struct Tile {
  static constexpr int NC = NC_;
  static constexpr int NPAD = 64 * NC;          // padded neuron count
  static constexpr int KCH = 2 * NC;            // K chunks of 32 along the contraction
  static constexpr int KG = KCH < 8 ? KCH : 8;  // chunks staged per register group
  static constexpr int NKG = KCH / KG;
  static constexpr int GW = (NC % 4 == 0) ? 4 : ((NC % 2 == 0) ? 2 : 1);  // LDS write granule
  static constexpr int SLOTS = KCH * 4 * 17;    // 16-byte operand slots per LDS buffer (padded groups)
};

// Operand-buffer groups (one per (K chunk, q)) hold 16 row slots and are spaced 17 slots apart: the
// 8-byte write-back of a wave then spreads over all banks (2-way, the minimum for 512 bytes) instead
// of landing 8-way on the same ones.
constexpr int XG = 17;

// Neuron ownership of the pipelined NC = 4 forward.  Its eight waves (w = 0..3, h = 0 "early" / 1 "late") each
// own two column tiles; tile cc, column n of wave (w,h) is neuron 64*w + 32*h + 2*n + cc, so the 16 lanes of an
// MFMA row group hold 32 consecutive neurons and a history store writes whole 128-byte lines.  The contraction
// index follows the same order, early waves first: position 128*h + 32*w + 2*n + cc <-> that neuron, which puts
// a wave's tile pair into one K chunk.  (The saved buffers keep the common tile order; see split_common_slot.)
__host__ __device__ __forceinline__ int split_k_neuron(int kappa) {
  const int h = kappa >> 7, s = kappa & 127;
  return 64 * (s >> 5) + 32 * h + (s & 31);
}

// Where the common tile order (tile c, column n <-> neuron 64*w + 4*n + c) keeps neuron 64*w + 32*h + 2*n + cc:
// column 8*h + n/2 of tile 2*(n%2) + cc.
__host__ __device__ __forceinline__ void split_common_slot(int h, int n, int cc, int& tile, int& col) {
  tile = 2 * (n & 1) + cc;
  col = 8 * h + (n >> 1);
}

// D = A(16x32 bf16) * B(32x16 bf16) + C(16x16 fp32).  Lane (q,n): A row n, B column n, both with
// K slots 8q..8q+7; C/D rows 4q..4q+3 of column n.
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the vector-memory
// counter, i.e. it would stall every time step on the HBM acknowledgement of that step's history
// stores; the recurrence only exchanges data through LDS, so waiting for lgkmcnt is sufficient.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// F(x) and F'(x).  gelu is the exact erf form (train/train_ring_attractor.py:16) and its derivative
// uses the normal density 1/sqrt(2*pi) as the torch path does (legacy/bwd_fp32.py:455-457).
// Branch-free activation pairs (F, F') for the per-step critical path of every recurrence kernel.
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
    const float th = fmaf(-2.f, __builtin_amdgcn_rcpf(e2 + 1.f), 1.f);
    F = th;
    D = fmaf(-th, th, 1.f);                       // written as one fused operation: the same bits in every kernel
  } else {
    const float xc = fmaxf(x, -87.f);
    const float s = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(xc * -1.44269504f));
    F = x * s;
    D = s * fmaf(x, 1.f - s, 1.f);
  }
}

// alpha * F(x) and alpha * F'(x) with alpha folded into the constants: what the leak update
// r' = (1 - alpha) r + alpha F(re) and the saved derivative record alpha * F'(re) need, in fewer vector
// instructions than scaling act_fast's results afterwards.  Same approximations as act_fast.
struct ActScale {
  float a, g0, g1, g2, g3, g4, gd;   // alpha; gelu: alpha/2 * erfc polynomial coefficients, alpha / sqrt(2 pi)
};

__device__ __forceinline__ ActScale act_scale_make(float alpha) {
  ActScale s;
  s.a = alpha;
  s.g4 = 0.5f * alpha * 1.061405429f;
  s.g3 = 0.5f * alpha * -1.453152027f;
  s.g2 = 0.5f * alpha * 1.421413741f;
  s.g1 = 0.5f * alpha * -0.284496736f;
  s.g0 = 0.5f * alpha * 0.254829592f;
  s.gd = alpha * 0.39894228f;
  return s;
}

template <int ACT>
__device__ __forceinline__ void act_scaled(float x, const ActScale& k, float& aF, float& aD) {
  if constexpr (ACT == ACT_RELU) {
    aF = k.a * fmaxf(x, 0.f);
    aD = x > 0.f ? k.a : 0.f;
  } else if constexpr (ACT == ACT_GELU) {
    const float t = __builtin_amdgcn_rcpf(fmaf(fabsf(x), 0.3275911f * 0.70710678f, 1.f));
    const float e = __builtin_amdgcn_exp2f(x * x * -0.72134752f);   // exp(-x^2/2)
    float poly = fmaf(t, k.g4, k.g3);
    poly = fmaf(t, poly, k.g2);
    poly = fmaf(t, poly, k.g1);
    poly = fmaf(t, poly, k.g0);
    const float h = poly * t * e;                 // alpha * Phi(-|x|)
    const float cdf = x >= 0.f ? k.a - h : h;     // alpha * Phi(x)
    aF = x * cdf;
    aD = fmaf(x * e, k.gd, cdf);
  } else if constexpr (ACT == ACT_TANH) {
    const float xc = __builtin_amdgcn_fmed3f(x, -15.f, 15.f);
    const float e2 = __builtin_amdgcn_exp2f(xc * 2.88539008f);      // exp(2x)
    const float th = fmaf(-2.f, __builtin_amdgcn_rcpf(e2 + 1.f), 1.f);
    aF = k.a * th;
    aD = fmaf(-th, aF, k.a);
  } else {
    const float xc = fmaxf(x, -87.f);
    const float s = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(xc * -1.44269504f));
    const float as = k.a * s;
    aF = x * as;
    aD = as * fmaf(x, 1.f - s, 1.f);
  }
}

// Sum over the 16 lanes that share q (one MFMA column group); every lane gets the total.
__device__ __forceinline__ float row16_sum(float v) {
  v += __shfl_xor(v, 1, 16);
  v += __shfl_xor(v, 2, 16);
  v += __shfl_xor(v, 4, 16);
  v += __shfl_xor(v, 8, 16);
  return v;
}

// The same sum with data-parallel-primitive adds (no LDS traffic): butterfly inside each row of 16 lanes.
__device__ __forceinline__ float row16_sum_dpp(float v) {
#define RING_DPP_ADD(CTRL) \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false))
  RING_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
  RING_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
  RING_DPP_ADD(0x141);   // row_half_mirror
  RING_DPP_ADD(0x140);   // row_mirror
#undef RING_DPP_ADD
  return v;
}

// LDS operand buffer: slot(kc,q,b) = (kc*4+q)*XG + b holds the 8 bf16 values
// x[b][32kc+8q .. +7]; an MFMA A-operand read by lane (q,b) is slot(kc,q,b): each group of 16 lanes
// reads 256 contiguous bytes.  This writes the lane's [4 rows][NC neurons] fp32 values as bf16.
template <int NC>
__device__ __forceinline__ void write_operand(bf16x8* xb, const float (&v)[4][NC], int w, int q, int n) {
  constexpr int G = Tile<NC>::GW;
  char* base = reinterpret_cast<char*>(xb);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int b = 4 * q + e;
#pragma unroll
    for (int c0 = 0; c0 < NC; c0 += G) {
      const int j = 16 * NC * w + NC * n + c0;
      const int slot = (((j >> 5) * 4 + ((j >> 3) & 3)) * XG + b);
      char* dst = base + slot * 16 + (j & 7) * 2;
      if constexpr (G == 4) {
        bf16x4 pk = {(__bf16)v[e][c0], (__bf16)v[e][c0 + 1], (__bf16)v[e][c0 + 2], (__bf16)v[e][c0 + 3]};
        *reinterpret_cast<bf16x4*>(dst) = pk;
      } else if constexpr (G == 2) {
        bf16x2 pk = {(__bf16)v[e][c0], (__bf16)v[e][c0 + 1]};
        *reinterpret_cast<bf16x2*>(dst) = pk;
      } else {
        *reinterpret_cast<__bf16*>(dst) = (__bf16)v[e][c0];
      }
    }
  }
}

// Saved F' (fp16) uses the lane order of the recurrence kernels,
//   S[t][bt][w][lane][c][e],  element = X[t][16*bt + 4q + e][16*NC*w + NC*n + c],
// so the forward writes and the BPTT reads 8*NC contiguous bytes per lane.
template <int NC>
__device__ __forceinline__ size_t side_offset(int t, int nbt, int bt, int w, int lane) {
  return ((((size_t)t * nbt + bt) * 4 + w) * 64 + lane) * (size_t)(4 * NC);
}

template <int NC, typename V4, typename S>
__device__ __forceinline__ void side_store(S* dst, const float (&v)[4][NC]) {
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    V4 pk = {(S)v[0][c], (S)v[1][c], (S)v[2][c], (S)v[3][c]};
    *reinterpret_cast<V4*>(dst + 4 * c) = pk;
  }
}

template <int NC>
__device__ __forceinline__ void side_load_f16(const _Float16* src, float (&v)[4][NC]) {
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    f16x4 pk = *reinterpret_cast<const f16x4*>(src + 4 * c);
    v[0][c] = (float)pk[0];
    v[1][c] = (float)pk[1];
    v[2][c] = (float)pk[2];
    v[3][c] = (float)pk[3];
  }
}

// The bf16 operand copies of r_prev and g feed the weight-gradient GEMM, whose MFMA K index runs
// over samples.  They are stored tile-major with two time steps paired,
//   P[t/2][bt][tile][lane][t%2][e],  tile = w*NC + c,  16 bytes per (pair, bt, tile, lane),
// i.e. exactly one MFMA operand fragment (K slot 8q + 4*(t%2) + e) per lane: a column tile of a K
// chunk is 1 KiB contiguous and goes global -> LDS -> MFMA without any transpose or repacking.
template <int NC>
__device__ __forceinline__ size_t pair_offset(int t, int nbt, int bt, int tile, int lane) {
  return (((((size_t)(t >> 1) * nbt + bt) * (4 * NC) + tile) * 64 + lane) * 2 + (t & 1)) * 4;
}

template <int NC>
__device__ __forceinline__ void pair_store(__bf16* base, int t, int nbt, int bt, int w, int lane, const float (&v)[4][NC]) {
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    bf16x4 pk = {(__bf16)v[0][c], (__bf16)v[1][c], (__bf16)v[2][c], (__bf16)v[3][c]};
    *reinterpret_cast<bf16x4*>(base + pair_offset<NC>(t, nbt, bt, w * NC + c, lane)) = pk;
  }
}

// With an odd sequence length the second half of the last pair has no time step; the writer of
// the buffer zeroes it so that readers need no special case.
template <int NC>
__device__ __forceinline__ void pair_zero_tail(__bf16* base, int T, int nbt, int bt, int w, int lane) {
  if ((T & 1) == 0) return;
  const bf16x4 z = {(__bf16)0.f, (__bf16)0.f, (__bf16)0.f, (__bf16)0.f};
#pragma unroll
  for (int c = 0; c < NC; ++c) *reinterpret_cast<bf16x4*>(base + pair_offset<NC>(T, nbt, bt, w * NC + c, lane)) = z;
}

// Masked fp32 [rows][N] <-> lane registers.  slab points at row 0 of a [B][N] matrix.
template <int NC>
__device__ __forceinline__ void rows_load(const float* slab, int N, int B, int b0, int i0, float (&v)[4][NC]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int b = b0 + e;
    if constexpr (NC % 4 == 0) {
      if ((N & 3) == 0 && i0 + NC <= N && b < B) {
        const float* row = slab + (size_t)b * N + i0;
#pragma unroll
        for (int c = 0; c < NC; c += 4) {
          f32x4 pk = *reinterpret_cast<const f32x4*>(row + c);
          v[e][c] = pk[0];
          v[e][c + 1] = pk[1];
          v[e][c + 2] = pk[2];
          v[e][c + 3] = pk[3];
        }
        continue;
      }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int i = i0 + c;
      v[e][c] = (b < B && i < N) ? slab[(size_t)b * N + i] : 0.f;
    }
  }
}

template <int NC>
__device__ __forceinline__ void rows_store(float* slab, int N, int B, int b0, int i0, const float (&v)[4][NC]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int b = b0 + e;
    if (b >= B) continue;
    float* row = slab + (size_t)b * N + i0;
    if constexpr (NC % 4 == 0) {
      // rows start 16-byte aligned when N % 4 == 0 (i0 is a multiple of NC)
      if ((N & 3) == 0 && i0 + NC <= N) {
#pragma unroll
        for (int c = 0; c < NC; c += 4) {
          f32x4 pk = {v[e][c], v[e][c + 1], v[e][c + 2], v[e][c + 3]};
          *reinterpret_cast<f32x4*>(row + c) = pk;
        }
        continue;
      }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c)
      if (i0 + c < N) row[c] = v[e][c];
  }
}
