// Fused decode + loss head over the state history, forward and backward.
//
// The training script turns bump_history [T,B,N] into a loss with a chain of full-size tensor ops
// (root train_general_ring_no_gain.py:113-116, 324-330; train/train_ring_attractor.py:190-220, 275-298):
//   proj = r @ W_delta7,  W_delta7[i][j] = cos(phi_i - phi_j),  phi_i = 2*pi*i/N
//   out  = proj / max_j proj
//   x = sum_j out_j cos(pa_j),  y = sum_j out_j sin(pa_j),  pa = linspace(0, 2*pi, N)   (end point included)
//   theta = atan2(y, x);  cos-sim loss = mean_{b,t} (cos theta - cos a)^2 + (sin theta - sin a)^2
//   amplitude loss = mean_{b,t} (sum_i |r_i| - target_b)^2,  target_b = sum_i |r_{t=0,i}| unless given
// W_delta7 has rank two: proj_j = C cos(phi_j) + S sin(phi_j) with C = sum_i r_i cos(phi_i),
// S = sum_i r_i sin(phi_i).  The positive row maximum cancels in atan2, so
//   theta = atan2(C*b1 + S*b2, C*a1 + S*a2),  a1 = sum_j cos(phi_j)cos(pa_j), a2 = sum_j sin(phi_j)cos(pa_j),
//                                             b1 = sum_j cos(phi_j)sin(pa_j), b2 = sum_j sin(phi_j)sin(pa_j)
// and everything a row contributes is three sums over its N values.  Forward: one pass over the
// history (three sums per row, loss partials in a fixed order).  Backward: one more pass that
// writes d loss / d r_i = kc cos(phi_i) + ks sin(phi_i) + beta sign(r_i) per row.  Both are pure
// HBM streams: 4N bytes read per row forward, 4N read + 4N written backward.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

namespace {

constexpr int L_ROWS_PER_BLOCK = 4;      // one wave per row at a time, four waves per workgroup
constexpr int L_MAXCH = 8;               // 256-element chunks per row held as per-lane constants (N <= 2048)

struct LossConsts {
  float a1, a2, b1, b2;
};

// Sum over the 64 lanes, result in every lane: butterfly inside each row of 16 lanes with DPP (no LDS
// traffic), then the four row totals through scalar registers.
__device__ __forceinline__ float wave_sum(float v) {
#define RING_DPP_ADD(CTRL) \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false))
  RING_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
  RING_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
  RING_DPP_ADD(0x141);   // row_half_mirror
  RING_DPP_ADD(0x140);   // row_mirror
#undef RING_DPP_ADD
  const int i = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 48));
  return (r0 + r1) + (r2 + r3);
}

// Element i of a row lives in lane (i / 4) % 64, slot i % 4 of chunk i / 256.
template <int NCH>
struct RowLanes {
  float cs[NCH][4], sn[NCH][4];
  __device__ __forceinline__ void init(int N, int lane) {
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int i = ch * 256 + lane * 4 + x;
        float s, c;
        sincosf(6.283185307179586f * (float)i / (float)N, &s, &c);
        cs[ch][x] = i < N ? c : 0.f;
        sn[ch][x] = i < N ? s : 0.f;
      }
  }
};

template <int NCH, bool VEC>
__device__ __forceinline__ void row_load(const float* row, int N, int lane, float (&v)[NCH][4]) {
#pragma unroll
  for (int ch = 0; ch < NCH; ++ch) {
    const int i0 = ch * 256 + lane * 4;
    if constexpr (VEC) {
      if (i0 < N) {
        const f32x4 p = *reinterpret_cast<const f32x4*>(row + i0);
        v[ch][0] = p[0]; v[ch][1] = p[1]; v[ch][2] = p[2]; v[ch][3] = p[3];
      } else {
        v[ch][0] = v[ch][1] = v[ch][2] = v[ch][3] = 0.f;
      }
    } else {
#pragma unroll
      for (int x = 0; x < 4; ++x) v[ch][x] = i0 + x < N ? row[i0 + x] : 0.f;
    }
  }
}

// stats[row] = (C, S, sum |r|, -); row = t*B + b.  A pure stream: three sums per row, nothing else.
template <int NCH, bool VEC>
__global__ __launch_bounds__(256) void ring_loss_stats_kernel(const float* __restrict__ hist, f32x4* __restrict__ stats, int N,
                                                              int T, int B) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  RowLanes<NCH> ph;
  ph.init(N, lane);
  const long rows = (long)T * B;
  // two rows per trip, so that two row loads are in flight per wave.  The sweep runs from the last row to the
  // first: the forward kernel has just written the history in time order, so its tail is what the memory-side
  // cache still holds.
  const long stride = (long)gridDim.x * L_ROWS_PER_BLOCK;
  for (long it = (long)blockIdx.x * L_ROWS_PER_BLOCK + wv; it < rows; it += 2 * stride) {
    const long row = rows - 1 - it;
    const long row2 = row - stride;
    const bool has2 = row2 >= 0;
    float v[2][NCH][4];
    row_load<NCH, VEC>(hist + row * N, N, lane, v[0]);
    row_load<NCH, VEC>(hist + (has2 ? row2 : row) * N, N, lane, v[1]);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float C = 0.f, S = 0.f, A = 0.f;
#pragma unroll
      for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          C = fmaf(v[h][ch][x], ph.cs[ch][x], C);
          S = fmaf(v[h][ch][x], ph.sn[ch][x], S);
          A += fabsf(v[h][ch][x]);
        }
      C = wave_sum(C);
      S = wave_sum(S);
      A = wave_sum(A);
      if (lane == 0 && (h == 0 || has2)) stats[h == 0 ? row : row2] = f32x4{C, S, A, 0.f};
    }
  }
}

// Per batch row, then per (t, b), in one launch.  A workgroup takes 16 batch rows at a time (sixteen threads per row
// stride over t):
//  1. target amplitude of the row, sum over t of the deviations (what flows into the target) and of their squares,
//     combined over the sixteen threads in a fixed order;
//  2. the decode and everything transcendental for the same rows: stats[row] is replaced by the row's gradient
//     coefficients (kc, ks, beta, theta), all still without the 1/(T*B) and upstream factors:
//       d total / d r_i = kc cos(phi_i) + ks sin(phi_i) + beta sign(r_i).
// partial[block] = sum of the block's cos-sim terms (fixed order); sq[b] = the row's sum of squared deviations.
__global__ __launch_bounds__(256) void ring_loss_decode_kernel(f32x4* __restrict__ stats, const float* __restrict__ angle,
                                                               const float* __restrict__ target_amp, float* __restrict__ sq,
                                                               float* __restrict__ partial, LossConsts k, float bump_weight,
                                                               int T, int B) {
  __shared__ float pd[16][16], ps[16][16];
  __shared__ float tg[16], ds[16];
  __shared__ float red[256];
  const int bi = threadIdx.x & 15, tl = threadIdx.x >> 4;
  const int groups = (B + 15) / 16;
  float acc = 0.f;
  for (int bg = blockIdx.x; bg < groups; bg += gridDim.x) {
    const int b = bg * 16 + bi, bc = b < B ? b : B - 1;
    const float target = target_amp ? target_amp[bc] : stats[bc][2];   // row t = 0 is stats[0*B + b]
    float d = 0.f, s = 0.f;
    for (int t = tl; t < T; t += 16) {
      const float dev = stats[(size_t)t * B + bc][2] - target;
      d += dev;
      s = fmaf(dev, dev, s);
    }
    pd[tl][bi] = d;
    ps[tl][bi] = s;
    __syncthreads();
    if (tl == 0) {
      float dd = 0.f, ss = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        dd += pd[j][bi];
        ss += ps[j][bi];
      }
      tg[bi] = target;
      ds[bi] = dd;
      if (b < B) sq[b] = ss;
    }
    __syncthreads();
    if (b < B) {
      const float tgt = tg[bi], dsum = ds[bi];
      for (int t = tl; t < T; t += 16) {
        const size_t row = (size_t)t * B + b;
        const f32x4 st = stats[row];
        const float C = st[0], S = st[1];
        const float X = C * k.a1 + S * k.a2, Y = C * k.b1 + S * k.b2;
        const float theta = atan2f(Y, X);
        const float a = angle[(size_t)b * T + t];
        float sth, cth, sa, ca;
        sincosf(theta, &sth, &cth);
        sincosf(a, &sa, &ca);
        acc += (cth - ca) * (cth - ca) + (sth - sa) * (sth - sa);
        // d/dtheta of (cos theta - cos a)^2 + (sin theta - sin a)^2 = 2 sin(theta - a)
        const float dth = 2.f * (sth * ca - cth * sa) / fmaxf(X * X + Y * Y, 1e-30f);
        // amplitude term: 2 (amp_t - target); the target (first step, unless given) collects minus the sum over t
        float beta = 2.f * (st[2] - tgt);
        if (!target_amp && t == 0) beta -= 2.f * dsum;
        stats[row] = f32x4{dth * (X * k.b1 - Y * k.a1), dth * (X * k.b2 - Y * k.a2), bump_weight * beta, theta};
      }
    }
    __syncthreads();          // pd / ps / tg / ds are reused by the next group of rows
  }
  red[threadIdx.x] = acc;
  __syncthreads();
  for (int o = 128; o >= 1; o >>= 1) {
    if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}

// out = (total, cos-sim loss, amplitude loss).  One workgroup: every thread sums a strided slice, the slices
// are combined by a fixed tree (bitwise repeatable).
__global__ __launch_bounds__(256) void ring_loss_final_kernel(const float* __restrict__ partial, int nparts,
                                                              const float* __restrict__ sq, int B, float inv_rows,
                                                              float bump_weight, float* __restrict__ out) {
  __shared__ double rc[256], ra[256];
  double c = 0.0, a = 0.0;
  for (int i = threadIdx.x; i < nparts; i += 256) c += partial[i];
  for (int i = threadIdx.x; i < B; i += 256) a += sq[i];
  rc[threadIdx.x] = c;
  ra[threadIdx.x] = a;
  __syncthreads();
  for (int o = 128; o >= 1; o >>= 1) {
    if ((int)threadIdx.x < o) {
      rc[threadIdx.x] += rc[threadIdx.x + o];
      ra[threadIdx.x] += ra[threadIdx.x + o];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float lc = (float)(rc[0] * inv_rows), la = (float)(ra[0] * inv_rows);
    out[0] = lc + bump_weight * la;
    out[1] = lc;
    out[2] = la;
  }
}

// grad[row][i] = up / (T*B) * (kc cos(phi_i) + ks sin(phi_i) + beta * sign(r_i)): a pure stream.
template <int NCH, bool VEC>
__global__ __launch_bounds__(256) void ring_loss_grad_kernel(const float* __restrict__ hist, const f32x4* __restrict__ coef,
                                                             const float* __restrict__ upstream, float* __restrict__ grad,
                                                             int N, int T, int B) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  RowLanes<NCH> ph;
  ph.init(N, lane);
  const long rows = (long)T * B;
  const float up = (upstream ? upstream[0] : 1.f) / (float)rows;
  const long stride = (long)gridDim.x * L_ROWS_PER_BLOCK;
  for (long row0 = (long)blockIdx.x * L_ROWS_PER_BLOCK + wv; row0 < rows; row0 += 2 * stride) {
    const bool has2 = row0 + stride < rows;
    float v[2][NCH][4];
    f32x4 cf[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const long row = (h == 1 && has2) ? row0 + stride : row0;
      cf[h] = coef[row];
      row_load<NCH, VEC>(hist + row * N, N, lane, v[h]);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (h == 1 && !has2) break;
      const long row = row0 + h * stride;
      const float kc = cf[h][0] * up, ks = cf[h][1] * up, beta = cf[h][2] * up;
#pragma unroll
      for (int ch = 0; ch < NCH; ++ch) {
        const int i0 = ch * 256 + lane * 4;
        float g[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const float r = v[h][ch][x];
          const float sg = r > 0.f ? 1.f : (r < 0.f ? -1.f : 0.f);
          g[x] = fmaf(kc, ph.cs[ch][x], fmaf(ks, ph.sn[ch][x], beta * sg));
        }
        float* dst = grad + row * N + i0;
        if constexpr (VEC) {
          if (i0 < N) *reinterpret_cast<f32x4*>(dst) = f32x4{g[0], g[1], g[2], g[3]};
        } else {
#pragma unroll
          for (int x = 0; x < 4; ++x)
            if (i0 + x < N) dst[x] = g[x];
        }
      }
    }
  }
}

LossConsts loss_consts(int N) {
  double a1 = 0, a2 = 0, b1 = 0, b2 = 0;
  for (int j = 0; j < N; ++j) {
    const double phi = 6.283185307179586476925 * j / N;
    const double pa = N > 1 ? 6.283185307179586476925 * j / (N - 1) : 0.0;
    a1 += cos(phi) * cos(pa);
    a2 += sin(phi) * cos(pa);
    b1 += cos(phi) * sin(pa);
    b2 += sin(phi) * sin(pa);
  }
  return LossConsts{(float)a1, (float)a2, (float)b1, (float)b2};
}

int loss_grid(long rows) {
  const long want = (rows + L_ROWS_PER_BLOCK - 1) / L_ROWS_PER_BLOCK;
  return (int)(want < 2048 ? want : 2048);
}

}  // namespace

size_t ring_loss_workspace_bytes(int T, int B) {
  const size_t rows = (size_t)T * B;
  return rows * sizeof(f32x4) + (size_t)3 * B * sizeof(float) + 2048 * sizeof(float) + 256;
}

#define LOSS_DISPATCH(CALL)                                                         \
  {                                                                                 \
    const int nch = (N + 255) / 256;                                                \
    const bool vec = (N % 4) == 0;                                                  \
    if (nch == 1 && vec) { constexpr int NCH = 1; constexpr bool VEC = true; CALL; } \
    else if (nch == 1) { constexpr int NCH = 1; constexpr bool VEC = false; CALL; } \
    else if (nch == 2 && vec) { constexpr int NCH = 2; constexpr bool VEC = true; CALL; } \
    else if (nch == 2) { constexpr int NCH = 2; constexpr bool VEC = false; CALL; } \
    else if (nch <= 4 && vec) { constexpr int NCH = 4; constexpr bool VEC = true; CALL; } \
    else if (nch <= 4) { constexpr int NCH = 4; constexpr bool VEC = false; CALL; } \
    else if (vec) { constexpr int NCH = L_MAXCH; constexpr bool VEC = true; CALL; } \
    else { constexpr int NCH = L_MAXCH; constexpr bool VEC = false; CALL; }         \
  }

struct LossWs {
  f32x4* stats;
  float *tgt, *dsum, *sq, *partial;
};

static LossWs carve(void* workspace, int T, int B) {
  LossWs w;
  char* p = (char*)workspace;
  w.stats = (f32x4*)p;
  p += (size_t)T * B * sizeof(f32x4);
  w.tgt = (float*)p;
  w.dsum = w.tgt + B;
  w.sq = w.dsum + B;
  w.partial = w.sq + B;
  return w;
}

// have_row_sums: the workspace's row-sum array (ring_loss_row_sums) is already filled (by the forward kernel); the
// pass over the history is skipped and `hist` is not read.
hipError_t ring_launch_loss_fwd(const float* hist, const float* angle, const float* target_amp, float bump_weight,
                                float* loss_out, int N, int T, int B, void* workspace, bool have_row_sums,
                                hipStream_t st) {
  if (N > 256 * L_MAXCH) return hipErrorInvalidValue;
  const LossWs w = carve(workspace, T, B);
  const LossConsts k = loss_consts(N);
  const long rows = (long)T * B;
  const int grid = loss_grid(rows);
  if (!have_row_sums) {
    LOSS_DISPATCH(hipLaunchKernelGGL((ring_loss_stats_kernel<NCH, VEC>), dim3(grid), dim3(256), 0, st, hist, w.stats, N, T, B));
  }
  const int dgrid = (B + 15) / 16 < 2048 ? (B + 15) / 16 : 2048;      // the workspace holds 2048 partial sums
  hipLaunchKernelGGL(ring_loss_decode_kernel, dim3(dgrid), dim3(256), 0, st, w.stats, angle, target_amp, w.sq, w.partial, k,
                     bump_weight, T, B);
  hipLaunchKernelGGL(ring_loss_final_kernel, dim3(1), dim3(256), 0, st, w.partial, dgrid, w.sq, B, 1.f / (float)rows,
                     bump_weight, loss_out);
  return hipGetLastError();
}

ring_f32x4* ring_loss_row_sums(void* workspace) {
  return reinterpret_cast<ring_f32x4*>(workspace);         // carve(): the per-row array leads the workspace
}

const ring_f32x4* ring_loss_row_coefficients(const void* workspace) {
  return reinterpret_cast<const ring_f32x4*>(workspace);   // carve(): the stats array leads the workspace
}

// The workspace must be the one ring_launch_loss_fwd filled for the same history: it holds the rows' coefficients.
hipError_t ring_launch_loss_bwd(const float* hist, const float* angle, const float* target_amp, float bump_weight,
                                const float* upstream, float* grad_hist, int N, int T, int B, const void* workspace,
                                hipStream_t st) {
  (void)angle;
  (void)target_amp;
  (void)bump_weight;
  if (N > 256 * L_MAXCH) return hipErrorInvalidValue;
  const LossWs w = carve(const_cast<void*>(workspace), T, B);
  const int grid = loss_grid((long)T * B);
  LOSS_DISPATCH(hipLaunchKernelGGL((ring_loss_grad_kernel<NCH, VEC>), dim3(grid), dim3(256), 0, st, hist, w.stats, upstream,
                                   grad_hist, N, T, B));
  return hipGetLastError();
}
