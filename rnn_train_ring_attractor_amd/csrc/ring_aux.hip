// Either side of the time loop, on the device: the synthetic input generator in front of it and the optimizer tail
// behind it.
//
// Input generator (utils/generate_av_integration_data.py:11-58, root train_general_ring_no_gain.py:176-229,
// train/train_ring_attractor.py:21-52 of the reference): angular-velocity trials, their integrated angle, the action
// signal and the initial bump, written where the time loop reads them, so that a training or benchmark step stages
// nothing from the host.  Per trial: the first n_initial_zeros steps are zero; of the remaining `rest` steps
// exactly rest - floor(rest * zero_ratio) randomly placed ones carry U(-max_av, max_av) draws (zero_ratio picked
// uniformly from a list); angle[0] = U(0, 2 pi), angle[t] = (angle[0] + sum_{s<t} av[s]) mod 2 pi.  The reference
// draws a random permutation per trial (argsort of uniform keys) and keeps the first n positions; choosing each
// position in turn with probability (still needed) / (still available) gives the same distribution over subsets
// (selection sampling) in one sequential pass, which the running sum for the angle needs anyway.  The random stream
// is this file's own counter-based generator (same distributions as the reference, not the same bits as torch's).
//
// Optimizer tail (root train_general_ring_no_gain.py:333-336: clip_grad_norm_(parameters, max_norm) then Adam.step()):
// the squared gradient norm over all tensors in a fixed order (two launches), then one launch that scales the
// gradients by min(1, max_norm / (norm + 1e-6)) and applies the Adam update to every tensor.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

namespace {

// splitmix64 finaliser over (seed, stream, counter): stateless, so any element can be drawn independently
__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ unsigned rand_u32(unsigned long long seed, unsigned stream, unsigned long long counter) {
  return (unsigned)(mix64(mix64(seed ^ ((unsigned long long)stream << 56)) + counter) >> 32);
}

__device__ __forceinline__ float rand_unit(unsigned long long seed, unsigned stream, unsigned long long counter) {
  return (float)(rand_u32(seed, stream, counter) >> 8) * (1.0f / 16777216.0f);   // [0, 1), 24 bits
}

}  // namespace

// av [B,T], angle [B,T], action [B,T,k].  A workgroup takes GEN_TRIALS trials through the sequence in chunks of
// GEN_TCH steps, in three phases per chunk: all threads draw the chunk's random numbers (the generator is stateless,
// so every (trial, step) draw is independent), one thread per trial walks its steps in order (selection sampling and
// the running angle are the only sequential parts: a compare, a subtract and an add per step), and all threads write
// the chunk out with consecutive threads on consecutive addresses.
namespace {
constexpr int GEN_TRIALS = 16;
constexpr int GEN_TCH = 128;
}  // namespace

__global__ __launch_bounds__(256) void ring_generate_trials_kernel(RingGenArgs p) {
  __shared__ float draw[GEN_TCH][GEN_TRIALS + 1];   // selection draw * positions left;  then the step's angle
  __shared__ float cand[GEN_TCH][GEN_TRIALS + 1];   // candidate velocity;               then the step's velocity
  const int tid = threadIdx.x, b0 = blockIdx.x * GEN_TRIALS;
  const int T = p.T, k = p.k;
  const int n0 = p.n_initial_zeros;
  const int rest = T - n0;
  const float two_pi = 6.283185307179586f;
  // per-trial state of the sequential phase (threads 0 .. GEN_TRIALS-1)
  const int bs = b0 + tid;
  float angle0 = 0.f, run = 0.f;                    // run: sum of av[s], s < t
  int need = 0;
  if (tid < GEN_TRIALS && bs < p.B) {
    angle0 = rand_unit(p.seed, 0, (unsigned long long)bs) * two_pi;
    const int pick = (int)(rand_u32(p.seed, 1, (unsigned long long)bs) % (unsigned)p.n_ratios);
    need = rest - (int)((float)rest * p.ratios[pick]);         // float32 product, truncated, as the reference
    need = need < 0 ? 0 : (need > rest ? rest : need);
  }
  for (int t0 = 0; t0 < T; t0 += GEN_TCH) {
    const int nt = T - t0 < GEN_TCH ? T - t0 : GEN_TCH;
    for (int idx = tid; idx < nt * GEN_TRIALS; idx += 256) {
      const int tl = idx / GEN_TRIALS, j = idx % GEN_TRIALS, b = b0 + j, t = t0 + tl;
      if (b < p.B) {
        const unsigned long long c = (unsigned long long)b * T + t;
        draw[tl][j] = rand_unit(p.seed, 2, c) * (float)(T - t);   // T - t positions are still available, this one included
        cand[tl][j] = (rand_unit(p.seed, 3, c) - 0.5f) * (2.f * p.max_av);
      }
    }
    __syncthreads();
    if (tid < GEN_TRIALS && bs < p.B) {
      for (int tl = 0; tl < nt; ++tl) {
        const int t = t0 + tl;
        float v = 0.f;
        if (t >= n0 && draw[tl][tid] < (float)need) {
          v = cand[tl][tid];
          --need;
        }
        float a = angle0 + run;
        a -= floorf(a / two_pi) * two_pi;                       // Python's %: result in [0, 2 pi)
        if (t == 0) a = angle0;
        cand[tl][tid] = v;
        draw[tl][tid] = a;
        run += v;
      }
    }
    __syncthreads();
    for (int idx = tid; idx < nt * GEN_TRIALS; idx += 256) {
      const int j = idx / nt, tl = idx % nt, b = b0 + j;
      if (b < p.B) {
        p.av[(size_t)b * T + t0 + tl] = cand[tl][j];
        p.angle[(size_t)b * T + t0 + tl] = draw[tl][j];
      }
    }
    for (int idx = tid; idx < nt * GEN_TRIALS * k; idx += 256) {
      const int c = idx % k, tl = (idx / k) % nt, j = idx / (k * nt), b = b0 + j;
      if (b >= p.B) continue;
      const float v = cand[tl][j];
      float out;
      if (p.spread) {
        const float scale = k > 1 ? -1.f + 2.f * (float)c / (float)(k - 1) : -1.f;   // linspace(-1, 1, k)
        out = fmaxf(v * scale, 0.f);
      } else {
        out = c == 0 ? fmaxf(-v, 0.f) : (c == 1 ? fmaxf(v, 0.f) : 0.f);
      }
      p.action[((size_t)b * T + t0 + tl) * k + c] = out;
    }
    __syncthreads();
  }
}

// One workgroup per trial: r_init[b][i] = bump(i; angle[b][0]) / its Euclidean norm.
// kind 0: exp(-d^2 / (2 w^2)), d the circular distance in neuron units to angle * N / (2 pi), w = N / param
// (train/train_ring_attractor.py:21-52); kind 1: von Mises, exp(param * cos(2 pi i / N - angle)).
__global__ __launch_bounds__(256) void ring_generate_bump_kernel(RingGenArgs p) {
  __shared__ float red[4];
  const int b = blockIdx.x, tid = threadIdx.x, N = p.N;
  const float a0 = p.angle[(size_t)b * p.T];
  const float two_pi = 6.283185307179586f;
  float ss = 0.f;
  for (int i = tid; i < N; i += 256) {
    float v;
    if (p.bump_kind == 0) {
      const float centre = a0 * (float)N / two_pi, w = (float)N / p.bump_param;
      const float d0 = fabsf((float)i - centre), d = fminf(d0, (float)N - d0);
      v = __expf(-(d * d) / (2.f * w * w));
    } else {
      v = __expf(p.bump_param * (cosf(two_pi * (float)i / (float)N - a0) - 1.f));   // scaled by exp(-kappa): cancels
    }
    p.r_init[(size_t)b * N + i] = v;
    ss = fmaf(v, v, ss);
  }
  ss = row16_sum_dpp(ss);
  {
    const int i = __builtin_bit_cast(int, ss);
    ss = (__builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 16))) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 48)));
  }
  if ((tid & 63) == 0) red[tid >> 6] = ss;
  __syncthreads();
  const float inv = 1.f / sqrtf((red[0] + red[1]) + (red[2] + red[3]));
  for (int i = tid; i < N; i += 256) p.r_init[(size_t)b * N + i] *= inv;
}

hipError_t ring_launch_generate(const RingGenArgs& a, hipStream_t st) {
  hipLaunchKernelGGL(ring_generate_trials_kernel, dim3((a.B + GEN_TRIALS - 1) / GEN_TRIALS), dim3(256), 0, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !a.r_init) return e;
  hipLaunchKernelGGL(ring_generate_bump_kernel, dim3(a.B), dim3(256), 0, st, a);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// clip_grad_norm_ + Adam
// ------------------------------------------------------------------------------------------------
namespace {
constexpr int OPT_BLOCK = 256;
constexpr int OPT_CHUNK = 4096;   // elements per workgroup
}  // namespace

// partial[blk] = sum of squares of the workgroup's chunk of the concatenated gradients (fixed order inside)
__global__ __launch_bounds__(OPT_BLOCK) void ring_gradnorm_partial_kernel(RingOptArgs p, float* partial) {
  __shared__ float red[OPT_BLOCK / 64];
  // which tensor does this workgroup's chunk belong to: chunks are dealt tensor after tensor
  int blk = blockIdx.x, ti = 0;
  while (ti < p.n && blk >= p.chunks[ti]) blk -= p.chunks[ti++];
  if (ti >= p.n) return;
  const float* g = p.grad[ti];
  const size_t lo = (size_t)blk * OPT_CHUNK, hi = lo + OPT_CHUNK < p.numel[ti] ? lo + OPT_CHUNK : p.numel[ti];
  float s = 0.f;
  {
    constexpr int U = 4;                       // loads of a trip issued together; the sum keeps its element order
    size_t i = lo + threadIdx.x;
    for (; i + (U - 1) * OPT_BLOCK < hi; i += U * OPT_BLOCK) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = g[i + u * OPT_BLOCK];
#pragma unroll
      for (int u = 0; u < U; ++u) s = fmaf(x[u], x[u], s);
    }
    for (; i < hi; i += OPT_BLOCK) s = fmaf(g[i], g[i], s);
  }
  s = row16_sum_dpp(s);
  const int si = __builtin_bit_cast(int, s);
  s = (__builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 16))) +
      (__builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 48)));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

// norm_out[0] = sqrt(sum of the partials, in order): one workgroup, fixed tree.  With a device step counter the same
// thread advances it and leaves Adam's two bias-correction factors of the new step in norm_out[1], norm_out[2].
__global__ __launch_bounds__(OPT_BLOCK) void ring_gradnorm_final_kernel(const float* partial, int nblk, float* norm_out,
                                                                        int* step_counter, float lr, float beta1,
                                                                        float beta2) {
  __shared__ float red[OPT_BLOCK];
  float s = 0.f;
  for (int i = threadIdx.x; i < nblk; i += OPT_BLOCK) s += partial[i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = OPT_BLOCK / 2; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    norm_out[0] = sqrtf(red[0]);
    if (step_counter) {
      const int t = step_counter[0] + 1;
      step_counter[0] = t;
      norm_out[1] = (float)((double)lr / (1.0 - pow((double)beta1, (double)t)));
      norm_out[2] = (float)(1.0 / sqrt(1.0 - pow((double)beta2, (double)t)));
    }
  }
}

// g <- g * min(1, max_norm / (norm + 1e-6)) (written back, as clip_grad_norm_ does); then torch.optim.Adam's update:
// m = b1 m + (1-b1) g;  v = b2 v + (1-b2) g^2;  p -= lr / (1 - b1^t) * m / (sqrt(v) / sqrt(1 - b2^t) + eps)
__global__ __launch_bounds__(OPT_BLOCK) void ring_clip_adam_kernel(RingOptArgs p, const float* norm) {
  int blk = blockIdx.x, ti = 0;
  while (ti < p.n && blk >= p.chunks[ti]) blk -= p.chunks[ti++];
  if (ti >= p.n) return;
  float clip = 1.f;
  if (p.max_norm > 0.f) clip = fminf(p.max_norm / (norm[0] + 1e-6f), 1.f);
  // the four arrays of a tensor are distinct allocations: all loads of a trip can be in flight together
  float* __restrict__ g = p.grad[ti];
  float* __restrict__ w = p.param[ti];
  float* __restrict__ m = p.exp_avg[ti];
  float* __restrict__ v = p.exp_avg_sq[ti];
  const size_t lo = (size_t)blk * OPT_CHUNK, hi = lo + OPT_CHUNK < p.numel[ti] ? lo + OPT_CHUNK : p.numel[ti];
  const float step_size = p.step_counter ? norm[1] : p.step_size;
  const float inv_sqrt_bc2 = p.step_counter ? norm[2] : p.inv_sqrt_bc2;
  auto update = [&](size_t i, float gr, float mo, float vo, float wo) {
    const float gi = gr * clip;
    const float mi = p.beta1 * mo + (1.f - p.beta1) * gi;
    const float vi = p.beta2 * vo + (1.f - p.beta2) * gi * gi;
    g[i] = gi;
    m[i] = mi;
    v[i] = vi;
    w[i] = wo - step_size * (mi / (sqrtf(vi) * inv_sqrt_bc2 + p.eps));
  };
  constexpr int U = 4;
  size_t i = lo + threadIdx.x;
  for (; i + (U - 1) * OPT_BLOCK < hi; i += U * OPT_BLOCK) {
    float gr[U], mo[U], vo[U], wo[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      gr[u] = g[i + u * OPT_BLOCK];
      mo[u] = m[i + u * OPT_BLOCK];
      vo[u] = v[i + u * OPT_BLOCK];
      wo[u] = w[i + u * OPT_BLOCK];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) update(i + u * OPT_BLOCK, gr[u], mo[u], vo[u], wo[u]);
  }
  for (; i < hi; i += OPT_BLOCK) update(i, g[i], m[i], v[i], w[i]);
}

int ring_opt_chunks(size_t numel) { return (int)((numel + OPT_CHUNK - 1) / OPT_CHUNK); }

// workspace: (total chunks + 3) floats; behind the partial sums: the gradient norm (before clipping) and, with a device
// step counter, the step's two bias-correction factors
hipError_t ring_launch_clip_adam(const RingOptArgs& a, float* workspace, hipStream_t st) {
  int total = 0;
  for (int i = 0; i < a.n; ++i) total += a.chunks[i];
  if (total <= 0) return hipErrorInvalidValue;
  float* norm = workspace + total;
  hipLaunchKernelGGL(ring_gradnorm_partial_kernel, dim3(total), dim3(OPT_BLOCK), 0, st, a, workspace);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ring_gradnorm_final_kernel, dim3(1), dim3(OPT_BLOCK), 0, st, workspace, total, norm, a.step_counter,
                     a.lr, a.beta1, a.beta2);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ring_clip_adam_kernel, dim3(total), dim3(OPT_BLOCK), 0, st, a, norm);
  return hipGetLastError();
}
