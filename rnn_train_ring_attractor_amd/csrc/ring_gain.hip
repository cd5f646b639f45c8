// Gain networks of the action signal, forward and backward, as two elementwise passes.
//
// The reference models scale each action channel by a learned gain (train/train_ring_attractor.py:70-79, 136-146;
// train/train_general_ring_attractor.py:38-46, 99-109): per sample, step and channel c
//     m = |x|,  u_j = w1_j m + b1_j,  a_j = gelu(u_j)  (j < h),  z = sum_j w2_j a_j + b2,  s = softplus(z),  A = x * s
// with one 1 -> h -> 1 network (Linear, GELU (exact erf), Linear, Softplus (beta 1, threshold 20)) per channel.
// The networks see only the input signal, not the recurrent state, so they are evaluated for all (b, t) at once in
// front of the time loop instead of inside it: 8 bytes per sample-step of traffic, and the time-loop kernels stay as
// they are.  Backward: from dL/dA (which the BPTT kernels produce) to the 3h + 1 parameter gradients per channel,
// summed over B*T samples in a fixed order (per-thread partial sums, fixed tree inside a workgroup, per-workgroup
// partials summed in a fixed order by a second launch), and optionally dL/dx.
//
// Parameters are packed per channel as [w1[0..h) | b1[0..h) | w2[0..h) | b2]; gradients use the same packing.
#include "ring_common.hpp"
#include "ring_kernels.hpp"

namespace {

constexpr int GAIN_THREADS = 256;

__device__ __forceinline__ void gelu_pair(float x, float& F, float& D) { act_fast<ACT_GELU>(x, F, D); }

// softplus(z) and its derivative sigmoid(z); torch's Softplus switches to the identity above its threshold of 20
__device__ __forceinline__ void softplus_pair(float z, float& s, float& ds) {
  const float e = __expf(-fabsf(z));                      // exp(-|z|) in (0, 1]
  const float sig_abs = 1.f / (1.f + e);                  // sigmoid(|z|)
  ds = z >= 0.f ? sig_abs : 1.f - sig_abs;
  s = z > 20.f ? z : fmaxf(z, 0.f) + log1pf(e);
  if (z > 20.f) ds = 1.f;
}

}  // namespace

// One thread per element (b, t, c) of the [B,T,k] signal.
template <int H>
__global__ __launch_bounds__(GAIN_THREADS) void ring_gain_fwd_kernel(const float* __restrict__ x,
                                                                     const float* __restrict__ params,
                                                                     float* __restrict__ out, int k, int h, long total) {
  extern __shared__ float prm[];                           // [k][3H+1], zero padded past h
  constexpr int PS = 3 * H + 1;
  for (int i = threadIdx.x; i < k * PS; i += GAIN_THREADS) {
    const int c = i / PS, o = i % PS;
    const int part = o / H, j = o % H;
    float v = 0.f;
    if (o == 3 * H) v = params[(size_t)c * (3 * h + 1) + 3 * h];
    else if (j < h) v = params[(size_t)c * (3 * h + 1) + part * h + j];
    prm[i] = v;
  }
  __syncthreads();
  for (long idx = (long)blockIdx.x * GAIN_THREADS + threadIdx.x; idx < total; idx += (long)gridDim.x * GAIN_THREADS) {
    const int c = (int)(idx % k);
    const float* pc = prm + c * PS;
    const float xv = x[idx], m = fabsf(xv);
    float z = pc[3 * H];
#pragma unroll
    for (int j = 0; j < H; ++j) {
      float a, d;
      gelu_pair(fmaf(pc[j], m, pc[H + j]), a, d);
      z = fmaf(pc[2 * H + j], a, z);
    }
    float s, ds;
    softplus_pair(z, s, ds);
    out[idx] = xv * s;
  }
}

// Thread `tid` of workgroup `blk` walks samples blk*256 + tid, + gridDim*256, ... of ONE channel (blockIdx.y), keeps
// the 3H + 1 partial sums in registers, and the workgroup reduces them in a fixed order into
// partial[blk][c][3H+1].  grad_x (optional) receives dL/dx = dL/dA * (s + x * s' * sign(x)).
template <int H>
__global__ __launch_bounds__(GAIN_THREADS) void ring_gain_bwd_kernel(const float* __restrict__ x,
                                                                     const float* __restrict__ params,
                                                                     const float* __restrict__ grad_A,
                                                                     float* __restrict__ grad_x,
                                                                     float* __restrict__ partial, int k, int h,
                                                                     long samples) {
  constexpr int PS = 3 * H + 1;
  __shared__ float prm[PS];
  __shared__ float red[GAIN_THREADS / 64][PS];
  const int c = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  for (int o = tid; o < PS; o += GAIN_THREADS) {
    const int part = o / H, j = o % H;
    float v = 0.f;
    if (o == 3 * H) v = params[(size_t)c * (3 * h + 1) + 3 * h];
    else if (j < h) v = params[(size_t)c * (3 * h + 1) + part * h + j];
    prm[o] = v;
  }
  __syncthreads();
  float gw1[H], gb1[H], gw2[H], gb2 = 0.f;
#pragma unroll
  for (int j = 0; j < H; ++j) gw1[j] = gb1[j] = gw2[j] = 0.f;
  for (long sidx = (long)blockIdx.x * GAIN_THREADS + tid; sidx < samples; sidx += (long)gridDim.x * GAIN_THREADS) {
    const long idx = sidx * k + c;
    const float xv = x[idx], m = fabsf(xv), go = grad_A[idx];
    float a[H], da[H];
    float z = prm[3 * H];
#pragma unroll
    for (int j = 0; j < H; ++j) {
      gelu_pair(fmaf(prm[j], m, prm[H + j]), a[j], da[j]);
      z = fmaf(prm[2 * H + j], a[j], z);
    }
    float s, ds;
    softplus_pair(z, s, ds);
    const float dz = go * xv * ds;                         // dL/dz
    gb2 += dz;
    float dm = 0.f;                                        // dz/dm / ... accumulated as dL/dm
#pragma unroll
    for (int j = 0; j < H; ++j) {
      gw2[j] = fmaf(dz, a[j], gw2[j]);
      const float du = dz * prm[2 * H + j] * da[j];
      gb1[j] += du;
      gw1[j] = fmaf(du, m, gw1[j]);
      dm = fmaf(du, prm[j], dm);
    }
    if (grad_x) grad_x[idx] = fmaf(go, s, xv > 0.f ? dm : (xv < 0.f ? -dm : 0.f));
  }
  // fixed-order reduction: 64 lanes with a butterfly, then the four waves in wave order
  auto wave_total = [&](float v) {
    v = row16_sum_dpp(v);
    const int i = __builtin_bit_cast(int, v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 48));
    return (r0 + r1) + (r2 + r3);
  };
#pragma unroll
  for (int j = 0; j < H; ++j) {
    const float t1 = wave_total(gw1[j]), t2 = wave_total(gb1[j]), t3 = wave_total(gw2[j]);
    if (lane == 0) {
      red[wv][j] = t1;
      red[wv][H + j] = t2;
      red[wv][2 * H + j] = t3;
    }
  }
  {
    const float t4 = wave_total(gb2);
    if (lane == 0) red[wv][3 * H] = t4;
  }
  __syncthreads();
  for (int o = tid; o < PS; o += GAIN_THREADS)
    partial[((size_t)blockIdx.x * k + c) * PS + o] = ((red[0][o] + red[1][o]) + red[2][o]) + red[3][o];
}

// grad_params[c][3h+1] = sum over workgroups of partial[blk][c][3H+1], un-padded.  One wave per output: lane l adds
// the partials of workgroups l, l + 64, ... in that order (independent loads, all in flight together), then the 64
// lane sums are combined by a fixed butterfly, so the result does not depend on scheduling.
template <int H>
__global__ __launch_bounds__(GAIN_THREADS) void ring_gain_reduce_kernel(const float* __restrict__ partial,
                                                                        float* __restrict__ grad_params, int k, int h,
                                                                        int nblk) {
  constexpr int PS = 3 * H + 1;
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * (GAIN_THREADS / 64) + (threadIdx.x >> 6);
  if (i >= k * (3 * h + 1)) return;                        // whole waves leave together
  const int c = i / (3 * h + 1), o = i % (3 * h + 1);
  const int po = o == 3 * h ? 3 * H : (o / h) * H + (o % h);
  float s = 0.f;
  for (int b = lane; b < nblk; b += 64) s += partial[((size_t)b * k + c) * PS + po];
  s = row16_sum_dpp(s);
  const int si = __builtin_bit_cast(int, s);
  const float total = (__builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 0)) +
                       __builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 16))) +
                      (__builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 32)) +
                       __builtin_bit_cast(float, __builtin_amdgcn_readlane(si, 48)));
  if (lane == 0) grad_params[i] = total;
}

static int gain_pad(int h) { return h <= 8 ? 8 : (h <= 16 ? 16 : (h <= 32 ? 32 : 0)); }

int ring_gain_blocks(long samples) {
  long b = (samples + GAIN_THREADS - 1) / GAIN_THREADS;
  return (int)(b < 1 ? 1 : (b > 512 ? 512 : b));
}

size_t ring_gain_workspace_bytes(int k, int h, long samples) {
  const int H = gain_pad(h);
  if (H == 0) return 0;
  return (size_t)ring_gain_blocks(samples) * k * (3 * H + 1) * sizeof(float);
}

hipError_t ring_launch_gain_fwd(const float* x, const float* params, float* out, int k, int h, long samples,
                                hipStream_t st) {
  const int H = gain_pad(h);
  if (H == 0) return hipErrorInvalidValue;
  const long total = samples * k;
  long blocks = (total + GAIN_THREADS - 1) / GAIN_THREADS;
  if (blocks > 4096) blocks = 4096;
  const size_t lds = (size_t)k * (3 * H + 1) * sizeof(float);
  if (lds > 48 * 1024) return hipErrorInvalidValue;
  switch (H) {
    case 8: hipLaunchKernelGGL(ring_gain_fwd_kernel<8>, dim3((unsigned)blocks), dim3(GAIN_THREADS), lds, st, x, params, out, k, h, total); break;
    case 16: hipLaunchKernelGGL(ring_gain_fwd_kernel<16>, dim3((unsigned)blocks), dim3(GAIN_THREADS), lds, st, x, params, out, k, h, total); break;
    default: hipLaunchKernelGGL(ring_gain_fwd_kernel<32>, dim3((unsigned)blocks), dim3(GAIN_THREADS), lds, st, x, params, out, k, h, total); break;
  }
  return hipGetLastError();
}

hipError_t ring_launch_gain_bwd(const float* x, const float* params, const float* grad_A, float* grad_params,
                                float* grad_x, int k, int h, long samples, void* workspace, hipStream_t st) {
  const int H = gain_pad(h);
  if (H == 0) return hipErrorInvalidValue;
  const int nblk = ring_gain_blocks(samples);
  float* partial = (float*)workspace;
  const dim3 grid((unsigned)nblk, (unsigned)k);
  switch (H) {
    case 8: hipLaunchKernelGGL(ring_gain_bwd_kernel<8>, grid, dim3(GAIN_THREADS), 0, st, x, params, grad_A, grad_x, partial, k, h, samples); break;
    case 16: hipLaunchKernelGGL(ring_gain_bwd_kernel<16>, grid, dim3(GAIN_THREADS), 0, st, x, params, grad_A, grad_x, partial, k, h, samples); break;
    default: hipLaunchKernelGGL(ring_gain_bwd_kernel<32>, grid, dim3(GAIN_THREADS), 0, st, x, params, grad_A, grad_x, partial, k, h, samples); break;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int n = k * (3 * h + 1);
  const unsigned rb = (unsigned)((n + GAIN_THREADS / 64 - 1) / (GAIN_THREADS / 64));   // one wave per output
  switch (H) {
    case 8: hipLaunchKernelGGL(ring_gain_reduce_kernel<8>, dim3(rb), dim3(GAIN_THREADS), 0, st, partial, grad_params, k, h, nblk); break;
    case 16: hipLaunchKernelGGL(ring_gain_reduce_kernel<16>, dim3(rb), dim3(GAIN_THREADS), 0, st, partial, grad_params, k, h, nblk); break;
    default: hipLaunchKernelGGL(ring_gain_reduce_kernel<32>, dim3(rb), dim3(GAIN_THREADS), 0, st, partial, grad_params, k, h, nblk); break;
  }
  return hipGetLastError();
}
