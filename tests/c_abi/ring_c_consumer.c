/*
 * A plain-C consumer of the ringattr C ABI: no Python, no torch, no C++.  It is what a C host that linked the
 * reference's fwd_cuda / bwd_cuda (cpp/fwd.cu:21-35, cpp/bwd.cu:4-30) would look like against this library: device
 * buffers from the HIP runtime, workspace sizes from the query functions, status codes checked after every call.
 *
 * The check uses a problem with a closed form: Wo = c * I, Wa = 0, J0 = 0, J1 = 1, relu, r_init > 0.  Then
 * re = c * r_prev > 0 and r_t = m^(t+1) * r_init with m = 1 - alpha + alpha * c, and with grad_output = 1 on the last
 * step only, dL/d r_init = m^T everywhere and dL/d Wo[i][i] = alpha * sum_b sum_t m^(T-1-t) * r_{t-1}[b][i] ... the
 * diagonal is checked against that sum accumulated on the host.  (The operands of the products are rounded to bf16,
 * hence the 1e-2 tolerance.)
 *
 * Built as a shared object (test_c_consumer() returns 0 on success and fills `msg`), so that a test process that
 * already owns the GPU can run it in-process.
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ringattr.h"

#define CHECK_HIP(call)                                                                         \
  do {                                                                                          \
    hipError_t e_ = (call);                                                                     \
    if (e_ != hipSuccess) {                                                                     \
      snprintf(msg, msg_len, "%s: %s", #call, hipGetErrorString(e_));                           \
      goto done;                                                                                \
    }                                                                                           \
  } while (0)

#define CHECK_RING(call)                                                                        \
  do {                                                                                          \
    int rc_ = (call);                                                                           \
    if (rc_ != RINGATTR_OK) {                                                                   \
      snprintf(msg, msg_len, "%s -> %d: %s", #call, rc_, ringattr_last_error());                \
      goto done;                                                                                \
    }                                                                                           \
  } while (0)

__attribute__((visibility("default"))) int test_c_consumer(int N, int B, int T, char* msg, size_t msg_len) {
  const int k = 2;
  const float alpha = 0.15f, c = 0.5f, m = 1.0f - alpha + alpha * c;
  const size_t nW = (size_t)N * N, nA = (size_t)B * T * k, nR = (size_t)B * N, nH = (size_t)T * B * N;
  int result = 1;
  float *hWo = NULL, *hR = NULL, *hH = NULL, *hG = NULL, *hgWo = NULL, *hgR = NULL;
  void *dA = NULL, *dWa = NULL, *dWo = NULL, *dR = NULL, *dH = NULL, *dG = NULL, *dgWa = NULL, *dgWo = NULL, *dgR = NULL;
  void *saved = NULL, *wsf = NULL, *wsb = NULL;
  msg[0] = 0;

  hWo = (float*)calloc(nW, sizeof(float));
  hR = (float*)malloc(nR * sizeof(float));
  hH = (float*)malloc(nH * sizeof(float));
  hG = (float*)calloc(nH, sizeof(float));
  hgWo = (float*)malloc(nW * sizeof(float));
  hgR = (float*)malloc(nR * sizeof(float));
  if (!hWo || !hR || !hH || !hG || !hgWo || !hgR) {
    snprintf(msg, msg_len, "host allocation failed");
    goto done;
  }
  for (int i = 0; i < N; ++i) hWo[(size_t)i * N + i] = c;
  for (size_t i = 0; i < nR; ++i) hR[i] = 0.25f + 0.5f * (float)((i * 2654435761u) % 1000u) / 1000.0f;
  for (size_t i = 0; i < nR; ++i) hG[(size_t)(T - 1) * nR + i] = 1.0f;      /* dL/d r_{T-1} = 1 */

  {
    const size_t sb = ringattr_saved_bytes(N, k, T, B), fb = ringattr_fwd_workspace_bytes(N, k, T, B);
    const size_t bb = ringattr_bwd_workspace_bytes(N, k, T, B, 1);
    if (!sb || !fb || !bb) {
      snprintf(msg, msg_len, "size query failed: %s", ringattr_last_error());
      goto done;
    }
    CHECK_HIP(hipMalloc(&dA, nA * 4));
    CHECK_HIP(hipMalloc(&dWa, k * nW * 4));
    CHECK_HIP(hipMalloc(&dWo, nW * 4));
    CHECK_HIP(hipMalloc(&dR, nR * 4));
    CHECK_HIP(hipMalloc(&dH, nH * 4));
    CHECK_HIP(hipMalloc(&dG, nH * 4));
    CHECK_HIP(hipMalloc(&dgWa, k * nW * 4));
    CHECK_HIP(hipMalloc(&dgWo, nW * 4));
    CHECK_HIP(hipMalloc(&dgR, nR * 4));
    CHECK_HIP(hipMalloc(&saved, sb));
    CHECK_HIP(hipMalloc(&wsf, fb));
    CHECK_HIP(hipMalloc(&wsb, bb));
    CHECK_HIP(hipMemset(dA, 0, nA * 4));
    CHECK_HIP(hipMemset(dWa, 0, k * nW * 4));
    CHECK_HIP(hipMemcpy(dWo, hWo, nW * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dR, hR, nR * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(dG, hG, nH * 4, hipMemcpyHostToDevice));

    CHECK_RING(ringattr_fwd(dA, dWa, 0.0f, 1.0f, dWo, dR, dH, alpha, N, k, T, B, /*relu*/ 0, saved, wsf, fb, NULL));
    CHECK_RING(ringattr_bwd(dG, dA, dWa, 0.0f, 1.0f, dWo, dH, dR, dgWa, dgWo, alpha, N, k, T, B, 0, /*accumulate*/ 0,
                            saved, NULL, dgR, wsb, bb, NULL));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(hH, dH, nH * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(hgWo, dgWo, nW * 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(hgR, dgR, nR * 4, hipMemcpyDeviceToHost));
  }

  {
    double worst_h = 0.0, worst_r = 0.0, worst_w = 0.0, off_diag = 0.0;
    for (int t = 0; t < T; ++t)
      for (size_t i = 0; i < nR; ++i) {
        const double want = pow((double)m, t + 1) * hR[i], err = fabs(hH[(size_t)t * nR + i] - want) / want;
        if (err > worst_h) worst_h = err;
      }
    for (size_t i = 0; i < nR; ++i) {
      const double want = pow((double)m, T), err = fabs(hgR[i] - want) / want;
      if (err > worst_r) worst_r = err;
    }
    /* g_t = alpha * F'(re) * G_t with G_t = m^(T-1-t) and F' = 1:  dWo[i][j] = J1 * sum_{b,t} g_t[b][i] * r_{t-1}[b][j] */
    for (int i = 0; i < N; ++i)
      for (int j = 0; j < N; ++j) {
        double want = 0.0;
        for (int b = 0; b < B; ++b)
          for (int t = 0; t < T; ++t)
            want += alpha * pow((double)m, T - 1 - t) * pow((double)m, t) * hR[(size_t)b * N + j];
        const double got = hgWo[(size_t)i * N + j], err = fabs(got - want) / want;
        if (i == j) {
          if (err > worst_w) worst_w = err;
        } else if (err > off_diag) {
          off_diag = err;   /* every row of g is the same here, so all entries of a column agree with the diagonal's */
        }
      }
    snprintf(msg, msg_len, "history %.2e, grad_r_init %.2e, grad_Wo diagonal %.2e, off-diagonal %.2e (relative)", worst_h,
             worst_r, worst_w, off_diag);
    result = (worst_h <= 1e-2 && worst_r <= 1e-2 && worst_w <= 1e-2 && off_diag <= 1e-2) ? 0 : 2;
  }

done:
  hipFree(dA); hipFree(dWa); hipFree(dWo); hipFree(dR); hipFree(dH); hipFree(dG); hipFree(dgWa); hipFree(dgWo);
  hipFree(dgR); hipFree(saved); hipFree(wsf); hipFree(wsb);
  free(hWo); free(hR); free(hH); free(hG); free(hgWo); free(hgR);
  return result;
}
