/*
 * A host written in plain C against include/fss_scan.h: no Python, no torch.
 * Allocates with the HIP runtime, runs the bf16 forward and backward scans (and the
 * state, gated and channel-major entry points' argument checks) on the current
 * device and compares with the CPU oracle (oracle/scan_oracle.c, linked in as the
 * checker).  Exit status 0 and a line starting "abi_check ok" on success.
 *
 * Built by tests/native/Makefile; run by tests/test_native_abi_gpu.py.
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "fss_scan.h"

/* the checker */
void oracle_scan_fwd_bf16_f32out(const uint16_t *alpha, const uint16_t *beta, float *h, int64_t bs, int64_t seq,
                                 int64_t d);
void oracle_scan_bwd_bf16_f32out(const uint16_t *alpha, const float *h, const uint16_t *dout, float *galpha,
                                 float *gbeta, int64_t bs, int64_t seq, int64_t d);
void oracle_f32_to_bf16(const float *src, uint16_t *dst, int64_t n);
void oracle_bf16_to_f32(const uint16_t *src, float *dst, int64_t n);

#define HIP_OK(call)                                                            \
  do {                                                                          \
    hipError_t e_ = (call);                                                     \
    if (e_ != hipSuccess) {                                                     \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));         \
      return 2;                                                                 \
    }                                                                           \
  } while (0)

#define FSS_OK_OR_FAIL(call)                                                    \
  do {                                                                          \
    int rc_ = (call);                                                           \
    if (rc_ != FSS_OK) {                                                        \
      fprintf(stderr, "%s -> %d (%s)\n", #call, rc_, fss_strerror(rc_));        \
      return 3;                                                                 \
    }                                                                           \
  } while (0)

static uint32_t rng_state = 12345u;
static float uniform01(void) { /* xorshift32 */
  rng_state ^= rng_state << 13;
  rng_state ^= rng_state >> 17;
  rng_state ^= rng_state << 5;
  return (float)(rng_state >> 8) * (1.0f / 16777216.0f);
}
static float normal(void) {
  const float u1 = uniform01() + 1e-7f, u2 = uniform01();
  return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
}

static int compare(const char *name, const uint16_t *got_bits, const float *want, int64_t n) {
  float *got = (float *)malloc(sizeof(float) * (size_t)n);
  oracle_bf16_to_f32(got_bits, got, n);
  int64_t bad = 0;
  double worst = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    const double err = fabs((double)got[i] - (double)want[i]);
    if (err > worst) worst = err;
    if (!(err <= 1e-2 + 1e-2 * fabs((double)want[i]))) ++bad;
  }
  free(got);
  if (bad) fprintf(stderr, "%s: %lld of %lld outside rtol=atol=1e-2 (worst %g)\n", name, (long long)bad, (long long)n, worst);
  return bad ? 1 : 0;
}

int main(void) {
  const int64_t bs = 2, seq = 1000, d = 768, n = bs * seq * d; /* several chunks, ragged last one */
  if (fss_abi_version() != FSS_ABI_VERSION) {
    fprintf(stderr, "header and library disagree on the ABI version\n");
    return 1;
  }
  float *tmp = (float *)malloc(sizeof(float) * (size_t)n);
  uint16_t *alpha = (uint16_t *)malloc(2 * (size_t)n), *beta = (uint16_t *)malloc(2 * (size_t)n),
           *dout = (uint16_t *)malloc(2 * (size_t)n);
  for (int64_t i = 0; i < n; ++i) tmp[i] = 1.0f / (1.0f + expf(-normal()));
  oracle_f32_to_bf16(tmp, alpha, n);
  for (int64_t i = 0; i < n; ++i) tmp[i] = normal();
  oracle_f32_to_bf16(tmp, beta, n);
  for (int64_t i = 0; i < n; ++i) tmp[i] = normal();
  oracle_f32_to_bf16(tmp, dout, n);

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  void *d_alpha, *d_beta, *d_dout, *d_h, *d_ga, *d_gb, *d_ws;
  const size_t bytes = 2 * (size_t)n;
  HIP_OK(hipMalloc(&d_alpha, bytes));
  HIP_OK(hipMalloc(&d_beta, bytes));
  HIP_OK(hipMalloc(&d_dout, bytes));
  HIP_OK(hipMalloc(&d_h, bytes));
  HIP_OK(hipMalloc(&d_ga, bytes));
  HIP_OK(hipMalloc(&d_gb, bytes));
  const size_t ws_bytes = fss_workspace_bytes_max(bs, seq, d);
  HIP_OK(hipMalloc(&d_ws, ws_bytes));
  HIP_OK(hipMemcpyAsync(d_alpha, alpha, bytes, hipMemcpyHostToDevice, stream));
  HIP_OK(hipMemcpyAsync(d_beta, beta, bytes, hipMemcpyHostToDevice, stream));
  HIP_OK(hipMemcpyAsync(d_dout, dout, bytes, hipMemcpyHostToDevice, stream));

  FSS_OK_OR_FAIL(fss_workspace_init(d_ws, ws_bytes, stream));
  FSS_OK_OR_FAIL(fss_scan_fwd_bf16(d_alpha, d_beta, d_h, bs, seq, d, d_ws, ws_bytes, stream));
  FSS_OK_OR_FAIL(fss_scan_bwd_bf16(d_alpha, d_h, d_dout, d_ga, d_gb, bs, seq, d, d_ws, ws_bytes, stream));
  FSS_OK_OR_FAIL(fss_workspace_status(d_ws, stream)); /* synchronises */

  uint16_t *h = (uint16_t *)malloc(bytes), *ga = (uint16_t *)malloc(bytes), *gb = (uint16_t *)malloc(bytes);
  HIP_OK(hipMemcpy(h, d_h, bytes, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(ga, d_ga, bytes, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(gb, d_gb, bytes, hipMemcpyDeviceToHost));

  float *h_ref = (float *)malloc(sizeof(float) * (size_t)n), *ga_ref = (float *)malloc(sizeof(float) * (size_t)n),
        *gb_ref = (float *)malloc(sizeof(float) * (size_t)n);
  oracle_scan_fwd_bf16_f32out(alpha, beta, h_ref, bs, seq, d);
  oracle_scan_bwd_bf16_f32out(alpha, h_ref, dout, ga_ref, gb_ref, bs, seq, d);
  int failed = compare("h", h, h_ref, n) + compare("grad_alpha", ga, ga_ref, n) + compare("grad_beta", gb, gb_ref, n);

  /* error behaviour of the other entry points, as a C caller sees it */
  if (fss_scan_fwd_state(FSS_BF16, d_alpha, d_beta, NULL, NULL, NULL, bs, seq, d, d_ws, ws_bytes, stream, NULL) !=
      FSS_ERR_NULL_POINTER)
    ++failed;
  if (fss_gated_scan_bwd(FSS_BF16, d_alpha, NULL, d_h, d_dout, d_ga, d_gb, bs, seq, d, d_ws, ws_bytes, stream, NULL) !=
      FSS_ERR_NULL_POINTER)
    ++failed;
  if (fss_gated_scan_bwd_state(FSS_BF16, d_alpha, d_beta, d_h, d_dout, NULL, NULL, d_ga, d_gb, (float *)d_ws, bs, seq, d,
                               d_ws, ws_bytes, stream, NULL) != FSS_ERR_NULL_POINTER)
    ++failed; /* grad_h_before without h_before */
  if (fss_scan_fwd_cm(FSS_BF16, d_alpha, d_beta, d_h, bs, d, seq, d_ws, 0, stream, NULL) != FSS_OK)
    ++failed; /* seq 1000 fits one workgroup: no workspace needed */
  if (fss_scan_fwd_bf16(d_alpha, d_beta, d_h, bs, seq, d, d_ws, 64, stream) != FSS_ERR_WORKSPACE_SMALL) ++failed;
  HIP_OK(hipStreamSynchronize(stream));

  hipFree(d_alpha); hipFree(d_beta); hipFree(d_dout); hipFree(d_h); hipFree(d_ga); hipFree(d_gb); hipFree(d_ws);
  hipStreamDestroy(stream);
  if (failed) {
    fprintf(stderr, "abi_check FAILED (%d)\n", failed);
    return 1;
  }
  printf("abi_check ok: bf16 fwd+bwd (%lld,%lld,%lld) from C within rtol=atol=1e-2 of the oracle\n", (long long)bs,
         (long long)seq, (long long)d);
  return 0;
}
