/*
 * CPU oracle for the first-order linear recurrence scan  h_t = a_t * h_{t-1} + b_t.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, the Python
 * package above it) may link, import or call this file; it is the checker that
 * tests, the smoke entry and the bench's cpu_baseline leg compare against.
 *
 * What it restates (reference file:line):
 *   forward   sequential_scan/common.py:46-59            h[0]=beta[0]; h[t]=h[t-1]*alpha[t]+beta[t]
 *             csrc/include/sequential_scan_cpu.hpp:5-34  same, fp32, row-major (bs, seq, d)
 *   backward  csrc/include/sequential_scan_cpu.hpp:36-115
 *                 g[T-1]=dout[T-1]; g[t]=alpha[t+1]*g[t+1]+dout[t];
 *                 grad_beta[t]=g[t]; grad_alpha[t]=g[t]*h[t-1] (t>=1); grad_alpha[0]=0
 *   bf16 I/O  csrc/include/sequential_scan_kernel_bf16.cuh:138-144 (bf16 -> fp32 on load,
 *             fp32 carry, round-to-nearest-even to bf16 on store, :50-56)
 *
 * Layout: every tensor is (bs, seq, d) row-major contiguous; the scan runs over
 * axis 1 independently per (batch, channel).  alpha[:,0,:] is never read.
 * Valid for every seq >= 1 (the reference kernels need seq >= 2 / >= 3).
 *
 * The backward carry g stays in fp32 in every variant; the reference's bf16
 * kernel re-rounds it to bf16 each step by accident
 * (sequential_scan_kernel_bf16.cuh:286), which the fp32-accumulated
 * specification this oracle serves does not ask for.
 *
 * `fused` selects how one step is rounded: 0 = multiply then add (two
 * roundings, what common.py and the C++ header compute), 1 = fmaf (one
 * rounding, what a GPU kernel built with contraction computes).
 *
 * Pinned by tests/test_oracle.py: closed forms (alpha==1 -> cumsum, alpha==0 ->
 * beta, constant alpha -> geometric series), an fp64 brute-force sum of
 * products on small shapes, autograd through an independent fp64 loop, the
 * reverse-scan identity, and - where it is built - the reference's own C++
 * header compiled unchanged (oracle/_ref).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t v) {
  uint32_t u = ((uint32_t)v) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet: the behaviour of __float2bfloat16 */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float step_f32(float a, float h, float b, int fused) {
  if (fused) return fmaf(a, h, b);
  volatile float m = a * h; /* volatile: forbid the compiler to contract */
  return m + b;
}

/* Loop order: batch, then time, then channel (unit stride), with one carry per
 * channel in a scratch row - the order of sequential_scan_cpu.hpp:18-33. */

#define SCAN_FWD(NAME, IN_T, OUT_T, ACC_T, LOAD, STORE, STEP)                    \
  void NAME(const IN_T *alpha, const IN_T *beta, OUT_T *h, int64_t bs,           \
            int64_t seq, int64_t d FUSED_PARAM) {                                \
    ACC_T *carry = (ACC_T *)malloc(sizeof(ACC_T) * (size_t)(d > 0 ? d : 1));     \
    for (int64_t b = 0; b < bs; ++b) {                                           \
      const int64_t base = b * seq * d;                                          \
      for (int64_t t = 0; t < seq; ++t) {                                        \
        const int64_t row = base + t * d;                                        \
        for (int64_t c = 0; c < d; ++c) {                                        \
          const int64_t i = row + c;                                             \
          if (t == 0)                                                            \
            carry[c] = LOAD(beta[i]);                                            \
          else                                                                   \
            carry[c] = STEP(LOAD(alpha[i]), carry[c], LOAD(beta[i]));            \
          h[i] = STORE(carry[c]);                                                \
        }                                                                        \
      }                                                                          \
    }                                                                            \
    free(carry);                                                                 \
  }

/* H_T/LOADH: type and loader of the saved forward states. */
#define SCAN_BWD(NAME, IN_T, H_T, OUT_T, ACC_T, LOAD, LOADH, STORE, STEP, ZERO)  \
  void NAME(const IN_T *alpha, const H_T *h, const IN_T *dout, OUT_T *galpha,    \
            OUT_T *gbeta, int64_t bs, int64_t seq, int64_t d FUSED_PARAM) {      \
    ACC_T *g = (ACC_T *)malloc(sizeof(ACC_T) * (size_t)(d > 0 ? d : 1));         \
    for (int64_t b = 0; b < bs; ++b) {                                           \
      const int64_t base = b * seq * d;                                          \
      for (int64_t t = seq - 1; t >= 0; --t) {                                   \
        const int64_t row = base + t * d;                                        \
        for (int64_t c = 0; c < d; ++c) {                                        \
          const int64_t i = row + c;                                             \
          if (t == seq - 1)                                                      \
            g[c] = LOAD(dout[i]);                                                \
          else                                                                   \
            g[c] = STEP(LOAD(alpha[i + d]), g[c], LOAD(dout[i]));                \
          gbeta[i] = STORE(g[c]);                                                \
          if (t >= 1)                                                            \
            galpha[i] = STORE(g[c] * LOADH(h[i - d]));                           \
          else                                                                   \
            galpha[i] = ZERO;                                                    \
        }                                                                        \
      }                                                                          \
    }                                                                            \
    free(g);                                                                     \
  }

#define ID(x) (x)
#define STEP32(a, h, b) step_f32((a), (h), (b), fused)
#define STEP32_UNFUSED(a, h, b) step_f32((a), (h), (b), 0)
#define STEP64(a, h, b) ((a) * (h) + (b))

/* ---- fp32 in, fp32 out ------------------------------------------------- */
#define FUSED_PARAM , int fused
SCAN_FWD(oracle_scan_fwd_f32, float, float, float, ID, ID, STEP32)
SCAN_BWD(oracle_scan_bwd_f32, float, float, float, float, ID, ID, ID, STEP32, 0.0f)

/* ---- bf16 in, bf16 out, fp32 carry -------------------------------------- *
 * The backward reads h as the STORED (bf16-rounded) forward output, which is
 * what the reference saves (sequential_scan/scan_cuda.py:20). */
SCAN_FWD(oracle_scan_fwd_bf16, uint16_t, uint16_t, float, bf16_to_f32, f32_to_bf16, STEP32)
SCAN_BWD(oracle_scan_bwd_bf16, uint16_t, uint16_t, uint16_t, float, bf16_to_f32,
         bf16_to_f32, f32_to_bf16, STEP32, (uint16_t)0)
#undef FUSED_PARAM

/* ---- bf16 in, fp32 out: the grading oracle ------------------------------ *
 * Same seeded bf16 inputs as the device kernel, every intermediate and every
 * output kept in fp32, multiply-then-add rounding; the backward takes the
 * fp32 forward states, not the rounded ones.  Device results are compared with
 * these at rtol = atol = 1e-2. */
#define FUSED_PARAM
SCAN_FWD(oracle_scan_fwd_bf16_f32out, uint16_t, float, float, bf16_to_f32, ID, STEP32_UNFUSED)
SCAN_BWD(oracle_scan_bwd_bf16_f32out, uint16_t, float, float, float, bf16_to_f32, ID,
         ID, STEP32_UNFUSED, 0.0f)

/* ---- fp64 throughout: used only to pin the fp32 variants ---------------- */
SCAN_FWD(oracle_scan_fwd_f64, double, double, double, ID, ID, STEP64)
SCAN_BWD(oracle_scan_bwd_f64, double, double, double, double, ID, ID, ID, STEP64, 0.0)
#undef FUSED_PARAM

/* bf16 helpers exported so tests can pin the rounding against torch's */
void oracle_f32_to_bf16(const float *src, uint16_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]);
}
void oracle_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}
