/*
 * CPU model of the HIP kernels' OWN arithmetic order for a chained scan.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships may link, import or call this file.
 *
 * This is not a restatement of the reference (whose scan walks each channel with one thread
 * in order, csrc/include/sequential_scan_kernel_bf16.cuh:121-151; that is oracle/scan_oracle.c).
 * It restates, one channel at a time and with plain sequential C, the order in which the
 * row-major HIP kernels of fast_sequential_scan_amd/csrc compose a long sequence out of
 * slices, waves and chunks - so that a test can demand that the device returns exactly these
 * bits, on every launch, whatever the timing of its workgroups:
 *
 *   slice   `steps` consecutive scan steps (one lane's registers); its effect on a state is
 *           the map x -> A*x + B with  B = fmaf(a, B, b), A = A*a  over its steps;
 *   chunk   `waves` consecutive slices (one workgroup); the slices' maps are composed in
 *           order, B = fma0(A_w, B, B_w), A = A*A_w, which also yields what the slices before
 *           slice w do to the chunk's incoming state (its prefix);
 *   chain   the state entering chunk k > 0 is composed from the maps of chunks k-1 .. a+1 and
 *           the outgoing state of chunk a = anchor(k) (the last chunk of the round of `period`
 *           chunks before, or the last multiple of look*span below k if nearer): the chunks are
 *           dealt out nearest first to `look` waves, ceil((k-a)/look) <= `span` consecutive
 *           chunks each; each wave composes its chunks nearest first, then the waves' results
 *           are folded in wave order;
 *   steps   every slice finally re-runs the recurrence from its true incoming state,
 *           state = fmaf(a, state, b), and the outputs are the states rounded to storage.
 *
 * fma0(a, x, b) is b when x == 0 and fmaf(a, x, b) otherwise.  Steps beyond the end of the
 * sequence are identity maps (a = 1, b = 0); the first step has coefficient 0.
 *
 * Pinned by tests/test_chained_model.py without a GPU: with one slice it equals the fused
 * sequential oracle bit for bit; on inputs whose arithmetic is exact (small integers) it
 * equals the sequential oracle bit for bit under every tiling, which pins its indexing;
 * on random inputs it stays within fp32 rounding of the sequential oracle.
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

static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float fma0(float a, float x, float b) { return x == 0.0f ? b : fmaf(a, x, b); }

typedef struct {
  int steps, waves, period, look, span;
} chain_cfg;

/* the last chunk of the round before, or the last multiple of `stride` below the chunk if nearer */
static int chain_anchor(int chunk, int period, int stride) {
  const int round_first = chunk - chunk % period;
  const int by_round = round_first > 0 ? round_first - 1 : 0;
  const int by_stride = (chunk - 1) / stride * stride;
  return by_round > by_stride ? by_round : by_stride;
}

/* One channel.  a[r], b[r] for r = 0..n-1 in scan order (a[0] is ignored: no predecessor);
 * out[r] receives the fp32 state after step r.  Scratch: 4 floats per chunk. */
static void chained_channel(const float *a, const float *b, float *out, int64_t n, const chain_cfg *cfg,
                            float *chunk_A, float *chunk_B, float *chunk_out) {
  const int S = cfg->steps, W = cfg->waves;
  const int64_t C = (int64_t)S * W;
  const int64_t n_chunks = (n + C - 1) / C;
  const int chained = n_chunks > 1;
  float mA[64], mB[64], pA[64], pB[64]; /* per wave of one chunk (W <= 64) */

  for (int64_t k = 0; k < n_chunks; ++k) {
    const int last = k == n_chunks - 1;
    /* slice maps */
    for (int w = 0; w < W; ++w) {
      float A = 1.0f, B = 0.0f;
      for (int s = 0; s < S; ++s) {
        const int64_t r = (k * W + w) * (int64_t)S + s;
        const float av = r >= n ? 1.0f : (r == 0 ? 0.0f : a[r]);
        const float bv = r >= n ? 0.0f : b[r];
        B = fmaf(av, B, bv);
        A *= av;
      }
      mA[w] = A;
      mB[w] = B;
    }
    float hin = 0.0f;
    if (!chained && W == 1) {
      pA[0] = 1.0f; /* the slice is the whole sequence: it starts from 0 */
      pB[0] = 0.0f;
    } else {
      /* prefixes and the chunk's map */
      float A = 1.0f, B = 0.0f;
      for (int w = 0; w < W; ++w) {
        pA[w] = A;
        pB[w] = B;
        B = fma0(mA[w], B, mB[w]);
        A *= mA[w];
      }
      chunk_A[k] = A;
      chunk_B[k] = B;
      if (k == 0) {
        chunk_out[0] = B; /* the sequence starts from 0 */
      } else {
        const int anchor = chain_anchor((int)k, cfg->period, cfg->look * cfg->span);
        /* chunks per look-back wave: as few as the waves allow (cfg->span is the most) */
        int span = ((int)k - anchor + cfg->look - 1) / cfg->look;
        span = span < 1 ? 1 : (span > cfg->span ? cfg->span : span);
        const int reach = cfg->look * span;
        float accA = 1.0f, accB = 0.0f;
        for (int nearest = (int)k - 1; nearest >= anchor; nearest -= reach) {
          for (int w = 0; w < cfg->look && nearest - w * span >= anchor; ++w) {
            const int j = nearest - w * span;
            float qA = j == anchor ? 0.0f : chunk_A[j];
            float qB = j == anchor ? chunk_out[j] : chunk_B[j];
            for (int kk = 1; kk < span && j - kk >= anchor; ++kk) {
              const int jj = j - kk;
              const float rA = jj == anchor ? 0.0f : chunk_A[jj];
              const float rB = jj == anchor ? chunk_out[jj] : chunk_B[jj];
              qB = fma0(qA, rB, qB);
              qA *= rA;
            }
            accB = fma0(accA, qB, accB);
            accA *= qA;
          }
        }
        hin = accB;
        if (!last) chunk_out[k] = fma0(A, hin, B);
      }
    }
    /* the recurrence from each slice's true incoming state */
    for (int w = 0; w < W; ++w) {
      float state;
      if (!chained && W == 1)
        state = 0.0f;
      else if (k == 0)
        state = pB[w];
      else
        state = fma0(pA[w], hin, pB[w]);
      for (int s = 0; s < S; ++s) {
        const int64_t r = (k * W + w) * (int64_t)S + s;
        if (r >= n) break;
        state = fmaf(r == 0 ? 0.0f : a[r], state, b[r]);
        out[r] = state;
      }
    }
  }
}

static int cfg_ok(const chain_cfg *c) {
  return c->steps >= 1 && c->waves >= 1 && c->waves <= 64 && c->period >= 1 && c->look >= 1 && c->span >= 1;
}

/* ---- fp32 tensors (bs, seq, d) ------------------------------------------------------------- */

int chained_scan_fwd_f32(const float *alpha, const float *beta, float *h, int64_t bs, int64_t seq, int64_t d,
                         int steps, int waves, int period, int look, int span) {
  const chain_cfg cfg = {steps, waves, period, look, span};
  if (!cfg_ok(&cfg)) return 1;
  if (bs <= 0 || seq <= 0 || d <= 0) return 0;
  const int64_t n_chunks = (seq + (int64_t)steps * waves - 1) / ((int64_t)steps * waves);
  float *buf = (float *)malloc(sizeof(float) * (size_t)(3 * seq + 3 * n_chunks));
  float *a = buf, *b = buf + seq, *o = buf + 2 * seq, *cA = buf + 3 * seq, *cB = cA + n_chunks, *cO = cB + n_chunks;
  for (int64_t bi = 0; bi < bs; ++bi)
    for (int64_t c = 0; c < d; ++c) {
      const int64_t base = bi * seq * d + c;
      for (int64_t t = 0; t < seq; ++t) {
        a[t] = alpha[base + t * d];
        b[t] = beta[base + t * d];
      }
      chained_channel(a, b, o, seq, &cfg, cA, cB, cO);
      for (int64_t t = 0; t < seq; ++t) h[base + t * d] = o[t];
    }
  free(buf);
  return 0;
}

/* backward: scan step r is timestep t = seq-1-r with coefficient alpha[t+1] and addend dout[t];
 * grad_beta[t] = g, grad_alpha[t] = g * h[t-1] (one fp32 multiply), grad_alpha[0] = 0 */
int chained_scan_bwd_f32(const float *alpha, const float *h, const float *dout, float *galpha, float *gbeta,
                         int64_t bs, int64_t seq, int64_t d, int steps, int waves, int period, int look,
                         int span) {
  const chain_cfg cfg = {steps, waves, period, look, span};
  if (!cfg_ok(&cfg)) return 1;
  if (bs <= 0 || seq <= 0 || d <= 0) return 0;
  const int64_t n_chunks = (seq + (int64_t)steps * waves - 1) / ((int64_t)steps * waves);
  float *buf = (float *)malloc(sizeof(float) * (size_t)(3 * seq + 3 * n_chunks));
  float *a = buf, *b = buf + seq, *o = buf + 2 * seq, *cA = buf + 3 * seq, *cB = cA + n_chunks, *cO = cB + n_chunks;
  for (int64_t bi = 0; bi < bs; ++bi)
    for (int64_t c = 0; c < d; ++c) {
      const int64_t base = bi * seq * d + c;
      for (int64_t r = 0; r < seq; ++r) {
        const int64_t t = seq - 1 - r;
        a[r] = r == 0 ? 0.0f : alpha[base + (t + 1) * d];
        b[r] = dout[base + t * d];
      }
      chained_channel(a, b, o, seq, &cfg, cA, cB, cO);
      for (int64_t r = 0; r < seq; ++r) {
        const int64_t t = seq - 1 - r;
        gbeta[base + t * d] = o[r];
        galpha[base + t * d] = t >= 1 ? o[r] * h[base + (t - 1) * d] : 0.0f;
      }
    }
  free(buf);
  return 0;
}

/* ---- bf16 tensors as bit patterns: fp32 inside, outputs rounded to nearest even --------------- */

int chained_scan_fwd_bf16(const uint16_t *alpha, const uint16_t *beta, uint16_t *h, int64_t bs, int64_t seq,
                          int64_t d, int steps, int waves, int period, int look, int span) {
  const chain_cfg cfg = {steps, waves, period, look, span};
  if (!cfg_ok(&cfg)) return 1;
  if (bs <= 0 || seq <= 0 || d <= 0) return 0;
  const int64_t n_chunks = (seq + (int64_t)steps * waves - 1) / ((int64_t)steps * waves);
  float *buf = (float *)malloc(sizeof(float) * (size_t)(3 * seq + 3 * n_chunks));
  float *a = buf, *b = buf + seq, *o = buf + 2 * seq, *cA = buf + 3 * seq, *cB = cA + n_chunks, *cO = cB + n_chunks;
  for (int64_t bi = 0; bi < bs; ++bi)
    for (int64_t c = 0; c < d; ++c) {
      const int64_t base = bi * seq * d + c;
      for (int64_t t = 0; t < seq; ++t) {
        a[t] = bf16_to_f32(alpha[base + t * d]);
        b[t] = bf16_to_f32(beta[base + t * d]);
      }
      chained_channel(a, b, o, seq, &cfg, cA, cB, cO);
      for (int64_t t = 0; t < seq; ++t) h[base + t * d] = f32_to_bf16(o[t]);
    }
  free(buf);
  return 0;
}

int chained_scan_bwd_bf16(const uint16_t *alpha, const uint16_t *h, const uint16_t *dout, uint16_t *galpha,
                          uint16_t *gbeta, int64_t bs, int64_t seq, int64_t d, int steps, int waves, int period,
                          int look, int span) {
  const chain_cfg cfg = {steps, waves, period, look, span};
  if (!cfg_ok(&cfg)) return 1;
  if (bs <= 0 || seq <= 0 || d <= 0) return 0;
  const int64_t n_chunks = (seq + (int64_t)steps * waves - 1) / ((int64_t)steps * waves);
  float *buf = (float *)malloc(sizeof(float) * (size_t)(3 * seq + 3 * n_chunks));
  float *a = buf, *b = buf + seq, *o = buf + 2 * seq, *cA = buf + 3 * seq, *cB = cA + n_chunks, *cO = cB + n_chunks;
  for (int64_t bi = 0; bi < bs; ++bi)
    for (int64_t c = 0; c < d; ++c) {
      const int64_t base = bi * seq * d + c;
      for (int64_t r = 0; r < seq; ++r) {
        const int64_t t = seq - 1 - r;
        a[r] = r == 0 ? 0.0f : bf16_to_f32(alpha[base + (t + 1) * d]);
        b[r] = bf16_to_f32(dout[base + t * d]);
      }
      chained_channel(a, b, o, seq, &cfg, cA, cB, cO);
      for (int64_t r = 0; r < seq; ++r) {
        const int64_t t = seq - 1 - r;
        gbeta[base + t * d] = f32_to_bf16(o[r]);
        galpha[base + t * d] = t >= 1 ? f32_to_bf16(o[r] * bf16_to_f32(h[base + (t - 1) * d])) : (uint16_t)0;
      }
    }
  free(buf);
  return 0;
}
