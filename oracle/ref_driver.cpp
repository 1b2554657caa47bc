// Thin C-ABI driver around the reference's own C++ CPU scan, compiled from where
// the header lies (-I$REFERENCE_DIR/csrc/include); nothing of the reference is
// copied here.  The header's entry points are templates over the shape
// (csrc/include/sequential_scan_cpu.hpp:5,36), so a fixed list of shapes is
// instantiated and dispatched at run time.  Test infrastructure only.
//
// The reference backward reads row seq-2 unconditionally
// (sequential_scan_cpu.hpp:55,62-64), so every listed shape has seq >= 2.
#include "sequential_scan_cpu.hpp"

#include <cstddef>
#include <cstdint>
#include <vector>

namespace {

template <int B, int T, int D>
void run_fwd(const float *alpha, const float *beta, float *h) {
  const std::size_t n = std::size_t(B) * T * D;
  std::vector<float> va(alpha, alpha + n), vb(beta, beta + n), vh(n, 0.0f);
  reference_scan_fwd<B, T, D>(&va, &vb, &vh);
  for (std::size_t i = 0; i < n; ++i) h[i] = vh[i];
}

template <int B, int T, int D>
void run_bwd(const float *alpha, const float *h, const float *dout,
             float *galpha, float *gbeta) {
  const std::size_t n = std::size_t(B) * T * D;
  std::vector<float> va(alpha, alpha + n), vh(h, h + n), vd(dout, dout + n);
  std::vector<float> ga(n, 0.0f), gb(n, 0.0f);
  reference_scan_bwd<B, T, D>(&va, &vh, &vd, &ga, &gb);
  for (std::size_t i = 0; i < n; ++i) {
    galpha[i] = ga[i];
    gbeta[i] = gb[i];
  }
}

}  // namespace

#define REF_SHAPES(X) \
  X(1, 2, 3)          \
  X(2, 4, 8)          \
  X(3, 7, 5)          \
  X(2, 33, 24)        \
  X(4, 128, 64)       \
  X(2, 1024, 768)

extern "C" {

// number of instantiated shapes, and the i-th one (bs, seq, d)
int ref_scan_num_shapes(void) {
  int n = 0;
#define X(B, T, D) ++n;
  REF_SHAPES(X)
#undef X
  return n;
}

int ref_scan_shape(int idx, int64_t *bs, int64_t *seq, int64_t *d) {
  int n = 0;
#define X(B, T, D)   \
  if (idx == n++) {  \
    *bs = B;         \
    *seq = T;        \
    *d = D;          \
    return 0;        \
  }
  REF_SHAPES(X)
#undef X
  return -1;
}

// 0 on success, -1 when (bs, seq, d) is not one of the instantiated shapes
int ref_scan_fwd(const float *alpha, const float *beta, float *h, int64_t bs,
                 int64_t seq, int64_t d) {
#define X(B, T, D)                        \
  if (bs == B && seq == T && d == D) {    \
    run_fwd<B, T, D>(alpha, beta, h);     \
    return 0;                             \
  }
  REF_SHAPES(X)
#undef X
  return -1;
}

int ref_scan_bwd(const float *alpha, const float *h, const float *dout,
                 float *galpha, float *gbeta, int64_t bs, int64_t seq,
                 int64_t d) {
#define X(B, T, D)                                      \
  if (bs == B && seq == T && d == D) {                  \
    run_bwd<B, T, D>(alpha, h, dout, galpha, gbeta);    \
    return 0;                                           \
  }
  REF_SHAPES(X)
#undef X
  return -1;
}

}  // extern "C"
