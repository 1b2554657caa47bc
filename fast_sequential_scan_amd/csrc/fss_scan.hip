// Linear-recurrence scan for MI355X (gfx950, wave64): kernels and the C ABI of
// include/fss_scan.h.
//
//   forward    h[t] = alpha[t]*h[t-1] + beta[t],  h[-1] = 0, alpha[0] never read
//   backward   g[t] = alpha[t+1]*g[t+1] + dout[t];  grad_beta = g;  grad_alpha[t] = g[t]*h[t-1]
//
// Semantics follow the reference's kernels
// (csrc/include/sequential_scan_kernel_bf16.cuh:58-167 forward, :169-390 backward;
// csrc/include/sequential_scan_kernel.cuh for fp32) except that the backward
// carry stays in fp32 (the reference re-rounds it to bf16 each step, :286) and
// that any seq >= 1 and any d are accepted.  The structure is not the
// reference's (one block per batch row walking the whole sequence): see below.
//
// Work decomposition
//   Tensors are (bs, seq, d) row-major, so one timestep of one batch item is a
//   contiguous row of d elements.  A lane owns VEC adjacent channels, a wave
//   owns 64*VEC adjacent channels (one coalesced row segment per load), and
//   keeps STEPS consecutive timesteps of them in registers.  The WAVES waves of a
//   workgroup take consecutive time slices of the SAME channels, so a workgroup
//   ("tile") covers 64*VEC channels x WAVES*STEPS timesteps ("chunk").
//
//   A tile runs in three phases, touching every input and output byte once:
//     1. every lane issues all its loads at once (STEPS rows x 2 or 3 tensors:
//        the memory-level parallelism that fills HBM), then folds its slice into
//        the affine map x -> A*x + B it applies to the incoming state;
//     2. wave 0 composes the waves' maps through LDS and publishes the chunk's map;
//        at the same time up to 8 waves each fetch what one earlier chunk of the
//        same channels offers (its outgoing state if it has one, else its map),
//        so the look-back over the nearest chunks costs one memory round trip, not
//        one per chunk (decoupled look-back over (A,B) pairs in global memory).
//        Wave 0 folds what they found into the chunk's incoming state, publishes
//        the outgoing state, and hands every wave its own incoming state via LDS;
//     3. every lane re-runs the recurrence over its register-resident slice from
//        its true incoming state, in sequential order, and stores the results.
//   Because phase 3 restarts from the incoming state, only that state is
//   computed by re-associated arithmetic; within a slice the operation order is
//   exactly the sequential one.
//
// Chaining across workgroups
//   The grid is persistent: it holds no more workgroups than the device keeps
//   resident at once, and each walks tiles blockIdx, blockIdx+gridDim, ... in
//   chunk-major order.  A tile only waits for lower-numbered tiles, each owned by
//   a resident workgroup that reaches it no later than the waiter reaches its
//   own, so the waits cannot deadlock - and no atomic ticket serialises the
//   start of the workgroups.  State handed between chunks travels as 64-bit
//   words {tag, fp32} written and read with relaxed agent-scope atomics; value
//   and validity arrive together, so no fence is needed.  The tag is a
//   per-workspace launch counter ("epoch", never 0), so words never need
//   clearing; workgroups count themselves out at the end (two-level counter) and
//   the last one advances the epoch for the next launch.  The counter wraps
//   after 2^32-1 launches; a host that can get there re-initialises the
//   workspace first.  Every wait is bounded: a wave that exhausts its budget
//   records an error in the workspace header and carries on with a zero state,
//   so the grid always drains.
//
// The backward runs the same machine over reversed time r = seq-1-t with
// a'[r] = alpha[t+1], b'[r] = dout[t], plus the elementwise g[t]*h[t-1].
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <initializer_list>

#include "../../include/fss_scan.h"

namespace fss {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct BF16 {
  static constexpr int kBytes = 2;
};
struct F32 {
  static constexpr int kBytes = 4;
};

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// Pins a wave-uniform pointer into scalar registers, so that `p + lane_offset`
// becomes the scalar-base + 32-bit-vector-offset form of a global access and
// costs no vector registers or 64-bit vector adds per row.
template <typename P>
__device__ __forceinline__ P *uniform_ptr(P *ptr) {
  const uint64_t u = reinterpret_cast<uint64_t>(ptr);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(u));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(u >> 32));
  return reinterpret_cast<P *>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Loads/stores of N dwords per lane.
template <int N>
struct DwordIO;
template <>
struct DwordIO<1> {
  static __device__ __forceinline__ void load(uint32_t *dst, const char *p) {
    dst[0] = *reinterpret_cast<const uint32_t *>(p);
  }
  static __device__ __forceinline__ void store(char *p, const uint32_t *src) {
    *reinterpret_cast<uint32_t *>(p) = src[0];
  }
};
template <>
struct DwordIO<2> {
  static __device__ __forceinline__ void load(uint32_t *dst, const char *p) {
    u32x2 v = *reinterpret_cast<const u32x2 *>(p);
    dst[0] = v.x;
    dst[1] = v.y;
  }
  static __device__ __forceinline__ void store(char *p, const uint32_t *src) {
    u32x2 v = {src[0], src[1]};
    *reinterpret_cast<u32x2 *>(p) = v;
  }
};
template <>
struct DwordIO<4> {
  static __device__ __forceinline__ void load(uint32_t *dst, const char *p) {
    u32x4 v = *reinterpret_cast<const u32x4 *>(p);
    dst[0] = v.x;
    dst[1] = v.y;
    dst[2] = v.z;
    dst[3] = v.w;
  }
  static __device__ __forceinline__ void store(char *p, const uint32_t *src) {
    u32x4 v = {src[0], src[1], src[2], src[3]};
    *reinterpret_cast<u32x4 *>(p) = v;
  }
};

// One row segment owned by a lane: VEC channels of element type E, kept packed.
template <typename E, int VEC>
struct Row;

template <int VEC>
struct Row<BF16, VEC> {
  static_assert(VEC == 2 || VEC == 4 || VEC == 8, "bf16 vector width");
  static constexpr int kDwords = VEC / 2;
  static constexpr int kBytes = VEC * 2;
  uint32_t dw[kDwords];
  __device__ __forceinline__ void load(const char *p) { DwordIO<kDwords>::load(dw, p); }
  __device__ __forceinline__ void store(char *p) const { DwordIO<kDwords>::store(p, dw); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = dw[i >> 1];
    return (i & 1) ? as_f32(w & 0xffff0000u) : as_f32(w << 16);
  }
  __device__ __forceinline__ void fill(float x) {  // x exactly representable in bf16
    const uint32_t hi = as_u32(x) >> 16;
#pragma unroll
    for (int i = 0; i < kDwords; ++i) dw[i] = hi | (hi << 16);
  }
  // round-to-nearest-even, as __float2bfloat16 of the reference (bf16.cuh:54)
  __device__ __forceinline__ void pack(const float *f) {
#pragma unroll
    for (int i = 0; i < kDwords; ++i) {
      f32x2 v = {f[2 * i], f[2 * i + 1]};
      dw[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
  }
};

template <>
struct Row<BF16, 1> {
  static constexpr int kDwords = 1;
  static constexpr int kBytes = 2;
  uint32_t dw[1];
  __device__ __forceinline__ void load(const char *p) {
    dw[0] = *reinterpret_cast<const uint16_t *>(p);
  }
  __device__ __forceinline__ void store(char *p) const {
    *reinterpret_cast<uint16_t *>(p) = static_cast<uint16_t>(dw[0]);
  }
  __device__ __forceinline__ float get(int) const { return as_f32(dw[0] << 16); }
  __device__ __forceinline__ void fill(float x) { dw[0] = as_u32(x) >> 16; }
  __device__ __forceinline__ void pack(const float *f) {
    f32x2 v = {f[0], 0.0f};
    dw[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2)) & 0xffffu;
  }
};

template <int VEC>
struct Row<F32, VEC> {
  static_assert(VEC == 1 || VEC == 2 || VEC == 4, "fp32 vector width");
  static constexpr int kDwords = VEC;
  static constexpr int kBytes = VEC * 4;
  uint32_t dw[kDwords];
  __device__ __forceinline__ void load(const char *p) { DwordIO<kDwords>::load(dw, p); }
  __device__ __forceinline__ void store(char *p) const { DwordIO<kDwords>::store(p, dw); }
  __device__ __forceinline__ float get(int i) const { return as_f32(dw[i]); }
  __device__ __forceinline__ void fill(float x) {
#pragma unroll
    for (int i = 0; i < kDwords; ++i) dw[i] = as_u32(x);
  }
  __device__ __forceinline__ void pack(const float *f) {
#pragma unroll
    for (int i = 0; i < kDwords; ++i) dw[i] = as_u32(f[i]);
  }
};

// Makes the compiler forget what it derived from a packed row: the rows stay
// packed in registers across the chaining phase and are unpacked again after
// it, instead of keeping an fp32 copy of every element alive next to them.
template <typename RowT>
__device__ __forceinline__ void keep_packed(RowT &r) {
#pragma unroll
  for (int i = 0; i < RowT::kDwords; ++i) asm volatile("" : "+v"(r.dw[i]));
}

// ---- workspace ----------------------------------------------------------------
//
// Header (kHeaderBytes): word 1 = top-level completion counter, word 2 = epoch,
// word 3 = sticky error flag, words 64+32*i (i < 16, one 128-byte line each) =
// first-level completion counters.  Then the tagged words,
// [chunk][column tile][kind: map A, map B, outgoing state][VEC][64 lanes].

enum : int { HDR_DONE = 1, HDR_EPOCH = 2, HDR_ERROR = 3, HDR_SLOT0 = 64, HDR_SLOT_STRIDE = 32 };
constexpr int kDoneSlots = 16;
constexpr size_t kHeaderBytes = 4096;
// Polls a wave makes before it gives up on an earlier chunk (each poll is a memory
// round trip plus a sleep: seconds in total, far beyond any healthy wait).
constexpr uint32_t kSpinLimit = 1u << 20;
// Most waves of a workgroup that look back in parallel, one earlier chunk each.
constexpr int kMaxLookWaves = 16;
enum : uint32_t { kPredNone = 0, kPredMap = 1, kPredState = 2 };

__device__ __forceinline__ uint32_t ld_u32(const uint32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u32(uint32_t *p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t add_u32(uint32_t *p, uint32_t v) {
  return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_word(const uint64_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_word(uint64_t *p, uint32_t tag, float v) {
  __hip_atomic_store(p, (static_cast<uint64_t>(tag) << 32) | as_u32(v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t word_tag(uint64_t w) { return static_cast<uint32_t>(w >> 32); }
__device__ __forceinline__ float word_val(uint64_t w) { return as_f32(static_cast<uint32_t>(w)); }

struct ScanArgs {
  const char *in_a;  // alpha
  const char *in_b;  // beta (forward) / dout (backward)
  const char *in_h;  // stored forward output (backward only)
  char *out0;        // h (forward) / grad_beta (backward)
  char *out1;        // grad_alpha (backward only)
  int64_t seq;
  int64_t d;
  int32_t tiles_per_row;  // ceil(d / (64*VEC))
  int32_t n_ctiles;       // bs * tiles_per_row
  int32_t n_chunks;       // ceil(seq / (WAVES*STEPS))
  int32_t n_tiles;        // n_ctiles * n_chunks
  int32_t look_waves;     // waves that look back in parallel (1..min(WAVES, kMaxLookWaves))
  uint32_t *hdr;          // workspace header
  uint64_t *words;        // tagged words
};

// ---- the kernel ----------------------------------------------------------------

template <typename E, int VEC, int STEPS, bool BWD>
__global__ __launch_bounds__(1024) void scan_kernel(const ScanArgs p) {
  using RowT = Row<E, VEC>;
  constexpr int kRowBytes = RowT::kBytes;
  constexpr int kLaneSlots = 64 * VEC;  // channels per tile

  extern __shared__ float lds[];
  __shared__ uint32_t s_kind[kMaxLookWaves];
  __shared__ uint32_t s_resolved;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n_waves = blockDim.x >> 6;
  const int look = p.look_waves;
  float2 *lds_map = reinterpret_cast<float2 *>(lds);   // [wave][v][lane] = (A, B), later .x = incoming state
  float2 *lds_pred = lds_map + n_waves * kLaneSlots;   // [look wave][v][lane] = what an earlier chunk offers

#ifdef FSS_RESIDENCY_PROBE
  // debug build only: header words 8/9 = workgroups resident now / the most ever seen
  if (threadIdx.x == 0 && p.hdr) {
    const uint32_t now = add_u32(p.hdr + 8, 1u) + 1u;
    __hip_atomic_fetch_max(p.hdr + 9, now, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#endif
  const bool chained = p.n_chunks > 1;
  // every workgroup of a launch reads the same value: it only changes when all are done
  const uint32_t tag = chained ? __builtin_amdgcn_readfirstlane(ld_u32(p.hdr + HDR_EPOCH)) : 0u;

  const int64_t seq = p.seq;
  const int64_t row_bytes = p.d * E::kBytes;
  const uint32_t lane_off = static_cast<uint32_t>(lane * kRowBytes);

  // The grid is sized to be resident all at once; each workgroup walks tiles
  // blockIdx, blockIdx + gridDim, ...  Tiles are numbered chunk-major, so a tile
  // only ever waits for tiles with smaller numbers: those belong to a resident
  // workgroup that reaches them no later than this one reaches its own.
  for (uint32_t tile = blockIdx.x; tile < static_cast<uint32_t>(p.n_tiles); tile += gridDim.x) {
    // unsigned, wave-uniform arithmetic: stays on the scalar unit
    const uint32_t uchunk = tile / static_cast<uint32_t>(p.n_ctiles);
    const uint32_t uctile = tile - uchunk * static_cast<uint32_t>(p.n_ctiles);
    const uint32_t batch = uctile / static_cast<uint32_t>(p.tiles_per_row);
    const uint32_t coltile = uctile - batch * static_cast<uint32_t>(p.tiles_per_row);
    const int chunk = static_cast<int>(uchunk);
    const int ctile = static_cast<int>(uctile);

    const int64_t col0 = static_cast<int64_t>(coltile) * kLaneSlots;  // first channel of the tile
    const bool col_ok = col0 + lane * VEC < p.d;                       // d % VEC == 0 (host)
    // byte offset of (batch, row 0, col0); uniform over the wave
    const int64_t tile_base = (static_cast<int64_t>(batch) * seq * p.d + col0) * E::kBytes;
    // first scan-order index of this wave's slice (forward: r = t, backward: r = seq-1-t)
    const int64_t r0 = (static_cast<int64_t>(chunk) * n_waves + wave) * STEPS;

    // Fast path: every row this wave touches exists, is interior, and every lane
    // has channels.  Forward touches rows r0..r0+STEPS-1 and must not be at r = 0;
    // backward additionally reads row t+1 and t-1.
    const bool full = (col0 + kLaneSlots <= p.d) && (r0 >= 1) &&
                      (BWD ? (r0 + STEPS <= seq - 1) : (r0 + STEPS <= seq));

    RowT a[STEPS], b[STEPS];
    RowT hp[BWD ? STEPS : 1];

    // ---- phase 1a: issue every load of the slice ----------------------------------
    if (full) {
      if (!BWD) {
        const char *pa = p.in_a + tile_base + r0 * row_bytes;
        const char *pb = p.in_b + tile_base + r0 * row_bytes;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          a[s].load(uniform_ptr(pa + s * row_bytes) + lane_off);
          b[s].load(uniform_ptr(pb + s * row_bytes) + lane_off);
        }
      } else {
        // t = seq-1-r: alpha row t+1, dout row t, h row t-1
        const int64_t t0 = seq - 1 - r0;
        const char *pa = p.in_a + tile_base + (t0 + 1) * row_bytes;
        const char *pb = p.in_b + tile_base + t0 * row_bytes;
        const char *ph = p.in_h + tile_base + (t0 - 1) * row_bytes;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          a[s].load(uniform_ptr(pa - s * row_bytes) + lane_off);
          b[s].load(uniform_ptr(pb - s * row_bytes) + lane_off);
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s) hp[s].load(uniform_ptr(ph - s * row_bytes) + lane_off);
      }
    } else {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        const int64_t r = r0 + s;
        const int64_t t = BWD ? seq - 1 - r : r;
        // Outside the sequence the step is the identity map (a=1, b=0); the first
        // step of the scan has no predecessor (a=0), whatever alpha holds there.
        a[s].fill(r >= seq ? 1.0f : 0.0f);
        b[s].fill(0.0f);
        if (BWD) hp[s].fill(0.0f);
        if (col_ok && r < seq) {
          if (r >= 1) a[s].load(uniform_ptr(p.in_a + tile_base + (BWD ? t + 1 : t) * row_bytes) + lane_off);
          b[s].load(uniform_ptr(p.in_b + tile_base + t * row_bytes) + lane_off);
          if (BWD && t >= 1) hp[s].load(uniform_ptr(p.in_h + tile_base + (t - 1) * row_bytes) + lane_off);
        }
      }
    }

    float state[VEC];
    const bool solo = !chained && n_waves == 1;  // the slice is the whole sequence: state starts at 0
    if (solo) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) state[v] = 0.0f;
    } else {
      // ---- phase 1b: the slice as an affine map --------------------------------------
      float mA[VEC], mB[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        mA[v] = 1.0f;
        mB[v] = 0.0f;
      }
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float av = a[s].get(v);
          mB[v] = __builtin_fmaf(av, mB[v], b[s].get(v));
          mA[v] *= av;
        }
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        lds_map[(wave * VEC + v) * 64 + lane] = make_float2(mA[v], mB[v]);
      __syncthreads();

      // ---- phase 2: compose the waves, chain the chunks --------------------------------
      // Wave 0 folds the waves' maps into the chunk's map and publishes it.  Meanwhile
      // wave w (w < look) fetches what chunk-1-w offers - its outgoing state if it has
      // one, else its map - so a look-back over `look` chunks costs one memory round
      // trip instead of one per chunk.  Chains longer than that repeat the step.
      const bool last = chunk == p.n_chunks - 1;
      uint64_t *mine = nullptr;
      float cA[VEC], cB[VEC], hin[VEC], accA[VEC], accB[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        cA[v] = accA[v] = 1.0f;
        cB[v] = accB[v] = hin[v] = 0.0f;
      }
      if (wave == 0) {
        for (int w = 0; w < n_waves; ++w) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const float2 m = lds_map[(w * VEC + v) * 64 + lane];
            cB[v] = __builtin_fmaf(m.x, cB[v], m.y);
            cA[v] *= m.x;
          }
        }
        if (chained) {
          mine = p.words + (static_cast<size_t>(chunk) * p.n_ctiles + ctile) * 3 * kLaneSlots + lane;
          if (chunk > 0 && !last) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
              st_word(mine + (0 * VEC + v) * 64, tag, cA[v]);
              st_word(mine + (1 * VEC + v) * 64, tag, cB[v]);
            }
          }
        }
      }
      if (chained && chunk > 0) {
        int nearest = chunk - 1;  // nearest earlier chunk not folded yet
        for (;;) {
          const int j = nearest - wave;
          if (wave < look && j >= 0) {
            const uint64_t *theirs =
                p.words + (static_cast<size_t>(j) * p.n_ctiles + ctile) * 3 * kLaneSlots + lane;
            float pA[VEC], pB[VEC];
            uint32_t kind = kPredNone;
            uint32_t polls = 0;
            while (kind == kPredNone) {
              uint64_t wa[VEC], wb[VEC], ws[VEC];
#pragma unroll
              for (int v = 0; v < VEC; ++v) {
                ws[v] = ld_word(theirs + (2 * VEC + v) * 64);
                wa[v] = ld_word(theirs + (0 * VEC + v) * 64);
                wb[v] = ld_word(theirs + (1 * VEC + v) * 64);
              }
              bool have_state = true, have_map = true;
#pragma unroll
              for (int v = 0; v < VEC; ++v) {
                have_state = have_state && word_tag(ws[v]) == tag;
                have_map = have_map && word_tag(wa[v]) == tag && word_tag(wb[v]) == tag;
              }
              // decide for the whole wave, so that one word per wave describes the slot
              if (__builtin_amdgcn_ballot_w64(have_state) == ~0ull) {
                kind = kPredState;
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                  pA[v] = 0.0f;
                  pB[v] = word_val(ws[v]);
                }
              } else if (j > 0 && __builtin_amdgcn_ballot_w64(have_map) == ~0ull) {
                kind = kPredMap;
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                  pA[v] = word_val(wa[v]);
                  pB[v] = word_val(wb[v]);
                }
              } else if (++polls > kSpinLimit) {
                if (lane == 0) st_u32(p.hdr + HDR_ERROR, 1u);
                kind = kPredState;  // give up: zero state, so that the grid still drains
#pragma unroll
                for (int v = 0; v < VEC; ++v) pA[v] = pB[v] = 0.0f;
              } else {
                __builtin_amdgcn_s_sleep(2);
              }
            }
#pragma unroll
            for (int v = 0; v < VEC; ++v)
              lds_pred[(wave * VEC + v) * 64 + lane] = make_float2(pA[v], pB[v]);
            if (lane == 0) s_kind[wave] = kind;
          }
          __syncthreads();
          if (wave == 0) {
            bool resolved = false;
            for (int w = 0; w < look && nearest - w >= 0 && !resolved; ++w) {
              const bool is_state = s_kind[w] == kPredState;
#pragma unroll
              for (int v = 0; v < VEC; ++v) {
                const float2 m = lds_pred[(w * VEC + v) * 64 + lane];
                if (is_state) {
                  hin[v] = __builtin_fmaf(accA[v], m.y, accB[v]);
                } else {
                  accB[v] = __builtin_fmaf(accA[v], m.y, accB[v]);
                  accA[v] *= m.x;
                }
              }
              resolved = is_state;
            }
            if (lane == 0) s_resolved = resolved ? 1u : 0u;
          }
          __syncthreads();
          if (s_resolved != 0u) break;  // chunk 0 always offers a state, so this is reached
          nearest -= look;
        }
      }

      if (wave == 0) {
        if (chained && !last) {
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            st_word(mine + (2 * VEC + v) * 64, tag, __builtin_fmaf(cA[v], hin[v], cB[v]));
        }
        // incoming state of every wave of this tile, left where the wave's map was
        for (int w = 0; w < n_waves; ++w) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const float2 m = lds_map[(w * VEC + v) * 64 + lane];
            lds_map[(w * VEC + v) * 64 + lane].x = hin[v];
            hin[v] = __builtin_fmaf(m.x, hin[v], m.y);
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int v = 0; v < VEC; ++v) state[v] = lds_map[(wave * VEC + v) * 64 + lane].x;
    }

    // ---- phase 3: the recurrence from the true incoming state, in order -------------
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      keep_packed(a[s]);
      keep_packed(b[s]);
      if (BWD) keep_packed(hp[s]);
    }
    if (full) {
      if (!BWD) {
        char *po = p.out0 + tile_base + r0 * row_bytes;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) state[v] = __builtin_fmaf(a[s].get(v), state[v], b[s].get(v));
          RowT o;
          o.pack(state);
          o.store(uniform_ptr(po + s * row_bytes) + lane_off);
        }
      } else {
        const int64_t t0 = seq - 1 - r0;
        char *pgb = p.out0 + tile_base + t0 * row_bytes;
        char *pga = p.out1 + tile_base + t0 * row_bytes;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          float ga[VEC];
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            state[v] = __builtin_fmaf(a[s].get(v), state[v], b[s].get(v));
            ga[v] = state[v] * hp[s].get(v);
          }
          RowT ob, oa;
          ob.pack(state);
          oa.pack(ga);
          ob.store(uniform_ptr(pgb - s * row_bytes) + lane_off);
          oa.store(uniform_ptr(pga - s * row_bytes) + lane_off);
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        const int64_t r = r0 + s;
        const int64_t t = BWD ? seq - 1 - r : r;
        float ga[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          state[v] = __builtin_fmaf(a[s].get(v), state[v], b[s].get(v));
          if (BWD) ga[v] = (t >= 1) ? state[v] * hp[s].get(v) : 0.0f;  // grad_alpha[0] = 0
        }
        if (col_ok && r < seq) {
          RowT o;
          o.pack(state);
          o.store(uniform_ptr(p.out0 + tile_base + t * row_bytes) + lane_off);
          if (BWD) {
            RowT oa;
            oa.pack(ga);
            oa.store(uniform_ptr(p.out1 + tile_base + t * row_bytes) + lane_off);
          }
        }
      }
    }
  }

#ifdef FSS_RESIDENCY_PROBE
  if (threadIdx.x == 0 && p.hdr) __hip_atomic_fetch_sub(p.hdr + 8, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
  // Two-level completion count (16 first-level counters on separate lines keep the
  // atomics off one hot address).  Whoever counts last knows that no workgroup will
  // read the workspace again and advances the epoch for the next launch.
  if (chained && threadIdx.x == 0) {
    const uint32_t slot = blockIdx.x % kDoneSlots;
    const uint32_t in_slot = (gridDim.x - slot + kDoneSlots - 1) / kDoneSlots;
    uint32_t *counter = p.hdr + HDR_SLOT0 + slot * HDR_SLOT_STRIDE;
    if (add_u32(counter, 1u) == in_slot - 1) {
      st_u32(counter, 0u);
      const uint32_t slots_used = gridDim.x < kDoneSlots ? gridDim.x : kDoneSlots;
      if (add_u32(p.hdr + HDR_DONE, 1u) == slots_used - 1) {
        st_u32(p.hdr + HDR_DONE, 0u);
        // 0 is the tag of never-written words: skip it when the counter wraps
        st_u32(p.hdr + HDR_EPOCH, tag + 1u == 0u ? 1u : tag + 1u);
      }
    }
  }
}

// Zero everywhere (tag 0 = "never written"), launch counter starting at 1.
__global__ void workspace_init_kernel(uint32_t *p, size_t n_words) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_words; i += stride)
    p[i] = (i == HDR_EPOCH) ? 1u : 0u;
}

__global__ void copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, size_t n_vec) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_vec; i += stride)
    dst[i] = src[i];
}

// ---- host side --------------------------------------------------------------------

thread_local int tls_hip_error = 0;

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Register budget: packed dwords a lane may hold per input tensor.
inline int max_vec_steps(int dtype) { return dtype == FSS_BF16 ? 64 : 32; }  // vec*steps

// LDS: one (A,B) slot per lane and vector element for every wave, plus the same
// for every wave that looks back.
constexpr size_t kLdsBudget = 60 * 1024;
inline int look_waves(int waves, int vec) {
  int look = waves < kMaxLookWaves ? waves : kMaxLookWaves;
  while (look > 1 && static_cast<size_t>(waves + look) * vec * 512 > kLdsBudget) --look;
  return look;
}
inline size_t lds_bytes(int waves, int vec) {
  return static_cast<size_t>(waves + look_waves(waves, vec)) * vec * 512;
}

inline bool config_valid(const fss_config &c, int dtype) {
  const bool vec_ok = dtype == FSS_BF16 ? (c.vec == 1 || c.vec == 2 || c.vec == 4 || c.vec == 8)
                                        : (c.vec == 1 || c.vec == 2 || c.vec == 4);
  const bool steps_ok = c.steps == 8 || c.steps == 16 || c.steps == 32;
  if (!vec_ok || !steps_ok) return false;
  if (c.vec * c.steps > max_vec_steps(dtype)) return false;
  if (dtype == FSS_BF16 && c.vec == 1 && c.steps > 32) return false;
  if (c.waves < 1 || c.waves > 16) return false;
  if (lds_bytes(c.waves, c.vec) > kLdsBudget) return false;
  return true;
}

// Fills the zero fields of `c`.  `align` is the common alignment in bytes of all
// tensors of the call.
void complete_config(fss_config &c, int64_t bs, int64_t seq, int64_t d, int dtype, int dir,
                     size_t align) {
  // Choices below come from sweeps on MI355X over the five measured workloads
  // (bs8 d1024 seq512..8192, bs16 d512 seq2048, bs4 d2048 seq8192, bs2 d768
  // seq1024, bs1 d256 seq65521).  What they showed: 4 bytes per lane per load
  // (bf16 x2) with as many timesteps in registers as fit beats wider vectors;
  // 8 waves per workgroup (two workgroups per CU, one loading while the other
  // chains and stores) beats 16 unless the chain of chunks is long; with few
  // channels, one channel per lane (twice the column tiles) and shorter slices
  // put more waves in flight.
  const int esize = dtype == FSS_BF16 ? 2 : 4;
  const int64_t channels = bs * d;
  if (c.vec == 0) {
    const bool can2 = d % 2 == 0 && align % (2 * static_cast<size_t>(esize)) == 0;
    int v = can2 ? 2 : 1;
    // few channels: more, narrower column tiles; also never pad a row to twice its width
    if (v == 2 && (channels < 8192 || ceil_div(d, 128) * 128 >= 2 * ceil_div(d, 64) * 64)) v = 1;
    c.vec = v;
  }
  // packed dwords one lane holds per timestep and tensor
  const int dwords = dtype == FSS_BF16 ? (c.vec + 1) / 2 : c.vec;
  if (c.steps == 0) {
    int s = (dir == FSS_BWD ? 16 : 32) / dwords;  // 2 (forward) or 3 (backward) tensors stay in registers
    if (s > 32) s = 32;
    if (s < 8) s = 8;
    // small problems: shorter slices until the machine has a few waves per SIMD
    const int64_t ctiles = bs * ceil_div(d, 64 * c.vec);
    while (s > 8 && ctiles * ceil_div(seq, s) < 1024) s >>= 1;
    // never longer than the sequence needs
    while (s > 8 && seq <= s / 2) s >>= 1;
    c.steps = s;
  }
  if (c.waves == 0) {
    int64_t w = ceil_div(seq, c.steps);
    // long chains of chunks (few channels, long sequence): the largest tile
    const int64_t cap = ceil_div(seq, static_cast<int64_t>(8) * c.steps) > 64 ? 16 : 8;
    if (w > cap) w = cap;
    while (w > 1 && lds_bytes(static_cast<int>(w), c.vec) > kLdsBudget) --w;
    c.waves = static_cast<int32_t>(w);
  }
}

struct Plan {
  fss_config cfg;
  int64_t tiles_per_row, n_ctiles, n_chunks, n_tiles;
  size_t ws_bytes;
};

int make_plan(Plan &pl, int64_t bs, int64_t seq, int64_t d, int dtype, int dir, size_t align,
              const fss_config *user) {
  if (bs < 0 || seq < 0 || d < 0) return FSS_ERR_BAD_SHAPE;
  if (dtype != FSS_BF16 && dtype != FSS_F32) return FSS_ERR_BAD_CONFIG;
  if (dir != FSS_FWD && dir != FSS_BWD) return FSS_ERR_BAD_CONFIG;
  const int esize = dtype == FSS_BF16 ? 2 : 4;
  // bs*seq*d*esize must fit int64
  if (bs > 0 && seq > 0 && d > 0) {
    const __int128 total = static_cast<__int128>(bs) * seq * d * esize;
    if (total > (static_cast<__int128>(1) << 62)) return FSS_ERR_BAD_SHAPE;
  }
  fss_config c = {0, 0, 0, 0};
  if (user) c = *user;
  if (c.max_groups < 0) return FSS_ERR_BAD_CONFIG;
  const int64_t dd = d > 0 ? d : 1, ss = seq > 0 ? seq : 1, bb = bs > 0 ? bs : 1;
  complete_config(c, bb, ss, dd, dtype, dir, align);
  if (!config_valid(c, dtype)) return FSS_ERR_BAD_CONFIG;
  if (dd % c.vec != 0) return FSS_ERR_BAD_CONFIG;
  if (align % (static_cast<size_t>(c.vec) * esize) != 0) return FSS_ERR_MISALIGNED;
  pl.cfg = c;
  pl.tiles_per_row = ceil_div(dd, 64 * c.vec);
  pl.n_ctiles = bb * pl.tiles_per_row;
  pl.n_chunks = ceil_div(ss, static_cast<int64_t>(c.waves) * c.steps);
  pl.n_tiles = pl.n_ctiles * pl.n_chunks;
  if (pl.n_ctiles > INT32_MAX || pl.n_chunks > INT32_MAX || pl.n_tiles > INT32_MAX) return FSS_ERR_BAD_SHAPE;
  pl.ws_bytes = kHeaderBytes;
  if (pl.n_chunks > 1) pl.ws_bytes += static_cast<size_t>(pl.n_tiles) * 3 * 64 * c.vec * sizeof(uint64_t);
  return FSS_OK;
}

size_t common_alignment(std::initializer_list<const void *> ptrs) {
  uintptr_t bits = 0;
  for (const void *p : ptrs) bits |= reinterpret_cast<uintptr_t>(p);
  bits |= 16;  // 16 bytes is all any path needs
  return static_cast<size_t>(bits & (~bits + 1));
}

int check_device() {
  static int cached[64];  // 0 unknown, 1 ok, 2 unsupported
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return FSS_ERR_LAUNCH;
  if (dev < 0 || dev >= 64) return FSS_OK;
  int state = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
  if (state == 0) {
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) {
      tls_hip_error = static_cast<int>(e);
      return FSS_ERR_LAUNCH;
    }
    state = strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
    __atomic_store_n(&cached[dev], state, __ATOMIC_RELAXED);
  }
  return state == 1 ? FSS_OK : FSS_ERR_UNSUPPORTED_DEVICE;
}

// Workgroups of `kernel` that are certainly resident together on the device (0 on
// error).  Deliberately not the runtime's occupancy query: the kernel's waits
// need a lower bound, and that query bounds by vector registers and LDS only.
// These kernels hold many scalar registers as well (a row pointer per load); a
// wave may be allocated 128 of the 800 a SIMD has, which caps a SIMD at 6 waves -
// the residency measured on MI355X for the scalar-heaviest variants.
template <typename Kernel>
int resident_workgroups(Kernel kernel, int waves, size_t lds) {
  static int cu_count = 0;
  if (cu_count == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return 0;
    cu_count = n;
  }
  hipFuncAttributes attr;
  const hipError_t e = hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kernel));
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return 0;
  }
  int vgprs = attr.numRegs > 0 ? attr.numRegs : 128;
  vgprs = (vgprs + 7) / 8 * 8;                    // allocation granule
  int per_simd = 512 / vgprs;                      // 512 vector registers per lane per SIMD
  if (per_simd > 6) per_simd = 6;                  // scalar-register bound, see above
  if (per_simd < 1) return 0;
  int per_cu;
  if (waves >= 4)
    per_cu = per_simd / ((waves + 3) / 4);         // a workgroup puts ceil(waves/4) waves on a SIMD
  else
    per_cu = per_simd * (waves == 1 ? 4 : waves == 2 ? 2 : 1);
  const size_t lds_alloc = (lds + attr.sharedSizeBytes + 1023) / 1024 * 1024;
  const int by_lds = static_cast<int>((160 * 1024) / (lds_alloc ? lds_alloc : 1024));
  if (per_cu > by_lds) per_cu = by_lds;
  if (per_cu > 32) per_cu = 32;
  return per_cu * cu_count;
}

template <typename E, int VEC, int STEPS, bool BWD>
int launch_one(const ScanArgs &args, const Plan &pl, hipStream_t stream) {
  // The kernel's waits are only safe if every workgroup of the grid is resident,
  // so the grid never exceeds what the device holds at once; workgroups loop.
  static int resident[17] = {0};  // by waves per workgroup; same answer on every call
  const int waves = pl.cfg.waves;
  const size_t lds = lds_bytes(waves, VEC);
  int fit = __atomic_load_n(&resident[waves], __ATOMIC_RELAXED);
  if (fit == 0) {
    fit = resident_workgroups(scan_kernel<E, VEC, STEPS, BWD>, waves, lds);
    if (fit <= 0) return FSS_ERR_LAUNCH;
    __atomic_store_n(&resident[waves], fit, __ATOMIC_RELAXED);
  }
  int64_t n_groups = pl.n_tiles < fit ? pl.n_tiles : fit;
  if (pl.cfg.max_groups > 0 && pl.cfg.max_groups < n_groups) n_groups = pl.cfg.max_groups;
  const dim3 grid(static_cast<uint32_t>(n_groups));
  const dim3 block(static_cast<uint32_t>(waves) * 64);
  hipLaunchKernelGGL((scan_kernel<E, VEC, STEPS, BWD>), grid, block, lds, stream, args);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

template <typename E, bool BWD>
int launch_typed(const ScanArgs &args, const Plan &pl, hipStream_t stream) {
  constexpr bool is_bf16 = E::kBytes == 2;
  const int key = pl.cfg.vec * 100 + pl.cfg.steps;
  switch (key) {
#define FSS_CASE(V, S) \
  case V * 100 + S:    \
    return launch_one<E, V, S, BWD>(args, pl, stream);
    FSS_CASE(1, 8)
    FSS_CASE(1, 16)
    FSS_CASE(1, 32)
    FSS_CASE(2, 8)
    FSS_CASE(2, 16)
    FSS_CASE(4, 8)
    default:
      break;
  }
  if constexpr (is_bf16) {
    switch (key) {
      FSS_CASE(2, 32)
      FSS_CASE(4, 16)
      FSS_CASE(8, 8)
      default:
        break;
    }
  }
#undef FSS_CASE
  return FSS_ERR_BAD_CONFIG;
}

int run_scan(int dtype, int dir, const void *alpha, const void *in_b, const void *in_h, void *out0,
             void *out1, int64_t bs, int64_t seq, int64_t d, void *workspace, size_t workspace_bytes,
             void *stream, const fss_config *cfg) {
  if (bs < 0 || seq < 0 || d < 0) return FSS_ERR_BAD_SHAPE;
  if (dtype != FSS_BF16 && dtype != FSS_F32) return FSS_ERR_BAD_CONFIG;
  if (bs == 0 || seq == 0 || d == 0) return FSS_OK;
  if (!alpha || !in_b || !out0) return FSS_ERR_NULL_POINTER;
  if (dir == FSS_BWD && (!in_h || !out1)) return FSS_ERR_NULL_POINTER;
  const size_t esize = dtype == FSS_BF16 ? 2 : 4;
  const size_t align = dir == FSS_BWD ? common_alignment({alpha, in_b, in_h, out0, out1})
                                      : common_alignment({alpha, in_b, out0});
  if (align < esize) return FSS_ERR_MISALIGNED;
  Plan pl;
  int rc = make_plan(pl, bs, seq, d, dtype, dir, align, cfg);
  if (rc != FSS_OK) return rc;
  if (pl.n_chunks > 1) {
    if (!workspace || workspace_bytes < pl.ws_bytes) return FSS_ERR_WORKSPACE_SMALL;
    if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0) return FSS_ERR_MISALIGNED;
  }
  rc = check_device();
  if (rc != FSS_OK) return rc;

  ScanArgs args;
  args.in_a = static_cast<const char *>(alpha);
  args.in_b = static_cast<const char *>(in_b);
  args.in_h = static_cast<const char *>(in_h);
  args.out0 = static_cast<char *>(out0);
  args.out1 = static_cast<char *>(out1);
  args.seq = seq;
  args.d = d;
  args.tiles_per_row = static_cast<int32_t>(pl.tiles_per_row);
  args.n_ctiles = static_cast<int32_t>(pl.n_ctiles);
  args.n_chunks = static_cast<int32_t>(pl.n_chunks);
  args.n_tiles = static_cast<int32_t>(pl.n_tiles);
  args.look_waves = look_waves(pl.cfg.waves, pl.cfg.vec);
  args.hdr = static_cast<uint32_t *>(workspace);
  args.words = workspace ? reinterpret_cast<uint64_t *>(static_cast<char *>(workspace) + kHeaderBytes) : nullptr;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == FSS_BF16)
    return dir == FSS_BWD ? launch_typed<BF16, true>(args, pl, s) : launch_typed<BF16, false>(args, pl, s);
  return dir == FSS_BWD ? launch_typed<F32, true>(args, pl, s) : launch_typed<F32, false>(args, pl, s);
}

}  // namespace fss

// ---- C ABI -------------------------------------------------------------------------

extern "C" {

int fss_abi_version(void) { return FSS_ABI_VERSION; }

const char *fss_strerror(int status) {
  switch (status) {
    case FSS_OK: return "ok";
    case FSS_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FSS_ERR_BAD_SHAPE: return "bs, seq or d is negative or too large";
    case FSS_ERR_MISALIGNED: return "a tensor (or the workspace) is not sufficiently aligned";
    case FSS_ERR_WORKSPACE_SMALL: return "workspace missing or smaller than fss_workspace_bytes";
    case FSS_ERR_BAD_CONFIG: return "unsupported dtype, direction or launch configuration";
    case FSS_ERR_LAUNCH: return "HIP reported an error (see fss_last_hip_error)";
    case FSS_ERR_CHAIN_TIMEOUT: return "a chunk gave up waiting for the state of its predecessor";
    case FSS_ERR_UNSUPPORTED_DEVICE: return "the current device is not gfx950";
    default: return "unknown status";
  }
}

int fss_last_hip_error(void) { return fss::tls_hip_error; }

size_t fss_workspace_bytes(int64_t bs, int64_t seq, int64_t d, int dtype, int dir, const fss_config *cfg) {
  fss::Plan pl;
  // alignment unknown here: assume the best the shape allows (the widest vector,
  // hence the most words per tile, is what a less aligned call can only shrink)
  if (fss::make_plan(pl, bs, seq, d, dtype, dir, 16, cfg) != FSS_OK) return fss::kHeaderBytes;
  return pl.ws_bytes;
}

size_t fss_workspace_bytes_max(int64_t bs, int64_t seq, int64_t d) {
  size_t best = fss::kHeaderBytes;
  for (int dtype = 0; dtype < 2; ++dtype)
    for (int dir = 0; dir < 2; ++dir)
      for (size_t align = 2; align <= 16; align <<= 1) {
        fss::Plan pl;
        if (fss::make_plan(pl, bs, seq, d, dtype, dir, align, nullptr) == FSS_OK && pl.ws_bytes > best)
          best = pl.ws_bytes;
      }
  return best;
}

int fss_choose_config(int64_t bs, int64_t seq, int64_t d, int dtype, int dir, size_t align_bytes,
                      fss_config *out) {
  if (!out) return FSS_ERR_NULL_POINTER;
  fss::Plan pl;
  const int rc = fss::make_plan(pl, bs, seq, d, dtype, dir, align_bytes ? align_bytes : 16, nullptr);
  if (rc == FSS_OK) *out = pl.cfg;
  return rc;
}

int fss_workspace_init(void *workspace, size_t bytes, void *stream) {
  if (!workspace) return FSS_ERR_NULL_POINTER;
  if (bytes < fss::kHeaderBytes) return FSS_ERR_WORKSPACE_SMALL;
  if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0 || bytes % 4 != 0) return FSS_ERR_MISALIGNED;
  const size_t n_words = bytes / 4;
  size_t blocks = (n_words + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fss::workspace_init_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint32_t *>(workspace), n_words);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fss::tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

int fss_workspace_status(void *workspace, void *stream) {
  if (!workspace) return FSS_ERR_NULL_POINTER;
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint32_t hdr[4] = {0, 0, 0, 0};
  hipError_t e = hipMemcpyAsync(hdr, workspace, sizeof(hdr), hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  if (e != hipSuccess) {
    fss::tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  if (hdr[fss::HDR_ERROR] != 0) {
    const uint32_t zero = 0;
    e = hipMemcpyAsync(static_cast<uint32_t *>(workspace) + fss::HDR_ERROR, &zero, 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    return FSS_ERR_CHAIN_TIMEOUT;
  }
  return FSS_OK;
}

int fss_scan_fwd_ex(int dtype, const void *alpha, const void *beta, void *h, int64_t bs, int64_t seq,
                    int64_t d, void *workspace, size_t workspace_bytes, void *stream,
                    const fss_config *cfg) {
  return fss::run_scan(dtype, FSS_FWD, alpha, beta, nullptr, h, nullptr, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg);
}

int fss_scan_bwd_ex(int dtype, const void *alpha, const void *h, const void *dout, void *grad_alpha,
                    void *grad_beta, int64_t bs, int64_t seq, int64_t d, void *workspace,
                    size_t workspace_bytes, void *stream, const fss_config *cfg) {
  return fss::run_scan(dtype, FSS_BWD, alpha, dout, h, grad_beta, grad_alpha, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg);
}

int fss_scan_fwd_bf16(const void *alpha, const void *beta, void *h, int64_t bs, int64_t seq, int64_t d,
                      void *workspace, size_t workspace_bytes, void *stream) {
  return fss_scan_fwd_ex(FSS_BF16, alpha, beta, h, bs, seq, d, workspace, workspace_bytes, stream, nullptr);
}

int fss_scan_bwd_bf16(const void *alpha, const void *h, const void *dout, void *grad_alpha,
                      void *grad_beta, int64_t bs, int64_t seq, int64_t d, void *workspace,
                      size_t workspace_bytes, void *stream) {
  return fss_scan_bwd_ex(FSS_BF16, alpha, h, dout, grad_alpha, grad_beta, bs, seq, d, workspace,
                         workspace_bytes, stream, nullptr);
}

int fss_scan_fwd_f32(const void *alpha, const void *beta, void *h, int64_t bs, int64_t seq, int64_t d,
                     void *workspace, size_t workspace_bytes, void *stream) {
  return fss_scan_fwd_ex(FSS_F32, alpha, beta, h, bs, seq, d, workspace, workspace_bytes, stream, nullptr);
}

int fss_scan_bwd_f32(const void *alpha, const void *h, const void *dout, void *grad_alpha,
                     void *grad_beta, int64_t bs, int64_t seq, int64_t d, void *workspace,
                     size_t workspace_bytes, void *stream) {
  return fss_scan_bwd_ex(FSS_F32, alpha, h, dout, grad_alpha, grad_beta, bs, seq, d, workspace,
                         workspace_bytes, stream, nullptr);
}

int fss_copy_bytes(const void *src, void *dst, size_t bytes, void *stream) {
  if (!src || !dst) return FSS_ERR_NULL_POINTER;
  if (bytes % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0)
    return FSS_ERR_MISALIGNED;
  if (bytes == 0) return FSS_OK;
  const size_t n_vec = bytes / 16;
  size_t blocks = (n_vec + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(fss::copy_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const fss::u32x4 *>(src),
                     static_cast<fss::u32x4 *>(dst), n_vec);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fss::tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

}  // extern "C"
