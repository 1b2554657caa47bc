// Linear-recurrence scan for MI355X (gfx950, wave64): kernels and the C ABI of
// include/fss_scan.h.
//
//   forward    h[t] = alpha[t]*h[t-1] + beta[t],  h[-1] = 0, alpha[0] never used
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
//
// Variants built on the same machine (none of them in the reference): scans with a
// state entering and leaving the sequence (STATE), the gated scan that computes
// alpha = sigmoid(gate) and beta = x*sqrt(1-alpha^2) in phase 1 (GATED, gated_tile),
// IEEE half next to bf16 and fp32, and the channel-major (bs, d, seq) layout with
// time across the lanes (cm_tile, cm_scan_kernel), whose rows are chained exactly
// as the channels are here.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <initializer_list>
#include <mutex>

#include "../../include/fss_scan.h"

namespace fss {

// Device pointers are kept in the global address space explicitly: the generic
// ("flat") form costs a 64-bit vector address per access and a slower instruction.
#define FSS_GLOBAL __attribute__((address_space(1)))
typedef const FSS_GLOBAL char *gcptr_t;
typedef FSS_GLOBAL char *gptr_t;

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// Storage types.  The 16-bit ones say how the two halves of a packed dword become
// fp32 and back (round to nearest even both ways).
struct BF16 {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float lo(uint32_t w) { return as_f32(w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return as_f32(w & 0xffff0000u); }
  // as __float2bfloat16 of the reference (csrc/include/sequential_scan_kernel_bf16.cuh:54)
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
  }
  static __device__ __forceinline__ uint32_t bits(float x) { return as_u32(x) >> 16; }  // x exactly representable
};
struct F16 {
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float lo(uint32_t w) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w)));
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w >> 16)));
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
  }
  static __device__ __forceinline__ uint32_t bits(float x) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x));
  }
};
struct F32 {
  static constexpr int kBytes = 4;
};

// Pins a wave-uniform pointer into scalar registers, so that `p + lane_offset`
// becomes the scalar-base + 32-bit-vector-offset form of a global access and
// costs no vector registers or 64-bit vector adds per row.
template <typename Ptr>
__device__ __forceinline__ Ptr uniform_ptr(Ptr ptr) {
  const uint64_t u = reinterpret_cast<uint64_t>(ptr);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(u));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(u >> 32));
  return reinterpret_cast<Ptr>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Loads/stores of N dwords per lane.  NT marks the access non-temporal: the data
// is touched once, so the caches should not keep it in preference to other lines.
template <int N, bool NT>
struct DwordIO;
template <bool NT>
struct DwordIO<1, NT> {
  static __device__ __forceinline__ void load(uint32_t *dst, gcptr_t p) {
    const FSS_GLOBAL uint32_t *q = reinterpret_cast<const FSS_GLOBAL uint32_t *>(p);
    dst[0] = NT ? __builtin_nontemporal_load(q) : *q;
  }
  static __device__ __forceinline__ void store(gptr_t p, const uint32_t *src) {
    FSS_GLOBAL uint32_t *q = reinterpret_cast<FSS_GLOBAL uint32_t *>(p);
    if (NT)
      __builtin_nontemporal_store(src[0], q);
    else
      *q = src[0];
  }
};
template <bool NT>
struct DwordIO<2, NT> {
  static __device__ __forceinline__ void load(uint32_t *dst, gcptr_t p) {
    const FSS_GLOBAL u32x2 *q = reinterpret_cast<const FSS_GLOBAL u32x2 *>(p);
    const u32x2 v = NT ? __builtin_nontemporal_load(q) : *q;
    dst[0] = v.x;
    dst[1] = v.y;
  }
  static __device__ __forceinline__ void store(gptr_t p, const uint32_t *src) {
    const u32x2 v = {src[0], src[1]};
    FSS_GLOBAL u32x2 *q = reinterpret_cast<FSS_GLOBAL u32x2 *>(p);
    if (NT)
      __builtin_nontemporal_store(v, q);
    else
      *q = v;
  }
};
template <bool NT>
struct DwordIO<4, NT> {
  static __device__ __forceinline__ void load(uint32_t *dst, gcptr_t p) {
    const FSS_GLOBAL u32x4 *q = reinterpret_cast<const FSS_GLOBAL u32x4 *>(p);
    const u32x4 v = NT ? __builtin_nontemporal_load(q) : *q;
    dst[0] = v.x;
    dst[1] = v.y;
    dst[2] = v.z;
    dst[3] = v.w;
  }
  static __device__ __forceinline__ void store(gptr_t p, const uint32_t *src) {
    const u32x4 v = {src[0], src[1], src[2], src[3]};
    FSS_GLOBAL u32x4 *q = reinterpret_cast<FSS_GLOBAL u32x4 *>(p);
    if (NT)
      __builtin_nontemporal_store(v, q);
    else
      *q = v;
  }
};

// One row segment owned by a lane: VEC channels of element type E, kept packed.
template <typename E, int VEC, int BYTES = E::kBytes>
struct Row;

template <typename E, int VEC>
struct Row<E, VEC, 2> {
  static_assert(VEC == 2 || VEC == 4 || VEC == 8, "16-bit vector width");
  static constexpr int kDwords = VEC / 2;
  static constexpr int kBytes = VEC * 2;
  uint32_t dw[kDwords];
  template <bool NT = false>
  __device__ __forceinline__ void load(gcptr_t p) {
    DwordIO<kDwords, NT>::load(dw, p);
  }
  template <bool NT = false>
  __device__ __forceinline__ void store(gptr_t p) const {
    DwordIO<kDwords, NT>::store(p, dw);
  }
  __device__ __forceinline__ float get(int i) const { return (i & 1) ? E::hi(dw[i >> 1]) : E::lo(dw[i >> 1]); }
  __device__ __forceinline__ void fill(float x) {  // x exactly representable in E
    const uint32_t b = E::bits(x);
#pragma unroll
    for (int i = 0; i < kDwords; ++i) dw[i] = b | (b << 16);
  }
  __device__ __forceinline__ void pack(const float *f) {
#pragma unroll
    for (int i = 0; i < kDwords; ++i) dw[i] = E::pack2(f[2 * i], f[2 * i + 1]);
  }
};

template <typename E>
struct Row<E, 1, 2> {
  static constexpr int kDwords = 1;
  static constexpr int kBytes = 2;
  uint32_t dw[1];
  template <bool NT = false>
  __device__ __forceinline__ void load(gcptr_t p) {
    const FSS_GLOBAL uint16_t *q = reinterpret_cast<const FSS_GLOBAL uint16_t *>(p);
    dw[0] = NT ? __builtin_nontemporal_load(q) : *q;
  }
  template <bool NT = false>
  __device__ __forceinline__ void store(gptr_t p) const {
    FSS_GLOBAL uint16_t *q = reinterpret_cast<FSS_GLOBAL uint16_t *>(p);
    if (NT)
      __builtin_nontemporal_store(static_cast<uint16_t>(dw[0]), q);
    else
      *q = static_cast<uint16_t>(dw[0]);
  }
  __device__ __forceinline__ float get(int) const { return E::lo(dw[0]); }
  __device__ __forceinline__ void fill(float x) { dw[0] = E::bits(x); }
  __device__ __forceinline__ void pack(const float *f) { dw[0] = E::pack2(f[0], 0.0f) & 0xffffu; }
};

template <typename E, int VEC>
struct Row<E, VEC, 4> {
  static_assert(VEC == 1 || VEC == 2 || VEC == 4, "fp32 vector width");
  static constexpr int kDwords = VEC;
  static constexpr int kBytes = VEC * 4;
  uint32_t dw[kDwords];
  template <bool NT = false>
  __device__ __forceinline__ void load(gcptr_t p) {
    DwordIO<kDwords, NT>::load(dw, p);
  }
  template <bool NT = false>
  __device__ __forceinline__ void store(gptr_t p) const {
    DwordIO<kDwords, NT>::store(p, dw);
  }
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
  return __hip_atomic_load((const FSS_GLOBAL uint32_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u32(uint32_t *p, uint32_t v) {
  __hip_atomic_store((FSS_GLOBAL uint32_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t add_u32(uint32_t *p, uint32_t v) {
  return __hip_atomic_fetch_add((FSS_GLOBAL uint32_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_word(const uint64_t *p) {
  return __hip_atomic_load((const FSS_GLOBAL uint64_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_word(uint64_t *p, uint32_t tag, float v) {
  __hip_atomic_store((FSS_GLOBAL uint64_t *)p, (static_cast<uint64_t>(tag) << 32) | as_u32(v), __ATOMIC_RELAXED,
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
  const char *in_x;       // gated backward only: the scan's input x (in_a is the gate there)
#ifdef FSS_TRACE
  uint64_t *trace;        // debug build: 8 timestamps per tile, written by lane 0 of every wave 0
#endif
};

// Optional (bs, d) fp32 rows of the scans with a state entering/leaving the sequence.
// The plain scan is compiled against the empty variant, whose members are constant
// nulls: it carries no kernel arguments for them and every use folds away.
template <bool STATE>
struct StateArgs {
  const float *state_in;  // forward: h[-1]; backward: gradient reaching the state after the last step
  float *state_out;       // forward: un-rounded state after the last step; backward: gradient w.r.t. h[-1]
  const float *h_before;  // backward only: h[-1] of the forward (grad_alpha[0] = g[0] * h[-1])
};
template <>
struct StateArgs<false> {
  static constexpr const float *state_in = nullptr;
  static constexpr float *state_out = nullptr;
  static constexpr const float *h_before = nullptr;
};

// ---- the kernel ----------------------------------------------------------------

// Which streams are accessed non-temporally (bit 0: alpha, 1: beta/dout, 2: saved h,
// 3: h output of the forward, 4: gradient outputs of the backward).  Measured on
// MI355X at bs8 seq4096 d1024, forward and backward alternating: marking the
// three output streams and the backward's reads of h non-temporal takes the step
// from 134 us to 113 us; marking the reads of alpha, beta or dout as well is slower.
#ifndef FSS_NT_MASK
#define FSS_NT_MASK 28
#endif
constexpr bool kNtA = (FSS_NT_MASK & 1) != 0;
constexpr bool kNtB = (FSS_NT_MASK & 2) != 0;
constexpr bool kNtH = (FSS_NT_MASK & 4) != 0;
constexpr bool kNtOutFwd = (FSS_NT_MASK & 8) != 0;
constexpr bool kNtOutBwd = (FSS_NT_MASK & 16) != 0;

#ifdef FSS_TRACE
#define FSS_STAMP(c, p, slot)                                                                   \
  do {                                                                                          \
    if ((p).trace && (c).lane == 0 && (c).wave == (c).trace_wave)                                \
      (p).trace[(static_cast<size_t>((c).chunk) * (p).n_ctiles + (c).ctile) * 8 + (slot)] =       \
          __builtin_amdgcn_s_memrealtime();                                                         \
  } while (0)
#else
#define FSS_STAMP(c, p, slot) \
  do {                        \
  } while (0)
#endif

// What is fixed for a wave while it works on one tile.
struct TileCtx {
  int lane, wave, n_waves, look;
  int chunk, ctile;      // position of the tile: chunk of the sequence, column tile
  bool chained, last;    // more than one chunk in the sequence; this is the last one
  uint32_t tag;          // epoch of this launch
  int64_t tile_base;     // byte offset of (batch, row 0, first channel of the tile)
  int64_t chan_row;      // index of (batch, first channel of the tile) in a (bs, d) array; wave-uniform
  int64_t r0;            // first scan-order index of this wave's slice
  int64_t seq, row_bytes;
  uint32_t lane_off;     // byte offset of the lane's channels inside the tile's row segment
  bool col_ok;           // the lane's channels exist (d % VEC == 0, so all or none)
  float2 *lds_map;       // [wave][v][lane] = (A, B) of this tile
  float2 *lds_pred;      // [look wave][v][lane] = what an earlier chunk offers
  float *lds_hin;        // [v][lane] = the chunk's incoming state, for every wave to read
  uint32_t *s_kind;      // [look wave] kind of that offer
  uint32_t *s_resolved;  // look-back finished (one word per workgroup)
#ifdef FSS_TRACE
  int trace_wave;
#endif
};

// One look at what chunk `j` of this column tile offers: its outgoing state if it
// has published one, else (j > 0) its map.  Split in two so that other work can be
// placed between the loads and the use of what they return.
template <int VEC>
struct ChunkWords {
  uint64_t a[VEC], b[VEC], s[VEC];
};

template <int VEC>
__device__ __forceinline__ void poll_issue(const ScanArgs &p, const TileCtx &c, int j, ChunkWords<VEC> &w) {
  const uint64_t *theirs = p.words + (static_cast<size_t>(j) * p.n_ctiles + c.ctile) * 3 * (64 * VEC) + c.lane;
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    w.s[v] = ld_word(theirs + (2 * VEC + v) * 64);
    w.a[v] = ld_word(theirs + (0 * VEC + v) * 64);
    w.b[v] = ld_word(theirs + (1 * VEC + v) * 64);
  }
}

// The answer is taken for the whole wave, so that one word per wave can describe
// it.  Returns kPredNone when neither a state nor a map is there yet.
template <int VEC>
__device__ __forceinline__ uint32_t poll_eval(const TileCtx &c, int j, const ChunkWords<VEC> &w, float *qA,
                                              float *qB) {
  bool have_state = true, have_map = true;
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    have_state = have_state && word_tag(w.s[v]) == c.tag;
    have_map = have_map && word_tag(w.a[v]) == c.tag && word_tag(w.b[v]) == c.tag;
  }
  if (__builtin_amdgcn_ballot_w64(have_state) == ~0ull) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      qA[v] = 0.0f;
      qB[v] = word_val(w.s[v]);
    }
    return kPredState;
  }
  if (j > 0 && __builtin_amdgcn_ballot_w64(have_map) == ~0ull) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      qA[v] = word_val(w.a[v]);
      qB[v] = word_val(w.b[v]);
    }
    return kPredMap;
  }
  return kPredNone;
}

template <int VEC>
__device__ __forceinline__ uint32_t poll_chunk(const ScanArgs &p, const TileCtx &c, int j, float *qA,
                                               float *qB) {
  ChunkWords<VEC> w;
  poll_issue<VEC>(p, c, j, w);
  return poll_eval<VEC>(c, j, w, qA, qB);
}

// (A, B) <- map[count-1] o ... o map[0] for this lane's channels: the maps of the
// first `count` waves of the workgroup composed in scan order.  Reads go out in
// small batches so that their LDS latencies overlap.
template <int VEC>
__device__ __forceinline__ void fold_wave_maps(const float2 *lds_map, int lane, int count, float *A,
                                               float *B) {
  constexpr int kBatch = 4;
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    A[v] = 1.0f;
    B[v] = 0.0f;
  }
  for (int w0 = 0; w0 < count; w0 += kBatch) {
    float2 m[kBatch][VEC];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const int w = w0 + i < count ? w0 + i : count - 1;  // clamped: the read stays in bounds
#pragma unroll
      for (int v = 0; v < VEC; ++v) m[i][v] = lds_map[(w * VEC + v) * 64 + lane];
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      if (w0 + i < count) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          B[v] = __builtin_fmaf(m[i][v].x, B[v], m[i][v].y);
          A[v] *= m[i][v].x;
        }
      }
    }
  }
}

// Phase 2.  In: this wave's slice as the map x -> mA*x + mB.  Out: the state
// entering the slice.  Every wave of the workgroup must call it (barriers).
//
// After one barrier every wave composes the maps of the waves before it (its state
// is then one multiply-add away from the chunk's incoming state), and wave 0 composes
// all of them into the chunk's map and publishes it.  Meanwhile wave w (w < look)
// fetches what chunk-1-w offers - its outgoing state if it has one, else its map -
// so a look-back over `look` chunks costs one memory round trip instead of one per
// chunk; wave 0 folds what they found and hands the chunk's incoming state to all
// waves through LDS.  Chains longer than `look` repeat the fetch.
template <int VEC>
__device__ __forceinline__ void chain_chunks(const ScanArgs &p, const TileCtx &c, const float *mA,
                                             const float *mB, const float *seq_in, float *state) {
  constexpr int kLaneSlots = 64 * VEC;
  const int lane = c.lane, wave = c.wave;
#pragma unroll
  for (int v = 0; v < VEC; ++v) c.lds_map[(wave * VEC + v) * 64 + lane] = make_float2(mA[v], mB[v]);
  __syncthreads();
  FSS_STAMP(c, p, 2);

  const bool look_back = c.chained && c.chunk > 0;
  uint64_t *mine = nullptr;
  float cA[VEC], cB[VEC];
  if (wave == 0 && c.chained && !c.last) {
    // the chunk's own map, needed by later chunks: out as early as possible
    fold_wave_maps<VEC>(c.lds_map, lane, c.n_waves, cA, cB);
    mine = p.words + (static_cast<size_t>(c.chunk) * p.n_ctiles + c.ctile) * 3 * kLaneSlots + lane;
    if (c.chunk > 0) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        st_word(mine + (0 * VEC + v) * 64, c.tag, cA[v]);
        st_word(mine + (1 * VEC + v) * 64, c.tag, cB[v]);
      }
    }
  }
  FSS_STAMP(c, p, 3);

  // (pA, pB): what the waves before this one do to the chunk's incoming state
  float pA[VEC], pB[VEC];
  if (!look_back) fold_wave_maps<VEC>(c.lds_map, lane, wave, pA, pB);

  if (!look_back) {
    // first chunk of the sequence (or the only one): the incoming state is the
    // sequence's own (0 in the plain scan)
    if (wave == 0 && c.chained && !c.last) {
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        st_word(mine + (2 * VEC + v) * 64, c.tag, seq_in ? __builtin_fmaf(cA[v], seq_in[v], cB[v]) : cB[v]);
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) state[v] = seq_in ? __builtin_fmaf(pA[v], seq_in[v], pB[v]) : pB[v];
    FSS_STAMP(c, p, 5);
    return;
  }

  float hin[VEC], accA[VEC], accB[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    accA[v] = 1.0f;
    accB[v] = hin[v] = 0.0f;
  }
  int nearest = c.chunk - 1;  // nearest earlier chunk not folded yet
  for (;;) {
    const int j = nearest - wave;
    if (wave < c.look && j >= 0) {
      float qA[VEC], qB[VEC];
      uint32_t kind = kPredNone;
      uint32_t polls = 0;
      while ((kind = poll_chunk<VEC>(p, c, j, qA, qB)) == kPredNone) {
        if (++polls > kSpinLimit) {
          if (lane == 0) st_u32(p.hdr + HDR_ERROR, 1u);
          kind = kPredState;  // give up: zero state, so that the grid still drains
#pragma unroll
          for (int v = 0; v < VEC; ++v) qA[v] = qB[v] = 0.0f;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) c.lds_pred[(wave * VEC + v) * 64 + lane] = make_float2(qA[v], qB[v]);
      if (lane == 0) c.s_kind[wave] = kind;
    }
    __syncthreads();
    if (wave == 0) {
      bool resolved = false;
      for (int w = 0; w < c.look && nearest - w >= 0 && !resolved; ++w) {
        const bool is_state = c.s_kind[w] == kPredState;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float2 m = c.lds_pred[(w * VEC + v) * 64 + lane];
          if (is_state) {
            hin[v] = __builtin_fmaf(accA[v], m.y, accB[v]);
          } else {
            accB[v] = __builtin_fmaf(accA[v], m.y, accB[v]);
            accA[v] *= m.x;
          }
        }
        resolved = is_state;
      }
      if (resolved) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) c.lds_hin[v * 64 + lane] = hin[v];
        if (!c.last) {
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            st_word(mine + (2 * VEC + v) * 64, c.tag, __builtin_fmaf(cA[v], hin[v], cB[v]));
        }
      }
      if (lane == 0) *c.s_resolved = resolved ? 1u : 0u;
    }
    __syncthreads();
    if (*c.s_resolved != 0u) break;  // chunk 0 always offers a state, so this is reached
    nearest -= c.look;
    if (nearest < 0) {  // cannot happen; never spin on a logic error
      if (threadIdx.x == 0) st_u32(p.hdr + HDR_ERROR, 1u);
      break;
    }
  }
  FSS_STAMP(c, p, 4);
  fold_wave_maps<VEC>(c.lds_map, lane, wave, pA, pB);  // after the polls: those are what is waited for
#pragma unroll
  for (int v = 0; v < VEC; ++v) state[v] = __builtin_fmaf(pA[v], c.lds_hin[v * 64 + lane], pB[v]);
  FSS_STAMP(c, p, 5);
}

// One tile, all three phases.  FULL: every row this wave touches exists and is
// interior and every lane has channels, so nothing is predicated; otherwise every
// access is guarded.  The two variants share no registers, so the guarded one
// costs the fast one nothing.
template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool FULL>
__device__ __forceinline__ void scan_tile(const ScanArgs &p, const StateArgs<STATE> &st, const TileCtx &c) {
  using RowT = Row<E, VEC>;
  const int64_t seq = c.seq, row_bytes = c.row_bytes, r0 = c.r0;
  const uint32_t lane_off = c.lane_off;

  RowT a[STEPS], b[STEPS];
  RowT hp[BWD ? STEPS : 1];

  // scan-order index r -> row: forward t = r; backward t = seq-1-r, with alpha taken
  // from row t+1 and the saved h from row t-1
  const int64_t t_first = BWD ? seq - 1 - r0 : r0;
  gcptr_t pa = (gcptr_t)p.in_a + c.tile_base + (BWD ? t_first + 1 : t_first) * row_bytes;
  gcptr_t pb = (gcptr_t)p.in_b + c.tile_base + t_first * row_bytes;
  const int64_t step_bytes = BWD ? -row_bytes : row_bytes;  // one step in scan order

  FSS_STAMP(c, p, 0);
  // ---- phase 1a: issue every load of the slice -------------------------------------
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    if (FULL) {
      // The scan's very first step (r = 0) has no predecessor: its coefficient is replaced
      // below, whatever is loaded here.  The backward would find it one row past the end
      // of the sequence, so it loads the row before instead.
      const int row = (BWD && s == 0 && r0 == 0) ? 1 : s;
      a[s].template load<kNtA>(uniform_ptr(pa + row * step_bytes) + lane_off);
      b[s].template load<kNtB>(uniform_ptr(pb + s * step_bytes) + lane_off);
    } else {
      const int64_t r = r0 + s;
      // Outside the sequence the step is the identity map (a=1, b=0).  The first step
      // of the plain scan has no predecessor (a=0), whatever alpha holds there; with a
      // state coming in, the forward applies alpha[0] to it and the backward adds it (a=1).
      a[s].fill((r >= seq || (STATE && BWD && r == 0 && st.state_in)) ? 1.0f : 0.0f);
      b[s].fill(0.0f);
      if (c.col_ok && r < seq) {
        if (r >= 1 || (STATE && !BWD && st.state_in))
          a[s].template load<kNtA>(uniform_ptr(pa + s * step_bytes) + lane_off);
        b[s].template load<kNtB>(uniform_ptr(pb + s * step_bytes) + lane_off);
      }
    }
  }

  if (FULL && r0 == 0) {
    // no predecessor: coefficient 0 - or, with a state coming in, alpha[0] as loaded
    // (forward) resp. 1, since the incoming gradient is added (backward)
    if (BWD)
      a[0].fill((STATE && st.state_in) ? 1.0f : 0.0f);
    else if (!(STATE && st.state_in))
      a[0].fill(0.0f);
  }

  // The backward's third stream, h[t-1], only feeds phase 3.  Its first kHEarly rows go
  // out now, behind the other two streams; the rest are loaded during phase 3 into
  // the registers that the steps already done have released, which is what lets a
  // lane of the backward hold as many timesteps as one of the forward.
  constexpr int kHEarly = (BWD && STEPS * Row<E, VEC>::kDwords > 16) ? STEPS / 2 : STEPS;
  gcptr_t ph = BWD ? (gcptr_t)p.in_h + c.tile_base + (t_first - 1) * row_bytes : (gcptr_t) nullptr;
  auto load_h = [&](int s) {
    if (FULL) {
      hp[s].template load<kNtH>(uniform_ptr(ph + s * step_bytes) + lane_off);
    } else {
      hp[s].fill(0.0f);
      if (c.col_ok && r0 + s < seq - 1)  // t - 1 >= 0
        hp[s].template load<kNtH>(uniform_ptr(ph + s * step_bytes) + lane_off);
    }
  };
  if (BWD) {
#pragma unroll
    for (int s = 0; s < kHEarly; ++s) load_h(s);
  }


  // the state the whole sequence starts from: only its first chunk needs it
  float seq_in[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) seq_in[v] = 0.0f;
  if (STATE && st.state_in && c.chunk == 0 && c.col_ok) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) seq_in[v] = st.state_in[c.chan_row + c.lane * VEC + v];
  }

  float state[VEC];
  if (!c.chained && c.n_waves == 1) {
    // the slice is the whole sequence: nothing to chain
#pragma unroll
    for (int v = 0; v < VEC; ++v) state[v] = seq_in[v];
  } else {
    // ---- phase 1b: the slice as an affine map ----------------------------------------
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
    FSS_STAMP(c, p, 1);
    chain_chunks<VEC>(p, c, mA, mB, STATE ? seq_in : nullptr, state);
  }

  // ---- phase 3: the recurrence from the true incoming state, in order ---------------
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    keep_packed(a[s]);
    keep_packed(b[s]);
    if (BWD && s < kHEarly) keep_packed(hp[s]);
  }
  gptr_t po0 = (gptr_t)p.out0 + c.tile_base + t_first * row_bytes;
  gptr_t po1 = BWD ? (gptr_t)p.out1 + c.tile_base + t_first * row_bytes : (gptr_t) nullptr;
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    float ga[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      state[v] = __builtin_fmaf(a[s].get(v), state[v], b[s].get(v));
      if (BWD) ga[v] = state[v] * hp[s].get(v);
    }
    const int64_t r = r0 + s;
    if (FULL || (c.col_ok && r < seq)) {
      RowT o;
      o.pack(state);
      o.template store<(BWD ? kNtOutBwd : kNtOutFwd)>(uniform_ptr(po0 + s * step_bytes) + lane_off);
      if (BWD) {
        if (!FULL && r == seq - 1) {  // t = 0: grad_alpha[0] = g[0] * h[-1], 0 in the plain scan
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            ga[v] = (STATE && st.h_before) ? state[v] * st.h_before[c.chan_row + c.lane * VEC + v] : 0.0f;
        }
        RowT oa;
        oa.pack(ga);
        oa.template store<kNtOutBwd>(uniform_ptr(po1 + s * step_bytes) + lane_off);
      }
    }
    if (BWD && s + kHEarly < STEPS) load_h(s + kHEarly);
  }
  // The wave whose slice holds the last step of the scan hands out the final state: the
  // forward as it is (the steps past the end are identity maps), the backward times
  // alpha[0] (the gradient with respect to h[-1]).
  if (STATE && st.state_out && c.col_ok && r0 <= seq - 1 && seq - 1 < r0 + STEPS) {
    if (BWD) {
      RowT a0;
      a0.template load<false>((gcptr_t)p.in_a + c.tile_base + lane_off);
#pragma unroll
      for (int v = 0; v < VEC; ++v) st.state_out[c.chan_row + c.lane * VEC + v] = a0.get(v) * state[v];
    } else {
#pragma unroll
      for (int v = 0; v < VEC; ++v) st.state_out[c.chan_row + c.lane * VEC + v] = state[v];
    }
  }
  FSS_STAMP(c, p, 6);
}

// Two-level completion count (16 first-level counters on separate lines keep the
// atomics off one hot address).  Whoever counts last knows that no workgroup will
// read the workspace again and advances the epoch for the next launch.
__device__ __forceinline__ void count_out(const ScanArgs &p, const TileCtx &c) {
  if (c.chained && threadIdx.x == 0) {
    const uint32_t slot = blockIdx.x % kDoneSlots;
    const uint32_t in_slot = (gridDim.x - slot + kDoneSlots - 1) / kDoneSlots;
    uint32_t *counter = p.hdr + HDR_SLOT0 + slot * HDR_SLOT_STRIDE;
    if (add_u32(counter, 1u) == in_slot - 1) {
      st_u32(counter, 0u);
      const uint32_t slots_used = gridDim.x < kDoneSlots ? gridDim.x : kDoneSlots;
      if (add_u32(p.hdr + HDR_DONE, 1u) == slots_used - 1) {
        st_u32(p.hdr + HDR_DONE, 0u);
        // 0 is the tag of never-written words: skip it when the counter wraps
        st_u32(p.hdr + HDR_EPOCH, c.tag + 1u == 0u ? 1u : c.tag + 1u);
      }
    }
  }
}

// ---- the gated scan --------------------------------------------------------------
//
//   alpha[t] = sigmoid(gate[t]),  beta[t] = x[t] * sqrt(1 - alpha[t]^2),  h = scan(alpha, beta)
//
// computed from the pre-activations inside the scan's own tile, so alpha and beta
// never exist in memory.  alpha and beta are rounded to the storage type where the
// plain scan would have read them from memory (they stay packed in registers), so
// the result is that of the plain scan on the rounded alpha and beta.

// 1/(1 + 2^(-z log2 e)): one exp2 and one reciprocal instruction, about 1 ulp each.
// +-inf and large |z| saturate to exactly 0 or 1.
__device__ __forceinline__ float sigmoid_f32(float z) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
}

// One tile of the gated scan.  Forward: in_a = gate, in_b = x, out0 = h.
// Backward: in_a = gate, in_b = dout, in_h = stored h, in_x = x, out0 = grad_x,
// out1 = grad_gate, with g the reversed-time scan of dout under alpha:
//   grad_x[t]    = g[t] * s[t]                                     s = sqrt(1 - alpha^2)
//   grad_gate[t] = g[t] * (h[t-1] - x[t]*alpha[t]/s[t]) * alpha[t]*(1 - alpha[t])
// (h[-1] = 0; the x term is dropped where alpha rounds to exactly 1, i.e. s = 0).
// The backward needs alpha[t+1] as the coefficient of step t and alpha[t] for its
// elementwise part: a slice of STEPS steps loads STEPS+1 rows of the gate.
template <typename E, int VEC, int STEPS, bool BWD, bool FULL>
__device__ __forceinline__ void gated_tile(const ScanArgs &p, const TileCtx &c) {
  using RowT = Row<E, VEC>;
  const int64_t seq = c.seq, row_bytes = c.row_bytes, r0 = c.r0;
  const uint32_t lane_off = c.lane_off;
  constexpr int kARows = BWD ? STEPS + 1 : STEPS;

  RowT a[kARows], b[STEPS];
  RowT hp[BWD ? STEPS : 1], xs[BWD ? STEPS : 1];

  // forward: a[s] = gate row t = r0+s.  backward: a[s] = gate row t+1 = seq-(r0+s), s = 0..STEPS
  const int64_t t_first = BWD ? seq - 1 - r0 : r0;
  gcptr_t pa = (gcptr_t)p.in_a + c.tile_base + (BWD ? t_first + 1 : t_first) * row_bytes;
  gcptr_t pb = (gcptr_t)p.in_b + c.tile_base + t_first * row_bytes;
  const int64_t step_bytes = BWD ? -row_bytes : row_bytes;

  // ---- phase 1a: loads ---------------------------------------------------------------
#pragma unroll
  for (int s = 0; s < kARows; ++s) {
    const int64_t r = r0 + s;
    // the gate row of a[s] exists: forward r < seq; backward 1 <= r <= seq
    const bool a_ok = FULL || (c.col_ok && (BWD ? (r >= 1 && r <= seq) : (r < seq)));
    if (!FULL) a[s].fill(0.0f);
    if (a_ok) a[s].template load<kNtA>(uniform_ptr(pa + s * step_bytes) + lane_off);
    if (s < STEPS) {
      if (!FULL) b[s].fill(0.0f);
      if (FULL || (c.col_ok && r < seq)) b[s].template load<kNtB>(uniform_ptr(pb + s * step_bytes) + lane_off);
    }
  }
  // x and the saved h only feed phase 3 of the backward: half of their rows now, the
  // rest during phase 3 into registers that finished steps have released
  constexpr int kEarly = BWD ? (STEPS >= 16 ? STEPS / 2 : STEPS) : 0;
  gcptr_t ph = BWD ? (gcptr_t)p.in_h + c.tile_base + (t_first - 1) * row_bytes : (gcptr_t) nullptr;
  gcptr_t px = BWD ? (gcptr_t)p.in_x + c.tile_base + t_first * row_bytes : (gcptr_t) nullptr;
  auto load_hx = [&](int s) {
    if (FULL) {
      hp[s].template load<kNtH>(uniform_ptr(ph + s * step_bytes) + lane_off);
      xs[s].template load<kNtH>(uniform_ptr(px + s * step_bytes) + lane_off);
    } else {
      hp[s].fill(0.0f);
      xs[s].fill(0.0f);
      if (c.col_ok && r0 + s < seq - 1)  // t - 1 >= 0
        hp[s].template load<kNtH>(uniform_ptr(ph + s * step_bytes) + lane_off);
      if (c.col_ok && r0 + s < seq) xs[s].template load<kNtH>(uniform_ptr(px + s * step_bytes) + lane_off);
    }
  };
  if (BWD) {
#pragma unroll
    for (int s = 0; s < kEarly; ++s) load_hx(s);
  }

  // ---- phase 1b: gate -> alpha (and x -> beta), in place; the slice as an affine map ----
  // The coefficient of a step outside the sequence is 1 (identity).  The first step of
  // the scan starts from a zero state, so its coefficient is immaterial as long as it
  // is finite: it is sigmoid(gate[0]) in the forward and sigmoid(0) in the backward.
  float mA[VEC], mB[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    mA[v] = 1.0f;
    mB[v] = 0.0f;
  }
#pragma unroll
  for (int s = 0; s < kARows; ++s) {
    const int64_t r = r0 + s;
    float al[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) al[v] = sigmoid_f32(a[s].get(v));
    if (!FULL && (r >= seq + (BWD ? 1 : 0) || !c.col_ok)) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) al[v] = 1.0f;
    }
    a[s].pack(al);
    if (s < STEPS) {
      if (!BWD) {
        float be[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          const float ar = a[s].get(v);  // as rounded
          be[v] = b[s].get(v) * __builtin_amdgcn_sqrtf(__builtin_fmaf(-ar, ar, 1.0f));
        }
        b[s].pack(be);  // rows outside the sequence hold x = 0, so beta = 0 there
      }
      // one step at a time: left to itself the compiler interleaves the gating of many steps
      // (for the latency of exp2/rcp/sqrt) and runs out of registers at 32 steps per lane
      keep_packed(a[s]);
      keep_packed(b[s]);
      const bool ident = !FULL && BWD && r >= seq;  // backward: a[s] with r == seq is alpha[0], not a coefficient
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float av = ident ? 1.0f : a[s].get(v);
        mB[v] = __builtin_fmaf(av, mB[v], b[s].get(v));
        mA[v] *= av;
      }
    }
  }

  float state[VEC];
  if (!c.chained && c.n_waves == 1) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) state[v] = 0.0f;
  } else {
    chain_chunks<VEC>(p, c, mA, mB, nullptr, state);
  }

  // ---- phase 3 -------------------------------------------------------------------------
#pragma unroll
  for (int s = 0; s < kARows; ++s) keep_packed(a[s]);
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    keep_packed(b[s]);
    if (BWD && s < kEarly) {
      keep_packed(hp[s]);
      keep_packed(xs[s]);
    }
  }
  gptr_t po0 = (gptr_t)p.out0 + c.tile_base + t_first * row_bytes;
  gptr_t po1 = BWD ? (gptr_t)p.out1 + c.tile_base + t_first * row_bytes : (gptr_t) nullptr;
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int64_t r = r0 + s;
    const bool ident = !FULL && BWD && r >= seq;
    float o0[VEC], o1[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      state[v] = __builtin_fmaf(ident ? 1.0f : a[s].get(v), state[v], b[s].get(v));
      if (BWD) {
        const float at = a[s + 1].get(v);  // alpha[t]
        const float om = __builtin_fmaf(-at, at, 1.0f);
        const float rs = om > 0.0f ? __builtin_amdgcn_rsqf(om) : 0.0f;
        o0[v] = state[v] * (om * rs);
        const float inner = __builtin_fmaf(-xs[s].get(v) * at, rs, hp[s].get(v));
        o1[v] = state[v] * inner * (at - at * at);
      } else {
        o0[v] = state[v];
      }
    }
    if (FULL || (c.col_ok && r < seq)) {
      RowT o;
      o.pack(o0);
      o.template store<(BWD ? kNtOutBwd : kNtOutFwd)>(uniform_ptr(po0 + s * step_bytes) + lane_off);
      if (BWD) {
        RowT oz;
        oz.pack(o1);
        oz.template store<kNtOutBwd>(uniform_ptr(po1 + s * step_bytes) + lane_off);
      }
    }
    if (BWD && s + kEarly < STEPS) load_hx(s + kEarly);
  }
}

// STATE: the variant that honours the optional incoming/outgoing state rows of ScanArgs;
// the plain scan is compiled without them.  GATED: the gated scan (never with STATE).
template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool GATED = false>
__global__ __launch_bounds__(1024) void scan_kernel(const ScanArgs p, const StateArgs<STATE> st) {
  constexpr int kLaneSlots = 64 * VEC;  // channels per tile

  extern __shared__ float lds[];
  __shared__ uint32_t s_kind[kMaxLookWaves];
  __shared__ uint32_t s_resolved;

  TileCtx c;
  c.lane = threadIdx.x & 63;
  c.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  c.n_waves = blockDim.x >> 6;
  c.look = p.look_waves;
  // LDS: two sets of per-wave maps (tiles alternate between them, so a wave that runs
  // ahead into the next tile cannot overwrite a map a slower wave still reads), then
  // the slots the look-back waves fill, then two rows for the chunk's incoming state
  float2 *const lds_maps = reinterpret_cast<float2 *>(lds);
  c.lds_pred = lds_maps + 2 * c.n_waves * kLaneSlots;
  float *const lds_hins = reinterpret_cast<float *>(c.lds_pred + c.look * kLaneSlots);
  c.s_kind = s_kind;
  c.s_resolved = &s_resolved;
  c.seq = p.seq;
  c.row_bytes = p.d * E::kBytes;
  c.lane_off = static_cast<uint32_t>(c.lane * Row<E, VEC>::kBytes);
#ifdef FSS_TRACE
  c.trace_wave = FSS_TRACE_WAVE < 0 ? c.n_waves - 1 : FSS_TRACE_WAVE;
#endif

#ifdef FSS_RESIDENCY_PROBE
  // debug build only: header words 8/9 = workgroups resident now / the most ever seen
  if (threadIdx.x == 0 && p.hdr) {
    const uint32_t now = add_u32(p.hdr + 8, 1u) + 1u;
    __hip_atomic_fetch_max(p.hdr + 9, now, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#endif
  c.chained = p.n_chunks > 1;
  // every workgroup of a launch reads the same value: it only changes when all are done
  c.tag = c.chained ? __builtin_amdgcn_readfirstlane(ld_u32(p.hdr + HDR_EPOCH)) : 0u;

  // The grid is sized to be resident all at once; each workgroup walks tiles
  // blockIdx, blockIdx + gridDim, ...  Tiles are numbered chunk-major, so a tile
  // only ever waits for tiles with smaller numbers: those belong to a resident
  // workgroup that reaches them no later than this one reaches its own.
  uint32_t parity = 0;
  for (uint32_t tile = blockIdx.x; tile < static_cast<uint32_t>(p.n_tiles); tile += gridDim.x, parity ^= 1u) {
    c.lds_map = lds_maps + parity * c.n_waves * kLaneSlots;
    c.lds_hin = lds_hins + parity * kLaneSlots;
    // unsigned, wave-uniform arithmetic: stays on the scalar unit
    // (the compiler divides through a vector-unit reciprocal: pin the quotients back)
    const uint32_t chunk = __builtin_amdgcn_readfirstlane(tile / static_cast<uint32_t>(p.n_ctiles));
    const uint32_t ctile = tile - chunk * static_cast<uint32_t>(p.n_ctiles);
    const uint32_t batch = __builtin_amdgcn_readfirstlane(ctile / static_cast<uint32_t>(p.tiles_per_row));
    const uint32_t coltile = ctile - batch * static_cast<uint32_t>(p.tiles_per_row);
    c.chunk = static_cast<int>(chunk);
    c.ctile = static_cast<int>(ctile);
    c.last = c.chunk == p.n_chunks - 1;

    const int64_t col0 = static_cast<int64_t>(coltile) * kLaneSlots;  // first channel of the tile
    c.col_ok = col0 + c.lane * VEC < p.d;
    c.tile_base = (static_cast<int64_t>(batch) * c.seq * p.d + col0) * E::kBytes;
    c.chan_row = static_cast<int64_t>(batch) * p.d + col0;
    c.r0 = (static_cast<int64_t>(chunk) * c.n_waves + c.wave) * STEPS;

    // Forward touches rows r0..r0+STEPS-1; the backward additionally reads row t+1 (the
    // unpredicated variant handles r = 0 itself, except in the gated backward) and row t-1.
    const bool full = (col0 + kLaneSlots <= p.d) && (c.r0 >= ((GATED && BWD) ? 1 : 0)) &&
                      (BWD ? (c.r0 + STEPS <= c.seq - 1) : (c.r0 + STEPS <= c.seq));
    // wave-uniform, but waves of one workgroup may differ: both variants execute the
    // same barriers, so they meet
    if constexpr (GATED) {
      if (full)
        gated_tile<E, VEC, STEPS, BWD, true>(p, c);
      else
        gated_tile<E, VEC, STEPS, BWD, false>(p, c);
    } else {
      if (full)
        scan_tile<E, VEC, STEPS, BWD, STATE, true>(p, st, c);
      else
        scan_tile<E, VEC, STEPS, BWD, STATE, false>(p, st, c);
    }
  }

#ifdef FSS_RESIDENCY_PROBE
  if (threadIdx.x == 0 && p.hdr) __hip_atomic_fetch_sub(p.hdr + 8, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
  count_out(p, c);
}

// ---- channel-major layout: (bs, d, seq), time contiguous ---------------------------
//
// Every (batch, channel) pair is a contiguous row of seq elements, so time runs
// across the lanes: a lane holds VEC consecutive timesteps of ROWS rows (one 16-byte
// load per row and tensor at full width), a wave 64*VEC consecutive timesteps of
// those rows, the waves of a workgroup consecutive slices of the same rows.  A lane
// folds its VEC steps into an affine map, a shuffle scan over the 64 lanes turns
// the maps into prefixes, and the last lane's prefix is the wave's map.  From
// there on the rows of a tile play the part the channels play in the row-major
// kernels: lane r carries row r's map into the same chain phase (other lanes carry
// identity maps), and gets back the state entering the wave's slice, which every
// lane then pushes through its own exclusive prefix before re-running its VEC steps.
// With 8 waves of 512 timesteps a workgroup covers 4096 timesteps, so sequences up
// to that length never touch the workspace.
//
// The backward runs over reversed time with lanes in scan order: lane l of slice k
// holds scan positions (k*64 + l)*VEC .. +VEC-1, i.e. timesteps descending from
// seq-1-(k*64+l)*VEC, and takes alpha[t+1] / h[t-1] of its first / last step from
// the neighbouring lane (or, at a slice edge, from a one-element load).

__device__ __forceinline__ float lane_read(float v, int lane) {
  return as_f32(__builtin_amdgcn_readlane(as_u32(v), lane));
}

template <typename E, int VEC, int ROWS, bool BWD>
__device__ __forceinline__ void cm_tile(const ScanArgs &p, const TileCtx &c, int64_t row0, int64_t n_rows) {
  using RowT = Row<E, VEC>;
  using OneT = Row<E, 1>;
  const int64_t seq = c.seq;
  const int lane = c.lane;
  const int64_t slice = static_cast<int64_t>(c.chunk) * c.n_waves + c.wave;
  const int64_t r_base = (slice * 64 + lane) * VEC;             // first scan position of this lane
  const bool in_seq = r_base < seq;                             // seq % VEC == 0: all of the vector or none
  const int64_t t_lo = BWD ? seq - r_base - VEC : r_base;       // lowest timestep of the vector
  const int64_t t_hi = t_lo + VEC - 1;
  // wave-uniform base (the lowest timestep any lane of the slice holds) + a 32-bit lane offset
  const int64_t t_base = BWD ? seq - (slice * 64 + 64) * VEC : slice * 64 * VEC;
  const uint32_t lane_off = static_cast<uint32_t>((BWD ? 63 - lane : lane) * RowT::kBytes);

  RowT a[ROWS], b[ROWS], hp[BWD ? ROWS : 1];
  float edge_a[BWD ? ROWS : 1], edge_h[BWD ? ROWS : 1];
  bool ok[ROWS];

  // ---- phase 1a: loads ---------------------------------------------------------------
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t row = row0 + r;
    ok[r] = in_seq && row < n_rows;
    a[r].fill(1.0f);  // outside: identity steps
    b[r].fill(0.0f);
    if (BWD) hp[r].fill(0.0f);
    if (ok[r]) {
      const int64_t off = (row * seq + t_base) * E::kBytes;
      a[r].template load<kNtA>(uniform_ptr((gcptr_t)p.in_a + off) + lane_off);
      b[r].template load<kNtB>(uniform_ptr((gcptr_t)p.in_b + off) + lane_off);
      if (BWD) hp[r].template load<kNtH>(uniform_ptr((gcptr_t)p.in_h + off) + lane_off);
    }
  }
  if (BWD) {
    // alpha[t_hi+1] for the first step and h[t_lo-1] for the last one: from the
    // neighbouring lanes, except at the two ends of the wave's slice
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int64_t row = row0 + r;
      OneT ea, eh;
      ea.fill(0.0f);
      eh.fill(0.0f);
      if (lane == 0 && ok[r] && t_hi + 1 < seq) ea.load((gcptr_t)p.in_a + (row * seq + t_hi + 1) * E::kBytes);
      if (lane == 63 && ok[r] && t_lo >= 1) eh.load((gcptr_t)p.in_h + (row * seq + t_lo - 1) * E::kBytes);
      const float from_prev = __shfl_up(a[r].get(0), 1);        // lane-1 holds timesteps just above ours
      const float from_next = __shfl_down(hp[r].get(VEC - 1), 1);  // lane+1 holds timesteps just below ours
      edge_a[r] = lane == 0 ? ea.get(0) : from_prev;
      edge_h[r] = lane == 63 ? eh.get(0) : from_next;
    }
  }

  // coefficient, addend and saved h of scan step j of row r
  auto coef = [&](int r, int j) -> float {
    if (BWD) return j == 0 ? edge_a[BWD ? r : 0] : a[r].get(VEC - j);
    return a[r].get(j);
  };
  auto addend = [&](int r, int j) -> float { return b[r].get(BWD ? VEC - 1 - j : j); };
  auto h_prev = [&](int r, int j) -> float {
    return j == VEC - 1 ? edge_h[BWD ? r : 0] : hp[BWD ? r : 0].get(VEC - 2 - j > 0 ? VEC - 2 - j : 0);
  };
  // the scan's first step has no predecessor, whatever alpha holds there
  const bool first_lane = slice == 0 && lane == 0;

  // ---- phase 1b: lane maps, then inclusive prefixes over the lanes --------------------
  float A[ROWS], B[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    A[r] = 1.0f;
    B[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float av = (j == 0 && first_lane) ? 0.0f : coef(r, j);
      B[r] = __builtin_fmaf(av, B[r], addend(r, j));
      A[r] *= av;
    }
  }
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const float pa = __shfl_up(A[r], off), pb = __shfl_up(B[r], off);
      if (lane >= off) {
        B[r] = __builtin_fmaf(A[r], pb, B[r]);
        A[r] *= pa;
      }
    }
  }
  // lane r takes row r's wave map into the chain phase; the other lanes identity maps
  float mA = 1.0f, mB = 0.0f;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const float wa = lane_read(A[r], 63), wb = lane_read(B[r], 63);
    if (lane == r) {
      mA = wa;
      mB = wb;
    }
  }
  // exclusive prefixes: what the lanes before this one do to the slice's incoming state
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const float pa = __shfl_up(A[r], 1), pb = __shfl_up(B[r], 1);
    A[r] = lane == 0 ? 1.0f : pa;
    B[r] = lane == 0 ? 0.0f : pb;
  }

  float slice_in = 0.0f;
  if (c.chained || c.n_waves > 1) chain_chunks<1>(p, c, &mA, &mB, nullptr, &slice_in);

  // ---- phase 3 ---------------------------------------------------------------------------
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    keep_packed(a[r]);
    keep_packed(b[r]);
    if (BWD) keep_packed(hp[r]);
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    float state = __builtin_fmaf(A[r], lane_read(slice_in, r), B[r]);
    float o0[VEC], o1[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float av = (j == 0 && first_lane) ? 0.0f : coef(r, j);
      state = __builtin_fmaf(av, state, addend(r, j));
      o0[BWD ? VEC - 1 - j : j] = state;
      if (BWD) o1[VEC - 1 - j] = state * h_prev(r, j);
    }
    if (ok[r]) {
      const int64_t off = ((row0 + r) * seq + t_base) * E::kBytes;
      RowT o;
      o.pack(o0);
      o.template store<(BWD ? kNtOutBwd : kNtOutFwd)>(uniform_ptr((gptr_t)p.out0 + off) + lane_off);
      if (BWD) {
        RowT oa;
        oa.pack(o1);
        oa.template store<kNtOutBwd>(uniform_ptr((gptr_t)p.out1 + off) + lane_off);
      }
    }
  }
}

// ScanArgs here: seq = the contiguous length, d = number of rows (bs * channels),
// n_ctiles = ceil(rows / ROWS) row groups, n_chunks = ceil(seq / (waves*64*VEC)).
template <typename E, int VEC, int ROWS, bool BWD>
__global__ __launch_bounds__(1024) void cm_scan_kernel(const ScanArgs p) {
  extern __shared__ float lds[];
  __shared__ uint32_t s_kind[kMaxLookWaves];
  __shared__ uint32_t s_resolved;

  TileCtx c;
  c.lane = threadIdx.x & 63;
  c.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  c.n_waves = blockDim.x >> 6;
  c.look = p.look_waves;
  float2 *const lds_maps = reinterpret_cast<float2 *>(lds);  // laid out as in scan_kernel with one slot per lane
  c.lds_pred = lds_maps + 2 * c.n_waves * 64;
  float *const lds_hins = reinterpret_cast<float *>(c.lds_pred + c.look * 64);
  c.s_kind = s_kind;
  c.s_resolved = &s_resolved;
  c.seq = p.seq;
  c.row_bytes = 0;
  c.lane_off = 0;
  c.col_ok = true;
  c.tile_base = c.chan_row = c.r0 = 0;
#ifdef FSS_TRACE
  c.trace_wave = 0;
#endif
  c.chained = p.n_chunks > 1;
  c.tag = c.chained ? __builtin_amdgcn_readfirstlane(ld_u32(p.hdr + HDR_EPOCH)) : 0u;

  uint32_t parity = 0;
  for (uint32_t tile = blockIdx.x; tile < static_cast<uint32_t>(p.n_tiles); tile += gridDim.x, parity ^= 1u) {
    c.lds_map = lds_maps + parity * c.n_waves * 64;
    c.lds_hin = lds_hins + parity * 64;
    const uint32_t chunk = __builtin_amdgcn_readfirstlane(tile / static_cast<uint32_t>(p.n_ctiles));
    const uint32_t ctile = tile - chunk * static_cast<uint32_t>(p.n_ctiles);
    c.chunk = static_cast<int>(chunk);
    c.ctile = static_cast<int>(ctile);
    c.last = c.chunk == p.n_chunks - 1;
    cm_tile<E, VEC, ROWS, BWD>(p, c, static_cast<int64_t>(ctile) * ROWS, p.d);
  }
  count_out(p, c);
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
#ifdef FSS_TRACE
uint64_t *g_trace = nullptr;
#ifndef FSS_TRACE_WAVE
#define FSS_TRACE_WAVE 0
#endif
#endif

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Register budget: packed dwords a lane may hold per input tensor.
inline int max_vec_steps(int dtype) { return dtype != FSS_F32 ? 64 : 32; }  // vec*steps

// LDS: one (A,B) slot per lane and vector element for every wave, twice (tiles
// alternate between two sets), the same for every wave that looks back, and two
// rows of incoming states.
constexpr size_t kLdsBudget = 60 * 1024;
inline int look_waves(int waves, int vec) {
  int look = waves < kMaxLookWaves ? waves : kMaxLookWaves;
  while (look > 1 && static_cast<size_t>(2 * waves + look + 1) * vec * 512 > kLdsBudget) --look;
  return look;
}
inline size_t lds_bytes(int waves, int vec) {
  return static_cast<size_t>(2 * waves + look_waves(waves, vec) + 1) * vec * 512;
}

inline bool config_valid(const fss_config &c, int dtype, bool gated = false, int dir = FSS_FWD) {
  // the gated kernels exist for 4 bytes (or one element) per lane; their backward holds
  // four tensors, so at most 16 timesteps per lane
  if (gated && (c.vec > (dtype != FSS_F32 ? 2 : 1) || (dir == FSS_BWD && c.steps > 16))) return false;
  const bool vec_ok = dtype != FSS_F32 ? (c.vec == 1 || c.vec == 2 || c.vec == 4 || c.vec == 8)
                                        : (c.vec == 1 || c.vec == 2 || c.vec == 4);
  const bool steps_ok = c.steps == 8 || c.steps == 16 || c.steps == 32;
  if (!vec_ok || !steps_ok) return false;
  if (c.vec * c.steps > max_vec_steps(dtype)) return false;
  if (dtype != FSS_F32 && c.vec == 1 && c.steps > 32) return false;
  if (c.waves < 1 || c.waves > 16) return false;
  if (lds_bytes(c.waves, c.vec) > kLdsBudget) return false;
  return true;
}

// Fills the zero fields of `c`.  `align` is the common alignment in bytes of all
// tensors of the call.
void complete_config(fss_config &c, int64_t bs, int64_t seq, int64_t d, int dtype, int dir,
                     size_t align, bool gated = false) {
  // Choices below come from sweeps on MI355X over the five measured workloads
  // (bs8 d1024 seq512..8192, bs16 d512 seq2048, bs4 d2048 seq8192, bs2 d768
  // seq1024, bs1 d256 seq65521).  What they showed: 4 bytes per lane per load
  // (bf16 x2) with as many timesteps in registers as fit beats wider vectors;
  // 8 waves per workgroup (two workgroups per CU, one loading while the other
  // chains and stores) beats 16 unless the chain of chunks is long; with few
  // channels, one channel per lane (twice the column tiles) and shorter slices
  // put more waves in flight.
  const int esize = dtype != FSS_F32 ? 2 : 4;
  const int64_t channels = bs * d;
  if (c.vec == 0) {
    // 4 bytes per lane and load either way: two bf16 channels or one fp32 channel
    const bool can2 = dtype != FSS_F32 && d % 2 == 0 && align % (2 * static_cast<size_t>(esize)) == 0;
    int v = can2 ? 2 : 1;
    // few channels: more, narrower column tiles; also never pad a row to twice its width
    if (v == 2 && (channels < 8192 || ceil_div(d, 128) * 128 >= 2 * ceil_div(d, 64) * 64)) v = 1;
    // forward: if two channels per lane leave at most one tile per resident workgroup, the whole
    // scan is a single round of load - chain - store with nothing overlapping; one channel per
    // lane gives twice the tiles (measured 8-9 % faster at bs16 seq2048 d512 and bs8 seq2048 d1024)
    if (v == 2 && dir == FSS_FWD && bs * ceil_div(d, 128) * ceil_div(seq, 256) <= 512) v = 1;
    c.vec = v;
  }
  // packed dwords one lane holds per timestep and tensor
  const int dwords = dtype != FSS_F32 ? (c.vec + 1) / 2 : c.vec;
  if (c.steps == 0) {
    int s = 32 / dwords;  // 32 packed dwords per lane and tensor (the backward loads half of its third one late)
    if (s > 32) s = 32;
    if (s < 8) s = 8;
    // backward: 32-step slices cost it a dozen spilled registers per lane (5 % more HBM
    // traffic); that only pays where the chain of chunks is long.  Elsewhere 16 steps are
    // as fast in bf16 and 6 % faster in fp32 (forward and backward alternating).
    if (dir == FSS_BWD && s == 32 && (gated || ceil_div(seq, static_cast<int64_t>(8) * 32) <= 16)) s = 16;
    // small problems: shorter slices until there are two 8-wave tiles per CU (512), as
    // long as the machine still gets a few waves per SIMD out of it
    const int64_t ctiles = bs * ceil_div(d, 64 * c.vec);
    while (s > 16 && ctiles * ceil_div(seq, static_cast<int64_t>(8) * s) < 512) s >>= 1;
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
    // many channels but a short sequence: half-size workgroups to reach 512 tiles
    if (w == 8 && bs * ceil_div(d, 64 * c.vec) >= 64 &&
        bs * ceil_div(d, 64 * c.vec) * ceil_div(seq, static_cast<int64_t>(8) * c.steps) < 512)
      w = 4;
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
  if (dtype != FSS_BF16 && dtype != FSS_F32 && dtype != FSS_F16) return FSS_ERR_BAD_CONFIG;
  if (dir < FSS_FWD || dir > FSS_GATED_BWD) return FSS_ERR_BAD_CONFIG;
  const bool gated = dir >= FSS_GATED_FWD;
  dir &= 1;
  const int esize = dtype != FSS_F32 ? 2 : 4;
  // bs*seq*d*esize must fit int64
  if (bs > 0 && seq > 0 && d > 0) {
    const __int128 total = static_cast<__int128>(bs) * seq * d * esize;
    if (total > (static_cast<__int128>(1) << 62)) return FSS_ERR_BAD_SHAPE;
  }
  fss_config c = {0, 0, 0, 0};
  if (user) c = *user;
  if (c.max_groups < 0) return FSS_ERR_BAD_CONFIG;
  const int64_t dd = d > 0 ? d : 1, ss = seq > 0 ? seq : 1, bb = bs > 0 ? bs : 1;
  complete_config(c, bb, ss, dd, dtype, dir, align, gated);
  if (!config_valid(c, dtype, gated, dir)) return FSS_ERR_BAD_CONFIG;
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

// Scans of one process never overlap on a device.  A scan's workgroups wait for each
// other and its grid is sized to fill the device, so two scans sharing the device
// could each hold the compute units the other's unscheduled workgroups need, and
// both would sit there until their waits give up.  Launches on one stream are
// ordered anyway; when the stream changes, the new launch is made to wait for
// everything queued on the previous stream.  The lock is held across the launch, so
// that the event recorded by the next caller lands behind this one's kernel.
// Streams under graph capture are left alone (a captured scan is ordered by its
// graph; do not replay two graphs holding scans concurrently).
struct ScanOrder {
  std::mutex lock;
  hipStream_t last = nullptr;
  bool any = false;
  hipEvent_t event = nullptr;
};
ScanOrder g_scan_order[64];

inline bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &status) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // unknown: do not touch it
  }
  return status != hipStreamCaptureStatusNone;
}

class ScanOrderGuard {
 public:
  explicit ScanOrderGuard(hipStream_t s) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
    order_ = &g_scan_order[dev];
    order_->lock.lock();
    if (stream_is_capturing(s)) return;
    if (order_->any && order_->last != s && !stream_is_capturing(order_->last)) {
      if (!order_->event && hipEventCreateWithFlags(&order_->event, hipEventDisableTiming) != hipSuccess) {
        order_->event = nullptr;
        (void)hipGetLastError();
      }
      // a stream the caller has destroyed since makes the record fail: nothing to wait for then
      if (order_->event && hipEventRecord(order_->event, order_->last) == hipSuccess)
        (void)hipStreamWaitEvent(s, order_->event, 0);
      (void)hipGetLastError();
    }
    order_->last = s;
    order_->any = true;
  }
  ~ScanOrderGuard() {
    if (order_) order_->lock.unlock();
  }
  ScanOrderGuard(const ScanOrderGuard &) = delete;
  ScanOrderGuard &operator=(const ScanOrderGuard &) = delete;

 private:
  ScanOrder *order_ = nullptr;
};

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

template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool GATED = false>
int launch_one(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, hipStream_t stream) {
  // The kernel's waits are only safe if every workgroup of the grid is resident,
  // so the grid never exceeds what the device holds at once; workgroups loop.
  static int resident[17] = {0};  // by waves per workgroup; same answer on every call
  const int waves = pl.cfg.waves;
  const size_t lds = lds_bytes(waves, VEC);
  int fit = __atomic_load_n(&resident[waves], __ATOMIC_RELAXED);
  if (fit == 0) {
    fit = resident_workgroups(scan_kernel<E, VEC, STEPS, BWD, STATE, GATED>, waves, lds);
    if (fit <= 0) return FSS_ERR_LAUNCH;
    __atomic_store_n(&resident[waves], fit, __ATOMIC_RELAXED);
  }
  int64_t n_groups = pl.n_tiles < fit ? pl.n_tiles : fit;
  if (pl.cfg.max_groups > 0 && pl.cfg.max_groups < n_groups) n_groups = pl.cfg.max_groups;
  const dim3 grid(static_cast<uint32_t>(n_groups));
  const dim3 block(static_cast<uint32_t>(waves) * 64);
  StateArgs<STATE> st;
  if constexpr (STATE) st = state;
  hipLaunchKernelGGL((scan_kernel<E, VEC, STEPS, BWD, STATE, GATED>), grid, block, lds, stream, args, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

template <typename E, bool BWD, bool STATE>
int launch_typed(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, hipStream_t stream) {
  constexpr bool is_16bit = E::kBytes == 2;
  const int key = pl.cfg.vec * 100 + pl.cfg.steps;
  switch (key) {
#define FSS_CASE(V, S) \
  case V * 100 + S:    \
    return launch_one<E, V, S, BWD, STATE>(args, state, pl, stream);
    FSS_CASE(1, 8)
    FSS_CASE(1, 16)
    FSS_CASE(1, 32)
    FSS_CASE(2, 8)
    FSS_CASE(2, 16)
    FSS_CASE(4, 8)
    default:
      break;
  }
  if constexpr (is_16bit) {
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

// The gated kernels: 4 bytes (bf16 x2, fp32 x1) or one bf16 element per lane.
template <typename E, bool BWD>
int launch_gated(const ScanArgs &args, const Plan &pl, hipStream_t stream) {
  constexpr bool is_16bit = E::kBytes == 2;
  const StateArgs<true> none = {nullptr, nullptr, nullptr};
  const int key = pl.cfg.vec * 100 + pl.cfg.steps;
  switch (key) {
#define FSS_CASE(V, S) \
  case V * 100 + S:    \
    return launch_one<E, V, S, BWD, false, true>(args, none, pl, stream);
    FSS_CASE(1, 8)
    FSS_CASE(1, 16)
    default:
      break;
  }
  if constexpr (!BWD) {
    if (key == 132) return launch_one<E, 1, 32, BWD, false, true>(args, none, pl, stream);
  }
  if constexpr (is_16bit) {
    switch (key) {
      FSS_CASE(2, 8)
      FSS_CASE(2, 16)
      default:
        break;
    }
    if constexpr (!BWD) {
      if (key == 232) return launch_one<E, 2, 32, BWD, false, true>(args, none, pl, stream);
    }
  }
#undef FSS_CASE
  return FSS_ERR_BAD_CONFIG;
}

int run_scan(int dtype, int dir, const void *alpha, const void *in_b, const void *in_h, void *out0,
             void *out1, int64_t bs, int64_t seq, int64_t d, void *workspace, size_t workspace_bytes,
             void *stream, const fss_config *cfg, const float *state_in = nullptr,
             float *state_out = nullptr, const float *h_before = nullptr, const void *in_x = nullptr) {
  const bool gated = dir >= FSS_GATED_FWD;
  const int plan_dir = dir;
  dir &= 1;
  if (bs < 0 || seq < 0 || d < 0) return FSS_ERR_BAD_SHAPE;
  if (dtype != FSS_BF16 && dtype != FSS_F32 && dtype != FSS_F16) return FSS_ERR_BAD_CONFIG;
  if (bs == 0 || seq == 0 || d == 0) return FSS_OK;
  if (!alpha || !in_b || !out0) return FSS_ERR_NULL_POINTER;
  if (dir == FSS_BWD && (!in_h || !out1)) return FSS_ERR_NULL_POINTER;
  if (gated && dir == FSS_BWD && !in_x) return FSS_ERR_NULL_POINTER;
  const size_t esize = dtype != FSS_F32 ? 2 : 4;
  const size_t align = dir == FSS_BWD ? common_alignment({alpha, in_b, in_h, out0, out1, in_x})
                                      : common_alignment({alpha, in_b, out0});
  if (align < esize) return FSS_ERR_MISALIGNED;
  if ((reinterpret_cast<uintptr_t>(state_in) | reinterpret_cast<uintptr_t>(state_out) |
       reinterpret_cast<uintptr_t>(h_before)) % 4 != 0)
    return FSS_ERR_MISALIGNED;
  Plan pl;
  int rc = make_plan(pl, bs, seq, d, dtype, plan_dir, align, cfg);
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
  args.in_x = static_cast<const char *>(in_x);
  args.seq = seq;
  args.d = d;
  args.tiles_per_row = static_cast<int32_t>(pl.tiles_per_row);
  args.n_ctiles = static_cast<int32_t>(pl.n_ctiles);
  args.n_chunks = static_cast<int32_t>(pl.n_chunks);
  args.n_tiles = static_cast<int32_t>(pl.n_tiles);
  args.look_waves = look_waves(pl.cfg.waves, pl.cfg.vec);
  const StateArgs<true> state = {state_in, state_out, h_before};
  args.hdr = static_cast<uint32_t *>(workspace);
  args.words = workspace ? reinterpret_cast<uint64_t *>(static_cast<char *>(workspace) + kHeaderBytes) : nullptr;
#ifdef FSS_TRACE
  args.trace = g_trace;
#endif
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool st = state_in || state_out || h_before;
  const bool bwd = dir == FSS_BWD;
  const ScanOrderGuard ordered(s);
#define FSS_DISPATCH(E)                                                                        \
  do {                                                                                         \
    if (gated) return bwd ? launch_gated<E, true>(args, pl, s) : launch_gated<E, false>(args, pl, s); \
    if (bwd) return st ? launch_typed<E, true, true>(args, state, pl, s) : launch_typed<E, true, false>(args, state, pl, s); \
    return st ? launch_typed<E, false, true>(args, state, pl, s) : launch_typed<E, false, false>(args, state, pl, s); \
  } while (0)
  if (dtype == FSS_BF16) FSS_DISPATCH(BF16);
  if (dtype == FSS_F16) FSS_DISPATCH(F16);
  FSS_DISPATCH(F32);
#undef FSS_DISPATCH
}

// ---- channel-major host side ------------------------------------------------------------

// rows per wave: 4 bytes-per-lane budgets as in the row-major kernels (two tensors of
// 8 rows x 16 bytes forward, three of 4 rows backward)
constexpr int kCmRowsFwd = 8, kCmRowsBwd = 4;

struct CmPlan {
  int vec, waves;
  int64_t n_rowtiles, n_chunks, n_tiles;
  size_t ws_bytes;
};

int make_cm_plan(CmPlan &pl, int64_t rows, int64_t seq, int dtype, int dir, size_t align, const fss_config *user) {
  if (rows < 0 || seq < 0) return FSS_ERR_BAD_SHAPE;
  if (dtype != FSS_BF16 && dtype != FSS_F32 && dtype != FSS_F16) return FSS_ERR_BAD_CONFIG;
  if (dir != FSS_FWD && dir != FSS_BWD) return FSS_ERR_BAD_CONFIG;
  const int esize = dtype != FSS_F32 ? 2 : 4;
  const int64_t rr = rows > 0 ? rows : 1, ss = seq > 0 ? seq : 1;
  if (static_cast<__int128>(rr) * ss * esize > (static_cast<__int128>(1) << 62)) return FSS_ERR_BAD_SHAPE;
  const int widest = 16 / esize;  // 16 bytes per lane and load
  int vec = user ? user->vec : 0, waves = user ? user->waves : 0;
  if (user && (user->max_groups < 0 || user->steps != 0)) return FSS_ERR_BAD_CONFIG;
  if (vec == 0) {
    vec = widest;
    // rows start at multiples of seq elements: every row must keep the vectors aligned
    while (vec > 2 || (vec == 2 && esize == 4)) {
      if (ss % vec == 0 && align % (static_cast<size_t>(vec) * esize) == 0) break;
      vec = 2;  // only 1, 2 and the widest are compiled (fp32: 1 and 4)
      if (esize == 4) vec = 1;
    }
    if (vec == 2 && (ss % 2 != 0 || align % (2 * static_cast<size_t>(esize)) != 0)) vec = 1;
  }
  const bool vec_ok = vec == 1 || vec == widest || (vec == 2 && esize == 2);
  if (!vec_ok) return FSS_ERR_BAD_CONFIG;
  if (ss % vec != 0) return FSS_ERR_BAD_CONFIG;
  if (align % (static_cast<size_t>(vec) * esize) != 0) return FSS_ERR_MISALIGNED;
  if (waves == 0) {
    const int64_t w = ceil_div(ss, static_cast<int64_t>(64) * vec);
    waves = static_cast<int>(w < 8 ? w : 8);
  }
  if (waves < 1 || waves > 16) return FSS_ERR_BAD_CONFIG;
  pl.vec = vec;
  pl.waves = waves;
  pl.n_rowtiles = ceil_div(rr, dir == FSS_BWD ? kCmRowsBwd : kCmRowsFwd);
  pl.n_chunks = ceil_div(ss, static_cast<int64_t>(waves) * 64 * vec);
  pl.n_tiles = pl.n_rowtiles * pl.n_chunks;
  if (pl.n_rowtiles > INT32_MAX || pl.n_chunks > INT32_MAX || pl.n_tiles > INT32_MAX) return FSS_ERR_BAD_SHAPE;
  pl.ws_bytes = kHeaderBytes;
  if (pl.n_chunks > 1) pl.ws_bytes += static_cast<size_t>(pl.n_tiles) * 3 * 64 * sizeof(uint64_t);
  return FSS_OK;
}

template <typename E, int VEC, bool BWD>
int launch_cm_one(const ScanArgs &args, const CmPlan &pl, int max_groups, hipStream_t stream) {
  constexpr int kRows = BWD ? kCmRowsBwd : kCmRowsFwd;
  static int resident[17] = {0};
  const int waves = pl.waves;
  const size_t lds = lds_bytes(waves, 1);
  int fit = __atomic_load_n(&resident[waves], __ATOMIC_RELAXED);
  if (fit == 0) {
    fit = resident_workgroups(cm_scan_kernel<E, VEC, kRows, BWD>, waves, lds);
    if (fit <= 0) return FSS_ERR_LAUNCH;
    __atomic_store_n(&resident[waves], fit, __ATOMIC_RELAXED);
  }
  int64_t n_groups = pl.n_tiles < fit ? pl.n_tiles : fit;
  if (max_groups > 0 && max_groups < n_groups) n_groups = max_groups;
  hipLaunchKernelGGL((cm_scan_kernel<E, VEC, kRows, BWD>), dim3(static_cast<uint32_t>(n_groups)),
                     dim3(static_cast<uint32_t>(waves) * 64), lds, stream, args);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

template <typename E, bool BWD>
int launch_cm(const ScanArgs &args, const CmPlan &pl, int max_groups, hipStream_t stream) {
  constexpr int kWidest = 16 / E::kBytes;
  if (pl.vec == kWidest) return launch_cm_one<E, kWidest, BWD>(args, pl, max_groups, stream);
  if (pl.vec == 1) return launch_cm_one<E, 1, BWD>(args, pl, max_groups, stream);
  if constexpr (E::kBytes == 2) {
    if (pl.vec == 2) return launch_cm_one<E, 2, BWD>(args, pl, max_groups, stream);
  }
  return FSS_ERR_BAD_CONFIG;
}

int run_cm_scan(int dtype, int dir, const void *alpha, const void *in_b, const void *in_h, void *out0, void *out1,
                int64_t bs, int64_t d, int64_t seq, void *workspace, size_t workspace_bytes, void *stream,
                const fss_config *cfg) {
  if (bs < 0 || seq < 0 || d < 0) return FSS_ERR_BAD_SHAPE;
  if (dtype != FSS_BF16 && dtype != FSS_F32 && dtype != FSS_F16) return FSS_ERR_BAD_CONFIG;
  if (bs == 0 || seq == 0 || d == 0) return FSS_OK;
  if (bs > INT64_MAX / d) return FSS_ERR_BAD_SHAPE;
  if (!alpha || !in_b || !out0) return FSS_ERR_NULL_POINTER;
  if (dir == FSS_BWD && (!in_h || !out1)) return FSS_ERR_NULL_POINTER;
  const size_t esize = dtype != FSS_F32 ? 2 : 4;
  const size_t align = dir == FSS_BWD ? common_alignment({alpha, in_b, in_h, out0, out1})
                                      : common_alignment({alpha, in_b, out0});
  if (align < esize) return FSS_ERR_MISALIGNED;
  CmPlan pl;
  int rc = make_cm_plan(pl, bs * d, seq, dtype, dir, align, cfg);
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
  args.in_x = nullptr;
  args.seq = seq;
  args.d = bs * d;  // rows
  args.tiles_per_row = 1;
  args.n_ctiles = static_cast<int32_t>(pl.n_rowtiles);
  args.n_chunks = static_cast<int32_t>(pl.n_chunks);
  args.n_tiles = static_cast<int32_t>(pl.n_tiles);
  args.look_waves = look_waves(pl.waves, 1);
  args.hdr = static_cast<uint32_t *>(workspace);
  args.words = workspace ? reinterpret_cast<uint64_t *>(static_cast<char *>(workspace) + kHeaderBytes) : nullptr;
#ifdef FSS_TRACE
  args.trace = nullptr;
#endif
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int max_groups = cfg ? cfg->max_groups : 0;
  const bool bwd = dir == FSS_BWD;
  const ScanOrderGuard ordered(s);
  if (dtype == FSS_BF16) return bwd ? launch_cm<BF16, true>(args, pl, max_groups, s) : launch_cm<BF16, false>(args, pl, max_groups, s);
  if (dtype == FSS_F16) return bwd ? launch_cm<F16, true>(args, pl, max_groups, s) : launch_cm<F16, false>(args, pl, max_groups, s);
  return bwd ? launch_cm<F32, true>(args, pl, max_groups, s) : launch_cm<F32, false>(args, pl, max_groups, s);
}

}  // namespace fss

// ---- C ABI -------------------------------------------------------------------------

extern "C" {

#ifdef FSS_TRACE
void fss_debug_set_trace(void *p) { fss::g_trace = static_cast<uint64_t *>(p); }
#endif

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
  for (int dtype = FSS_BF16; dtype <= FSS_F16; ++dtype)
    for (int dir = FSS_FWD; dir <= FSS_GATED_BWD; ++dir)
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

int fss_scan_fwd_state(int dtype, const void *alpha, const void *beta, void *h, const float *h_before,
                       float *h_last, int64_t bs, int64_t seq, int64_t d, void *workspace,
                       size_t workspace_bytes, void *stream, const fss_config *cfg) {
  return fss::run_scan(dtype, FSS_FWD, alpha, beta, nullptr, h, nullptr, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg, h_before, h_last, nullptr);
}

int fss_scan_bwd_state(int dtype, const void *alpha, const void *h, const void *dout, const float *h_before,
                       const float *grad_h_last, void *grad_alpha, void *grad_beta, float *grad_h_before,
                       int64_t bs, int64_t seq, int64_t d, void *workspace, size_t workspace_bytes,
                       void *stream, const fss_config *cfg) {
  if (grad_h_before && !h_before) return FSS_ERR_NULL_POINTER;
  return fss::run_scan(dtype, FSS_BWD, alpha, dout, h, grad_beta, grad_alpha, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg, grad_h_last, grad_h_before, h_before);
}

int fss_gated_scan_fwd(int dtype, const void *gate, const void *x, void *h, int64_t bs, int64_t seq,
                       int64_t d, void *workspace, size_t workspace_bytes, void *stream,
                       const fss_config *cfg) {
  return fss::run_scan(dtype, FSS_GATED_FWD, gate, x, nullptr, h, nullptr, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg);
}

int fss_gated_scan_bwd(int dtype, const void *gate, const void *x, const void *h, const void *dout,
                       void *grad_gate, void *grad_x, int64_t bs, int64_t seq, int64_t d,
                       void *workspace, size_t workspace_bytes, void *stream, const fss_config *cfg) {
  return fss::run_scan(dtype, FSS_GATED_BWD, gate, dout, h, grad_x, grad_gate, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg, nullptr, nullptr, nullptr, x);
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

size_t fss_cm_workspace_bytes(int64_t bs, int64_t d, int64_t seq, int dtype, int dir, const fss_config *cfg) {
  fss::CmPlan pl;
  if (bs < 0 || d < 0 || (d > 0 && bs > INT64_MAX / d)) return fss::kHeaderBytes;
  // alignment unknown here: the narrowest vector gives the most chunks, hence the upper bound
  size_t best = fss::kHeaderBytes;
  for (size_t align = 2; align <= 16; align <<= 1)
    if (fss::make_cm_plan(pl, bs * d, seq, dtype, dir, align, cfg) == FSS_OK && pl.ws_bytes > best) best = pl.ws_bytes;
  return best;
}

int fss_scan_fwd_cm(int dtype, const void *alpha, const void *beta, void *h, int64_t bs, int64_t d, int64_t seq,
                    void *workspace, size_t workspace_bytes, void *stream, const fss_config *cfg) {
  return fss::run_cm_scan(dtype, FSS_FWD, alpha, beta, nullptr, h, nullptr, bs, d, seq, workspace, workspace_bytes,
                          stream, cfg);
}

int fss_scan_bwd_cm(int dtype, const void *alpha, const void *h, const void *dout, void *grad_alpha,
                    void *grad_beta, int64_t bs, int64_t d, int64_t seq, void *workspace, size_t workspace_bytes,
                    void *stream, const fss_config *cfg) {
  return fss::run_cm_scan(dtype, FSS_BWD, alpha, dout, h, grad_beta, grad_alpha, bs, d, seq, workspace,
                          workspace_bytes, stream, cfg);
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
