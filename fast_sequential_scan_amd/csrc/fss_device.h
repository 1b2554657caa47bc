// Device-side building blocks shared by the scan kernels: packed rows, the workspace
// words, and the chain phase that carries state from chunk to chunk.  See the
// comment at the top of fss_scan_rm.hip for how the kernels use them.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fss_scan.h"

#if defined(FSS_TRACE) && !defined(FSS_TRACE_WAVE)
#define FSS_TRACE_WAVE 0
#endif

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

// seq - r0 clamped to [-1, cap] as a wave-uniform 32-bit integer: how many steps of a slice
// that starts at scan-order index r0 lie inside the sequence.  With it, "r0 + s < seq" is
// "s < n", "r0 + s <= seq" is "s <= n" and so on for every step s >= 0 of the slice; -1
// (the slice starts beyond index seq) keeps "s <= n" false where 0 would make it true for s = 0.
__device__ __forceinline__ int slice_steps_inside(int64_t seq, int64_t r0, int cap) {
  const int64_t left = seq - r0;
  const int n = left < 0 ? -1 : (left >= cap ? cap : static_cast<int>(left));
  return __builtin_amdgcn_readfirstlane(n);
}

// A constant the compiler materialises where it is used.  Constants it recognises as
// loop-invariant are otherwise put into registers ahead of the tile loop and kept there for
// the whole kernel (or spilled, and reloaded in the middle of the look-back): four to six
// registers in kernels that have none to spare.
__device__ __forceinline__ float local_const(float x) {
  asm volatile("" : "+v"(x));
  return x;
}

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
// Header (kHeaderBytes): word 1 = top-level completion counter, word 2 = epoch (the tag
// of the next launch minus 1: an all-zero workspace is ready for use),
// word 3 = sticky error flag, words 4-5 = address of an optional 32-bit word the host
// can read without a device call (0: none), which a wave that gives up also sets,
// words 64+32*i (i < 16, one 128-byte line each) = first-level completion counters.
// Then the tagged words,
// [chunk][column tile][kind: map A, map B, outgoing state][VEC][64 lanes].

enum : int { HDR_DONE = 1, HDR_EPOCH = 2, HDR_ERROR = 3, HDR_FLAG_LO = 4, HDR_FLAG_HI = 5, HDR_SLOT0 = 64, HDR_SLOT_STRIDE = 32 };
constexpr int kDoneSlots = 16;
constexpr size_t kHeaderBytes = 4096;
// Polls a wave makes before it gives up on an earlier chunk (each poll is a memory
// round trip plus a sleep: seconds in total, far beyond any healthy wait).  The limit
// travels as a kernel argument so that a test can lower it from the host; 0 makes every
// look-back give up before its first poll.
constexpr uint32_t kSpinLimit = 1u << 20;
// Most waves of a workgroup that look back in parallel, one earlier chunk each.
constexpr int kMaxLookWaves = 16;
// chunks one look-back wave covers at most (measured: 2 -> 4 gains up to 12 % on chains of
// hundreds of chunks, 8 nothing more)
constexpr int kMaxSpan = 4;

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

// a*x + b where x is a state (or the constant part of a composed map) and a the
// coefficient it meets.  A coefficient that is a product of many |alpha| > 1 may have
// overflowed to inf while x is exactly 0; the sequential recurrence keeps such a state
// at 0, inf*0 would make it NaN.  (A NaN x - the mark of a look-back that gave up -
// still propagates.)
__device__ __forceinline__ float fma0(float a, float x, float b) {
  return x == 0.0f ? b : __builtin_fmaf(a, x, b);
}

// A wave that gives up on an earlier chunk: sticky error word, the host-visible word
// if one is attached, and (by the caller) a NaN state, so that every output from here
// to the end of the sequence is visibly poisoned.
__device__ __forceinline__ void report_timeout(uint32_t *hdr) {
  st_u32(hdr + HDR_ERROR, 1u);
  const uint64_t addr = (static_cast<uint64_t>(ld_u32(hdr + HDR_FLAG_HI)) << 32) | ld_u32(hdr + HDR_FLAG_LO);
  if (addr != 0)
    __hip_atomic_store(reinterpret_cast<uint32_t *>(addr), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

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
  int32_t n_tiles;        // tiles the workgroups walk: n_groups * n_chunks
  int32_t n_groups;       // column groups per chunk: n_ctiles / wg_cols
  int32_t wg_cols;        // adjacent column tiles a workgroup covers side by side (1 or 2)
  int32_t look_waves;     // waves per column tile that look back in parallel (1..kMaxLookWaves)
  int32_t period;         // chunks of one sequence that a full grid works on at once (chain_anchor), >= 1
  uint32_t spin_limit;    // polls before a look-back gives up (kSpinLimit unless a test lowered it)
  uint32_t *hdr;          // workspace header
  uint64_t *words;        // tagged words
  const char *in_x;       // gated backward only: the scan's input x (in_a is the gate there)
#ifdef FSS_TRACE
  uint64_t *trace;        // debug build: 8 timestamps per tile, written by lane 0 of every wave 0
#endif
};

// Which column group the workgroup that takes slot `slot` of chunk `chunk` works on (tiles are
// numbered chunk-major: tile = chunk * n_groups + slot, and workgroup b takes tiles b,
// b + grid, ...).  Workgroup b runs on XCD b % 8, so with the groups dealt out in eighths the
// workgroups of one XCD share consecutive groups: whole rows of a few batch items instead of
// one 256-byte stripe of every row (`per` groups each; 0: the number of groups does not
// divide by 8, slot s takes group s).  Within its eighth the deal moves on by one group from one
// round of the grid to the next (`in_flight` chunks make a round), so that a workgroup meets a
// different column stripe with every tile: the memory system serves some stripes more slowly
// than others (measured on MI355X: byte offsets 256-511 of every KiB by 12 %), and the kernel ends
// with its slowest workgroup.  A column's chunks stay on one XCD, and so do the words that
// chain them.  The turn depends on the chunk alone, so every chunk's slots map onto its groups
// one to one whatever the grid.
struct TileOrder {
  uint32_t n_groups, per, in_flight;
};
__host__ __device__ inline uint32_t wave_uniform(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_readfirstlane(x);  // (divisions run on the vector unit: pin the result back)
#else
  return x;
#endif
}
__host__ __device__ inline TileOrder tile_order(uint32_t n_groups, uint32_t grid) {
  TileOrder o;
  o.n_groups = n_groups;
  o.per = (n_groups & 7u) == 0 ? n_groups >> 3 : 0u;
  o.in_flight = wave_uniform((grid + n_groups - 1) / n_groups);
  if (o.in_flight < 1) o.in_flight = 1;
  return o;
}
__host__ __device__ inline uint32_t tile_group(const TileOrder &o, uint32_t slot, uint32_t chunk) {
  if (o.per <= 1) return slot;
  const uint32_t turn = wave_uniform((chunk / o.in_flight) % o.per);
  uint32_t k = (slot >> 3) + turn;
  if (k >= o.per) k -= o.per;
  return (slot & 7u) * o.per + k;
}

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

// Which streams are accessed non-temporally (bit 0: alpha in the forward, 1: beta,
// 2: the saved h in the backward, 3: the forward's output h, 4: the backward's two
// gradient outputs, 5: alpha in the backward, 6: dout).  Measured on MI355X at bs8
// seq4096 d1024 with 16-wave workgroups, forward and backward alternating on one set
// of tensors (the way the reference benchmarks): no hints 115 us per step; hints on the
// three output streams and on the backward's reads of h (their last use) 94 us; hints
// on the reads of alpha, beta or dout as well 96-105 us.  With nothing cached between
// launches (eight sets of tensors in rotation) the same settings read 114 / 113 /
// 106-108 us: hints on the input reads would be worth 5 % there and cost up to 15 % in
// the first setting.
#ifndef FSS_NT_MASK
#define FSS_NT_MASK 28
#endif
constexpr bool kNtAFwd = (FSS_NT_MASK & 1) != 0;
constexpr bool kNtBFwd = (FSS_NT_MASK & 2) != 0;
constexpr bool kNtABwd = (FSS_NT_MASK & 32) != 0;
constexpr bool kNtBBwd = (FSS_NT_MASK & 64) != 0;
constexpr bool kNtH = (FSS_NT_MASK & 4) != 0;
constexpr bool kNtOutFwd = (FSS_NT_MASK & 8) != 0;
constexpr bool kNtOutBwd = (FSS_NT_MASK & 16) != 0;

// The forward's output is the one stream with a reader waiting: the next kernel of any
// pipeline, or the backward in a benchmark loop.  A small h is therefore stored without
// the hint and found in the 256 MiB memory-side cache by its reader (forward and backward
// alternating, bf16: bs16 seq2048 d512 52.4 -> 49.0 us per step, bs8 seq3000 d1024
// 74.0 -> 69.8 us).  "Small" means that h and the three inputs of such a step fill at
// most three quarters of that cache; at bs8 seq4096 d1024 (4 x 64 MiB, all of it) the
// same change read -4 us or +4 us depending on where the tensors happened to lie, and
// a larger h only pushes the inputs out (bs8 seq8192: the forward on its own 69 -> 89 us).
constexpr int64_t kKeepOutBytes = static_cast<int64_t>(48) << 20;

// dout is read once per step.  While the three inputs of a step (alpha, h or beta, dout)
// fit the memory-side cache together, a benchmark loop over one set of tensors finds it
// there again and a hint on its reads costs 4 % (bs8 seq4096 d1024 bf16, 64 MiB per
// tensor: 93.6 -> 97.3 us per step); beyond that the hint keeps dout from evicting alpha,
// which the backward reads a second time (128 MiB per tensor: bs8 seq8192 d1024
// 201.7 -> 192.6 us, fp32 at seq4096 194.4 -> 182.3 us).  With nothing cached between
// launches the hint is worth 5 % at any size.  The forward treats beta, which nothing
// reads again, the same way from the same size on (its 32-steps-per-lane kernels, the ones
// such tensors run): with nothing cached between launches the hint takes 2-4 % off a step
// at any size (bs8 seq4096 d1024 103.2 -> 100.9 us, seq8192 194.5 -> 187.5 us); in a loop
// over one set of tensors it costs 2 % at 64 MiB per tensor, where part of beta is still
// cached from the step before, and nothing measurable at 128 MiB.
constexpr int64_t kStreamDoutBytes = static_cast<int64_t>(80) << 20;

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
  int lane, wave, n_waves, look;   // wave, n_waves: along time, within this wave's column tile
  int wcol;              // which of the workgroup's column tiles this wave belongs to
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
  float2 *lds_pred;      // [look wave][v][lane] = what that wave's earlier chunks do to a state
  int span;              // chunks one look-back wave of this tile covers, one after the other (chunk_span)
  int anchor;            // the earlier chunk whose outgoing state this chunk's chain starts from (chain_anchor)
  uint32_t *s_ready;     // [wave] of this column tile: the number of the last tile whose map the wave has left in LDS
  uint32_t tile_no;      // number of this tile among the workgroup's tiles, from 1
#ifdef FSS_TRACE
  int trace_wave;
#endif
};

// ---- the order in which a chunk's incoming state is composed -----------------------------
//
// The state entering chunk k is  map[k-1] o map[k-2] o ... o map[a+1] (state[a])  for one earlier
// chunk a = chain_anchor(k), the "anchor" of k.  Which chunk that is, and how the maps between are
// grouped when they are composed, is fixed by k and by the plan (period, look-back waves, span)
// - never by which of the earlier chunks happen to have finished when k looks back.  The
// composition of affine maps is associative only up to fp32 rounding, so this is what makes
// the result of a chained scan a function of its inputs and its launch configuration alone:
// the same bits from run to run, on any stream, whatever else the device is doing.
//
// `period` is the number of chunks of one sequence that a full grid works on at once (tiles are
// numbered chunk-major, so the chunks of a sequence in flight together are consecutive).  Chunk
// k of round R = k / period takes the maps of its own round's earlier chunks - published as soon
// as their rows are loaded - and the outgoing state of the last chunk of round R-1, which a
// grid of the planned size finished a round ago (in round 0: of chunk 0, which needs no
// look-back).  The period is planned from the nominal device, not from the grid actually
// launched: a smaller grid or device meets the same anchors (and merely finds the maps
// already there), so the results do not depend on it either.
//
// Where a round holds more chunks than one round of the look-back reaches (`stride` = look-back
// waves x kMaxSpan chunks; a single long sequence whose chunks are all in flight at once), every
// stride-th chunk is an anchor as well: a chunk then never composes more than `stride` maps, at
// the price of a chain of states stride chunks apart (each available one look-back after the
// one before).  bs 1 seq 65521 d 256 bf16: backward 34.0 -> 31.3 us, forward+backward 60.6 -> 57.7 us.
__host__ __device__ inline int chain_anchor(int chunk, int period, int stride) {
  const int round_first = chunk - chunk % period;
  const int by_round = round_first > 0 ? round_first - 1 : 0;
  const int by_stride = (chunk - 1) / stride * stride;
  return by_round > by_stride ? by_round : by_stride;
}

// Chunks one look-back wave covers, one after the other, when `items` chunks (the anchor
// included; never more than look * kMaxSpan) are dealt out to `look` waves: as few as the waves allow.
__host__ __device__ inline int chunk_span(int items, int look) {
  const int span = (items + look - 1) / look;
  return span < 1 ? 1 : (span > kMaxSpan ? kMaxSpan : span);
}

// One look at chunk `j` of this column tile: at its outgoing state (`want_state`: j is the
// anchor) or at its map.  Split in two so that other work can be placed between the loads and
// the use of what they return.
template <int VEC>
struct ChunkWords {
  uint64_t a[VEC], b[VEC];
};

template <int VEC>
__device__ __forceinline__ void poll_issue(const ScanArgs &p, const TileCtx &c, int j, bool want_state,
                                           ChunkWords<VEC> &w) {
  const uint64_t *theirs = p.words + (static_cast<size_t>(j) * p.n_ctiles + c.ctile) * 3 * (64 * VEC) + c.lane;
  // (a state is asked for as both halves of a "map": the same straight-line code either way)
  const uint64_t *word_a = theirs + (want_state ? 2 * VEC * 64 : 0);
  const uint64_t *word_b = theirs + (want_state ? 2 * VEC * 64 : VEC * 64);
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    w.a[v] = ld_word(word_a + v * 64);
    w.b[v] = ld_word(word_b + v * 64);
  }
}

// True once every lane of the wave has what it asked for (the answer is taken for the whole
// wave); then (qA, qB) is the map, a state s being the map x -> 0*x + s.
template <int VEC>
__device__ __forceinline__ bool poll_eval(const TileCtx &c, bool want_state, const ChunkWords<VEC> &w, float *qA,
                                          float *qB) {
  bool have = true;
#pragma unroll
  for (int v = 0; v < VEC; ++v) have = have && word_tag(w.a[v]) == c.tag && word_tag(w.b[v]) == c.tag;
  if (__builtin_amdgcn_ballot_w64(have) != ~0ull) return false;
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    qA[v] = want_state ? 0.0f : word_val(w.a[v]);
    qB[v] = word_val(w.b[v]);
  }
  return true;
}

// Waits (bounded) for chunk j's state or map.  A wave that gives up reports it and carries on
// with a NaN state, so that the grid still drains and everything downstream is visibly poisoned.
template <int VEC>
__device__ __forceinline__ void await_chunk(const ScanArgs &p, const TileCtx &c, int j, bool want_state, float *qA,
                                            float *qB) {
  uint32_t polls = 0;
  for (;;) {
    if (polls >= p.spin_limit) {
      if (c.lane == 0) report_timeout(p.hdr);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        qA[v] = 0.0f;
        qB[v] = local_const(__builtin_nanf(""));
      }
      return;
    }
    ChunkWords<VEC> w;
    poll_issue<VEC>(p, c, j, want_state, w);
    if (poll_eval<VEC>(c, want_state, w, qA, qB)) return;
    ++polls;
    __builtin_amdgcn_s_sleep(2);
  }
}

// ---- hand-over of the waves' maps inside a workgroup ------------------------------------------
//
// A wave that has left its map in LDS says so in its word of `ready` (release; the number of the
// tile, which only grows, so nothing is ever reset).  Wave 0 composes the maps in wave order as
// they arrive, instead of behind a barrier that waits for the slowest wave before the first
// map is touched: a wave's rows arrive microseconds apart, and when the last map lands the
// others are already composed, so the chunk's map goes out a microsecond earlier - to every later
// chunk that is waiting for it.
__device__ __forceinline__ void announce_map(uint32_t *ready, int wave, uint32_t seq) {
  __hip_atomic_store(ready + wave, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void await_map(const uint32_t *ready, int wave, uint32_t seq) {
  // (wave-uniform address: one LDS word, broadcast)
  while (__hip_atomic_load(ready + wave, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < seq)
    __builtin_amdgcn_s_sleep(1);
}
// every wave of the column tile has left its map (lane l looks at wave l's word)
__device__ __forceinline__ void await_all_maps(const uint32_t *ready, int lane, int n_waves, uint32_t seq) {
  for (;;) {
    const uint32_t r = lane < n_waves
                           ? __hip_atomic_load(ready + lane, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)
                           : seq;
    if (__builtin_amdgcn_ballot_w64(r < seq) == 0ull) return;
    __builtin_amdgcn_s_sleep(1);
  }
}

// (A, B) <- map[count-1] o ... o map[0], composed by one wave for the whole workgroup as the maps
// arrive: slot w receives what the waves before w do to the chunk's incoming state (the
// composition of maps 0 .. w-1, in place of map w, which nobody else reads), and (A, B) the
// chunk's map.  Every other wave then finds its prefix with one LDS read behind the next barrier.
// The order of the composition is the waves' order, whatever the order of their arrival.
template <int VEC>
__device__ __forceinline__ void fold_arriving_maps(float2 *lds_map, const uint32_t *ready, uint32_t seq, int lane,
                                                   int count, float *A, float *B) {
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    A[v] = 1.0f;
    B[v] = 0.0f;
  }
  for (int w = 0; w < count; ++w) {
    if (w > 0) await_map(ready, w, seq);  // (slot 0 is this wave's own)
    float2 m[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) m[v] = lds_map[(w * VEC + v) * 64 + lane];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      lds_map[(w * VEC + v) * 64 + lane] = make_float2(A[v], B[v]);
      B[v] = fma0(m[v].x, B[v], m[v].y);
      A[v] *= m[v].x;
    }
  }
}

// Phase 2.  In: this wave's slice as the map x -> mA*x + mB.  Out: the state
// entering the slice.  Every wave of the workgroup must call it (barriers).
//
// Every wave leaves its map in LDS and says so (announce_map); wave 0 composes the maps into the
// chunk's map as they arrive and publishes it, leaving in every wave's slot the composition of
// the waves before it.  Meanwhile the look-back: the chunks from chunk-1 down to the anchor
// (chain_anchor) are dealt out to `look` waves, `span` consecutive chunks each, nearest first;
// each such wave waits for its chunks' maps (the anchor's outgoing state) and composes them, so a
// look-back over look*span chunks costs `span` memory round trips instead of one per chunk.
// After the one barrier of the phase every wave folds what the look-back waves left in LDS into
// the chunk's incoming state itself (a few multiply-adds: cheaper than another barrier and a
// broadcast), wave 0 also publishes the chunk's outgoing state, and every wave applies the
// composition of the waves before it (one LDS read).  Who looks at which chunk, and the order of
// every composition, depend on the chunk's index and the plan alone.
//
// `mid` (only with HAS_MID) is called once by every wave, by the look-back waves right after their
// first fetch has been issued: loads it issues travel while the chain is resolved and
// return after the fetch (loads return in issue order).
template <int VEC, bool HAS_MID, typename Mid>
__device__ __forceinline__ void chain_chunks(const ScanArgs &p, const TileCtx &c, const float *mA,
                                             const float *mB, const float *seq_in, float *state, Mid &&mid) {
  constexpr int kLaneSlots = 64 * VEC;
  const int lane = c.lane, wave = c.wave;
#pragma unroll
  for (int v = 0; v < VEC; ++v) c.lds_map[(wave * VEC + v) * 64 + lane] = make_float2(mA[v], mB[v]);
  announce_map(c.s_ready, wave, c.tile_no);
  FSS_STAMP(c, p, 2);

  const bool look_back = c.chained && c.chunk > 0;
  uint64_t *mine = nullptr;
  float cA[VEC], cB[VEC];
  if (wave == 0) {
    // the chunk's own map, needed by later chunks: out as early as possible - and on the way
    // every wave's prefix, left where its map was (the waves read it behind the next barrier)
    fold_arriving_maps<VEC>(c.lds_map, c.s_ready, c.tile_no, lane, c.n_waves, cA, cB);
    if (c.chained && !c.last) {
      mine = p.words + (static_cast<size_t>(c.chunk) * p.n_ctiles + c.ctile) * 3 * kLaneSlots + lane;
      if (look_back) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          st_word(mine + (0 * VEC + v) * 64, c.tag, cA[v]);
          st_word(mine + (1 * VEC + v) * 64, c.tag, cB[v]);
        }
      } else {
        // first chunk of a chained sequence: nobody asks for its map, only for its outgoing state
#pragma unroll
        for (int v = 0; v < VEC; ++v)
          st_word(mine + (2 * VEC + v) * 64, c.tag, seq_in ? fma0(cA[v], seq_in[v], cB[v]) : cB[v]);
      }
    }
  }
  FSS_STAMP(c, p, 3);

  // (pA, pB): what the waves before this one do to the chunk's incoming state
  float pA[VEC], pB[VEC];
  if (!look_back) {
    // first chunk of the sequence (or the only one): the incoming state is the
    // sequence's own (0 in the plain scan)
    if constexpr (HAS_MID) {
      if (wave != 0) await_all_maps(c.s_ready, lane, c.n_waves, c.tile_no);  // (as below: not before the others' rows are in)
      mid();
    }
    __syncthreads();  // wave 0 has left every wave's prefix
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float2 e = c.lds_map[(wave * VEC + v) * 64 + lane];
      pA[v] = e.x;
      pB[v] = e.y;
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) state[v] = seq_in ? fma0(pA[v], seq_in[v], pB[v]) : pB[v];
    FSS_STAMP(c, p, 5);
    return;
  }

  float hin[VEC], accA[VEC], accB[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    accA[v] = local_const(1.0f);
    accB[v] = local_const(0.0f);
    hin[v] = local_const(0.0f);
  }
  const int anchor = c.anchor;
  // Which wave asks which chunk: look index 0 asks the nearest chunk.  Where the waves issue loads
  // of their own inside this phase (`mid`), the look-back is the work of the LAST waves (look
  // index 0 = the last wave): wave 0 is busy composing and publishing the chunk's own map and
  // would ask behind that and behind its own loads (bs 8 seq 4096 d 1024 bf16 backward 54.8 ->
  // 54.0 us, 60.3 -> 58.4 us over tensor sets in rotation; the forward, which issues nothing
  // here, measured 0.3-0.6 us slower that way and keeps the first waves).
  const int li = HAS_MID ? c.n_waves - 1 - wave : wave;
  // The chunks chunk-1 .. anchor, `span` consecutive ones per look-back wave: one round always
  // reaches the anchor (chain_anchor keeps it within look * kMaxSpan chunks, chunk_span deals
  // them out).  This wave's are j, j-1, ..., down to the anchor at most.
  const int j = c.chunk - 1 - li * c.span;
  const bool looks = li < c.look && j >= anchor;
  // The first look goes out with `mid` in a straight line between the issue of its loads and
  // their use: only so does the compiler wait for exactly those loads and not for the ones
  // `mid` has issued behind them.
  bool have0 = false;
  float qA[VEC], qB[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) qA[v] = qB[v] = local_const(0.0f);
  // The look-back starts once every wave of the column tile has its rows (the chunks it asks run
  // in step with this one: asking earlier only polls for longer).  Waves with loads of their own
  // to issue here wait for that moment too (issued while the other waves' rows are still on
  // their way, those loads only delay them: bs 8 seq 4096 d 1024 backward 53.5 -> 56.4 us); the
  // rest go straight on to the barrier.
  if (looks || (HAS_MID && wave != 0)) await_all_maps(c.s_ready, lane, c.n_waves, c.tile_no);
  if constexpr (HAS_MID) {
    if (looks && p.spin_limit != 0) {
      ChunkWords<VEC> w;
      poll_issue<VEC>(p, c, j, j == anchor, w);
      mid();
      have0 = poll_eval<VEC>(c, j == anchor, w, qA, qB);
    } else {
      mid();
    }
  }
  if (looks) {
    if (!have0) await_chunk<VEC>(p, c, j, j == anchor, qA, qB);
    // long chains: the wave also takes the chunks before that one (by now they have nearly
    // always published), so that the look-back reaches `span` times as far
    for (int k = 1; k < c.span && j - k >= anchor; ++k) {
      float rA[VEC], rB[VEC];
      await_chunk<VEC>(p, c, j - k, j - k == anchor, rA, rB);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        qB[v] = fma0(qA[v], rB[v], qB[v]);
        qA[v] *= rA[v];
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) c.lds_pred[(li * VEC + v) * 64 + lane] = make_float2(qA[v], qB[v]);
  }
  __syncthreads();
  // every wave folds what the look-back waves found (the same few LDS reads in each wave
  // cost less than a second barrier and a broadcast by wave 0)
  for (int w = 0; w < c.look && c.chunk - 1 - w * c.span >= anchor; ++w) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float2 m = c.lds_pred[(w * VEC + v) * 64 + lane];
      accB[v] = fma0(accA[v], m.y, accB[v]);
      accA[v] *= m.x;
    }
  }
  // (the last group folded ended with the anchor's state, the map x -> 0*x + s: accB is the state)
#pragma unroll
  for (int v = 0; v < VEC; ++v) hin[v] = accB[v];
  if (wave == 0 && !c.last) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) st_word(mine + (2 * VEC + v) * 64, c.tag, fma0(cA[v], hin[v], cB[v]));
  }
  FSS_STAMP(c, p, 4);
  // (the prefix wave 0 left in this wave's slot, behind the loop's barrier)
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    const float2 e = c.lds_map[(wave * VEC + v) * 64 + lane];
    pA[v] = e.x;
    pB[v] = e.y;
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) state[v] = fma0(pA[v], hin[v], pB[v]);
  FSS_STAMP(c, p, 5);
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
        // the header holds the next launch's tag minus 1, so that zero-filled memory is a
        // ready workspace; 0 is the tag of never-written words: skip it when the counter wraps
        st_u32(p.hdr + HDR_EPOCH, (c.tag + 1u == 0u ? 1u : c.tag + 1u) - 1u);
      }
    }
  }
}

}  // namespace fss
