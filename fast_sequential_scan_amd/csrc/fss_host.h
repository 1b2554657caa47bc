// Host-side pieces shared by the translation units of the library: launch planning,
// device checks, the ordering of scans across streams, residency of a kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <initializer_list>
#include <mutex>

#include "../../include/fss_scan.h"
#include "fss_device.h"

namespace fss {

extern thread_local int tls_hip_error;  // hipError_t of this thread's last failed HIP call
extern uint32_t g_spin_limit;           // polls before a look-back gives up (a test may lower it)
#ifdef FSS_TRACE
extern uint64_t *g_trace;
#endif

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Register budget: packed dwords a lane may hold per input tensor.
inline int max_vec_steps(int dtype) { return dtype != FSS_F32 ? 64 : 32; }  // vec*steps

// Most waves a workgroup of the row-major kernels may have, by what a lane holds: the kernels
// are compiled for that many (launch bounds), so that their registers fit without spilling.
// 16 waves leave a lane 128 registers: enough for 64 dwords of rows with up to two channels
// per lane.  Wider lanes (whose chaining state grows with the channels) and the plain
// backward with 32 steps of two channels (three tensors) get 256 or 512 registers instead.
constexpr int max_waves(int esize, int vec, int steps, bool bwd, bool gated) {
  const int dwords = vec * esize >= 4 ? vec * esize / 4 : 1;  // per lane and row
  if (vec >= 8) return 4;
  if (vec >= 4) return 8;
  if (!gated && vec >= 2 && dwords * steps * (bwd ? 3 : 2) > 64) return 8;
  return 16;
}

// LDS: one (A,B) slot per lane and vector element for every wave, twice (tiles
// alternate between two sets), and the same for every wave that looks back (per
// column tile of the workgroup).  `waves` counts all waves of the workgroup, of which
// waves/cols lie along time.
constexpr size_t kLdsBudget = 60 * 1024;
inline int look_waves(int waves, int vec, int cols = 1) {
  const int along_time = waves / cols;
  int look = along_time < kMaxLookWaves ? along_time : kMaxLookWaves;
  while (look > 1 && static_cast<size_t>(2 * waves + look * cols) * vec * 512 > kLdsBudget) --look;
  return look;
}
inline size_t lds_bytes(int waves, int vec, int cols = 1) {
  return static_cast<size_t>(2 * waves + look_waves(waves, vec, cols) * cols) * vec * 512;
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
  if (c.waves < 1 || c.waves > max_waves(dtype != FSS_F32 ? 2 : 4, c.vec, c.steps, (dir & 1) == FSS_BWD, gated)) return false;
  if (c.cols != 1 && c.cols != 2) return false;
  if (c.waves % c.cols != 0) return false;
  if (lds_bytes(c.waves, c.vec, c.cols) > kLdsBudget) return false;
  return true;
}

// CUs of an unpartitioned MI355X: what "one tile per CU" means when a launch is planned
// (planning must work without a device; the grid itself is sized from the runtime's count).
constexpr int64_t kCus = 256;

// Chunks of one sequence that a full grid works on at once: the spacing of the chain's anchors
// (chain_anchor in fss_device.h).  Planned from the nominal device - kCus compute units holding
// 16 waves of a scan each - and from nothing that can differ between two launches of one
// configuration (not the grid actually launched, not the device's own CU count), so that the
// order in which carries are composed, and with it every bit of the result, is fixed by the
// shape and the configuration.
inline int chain_period(int64_t n_groups, int waves) {
  const int64_t per_cu = waves >= 16 ? 1 : 16 / (waves > 0 ? waves : 1);
  const int64_t nominal_grid = kCus * per_cu;
  const int64_t period = ceil_div(nominal_grid, n_groups > 0 ? n_groups : 1);
  return static_cast<int>(period < 1 ? 1 : (period > (1 << 20) ? (1 << 20) : period));
}

// One candidate launch configuration: taken when it yields at least `need` tiles.
struct Rung {
  int vec, steps, waves;
  int64_t need;
};

// Column tiles a workgroup covers side by side (fss_config.cols) when the caller leaves the
// choice open; vec, steps and waves of `c` are already fixed.  Two column tiles make every row a
// workgroup touches 512 contiguous bytes instead of 256 and its chunks half as long.  Measured in
// the forward with 4 bytes per lane, 32 steps and 16 waves (bf16, 49 shapes, bs 2..16, seq
// 2048..16384, d 512..4096, tensor sets in rotation so that nothing is found in a cache): where
// the launch has more than one and at most two tiles per CU, 5-13 % faster on 8 shapes of 9;
// with four tiles per CU +-0, with eight 1 % slower; in the backward, whose chunks would shrink
// to 128 steps, slower throughout.  At bs 8 seq 4096 d 1024: forward 42.8 -> 40.9 us and the
// forward+backward step 105.4 -> 103.3 us over tensor sets in rotation, a forward behind flushed
// caches 48.2 -> 45.6 us; when the tensors are found in the memory-side cache again (forward and
// backward alternating on one set of tensors) forward 31.0 -> 32.2 us, step 88.6 -> 90.5 us.  The
// library cannot know which of the two it is in and takes what serves the caller whose tensors
// come from memory.  The choice depends on the shape alone - never on a policy or on earlier
// calls - because a different tiling rounds the carries differently.
inline int choose_cols(const fss_config &c, int64_t bs, int64_t seq, int64_t d, int dtype, int dir, bool gated) {
  if (gated || dir != FSS_FWD) return 1;
  const int esize = dtype != FSS_F32 ? 2 : 4;
  if (c.vec * esize != 4 || c.steps != 32 || c.waves != 16) return 1;
  const int64_t tiles_per_row = ceil_div(d, 64 * static_cast<int64_t>(c.vec));
  if (tiles_per_row % 2 != 0) return 1;
  const int64_t tiles = bs * tiles_per_row * ceil_div(seq, static_cast<int64_t>(c.steps) * c.waves);
  return tiles > kCus && tiles <= 2 * kCus ? 2 : 1;
}

// Fills the zero fields of `c`.  `align` is the common alignment in bytes of all
// tensors of the call.
//
// From sweeps over bs 1..64, seq 256..16384, d 256..4096 per storage type and kernel
// family (every shape against 8-11 configurations), which all show the same thing: the
// largest tile that still leaves one tile per CU wins.  Large tiles mean few chunks per
// sequence (a short chain) and long uninterrupted streams per wave; 16 waves of 32
// (backward 16) timesteps with 4 bytes per lane is the largest that fits the register
// file.  So the choice walks down a ladder of tile sizes, each half the one before, and
// takes the first with at least one tile per CU; which of time, channels per lane and waves
// is halved at each rung is what the sweeps decided.  Below the last rung the problem
// is latency-bound and the smallest tile is as good as any.
inline void complete_config(fss_config &c, int64_t bs, int64_t seq, int64_t d, int dtype, int dir,
                     size_t align, bool gated = false) {
  const bool narrow = dtype != FSS_F32;  // 16-bit storage
  const int esize = narrow ? 2 : 4;
  // two channels per lane: even d, 2-element alignment, and never pad a row to twice its width
  const bool can2 = d % 2 == 0 && align % (2 * static_cast<size_t>(esize)) == 0 &&
                    ceil_div(d, 128) * 128 < 2 * ceil_div(d, 64) * 64;
  // fp32, very large tensors with wide rows (56 shapes of 2^24..2^27 elements, d 512..4096, seq
  // 512..8192, six configurations each).  Forward from 2^26 elements: 16 steps per lane are 2-6 %
  // faster than 32 up to seq 4096, and 8 bytes per lane another 3-8 % at seq 512 (4-9 % slower
  // from seq 2048).  Backward: 8 bytes per lane with 8 steps are 4-11 % faster from 2^27 elements
  // and 3-10 % slower at 2^26.
  const int64_t elems = bs * seq * d;
  const bool big32 = !narrow && !gated && d >= 512 && elems >= (static_cast<int64_t>(1) << 26);
  const bool wide32_fwd = big32 && can2 && seq <= 512;
  const bool wide32_bwd = big32 && can2 && elems >= (static_cast<int64_t>(1) << 27);
  Rung ladder[8];
  int n = 0;
  auto rung = [&](int v, int s, int w, int64_t need = kCus) { ladder[n++] = Rung{v, s, w, need}; };
  const bool fwd = dir == FSS_FWD;
  if (!gated && fwd) {
    if (narrow) rung(2, 32, 16);
    if (wide32_fwd) rung(2, 16, 16);
    else if (big32 && seq <= 4096) rung(1, 16, 16);
    rung(1, 32, 16);
    if (seq <= 2048) rung(1, 16, 16);
    rung(1, 32, 8, 0);
  } else if (!gated) {
    // 32-step slices would cost the backward a dozen spilled registers per lane
    if (narrow) {
      rung(2, 16, 16);
      if (seq >= 16384) rung(1, 16, 16); else rung(2, 16, 8);
      if (seq > 256) rung(1, 16, 8); else rung(2, 8, 8);
    } else {
      if (wide32_bwd) rung(2, 8, 16);
      rung(1, 16, 16);
      rung(1, 16, 8);
    }
    if (seq >= 2048) rung(1, 16, 8, 0); else rung(1, 8, 8, 0);
  } else if (fwd) {
    // The gated kernels spend as much time on arithmetic as on memory and like more, smaller
    // waves; a sequence that 8 waves cover wants two workgroups per CU before it takes them.
    if (narrow) {
      // (from 8192 steps two 8-wave workgroups per CU are 3-5 % faster than one of 16 waves: 8 shapes of 9)
      if (seq >= 8192) rung(2, 32, 8, 2 * kCus);
      if (seq > 256) rung(2, 32, 16); else rung(2, 32, 8, 2 * kCus);
      if (seq >= 4096) rung(1, 32, 16); else rung(2, 16, 16);
      if (seq >= 16384) rung(1, 32, 8);
      rung(1, 16, 16);
      if (seq >= 1024) rung(1, 16, 8, 0); else rung(1, 16, 16, 0);
    } else {
      if (seq > 256) rung(1, 32, 16); else rung(1, 32, 8, 2 * kCus);
      rung(1, 16, 16, 0);
    }
  } else {
    // gated backward: four tensors per timestep, at most 16 steps per lane (fp32: 8 are faster)
    if (narrow) {
      // (many short sequences: two 8-wave workgroups per CU are 3-16 % faster: 6 shapes of 7 at 2^25 elements)
      if (seq <= 1024) rung(2, 16, 8, 8 * kCus);
      if (seq > 256) rung(2, 16, 16); else rung(2, 16, 8, 4 * kCus);
      rung(2, 8, 16);
      rung(2, 8, 8, seq <= 256 ? 1 : kCus);
      rung(1, 8, 8, 0);
    } else {
      if (seq > 256) rung(1, 8, 16);
      rung(1, 8, 8, 0);
    }
  }
  fss_config pick = {0, 0, 0, 0, 0};
  for (int i = 0; i < n; ++i) {
    // what the caller fixed stays fixed
    int v = c.vec ? c.vec : ladder[i].vec;
    int s = c.steps ? c.steps : ladder[i].steps;
    int w = c.waves ? c.waves : ladder[i].waves;
    if (!c.vec && v == 2 && !can2) continue;
    // never more waves or steps than the sequence needs
    while (!c.waves && w > 1 && static_cast<int64_t>(s) * (w / 2) >= seq) w /= 2;
    while (!c.steps && s > 8 && s / 2 >= seq) s /= 2;
    while (!c.waves && w > max_waves(esize, v, s, !fwd, gated)) w /= 2;  // (only when the caller fixed a wide lane)
    while (!c.waves && w > 1 && lds_bytes(w, v) > kLdsBudget) --w;
    pick = fss_config{v, s, w, 0, 0};
    if (bs * ceil_div(d, 64 * static_cast<int64_t>(v)) * ceil_div(seq, static_cast<int64_t>(s) * w) >= ladder[i].need) break;
  }
  // Forward and gated backward, 16-wave workgroups (one per CU) whose last round would fill less than 90 % of the
  // CUs: the same tile shape as 8-wave workgroups, two per CU, spreads that round over all CUs
  // (7-18 % faster on 59 of 182 shapes with lengths and widths that are no powers of two; the
  // plain backward measured no gain from it, the gated backward 5-16 % on 6 shapes of 6).
  if ((fwd || gated) && !c.waves && pick.waves == 16) {
    const int64_t tiles = bs * ceil_div(d, 64 * static_cast<int64_t>(pick.vec)) * ceil_div(seq, static_cast<int64_t>(pick.steps) * 16);
    const int64_t rounds = ceil_div(tiles, kCus);
    if (rounds >= 2 && tiles * 10 < rounds * kCus * 9) pick.waves = 8;
  }
  c.vec = pick.vec;
  c.steps = pick.steps;
  c.waves = pick.waves;
  if (!c.cols) c.cols = choose_cols(c, bs, seq, d, dtype, dir, gated);
}

struct Plan {
  fss_config cfg;
  int alt_policy = 0;  // plain scan: which cache hints the kernel carries (see kKeepOutBytes, kStreamDoutBytes)
  int64_t tiles_per_row, n_ctiles, n_chunks;
  int64_t n_groups;  // column groups per chunk: n_ctiles / cfg.cols
  int64_t n_tiles;   // what the workgroups walk: n_groups * n_chunks
  size_t ws_bytes;
};

inline int make_plan(Plan &pl, int64_t bs, int64_t seq, int64_t d, int dtype, int dir, size_t align,
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
  fss_config c = {0, 0, 0, 0, 0};
  if (user) c = *user;
  if (c.max_groups < 0 || c.cols < 0) return FSS_ERR_BAD_CONFIG;
  const int64_t dd = d > 0 ? d : 1, ss = seq > 0 ? seq : 1, bb = bs > 0 ? bs : 1;
  complete_config(c, bb, ss, dd, dtype, dir, align, gated);
  if (!config_valid(c, dtype, gated, dir)) return FSS_ERR_BAD_CONFIG;
  if (dd % c.vec != 0) return FSS_ERR_BAD_CONFIG;
  if (align % (static_cast<size_t>(c.vec) * esize) != 0) return FSS_ERR_MISALIGNED;
  pl.cfg = c;
  pl.tiles_per_row = ceil_div(dd, 64 * c.vec);
  if (pl.tiles_per_row % c.cols != 0) return FSS_ERR_BAD_CONFIG;
  pl.n_ctiles = bb * pl.tiles_per_row;
  pl.n_chunks = ceil_div(ss, static_cast<int64_t>(c.waves / c.cols) * c.steps);
  pl.n_groups = pl.n_ctiles / c.cols;
  pl.n_tiles = pl.n_groups * pl.n_chunks;
  if (pl.n_ctiles > INT32_MAX || pl.n_chunks > INT32_MAX || pl.n_ctiles * pl.n_chunks > INT32_MAX) return FSS_ERR_BAD_SHAPE;
  pl.ws_bytes = kHeaderBytes;
  if (pl.n_chunks > 1)
    pl.ws_bytes += static_cast<size_t>(pl.n_ctiles * pl.n_chunks) * 3 * 64 * c.vec * sizeof(uint64_t);
  return FSS_OK;
}

inline size_t common_alignment(std::initializer_list<const void *> ptrs) {
  uintptr_t bits = 0;
  for (const void *p : ptrs) bits |= reinterpret_cast<uintptr_t>(p);
  bits |= 16;  // 16 bytes is all any path needs
  return static_cast<size_t>(bits & (~bits + 1));
}

inline int check_device() {
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
extern ScanOrder g_scan_order[64];

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

inline int cu_count_of_current_device() {
  static int cached[64];  // by device; 0 = not asked yet
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  const bool slot = dev >= 0 && dev < 64;
  if (slot && (n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED)) > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
  if (slot) __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
  return n;
}

// Workgroups of `kernel` that are certainly resident together on one compute unit (0 on
// error).  Deliberately not the runtime's occupancy query: the kernel's waits
// need a lower bound, and that query bounds by vector registers and LDS only.
// These kernels hold many scalar registers as well (a row pointer per load); a
// wave may be allocated 128 of the 800 a SIMD has, which caps a SIMD at 6 waves -
// the residency measured on MI355X for the scalar-heaviest variants.
template <typename Kernel>
int resident_workgroups_per_cu(Kernel kernel, int waves, size_t lds) {
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
  return per_cu;
}

// The same for the whole current device.  `cache` (one slot per waves-per-workgroup value
// of one kernel instantiation) keeps the per-CU answer, which is a property of the code
// object; the CU count is the current device's.
template <typename Kernel>
int resident_workgroups(Kernel kernel, int waves, size_t lds, int *cache) {
  int per_cu = __atomic_load_n(&cache[waves], __ATOMIC_RELAXED);
  if (per_cu == 0) {
    per_cu = resident_workgroups_per_cu(kernel, waves, lds);
    if (per_cu <= 0) return 0;
    __atomic_store_n(&cache[waves], per_cu, __ATOMIC_RELAXED);
  }
  return per_cu * cu_count_of_current_device();
}

// ---- channel-major planning -------------------------------------------------------------

// rows per wave: 4 bytes-per-lane budgets as in the row-major kernels (two tensors of
// 8 rows x 16 bytes forward, three of 4 rows backward)
constexpr int kCmRowsFwd = 8, kCmRowsBwd = 4;

struct CmPlan {
  int vec, waves;
  int64_t n_rowtiles, n_chunks, n_tiles;
  size_t ws_bytes;
};

inline int make_cm_plan(CmPlan &pl, int64_t rows, int64_t seq, int dtype, int dir, size_t align, const fss_config *user) {
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
    // forward, a chained sequence with few rows: half-size workgroups double the tiles in
    // flight (10-15 % at bs1 d256 seq16384)
    const int64_t chunks8 = ceil_div(ss, static_cast<int64_t>(8) * 64 * vec);
    if (dir == FSS_FWD && waves == 8 && chunks8 >= 2 && ceil_div(rr, kCmRowsFwd) * chunks8 < 1024) waves = 4;
    // a chained sequence that half-size workgroups cover with less padding (seq 5120: three
    // chunks of 2048 steps instead of two of 4096; 7-9 % faster)
    const int64_t reach4 = static_cast<int64_t>(4) * 64 * vec;
    if (waves == 8 && chunks8 >= 2 && ceil_div(ss, reach4) * reach4 < chunks8 * 2 * reach4) waves = 4;
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


// ---- what each translation unit provides --------------------------------------------------

// fss_scan_rm.hip, compiled once per storage type and direction: launches the row-major
// kernel (plain, with states, or gated) the plan asks for.
#define FSS_DECLARE_RM_LAUNCH(name)                                                                        \
  int name(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, bool gated, bool with_state, \
           hipStream_t stream)
FSS_DECLARE_RM_LAUNCH(launch_rm_bf16_fwd);
FSS_DECLARE_RM_LAUNCH(launch_rm_bf16_bwd);
FSS_DECLARE_RM_LAUNCH(launch_rm_f16_fwd);
FSS_DECLARE_RM_LAUNCH(launch_rm_f16_bwd);
FSS_DECLARE_RM_LAUNCH(launch_rm_f32_fwd);
FSS_DECLARE_RM_LAUNCH(launch_rm_f32_bwd);
#undef FSS_DECLARE_RM_LAUNCH

// fss_scan_cm.hip
int run_cm_scan(int dtype, int dir, const void *alpha, const void *in_b, const void *in_h, void *out0, void *out1,
                int64_t bs, int64_t d, int64_t seq, void *workspace, size_t workspace_bytes, void *stream,
                const fss_config *cfg);

}  // namespace fss
