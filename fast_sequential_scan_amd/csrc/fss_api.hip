// The C ABI of include/fss_scan.h: argument checking, planning, and the hand-off to the
// kernels' translation units (fss_scan_rm.hip per storage type, fss_scan_cm.hip).
#include "fss_device.h"
#include "fss_host.h"

namespace fss {

thread_local int tls_hip_error = 0;
#ifdef FSS_TRACE
uint64_t *g_trace = nullptr;
#endif
ScanOrder g_scan_order[64];

// Zero everywhere: tag 0 = "never written", and the first launch takes tag 1.
__global__ void workspace_init_kernel(uint32_t *p, size_t n_words) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_words; i += stride) p[i] = 0u;
}

__global__ void workspace_attach_kernel(uint32_t *hdr, uint64_t flag_address) {
  hdr[HDR_FLAG_LO] = static_cast<uint32_t>(flag_address);
  hdr[HDR_FLAG_HI] = static_cast<uint32_t>(flag_address >> 32);
}

__global__ void copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, size_t n_vec) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_vec; i += stride)
    dst[i] = src[i];
}

// Calibration: the plainest kernel that moves a scan's mix of streams - R buffers read, W written,
// each lane 16 bytes at a time, linearly, no dependence between elements.  What it reaches is
// what this machine's memory system gives a kernel with that read/write mix; the scan kernels
// are judged against it as well as against the nominal peak.  out0 = XOR of the reads,
// out1 = ~out0 (so that every load is used and the result can be checked).
struct StreamMixArgs {
  const u32x4 *rd[3];
  u32x4 *wr[2];
  size_t n_vec;
};
template <bool NT>
__device__ __forceinline__ u32x4 stream_load(const u32x4 *p) {
  return NT ? __builtin_nontemporal_load(p) : *p;
}
template <int R, int W, bool NTW, bool NTR>
__device__ __forceinline__ void stream_mix_finish(const StreamMixArgs &a, size_t i, u32x4 v) {
  if (R > 1) v ^= stream_load<NTR>(a.rd[1] + i);
  if (R > 2) v ^= stream_load<NTR>(a.rd[2] + i);
  if (W > 0) {
    if (NTW) __builtin_nontemporal_store(v, a.wr[0] + i); else a.wr[0][i] = v;
  }
  if (W > 1) {
    if (NTW) __builtin_nontemporal_store(~v, a.wr[1] + i); else a.wr[1][i] = ~v;
  }
  if (W == 0) {
    // read-only: the loads must not be optimised away; the store never happens in practice
    // (the caller passes a 16-byte sink for the one value that would trigger it)
    if (v.x == 0x9e3779b9u && v.y == 0x7f4a7c15u && v.z == 0xf39cc060u && v.w == 0x5cedc834u) a.wr[0][0] = v;
  }
}
// U vectors per lane and iteration, a grid stride apart: their first loads are issued together.
template <int R, int W, bool NTW, bool NTR, int U>
__global__ __launch_bounds__(1024) void stream_mix_kernel(const StreamMixArgs a) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; i + (U - 1) * stride < a.n_vec; i += U * stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = stream_load<NTR>(a.rd[0] + i + u * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) stream_mix_finish<R, W, NTW, NTR>(a, i + u * stride, v[u]);
  }
  for (; i < a.n_vec; i += stride) stream_mix_finish<R, W, NTW, NTR>(a, i, stream_load<NTR>(a.rd[0] + i));
}

struct StreamMixShape {
  int blocks, threads, per_lane;
  bool nt_writes, nt_reads;
};
template <int R, int W, bool NTW, bool NTR>
static void launch_stream_mix_u(const StreamMixArgs &a, const StreamMixShape &sh, hipStream_t stream) {
  const dim3 grid(sh.blocks), block(sh.threads);
  if (sh.per_lane == 2)
    hipLaunchKernelGGL((stream_mix_kernel<R, W, NTW, NTR, 2>), grid, block, 0, stream, a);
  else
    hipLaunchKernelGGL((stream_mix_kernel<R, W, NTW, NTR, 1>), grid, block, 0, stream, a);
}
template <int R, int W>
static void launch_stream_mix(const StreamMixArgs &a, const StreamMixShape &sh, hipStream_t stream) {
  if (sh.nt_writes) {
    if (sh.nt_reads) launch_stream_mix_u<R, W, true, true>(a, sh, stream);
    else launch_stream_mix_u<R, W, true, false>(a, sh, stream);
  } else {
    if (sh.nt_reads) launch_stream_mix_u<R, W, false, true>(a, sh, stream);
    else launch_stream_mix_u<R, W, false, false>(a, sh, stream);
  }
}

int g_cache_policy = FSS_CACHE_AUTO;  // fss_set_cache_policy
uint32_t g_spin_limit = kSpinLimit;    // fss_debug_set_spin_limit

// ---- the chaining scratch of the entry point that allocates nothing ----------------------
//
// One array per device (every GPU the library runs on holds its own copy, at its own
// address, until the process ends).  Zero-initialised memory is a ready workspace, so it
// needs no reset before its first use.  In host code the array's name is only a handle
// for hipGetSymbolAddress: what the kernels get is the address looked up once per device.
static __device__ __align__(256) unsigned char scratch[FSS_NOALLOC_SCRATCH_BYTES];

struct ScratchSlot {
  std::mutex lock;
  void *ptr = nullptr;
  uint64_t launches = 0;  // chained or not: an upper bound on how far the array's launch tag has advanced
  uint32_t *flag = nullptr;  // host-visible word attached through fss_workspace_attach_flag(NULL, ...)
};
static ScratchSlot g_scratch[64];

// The validity tags of the chaining words are a 32-bit launch counter kept in the array itself.
// A caller's workspace is re-initialised by its owner before the counter can wrap; nobody but
// the library can reach this array, so the library counts the launches through it and zeroes it
// again (a fill kernel on the call's stream: nothing is allocated) long before that.  Without
// this, words left behind by an earlier, larger shape could carry a live tag again after the wrap.
constexpr uint64_t kScratchReinitAfter = 1ull << 31;
static uint64_t g_scratch_reinit_after = kScratchReinitAfter;  // fss_debug_noalloc_reinit_after

// Address of the current device's copy of `scratch`; looked up at the first call on that
// device.  The same set-up creates the event that orders scans across streams, so that no
// later call through this entry point has anything left to create.
static int scratch_of_current_device(void **out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  if (dev < 0 || dev >= 64) return FSS_ERR_UNSUPPORTED_DEVICE;
  ScratchSlot &slot = g_scratch[dev];
  std::lock_guard<std::mutex> guard(slot.lock);
  if (!slot.ptr) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      tls_hip_error = static_cast<int>(e);
      (void)hipGetLastError();
      return FSS_ERR_LAUNCH;
    }
    ScanOrder &order = g_scan_order[dev];
    std::lock_guard<std::mutex> order_guard(order.lock);
    if (!order.event && hipEventCreateWithFlags(&order.event, hipEventDisableTiming) != hipSuccess) {
      order.event = nullptr;
      (void)hipGetLastError();
    }
    slot.ptr = ptr;
  }
  *out = slot.ptr;
  return FSS_OK;
}

static int launch_workspace_init(void *workspace, size_t bytes, hipStream_t stream) {
  const size_t n_words = bytes / 4;
  size_t blocks = (n_words + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(workspace_init_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                     static_cast<uint32_t *>(workspace), n_words);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

static int launch_workspace_attach(void *workspace, uint32_t *flag, hipStream_t stream) {
  hipLaunchKernelGGL(workspace_attach_kernel, dim3(1), dim3(1), 0, stream, static_cast<uint32_t *>(workspace),
                     static_cast<uint64_t>(reinterpret_cast<uintptr_t>(flag)));
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

// Counts one launch through the current device's scratch array and, when the count says that
// its launch tag could come near wrapping, zeroes the array on `stream` first (and attaches the
// host-visible word again).  The fill is ordered against scans on other streams like a scan.
static int count_scratch_launch(void *ptr, hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return FSS_ERR_LAUNCH;
  ScratchSlot &slot = g_scratch[dev];
  uint32_t *flag = nullptr;
  {
    std::lock_guard<std::mutex> guard(slot.lock);
    if (++slot.launches <= __atomic_load_n(&g_scratch_reinit_after, __ATOMIC_RELAXED)) return FSS_OK;
    slot.launches = 1;
    flag = slot.flag;
  }
  const ScanOrderGuard ordered(stream);
  int rc = launch_workspace_init(ptr, FSS_NOALLOC_SCRATCH_BYTES, stream);
  if (rc == FSS_OK && flag) rc = launch_workspace_attach(ptr, flag, stream);
  return rc;
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
  const bool streaming = __atomic_load_n(&g_cache_policy, __ATOMIC_RELAXED) == FSS_CACHE_STREAMING;
  const bool with_state = state_in || state_out || h_before;
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
  args.n_groups = static_cast<int32_t>(pl.n_groups);
  args.wg_cols = pl.cfg.cols;
  args.look_waves = look_waves(pl.cfg.waves, pl.cfg.vec, pl.cfg.cols);
  args.period = chain_period(pl.n_groups, pl.cfg.waves);
  args.spin_limit = __atomic_load_n(&g_spin_limit, __ATOMIC_RELAXED);
  const int64_t tensor_bytes = bs * seq * d * static_cast<int64_t>(esize);
  // (variant 2 exists for the kernels large shapes run - the forward with 32 steps per lane, the
  // backward with 16 steps and 4 bytes per lane; elsewhere the forward runs as 0, the backward as 1)
  const bool large = streaming || tensor_bytes > kStreamDoutBytes;
  if (gated)
    pl.alt_policy = 0;
  else if (dir == FSS_FWD)
    pl.alt_policy = large ? 2 : (tensor_bytes <= kKeepOutBytes ? 1 : 0);
  else
    pl.alt_policy = streaming ? 2 : (large ? 1 : 0);
  const StateArgs<true> state = {state_in, state_out, h_before};
  args.hdr = static_cast<uint32_t *>(workspace);
  args.words = workspace ? reinterpret_cast<uint64_t *>(static_cast<char *>(workspace) + kHeaderBytes) : nullptr;
#ifdef FSS_TRACE
  args.trace = g_trace;
#endif
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool st = with_state;
  const bool bwd = dir == FSS_BWD;
  const ScanOrderGuard ordered(s);
  if (dtype == FSS_BF16)
    return bwd ? launch_rm_bf16_bwd(args, state, pl, gated, st, s) : launch_rm_bf16_fwd(args, state, pl, gated, st, s);
  if (dtype == FSS_F16)
    return bwd ? launch_rm_f16_bwd(args, state, pl, gated, st, s) : launch_rm_f16_fwd(args, state, pl, gated, st, s);
  return bwd ? launch_rm_f32_bwd(args, state, pl, gated, st, s) : launch_rm_f32_fwd(args, state, pl, gated, st, s);
}

}  // namespace fss

// ---- C ABI -------------------------------------------------------------------------

extern "C" {

#ifdef FSS_TRACE
void fss_debug_set_trace(void *p) { fss::g_trace = static_cast<uint64_t *>(p); }
#endif

int fss_abi_version(void) { return FSS_ABI_VERSION; }

int fss_set_cache_policy(int policy) {
  if (policy != FSS_CACHE_AUTO && policy != FSS_CACHE_STREAMING) return -1;
  return __atomic_exchange_n(&fss::g_cache_policy, policy, __ATOMIC_RELAXED);
}

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
    case FSS_ERR_TOO_LARGE:
      return "the shape needs more chaining scratch than the entry point that allocates nothing holds "
             "(FSS_NOALLOC_SCRATCH_BYTES): use fss_scan_fwd_ex with a workspace";
    default: return "unknown status";
  }
}

int fss_last_hip_error(void) { return fss::tls_hip_error; }

size_t fss_workspace_bytes(int64_t bs, int64_t seq, int64_t d, int dtype, int dir, const fss_config *cfg) {
  // The tensors' alignment is unknown here and changes the plan (less aligned tensors take
  // fewer channels per lane, which can mean more, smaller tiles and more chaining words):
  // the answer covers every alignment.
  size_t best = fss::kHeaderBytes;
  for (size_t align = 2; align <= 16; align <<= 1) {
    fss::Plan pl;
    if (fss::make_plan(pl, bs, seq, d, dtype, dir, align, cfg) == FSS_OK && pl.ws_bytes > best) best = pl.ws_bytes;
  }
  return best;
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
  return fss::launch_workspace_init(workspace, bytes, static_cast<hipStream_t>(stream));
}

int fss_workspace_attach_flag(void *workspace, uint32_t *flag, void *stream) {
  if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0 || reinterpret_cast<uintptr_t>(flag) % 4 != 0)
    return FSS_ERR_MISALIGNED;
  if (!workspace) {
    // the static array of fss_scan_fwd_noalloc on the current device; remembered, so that the
    // word stays attached when the library zeroes that array again
    const int rc = fss::scratch_of_current_device(&workspace);
    if (rc != FSS_OK) return rc;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return FSS_ERR_LAUNCH;
    std::lock_guard<std::mutex> guard(fss::g_scratch[dev].lock);
    fss::g_scratch[dev].flag = flag;
  }
  return fss::launch_workspace_attach(workspace, flag, static_cast<hipStream_t>(stream));
}

uint64_t fss_debug_noalloc_reinit_after(uint64_t launches) {
  if (launches == 0) launches = fss::kScratchReinitAfter;
  return __atomic_exchange_n(&fss::g_scratch_reinit_after, launches, __ATOMIC_RELAXED);
}

int fss_debug_tile_groups(int32_t n_groups, int32_t grid, int32_t n_tiles, int32_t *groups) {
  if (!groups) return FSS_ERR_NULL_POINTER;
  if (n_groups <= 0 || grid <= 0 || n_tiles < 0) return FSS_ERR_BAD_SHAPE;
  const fss::TileOrder order = fss::tile_order(static_cast<uint32_t>(n_groups), static_cast<uint32_t>(grid));
  for (int32_t tile = 0; tile < n_tiles; ++tile)
    groups[tile] = static_cast<int32_t>(
        fss::tile_group(order, static_cast<uint32_t>(tile % n_groups), static_cast<uint32_t>(tile / n_groups)));
  return FSS_OK;
}

int fss_debug_chain_plan(int64_t bs, int64_t seq, int64_t d, int dtype, int dir, size_t align_bytes,
                         const fss_config *cfg, int32_t *out) {
  if (!out) return FSS_ERR_NULL_POINTER;
  fss::Plan pl;
  const int rc = fss::make_plan(pl, bs, seq, d, dtype, dir, align_bytes ? align_bytes : 16, cfg);
  if (rc != FSS_OK) return rc;
  const int look = fss::look_waves(pl.cfg.waves, pl.cfg.vec, pl.cfg.cols);
  const int period = fss::chain_period(pl.n_groups, pl.cfg.waves);
  out[0] = static_cast<int32_t>(pl.n_chunks);
  out[1] = pl.cfg.waves / pl.cfg.cols;
  out[2] = pl.cfg.steps;
  out[3] = period;
  out[4] = look;
  out[5] = fss::kMaxSpan;
  out[6] = pl.cfg.vec;
  out[7] = pl.cfg.cols;
  return FSS_OK;
}

int32_t fss_debug_chain_anchor(int32_t chunk, int32_t period, int32_t stride) {
  if (chunk < 0 || period < 1 || stride < 1) return -1;
  return fss::chain_anchor(chunk, period, stride);
}

uint32_t fss_debug_set_spin_limit(uint32_t polls) {
  return __atomic_exchange_n(&fss::g_spin_limit, polls, __ATOMIC_RELAXED);
}

int fss_workspace_status(void *workspace, void *stream) {
  if (!workspace) {  // the static array of fss_scan_fwd_noalloc on the current device
    const int rc = fss::scratch_of_current_device(&workspace);
    if (rc != FSS_OK) return rc;
  }
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

int fss_scan_fwd_noalloc(int dtype, const void *alpha, const void *beta, void *h, int64_t bs, int64_t seq,
                         int64_t d, void *stream) {
  if (bs < 0 || seq < 0 || d < 0) return FSS_ERR_BAD_SHAPE;
  if (bs == 0 || seq == 0 || d == 0) return FSS_OK;
  if (fss_workspace_bytes(bs, seq, d, dtype, FSS_FWD, nullptr) > FSS_NOALLOC_SCRATCH_BYTES) return FSS_ERR_TOO_LARGE;
  void *ptr = nullptr;
  int rc = fss::scratch_of_current_device(&ptr);
  if (rc != FSS_OK) return rc;
  rc = fss::count_scratch_launch(ptr, static_cast<hipStream_t>(stream));
  if (rc != FSS_OK) return rc;
  return fss::run_scan(dtype, FSS_FWD, alpha, beta, nullptr, h, nullptr, bs, seq, d, ptr, FSS_NOALLOC_SCRATCH_BYTES,
                       stream, nullptr);
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

int fss_gated_scan_fwd_state(int dtype, const void *gate, const void *x, void *h, const float *h_before,
                             float *h_last, int64_t bs, int64_t seq, int64_t d, void *workspace,
                             size_t workspace_bytes, void *stream, const fss_config *cfg) {
  return fss::run_scan(dtype, FSS_GATED_FWD, gate, x, nullptr, h, nullptr, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg, h_before, h_last, nullptr);
}

int fss_gated_scan_bwd_state(int dtype, const void *gate, const void *x, const void *h, const void *dout,
                             const float *h_before, const float *grad_h_last, void *grad_gate, void *grad_x,
                             float *grad_h_before, int64_t bs, int64_t seq, int64_t d, void *workspace,
                             size_t workspace_bytes, void *stream, const fss_config *cfg) {
  if (grad_h_before && !h_before) return FSS_ERR_NULL_POINTER;
  return fss::run_scan(dtype, FSS_GATED_BWD, gate, dout, h, grad_x, grad_gate, bs, seq, d, workspace,
                       workspace_bytes, stream, cfg, grad_h_last, grad_h_before, h_before, x);
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

int fss_stream_mix(const void *const *reads, int n_reads, void *const *writes, int n_writes, size_t bytes,
                   int nontemporal_writes, const int *launch_shape, void *stream) {
  if (!reads || n_reads < 1 || n_reads > 3 || n_writes < 0 || n_writes > 2) return FSS_ERR_BAD_CONFIG;
  fss::StreamMixShape sh = {2048, 256, 1, nontemporal_writes != 0, false};
  if (launch_shape) {
    sh.blocks = launch_shape[0];
    sh.threads = launch_shape[1];
    sh.per_lane = launch_shape[2];
    sh.nt_reads = launch_shape[3] != 0;
    if (sh.blocks < 1 || sh.blocks > (1 << 20) || sh.threads < 64 || sh.threads > 1024 || sh.threads % 64 != 0 ||
        (sh.per_lane != 1 && sh.per_lane != 2) || (launch_shape[3] != 0 && launch_shape[3] != 1))
      return FSS_ERR_BAD_CONFIG;
  }
  if (!writes) return FSS_ERR_NULL_POINTER;  // (read-only runs still name one 16-byte sink)
  if (bytes % 16 != 0) return FSS_ERR_MISALIGNED;
  fss::StreamMixArgs a = {{nullptr, nullptr, nullptr}, {nullptr, nullptr}, bytes / 16};
  for (int i = 0; i < n_reads; ++i) {
    if (!reads[i]) return FSS_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(reads[i]) % 16 != 0) return FSS_ERR_MISALIGNED;
    a.rd[i] = static_cast<const fss::u32x4 *>(reads[i]);
  }
  for (int i = 0; i < (n_writes > 0 ? n_writes : 1); ++i) {
    if (!writes[i]) return FSS_ERR_NULL_POINTER;
    if (reinterpret_cast<uintptr_t>(writes[i]) % 16 != 0) return FSS_ERR_MISALIGNED;
    a.wr[i] = static_cast<fss::u32x4 *>(writes[i]);
  }
  if (bytes == 0) return FSS_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (n_reads * 10 + n_writes) {
    case 10: fss::launch_stream_mix<1, 0>(a, sh, s); break;
    case 11: fss::launch_stream_mix<1, 1>(a, sh, s); break;
    case 12: fss::launch_stream_mix<1, 2>(a, sh, s); break;
    case 20: fss::launch_stream_mix<2, 0>(a, sh, s); break;
    case 21: fss::launch_stream_mix<2, 1>(a, sh, s); break;
    case 22: fss::launch_stream_mix<2, 2>(a, sh, s); break;
    case 30: fss::launch_stream_mix<3, 0>(a, sh, s); break;
    case 31: fss::launch_stream_mix<3, 1>(a, sh, s); break;
    default: fss::launch_stream_mix<3, 2>(a, sh, s); break;
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    fss::tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

}  // extern "C"
