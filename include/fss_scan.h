/*
 * fss_scan.h - C ABI of the MI355X (gfx950) linear-recurrence scan library.
 *
 * Computes, independently for each of the bs*d channels of row-major
 * contiguous (bs, seq, d) tensors,
 *
 *   forward    h[0] = beta[0];  h[t] = alpha[t]*h[t-1] + beta[t]      (t = 1..seq-1)
 *   backward   g[seq-1] = dout[seq-1];  g[t] = alpha[t+1]*g[t+1] + dout[t]
 *              grad_beta[t] = g[t];  grad_alpha[t] = g[t]*h[t-1] (t >= 1);  grad_alpha[0] = 0
 *
 * with fp32 carries in both directions.  The values in alpha[:,0,:] are never used
 * (they may be NaN).  Long sequences are scanned in chunks whose effect on the state is
 * handed on as x -> A*x + B with A the product of the chunk's alphas (up to 512 of them):
 * with |alpha| <= 1, the recurrence's regime, this matches the sequential order to fp32
 * rounding.  With |alpha| > 1 over long stretches A can overflow to inf; a state of exactly
 * 0 still stays 0 (as sequentially), but a tiny non-zero state times such an A is inf where
 * the sequential order might have stayed finite.  An alpha that is itself +-inf or NaN makes
 * exactly the outputs non-finite that the sequential order makes non-finite (that step and
 * every later one of its channel); which of NaN and +-inf an output then holds can depend on
 * the launch configuration (a composed map with an infinite coefficient can turn the
 * sequential order's -inf into inf - inf = NaN).
 *
 * What is guaranteed about the bits.  The order in which the chunks' maps are composed is
 * fixed by the shape and the launch configuration (fss_config: vec, steps, waves, cols) and
 * by nothing else: not the timing of the workgroups, the stream, the cache policy, the number
 * of workgroups launched (max_groups), the device's CU count, the workspace (the caller's or
 * the static one of fss_scan_fwd_noalloc) or earlier calls.  So one call returns the same
 * bits on every run, as the reference does by walking each channel with one thread
 * (csrc/include/sequential_scan_kernel_bf16.cuh:121-151).  Two DIFFERENT configurations agree
 * only to fp32 rounding of the carries (they cut the sequence at different places); where no
 * chunk is needed (one wave covers the sequence) the result is the sequential one bit for bit
 * given fused multiply-adds.  The configuration the library chooses by itself is a function
 * of shape, dtype, direction and the tensors' common alignment (fss_choose_config).
 *
 * This header replaces, for a host written in any language, the pybind11 module
 * `sequential_scan_cuda` of the reference (csrc/sequential_scan.cpp:13-22) and
 * the host launchers behind it (csrc/sequential_scan_kernel.cu).  The entry
 * points take plain device pointers, sizes and a HIP stream; no torch types.
 *
 * Conventions
 *   - Every pointer is a device pointer on the current HIP device.
 *   - The library never allocates or frees device memory.  Outputs and the
 *     workspace are the caller's.
 *   - Calls are asynchronous on `stream` (a hipStream_t passed as void*; NULL is
 *     the null stream).  No entry point synchronises except fss_workspace_status.
 *   - Scans launched by one process on different streams of a device do not overlap:
 *     a scan fills the device with workgroups that wait for each other, so the library
 *     makes a launch on a new stream wait (hipStreamWaitEvent) for the work queued on
 *     the stream of the previous scan.  Streams under graph capture are exempt: do not
 *     replay two graphs containing scans concurrently, and do not share the device
 *     between processes that scan at the same time - co-scheduled scans can stall each
 *     other until their bounded waits give up (FSS_ERR_CHAIN_TIMEOUT).
 *   - Every entry point returns an fss_status (0 = ok); nothing throws.
 *   - Any seq >= 1 and any d >= 1 are accepted (the reference needs seq >= 2/3 and
 *     d in {512,768,1024,1536,2048}: csrc/sequential_scan_kernel.cu:136-184).
 *     Tensors need only their element alignment; 4/8/16-byte aligned tensors
 *     with d a multiple of 2/4/8 elements take the vectorised paths.
 *   - Offsets are 64-bit (the reference's are 32-bit:
 *     csrc/include/sequential_scan_kernel_bf16.cuh:63-70).
 *
 * Workspace
 *   When the sequence is split into more than one chunk the kernels chain the
 *   chunks through a small workspace (per-chunk carries with validity tags,
 *   completion counters).  Size it with fss_workspace_bytes, reset it ONCE with
 *   fss_workspace_init; after that every scan call leaves it ready for the
 *   next one, so steady-state calls launch exactly one kernel.  One workspace
 *   must not be used by two calls that may run concurrently (use one per
 *   stream).  A workspace sized for one shape serves any shape whose
 *   fss_workspace_bytes is not larger.  Validity tags are a 32-bit launch
 *   counter kept in the workspace: call fss_workspace_init again before a
 *   workspace has served 2^32-1 chained launches.
 */
#ifndef FSS_SCAN_H_
#define FSS_SCAN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSS_ABI_VERSION 3

typedef enum fss_status {
  FSS_OK = 0,
  FSS_ERR_NULL_POINTER = 1,    /* a required pointer is NULL                      */
  FSS_ERR_BAD_SHAPE = 2,       /* bs, seq or d < 0, or a product overflows        */
  FSS_ERR_MISALIGNED = 3,      /* a tensor is not aligned to its element size     */
  FSS_ERR_WORKSPACE_SMALL = 4, /* workspace NULL or smaller than fss_workspace_bytes */
  FSS_ERR_BAD_CONFIG = 5,      /* explicit launch configuration not supported     */
  FSS_ERR_LAUNCH = 6,          /* HIP reported an error at launch (see fss_last_hip_error) */
  FSS_ERR_CHAIN_TIMEOUT = 7,   /* reported by fss_workspace_status: a chunk gave up waiting */
  FSS_ERR_UNSUPPORTED_DEVICE = 8, /* current device is not gfx950                 */
  FSS_ERR_TOO_LARGE = 9        /* fss_scan_fwd_noalloc: the shape needs more than FSS_NOALLOC_SCRATCH_BYTES */
} fss_status;

/* FSS_F16 (IEEE half) has no counterpart in the reference; same kernels, same fp32 carries */
typedef enum fss_dtype { FSS_BF16 = 0, FSS_F32 = 1, FSS_F16 = 2 } fss_dtype;
/* FSS_GATED_*: the gated scans below (they chunk the sequence differently) */
typedef enum fss_dir { FSS_FWD = 0, FSS_BWD = 1, FSS_GATED_FWD = 2, FSS_GATED_BWD = 3 } fss_dir;

/*
 * Launch configuration.  Zero in a field means "choose for me".
 *   vec    channels per lane (bf16/fp16: 1,2,4,8; fp32: 1,2,4); needs d % vec == 0 and
 *          tensors aligned to vec elements
 *   steps  timesteps each lane keeps in registers (8, 16 or 32; vec*steps bounded
 *          by the register budget of the direction)
 *   waves  wavefronts per workgroup: 1..16; at most 8 with vec = 4 and wherever a lane with
 *          vec = 2 holds more than 64 dwords of rows (the plain backward at 32 steps); at most
 *          4 with vec = 8 (the kernels are compiled so that what a lane holds fits its registers)
 *   max_groups  upper bound on the workgroups launched; 0 = as many as the device
 *          holds resident at once (the grid is persistent: workgroups loop over
 *          tiles, and never more are launched than are resident together)
 *   cols   adjacent column tiles (of 64*vec channels each) a workgroup covers side by
 *          side, 1 or 2 (row-major kernels only; must divide waves, and with 2 the row
 *          must hold an even number of column tiles).  A workgroup scans
 *          (waves/cols)*steps consecutive timesteps of 64*vec*cols channels at a time;
 *          two column tiles side by side make every row a workgroup touches 512
 *          contiguous bytes instead of 256, which the memory system serves faster
 * Results depend on vec, steps, waves and cols only through fp32 rounding of the carries
 * handed between chunks (a different tiling cuts the sequence at different places), and not at
 * all on max_groups: see "What is guaranteed about the bits" above.
 */
typedef struct fss_config {
  int32_t vec;
  int32_t steps;
  int32_t waves;
  int32_t max_groups;
  int32_t cols;
} fss_config;

int fss_abi_version(void);
const char *fss_strerror(int status);
/* hipError_t of the most recent failed HIP call made by this thread, 0 if none */
int fss_last_hip_error(void);

/* Bytes of workspace a scan of this shape needs (a multiple of 256, never 0), whatever
 * the alignment of its tensors (which changes how the library tiles the scan).
 * cfg may be NULL. */
size_t fss_workspace_bytes(int64_t bs, int64_t seq, int64_t d, int dtype, int dir,
                           const fss_config *cfg);
/* Upper bound over all directions (gated included), all three dtypes and every
 * configuration the library may choose by itself. */
size_t fss_workspace_bytes_max(int64_t bs, int64_t seq, int64_t d);
/* Resets the workspace with a fill kernel on `stream` (graph-capturable). */
int fss_workspace_init(void *workspace, size_t bytes, void *stream);
/* Synchronises `stream`, then reports FSS_OK or FSS_ERR_CHAIN_TIMEOUT and clears
 * the sticky error word.  For tests and debugging.  workspace = NULL stands for the static
 * array of fss_scan_fwd_noalloc on the current device. */
int fss_workspace_status(void *workspace, void *stream);
/*
 * A chunk that gives up waiting (see FSS_ERR_CHAIN_TIMEOUT above) hands on a NaN state, so
 * every output from there to the end of its sequence is NaN, and sets the workspace's
 * sticky error word.  To learn of it without a device call or a synchronisation, attach a
 * 32-bit word that the device can write and the host can read (hipHostMalloc memory): a
 * kernel that gives up stores 1 there as well.  The host polls the word whenever it likes
 * (it is set by the time the kernel has finished) and clears it itself.  Asynchronous on
 * `stream` (a small kernel, graph-capturable); fss_workspace_init detaches the word; flag =
 * NULL detaches it too.  workspace = NULL stands for the static array of fss_scan_fwd_noalloc
 * on the current device (the word then stays attached when the library zeroes that array
 * again).  No counterpart in the reference, whose kernels never wait.
 */
int fss_workspace_attach_flag(void *workspace, uint32_t *flag, void *stream);
/*
 * Test hook: the number of polls after which a look-back gives up (default 2^20, seconds of
 * waiting).  0 makes every look-back give up before its first poll, which exercises the
 * time-out path on a healthy device with every kernel still running to completion.
 * Process-wide; returns the previous value.
 */
uint32_t fss_debug_set_spin_limit(uint32_t polls);
/*
 * Test hook: after how many calls per device fss_scan_fwd_noalloc zeroes its static array again
 * (default 2^31; 0 restores the default).  Process-wide; returns the previous value.
 */
uint64_t fss_debug_noalloc_reinit_after(uint64_t launches);
/*
 * Test hook (host only, no device call): the order in which the row-major kernels take
 * their tiles.  Tiles are numbered chunk-major (tile = chunk * n_groups + slot) and workgroup b
 * of a grid of `grid` workgroups takes tiles b, b + grid, ...; groups[tile] receives the column
 * group that tile stands for, for tile = 0 .. n_tiles-1.  Every chunk's slots must map onto its
 * groups one to one.  No counterpart in the reference (one block per batch row, no tiles).
 */
int fss_debug_tile_groups(int32_t n_groups, int32_t grid, int32_t n_tiles, int32_t *groups);

/*
 * Test hooks (host only, no device call): how a row-major scan of this shape chains its chunks.
 * The state entering chunk k of a sequence is composed from the maps of chunks k-1 .. a+1 and
 * the outgoing state of chunk a = fss_debug_chain_anchor(k, period, look * max_span): the last
 * chunk of the round of `period` chunks before k's, or the last multiple of look * max_span
 * below k if that is nearer.  The k - a chunks are dealt out nearest first to `look` waves,
 * ceil((k - a) / look) consecutive chunks each; each wave composes its chunks nearest first,
 * then the waves' results are folded in wave order.  None of this depends on timing, so a
 * chained scan returns the same bits from run to run.  out[0..7] = number of chunks, waves
 * along time per chunk, timesteps per lane (a chunk is their product), period, look, max_span,
 * vec, cols.  No counterpart in the reference, where one thread walks a channel in order
 * (csrc/include/sequential_scan_kernel_bf16.cuh:121-151).
 */
int fss_debug_chain_plan(int64_t bs, int64_t seq, int64_t d, int dtype, int dir, size_t align_bytes,
                         const fss_config *cfg, int32_t *out);
int32_t fss_debug_chain_anchor(int32_t chunk, int32_t period, int32_t stride);

/* The configuration the library would choose for this shape (for reporting). */
int fss_choose_config(int64_t bs, int64_t seq, int64_t d, int dtype, int dir,
                      size_t align_bytes, fss_config *out);

/*
 * bf16 forward.  Replaces scan_forward_half
 * (csrc/sequential_scan.cpp:19, csrc/sequential_scan_kernel.cu:126-187, kernel
 * csrc/include/sequential_scan_kernel_bf16.cuh:58-167).  h is written in full.
 */
int fss_scan_fwd_bf16(const void *alpha, const void *beta, void *h, int64_t bs,
                      int64_t seq, int64_t d, void *workspace,
                      size_t workspace_bytes, void *stream);

/*
 * bf16 backward.  Replaces scan_backward_half
 * (csrc/sequential_scan.cpp:21, csrc/sequential_scan_kernel.cu:189-268, kernel
 * csrc/include/sequential_scan_kernel_bf16.cuh:169-390).  `h` is the stored
 * forward output.  The tensors must not overlap, with one exception: grad_beta may
 * be dout itself (the same address: the gradient is then computed in place, and the
 * backward allocates one tensor, as the reference's does) - every lane has read the
 * rows of dout it owns before it stores one of them, and no other lane touches them.
 * The reference writes grad_beta over `h` instead (csrc/sequential_scan_kernel.cu:197),
 * which is only safe when one thread walks a channel's whole sequence in order; here
 * neighbouring chunks of a sequence run concurrently and each reads the last row of
 * `h` before its own chunk, so grad_beta over `h` (or any partial overlap) stays
 * forbidden.  The same holds for fss_scan_bwd_f32, fss_scan_bwd_ex and
 * fss_scan_bwd_state (row-major layout only).
 */
int fss_scan_bwd_bf16(const void *alpha, const void *h, const void *dout,
                      void *grad_alpha, void *grad_beta, int64_t bs, int64_t seq,
                      int64_t d, void *workspace, size_t workspace_bytes,
                      void *stream);

/* fp32 forward.  Replaces scan_forward (csrc/sequential_scan.cpp:15,
 * csrc/sequential_scan_kernel.cu:7-58, csrc/include/sequential_scan_kernel.cuh:35-129). */
int fss_scan_fwd_f32(const void *alpha, const void *beta, void *h, int64_t bs,
                     int64_t seq, int64_t d, void *workspace,
                     size_t workspace_bytes, void *stream);

/* fp32 backward.  Replaces scan_backward (csrc/sequential_scan.cpp:17,
 * csrc/sequential_scan_kernel.cu:60-124, csrc/include/sequential_scan_kernel.cuh:131-301). */
int fss_scan_bwd_f32(const void *alpha, const void *h, const void *dout,
                     void *grad_alpha, void *grad_beta, int64_t bs, int64_t seq,
                     int64_t d, void *workspace, size_t workspace_bytes,
                     void *stream);

/*
 * How the scans treat the memory-side cache (process-wide; no counterpart in the reference).
 *   FSS_CACHE_AUTO       (default) assumes that the tensors of a step are touched again soon,
 *                        as in a benchmark loop or a short pipeline: a small forward output is
 *                        left in the cache for its reader, and the tensors nothing reads again
 *                        (beta in the forward, dout in the backward) are read with the
 *                        streaming hint only when the inputs of a step cannot fit the cache.
 *   FSS_CACHE_STREAMING  assumes that nothing is found in the cache again (a scan inside a
 *                        large model): the forward output always carries the streaming hint,
 *                        beta and dout are always read with it, and so is alpha at its last use,
 *                        in the backward (measured 1-6 % faster then, 3-8 % slower in a loop
 *                        over one set of tensors).
 * The policy selects cache hints on loads and stores and nothing else - never the tiling - so
 * results are bit-identical under both.  It acts on the plain scans over (bs, seq, d) tensors,
 * with or without states (with states: in the kernels that large shapes run - 32 steps per lane
 * in the forward, 16 steps and 4 bytes per lane in the backward); the gated and the channel-major
 * scans carry the same hints under both (outputs and the backward's reads of h streamed,
 * everything else cached).  Returns the previous policy, or -1 for an unknown one.
 */
enum fss_cache_policy { FSS_CACHE_AUTO = 0, FSS_CACHE_STREAMING = 1 };
int fss_set_cache_policy(int policy);

/*
 * fss_scan_fwd_ex with cfg = NULL for callers that cannot allocate device memory and have
 * no workspace to bring (code under graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): the chaining words live in a static device array of
 * FSS_NOALLOC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process
 * ends.  No counterpart in the reference.  The call allocates and frees nothing, in the
 * library or in the HIP runtime (the first call on a device looks up the array's address
 * and creates the event that orders scans across streams).  A shape whose
 * fss_workspace_bytes(.., FSS_FWD, NULL) exceeds the array is refused with
 * FSS_ERR_TOO_LARGE.  All calls of one process on one GPU share that GPU's array (another
 * process has its own copy): calls that can overlap on one GPU race - the library already
 * orders scans across streams; replays of different captured graphs are the caller's to keep
 * apart.  Results are bit-identical to fss_scan_fwd_ex with cfg = NULL (same kernel, same
 * plan; only where the chaining words live differs).  The validity tags of the array are a
 * 32-bit launch counter like a workspace's; the library counts the calls through this entry
 * point per device and zeroes the array again (a fill kernel on the call's stream) every 2^31
 * calls, so a long-lived process never meets a wrapped tag.  A chain time-out is reported as
 * for any workspace: fss_workspace_status(NULL, stream), or a word attached with
 * fss_workspace_attach_flag(NULL, flag, stream).
 */
#define FSS_NOALLOC_SCRATCH_BYTES (16u << 20)
int fss_scan_fwd_noalloc(int dtype, const void *alpha, const void *beta, void *h, int64_t bs,
                         int64_t seq, int64_t d, void *stream);

/* Same four operations with an explicit dtype and launch configuration (tuning,
 * and tests that results do not depend on how the sequence is chunked). */
int fss_scan_fwd_ex(int dtype, const void *alpha, const void *beta, void *h,
                    int64_t bs, int64_t seq, int64_t d, void *workspace,
                    size_t workspace_bytes, void *stream, const fss_config *cfg);
int fss_scan_bwd_ex(int dtype, const void *alpha, const void *h, const void *dout,
                    void *grad_alpha, void *grad_beta, int64_t bs, int64_t seq,
                    int64_t d, void *workspace, size_t workspace_bytes,
                    void *stream, const fss_config *cfg);

/*
 * The same scans with a state entering and leaving the sequence, for streaming
 * over segments of a longer sequence (and for sharding one over devices).  No
 * counterpart in the reference, whose scan always starts from h[-1] = 0.
 * States are fp32 (bs, d) row-major whatever the tensors' dtype; any may be NULL.
 *
 *   forward   h[-1] = h_before (then alpha[:,0,:] IS read: h[0] = alpha[0]*h[-1] + beta[0]);
 *             h_last = the un-rounded state after the last step.
 *   backward  g[seq-1] = dout[seq-1] + grad_h_last;
 *             grad_alpha[0] = g[0]*h_before (0 without h_before);
 *             grad_h_before = alpha[0]*g[0] (needs h_before).
 * Scanning two adjacent segments with h_last of the first as h_before of the second,
 * and grad_h_before of the second as grad_h_last of the first, equals scanning their
 * concatenation.
 */
int fss_scan_fwd_state(int dtype, const void *alpha, const void *beta, void *h,
                       const float *h_before, float *h_last, int64_t bs, int64_t seq,
                       int64_t d, void *workspace, size_t workspace_bytes,
                       void *stream, const fss_config *cfg);
int fss_scan_bwd_state(int dtype, const void *alpha, const void *h, const void *dout,
                       const float *h_before, const float *grad_h_last,
                       void *grad_alpha, void *grad_beta, float *grad_h_before,
                       int64_t bs, int64_t seq, int64_t d, void *workspace,
                       size_t workspace_bytes, void *stream, const fss_config *cfg);

/*
 * Gated scan: the gating of a Hawk / RG-LRU style block fused in front of the scan,
 *
 *   alpha = sigmoid(gate),  beta = x * sqrt(1 - alpha^2),  h = scan(alpha, beta)
 *
 * from the pre-activations `gate` and `x`, both (bs, seq, d) of `dtype`; alpha and beta
 * never exist in memory (forward 3 tensors of traffic instead of 7, forward+backward 9
 * instead of 18).  No counterpart in the reference, which is handed alpha and beta
 * (sequential_scan/scan_cuda.py:16-27); a model computes them with elementwise kernels first.
 * alpha and beta are rounded to `dtype` exactly where the plain scan would have read
 * them from memory, so h equals fss_scan_fwd on those rounded tensors.
 *
 * Backward, with g the reversed-time scan of dout under alpha (as in fss_scan_bwd) and
 * s = sqrt(1 - alpha^2):
 *   grad_x[t]    = g[t] * s[t]
 *   grad_gate[t] = g[t] * (h[t-1] - x[t]*alpha[t]/s[t]) * alpha[t]*(1 - alpha[t])   (h[-1] = 0)
 * Where alpha rounds to exactly 1 (s = 0) the x term is dropped (torch's autograd gives
 * inf/nan there).  gate[:,0,:] is read (beta[0] depends on it).  The six tensors of a
 * backward must not overlap.  vec is 1 or 2 (bf16, fp16) / 1 (fp32); steps at most 16 in the
 * backward.  Use FSS_GATED_FWD / FSS_GATED_BWD as `dir` of fss_workspace_bytes and
 * fss_choose_config.
 */
int fss_gated_scan_fwd(int dtype, const void *gate, const void *x, void *h, int64_t bs,
                       int64_t seq, int64_t d, void *workspace, size_t workspace_bytes,
                       void *stream, const fss_config *cfg);
int fss_gated_scan_bwd(int dtype, const void *gate, const void *x, const void *h,
                       const void *dout, void *grad_gate, void *grad_x, int64_t bs,
                       int64_t seq, int64_t d, void *workspace, size_t workspace_bytes,
                       void *stream, const fss_config *cfg);

/*
 * The gated scan with a state entering and leaving the sequence: fss_gated_scan_fwd /
 * fss_gated_scan_bwd with the state arguments, semantics and chaining property of
 * fss_scan_fwd_state / fss_scan_bwd_state (alpha there = sigmoid(gate) here):
 *   forward   h[-1] = h_before;  h_last = the un-rounded state after the last step.
 *   backward  g[seq-1] = dout[seq-1] + grad_h_last;  h[-1] = h_before in grad_gate[0];
 *             grad_h_before = alpha[0]*g[0] (needs h_before).
 * No counterpart in the reference.  States are fp32 (bs, d); any may be NULL.
 */
int fss_gated_scan_fwd_state(int dtype, const void *gate, const void *x, void *h,
                             const float *h_before, float *h_last, int64_t bs, int64_t seq,
                             int64_t d, void *workspace, size_t workspace_bytes, void *stream,
                             const fss_config *cfg);
int fss_gated_scan_bwd_state(int dtype, const void *gate, const void *x, const void *h,
                             const void *dout, const float *h_before, const float *grad_h_last,
                             void *grad_gate, void *grad_x, float *grad_h_before, int64_t bs,
                             int64_t seq, int64_t d, void *workspace, size_t workspace_bytes,
                             void *stream, const fss_config *cfg);

/*
 * Channel-major layout: tensors are (bs, d, seq) row-major, i.e. every (batch, channel)
 * pair is a contiguous run of seq timesteps - the layout of the `accelerated-scan`
 * package the reference benchmarks against after a permute().contiguous() of its own
 * (bs, seq, d) tensors (benchmark.py:67-72).  Same recurrences and gradients as
 * fss_scan_fwd_ex / fss_scan_bwd_ex, per run; the values in alpha[..., 0] are never used.  Note the
 * argument order bs, d, seq.  Of `cfg` only vec (timesteps per lane: 1, 2 or 8 for the
 * 16-bit types, 1 or 4 for fp32; seq % vec == 0 and tensors aligned to vec elements),
 * waves and max_groups are used; steps must be 0.  A workgroup of 8 waves covers
 * 4096 (16-bit) / 2048 (fp32) timesteps, and only longer sequences use the workspace:
 * size it with fss_cm_workspace_bytes (an upper bound over alignments).
 */
size_t fss_cm_workspace_bytes(int64_t bs, int64_t d, int64_t seq, int dtype, int dir,
                              const fss_config *cfg);
int fss_scan_fwd_cm(int dtype, const void *alpha, const void *beta, void *h, int64_t bs,
                    int64_t d, int64_t seq, void *workspace, size_t workspace_bytes,
                    void *stream, const fss_config *cfg);
int fss_scan_bwd_cm(int dtype, const void *alpha, const void *h, const void *dout,
                    void *grad_alpha, void *grad_beta, int64_t bs, int64_t d, int64_t seq,
                    void *workspace, size_t workspace_bytes, void *stream,
                    const fss_config *cfg);

/* Plain device-to-device copy kernel of `bytes` bytes (a multiple of 16; both
 * pointers 16-byte aligned).  Exists so that hardware counters read for the
 * scan kernels can be scaled by what the same counters read for a transfer of
 * known size. */
int fss_copy_bytes(const void *src, void *dst, size_t bytes, void *stream);

/*
 * Calibration kernel: the plainest kernel that moves a scan's mix of streams.  Reads `n_reads`
 * (1..3) buffers and writes `n_writes` (0..2) buffers of `bytes` bytes each (a multiple of 16;
 * all pointers 16-byte aligned), linearly, 16 bytes per lane and access, with no dependence
 * between elements; `nontemporal_writes` marks the stores as the scans mark theirs.  writes[0]
 * receives the XOR of the reads, writes[1] its complement.  With n_writes = 0, writes[0] must
 * still name 16 writable bytes (a sink that is not written in practice).  `launch_shape` is
 * NULL (2048 workgroups of 256 threads, one vector per lane and iteration, ordinary loads) or
 * names four ints: workgroups (1..2^20), threads per workgroup (a multiple of 64, at most
 * 1024), vectors per lane and iteration (1 or 2, a grid stride apart, first loads issued
 * together), non-temporal loads (0 or 1); which shape streams fastest depends on the mix, so a
 * calibration tries a few and keeps the best.  The forward scan's mix is 2 reads + 1 write,
 * the backward's 3 reads + 2 writes: what this kernel reaches over buffers that fit no cache is
 * what the machine's memory system gives that mix, and bench.py reports the scans against it
 * next to the nominal 8 TB/s.  No counterpart in the reference.
 */
int fss_stream_mix(const void *const *reads, int n_reads, void *const *writes, int n_writes,
                   size_t bytes, int nontemporal_writes, const int *launch_shape, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FSS_SCAN_H_ */
