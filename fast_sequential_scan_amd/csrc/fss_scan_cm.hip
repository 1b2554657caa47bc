// Channel-major (bs, d, seq) scan kernels and their host side.
#include "fss_device.h"
#include "fss_host.h"

namespace fss {

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
    if (ok[r]) {
      const int64_t off = (row * seq + t_base) * E::kBytes;
      a[r].template load<(BWD ? kNtABwd : kNtAFwd)>(uniform_ptr((gcptr_t)p.in_a + off) + lane_off);
      b[r].template load<(BWD ? kNtBBwd : kNtBFwd)>(uniform_ptr((gcptr_t)p.in_b + off) + lane_off);
    }
  }
  if (BWD) {
    // alpha[t_hi+1] for the first step: from the neighbouring lane, except at the end of
    // the wave's slice
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      OneT ea;
      ea.fill(0.0f);
      if (lane == 0 && ok[r] && t_hi + 1 < seq) ea.load((gcptr_t)p.in_a + ((row0 + r) * seq + t_hi + 1) * E::kBytes);
      const float from_prev = __shfl_up(a[r].get(0), 1);  // lane-1 holds timesteps just above ours
      edge_a[r] = lane == 0 ? ea.get(0) : from_prev;
    }
  }
  // The saved h only feeds phase 3: its loads go out inside the chain phase, behind the
  // look-back's, and travel while the chain is resolved.
  OneT eh[BWD ? ROWS : 1];
  auto load_h = [&] {
    if (BWD) {
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        eh[r].fill(0.0f);
        hp[r].fill(0.0f);
        if (ok[r]) {
          const int64_t off = ((row0 + r) * seq + t_base) * E::kBytes;
          hp[r].template load<kNtH>(uniform_ptr((gcptr_t)p.in_h + off) + lane_off);
        }
        if (lane == 63 && ok[r] && t_lo >= 1) eh[r].load((gcptr_t)p.in_h + ((row0 + r) * seq + t_lo - 1) * E::kBytes);
      }
    }
  };

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
        B[r] = fma0(A[r], pb, B[r]);
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
  if (c.chained || c.n_waves > 1)
    chain_chunks<1, BWD>(p, c, &mA, &mB, nullptr, &slice_in, load_h);
  else
    load_h();
  if (BWD) {
    // h[t_lo-1] for the last step: from the neighbouring lane, except at the end of the slice
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const float from_next = __shfl_down(hp[r].get(VEC - 1), 1);  // lane+1 holds timesteps just below ours
      edge_h[r] = lane == 63 ? eh[r].get(0) : from_next;
    }
  }

  // ---- phase 3 ---------------------------------------------------------------------------
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    keep_packed(a[r]);
    keep_packed(b[r]);
    if (BWD) keep_packed(hp[r]);
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    float state = fma0(A[r], lane_read(slice_in, r), B[r]);
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
  __shared__ uint32_t s_ready[16];  // per wave: see announce_map

  TileCtx c;
  c.wcol = 0;
  c.lane = threadIdx.x & 63;
  c.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  c.n_waves = blockDim.x >> 6;
  c.look = p.look_waves;
  float2 *const lds_maps = reinterpret_cast<float2 *>(lds);  // laid out as in scan_kernel with one slot per lane
  c.lds_pred = lds_maps + 2 * c.n_waves * 64;
  c.seq = p.seq;
  c.s_ready = s_ready;
  if (threadIdx.x < 16) s_ready[threadIdx.x] = 0u;
  __syncthreads();
  c.row_bytes = 0;
  c.lane_off = 0;
  c.col_ok = true;
  c.tile_base = c.chan_row = c.r0 = 0;
#ifdef FSS_TRACE
  c.trace_wave = 0;
#endif
  c.chained = p.n_chunks > 1;
  c.tag = c.chained ? __builtin_amdgcn_readfirstlane(ld_u32(p.hdr + HDR_EPOCH)) + 1u : 0u;

  uint32_t parity = 0;
  uint32_t tile_no = 0;
  for (uint32_t tile = blockIdx.x; tile < static_cast<uint32_t>(p.n_tiles); tile += gridDim.x, parity ^= 1u) {
    c.tile_no = ++tile_no;
    c.lds_map = lds_maps + parity * c.n_waves * 64;
    const uint32_t chunk = __builtin_amdgcn_readfirstlane(tile / static_cast<uint32_t>(p.n_ctiles));
    const uint32_t ctile = tile - chunk * static_cast<uint32_t>(p.n_ctiles);
    c.chunk = static_cast<int>(chunk);
    c.ctile = static_cast<int>(ctile);
    c.last = c.chunk == p.n_chunks - 1;
    c.anchor = __builtin_amdgcn_readfirstlane(chain_anchor(c.chunk, p.period, p.look_waves * kMaxSpan));
    c.span = __builtin_amdgcn_readfirstlane(chunk_span(c.chunk - c.anchor, p.look_waves));
    cm_tile<E, VEC, ROWS, BWD>(p, c, static_cast<int64_t>(ctile) * ROWS, p.d);
  }
  count_out(p, c);
}

// ---- launching ---------------------------------------------------------------------

template <typename E, int VEC, bool BWD>
int launch_cm_one(const ScanArgs &args, const CmPlan &pl, int max_groups, hipStream_t stream) {
  constexpr int kRows = BWD ? kCmRowsBwd : kCmRowsFwd;
  static int resident[17] = {0};
  const int waves = pl.waves;
  const size_t lds = lds_bytes(waves, 1);
  const int fit = resident_workgroups(cm_scan_kernel<E, VEC, kRows, BWD>, waves, lds, resident);
  if (fit <= 0) return FSS_ERR_LAUNCH;
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
  args.n_groups = static_cast<int32_t>(pl.n_rowtiles);
  args.wg_cols = 1;
  args.look_waves = look_waves(pl.waves, 1);
  args.period = chain_period(pl.n_rowtiles, pl.waves);
  args.spin_limit = __atomic_load_n(&g_spin_limit, __ATOMIC_RELAXED);
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
