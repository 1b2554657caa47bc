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
//     2. wave 0 composes the waves' maps through LDS as they arrive and publishes the chunk's
//        map; at the same time up to 16 waves fetch the maps of the earlier chunks the chunk is
//        to compose and the outgoing state of the one it starts from (its "anchor"), up to four
//        chunks per wave, so the look-back over the nearest chunks costs a few memory round
//        trips, not one per chunk (a look-back over (A,B) pairs in global memory whose order of
//        composition is fixed by the chunk's index: see chain_anchor in fss_device.h).
//        Every wave folds what they found into the chunk's incoming state and applies the maps
//        of the waves before it; wave 0 publishes the outgoing state.  The backward issues the
//        loads of its third tensor, which only phase 3 needs, inside this phase;
//     3. every lane re-runs the recurrence over its register-resident slice from
//        its true incoming state, in sequential order, and stores the results.
//   Because phase 3 restarts from the incoming state, only that state is
//   computed by re-associated arithmetic; within a slice the operation order is
//   exactly the sequential one.  And because which chunks are composed, and in which
//   grouping, depends on the chunk's index and the plan alone - never on which
//   earlier chunk happens to have finished - the result is a function of the inputs
//   and the launch configuration: the same bits on every run.
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
//   records an error in the workspace header (and in the host-visible word attached
//   to the workspace, if any) and carries on with a NaN state, so the grid always
//   drains and the outputs from there on are visibly poisoned.
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
#include "fss_device.h"
#include "fss_host.h"

// This file is compiled once per storage type and direction: FSS_RM_ELEM names the element
// type (BF16, F16 or F32), FSS_RM_BWD the direction (0 forward, 1 backward) and
// FSS_RM_LAUNCH the entry it defines (launch_rm_bf16_fwd, ...).
#if !defined(FSS_RM_ELEM) || !defined(FSS_RM_LAUNCH) || !defined(FSS_RM_BWD)
#error "define FSS_RM_ELEM, FSS_RM_BWD and FSS_RM_LAUNCH"
#endif

namespace fss {

// One tile, all three phases.  FULL: every row this wave touches exists and is
// interior and every lane has channels, so nothing is predicated; otherwise every
// access is guarded.  The two variants share no registers, so the guarded one
// costs the fast one nothing.
template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool FULL, int ALT>
__device__ __forceinline__ void scan_tile(const ScanArgs &p, const StateArgs<STATE> &st, const TileCtx &c) {
  using RowT = Row<E, VEC>;
  const int64_t seq = c.seq, row_bytes = c.row_bytes, r0 = c.r0;
  const uint32_t lane_off = c.lane_off;

  RowT a[STEPS], b[STEPS];
  RowT hp[BWD ? STEPS : 1];

  // How many steps of the slice lie inside the sequence, as a small wave-uniform integer (capped
  // one above the slice), and whether the slice starts the scan: the guards of the ragged variant
  // are then 32-bit scalar compares against constants (a 64-bit "r < seq" per row is a
  // vector compare whose lane mask the compiler keeps for phase 3, one register pair per row).
  const int valid = FULL ? STEPS + 1 : slice_steps_inside(seq, r0, STEPS + 1);
  const bool at_start = r0 == 0;

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
      const int row = (BWD && s == 0 && at_start) ? 1 : s;
      a[s].template load<(BWD ? (kNtABwd || ALT == 2) : kNtAFwd)>(uniform_ptr(pa + row * step_bytes) + lane_off);
      b[s].template load<(BWD ? (kNtBBwd || ALT != 0) : (kNtBFwd || ALT == 2))>(uniform_ptr(pb + s * step_bytes) + lane_off);
    } else {
      // Outside the sequence the step is the identity map (a=1, b=0).  The first step
      // of the plain scan has no predecessor (a=0), whatever alpha holds there; with a
      // state coming in, the forward applies alpha[0] to it and the backward adds it (a=1).
      a[s].fill((s >= valid || (STATE && BWD && s == 0 && at_start && st.state_in)) ? 1.0f : 0.0f);
      b[s].fill(0.0f);
      if (c.col_ok && s < valid) {
        if (s >= 1 || !at_start || (STATE && !BWD && st.state_in))
          a[s].template load<(BWD ? (kNtABwd || ALT == 2) : kNtAFwd)>(uniform_ptr(pa + s * step_bytes) + lane_off);
        b[s].template load<(BWD ? (kNtBBwd || ALT != 0) : (kNtBFwd || ALT == 2))>(uniform_ptr(pb + s * step_bytes) + lane_off);
      }
    }
  }

  if (FULL && at_start) {
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
      if (c.col_ok && s + 1 < valid)  // t - 1 >= 0
        hp[s].template load<kNtH>(uniform_ptr(ph + s * step_bytes) + lane_off);
    }
  };
  auto load_h_early = [&] {
    if (BWD) {
#pragma unroll
      for (int s = 0; s < kHEarly; ++s) load_h(s);
    }
  };

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
    load_h_early();
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
    chain_chunks<VEC, BWD>(p, c, mA, mB, STATE ? seq_in : nullptr, state, load_h_early);
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
    if (FULL || (c.col_ok && s < valid)) {
      RowT o;
      o.pack(state);
      o.template store<(BWD ? kNtOutBwd : (kNtOutFwd && ALT != 1))>(uniform_ptr(po0 + s * step_bytes) + lane_off);
      if (BWD) {
        if (!FULL && s + 1 == valid) {  // t = 0: grad_alpha[0] = g[0] * h[-1], 0 in the plain scan
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
  if (STATE && st.state_out && c.col_ok && r0 <= seq - 1 && seq - 1 < r0 + STEPS) {  // (once per tile)
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
// STATE: h[-1] and the gradient reaching the last state come in, the last state and the
// gradient with respect to h[-1] go out, exactly as in the plain scan (scan_tile).
// The backward needs alpha[t+1] as the coefficient of step t and alpha[t] for its
// elementwise part: a slice of STEPS steps loads STEPS+1 rows of the gate.
template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool FULL>
__device__ __forceinline__ void gated_tile(const ScanArgs &p, const StateArgs<STATE> &st, const TileCtx &c) {
  using RowT = Row<E, VEC>;
  const int64_t seq = c.seq, row_bytes = c.row_bytes, r0 = c.r0;
  const uint32_t lane_off = c.lane_off;
  constexpr int kARows = BWD ? STEPS + 1 : STEPS;

  RowT a[kARows], b[STEPS];
  RowT hp[BWD ? STEPS : 1], xs[BWD ? STEPS : 1];
  // (steps of the slice inside the sequence, capped two above the slice; see scan_tile)
  const int valid = FULL ? STEPS + 2 : slice_steps_inside(seq, r0, STEPS + 2);
  const bool at_start = r0 == 0;

  // forward: a[s] = gate row t = r0+s.  backward: a[s] = gate row t+1 = seq-(r0+s), s = 0..STEPS
  const int64_t t_first = BWD ? seq - 1 - r0 : r0;
  gcptr_t pa = (gcptr_t)p.in_a + c.tile_base + (BWD ? t_first + 1 : t_first) * row_bytes;
  gcptr_t pb = (gcptr_t)p.in_b + c.tile_base + t_first * row_bytes;
  const int64_t step_bytes = BWD ? -row_bytes : row_bytes;

  // ---- phase 1a: loads ---------------------------------------------------------------
#pragma unroll
  for (int s = 0; s < kARows; ++s) {
    // the gate row of a[s] exists: forward r < seq; backward 1 <= r <= seq  (r = r0 + s)
    const bool a_ok = FULL || (c.col_ok && (BWD ? ((s >= 1 || !at_start) && s <= valid) : (s < valid)));
    if (!FULL) a[s].fill(0.0f);
    if (a_ok) a[s].template load<(BWD ? kNtABwd : kNtAFwd)>(uniform_ptr(pa + s * step_bytes) + lane_off);
    if (s < STEPS) {
      if (!FULL) b[s].fill(0.0f);
      if (FULL || (c.col_ok && s < valid)) b[s].template load<(BWD ? kNtBBwd : kNtBFwd)>(uniform_ptr(pb + s * step_bytes) + lane_off);
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
      if (c.col_ok && s + 1 < valid)  // t - 1 >= 0
        hp[s].template load<kNtH>(uniform_ptr(ph + s * step_bytes) + lane_off);
      if (c.col_ok && s < valid) xs[s].template load<kNtH>(uniform_ptr(px + s * step_bytes) + lane_off);
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
    float al[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) al[v] = sigmoid_f32(a[s].get(v));
    // (backward with a gradient coming in through the last state: it is added, coefficient 1)
    if (!FULL && (s >= valid + (BWD ? 1 : 0) || !c.col_ok || (STATE && BWD && s == 0 && at_start && st.state_in))) {
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
      const bool ident = !FULL && BWD && s >= valid;  // backward: a[s] with r == seq is alpha[0], not a coefficient
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float av = ident ? 1.0f : a[s].get(v);
        mB[v] = __builtin_fmaf(av, mB[v], b[s].get(v));
        mA[v] *= av;
      }
    }
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
#pragma unroll
    for (int v = 0; v < VEC; ++v) state[v] = seq_in[v];
  } else {
    chain_chunks<VEC, false>(p, c, mA, mB, STATE ? seq_in : nullptr, state, [] {});
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
    const bool ident = !FULL && BWD && s >= valid;
    float o0[VEC], o1[VEC];
    // t = 0 with a state coming in: h[-1] is that state, and alpha[0]*g[0] goes out
    const bool t_zero = STATE && BWD && !FULL && s + 1 == valid;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      state[v] = __builtin_fmaf(ident ? 1.0f : a[s].get(v), state[v], b[s].get(v));
      if (BWD) {
        const float at = a[s + 1].get(v);  // alpha[t]
        const float om = __builtin_fmaf(-at, at, 1.0f);
        const float rs = om > 0.0f ? __builtin_amdgcn_rsqf(om) : 0.0f;
        o0[v] = state[v] * (om * rs);
        float h_prev = hp[s].get(v);
        if constexpr (STATE) {
          if (t_zero && c.col_ok) {
            const int64_t ch = c.chan_row + c.lane * VEC + v;
            if (st.h_before) h_prev = st.h_before[ch];
            if (st.state_out) st.state_out[ch] = at * state[v];
          }
        }
        const float inner = __builtin_fmaf(-xs[s].get(v) * at, rs, h_prev);
        o1[v] = state[v] * inner * (at - at * at);
      } else {
        o0[v] = state[v];
      }
    }
    if (FULL || (c.col_ok && s < valid)) {
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
  // forward: the wave whose slice holds the last step hands out the final state (the steps
  // past the end are identity maps)
  if (STATE && !BWD && st.state_out && c.col_ok && r0 <= seq - 1 && seq - 1 < r0 + STEPS) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) st.state_out[c.chan_row + c.lane * VEC + v] = state[v];
  }
}

// STATE: the variant that honours the optional incoming/outgoing state rows of ScanArgs;
// the plain and the gated scan are compiled without them.  GATED: the gated scan.
// ALT: the cache policy of the plain scan (hints only, never the arithmetic).  Forward: 0 stores
// h with the non-temporal hint, 1 without it (small outputs, left in the cache for their reader),
// 2 = 0 and reads beta, which nothing reads again, with the hint (large tensors).  Backward:
// 1 reads dout with the hint (large tensors), 2 = 1 and reads alpha with it as well (its last
// use in a step; only when the caller says that nothing is found in the cache again, because
// the forward of a loop over one set of tensors does find it there).
// COLS: column tiles a workgroup covers side by side (compile-time, so that the common
// one-column kernels keep their compile-time LDS addresses and scalar register count).
// MAXW: the most waves a workgroup may have (max_waves of the planner): what the registers are allotted for.
template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool GATED, int ALT, int COLS, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void scan_kernel(const ScanArgs p, const StateArgs<STATE> st) {
  constexpr int kLaneSlots = 64 * VEC;  // channels per tile

  extern __shared__ float lds[];
  __shared__ uint32_t s_ready[2 * 16];  // per column tile and wave: see announce_map

  // The waves of a workgroup: wg_cols column tiles side by side, each with n_waves waves
  // that take consecutive time slices.  Everything the chain phase touches is per column tile.
  TileCtx c;
  c.lane = threadIdx.x & 63;
  // (wave-uniform values, pinned to scalar registers: the row addresses derive from them)
  const int wave_in_group = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int waves_total = __builtin_amdgcn_readfirstlane(blockDim.x >> 6);
  c.n_waves = waves_total / COLS;
  // (adjacent waves side by side: they issue the two halves of a 512-byte row segment together)
  c.wcol = COLS > 1 ? (wave_in_group & 1) : 0;
  c.wave = COLS > 1 ? (wave_in_group >> 1) : wave_in_group;
  c.look = p.look_waves;
  // LDS: two sets of per-wave maps (tiles alternate between them, so a wave that runs
  // ahead into the next tile cannot overwrite a map a slower wave still reads), then
  // the slots the look-back waves fill
  float2 *const lds_maps = reinterpret_cast<float2 *>(lds);
  c.lds_pred = lds_maps + (2 * waves_total + c.wcol * c.look) * kLaneSlots;
  c.seq = p.seq;
  c.row_bytes = p.d * E::kBytes;
  c.s_ready = s_ready + c.wcol * 16;
  if (threadIdx.x < 2 * 16) s_ready[threadIdx.x] = 0u;
  __syncthreads();
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
  c.tag = c.chained ? __builtin_amdgcn_readfirstlane(ld_u32(p.hdr + HDR_EPOCH)) + 1u : 0u;

  // The grid is sized to be resident all at once; each workgroup walks tiles
  // blockIdx, blockIdx + gridDim, ...  Tiles are numbered chunk-major, so a tile
  // only ever waits for tiles with smaller numbers: those belong to a resident
  // workgroup that reaches them no later than this one reaches its own.
  // (which column group a slot of a chunk stands for: tile_order; bs 8 seq 4096 d 1024 bf16, forward +
  // backward, against slot s = group s: 96.3 -> 94.3 us on one set of tensors, 117.7 -> 111.0 us
  // over eight sets in rotation)
  const TileOrder order = tile_order(static_cast<uint32_t>(p.n_groups), gridDim.x);
  const uint32_t n_groups = order.n_groups;
  uint32_t parity = 0;
  uint32_t tile_no = 0;
  for (uint32_t tile = blockIdx.x; tile < static_cast<uint32_t>(p.n_tiles); tile += gridDim.x, parity ^= 1u) {
    c.tile_no = ++tile_no;
    c.lds_map = lds_maps + (parity * waves_total + c.wcol * c.n_waves) * kLaneSlots;
    // unsigned, wave-uniform arithmetic: stays on the scalar unit
    // (the compiler divides through a vector-unit reciprocal: pin the quotients back)
    const uint32_t chunk = __builtin_amdgcn_readfirstlane(tile / n_groups);
    const uint32_t group = tile_group(order, tile - chunk * n_groups, chunk);
    const uint32_t ctile = group * COLS + static_cast<uint32_t>(c.wcol);
    const uint32_t batch = __builtin_amdgcn_readfirstlane(ctile / static_cast<uint32_t>(p.tiles_per_row));
    const uint32_t coltile = ctile - batch * static_cast<uint32_t>(p.tiles_per_row);
    c.chunk = static_cast<int>(chunk);
    c.ctile = static_cast<int>(ctile);
    c.last = c.chunk == p.n_chunks - 1;
    c.anchor = __builtin_amdgcn_readfirstlane(chain_anchor(c.chunk, p.period, p.look_waves * kMaxSpan));
    c.span = __builtin_amdgcn_readfirstlane(chunk_span(c.chunk - c.anchor, p.look_waves));

    const int64_t col0 = static_cast<int64_t>(coltile) * kLaneSlots;  // first channel of the tile
    c.col_ok = col0 + c.lane * VEC < p.d;
    c.lane_off = static_cast<uint32_t>(c.lane * Row<E, VEC>::kBytes);
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
        gated_tile<E, VEC, STEPS, BWD, STATE, true>(p, st, c);
      else
        gated_tile<E, VEC, STEPS, BWD, STATE, false>(p, st, c);
    } else {
      if (full)
        scan_tile<E, VEC, STEPS, BWD, STATE, true, ALT>(p, st, c);
      else
        scan_tile<E, VEC, STEPS, BWD, STATE, false, ALT>(p, st, c);
    }
  }

#ifdef FSS_RESIDENCY_PROBE
  if (threadIdx.x == 0 && p.hdr) __hip_atomic_fetch_sub(p.hdr + 8, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
  count_out(p, c);
}

// ---- launching ---------------------------------------------------------------------

template <typename E, int VEC, int STEPS, bool BWD, bool STATE, bool GATED = false, int ALT = 0, int COLS = 1>
int launch_one(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, hipStream_t stream) {
  // The kernel's waits are only safe if every workgroup of the grid is resident,
  // so the grid never exceeds what the device holds at once; workgroups loop.
  static int resident[17] = {0};  // workgroups per CU by waves per workgroup
  const int waves = pl.cfg.waves;
  const size_t lds = lds_bytes(waves, VEC, pl.cfg.cols);
  constexpr int kMaxW = max_waves(E::kBytes, VEC, STEPS, BWD, GATED);
  if (waves > kMaxW) return FSS_ERR_BAD_CONFIG;
  const int fit = resident_workgroups(scan_kernel<E, VEC, STEPS, BWD, STATE, GATED, ALT, COLS, kMaxW>, waves, lds, resident);
  if (fit <= 0) return FSS_ERR_LAUNCH;
  int64_t n_groups = pl.n_tiles < fit ? pl.n_tiles : fit;
  if (pl.cfg.max_groups > 0 && pl.cfg.max_groups < n_groups) n_groups = pl.cfg.max_groups;
  const dim3 grid(static_cast<uint32_t>(n_groups));
  const dim3 block(static_cast<uint32_t>(waves) * 64);
  StateArgs<STATE> st;
  if constexpr (STATE) st = state;
  hipLaunchKernelGGL((scan_kernel<E, VEC, STEPS, BWD, STATE, GATED, ALT, COLS, kMaxW>), grid, block, lds, stream, args, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    tls_hip_error = static_cast<int>(e);
    return FSS_ERR_LAUNCH;
  }
  return FSS_OK;
}

// Two column tiles per workgroup exist for the plain scan's 4-byte-per-lane kernels (the ones
// large shapes run), with 16 steps per lane in both directions and with 32 in the forward; the
// forward also with states (the library takes two columns by itself there, and the scan with
// states must cut the sequence where the plain scan does).
template <typename E, bool BWD, bool STATE>
int launch_two_columns(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, hipStream_t stream) {
  constexpr int V = E::kBytes == 2 ? 2 : 1;
  if (pl.cfg.vec != V) return FSS_ERR_BAD_CONFIG;
  if constexpr (STATE) {
    if constexpr (!BWD) {
      if (pl.cfg.steps == 32) {
        if (pl.alt_policy == 2) return launch_one<E, V, 32, BWD, true, false, 2, 2>(args, state, pl, stream);
        if (pl.alt_policy == 1) return launch_one<E, V, 32, BWD, true, false, 1, 2>(args, state, pl, stream);
        return launch_one<E, V, 32, BWD, true, false, 0, 2>(args, state, pl, stream);
      }
    }
    return FSS_ERR_BAD_CONFIG;
  } else {
  switch (pl.cfg.steps) {
#define FSS_CASE2(S)                                                                                   \
  case S:                                                                                              \
    if constexpr (!BWD && S == 32) {                                                                   \
      if (pl.alt_policy == 2) return launch_one<E, V, S, BWD, false, false, 2, 2>(args, state, pl, stream); \
    }                                                                                                  \
    if (pl.alt_policy == 1 || (BWD && pl.alt_policy == 2))                                             \
      return launch_one<E, V, S, BWD, false, false, 1, 2>(args, state, pl, stream);                    \
    return launch_one<E, V, S, BWD, false, false, 0, 2>(args, state, pl, stream);
    FSS_CASE2(16)
    default:
      break;
  }
  if constexpr (!BWD) {
    switch (pl.cfg.steps) {
      FSS_CASE2(32)
      default:
        break;
    }
  }
#undef FSS_CASE2
  return FSS_ERR_BAD_CONFIG;
  }
}

template <typename E, bool BWD, bool STATE>
int launch_typed(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, hipStream_t stream) {
  constexpr bool is_16bit = E::kBytes == 2;
  if (pl.cfg.cols == 2) return launch_two_columns<E, BWD, STATE>(args, state, pl, stream);
  const int key = pl.cfg.vec * 100 + pl.cfg.steps;
  switch (key) {
#define FSS_CASE(V, S)                                                                            \
  case V * 100 + S:                                                                               \
    /* the scans with states carry the policy in the kernels large shapes run, the plain scan in all */ \
    if constexpr ((!BWD && S == 32) || (BWD && S == 16 && V * E::kBytes == 4)) {                  \
      if (pl.alt_policy == 2) return launch_one<E, V, S, BWD, STATE, false, 2>(args, state, pl, stream); \
      if (pl.alt_policy == 1) return launch_one<E, V, S, BWD, STATE, false, 1>(args, state, pl, stream); \
    } else if constexpr (!STATE) {                                                                \
      if (pl.alt_policy == 1 || (BWD && pl.alt_policy == 2))                                      \
        return launch_one<E, V, S, BWD, STATE, false, 1>(args, state, pl, stream);                \
    }                                                                                             \
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
template <typename E, bool BWD, bool STATE>
int launch_gated(const ScanArgs &args, const StateArgs<true> &none, const Plan &pl, hipStream_t stream) {
  constexpr bool is_16bit = E::kBytes == 2;
  if (pl.cfg.cols != 1) return FSS_ERR_BAD_CONFIG;
  const int key = pl.cfg.vec * 100 + pl.cfg.steps;
  switch (key) {
#define FSS_CASE(V, S) \
  case V * 100 + S:    \
    return launch_one<E, V, S, BWD, STATE, true>(args, none, pl, stream);
    FSS_CASE(1, 8)
    FSS_CASE(1, 16)
    default:
      break;
  }
  if constexpr (!BWD) {
    if (key == 132) return launch_one<E, 1, 32, BWD, STATE, true>(args, none, pl, stream);
  }
  if constexpr (is_16bit) {
    switch (key) {
      FSS_CASE(2, 8)
      FSS_CASE(2, 16)
      default:
        break;
    }
    if constexpr (!BWD) {
      if (key == 232) return launch_one<E, 2, 32, BWD, STATE, true>(args, none, pl, stream);
    }
  }
#undef FSS_CASE
  return FSS_ERR_BAD_CONFIG;
}

int FSS_RM_LAUNCH(const ScanArgs &args, const StateArgs<true> &state, const Plan &pl, bool gated, bool with_state,
                  hipStream_t stream) {
  using E = FSS_RM_ELEM;
  constexpr bool kBwd = FSS_RM_BWD != 0;
  if (gated)
    return with_state ? launch_gated<E, kBwd, true>(args, state, pl, stream)
                      : launch_gated<E, kBwd, false>(args, state, pl, stream);
  return with_state ? launch_typed<E, kBwd, true>(args, state, pl, stream)
                    : launch_typed<E, kBwd, false>(args, state, pl, stream);
}

}  // namespace fss
