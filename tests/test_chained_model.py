"""CPU checks of the fixed composition order of chained scans.

Two things are pinned here without a GPU:

* the host side of the order (`fss_debug_chain_plan`, `fss_debug_chain_anchor`): which earlier
  chunk's state a chunk starts from and which maps it composes depends on the chunk's index and
  the plan alone, covers every chunk in between exactly once, and never asks for more than one
  period of maps nor for more than one round of the look-back reaches;
* `oracle/chained_model.c`, the sequential C restatement of the kernels' composition order that
  the GPU tests demand bit-for-bit agreement with: one slice equals the fused sequential oracle
  exactly, exact-arithmetic inputs equal it exactly under every tiling (which pins the model's
  indexing: a wrong chunk, anchor or prefix changes integers), and random inputs stay within
  fp32 rounding of the sequential fp64 oracle.

The reference walks every channel with one thread in order
(csrc/include/sequential_scan_kernel_bf16.cuh:121-151), so its results are the same bits from
run to run; this is how the chunked scan keeps that property.
"""
import ctypes

import numpy as np
import pytest

import oracle
from fast_sequential_scan_amd import _native

TILINGS = [
    # steps, waves, period, look, most chunks per look-back wave
    (8, 1, 1, 1, 1),
    (8, 2, 1, 2, 1),
    (8, 2, 3, 2, 1),
    (8, 2, 5, 2, 2),
    (16, 4, 4, 4, 1),
    (32, 16, 4, 16, 1),
    (16, 16, 128, 16, 4),
    (8, 8, 1000, 8, 4),
    (8, 3, 7, 2, 3),
]


def chain_plan(bs, seq, d, dtype, direction, cfg=None, align=16):
    out = (ctypes.c_int32 * 8)()
    rc = _native.lib().fss_debug_chain_plan(bs, seq, d, dtype, direction, align, _native.make_config(cfg), out)
    assert rc == 0, rc
    keys = ("n_chunks", "waves", "steps", "period", "look", "max_span", "vec", "cols")
    return dict(zip(keys, list(out)))


def fold_items(chunk, period, look, max_span):
    """The order in which the kernels fold earlier chunks into the state entering `chunk`:
    a list of groups (one per look-back wave), each a list of chunk indices, nearest first; the
    very last index is the anchor, whose outgoing state is taken."""
    anchor = _native.lib().fss_debug_chain_anchor(chunk, period, look * max_span)
    items = chunk - anchor
    span = min(max_span, max(1, -(-items // look)))
    groups = []
    nearest = chunk - 1
    while nearest >= anchor:
        for w in range(look):
            j = nearest - w * span
            if j < anchor:
                break
            groups.append([j - k for k in range(span) if j - k >= anchor])
        nearest -= look * span
    return anchor, groups


def test_anchor_is_a_function_of_chunk_and_plan_only():
    lib = _native.lib()
    for period in (1, 2, 3, 4, 7, 64, 128, 1000):
        for stride in (1, 4, 8, 64, 52, 1 << 20):
            for chunk in range(1, 600):
                a = lib.fss_debug_chain_anchor(chunk, period, stride)
                assert 0 <= a < chunk
                # the last chunk of the round before (chunk 0 within the first round), or the last
                # multiple of the stride below the chunk if that is nearer
                first = chunk - chunk % period
                by_round = first - 1 if first > 0 else 0
                by_stride = (chunk - 1) // stride * stride
                assert a == max(by_round, by_stride)
                assert chunk - a <= min(period, stride)  # never more than that many chunks to fold
                # an anchor's own chain ends at chunk 0 after finitely many hops
                hops, k = 0, a
                while k > 0:
                    k = lib.fss_debug_chain_anchor(k, period, stride)
                    hops += 1
                assert hops <= chunk
    assert lib.fss_debug_chain_anchor(-1, 4, 64) == -1
    assert lib.fss_debug_chain_anchor(3, 0, 64) == -1
    assert lib.fss_debug_chain_anchor(3, 4, 0) == -1


@pytest.mark.parametrize("period,look,max_span", [(1, 1, 1), (4, 16, 4), (4, 2, 1), (128, 16, 4), (7, 2, 3), (300, 16, 4), (300, 5, 4)])
def test_fold_covers_every_chunk_between_once_nearest_first(period, look, max_span):
    for chunk in range(1, 700):
        anchor, groups = fold_items(chunk, period, look, max_span)
        flat = [j for g in groups for j in g]
        assert flat == list(range(chunk - 1, anchor - 1, -1))
        assert all(1 <= len(g) <= max_span for g in groups)
        assert len(groups) <= look  # one round of the look-back always reaches the anchor


def test_chain_plan_of_the_measured_workloads():
    # (shape, dtype, dir) -> chunk length and period: the planned grid holds 256 workgroups of 16 waves
    # (the forward at this shape is a two-round launch: two column tiles per workgroup, so 8 of its
    # 16 waves lie along time and a chunk is 256 steps)
    p = chain_plan(8, 4096, 1024, _native.FSS_BF16, _native.FSS_FWD)
    assert (p["steps"], p["waves"], p["vec"], p["cols"]) == (32, 8, 2, 2)
    assert p["n_chunks"] == 16 and p["period"] == 8 and p["max_span"] == 4
    p = chain_plan(8, 8192, 1024, _native.FSS_BF16, _native.FSS_FWD)
    assert (p["steps"], p["waves"], p["vec"], p["cols"]) == (32, 16, 2, 1)
    assert p["n_chunks"] == 16 and p["period"] == 4 and p["look"] == 16
    p = chain_plan(8, 4096, 1024, _native.FSS_BF16, _native.FSS_BWD)
    assert (p["steps"], p["waves"]) == (16, 16) and p["n_chunks"] == 16 and p["period"] == 4
    p = chain_plan(1, 65521, 256, _native.FSS_BF16, _native.FSS_FWD)
    # two column tiles of 128 channels, 128 chunks of 512 steps: every chunk is in flight at once
    # (so every 64th chunk is an anchor as well: 16 look-back waves x 4 chunks)
    assert (p["n_chunks"], p["steps"] * p["waves"], p["period"], p["look"], p["max_span"]) == (128, 512, 128, 16, 4)
    assert _native.lib().fss_debug_chain_anchor(127, 128, 64) == 64 and _native.lib().fss_debug_chain_anchor(64, 128, 64) == 0
    # an explicit configuration and a grid cap: the cap does not enter the plan
    a = chain_plan(2, 4099, 256, _native.FSS_BF16, _native.FSS_FWD, cfg=(1, 8, 2))
    b = chain_plan(2, 4099, 256, _native.FSS_BF16, _native.FSS_FWD, cfg=(1, 8, 2, 3))
    assert a == b and a["n_chunks"] == -(-4099 // 16)


def _exact_inputs(rng, bs, seq, d):
    alpha = rng.choice(np.array([0.0, 1.0, -1.0, 1.0, 1.0], dtype=np.float32), size=(bs, seq, d))
    beta = rng.integers(-3, 4, size=(bs, seq, d)).astype(np.float32)
    return alpha, beta


@pytest.mark.parametrize("tiling", TILINGS)
def test_model_equals_sequential_oracle_on_exact_arithmetic(tiling):
    rng = np.random.default_rng(7)
    for seq in (1, 2, 9, 64, 257, 1031):
        alpha, beta = _exact_inputs(rng, 2, seq, 5)
        want = oracle.scan_fwd_f32(alpha, beta)
        got = oracle.chained_scan_fwd(alpha, beta, *tiling)
        assert np.array_equal(got, want), (seq, tiling)
        dout = rng.integers(-2, 3, size=alpha.shape).astype(np.float32)
        # (keep the stored h small enough for g*h to stay exact)
        h = rng.integers(-4, 5, size=alpha.shape).astype(np.float32)
        ga_want, gb_want = oracle.scan_bwd_f32(alpha, h, dout)
        ga, gb = oracle.chained_scan_bwd(alpha, h, dout, *tiling)
        assert np.array_equal(gb, gb_want), (seq, tiling)
        assert np.array_equal(ga, ga_want), (seq, tiling)


def test_model_with_one_slice_is_the_fused_sequential_oracle():
    rng = np.random.default_rng(11)
    bs, seq, d = 2, 200, 9
    alpha = rng.uniform(-1.1, 1.1, size=(bs, seq, d)).astype(np.float32)
    beta = rng.standard_normal((bs, seq, d)).astype(np.float32)
    dout = rng.standard_normal((bs, seq, d)).astype(np.float32)
    h = oracle.scan_fwd_f32(alpha, beta, fused=True)
    assert np.array_equal(oracle.chained_scan_fwd(alpha, beta, 256, 1, 1, 1, 1), h)
    ga_want, gb_want = oracle.scan_bwd_f32(alpha, h, dout, fused=True)
    ga, gb = oracle.chained_scan_bwd(alpha, h, dout, 256, 1, 1, 1, 1)
    assert np.array_equal(gb, gb_want) and np.array_equal(ga, ga_want)
    # bf16 storage: same carries, outputs rounded to nearest even
    ab, bb = oracle.f32_to_bf16_bits(alpha), oracle.f32_to_bf16_bits(beta)
    assert np.array_equal(oracle.chained_scan_fwd(ab, bb, 256, 1, 1, 1, 1), oracle.scan_fwd_bf16(ab, bb, fused=True))


@pytest.mark.parametrize("tiling", TILINGS)
@pytest.mark.parametrize("recipe", ["sigmoid", "near_one", "constant_0.999"])
def test_model_within_fp32_rounding_of_sequential(tiling, recipe):
    rng = np.random.default_rng(3)
    bs, seq, d = 1, 3001, 6
    z = rng.standard_normal((bs, seq, d))
    if recipe == "sigmoid":
        alpha = 1.0 / (1.0 + np.exp(-z))
    elif recipe == "near_one":
        alpha = 1.0 / (1.0 + np.exp(-(z + 6.0)))
    else:
        alpha = np.full_like(z, 0.999)
    alpha = alpha.astype(np.float32)
    beta = rng.standard_normal((bs, seq, d)).astype(np.float32)
    want = oracle.scan_fwd_f64(alpha.astype(np.float64), beta.astype(np.float64))
    got = oracle.chained_scan_fwd(alpha, beta, *tiling)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-5 * scale
    # the long-memory recipes really exercise the composed carries: a chunk's coefficient is not 0
    if recipe != "sigmoid" and tiling[0] * tiling[1] <= 512:
        assert np.prod(alpha[0, 1 : 1 + tiling[0] * tiling[1], 0].astype(np.float64)) > 1e-3
