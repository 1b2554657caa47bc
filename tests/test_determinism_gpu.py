"""GPU tests that a chained scan is a function of its inputs and its launch configuration alone.

The reference walks every channel with one thread in order
(csrc/include/sequential_scan_kernel_bf16.cuh:121-151, sequential_scan_cpu.hpp:18-33): the same
inputs give the same bits on every run.  Here chunks of a sequence run concurrently and hand
each other affine maps, whose composition is associative only up to fp32 rounding - so the order
of composition is fixed by the chunk index and the plan (tests/test_chained_model.py), and these
tests hold the device to it in the regime where it matters: alphas so close to 1 that the
product over a chunk is far from 0 (with the sigmoid(N(0,1)) alphas of the measured workloads
that product underflows and every order of composition gives the same bits trivially).

  * bit for bit against oracle/chained_model.c, the sequential C program that composes in that
    fixed order: if the device's bits are those of a sequential program, they cannot depend on
    the timing of its workgroups;
  * the same bits over back-to-back launches, on a second stream, under both cache policies,
    through the entry point that allocates nothing, and with the grid capped;
  * and all of it within the grading tolerance of the sequential fp32 oracle.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import fast_sequential_scan_amd as pkg  # noqa: E402
from fast_sequential_scan_amd import _native  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402
from fast_sequential_scan_amd.workloads import make_inputs  # noqa: E402

DEV = "cuda:0"
CODE = {torch.bfloat16: _native.FSS_BF16, torch.float32: _native.FSS_F32}


def chain_plan(shape, dtype, direction, cfg=None):
    out = (ctypes.c_int32 * 8)()
    rc = _native.lib().fss_debug_chain_plan(*shape, CODE[dtype], direction, 16, _native.make_config(cfg), out)
    assert rc == 0, rc
    n_chunks, waves, steps, period, look, max_span, _vec, _cols = list(out)
    return dict(n_chunks=n_chunks, steps=steps, waves=waves, period=period, look=look, span=max_span)


def long_memory_inputs(recipe, shape, dtype, seed):
    """near_one: alpha = sigmoid(N(0,1)+6); constant: alpha = the storage type's value next below
    0.9995 (bf16: 0.99609375, fp32: 0.999)."""
    if recipe == "near_one":
        return make_inputs("near_one", *shape, dtype=dtype, seed=seed)
    _alpha, beta, dout = make_inputs("sigmoid", *shape, dtype=dtype, seed=seed)
    value = 0.99609375 if dtype == torch.bfloat16 else 0.999
    return torch.full(shape, value, dtype=dtype), (beta.float() * 0.05).to(dtype), dout


def as_model_array(t):
    if t.dtype == torch.bfloat16:
        return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
    return t.detach().cpu().contiguous().numpy()


def for_backward(cfg):
    if cfg is not None and cfg[0] == 2 and cfg[1] == 32 and cfg[2] > 8:
        return (cfg[0], cfg[1], 8) + tuple(cfg[3:])
    return cfg


CASES = [
    # dtype, shape, explicit configuration (vec, steps, waves[, max_groups])
    (torch.bfloat16, (8, 4096, 1024), None),
    (torch.float32, (8, 4096, 1024), None),
    (torch.bfloat16, (2, 4099, 256), (1, 8, 2)),
    (torch.bfloat16, (2, 4099, 256), (1, 8, 2, 3)),   # three workgroups walk all 2056 tiles
    (torch.float32, (2, 4099, 256), (1, 8, 2, 5)),
    (torch.bfloat16, (1, 65521, 256), None),          # every chunk of the sequence in flight at once
    (torch.bfloat16, (4, 8192, 2048), None),
    (torch.bfloat16, (3, 3000, 384), (2, 16, 4)),
    (torch.float32, (2, 2500, 192), (1, 16, 8)),
]


@pytest.mark.parametrize("recipe", ["near_one", "constant"])
@pytest.mark.parametrize("dtype,shape,cfg", CASES, ids=lambda v: str(v).replace("torch.", ""))
def test_device_bits_are_those_of_the_sequential_model(oracle, dtype, shape, cfg, recipe):
    if recipe == "constant" and shape[0] * shape[1] * shape[2] > (1 << 25):
        pytest.skip("covered by near_one at this size")
    alpha, beta, dout = long_memory_inputs(recipe, shape, dtype, seed=sum(shape))
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(dtype, a, b, cfg)
    ga, gb = ext._backward(dtype, a, h, do, for_backward(cfg))
    ext.workspace_status()

    fwd = chain_plan(shape, dtype, _native.FSS_FWD, cfg)
    bwd = chain_plan(shape, dtype, _native.FSS_BWD, for_backward(cfg))
    assert fwd["n_chunks"] > 1 and bwd["n_chunks"] > 1
    a_m, b_m, do_m = as_model_array(alpha), as_model_array(beta), as_model_array(dout)
    order = ("steps", "waves", "period", "look", "span")
    h_model = oracle.chained_scan_fwd(a_m, b_m, *(fwd[k] for k in order))
    np.testing.assert_array_equal(as_model_array(h), h_model, err_msg="h")
    ga_model, gb_model = oracle.chained_scan_bwd(a_m, as_model_array(h), do_m, *(bwd[k] for k in order))
    np.testing.assert_array_equal(as_model_array(gb), gb_model, err_msg="grad_beta")
    np.testing.assert_array_equal(as_model_array(ga), ga_model, err_msg="grad_alpha")

    # the carries really are composed: over one chunk the alphas' product is far from 0
    chunk = fwd["steps"] * fwd["waves"]
    product = np.prod(alpha[0, 1:1 + chunk, 0].double().numpy())
    assert product > 1e-4, product

    # and the model (hence the device) is within the grading tolerance of the sequential oracle
    if dtype == torch.bfloat16:
        h32 = oracle.scan_fwd_bf16_f32out(a_m, b_m)
        ga32, gb32 = oracle.scan_bwd_bf16_f32out(a_m, h32, do_m)
        tol = dict(rtol=1e-2, atol=1e-2)
    else:
        h32 = oracle.scan_fwd_f32(a_m, b_m)
        ga32, gb32 = oracle.scan_bwd_f32(a_m, h32, do_m)
        tol = dict(rtol=1e-4, atol=1e-4)
    for name, got, want in (("h", h, h32), ("grad_beta", gb, gb32), ("grad_alpha", ga, ga32)):
        got = got.float().cpu().numpy()
        # (outputs of size up to ~30: atol scaled to the result's own magnitude)
        scale = max(1.0, float(np.abs(want).max()) / 8.0)
        assert np.allclose(got, want, rtol=tol["rtol"], atol=tol["atol"] * scale), name


def _launch_fwd_bwd(dtype, a, b, do, cfg):
    h = ext._forward(dtype, a, b, cfg)
    ga, gb = ext._backward(dtype, a, h, do, for_backward(cfg))
    return h, ga, gb


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("shape,cfg", [((8, 4096, 1024), None), ((2, 4099, 256), (1, 8, 2))], ids=["headline", "small_tiles"])
@pytest.mark.parametrize("recipe", ["near_one", "constant"])
def test_same_bits_from_run_to_run(dtype, shape, cfg, recipe):
    """Ten launches back to back, a second stream, both cache policies, a capped grid and the entry
    point that allocates nothing: one set of bits."""
    alpha, beta, dout = long_memory_inputs(recipe, shape, dtype, seed=5 + sum(shape))
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    first = _launch_fwd_bwd(dtype, a, b, do, cfg)
    torch.cuda.synchronize()
    # (a device-side comparison per launch: the launches stay back to back)
    same = []
    for _ in range(10):
        again = _launch_fwd_bwd(dtype, a, b, do, cfg)
        same.append(torch.stack([(x == y).all() for x, y in zip(first, again)]))
    assert bool(torch.stack(same).all())
    for x in first:
        assert bool(torch.isfinite(x.float()).all())

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = _launch_fwd_bwd(dtype, a, b, do, cfg)
    side.synchronize()
    for x, y in zip(first, other):
        assert torch.equal(x, y)

    previous = pkg.set_cache_policy("streaming")
    try:
        # with an explicit configuration the policy cannot change the tiling; with the library's own
        # choice it may not either
        assert chain_plan(shape, dtype, _native.FSS_FWD, cfg) == _with_policy("auto", lambda: chain_plan(shape, dtype, _native.FSS_FWD, cfg))
        streamed = _launch_fwd_bwd(dtype, a, b, do, cfg)
    finally:
        pkg.set_cache_policy(previous)
    for x, y in zip(first, streamed):
        assert torch.equal(x, y)

    # a capped grid walks the same tiles in more rounds: the plan, and so the bits, do not change
    if cfg is not None:
        capped = _launch_fwd_bwd(dtype, a, b, do, tuple(cfg) + (7,))
        for x, y in zip(first, capped):
            assert torch.equal(x, y)

    lib = _native.lib()
    if cfg is None:
        out = torch.empty_like(a)
        for _ in range(2):
            _native.check(lib.fss_scan_fwd_noalloc(CODE[dtype], a.data_ptr(), b.data_ptr(), out.data_ptr(), *shape,
                                                   torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(out, first[0])
    ext.workspace_status()


def _with_policy(policy, fn):
    previous = pkg.set_cache_policy(policy)
    try:
        return fn()
    finally:
        pkg.set_cache_policy(previous)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("cfg", [(1, 8, 2), (2, 16, 4), None], ids=str)
def test_infinite_alpha_poisons_exactly_what_it_poisons_sequentially(oracle, dtype, cfg):
    """alpha = +inf meeting a state of exactly 0 gives NaN, meeting anything else +-inf, and every
    later state of that channel is NaN or +-inf - in the sequential loop
    (sequential_scan/common.py:46-59) and here alike: the same elements are non-finite, nothing else
    is touched, whether the inf sits inside a lane's slice of timesteps, on its first step or on the
    first step of a chunk.  WHICH non-finite value comes out can differ: where the sequential order
    keeps -inf, a composed map with an infinite coefficient can give inf - inf = NaN, so with a
    non-finite alpha only the finiteness of an output is independent of the tiling.  (The
    composition keeps a zero state at 0 when a PRODUCT of finite alphas overflowed, which the
    sequential order also does: tests/test_scan_gpu.py's growing-recurrence case.)"""
    bs, seq, d = 2, 600, 128
    alpha, beta, dout = make_inputs("sigmoid", bs, seq, d, dtype=dtype, seed=31)
    beta[:, :300, :64] = 0  # channels 0-63: the state is exactly 0 until step 300
    steps = 8 if cfg is None else cfg[1]
    for t in (16, 16 + 3, 128, 256 + steps, 299):  # chunk starts, slice starts and steps inside a slice, whatever the tiling
        alpha[0, t, 0:2] = float("inf")      # meets 0 -> NaN
        alpha[0, t, 64:66] = float("inf")    # meets a non-zero state -> +-inf
    a, b = alpha.to(DEV), beta.to(DEV)
    h = ext._forward(dtype, a, b, cfg)
    ext.workspace_status()
    if dtype == torch.bfloat16:
        want = oracle.bf16_bits_to_f32(oracle.scan_fwd_bf16(as_model_array(alpha), as_model_array(beta), fused=True))
    else:
        want = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy(), fused=True)
    got = h.float().cpu().numpy()
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    assert np.isnan(got[0, 16:, 0]).all() and np.isfinite(got[0, :16, 0]).all()   # inf * 0: NaN in both
    assert np.isinf(got[0, 16, 64]) and not np.isfinite(got[0, 16:, 64]).any()
    finite = np.isfinite(want)
    assert finite[1].all() and finite[0, :, 2:64].all() and finite[0, :, 66:].all()
    tol = 1e-2 if dtype == torch.bfloat16 else 1e-4
    assert np.allclose(got[finite], want[finite], rtol=tol, atol=tol)


def _random_tilings(n, seed):
    """(dtype, shape, forward configuration, backward configuration) drawn at random from what the
    row-major kernels are compiled for, with short chunks so that sequences chain many of them."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
        vec = int(rng.choice([1, 2, 4, 8] if dtype == torch.bfloat16 else [1, 2, 4]))
        steps = int(rng.choice([8, 16, 32]))
        budget = 64 if dtype == torch.bfloat16 else 32
        if vec * steps > budget:
            continue
        max_waves = 4 if vec >= 8 else 8 if vec >= 4 else 16
        waves = int(rng.integers(1, max_waves + 1))
        cols = 1
        if vec * (2 if dtype == torch.bfloat16 else 4) == 4 and steps in (16, 32) and waves % 2 == 0 and rng.random() < 0.4:
            cols = 2
        bs = int(rng.integers(1, 4))
        d = 64 * vec * cols * int(rng.integers(1, 4))
        seq = int(rng.integers(steps * max(waves // cols, 1) + 1, 40 * steps * max(waves // cols, 1)))
        seq = min(seq, 6000)
        groups = int(rng.choice([0, 0, 1, 2, 5, 16]))
        fwd = (vec, steps, waves, groups, cols)
        # the backward has no 32-step kernels beyond 8 waves at two channels per lane, none with two
        # column tiles at 32 steps, and holds three tensors: stay within what it is compiled for
        b_steps = steps if vec * steps * 3 <= budget * 2 or vec < 2 else 16 if vec * 16 <= budget else 8
        if dtype == torch.float32 and vec * b_steps > 32:
            b_steps = 8
        b_cols = cols if b_steps == 16 else 1
        b_waves = waves if not (vec >= 2 and b_steps == 32 and waves > 8) else 8
        if b_cols == 2 and b_waves % 2:
            b_cols = 1
        bwd = (vec, b_steps, b_waves, groups, b_cols)
        out.append((dtype, (bs, seq, d), fwd, bwd))
    return out


TWO_COLUMN_TILINGS = [
    (torch.bfloat16, (2, 3000, 512), (2, 32, 8, 0, 2), (2, 16, 8, 0, 2)),
    (torch.bfloat16, (1, 5000, 256), (2, 16, 6, 3, 2), (2, 16, 6, 3, 2)),
    (torch.bfloat16, (3, 2222, 1024), (2, 32, 16, 0, 2), (2, 16, 16, 7, 2)),
    (torch.float32, (2, 2000, 256), (1, 32, 4, 0, 2), (1, 16, 4, 0, 2)),
]


@pytest.mark.parametrize("dtype,shape,fwd_cfg,bwd_cfg", _random_tilings(36, seed=20) + TWO_COLUMN_TILINGS,
                         ids=lambda v: str(v).replace("torch.", "").replace(" ", ""))
def test_random_tilings_return_the_models_bits(oracle, dtype, shape, fwd_cfg, bwd_cfg):
    """Any tiling the kernels are compiled for, capped grids and two column tiles included: the device
    returns the bits of the sequential model of that tiling (alphas near 1)."""
    lib = _native.lib()
    plan = (ctypes.c_int32 * 8)()
    for direction, cfg in ((_native.FSS_FWD, fwd_cfg), (_native.FSS_BWD, bwd_cfg)):
        if lib.fss_debug_chain_plan(*shape, CODE[dtype], direction, 16, _native.make_config(cfg), plan) != 0:
            pytest.skip(f"configuration {cfg} is not one the library has a kernel for")
    alpha, beta, dout = long_memory_inputs("near_one", shape, dtype, seed=sum(shape) + fwd_cfg[1])
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(dtype, a, b, fwd_cfg)
    ga, gb = ext._backward(dtype, a, h, do, bwd_cfg)
    ext.workspace_status()
    order = ("steps", "waves", "period", "look", "span")
    fwd = chain_plan(shape, dtype, _native.FSS_FWD, fwd_cfg)
    bwd = chain_plan(shape, dtype, _native.FSS_BWD, bwd_cfg)
    a_m, b_m, do_m = as_model_array(alpha), as_model_array(beta), as_model_array(dout)
    np.testing.assert_array_equal(as_model_array(h), oracle.chained_scan_fwd(a_m, b_m, *(fwd[k] for k in order)))
    ga_model, gb_model = oracle.chained_scan_bwd(a_m, as_model_array(h), do_m, *(bwd[k] for k in order))
    np.testing.assert_array_equal(as_model_array(gb), gb_model)
    np.testing.assert_array_equal(as_model_array(ga), ga_model)


def test_the_other_kernel_families_return_the_same_bits_from_run_to_run():
    """The gated scan, the scans with states and the channel-major scan chain their chunks through the
    same phase: eight launches of each, long-memory inputs, one set of bits (outputs finite)."""
    shape = (4, 6000, 256)
    alpha, beta, dout = make_inputs("near_one", *shape, seed=77)
    g = torch.Generator().manual_seed(78)
    gate = (torch.randn(shape, generator=g) + 6.0).to(torch.bfloat16).to(DEV)
    h0 = torch.randn(shape[0], shape[2], generator=g).to(DEV)
    g_last = torch.randn(shape[0], shape[2], generator=g).to(DEV)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    # channel-major: (bs, d, seq) with a sequence long enough to be chained through memory
    a_cm, b_cm, do_cm = (t[:2, :, :64].transpose(1, 2).contiguous().repeat(1, 1, 3) for t in (a, b, do))

    def gated():
        h = ext.gated_scan_forward(gate, b)
        return (h, *ext.gated_scan_backward(gate, b, h, do))

    def with_states():
        h, h_last = ext.scan_forward_state(a, b, h0)
        return (h, h_last, *ext.scan_backward_state(a, h, do, h0, g_last))

    def gated_with_states():
        h, h_last = ext.gated_scan_forward_state(gate, b, h0)
        return (h, h_last, *ext.gated_scan_backward_state(gate, b, h, do, h0, g_last))

    def channel_major():
        h = ext.scan_forward_cm(a_cm, b_cm)
        return (h, *ext.scan_backward_cm(a_cm, h, do_cm))

    assert a_cm.shape == (2, 64, 18000)
    for run in (gated, with_states, gated_with_states, channel_major):
        first = run()
        torch.cuda.synchronize()
        same = []
        for _ in range(8):
            same.append(torch.stack([(x == y).all() for x, y in zip(first, run())]))
        assert bool(torch.stack(same).all()), run.__name__
        for x in first:
            assert bool(torch.isfinite(x.float()).all()), run.__name__
    ext.workspace_status()
