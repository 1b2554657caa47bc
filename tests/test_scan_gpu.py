"""GPU parity tests: the HIP kernels, called through the C ABI, against the CPU oracle.

Bars
  * grading bar: every output within rtol = atol = 1e-2 of the fp32-accumulated
    sequential scan fed the same seeded bf16 inputs (oracle.*_f32out);
  * tight bar: bf16 outputs within 2 bf16 ulps of the oracle that rounds exactly
    where the kernel does (fp32 carry, fused multiply-add, round-to-nearest-even
    on store, backward fed the same stored h) - bit-exact when one wave scans
    the whole sequence, because then the operation order is identical;
  * fp32: relative L2 error < 1e-6, the reference's SINGLE_TOL
    (sequential_scan/common.py:6,14-17).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import _native, scan_cu, scan_cu_single  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402
from fast_sequential_scan_amd.workloads import BASELINE_CASES, make_inputs  # noqa: E402

DEV = "cuda:0"
RTOL = ATOL = 1e-2


def bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def ulp_distance(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in representable bf16 values (sign-magnitude -> ordered integers)."""
    def ordered(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)
    return np.abs(ordered(a_bits) - ordered(b_bits))


def assert_close_f32(got: torch.Tensor, want: np.ndarray, what: str):
    got = got.detach().float().cpu().numpy()
    bad = ~(np.abs(got - want) <= ATOL + RTOL * np.abs(want))
    assert not bad.any(), (
        f"{what}: {bad.sum()} of {bad.size} elements outside rtol=atol=1e-2; "
        f"worst abs err {np.abs(got - want)[bad].max():.4g} at {np.argwhere(bad)[0]}"
    )


def rel_l2(x: np.ndarray, y: np.ndarray) -> float:
    return float(np.linalg.norm((x - y).ravel()) / max(np.linalg.norm(y.ravel()), 1e-30))


def for_backward(config):
    """The same tiling for the backward: its 32-step kernels with two channels per lane hold three
    tensors and are built for 8 waves at most."""
    if config is not None and config[0] == 2 and config[1] == 32 and config[2] > 8:
        return (config[0], config[1], 8) + tuple(config[3:])
    return config


def run_bf16(alpha, beta, dout, config=None):
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(torch.bfloat16, a, b, config)
    ga, gb = ext._backward(torch.bfloat16, a, h, do, for_backward(config))
    torch.cuda.synchronize()
    return h, ga, gb


def check_bf16(oracle, alpha, beta, dout, config=None, exact=False, max_ulp=2, what=""):
    h, ga, gb = run_bf16(alpha, beta, dout, config)
    a_bits, b_bits, d_bits = bits(alpha), bits(beta), bits(dout)
    # grading bar
    h32 = oracle.scan_fwd_bf16_f32out(a_bits, b_bits)
    ga32, gb32 = oracle.scan_bwd_bf16_f32out(a_bits, h32, d_bits)
    assert_close_f32(h, h32, f"{what} h")
    assert_close_f32(gb, gb32, f"{what} grad_beta")
    assert_close_f32(ga, ga32, f"{what} grad_alpha")
    # tight bar: same rounding points as the kernel
    h_or = oracle.scan_fwd_bf16(a_bits, b_bits, fused=True)
    ga_or, gb_or = oracle.scan_bwd_bf16(a_bits, bits(h), d_bits, fused=True)
    for name, got, want in (("h", bits(h), h_or), ("grad_beta", bits(gb), gb_or), ("grad_alpha", bits(ga), ga_or)):
        if exact:
            np.testing.assert_array_equal(got, want, err_msg=f"{what} {name}")
        else:
            finite = np.isfinite(oracle.bf16_bits_to_f32(want))
            dist = ulp_distance(got[finite], want[finite])
            # re-associated carries may move a value across a rounding boundary, or - where
            # the result nearly cancels - by a few ulps of a much smaller number
            close = np.abs(oracle.bf16_bits_to_f32(got[finite]) - oracle.bf16_bits_to_f32(want[finite])) <= 1e-3
            assert ((dist <= max_ulp) | close).all(), f"{what} {name}: max ulp distance {dist.max()}"
    return h, ga, gb


# ------------------------------------------------------------------ small shapes


@pytest.mark.parametrize("seq", [1, 2, 3, 7, 8])
@pytest.mark.parametrize("d", [1, 2, 6, 64, 100, 136, 520])
def test_bf16_one_wave_is_bit_exact(oracle, seq, d):
    """seq <= steps with one wave: no re-association anywhere -> identical bits."""
    alpha, beta, dout = make_inputs("normal", 3, seq, d, seed=seq * 1000 + d)
    vec = 8 if d % 8 == 0 else 4 if d % 4 == 0 else 2 if d % 2 == 0 else 1
    for v in {1, vec, min(vec, 2)}:
        check_bf16(oracle, alpha, beta, dout, config=(v, 8, 1), exact=True, what=f"v{v}")
    check_bf16(oracle, alpha, beta, dout, config=None, exact=True, what="default")


@pytest.mark.parametrize("seq", [9, 31, 64, 65, 257, 1000])
@pytest.mark.parametrize("d", [2, 24, 128, 192, 768])
@pytest.mark.parametrize("recipe", ["normal", "sigmoid"])
def test_bf16_default_config(oracle, recipe, seq, d):
    alpha, beta, dout = make_inputs(recipe, 2, seq, d, seed=seq + d)
    check_bf16(oracle, alpha, beta, dout, what=f"{recipe} {seq}x{d}")


CONFIGS = [
    (1, 8, 1), (1, 16, 3), (1, 32, 16),
    (2, 8, 2), (2, 16, 8), (2, 32, 4), (2, 32, 16),
    (4, 8, 5), (4, 16, 8), (4, 8, 7),
    (8, 8, 1), (8, 8, 3),
]


@pytest.mark.parametrize("config", CONFIGS, ids=lambda c: "v%d_s%d_w%d" % c)
def test_bf16_result_does_not_depend_on_chunking(oracle, config):
    """Same inputs through every tiling: many chunks, ragged tails, partial column tiles."""
    alpha, beta, dout = make_inputs("hawk", 2, 777, 328, seed=7)  # 328 = 8*41: partial tiles for every vec
    check_bf16(oracle, alpha, beta, dout, config=config, what=str(config))


# (forward config, backward config): two column tiles per workgroup exist for 4 bytes per lane with
# 16 steps (both directions) and 32 steps (forward)
TWO_COLUMN_CONFIGS = [
    ((2, 32, 16, 0, 2), (2, 16, 16, 0, 2)), ((2, 16, 8, 0, 2), (2, 16, 8, 0, 2)), ((2, 32, 4, 3, 2), (2, 16, 4, 3, 2)),
    ((2, 16, 2, 0, 2), (2, 16, 2, 0, 2)), ((2, 32, 2, 5, 2), (2, 16, 2, 5, 2)), ((2, 16, 6, 0, 2), (2, 16, 12, 0, 2)),
]


@pytest.mark.parametrize("fwd_cfg,bwd_cfg", TWO_COLUMN_CONFIGS, ids=lambda c: "v%d_s%d_w%d_g%d_c%d" % c)
def test_bf16_two_column_tiles_per_workgroup(oracle, fwd_cfg, bwd_cfg):
    """Workgroups that cover two adjacent column tiles (512 contiguous bytes per row) run two
    look-backs side by side behind shared barriers.  Short chains resolve in one round; with one
    wave per column tile the sequence is ~49 chunks, so the two look-backs take several rounds and
    must agree on when to leave.  Capped grids make workgroups walk many tiles."""
    alpha, beta, dout = make_inputs("hawk", 2, 777, 512, seed=19)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(torch.bfloat16, a, b, fwd_cfg)
    ga, gb = ext._backward(torch.bfloat16, a, h, do, bwd_cfg)
    ext.workspace_status()
    a_bits, b_bits, d_bits = bits(alpha), bits(beta), bits(dout)
    h32 = oracle.scan_fwd_bf16_f32out(a_bits, b_bits)
    ga32, gb32 = oracle.scan_bwd_bf16_f32out(a_bits, h32, d_bits)
    assert_close_f32(h, h32, "h")
    assert_close_f32(gb, gb32, "grad_beta")
    assert_close_f32(ga, ga32, "grad_alpha")
    # the same bits as one column tile per workgroup with the same time slicing
    one = lambda c: (c[0], c[1], c[2] // 2, c[3], 1)  # noqa: E731
    h1 = ext._forward(torch.bfloat16, a, b, one(fwd_cfg))
    ga1, gb1 = ext._backward(torch.bfloat16, a, h, do, one(bwd_cfg))
    assert torch.equal(h, h1) and torch.equal(ga, ga1) and torch.equal(gb, gb1)


def test_two_column_tiles_f32_and_refusals(oracle):
    import ctypes

    alpha, beta, dout = make_inputs("sigmoid", 3, 515, 256, dtype=torch.float32, seed=23)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    for fwd_cfg, bwd_cfg in [((1, 32, 8, 0, 2), (1, 16, 8, 0, 2)), ((1, 16, 16, 0, 2), (1, 16, 2, 0, 2))]:
        h = ext._forward(torch.float32, a, b, fwd_cfg)
        ga, gb = ext._backward(torch.float32, a, h, do, bwd_cfg)
        h_or = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy(), fused=True)
        ga_or, gb_or = oracle.scan_bwd_f32(alpha.numpy(), h.cpu().numpy(), dout.numpy(), fused=True)
        np.testing.assert_allclose(h.cpu().numpy(), h_or, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(gb.cpu().numpy(), gb_or, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(ga.cpu().numpy(), ga_or, rtol=1e-4, atol=1e-5)
    ext.workspace_status()
    # what has no two-column kernel is refused, never run wrongly
    lib = _native.lib()
    sp = torch.cuda.current_stream().cuda_stream
    t = torch.zeros(2, 64, 328, dtype=torch.bfloat16, device=DEV)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)

    def fwd(cfg, d=256):
        return lib.fss_scan_fwd_ex(0, t.data_ptr(), t.data_ptr(), t.data_ptr(), 2, 64, d, ws.data_ptr(), ws.numel(), sp,
                                   ctypes.byref(_native.FssConfig(*cfg)))

    assert fwd((2, 16, 4, 0, 2)) == 0
    assert fwd((2, 16, 4, 0, 2), d=328) == 5      # three column tiles per row cannot be paired
    assert fwd((2, 16, 3, 0, 2)) == 5             # the waves do not split over two columns
    assert fwd((2, 8, 4, 0, 2)) == 5 and fwd((1, 16, 4, 0, 2)) == 5 and fwd((2, 16, 4, 0, 3)) == 5
    h0 = torch.zeros(2, 256, device=DEV)
    assert lib.fss_scan_fwd_state(0, t.data_ptr(), t.data_ptr(), t.data_ptr(), h0.data_ptr(), None, 2, 64, 256,
                                  ws.data_ptr(), ws.numel(), sp, ctypes.byref(_native.FssConfig(2, 16, 4, 0, 2))) == 5
    assert lib.fss_gated_scan_fwd(0, t.data_ptr(), t.data_ptr(), t.data_ptr(), 2, 64, 256, ws.data_ptr(), ws.numel(), sp,
                                  ctypes.byref(_native.FssConfig(2, 16, 4, 0, 2))) == 5
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_grad_beta_in_place_over_dout(dtype):
    """grad_beta written over dout itself - the one overlap the kernels allow, which gives the
    backward the reference's footprint of one allocation (it aliases grad_beta onto the saved h,
    csrc/sequential_scan_kernel.cu:197): bit-identical to the out-of-place result, for chained,
    ragged and capped launches and for two column tiles per workgroup."""
    narrow = dtype != torch.float32
    for shape, config in [((2, 777, 328), None), ((3, 1000, 256), (2 if narrow else 1, 16, 4)), ((2, 515, 204), (1, 8, 2, 3)),
                          ((1, 2049, 512), (2 if narrow else 1, 16, 8, 0, 2)), ((8, 4096, 1024), None), ((2, 5, 7), None)]:
        alpha, beta, dout = make_inputs("hawk", *shape, dtype=dtype, seed=41)
        a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
        h = ext._forward(dtype, a, b)
        ga_ref, gb_ref = ext._backward(dtype, a, h, do, config)
        work = do.clone()
        ga, gb = ext._backward(dtype, a, h, work, config, overwrite_grad_out=True)
        ext.workspace_status()
        assert gb.data_ptr() == work.data_ptr()
        assert torch.equal(gb, gb_ref) and torch.equal(ga, ga_ref), (shape, config)
    # the public callee of the reference's name takes the option too
    ga, gb = ext.scan_backward_half(a.bfloat16(), h.bfloat16(), do.bfloat16().clone(), overwrite_grad_out=True) if not narrow else \
        ext.scan_backward_half(a, h, do.clone(), overwrite_grad_out=True)
    assert ga.shape == gb.shape == a.shape


@pytest.mark.parametrize("groups", [1, 3, 7, 64])
@pytest.mark.parametrize("config", [(1, 8, 1), (2, 8, 3), (2, 16, 8), (2, 32, 2), (4, 8, 6)],
                         ids=lambda c: "v%d_s%d_w%d" % c)
def test_bf16_few_workgroups_walk_many_tiles(oracle, config, groups):
    """The grid is persistent: cap it far below the tile count, so that every workgroup
    loops over many tiles and chunks wait on tiles of the same workgroup's earlier rounds."""
    alpha, beta, dout = make_inputs("sigmoid", 2, 1531, 200, seed=13)
    check_bf16(oracle, alpha, beta, dout, config=config + (groups,), what=f"{config} groups={groups}")
    ext.workspace_status()


@pytest.mark.parametrize("config", [(1, 8, 1), (1, 8, 2), (1, 8, 4), (2, 8, 2), (1, 16, 1), (2, 8, 8)],
                         ids=lambda c: "v%d_s%d_w%d" % c)
def test_bf16_full_grid_is_resident(oracle, config):
    """Small workgroups at a size where the uncapped grid fills the device: every wait
    must be served (no chain timeout), i.e. the grid really is resident all at once."""
    alpha, beta, dout = make_inputs("sigmoid", 8, 4096, 1024, seed=17)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(torch.bfloat16, a, b, config)
    ga, gb = ext._backward(torch.bfloat16, a, h, do, config)
    ext.workspace_status()  # raises on a chain timeout
    h_ref = ext._forward(torch.bfloat16, a, b, (2, 32, 16))
    ga_ref, gb_ref = ext._backward(torch.bfloat16, a, h_ref, do, (2, 16, 16))
    for got, want in ((h, h_ref), (ga, ga_ref), (gb, gb_ref)):
        close = (got.float() - want.float()).abs().cpu().numpy() <= 1e-3
        assert ((ulp_distance(bits(got), bits(want)) <= 2) | close).all()


@pytest.mark.parametrize("config", [(1, 8, 4), (2, 8, 16), (2, 16, 2), (4, 8, 8), (1, 32, 1)],
                         ids=lambda c: "v%d_s%d_w%d" % c)
def test_f32_chunking(oracle, config):
    alpha, beta, dout = make_inputs("sigmoid", 3, 515, 204, dtype=torch.float32, seed=11)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(torch.float32, a, b, config)
    ga, gb = ext._backward(torch.float32, a, h, do, config)
    h_or = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy(), fused=True)
    ga_or, gb_or = oracle.scan_bwd_f32(alpha.numpy(), h.cpu().numpy(), dout.numpy(), fused=True)
    assert rel_l2(h.cpu().numpy(), h_or) < 1e-6
    assert rel_l2(gb.cpu().numpy(), gb_or) < 1e-6
    assert rel_l2(ga.cpu().numpy(), ga_or) < 1e-6
    np.testing.assert_allclose(h.cpu().numpy(), h_or, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gb.cpu().numpy(), gb_or, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ga.cpu().numpy(), ga_or, rtol=1e-4, atol=1e-5)


def test_f32_one_wave_bit_exact(oracle):
    alpha, beta, dout = make_inputs("normal", 2, 8, 100, dtype=torch.float32, seed=3)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(torch.float32, a, b, (1, 8, 1))
    ga, gb = ext._backward(torch.float32, a, h, do, (1, 8, 1))
    np.testing.assert_array_equal(h.cpu().numpy(), oracle.scan_fwd_f32(alpha.numpy(), beta.numpy(), fused=True))
    ga_or, gb_or = oracle.scan_bwd_f32(alpha.numpy(), h.cpu().numpy(), dout.numpy(), fused=True)
    np.testing.assert_array_equal(gb.cpu().numpy(), gb_or)
    np.testing.assert_array_equal(ga.cpu().numpy(), ga_or)


# ------------------------------------------------- the measured configurations


@pytest.mark.parametrize("case", list(BASELINE_CASES), ids=list(BASELINE_CASES))
def test_baseline_configs_full_size(oracle, case):
    recipe, bs, seq, d = BASELINE_CASES[case]
    alpha, beta, dout = make_inputs(recipe, bs, seq, d)
    # N(0,1) alphas exceed 1 a third of the time: a product of a few of them can
    # amplify the fp32 rounding of a re-associated carry, so allow more ulps there
    check_bf16(oracle, alpha, beta, dout, max_ulp=2 if recipe != "normal" else 4, what=case)
    ext.workspace_status()


@pytest.mark.parametrize(
    "bs,seq,d",
    [(12, 2048, 1024), (8, 1536, 1536), (5, 2048, 1024), (2, 4096, 1792), (16, 1024, 2048)],
    ids=["96_groups", "96_groups_12_stripes", "40_groups", "28_groups", "256_groups"],
)
def test_tile_orders_of_full_grids(oracle, bs, seq, d):
    """Shapes whose launches fill the device and take their tiles in the different orders the
    kernels know: column groups in eighths that do not divide the grid (96, 40), that equal it
    (256), and a number of groups that does not divide by 8 (28)."""
    alpha, beta, dout = make_inputs("sigmoid", bs, seq, d, seed=bs + d)
    check_bf16(oracle, alpha, beta, dout, what=f"({bs},{seq},{d})")
    ext.workspace_status()


def test_fp32_at_headline_shape(oracle):
    """fp32 at bs 8, seq 4096, d 1024: 128 MiB per tensor, so the backward runs the instantiation
    that reads dout with the streaming hint.  Against the fp32 oracle, the reference's fp32 bar
    (relative L2 error below 1e-6) and elementwise."""
    alpha, beta, dout = make_inputs("sigmoid", 8, 4096, 1024, dtype=torch.float32, seed=83)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext.scan_forward(a, b)
    ga, gb = ext.scan_backward(a, h, do)
    ext.workspace_status()
    h_ref = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy())
    ga_ref, gb_ref = oracle.scan_bwd_f32(alpha.numpy(), h_ref, dout.numpy())
    for name, got, want in (("h", h, h_ref), ("grad_alpha", ga, ga_ref), ("grad_beta", gb, gb_ref)):
        got = got.cpu().numpy()
        assert rel_l2(got, want) < 1e-6, name
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5), name


def test_cache_policies_give_identical_results():
    """The cache policy selects hints on loads and stores, never the tiling: every output bit stays.
    Shapes on both sides of the sizes at which the automatic policy switches its hints (the same
    with alphas near 1, where the composed carries matter: tests/test_determinism_gpu.py)."""
    import fast_sequential_scan_amd as pkg

    for shape in ((4, 1000, 512), (8, 4096, 1024)):
        alpha, beta, dout = make_inputs("sigmoid", *shape, seed=84)
        a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
        results = {}
        for policy in ("auto", "streaming"):
            previous = pkg.set_cache_policy(policy)
            try:
                h = ext.scan_forward_half(a, b)
                results[policy] = (h, *ext.scan_backward_half(a, h, do))
            finally:
                pkg.set_cache_policy(previous)
        for x, y in zip(results["auto"], results["streaming"]):
            assert torch.equal(x, y)
    ext.workspace_status()


def test_closed_forms_at_headline_shape():
    """Size-independent properties at the full headline size (bs 8, seq 4096, d 1024)."""
    bs, seq, d = 8, 4096, 1024
    beta = torch.randn(bs, seq, d, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(DEV)
    zeros = torch.zeros_like(beta)
    # alpha == 0 -> h == beta exactly
    h = ext.scan_forward_half(zeros, beta)
    assert torch.equal(h, beta)
    # linearity in beta for fixed alpha: scan(a, 2b) == 2 scan(a, b) exactly (power of two)
    alpha = torch.sigmoid(torch.randn(bs, seq, d, generator=torch.Generator().manual_seed(6))).to(torch.bfloat16).to(DEV)
    h1 = ext.scan_forward_half(alpha, beta)
    h2 = ext.scan_forward_half(alpha, beta * 2)
    assert torch.equal(h2.float(), h1.float() * 2)
    # alpha == 1, beta == 1/64: h[t] = (t+1)/64, exact in fp32, compare after bf16 rounding
    ones = torch.ones_like(beta)
    small = torch.full_like(beta, 1.0 / 64)
    h = ext.scan_forward_half(ones, small)
    expect = ((torch.arange(seq, device=DEV, dtype=torch.float32) + 1) / 64).to(torch.bfloat16)
    assert torch.equal(h, expect[None, :, None].expand_as(h))
    # backward with dout == 0 -> both grads exactly zero; with alpha == 0 -> grad_beta == dout
    ga, gb = ext.scan_backward_half(alpha, h1, zeros)
    assert not ga.any() and not gb.any()
    ga, gb = ext.scan_backward_half(zeros, h1, beta)
    assert torch.equal(gb, beta)
    assert torch.equal(ga[:, 1:].float(), (beta[:, 1:].float() * h1[:, :-1].float()).to(torch.bfloat16).float())
    assert not ga[:, 0].any()
    ext.workspace_status()


@pytest.mark.parametrize("shape", [(32, 4096, 1024), (256, 512, 512)], ids=["2^27", "2^26_seq512"])
def test_fp32_closed_forms_at_the_sizes_that_change_the_launch_configuration(shape):
    """fp32 tensors of 2^26 and 2^27 elements take other launch configurations (16 steps or 8 bytes per
    lane).  alpha == 1 and beta, dout powers of two that differ by channel and batch row: every
    partial sum and product is exact in fp32 whatever the chunking, so the results are known bit for
    bit: h[t] = (t+1) beta, grad_beta[t] = (seq-t) dout, grad_alpha[t] = h[t-1] grad_beta[t]."""
    bs, seq, d = shape
    t = torch.arange(seq, device=DEV, dtype=torch.float32)[None, :, None]
    c = torch.arange(d, device=DEV)[None, None, :]
    b = torch.arange(bs, device=DEV)[:, None, None]
    beta_bc = torch.ldexp(torch.ones((), device=DEV), (c % 4 + b % 2 - 6).to(torch.int32)).to(torch.float32)
    dout_bc = torch.ldexp(torch.ones((), device=DEV), (c % 2 - 6 + 0 * b).to(torch.int32)).to(torch.float32)
    alpha = torch.ones(shape, device=DEV)
    beta = beta_bc.expand(shape).contiguous()
    h = ext.scan_forward(alpha, beta)
    assert torch.equal(h, ((t + 1) * beta_bc).expand(shape))
    del beta
    dout = dout_bc.expand(shape).contiguous()
    ga, gb = ext.scan_backward(alpha, h, dout)
    ext.workspace_status()
    assert torch.equal(gb, ((seq - t) * dout_bc).expand(shape))
    assert torch.equal(ga, (t * beta_bc * (seq - t) * dout_bc).expand(shape))


# -------------------------------------------------------------------- edge cases


def test_alpha_row_zero_is_never_used(oracle):
    alpha, beta, dout = make_inputs("sigmoid", 2, 300, 64, seed=21)
    h0, ga0, gb0 = run_bf16(alpha, beta, dout)
    alpha2 = alpha.clone()
    alpha2[:, 0, :] = float("nan")
    h1, ga1, gb1 = run_bf16(alpha2, beta, dout)
    assert torch.equal(h0, h1) and torch.equal(gb0, gb1) and torch.equal(ga0, ga1)
    assert not ga1[:, 0].any()


def test_empty_tensors():
    for shape in [(0, 5, 8), (2, 0, 8), (2, 5, 0)]:
        a = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
        h = ext.scan_forward_half(a, a)
        assert h.shape == a.shape
        ga, gb = ext.scan_backward_half(a, h, a)
        assert ga.shape == a.shape and gb.shape == a.shape


def test_non_contiguous_and_offset_inputs(oracle):
    alpha, beta, dout = make_inputs("sigmoid", 2, 130, 70, seed=31)
    # time-major storage viewed as (bs, seq, d): not contiguous
    a_nc = alpha.to(DEV).transpose(0, 1).contiguous().transpose(0, 1)
    b_nc = beta.to(DEV).transpose(0, 1).contiguous().transpose(0, 1)
    assert not a_nc.is_contiguous()
    h = ext.scan_forward_half(a_nc, b_nc)
    h_ref = ext.scan_forward_half(alpha.to(DEV), beta.to(DEV))
    assert torch.equal(h, h_ref)
    # a contiguous view that starts 2 bytes into its storage: only element alignment
    flat = torch.empty(alpha.numel() + 1, dtype=torch.bfloat16, device=DEV)
    a_off = flat[1:].view(alpha.shape)
    a_off.copy_(alpha)
    assert a_off.data_ptr() % 4 == 2
    h_off = ext.scan_forward_half(a_off, beta.to(DEV))
    assert torch.equal(h_off, h_ref)
    ga, gb = ext.scan_backward_half(a_off, h_ref, dout.to(DEV))
    ga_ref, gb_ref = ext.scan_backward_half(alpha.to(DEV), h_ref, dout.to(DEV))
    assert torch.equal(ga, ga_ref) and torch.equal(gb, gb_ref)


def test_non_default_stream_and_back_to_back_launches(oracle):
    alpha, beta, dout = make_inputs("sigmoid", 4, 2000, 256, seed=41)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h_ref, ga_ref, gb_ref = run_bf16(alpha, beta, dout)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        outs = []
        for _ in range(20):  # back-to-back chained launches reuse one workspace
            h = ext.scan_forward_half(a, b)
            ga, gb = ext.scan_backward_half(a, h, do)
            outs.append((h, ga, gb))
        ext.workspace_status()
    s.synchronize()
    for h, ga, gb in outs:
        assert torch.equal(h, h_ref) and torch.equal(ga, ga_ref) and torch.equal(gb, gb_ref)


# ----------------------------------------------------- the public autograd API


def test_scan_cu_autograd_matches_oracle(oracle):
    alpha, beta, dout = make_inputs("sigmoid", 3, 600, 512, seed=51)
    a = alpha.to(DEV).requires_grad_(True)
    b = beta.to(DEV).requires_grad_(True)
    out = scan_cu(a, b)
    out.backward(dout.to(DEV), retain_graph=True)
    h32 = oracle.scan_fwd_bf16_f32out(bits(alpha), bits(beta))
    ga32, gb32 = oracle.scan_bwd_bf16_f32out(bits(alpha), h32, bits(dout))
    assert_close_f32(out, h32, "h")
    assert_close_f32(a.grad, ga32, "grad_alpha")
    assert_close_f32(b.grad, gb32, "grad_beta")
    # a second backward works: the forward output is not overwritten by the first
    # (the reference aliases grad_beta onto it: csrc/sequential_scan_kernel.cu:197)
    first = (a.grad.clone(), b.grad.clone())
    a.grad = b.grad = None
    out.backward(dout.to(DEV))
    assert torch.equal(a.grad, first[0]) and torch.equal(b.grad, first[1])
    assert_close_f32(out, h32, "h after two backwards")


def test_scan_cu_under_autocast_casts_to_bf16(oracle):
    alpha, beta, _ = make_inputs("sigmoid", 2, 100, 64, dtype=torch.float32, seed=61)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = scan_cu(alpha.to(DEV), beta.to(DEV))
    assert out.dtype == torch.bfloat16
    want = oracle.scan_fwd_bf16(bits(alpha.to(torch.bfloat16)), bits(beta.to(torch.bfloat16)), fused=True)
    assert (ulp_distance(bits(out), want) <= 2).all()
    with pytest.raises(RuntimeError):  # outside autocast fp32 input is a dtype error, as in the reference
        scan_cu(alpha.to(DEV), beta.to(DEV))


@pytest.mark.parametrize("bs,sq,d", [(9, 128, 512), (2, 1024, 768), (12, 256, 1024)])
def test_reference_test_matrix_fp32(oracle, bs, sq, d):
    """The reference's own fp32 test (sequential_scan/test_scan_cuda.py:27-72): N(0,1)
    inputs, relative L2 error below 1e-6 for the output and both gradients."""
    g = torch.Generator().manual_seed(0)
    alpha = torch.randn(bs, sq, d, generator=g)
    beta = torch.randn(bs, sq, d, generator=g)
    dy = torch.randn(bs, sq, d, generator=g)
    a = alpha.to(DEV).requires_grad_(True)
    b = beta.to(DEV).requires_grad_(True)
    out = scan_cu_single(a, b)
    out.backward(dy.to(DEV))
    h = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy())
    ga, gb = oracle.scan_bwd_f32(alpha.numpy(), h, dy.numpy())
    assert rel_l2(out.detach().cpu().numpy(), h) < 1e-6
    assert rel_l2(a.grad.cpu().numpy(), ga) < 1e-6
    assert rel_l2(b.grad.cpu().numpy(), gb) < 1e-6


@pytest.mark.parametrize("bs,sq,d", [(5, 128, 512), (13, 512, 768), (3, 1024, 1024)])
def test_reference_test_matrix_bf16(oracle, bs, sq, d):
    """The reference's bf16 test (test_scan_cuda.py:80-124): relative L2 error below 0.1
    against the scan evaluated in bf16 arithmetic; here against the fp32-accumulated one."""
    alpha, beta, dy = make_inputs("normal", bs, sq, d, seed=71)
    a = alpha.to(DEV).requires_grad_(True)
    b = beta.to(DEV).requires_grad_(True)
    out = scan_cu(a, b)
    out.backward(dy.to(DEV))
    h32 = oracle.scan_fwd_bf16_f32out(bits(alpha), bits(beta))
    ga32, gb32 = oracle.scan_bwd_bf16_f32out(bits(alpha), h32, bits(dy))
    assert rel_l2(out.detach().float().cpu().numpy(), h32) < 1e-2
    assert rel_l2(a.grad.float().cpu().numpy(), ga32) < 1e-2
    assert rel_l2(b.grad.float().cpu().numpy(), gb32) < 1e-2


def test_c_abi_rejects_bad_arguments():
    lib = _native.lib()
    a = torch.zeros(2, 300, 64, dtype=torch.bfloat16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.fss_scan_fwd_bf16(None, a.data_ptr(), a.data_ptr(), 2, 300, 64, None, 0, s) == 1
    assert lib.fss_scan_fwd_bf16(a.data_ptr(), a.data_ptr(), a.data_ptr(), -1, 300, 64, None, 0, s) == 2
    # 300 steps need more than one chunk here -> a workspace is required
    cfg = _native.FssConfig(2, 8, 2, 0)
    import ctypes
    assert lib.fss_scan_fwd_ex(0, a.data_ptr(), a.data_ptr(), a.data_ptr(), 2, 300, 64, None, 0, s, ctypes.byref(cfg)) == 4
    bad = _native.FssConfig(3, 8, 2, 0)
    assert lib.fss_scan_fwd_ex(0, a.data_ptr(), a.data_ptr(), a.data_ptr(), 2, 300, 64, None, 0, s, ctypes.byref(bad)) == 5
    odd = _native.FssConfig(2, 8, 1, 0)  # vec 2 needs 4-byte alignment
    assert lib.fss_scan_fwd_ex(0, a.data_ptr() + 2, a.data_ptr(), a.data_ptr(), 1, 8, 64, None, 0, s, ctypes.byref(odd)) == 3
    torch.cuda.synchronize()


def test_hip_graph_replays_match_eager(oracle):
    """A captured forward+backward step replays correctly: the chaining workspace keeps its
    launch counter on the device, so every replay sees fresh tags.  Replays alternate with
    eager launches and synchronisations, and each replay is checked."""
    alpha, beta, dout = make_inputs("sigmoid", 4, 3000, 256, seed=81)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h_ref, ga_ref, gb_ref = run_bf16(alpha, beta, dout)
    lib = _native.lib()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sp = side.cuda_stream
        ws = torch.empty(lib.fss_workspace_bytes_max(*a.shape), dtype=torch.uint8, device=DEV)
        _native.check(lib.fss_workspace_init(ws.data_ptr(), ws.numel(), sp))
        h, ga, gb = torch.empty_like(a), torch.empty_like(a), torch.empty_like(a)

        def step():
            _native.check(lib.fss_scan_fwd_bf16(a.data_ptr(), b.data_ptr(), h.data_ptr(), *a.shape,
                                                ws.data_ptr(), ws.numel(), sp))
            _native.check(lib.fss_scan_bwd_bf16(a.data_ptr(), h.data_ptr(), do.data_ptr(), ga.data_ptr(),
                                                gb.data_ptr(), *a.shape, ws.data_ptr(), ws.numel(), sp))

        step()  # warm: device check, residency query
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        for i in range(5):
            h.zero_(), ga.zero_(), gb.zero_()
            graph.replay()
            side.synchronize()
            assert torch.equal(h, h_ref) and torch.equal(ga, ga_ref) and torch.equal(gb, gb_ref), i
            step()  # eager work between replays, same workspace
            side.synchronize()
        assert lib.fss_workspace_status(ws.data_ptr(), sp) == 0


def test_tensors_larger_than_4_GiB():
    """Byte offsets beyond 2^32 (the reference's index math is 32-bit:
    csrc/include/sequential_scan_kernel_bf16.cuh:63-70).  Checked through closed forms, on the device."""
    bs, seq, d = 3, 8192, 90000  # 2.2e9 elements, 4.4 GB per bf16 tensor
    g = torch.Generator(device=DEV).manual_seed(3)
    beta = torch.randn(bs, seq, d, generator=g, device=DEV, dtype=torch.bfloat16)
    alpha = torch.zeros_like(beta)
    h = ext.scan_forward_half(alpha, beta)
    assert torch.equal(h, beta)
    # alpha == 1 on one channel per batch row, beta == 1/128 there: h[t] = (t+1)/128
    alpha[:, :, d - 2] = 1.0
    beta[:, :, d - 2] = 1.0 / 128
    h = ext.scan_forward_half(alpha, beta)
    expect = ((torch.arange(seq, device=DEV, dtype=torch.float32) + 1) / 128).to(torch.bfloat16)
    assert torch.equal(h[:, :, d - 2], expect[None, :].expand(bs, seq))
    assert torch.equal(h[:, :, d - 1], beta[:, :, d - 1])
    # backward: alpha == 0 elsewhere -> grad_beta == dout, grad_alpha[t] = dout[t]*h[t-1]
    ga, gb = ext.scan_backward_half(alpha, h, beta)
    assert torch.equal(gb[:, :, : d - 2], beta[:, :, : d - 2])
    last = (slice(None), slice(1, None), d - 1)
    assert torch.equal(ga[last].float(), (beta[last].float() * h[:, :-1, d - 1].float()).to(torch.bfloat16).float())
    ext.workspace_status()
    del alpha, beta, h, ga, gb
    torch.cuda.empty_cache()


def test_scans_on_two_streams_do_not_overlap(oracle):
    """A scan fills the device with workgroups that wait for each other; the library chains launches
    that arrive on different streams, so interleaved launches stay correct and never time out."""
    shape = (8, 2048, 1024)
    sets = []
    for seed in (41, 42):
        alpha, beta, dout = make_inputs("sigmoid", *shape, seed=seed)
        sets.append(tuple(t.to(DEV) for t in (alpha, beta, dout)))
    want = []
    for a, b, do in sets:
        h = ext.scan_forward_half(a, b)
        want.append((h, *ext.scan_backward_half(a, h, do)))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [None, None]
    for _ in range(8):  # no host synchronisation between the launches
        for i, s in enumerate(streams):
            with torch.cuda.stream(s):
                a, b, do = sets[i]
                h = ext.scan_forward_half(a, b)
                got[i] = (h, *ext.scan_backward_half(a, h, do))
    for i, s in enumerate(streams):
        with torch.cuda.stream(s):
            ext.workspace_status()  # synchronises the stream; raises on a chain time-out
    torch.cuda.synchronize()
    for i in range(2):
        for g, w in zip(got[i], want[i]):
            assert torch.equal(g, w)


# ------------------------------------------- tensors with only their element alignment


def _offset_view(t: torch.Tensor, offset_bytes: int) -> torch.Tensor:
    """A contiguous copy of `t` on the device that starts `offset_bytes` into a 256-byte aligned
    allocation."""
    n_off = offset_bytes // t.element_size()
    flat = torch.empty(t.numel() + n_off, dtype=t.dtype, device=DEV)
    view = flat[n_off:].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 256 == offset_bytes and view.is_contiguous()
    return view


@pytest.mark.parametrize("offset", [2, 4])
@pytest.mark.parametrize("shape", [(1, 4096, 2048), (8, 3000, 1024), (1, 20000, 512)], ids=str)
def test_offset_views_at_sizes_that_chain_many_chunks(oracle, shape, offset):
    """Contiguous tensors that start 2 or 4 bytes into their storage take fewer channels per lane
    and smaller tiles than aligned ones, so they chain more chunks and need a larger workspace
    than the 16-byte aligned plan of the same shape: the public wrappers must size for that.
    Forward and backward against the oracle; the reference takes any contiguous tensor
    (csrc/sequential_scan_kernel.cu:126-187)."""
    alpha, beta, dout = make_inputs("sigmoid", *shape, seed=91 + offset)
    a, b, do = (_offset_view(t, offset) for t in (alpha, beta, dout))
    h = ext.scan_forward_half(a, b)
    ga, gb = ext.scan_backward_half(a, _offset_view(h, offset), do)
    ext.workspace_status()
    a_bits, b_bits, d_bits = bits(alpha), bits(beta), bits(dout)
    h32 = oracle.scan_fwd_bf16_f32out(a_bits, b_bits)
    ga32, gb32 = oracle.scan_bwd_bf16_f32out(a_bits, h32, d_bits)
    assert_close_f32(h, h32, "h")
    assert_close_f32(gb, gb32, "grad_beta")
    assert_close_f32(ga, ga32, "grad_alpha")
    # and through autograd, as a user would
    a_req, b_req = a.detach().requires_grad_(True), b.detach().requires_grad_(True)
    scan_cu(a_req, b_req).backward(do)
    assert torch.equal(a_req.grad, ga) and torch.equal(b_req.grad, gb)


# ------------------------------------------------------- |alpha| > 1 over long stretches


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_growing_recurrence_with_zero_state_stays_zero(oracle, dtype):
    """alpha == 2 over 300 steps: the product of a chunk's alphas overflows fp32 (2^128) long
    before the sequence ends.  Where the state is exactly 0 the sequential recurrence keeps it 0
    (sequential_scan/common.py:55) and so must the chunked one (inf * 0 would be NaN); where it
    is not, both overflow to inf at the same step.  Every tiling, forward and backward."""
    bs, seq, d = 2, 300, 128
    alpha = torch.full((bs, seq, d), 2.0, dtype=dtype)
    zeros = torch.zeros_like(alpha)
    e0 = zeros.clone()
    e0[:, 0] = 1.0
    e_last = zeros.clone()
    e_last[:, -1] = 1.0
    small = torch.full_like(alpha, 2.0 ** -20)

    def run(beta, dout, h_for_bwd, config):
        h = ext._forward(dtype, alpha.to(DEV), beta.to(DEV), config)
        ga, gb = ext._backward(dtype, alpha.to(DEV), h_for_bwd.to(DEV), dout.to(DEV), config)
        ext.workspace_status()
        return h.float().cpu().numpy(), ga.float().cpu().numpy(), gb.float().cpu().numpy()

    def want(beta, dout, h_for_bwd):
        if dtype == torch.float32:
            h = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy(), fused=True)
            ga, gb = oracle.scan_bwd_f32(alpha.numpy(), h_for_bwd.numpy(), dout.numpy(), fused=True)
            return h, ga, gb
        h = oracle.scan_fwd_bf16(bits(alpha), bits(beta), fused=True)
        ga, gb = oracle.scan_bwd_bf16(bits(alpha), bits(h_for_bwd), bits(dout), fused=True)
        return tuple(oracle.bf16_bits_to_f32(x) for x in (h, ga, gb))

    with np.errstate(over="ignore", invalid="ignore"):
        for config in [None, (1, 8, 4), (2, 16, 8), (2, 8, 16), (1, 32, 2)]:
            # zero everywhere: stays zero, no NaN from inf * 0
            h, ga, gb = run(zeros, zeros, small, config)
            assert not h.any() and not ga.any() and not gb.any(), config
            # one impulse: exact powers of two until fp32 (or bf16) overflows, then inf - never NaN
            h, ga, gb = run(e0, e_last, small, config)
            h_w, ga_w, gb_w = want(e0, e_last, small)
            assert not np.isnan(h).any() and not np.isnan(gb).any() and not np.isnan(ga).any(), config
            np.testing.assert_array_equal(h, h_w, err_msg=str(config))
            np.testing.assert_array_equal(gb, gb_w, err_msg=str(config))
            np.testing.assert_array_equal(ga, ga_w, err_msg=str(config))


# ------------------------------------------------------------------ chain time-outs


def test_chain_timeout_poisons_the_output_and_is_reported(oracle):
    """A look-back that gives up must be impossible to miss: NaN from the affected chunk on, the
    workspace's sticky word, and the host-visible word that makes the NEXT call on that stream
    raise without any synchronisation.  Forced from the host (a poll budget of zero makes every
    look-back give up at once), so every kernel runs to completion."""
    lib = _native.lib()
    alpha, beta, dout = make_inputs("sigmoid", 2, 3000, 256, seed=95)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    good = ext.scan_forward_half(a, b)
    ext.workspace_status()
    first_chunk = 32 * 16  # rows of the largest tile any configuration covers in one chunk
    previous = lib.fss_debug_set_spin_limit(0)
    try:
        assert previous == 1 << 20
        h = ext.scan_forward_half(a, b)
        torch.cuda.synchronize()
        assert torch.isnan(h[:, first_chunk:].float()).all()      # everything behind the first chunk
        assert torch.equal(h[:, :8], good[:, :8])                  # the first chunk needs no look-back
        with pytest.raises(_native.FssError) as err:              # the next call reports it, before launching
            ext.scan_forward_half(a, b)
        assert err.value.status == _native.FSS_ERR_CHAIN_TIMEOUT
        # the backward path and the debug query report it as well
        ga, gb = ext.scan_backward_half(a, good, do)
        torch.cuda.synchronize()
        assert torch.isnan(gb[:, : 3000 - first_chunk].float()).all()
        with pytest.raises(_native.FssError):
            ext.workspace_status()
    finally:
        lib.fss_debug_set_spin_limit(previous)
    # back to normal: same workspace, correct results, nothing pending
    h = ext.scan_forward_half(a, b)
    ext.workspace_status()
    assert torch.equal(h, good)
    # through the C ABI without the Python layer: sticky word and attached flag
    ws = torch.zeros(lib.fss_workspace_bytes_max(*a.shape), dtype=torch.uint8, device=DEV)
    flag = torch.zeros(1, dtype=torch.int32).pin_memory()
    sp = torch.cuda.current_stream().cuda_stream
    _native.check(lib.fss_workspace_init(ws.data_ptr(), ws.numel(), sp))
    _native.check(lib.fss_workspace_attach_flag(ws.data_ptr(), flag.data_ptr(), sp))
    out = torch.empty_like(a)
    lib.fss_debug_set_spin_limit(0)
    try:
        _native.check(lib.fss_scan_fwd_bf16(a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, ws.data_ptr(), ws.numel(), sp))
        torch.cuda.synchronize()
    finally:
        lib.fss_debug_set_spin_limit(1 << 20)
    assert int(flag[0]) == 1
    assert lib.fss_workspace_status(ws.data_ptr(), sp) == _native.FSS_ERR_CHAIN_TIMEOUT
    assert lib.fss_workspace_status(ws.data_ptr(), sp) == 0  # cleared by the query
    _native.check(lib.fss_scan_fwd_bf16(a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, ws.data_ptr(), ws.numel(), sp))
    torch.cuda.synchronize()
    assert torch.equal(out, good)


# --------------------------------- residency of every kernel family (no wait is left unserved)


def _big(dtype, shape=(8, 4096, 1024), seed=97):
    return tuple(t.to(DEV) for t in make_inputs("sigmoid", *shape, dtype=dtype, seed=seed))


def test_full_grids_of_small_workgroups_are_resident_in_every_kernel_family(oracle):
    """The grid of a chained scan is sized from a hand-derived bound on how many workgroups are
    resident at once; were it too high for some instantiation, workgroups that are not running
    would be waited for and the scan would time out.  One case per kernel family with the
    smallest workgroups and far more tiles than the device holds, each checked for a time-out
    and against the same kernel run with large workgroups."""
    from fast_sequential_scan_amd.sequential_scan_cuda import (
        gated_scan_backward, gated_scan_forward, scan_backward_cm, scan_backward_state, scan_forward_cm,
        scan_forward_state)

    def same(x, y, tol):
        assert torch.allclose(x.float(), y.float(), rtol=tol, atol=tol)

    for dtype, small_cfgs, tol in ((torch.float32, [(1, 8, 1), (1, 8, 2), (2, 8, 1)], 1e-4),
                                   (torch.float16, [(1, 8, 1), (2, 8, 2)], 2e-3)):
        a, b, do = _big(dtype)
        h_ref = ext._forward(dtype, a, b, (1, 16, 16))
        ga_ref, gb_ref = ext._backward(dtype, a, h_ref, do, (1, 16, 16))
        for cfg in small_cfgs:
            h = ext._forward(dtype, a, b, cfg)
            ga, gb = ext._backward(dtype, a, h_ref, do, cfg)
            ext.workspace_status()
            same(h, h_ref, tol), same(ga, ga_ref, tol), same(gb, gb_ref, tol)
    # bf16: the state kernels, the gated kernels, and the other cache policies of the plain scan
    a, b, do = _big(torch.bfloat16)
    h0 = torch.randn(8, 1024, device=DEV)
    h_ref, last_ref = scan_forward_state(a, b, h0, (2, 32, 16))
    ref = scan_backward_state(a, h_ref, do, h0, None, (2, 16, 16))
    for cfg in [(1, 8, 1), (2, 8, 2)]:
        h, last = scan_forward_state(a, b, h0, cfg)
        got = scan_backward_state(a, h_ref, do, h0, None, cfg)
        ext.workspace_status()
        same(h, h_ref, 2e-2), same(last, last_ref, 2e-2)
        for x, y in zip(got, ref):
            same(x, y, 2e-2)
    gate = (a.float() * 4 - 2).to(torch.bfloat16)
    g_ref = gated_scan_forward(gate, b, (2, 32, 16))
    gb_ref = gated_scan_backward(gate, b, g_ref, do, (2, 16, 16))
    for cfg in [(1, 8, 1), (2, 8, 2)]:
        hg = gated_scan_forward(gate, b, cfg)
        got = gated_scan_backward(gate, b, g_ref, do, cfg)
        ext.workspace_status()
        same(hg, g_ref, 2e-2)
        for x, y in zip(got, gb_ref):
            same(x, y, 2e-2)
    # plain forward with a kept output (tensors up to 48 MiB) and plain backward that streams dout
    # (tensors above 80 MiB): both are separate instantiations
    a, b, do = _big(torch.bfloat16, (8, 2048, 1024))
    h_ref = ext._forward(torch.bfloat16, a, b, (2, 32, 16))
    for cfg in [(1, 8, 1), (2, 8, 2)]:
        assert torch.equal(ext._forward(torch.bfloat16, a, b, cfg)[:, :8], h_ref[:, :8])
        ext.workspace_status()
    a, b, do = _big(torch.bfloat16, (8, 8192, 1024))
    h_ref = ext._forward(torch.bfloat16, a, b, (2, 32, 16))
    ga_ref, gb_ref = ext._backward(torch.bfloat16, a, h_ref, do, (2, 16, 16))
    for cfg in [(1, 8, 1), (2, 8, 2)]:
        ga, gb = ext._backward(torch.bfloat16, a, h_ref, do, cfg)
        ext.workspace_status()
        same(ga, ga_ref, 2e-2), same(gb, gb_ref, 2e-2)
    del a, b, do, h_ref, ga_ref, gb_ref
    # channel-major, chained (sequences beyond one workgroup's reach), one-wave workgroups
    for dtype, vec in ((torch.bfloat16, 8), (torch.float32, 4)):
        a, b, do = (t.transpose(1, 2).contiguous() for t in _big(dtype, (4, 8192, 1024)))
        h_ref = scan_forward_cm(a, b)
        ga_ref, gb_ref = scan_backward_cm(a, h_ref, do)
        h = scan_forward_cm(a, b, (vec, 0, 1))
        ga, gb = scan_backward_cm(a, h_ref, do, (vec, 0, 1))
        ext.workspace_status()
        tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
        same(h, h_ref, tol), same(ga, ga_ref, tol), same(gb, gb_ref, tol)
    torch.cuda.empty_cache()
