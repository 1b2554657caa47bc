"""Seeded random shapes and launch configurations through every entry point, against the oracle.

Shapes are drawn to hit the edges the fixed cases may miss: odd d, d just off a multiple of the
tile width, sequences just off a multiple of the tile length, one-element dimensions; explicit
configurations are drawn from what the library accepts for the dtype and direction.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402

DEV = "cuda:0"
TOL = {torch.bfloat16: (1e-2, 1e-2), torch.float16: (2e-3, 2e-3), torch.float32: (1e-4, 1e-5)}
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _draw_shape(rng):
    bs = int(rng.choice([1, 2, 3, 5]))
    d = int(rng.choice([1, 2, 7, 64, 126, 128, 130, 200, 384, 520]))
    seq = int(rng.choice([1, 2, 9, 63, 64, 65, 255, 256, 257, 511, 1000, 1025, 2049, 3001]))
    return bs, seq, d


def _draw_config(rng, dtype, d, backward, gated=False):
    if rng.random() < 0.4:
        return None
    wide = dtype != torch.float32
    vecs = [v for v in ((1, 2, 4, 8) if wide else (1, 2, 4)) if d % v == 0]
    if gated:
        vecs = [v for v in vecs if v <= (2 if wide else 1)]
    vec = int(rng.choice(vecs))
    budget = (64 if wide else 32) // vec
    steps = [s for s in (8, 16, 32) if s <= budget and not (gated and backward and s > 16)]
    step = int(rng.choice(steps))
    # wide lanes and the 32-step backward are built for 8 (4) waves at most: what a lane holds must fit its registers
    dwords = max(1, vec * (2 if wide else 4) // 4)
    most = 4 if vec >= 8 else 8 if (vec >= 4 or (not gated and vec >= 2 and dwords * step * (3 if backward else 2) > 64)) else 16
    for _ in range(20):
        waves = int(rng.integers(1, most + 1))
        look = min(waves, 16)
        while look > 1 and (2 * waves + look + 1) * vec * 512 > 60 * 1024:
            look -= 1
        if (2 * waves + look + 1) * vec * 512 <= 60 * 1024:
            break
    else:
        waves = 1
    groups = int(rng.choice([0, 0, 1, 3, 17]))
    return (vec, step, waves, groups)


def _tensors(rng, shape, dtype):
    g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
    alpha = torch.sigmoid(1.5 * torch.randn(shape, generator=g)).to(dtype)
    beta = torch.randn(shape, generator=g).to(dtype)
    dout = torch.randn(shape, generator=g).to(dtype)
    return alpha, beta, dout


def _check(got, want, dtype, what, outliers=0.0):
    rtol, atol = TOL[dtype]
    got = got.detach().float().cpu().numpy()
    bad = ~(np.abs(got - want) <= atol + rtol * np.abs(want))
    assert bad.mean() <= outliers, f"{what}: {bad.sum()} of {bad.size} off, worst {np.abs(got - want).max():.4g}"


@pytest.mark.parametrize("seed", range(24))
def test_plain_and_state_scans(oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = DTYPES[seed % 3]
    bs, seq, d = _draw_shape(rng)
    alpha, beta, dout = _tensors(rng, (bs, seq, d), dtype)
    fwd_cfg, bwd_cfg = _draw_config(rng, dtype, d, False), _draw_config(rng, dtype, d, True)
    what = f"seed {seed} {dtype} {(bs, seq, d)} fwd {fwd_cfg} bwd {bwd_cfg}"
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(dtype, a, b, fwd_cfg)
    ga, gb = ext._backward(dtype, a, h, do, bwd_cfg)
    a32, b32, d32 = alpha.float().numpy(), beta.float().numpy(), dout.float().numpy()
    _check(h, oracle.scan_fwd_f32(a32, b32), dtype, what + " h")
    ga_or, gb_or = oracle.scan_bwd_f32(a32, h.float().cpu().numpy(), d32)
    _check(gb, gb_or, dtype, what + " grad_beta")
    _check(ga, ga_or, dtype, what + " grad_alpha")
    # the state entry points: a state in, against the plain oracle on the sequence one step longer
    g = torch.Generator().manual_seed(seed)
    h0 = torch.randn(bs, d, generator=g)
    hs, h_last = ext.scan_forward_state(a, b, h0.to(DEV), fwd_cfg)
    a_ext = np.concatenate([np.zeros((bs, 1, d), np.float32), a32], axis=1)
    b_ext = np.concatenate([h0.numpy()[:, None, :], b32], axis=1)
    h_ext = oracle.scan_fwd_f32(a_ext, b_ext)
    _check(hs, h_ext[:, 1:], dtype, what + " h with state")
    np.testing.assert_allclose(h_last.cpu().numpy(), h_ext[:, -1], rtol=1e-4, atol=1e-4)
    ext.workspace_status()


@pytest.mark.parametrize("seed", range(12))
def test_many_column_groups_under_random_grids(oracle, seed):
    """Shapes with enough column groups for the tile orders that deal them out by XCD (a multiple
    of 8 groups: 24 to 128 here), small tiles (many chunks per sequence) and grids capped at random,
    so that rounds of the grid cut through chunks at every offset."""
    rng = np.random.default_rng(4000 + seed)
    dtype = DTYPES[seed % 3]
    bs = int(rng.choice([3, 5, 8, 12, 16]))
    d = int(rng.choice([512, 1024]))
    seq = int(rng.choice([257, 513, 1000]))
    alpha, beta, dout = _tensors(rng, (bs, seq, d), dtype)
    vec = 2 if dtype != torch.float32 else 1  # 128 (64) channels per column tile
    grids = [0, 8, 24, 40, 64, 100, 136]
    fwd_cfg = (vec, int(rng.choice([8, 16])), int(rng.choice([1, 2, 4])), int(rng.choice(grids)))
    bwd_cfg = (vec, int(rng.choice([8, 16])), int(rng.choice([1, 2, 4])), int(rng.choice(grids)))
    what = f"seed {seed} {dtype} {(bs, seq, d)} fwd {fwd_cfg} bwd {bwd_cfg}"
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext._forward(dtype, a, b, fwd_cfg)
    ga, gb = ext._backward(dtype, a, h, do, bwd_cfg)
    a32, b32, d32 = alpha.float().numpy(), beta.float().numpy(), dout.float().numpy()
    _check(h, oracle.scan_fwd_f32(a32, b32), dtype, what + " h")
    ga_or, gb_or = oracle.scan_bwd_f32(a32, h.float().cpu().numpy(), d32)
    _check(gb, gb_or, dtype, what + " grad_beta")
    _check(ga, ga_or, dtype, what + " grad_alpha")
    ext.workspace_status()


@pytest.mark.parametrize("seed", range(12))
def test_gated_scans(oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    dtype = DTYPES[seed % 3]
    bs, seq, d = _draw_shape(rng)
    gate, x, dout = _tensors(rng, (bs, seq, d), dtype)
    gate = (torch.logit(gate.float().clamp(1e-3, 1 - 1e-3))).to(dtype)  # back to a pre-activation
    fwd_cfg = _draw_config(rng, dtype, d, False, gated=True)
    bwd_cfg = _draw_config(rng, dtype, d, True, gated=True)
    what = f"seed {seed} {dtype} {(bs, seq, d)} fwd {fwd_cfg} bwd {bwd_cfg}"
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h = ext.gated_scan_forward(gd, xd, fwd_cfg)
    gg, gx = ext.gated_scan_backward(gd, xd, h, dd, bwd_cfg)
    rounding = {torch.bfloat16: "bf16", torch.float32: "f32", torch.float16: "f16"}[dtype]
    g32, x32, d32 = gate.float().numpy(), x.float().numpy(), dout.float().numpy()
    h_dev = h.float().cpu().numpy()
    rtol, atol = TOL[dtype]

    # every element within tolerance of the interval spanned by the two roundings of alpha (they
    # differ only where sigmoid(gate) sits on a rounding boundary of the storage type)
    def check(got, want, other, name):
        ok = oracle.within_rounding_envelope(got.detach().float().cpu().numpy(), want, other, rtol, atol)
        assert ok.all(), f"{what} {name}: {(~ok).sum()} of {ok.size} off"

    check(h, oracle.gated_scan_fwd(g32, x32, rounding), oracle.gated_scan_fwd(g32, x32, rounding, True), "h")
    want_gg, want_gx = oracle.gated_scan_bwd(g32, x32, h_dev, d32, rounding)
    other_gg, other_gx = oracle.gated_scan_bwd(g32, x32, h_dev, d32, rounding, True)
    check(gx, want_gx, other_gx, "grad_x")
    check(gg, want_gg, other_gg, "grad_gate")
    ext.workspace_status()


@pytest.mark.parametrize("seed", range(12))
def test_channel_major_scans(oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    dtype = DTYPES[seed % 3]
    bs, seq, d = _draw_shape(rng)
    seq = int(rng.choice([seq, seq * 2, 4100, 9001]))
    alpha, beta, dout = _tensors(rng, (bs, d, seq), dtype)
    widest = 8 if dtype != torch.float32 else 4
    vecs = [v for v in ({1, 2, widest} if dtype != torch.float32 else {1, widest}) if seq % v == 0]
    cfg = None if rng.random() < 0.4 else (int(rng.choice(sorted(vecs))), 0, int(rng.integers(1, 17)), int(rng.choice([0, 0, 2])))
    what = f"seed {seed} {dtype} {(bs, d, seq)} cfg {cfg}"
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext.scan_forward_cm(a, b, cfg)
    ga, gb = ext.scan_backward_cm(a, h, do, cfg)

    def t(x):
        return np.ascontiguousarray(x.detach().float().cpu().numpy().transpose(0, 2, 1))

    _check(h.transpose(1, 2), oracle.scan_fwd_f32(t(alpha), t(beta)), dtype, what + " h")
    ga_or, gb_or = oracle.scan_bwd_f32(t(alpha), t(h), t(dout))
    _check(gb.transpose(1, 2), gb_or, dtype, what + " grad_beta")
    _check(ga.transpose(1, 2), ga_or, dtype, what + " grad_alpha")
    ext.workspace_status()


# Mid-size shapes whose lengths and widths are no powers of two, with the library's own
# choices: they land on different rungs of the planning ladder (16- and 8-wave workgroups,
# one and two channels per lane, ragged last chunks and column tiles).
DEFAULT_CHOICE_SHAPES = [
    (3, 3000, 1536), (8, 3000, 1024), (5, 1500, 2560), (2, 5000, 768), (1, 12000, 520),
    (7, 700, 200), (2, 6000, 1030), (16, 1000, 384), (1, 40000, 130), (4, 2049, 1537),
]


@pytest.mark.parametrize("shape", DEFAULT_CHOICE_SHAPES, ids=[str(s) for s in DEFAULT_CHOICE_SHAPES])
def test_library_choices_at_odd_mid_size_shapes(oracle, shape):
    rng = np.random.default_rng(sum(shape))
    for dtype in (torch.bfloat16, torch.float32):
        alpha, beta, dout = _tensors(rng, shape, dtype)
        a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
        h = ext._forward(dtype, a, b)
        ga, gb = ext._backward(dtype, a, h, do)
        a32, b32, d32 = alpha.float().numpy(), beta.float().numpy(), dout.float().numpy()
        what = f"{dtype} {shape}"
        _check(h, oracle.scan_fwd_f32(a32, b32), dtype, what + " h")
        ga_or, gb_or = oracle.scan_bwd_f32(a32, h.float().cpu().numpy(), d32)
        _check(gb, gb_or, dtype, what + " grad_beta")
        _check(ga, ga_or, dtype, what + " grad_alpha")
    ext.workspace_status()
