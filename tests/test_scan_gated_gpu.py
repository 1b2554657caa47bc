"""GPU tests of the gated scan (fss_gated_scan_fwd / fss_gated_scan_bwd, scan_gated):
alpha = sigmoid(gate), beta = x*sqrt(1-alpha^2) computed inside the scan kernels.

Tolerances: rtol = atol = 1e-2 in bf16 (the bar of the plain bf16 scan), 1e-4 / 1e-5 in
fp32, for every element.  In bf16 the device's sigmoid (hardware exp2 and reciprocal, a few
fp32 ulps) can land on the other side of a bf16 rounding boundary than the oracle's float64
one for a few elements in 10^4; alpha then differs by one bf16 ulp there, and near
alpha -> 1 the backward amplifies that (alpha/s).  The oracle therefore evaluates twice -
alpha rounded to nearest, and to the other neighbour wherever the exact sigmoid lies within
8 fp32 ulps of the rounding boundary - and every element must lie within the tolerance of
the interval the two evaluations span.  Where no such element influences a result the two
agree and the check is the plain tolerance: nothing is ever let through unexplained.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import _native, scan_cu_single, scan_gated  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402

DEV = "cuda:0"


def _inputs(shape, dtype, seed, gate_scale=1.5):
    g = torch.Generator().manual_seed(seed)
    gate = (gate_scale * torch.randn(shape, generator=g)).to(dtype)
    x = torch.randn(shape, generator=g).to(dtype)
    dout = torch.randn(shape, generator=g).to(dtype)
    return gate, x, dout


def _check(oracle, got, want, want_other, rtol, atol, what):
    got = got.detach().float().cpu().numpy()
    assert np.isfinite(got).all(), what
    ok = oracle.within_rounding_envelope(got, want, want_other, rtol, atol)
    assert ok.all(), (
        f"{what}: {(~ok).sum()} of {ok.size} outside tolerance of both roundings, first at {np.argwhere(~ok)[0]}, "
        f"worst {np.abs(got - want)[~ok].max():.4g}")


def _check_all(oracle, rounding, rtol, atol, gate, x, dout, h, grad_gate, grad_x):
    g32, x32, d32 = gate.float().numpy(), x.float().numpy(), dout.float().numpy()
    h_dev = h.float().cpu().numpy()
    _check(oracle, h, oracle.gated_scan_fwd(g32, x32, rounding), oracle.gated_scan_fwd(g32, x32, rounding, True),
           rtol, atol, "h")
    # the backward is fed the stored (rounded) h, as the product path does
    want_gate, want_x = oracle.gated_scan_bwd(g32, x32, h_dev, d32, rounding)
    other_gate, other_x = oracle.gated_scan_bwd(g32, x32, h_dev, d32, rounding, True)
    _check(oracle, grad_x, want_x, other_x, rtol, atol, "grad_x")
    _check(oracle, grad_gate, want_gate, other_gate, rtol, atol, "grad_gate")


CASES = [
    ((2, 1, 5), None, None), ((1, 2, 64), None, None), ((3, 7, 64), (1, 8, 1), (1, 8, 1)),
    ((2, 200, 130), None, None), ((2, 777, 328), (2, 8, 3), (2, 8, 3)), ((4, 2000, 256), None, None),
    ((2, 1531, 200), (2, 16, 8, 3), (2, 16, 8, 3)), ((2, 1024, 768), (2, 32, 8), (2, 16, 4)),
    ((1, 4099, 128), (1, 32, 16), (1, 16, 16)), ((16, 2048, 512), None, None),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape,fwd_cfg,bwd_cfg", CASES)
def test_gated_scan_matches_oracle(oracle, dtype, shape, fwd_cfg, bwd_cfg):
    bf16 = dtype == torch.bfloat16
    if not bf16:  # fp32 kernels are one element per lane
        fwd_cfg = (1,) + tuple(fwd_cfg[1:]) if fwd_cfg else None
        bwd_cfg = (1,) + tuple(bwd_cfg[1:]) if bwd_cfg else None
    rounding = "bf16" if bf16 else "f32"
    rtol, atol = (1e-2, 1e-2) if bf16 else (1e-4, 1e-5)
    gate, x, dout = _inputs(shape, dtype, seed=sum(shape))
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h = ext.gated_scan_forward(gd, xd, fwd_cfg)
    grad_gate, grad_x = ext.gated_scan_backward(gd, xd, h, dd, bwd_cfg)
    ext.workspace_status()
    _check_all(oracle, rounding, rtol, atol, gate, x, dout, h, grad_gate, grad_x)


def test_every_chunking_gives_the_same_result():
    """fp32: results depend on the launch configuration only through the carries' rounding."""
    gate, x, dout = (t.to(DEV) for t in _inputs((2, 1200, 192), torch.float32, seed=5))
    ref_h = ext.gated_scan_forward(gate, x, (1, 8, 1))
    ref_g = ext.gated_scan_backward(gate, x, ref_h, dout, (1, 8, 1))
    for cfg in [(1, 8, 4), (1, 16, 8), (1, 16, 16), (1, 16, 8, 2), (1, 8, 16, 5)]:
        h = ext.gated_scan_forward(gate, x, cfg)
        torch.testing.assert_close(h, ref_h, rtol=1e-5, atol=1e-5)
        for got, want in zip(ext.gated_scan_backward(gate, x, ref_h, dout, cfg), ref_g):
            torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5)
    h32 = ext.gated_scan_forward(gate, x, (1, 32, 8))
    torch.testing.assert_close(h32, ref_h, rtol=1e-5, atol=1e-5)
    ext.workspace_status()


def test_equals_plain_scan_on_the_gpu_in_fp32():
    """The fused kernels against the unfused pipeline (torch elementwise ops + the plain scan)."""
    gate, x, dout = (t.to(DEV) for t in _inputs((3, 900, 160), torch.float32, seed=6))
    g1, x1 = gate.clone().requires_grad_(True), x.clone().requires_grad_(True)
    a = torch.sigmoid(g1)
    h_ref = scan_cu_single(a, x1 * torch.sqrt(1.0 - a * a))
    h_ref.backward(dout)
    g2, x2 = gate.clone().requires_grad_(True), x.clone().requires_grad_(True)
    h = scan_gated(g2, x2)
    h.backward(dout)
    torch.testing.assert_close(h, h_ref, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(x2.grad, x1.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(g2.grad, g1.grad, rtol=1e-4, atol=1e-5)


def test_saturated_gates_stay_finite():
    shape = (2, 300, 128)
    for dtype in (torch.bfloat16, torch.float32):
        gate, x, dout = _inputs(shape, dtype, seed=7)
        gate[:, 0::3] = 30.0   # alpha == 1 exactly in both dtypes
        gate[:, 1::3] = -120.0  # alpha == 0
        gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
        h = ext.gated_scan_forward(gd, xd)
        grad_gate, grad_x = ext.gated_scan_backward(gd, xd, h, dd)
        for t in (h, grad_gate, grad_x):
            assert torch.isfinite(t.float()).all()
        assert (grad_gate[:, 0::3] == 0).all() and (grad_x[:, 0::3] == 0).all()
        assert (grad_gate[:, 1::3] == 0).all()
        assert torch.equal(h[:, 1::3], xd[:, 1::3])  # alpha = 0: h = beta = x


def test_scaling_x_by_two_scales_everything_bit_exactly_at_the_headline_size():
    """Size-independent property at bs8 seq4096 d1024 bf16: powers of two commute with every
    rounding, so h(gate, 2x) == 2 h(gate, x) and grad_x(2 dout) == 2 grad_x(dout) exactly."""
    gate, x, dout = (t.to(DEV) for t in _inputs((8, 4096, 1024), torch.bfloat16, seed=8))
    h = ext.gated_scan_forward(gate, x)
    h2 = ext.gated_scan_forward(gate, 2 * x)
    assert torch.equal(h2, 2 * h)
    gg, gx = ext.gated_scan_backward(gate, x, h, dout)
    gg2, gx2 = ext.gated_scan_backward(gate, x, h, 2 * dout)
    assert torch.equal(gx2, 2 * gx) and torch.equal(gg2, 2 * gg)
    # and the gate's first row matters (beta[0] depends on it), unlike alpha[:,0] of the plain scan
    gate2 = gate.clone()
    gate2[:, 0] = -gate2[:, 0]
    assert not torch.equal(ext.gated_scan_forward(gate2, x)[:, 0], h[:, 0])
    ext.workspace_status()


def test_headline_size_against_oracle(oracle):
    shape = (8, 4096, 1024)
    gate, x, dout = _inputs(shape, torch.bfloat16, seed=9)
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h = ext.gated_scan_forward(gd, xd)
    grad_gate, grad_x = ext.gated_scan_backward(gd, xd, h, dd)
    ext.workspace_status()
    _check_all(oracle, "bf16", 1e-2, 1e-2, gate, x, dout, h, grad_gate, grad_x)


@pytest.mark.parametrize("shape", [(2, 8192, 1024), (64, 512, 1024), (5, 2048, 1024)])
def test_shapes_the_library_gives_two_workgroups_per_cu(oracle, shape):
    """The library's own choices where they are 8-wave workgroups: a forward of 8192 steps, a backward
    over many short sequences, a backward whose last round of 16-wave tiles would be ragged."""
    gate, x, dout = _inputs(shape, torch.bfloat16, seed=sum(shape))
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h = ext.gated_scan_forward(gd, xd)
    grad_gate, grad_x = ext.gated_scan_backward(gd, xd, h, dd)
    ext.workspace_status()
    _check_all(oracle, "bf16", 1e-2, 1e-2, gate, x, dout, h, grad_gate, grad_x)


def test_autograd_and_validation():
    gate, x, dout = (t.to(DEV) for t in _inputs((2, 50, 24), torch.bfloat16, seed=10))
    g1, x1 = gate.clone().requires_grad_(True), x.clone().requires_grad_(True)
    out = scan_gated(g1, x1)
    out.backward(dout)
    assert g1.grad.dtype == torch.bfloat16 and x1.grad.shape == x.shape
    assert scan_gated(gate[:, :0], x[:, :0]).shape == (2, 0, 24)
    with pytest.raises(RuntimeError):
        scan_gated(gate, x.float())
    with pytest.raises(RuntimeError):
        scan_gated(gate, x[:, :10])
    with pytest.raises(RuntimeError):
        scan_gated(gate.double(), x.double())


def test_c_abi_rejects_what_the_gated_kernels_do_not_cover():
    lib = _native.lib()
    t = torch.zeros(2, 64, 128, dtype=torch.bfloat16, device=DEV)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    sp = torch.cuda.current_stream().cuda_stream
    args = (2, 64, 128, ws.data_ptr(), ws.numel(), sp)
    p = t.data_ptr()
    bad_vec = ctypes.byref(_native.FssConfig(4, 8, 2, 0))
    assert lib.fss_gated_scan_fwd(_native.FSS_BF16, p, p, p, *args, bad_vec) == 5
    long_bwd = ctypes.byref(_native.FssConfig(2, 32, 2, 0))
    assert lib.fss_gated_scan_bwd(_native.FSS_BF16, p, p, p, p, p, p, *args, long_bwd) == 5
    assert lib.fss_gated_scan_bwd(_native.FSS_BF16, p, None, p, p, p, p, *args, None) == 1
    assert lib.fss_gated_scan_fwd(_native.FSS_BF16, p, p, None, *args, None) == 1
    assert lib.fss_gated_scan_fwd(_native.FSS_F32, p, p, p, *args, ctypes.byref(_native.FssConfig(2, 8, 2, 0))) == 5
    assert lib.fss_gated_scan_fwd(7, p, p, p, *args, None) == 5
    assert lib.fss_gated_scan_fwd(_native.FSS_BF16, p, p, p, 0, 64, 128, ws.data_ptr(), ws.numel(), sp, None) == 0
    assert lib.fss_workspace_bytes(8, 4096, 1024, _native.FSS_BF16, _native.FSS_GATED_BWD, None) <= \
        lib.fss_workspace_bytes_max(8, 4096, 1024)
