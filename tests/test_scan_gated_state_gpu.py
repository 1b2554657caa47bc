"""GPU tests of the gated scan with a state entering and leaving the sequence
(fss_gated_scan_fwd_state / fss_gated_scan_bwd_state, scan_gated_with_state).

The oracle is the pinned gating oracle around the pinned plain scan on a sequence one
step longer, as for the plain state scan: with beta'[0] = h_before, alpha'[1:] = alpha and
beta'[1:] = beta, the plain scan gives h'[1:] = h and h'[-1] = h_last; its backward with
dout'[0] = 0 and grad_h_last added to dout'[-1] gives grad_beta'[0] = grad_h_before and
grad_alpha'[1:], grad_beta'[1:], which the chain rule through the gating turns into
grad_gate and grad_x.  Tolerances are those of tests/test_scan_gated_gpu.py, as is the way
elements whose alpha sits on a bf16 rounding boundary are treated (two oracle evaluations,
every element within tolerance of the interval they span).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import scan_gated, scan_gated_with_state  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402

DEV = "cuda:0"


def _inputs(shape, dtype, seed, gate_scale=1.5):
    g = torch.Generator().manual_seed(seed)
    gate = (gate_scale * torch.randn(shape, generator=g)).to(dtype)
    x = torch.randn(shape, generator=g).to(dtype)
    dout = torch.randn(shape, generator=g).to(dtype)
    h0 = torch.randn(shape[0], shape[2], generator=g)
    g_last = torch.randn(shape[0], shape[2], generator=g)
    return gate, x, dout, h0, g_last


def _check(oracle, got, want, want_other, rtol, atol, what):
    got = got.detach().float().cpu().numpy()
    assert np.isfinite(got).all(), what
    ok = oracle.within_rounding_envelope(got, want, want_other, rtol, atol)
    assert ok.all(), (
        f"{what}: {(~ok).sum()} of {ok.size} outside tolerance of both roundings, worst {np.abs(got - want)[~ok].max():.4g}")


def _extended_gated_oracle(oracle, gate, x, dout, h0, g_last, rounding, other_rounding=False):
    """fp32 numpy in, (h, h_last, grad_gate, grad_x, grad_h_before) out."""
    bs, seq, d = gate.shape
    alpha, beta = oracle.gate_transform(gate, x, rounding, other_rounding)
    a_ext = np.concatenate([np.zeros((bs, 1, d), np.float32), alpha], axis=1)
    b_ext = np.concatenate([h0[:, None, :], beta], axis=1)
    h_ext = oracle.scan_fwd_f32(a_ext, b_ext)
    d_ext = np.concatenate([np.zeros((bs, 1, d), np.float32), dout], axis=1)
    d_ext[:, -1, :] += g_last
    ga_ext, gb_ext = oracle.scan_bwd_f32(a_ext, h_ext, d_ext)
    grad_alpha, grad_beta = ga_ext[:, 1:].astype(np.float64), gb_ext[:, 1:].astype(np.float64)
    a = alpha.astype(np.float64)
    om = np.maximum(1.0 - a * a, 0.0)
    s = np.sqrt(om)
    with np.errstate(divide="ignore", invalid="ignore"):
        a_over_s = np.where(om > 0.0, a / s, 0.0)
    grad_x = grad_beta * s
    grad_gate = (grad_alpha - grad_beta * x.astype(np.float64) * a_over_s) * a * (1.0 - a)
    return (h_ext[:, 1:], h_ext[:, -1], grad_gate.astype(np.float32), grad_x.astype(np.float32), gb_ext[:, 0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize(
    "shape,fwd_cfg,bwd_cfg",
    [((2, 1, 5), None, None), ((3, 7, 64), (1, 8, 1), (1, 8, 1)), ((2, 200, 130), None, None),
     ((2, 777, 328), (2, 8, 3), (2, 8, 3)), ((4, 2000, 256), None, None),
     ((2, 1531, 200), (2, 16, 8, 3), (2, 16, 8, 3)), ((2, 4099, 128), (1, 32, 16), (1, 16, 16))],
)
def test_gated_state_scan_matches_extended_oracle(oracle, dtype, shape, fwd_cfg, bwd_cfg):
    bf16 = dtype == torch.bfloat16
    if not bf16:  # fp32 kernels are one element per lane
        fwd_cfg = (1,) + tuple(fwd_cfg[1:]) if fwd_cfg else None
        bwd_cfg = (1,) + tuple(bwd_cfg[1:]) if bwd_cfg else None
    rounding = "bf16" if bf16 else "f32"
    rtol, atol = (1e-2, 1e-2) if bf16 else (1e-4, 1e-5)
    gate, x, dout, h0, g_last = _inputs(shape, dtype, seed=sum(shape) + 7)
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h, h_last = ext.gated_scan_forward_state(gd, xd, h0.to(DEV), fwd_cfg)
    gg, gx, gh0 = ext.gated_scan_backward_state(gd, xd, h, dd, h0.to(DEV), g_last.to(DEV), bwd_cfg)
    ext.workspace_status()
    args = (gate.float().numpy(), x.float().numpy(), dout.float().numpy(), h0.numpy(), g_last.numpy(), rounding)
    want = _extended_gated_oracle(oracle, *args)
    other = _extended_gated_oracle(oracle, *args, other_rounding=True)
    names = ("h", "h_last", "grad_gate", "grad_x", "grad_h_before")
    for name, got, ref, ref_other in zip(names, (h, h_last, gg, gx, gh0), want, other):
        _check(oracle, got, ref, ref_other, rtol, atol, name)


def test_without_state_equals_the_gated_scan():
    gate, x, dout, _, _ = _inputs((3, 900, 192), torch.bfloat16, seed=41)
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h, h_last = ext.gated_scan_forward_state(gd, xd, None)
    h_plain = ext.gated_scan_forward(gd, xd)
    assert torch.equal(h, h_plain)
    assert torch.equal(h_last.to(torch.bfloat16), h_plain[:, -1, :])
    gg, gx, gh0 = ext.gated_scan_backward_state(gd, xd, h, dd)
    gg_p, gx_p = ext.gated_scan_backward(gd, xd, h, dd)
    assert gh0 is None and torch.equal(gg, gg_p) and torch.equal(gx, gx_p)


@pytest.mark.parametrize("cut", [1, 257, 1000, 2999])
def test_two_gated_segments_equal_the_whole_sequence(cut):
    """fp32, so only the re-association of the carried state separates the two."""
    gate, x, dout, _, _ = _inputs((2, 3000, 192), torch.float32, seed=42)
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h = ext.gated_scan_forward(gd, xd)
    gg, gx = ext.gated_scan_backward(gd, xd, h, dd)
    g1, x1, d1 = (t[:, :cut].contiguous() for t in (gd, xd, dd))
    g2, x2, d2 = (t[:, cut:].contiguous() for t in (gd, xd, dd))
    h1, last1 = ext.gated_scan_forward_state(g1, x1, None)
    h2, last2 = ext.gated_scan_forward_state(g2, x2, last1)
    torch.testing.assert_close(torch.cat([h1, h2], 1), h, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(last2, h[:, -1, :], rtol=1e-5, atol=1e-5)
    gg2, gx2, gh = ext.gated_scan_backward_state(g2, x2, h2, d2, last1, None)
    gg1, gx1, none = ext.gated_scan_backward_state(g1, x1, h1, d1, None, gh)
    assert none is None
    torch.testing.assert_close(torch.cat([gx1, gx2], 1), gx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(torch.cat([gg1, gg2], 1), gg, rtol=1e-4, atol=1e-5)
    ext.workspace_status()


def test_scan_gated_with_state_autograd():
    """Gradients through both outputs and into all three inputs, against autograd through a float64 loop."""
    g = torch.Generator().manual_seed(43)
    bs, seq, d = 2, 70, 48
    gate = torch.randn(bs, seq, d, generator=g)
    x = torch.randn(bs, seq, d, generator=g)
    h0 = torch.randn(bs, d, generator=g)
    w_h = torch.randn(bs, seq, d, generator=g)
    w_last = torch.randn(bs, d, generator=g)

    def loss_ref(gt, xt, s):
        a = torch.sigmoid(gt)
        b = xt * torch.sqrt(1 - a * a)
        hs, cur = [], s
        for t in range(seq):
            cur = a[:, t] * cur + b[:, t]
            hs.append(cur)
        return (torch.stack(hs, 1) * w_h).sum() + (cur * w_last).sum()

    gr, xr, sr = (t.clone().double().requires_grad_(True) for t in (gate, x, h0))
    loss_ref(gr, xr, sr).backward()

    gdv, xdv, sdv = (t.clone().to(DEV).requires_grad_(True) for t in (gate, x, h0))
    h, h_last = scan_gated_with_state(gdv, xdv, sdv)
    ((h * w_h.to(DEV)).sum() + (h_last * w_last.to(DEV)).sum()).backward()
    torch.testing.assert_close(gdv.grad.cpu().double(), gr.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(xdv.grad.cpu().double(), xr.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(sdv.grad.cpu().double(), sr.grad, rtol=1e-4, atol=1e-5)
    # and the plain gated entry point is untouched by all this
    assert scan_gated(gate.to(DEV), x.to(DEV)).shape == (bs, seq, d)


def test_gated_state_error_paths():
    gate, x, dout, h0, _ = _inputs((2, 16, 64), torch.float32, seed=44)
    gd, xd = gate.to(DEV), x.to(DEV)
    with pytest.raises((RuntimeError, ValueError)):
        ext.gated_scan_forward_state(gd, xd, h0.to(DEV)[:, :32])  # wrong state shape
    with pytest.raises((RuntimeError, ValueError)):
        ext.gated_scan_forward_state(gd, xd, h0.to(DEV).to(torch.bfloat16))  # states are fp32
