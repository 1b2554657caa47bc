"""Pins the gated-scan oracle (oracle.gate_transform / gated_scan_fwd / gated_scan_bwd).

The scans underneath are pinned in test_oracle.py.  What is new here is elementwise:
alpha = sigmoid(gate), beta = x*sqrt(1-alpha^2), and the chain rule back through them.
Checked against torch's own sigmoid/sqrt, against autograd through an independent
float64 loop, closed forms, saturation, and finite differences -- none of which
retypes the oracle's formulas.
"""
import numpy as np
import pytest
import torch


def _rand(rng, shape, scale=1.0):
    return (scale * rng.standard_normal(shape)).astype(np.float32)


def test_gate_transform_matches_torch_ops(oracle):
    rng = np.random.default_rng(10)
    gate, x = _rand(rng, (3, 17, 9), 2.0), _rand(rng, (3, 17, 9))
    alpha, beta = oracle.gate_transform(gate, x, "f32")
    a_t = torch.sigmoid(torch.from_numpy(gate).double())
    b_t = torch.from_numpy(x).double() * torch.sqrt(1.0 - a_t * a_t)
    np.testing.assert_allclose(alpha, a_t.numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(beta, b_t.numpy(), rtol=2e-6, atol=1e-7)


def test_gate_transform_bf16_rounds_alpha_then_uses_the_rounded_value(oracle):
    rng = np.random.default_rng(11)
    gate = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(_rand(rng, (2, 64, 33), 2.0)))
    x = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(_rand(rng, (2, 64, 33))))
    alpha, beta = oracle.gate_transform(gate, x, "bf16")
    # alpha is torch's bf16 sigmoid of the same bf16 gate (fp32 inside, rounded once)
    a_t = torch.sigmoid(torch.from_numpy(gate).to(torch.bfloat16)).float().numpy()
    assert (alpha == a_t).mean() > 0.999
    np.testing.assert_allclose(alpha, a_t, rtol=2 ** -7, atol=0)
    # beta is computed from the ROUNDED alpha: exact identity beta = bf16(x * sqrt(1 - alpha^2))
    want = torch.from_numpy(x.astype(np.float64) * np.sqrt(1.0 - alpha.astype(np.float64) ** 2)).to(torch.bfloat16)
    np.testing.assert_array_equal(beta, want.float().numpy())
    # both are bf16 values
    for t in (alpha, beta):
        np.testing.assert_array_equal(t, oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(t)))


def test_gated_fwd_closed_forms(oracle):
    bs, seq, d = 2, 400, 3
    ones = np.ones((bs, seq, d), np.float32)
    # gate = 0: alpha = 1/2, s = sqrt(3)/2; constant x = 1 -> h[t] = 2 s (1 - 2^-(t+1))
    h = oracle.gated_scan_fwd(np.zeros_like(ones), ones, "f32")
    t = np.arange(seq, dtype=np.float64)[None, :, None]
    np.testing.assert_allclose(h, np.sqrt(3.0) * (1.0 - 0.5 ** (t + 1)) * np.ones((bs, 1, d)), rtol=1e-6)
    # saturated high: alpha = 1 exactly, beta = 0 -> h stays 0
    h = oracle.gated_scan_fwd(40.0 * ones, ones, "f32")
    np.testing.assert_array_equal(h, np.zeros_like(h))
    # saturated low: alpha -> 0, beta = x -> h = x
    rng = np.random.default_rng(12)
    x = _rand(rng, (bs, seq, d))
    np.testing.assert_allclose(oracle.gated_scan_fwd(-100.0 * ones, x, "f32"), x, rtol=0, atol=0)


@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 5, 3), (3, 41, 7)])
def test_gated_bwd_matches_autograd_through_an_independent_loop(oracle, shape):
    rng = np.random.default_rng(13)
    gate, x, dout = _rand(rng, shape, 1.5), _rand(rng, shape), _rand(rng, shape)
    g_t = torch.from_numpy(gate).double().requires_grad_(True)
    x_t = torch.from_numpy(x).double().requires_grad_(True)
    a = torch.sigmoid(g_t)
    b = x_t * torch.sqrt(1.0 - a * a)
    hs, cur = [], torch.zeros(shape[0], shape[2], dtype=torch.float64)
    for t in range(shape[1]):
        cur = a[:, t] * cur + b[:, t]
        hs.append(cur)
    h_t = torch.stack(hs, 1)
    (h_t * torch.from_numpy(dout).double()).sum().backward()
    h = oracle.gated_scan_fwd(gate, x, "f32")
    np.testing.assert_allclose(h, h_t.detach().numpy(), rtol=1e-5, atol=1e-6)
    grad_gate, grad_x = oracle.gated_scan_bwd(gate, x, h, dout, "f32")
    np.testing.assert_allclose(grad_x, x_t.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(grad_gate, g_t.grad.numpy(), rtol=1e-4, atol=1e-5)


def test_gated_bwd_finite_differences(oracle):
    rng = np.random.default_rng(14)
    shape = (1, 6, 2)
    gate, x, dout = (rng.standard_normal(shape).astype(np.float32) for _ in range(3))

    def loss(g, xx):
        return float((oracle.gated_scan_fwd(g, xx, "f32").astype(np.float64) * dout).sum())

    h = oracle.gated_scan_fwd(gate, x, "f32")
    grad_gate, grad_x = oracle.gated_scan_bwd(gate, x, h, dout, "f32")
    eps = 1e-2
    for idx in [(0, 0, 0), (0, 3, 1), (0, 5, 0)]:
        for arr, grad, which in ((gate, grad_gate, 0), (x, grad_x, 1)):
            hi, lo = arr.copy(), arr.copy()
            hi[idx] += eps
            lo[idx] -= eps
            fd = (loss(hi, x) - loss(lo, x)) / (2 * eps) if which == 0 else (loss(gate, hi) - loss(gate, lo)) / (2 * eps)
            assert abs(fd - grad[idx]) <= 2e-3 + 2e-3 * abs(fd), (idx, which, fd, grad[idx])


def test_gated_bwd_where_alpha_saturates(oracle):
    """alpha == 1 exactly: s = 0, the x term is dropped, everything stays finite."""
    shape = (1, 8, 2)
    gate = np.full(shape, 40.0, np.float32)
    gate[:, ::2] = 0.0
    rng = np.random.default_rng(15)
    x, dout = _rand(rng, shape), _rand(rng, shape)
    h = oracle.gated_scan_fwd(gate, x, "f32")
    grad_gate, grad_x = oracle.gated_scan_bwd(gate, x, h, dout, "f32")
    assert np.isfinite(grad_gate).all() and np.isfinite(grad_x).all()
    assert (grad_gate[:, 1::2] == 0).all() and (grad_x[:, 1::2] == 0).all()


@pytest.mark.parametrize("rounding,dtype", [("f32", torch.float32), ("bf16", torch.bfloat16)])
def test_torch_gated_baseline_equals_numpy_oracle(oracle, rounding, dtype):
    from oracle.torch_loop import torch_gated_bwd, torch_gated_fwd

    g = torch.Generator().manual_seed(16)
    gate = (1.5 * torch.randn(2, 50, 12, generator=g)).to(dtype)
    x, dout = torch.randn(2, 50, 12, generator=g).to(dtype), torch.randn(2, 50, 12, generator=g).to(dtype)
    alpha, h = torch_gated_fwd(gate, x)
    g32, x32, d32 = gate.float().numpy(), x.float().numpy(), dout.float().numpy()
    a_or, _ = oracle.gate_transform(g32, x32, rounding)
    if rounding == "f32":
        np.testing.assert_allclose(alpha.numpy(), a_or, rtol=3e-7, atol=0)  # fp32 sigmoid against float64
    else:
        # one rounding to bf16 on either side: identical unless an fp32 ulp decides the boundary (not in this draw)
        np.testing.assert_array_equal(alpha.float().numpy(), a_or)
    np.testing.assert_allclose(h.numpy(), oracle.gated_scan_fwd(g32, x32, rounding), rtol=1e-5, atol=1e-5)
    gg, gx = torch_gated_bwd(alpha, x, h, dout)
    want_gg, want_gx = oracle.gated_scan_bwd(g32, x32, h.numpy(), d32, rounding)
    np.testing.assert_allclose(gx.numpy(), want_gx, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gg.numpy(), want_gg, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("rounding", ["bf16", "f16"])
def test_ambiguous_roundings_of_alpha(oracle, rounding):
    """gate_alpha_variants: the elements it calls ambiguous are exactly those whose sigmoid sits on
    a midpoint between two storage values (to a few fp32 ulps); the other rounding differs from
    the nearest one there by one storage step and nowhere else.  Pinned on gates constructed from
    the midpoints themselves (logit of the midpoint), without using the oracle's own formula."""
    if rounding == "bf16":  # pairs of adjacent storage values in [0.25, 1)
        bits = np.arange(0x3E80, 0x3F7F, dtype=np.uint16)
        lo, hi = (oracle.bf16_bits_to_f32(b).astype(np.float64) for b in (bits, bits + 1))
    else:
        bits = np.arange(0x3400, 0x3BFF, 7, dtype=np.uint16)
        lo, hi = (b.view(np.float16).astype(np.float64) for b in (bits, bits + 1))
    mid = 0.5 * (lo + hi)
    gate_at_mid = np.log(mid / (1.0 - mid))  # float64 gates: sigmoid lands on the midpoint to ~1e-16
    alpha, other, ambiguous = oracle.gate_alpha_variants(gate_at_mid.reshape(1, -1, 1), rounding)
    assert ambiguous.all()
    a, o = alpha.ravel().astype(np.float64), other.ravel().astype(np.float64)
    assert (np.minimum(a, o) == lo).all() and (np.maximum(a, o) == hi).all()
    # a quarter of a storage step away from the midpoint nothing is ambiguous, and both variants agree
    quarter = lo + 0.25 * (hi - lo)
    alpha, other, ambiguous = oracle.gate_alpha_variants(np.log(quarter / (1.0 - quarter)).reshape(1, -1, 1), rounding)
    assert not ambiguous.any()
    np.testing.assert_array_equal(alpha, other)
    np.testing.assert_array_equal(alpha.ravel(), lo.astype(np.float32))
    # random gates: the ambiguous share is the window over the storage step (a few in 10^4)
    rng = np.random.default_rng(21)
    gate = (1.5 * rng.standard_normal((4, 500, 100))).astype(np.float32)
    alpha, other, ambiguous = oracle.gate_alpha_variants(gate, rounding)
    assert 0 < ambiguous.mean() < (2e-3 if rounding == "bf16" else 2e-2)
    changed = alpha != other
    np.testing.assert_array_equal(changed, ambiguous & changed)
    # fp32 storage: never ambiguous
    assert not oracle.gate_alpha_variants(gate, "f32")[2].any()


def test_rounding_envelope_is_the_plain_tolerance_where_the_variants_agree(oracle):
    want = np.array([1.0, -2.0, 0.0, 5.0], np.float32)
    other = np.array([1.0, -2.0, 0.0, 6.0], np.float32)
    got = np.array([1.02, -2.05, 0.011, 5.5], np.float32)
    ok = oracle.within_rounding_envelope(got, want, other, 1e-2, 1e-2)
    np.testing.assert_array_equal(ok, [True, False, False, True])
    got = np.array([1.0, -2.0, 0.0, 6.2], np.float32)
    np.testing.assert_array_equal(oracle.within_rounding_envelope(got, want, other, 1e-2, 1e-2), [True, True, True, False])
    # the other-rounding evaluation equals the nearest one when no element is ambiguous
    rng = np.random.default_rng(22)
    gate, x = _rand(rng, (1, 30, 4)), _rand(rng, (1, 30, 4))
    if not oracle.gate_alpha_variants(gate, "bf16")[2].any():
        np.testing.assert_array_equal(oracle.gated_scan_fwd(gate, x, "bf16"), oracle.gated_scan_fwd(gate, x, "bf16", True))
