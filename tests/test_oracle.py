"""Pins the CPU oracle (oracle/scan_oracle.c) before anything is compared with it.

Each check is chosen so that a plausible mistake fails it: a dropped carry, an
off-by-one in the alpha shift of the backward, a wrong sign, a transposed axis,
alpha[:,0] leaking into the result, truncation instead of round-to-nearest-even.
None of them retypes the oracle's loop: they use closed forms, an explicit
sum-of-products, autograd through an independent torch loop, the reverse-scan
identity, the golden vectors written by the reference's own C++ CPU scan, and
that library itself where it has been built.
"""
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ref_cpu_vectors.npz")


def _rand(rng, shape, dtype=np.float32):
    return rng.standard_normal(shape).astype(dtype)


# ----------------------------------------------------------------- forward


def test_fwd_alpha_one_is_cumsum(oracle):
    rng = np.random.default_rng(0)
    beta = _rand(rng, (3, 37, 11), np.float64)
    h = oracle.scan_fwd_f64(np.ones_like(beta), beta)
    np.testing.assert_allclose(h, np.cumsum(beta, axis=1), rtol=1e-12, atol=1e-12)


def test_fwd_alpha_zero_is_beta(oracle):
    rng = np.random.default_rng(1)
    beta = _rand(rng, (2, 9, 5))
    for fused in (False, True):
        h = oracle.scan_fwd_f32(np.zeros_like(beta), beta, fused=fused)
        np.testing.assert_array_equal(h, beta)


def test_fwd_constant_alpha_geometric_series(oracle):
    c, T = 0.75, 40
    alpha = np.full((1, T, 4), c, np.float64)
    beta = np.ones((1, T, 4), np.float64)
    h = oracle.scan_fwd_f64(alpha, beta)
    t = np.arange(T, dtype=np.float64)
    expect = (1.0 - c ** (t + 1)) / (1.0 - c)
    np.testing.assert_allclose(h[0, :, 2], expect, rtol=1e-13)


def test_fwd_closed_form_survey_values(oracle):
    alpha = np.full((2, 4, 8), 0.5, np.float32)
    beta = np.ones((2, 4, 8), np.float32)
    h = oracle.scan_fwd_f32(alpha, beta)
    np.testing.assert_array_equal(h[1, :, 3], np.array([1, 1.5, 1.75, 1.875], np.float32))
    ga, gb = oracle.scan_bwd_f32(alpha, h, np.ones_like(h))
    np.testing.assert_array_equal(gb[0, :, 0], np.array([1.875, 1.75, 1.5, 1.0], np.float32))
    np.testing.assert_array_equal(ga[0, :, 0], np.array([0.0, 1.75, 2.25, 1.75], np.float32))


def _brute_force_fwd(alpha, beta):
    """h_t = sum_{s<=t} (prod_{r=s+1..t} a_r) b_s, written as the explicit sum."""
    bs, T, d = alpha.shape
    h = np.zeros_like(alpha)
    for t in range(T):
        acc = np.zeros((bs, d), alpha.dtype)
        for s in range(t + 1):
            prod = np.ones((bs, d), alpha.dtype)
            for r in range(s + 1, t + 1):
                prod = prod * alpha[:, r, :]
            acc = acc + prod * beta[:, s, :]
        h[:, t, :] = acc
    return h


@pytest.mark.parametrize("shape", [(1, 1, 3), (2, 2, 4), (2, 3, 1), (3, 9, 5)])
def test_fwd_brute_force_sum_of_products(oracle, shape):
    rng = np.random.default_rng(2)
    alpha, beta = _rand(rng, shape, np.float64), _rand(rng, shape, np.float64)
    np.testing.assert_allclose(
        oracle.scan_fwd_f64(alpha, beta), _brute_force_fwd(alpha, beta), rtol=1e-11, atol=1e-12
    )
    # the fp32 variants follow the fp64 one to fp32 accuracy
    h32 = oracle.scan_fwd_f32(alpha.astype(np.float32), beta.astype(np.float32))
    h64 = oracle.scan_fwd_f64(alpha.astype(np.float32).astype(np.float64), beta.astype(np.float32).astype(np.float64))
    np.testing.assert_allclose(h32, h64, rtol=2e-5, atol=2e-5)


def test_fwd_ignores_alpha_row_zero(oracle):
    rng = np.random.default_rng(3)
    alpha, beta = _rand(rng, (2, 6, 4)), _rand(rng, (2, 6, 4))
    h0 = oracle.scan_fwd_f32(alpha, beta)
    alpha2 = alpha.copy()
    alpha2[:, 0, :] = np.nan
    np.testing.assert_array_equal(oracle.scan_fwd_f32(alpha2, beta), h0)
    bits = oracle.f32_to_bf16_bits
    hb0 = oracle.scan_fwd_bf16(bits(alpha), bits(beta))
    np.testing.assert_array_equal(oracle.scan_fwd_bf16(bits(alpha2), bits(beta)), hb0)


def test_fwd_channels_and_batches_are_independent(oracle):
    rng = np.random.default_rng(4)
    alpha, beta = _rand(rng, (3, 12, 7)), _rand(rng, (3, 12, 7))
    h = oracle.scan_fwd_f32(alpha, beta)
    perm_c, perm_b = rng.permutation(7), rng.permutation(3)
    h2 = oracle.scan_fwd_f32(alpha[perm_b][:, :, perm_c], beta[perm_b][:, :, perm_c])
    np.testing.assert_array_equal(h2, h[perm_b][:, :, perm_c])
    # time is the middle axis: scanning a transposed copy must differ
    assert not np.allclose(
        oracle.scan_fwd_f32(alpha.transpose(0, 2, 1).copy(), beta.transpose(0, 2, 1).copy()).transpose(0, 2, 1), h
    )


def test_fused_and_unfused_differ_only_by_rounding(oracle):
    rng = np.random.default_rng(5)
    alpha, beta = _rand(rng, (2, 200, 16)) * 0.9, _rand(rng, (2, 200, 16))
    a = oracle.scan_fwd_f32(alpha, beta, fused=False)
    b = oracle.scan_fwd_f32(alpha, beta, fused=True)
    assert not np.array_equal(a, b)  # the switch does something
    ref = oracle.scan_fwd_f64(alpha.astype(np.float64), beta.astype(np.float64))
    scale = np.abs(ref).max()
    assert np.abs(a - ref).max() / scale < 1e-5
    assert np.abs(b - ref).max() / scale < 1e-5


# ---------------------------------------------------------------- backward


def _torch_loop(alpha, beta):
    """Independent statement of the forward in torch (autograd supplies the backward)."""
    hs = [beta[:, 0, :]]
    for t in range(1, alpha.shape[1]):
        hs.append(hs[-1] * alpha[:, t, :] + beta[:, t, :])
    return torch.stack(hs, dim=1)


@pytest.mark.parametrize("shape", [(1, 1, 2), (2, 2, 3), (2, 3, 3), (3, 17, 6)])
def test_bwd_matches_autograd_fp64(oracle, shape):
    g = torch.Generator().manual_seed(6)
    alpha = torch.randn(shape, dtype=torch.float64, generator=g, requires_grad=True)
    beta = torch.randn(shape, dtype=torch.float64, generator=g, requires_grad=True)
    dout = torch.randn(shape, dtype=torch.float64, generator=g)
    h = _torch_loop(alpha, beta)
    h.backward(dout)
    np.testing.assert_allclose(oracle.scan_fwd_f64(alpha.detach().numpy(), beta.detach().numpy()), h.detach().numpy(), rtol=1e-12, atol=1e-12)
    ga, gb = oracle.scan_bwd_f64(alpha.detach().numpy(), h.detach().numpy(), dout.numpy())
    np.testing.assert_allclose(gb, beta.grad.numpy(), rtol=1e-11, atol=1e-12)
    # seq == 1 never touches alpha: autograd leaves its grad unset, the scan returns zeros
    alpha_grad = alpha.grad.numpy() if alpha.grad is not None else np.zeros(shape)
    np.testing.assert_allclose(ga, alpha_grad, rtol=1e-11, atol=1e-12)
    assert np.all(ga[:, 0, :] == 0.0)


def test_bwd_is_forward_of_flipped_shifted_inputs(oracle):
    """grad_beta = flip(scan(flip(shift(alpha)), flip(dout))): reduces bwd to the pinned fwd."""
    rng = np.random.default_rng(7)
    shape = (2, 23, 5)
    alpha, beta, dout = (_rand(rng, shape, np.float64) for _ in range(3))
    h = oracle.scan_fwd_f64(alpha, beta)
    ga, gb = oracle.scan_bwd_f64(alpha, h, dout)
    shifted = np.zeros_like(alpha)
    shifted[:, :-1, :] = alpha[:, 1:, :]  # a'_t = alpha_{t+1}
    gb2 = oracle.scan_fwd_f64(shifted[:, ::-1, :].copy(), dout[:, ::-1, :].copy())[:, ::-1, :]
    np.testing.assert_allclose(gb, gb2, rtol=1e-13, atol=1e-13)
    expect_ga = np.zeros_like(ga)
    expect_ga[:, 1:, :] = gb[:, 1:, :] * h[:, :-1, :]
    np.testing.assert_allclose(ga, expect_ga, rtol=1e-13, atol=1e-13)


def test_bwd_finite_differences(oracle):
    rng = np.random.default_rng(8)
    shape = (1, 6, 2)
    alpha, beta, dout = (_rand(rng, shape, np.float64) for _ in range(3))
    h = oracle.scan_fwd_f64(alpha, beta)
    ga, gb = oracle.scan_bwd_f64(alpha, h, dout)
    eps = 1e-6
    for t in range(shape[1]):
        for which, grad in (("a", ga), ("b", gb)):
            ap, bp = alpha.copy(), beta.copy()
            am, bm = alpha.copy(), beta.copy()
            (ap if which == "a" else bp)[0, t, 1] += eps
            (am if which == "a" else bm)[0, t, 1] -= eps
            fd = ((oracle.scan_fwd_f64(ap, bp) - oracle.scan_fwd_f64(am, bm)) * dout).sum() / (2 * eps)
            assert abs(fd - grad[0, t, 1]) < 1e-6, (which, t)


# -------------------------------------------------------------------- bf16


def test_bf16_rounding_matches_torch(oracle):
    g = torch.Generator().manual_seed(9)
    x = torch.randn(100000, generator=g) * torch.logspace(-20, 20, 100000)
    x[:7] = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 1.00390625, 1.01171875, 3.3895314e38])
    bits = oracle.f32_to_bf16_bits(x.numpy())
    expect = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(bits, expect)
    np.testing.assert_array_equal(oracle.bf16_bits_to_f32(bits), x.to(torch.bfloat16).float().numpy())
    nan_bits = oracle.f32_to_bf16_bits(np.array([np.nan], np.float32))
    assert np.isnan(oracle.bf16_bits_to_f32(nan_bits))[0]


def test_bf16_variants_follow_fp32(oracle):
    rng = np.random.default_rng(10)
    shape = (2, 50, 8)
    a_bits = oracle.f32_to_bf16_bits(1.0 / (1.0 + np.exp(-_rand(rng, shape))))
    b_bits = oracle.f32_to_bf16_bits(_rand(rng, shape))
    d_bits = oracle.f32_to_bf16_bits(_rand(rng, shape))
    a, b, do = (oracle.bf16_bits_to_f32(x) for x in (a_bits, b_bits, d_bits))
    h32 = oracle.scan_fwd_f32(a, b)
    np.testing.assert_array_equal(oracle.scan_fwd_bf16_f32out(a_bits, b_bits), h32)
    h_bits = oracle.scan_fwd_bf16(a_bits, b_bits)
    # storing bf16 never feeds back into the carry: output == round(fp32 carry)
    np.testing.assert_array_equal(h_bits, oracle.f32_to_bf16_bits(h32))
    ga32, gb32 = oracle.scan_bwd_f32(a, h32, do)
    ga_o, gb_o = oracle.scan_bwd_bf16_f32out(a_bits, h32, d_bits)
    np.testing.assert_array_equal(ga_o, ga32)
    np.testing.assert_array_equal(gb_o, gb32)
    ga_bits, gb_bits = oracle.scan_bwd_bf16(a_bits, h_bits, d_bits)
    np.testing.assert_array_equal(gb_bits, oracle.f32_to_bf16_bits(gb32))
    ga_saved, _ = oracle.scan_bwd_f32(a, oracle.bf16_bits_to_f32(h_bits), do)
    np.testing.assert_array_equal(ga_bits, oracle.f32_to_bf16_bits(ga_saved))


# ----------------------------------- the reference's own C++ CPU implementation


def test_golden_vectors_from_reference_cpu_scan(oracle):
    z = np.load(GOLDEN)
    keys = sorted({k.split("/")[0] for k in z.files})
    assert "2x33x24" in keys and "const" in keys
    for key in keys:
        alpha, beta, dout = z[f"{key}/alpha"], z[f"{key}/beta"], z[f"{key}/dout"]
        h = oracle.scan_fwd_f32(alpha, beta)
        np.testing.assert_array_equal(h, z[f"{key}/h"], err_msg=key)
        ga, gb = oracle.scan_bwd_f32(alpha, h, dout)
        np.testing.assert_array_equal(gb, z[f"{key}/gbeta"], err_msg=key)
        np.testing.assert_array_equal(ga, z[f"{key}/galpha"], err_msg=key)


def test_against_compiled_reference_header(oracle):
    if not oracle.ref_available():
        pytest.skip("oracle/_ref is not built on this machine")
    rng = np.random.default_rng(11)
    for shape in oracle.ref_shapes():
        alpha, beta, dout = (_rand(rng, shape) for _ in range(3))
        h_ref = oracle.ref_scan_fwd(alpha, beta)
        h = oracle.scan_fwd_f32(alpha, beta)
        np.testing.assert_array_equal(h, h_ref, err_msg=str(shape))
        ga_ref, gb_ref = oracle.ref_scan_bwd(alpha, h_ref, dout)
        ga, gb = oracle.scan_bwd_f32(alpha, h, dout)
        np.testing.assert_array_equal(gb, gb_ref, err_msg=str(shape))
        np.testing.assert_array_equal(ga, ga_ref, err_msg=str(shape))


def test_torch_loop_baseline_equals_c_oracle(oracle):
    """The CPU baseline timed by the bench (oracle/torch_loop.py) computes what the C oracle computes."""
    from oracle.torch_loop import torch_loop_bwd, torch_loop_fwd

    g = torch.Generator().manual_seed(12)
    for shape in [(1, 1, 3), (2, 2, 4), (3, 40, 9)]:
        alpha = torch.randn(shape, generator=g).to(torch.bfloat16)
        beta = torch.randn(shape, generator=g).to(torch.bfloat16)
        dout = torch.randn(shape, generator=g).to(torch.bfloat16)
        bits = oracle.torch_bf16_to_bits
        h = torch_loop_fwd(alpha, beta)
        h_c = oracle.scan_fwd_bf16_f32out(bits(alpha), bits(beta))
        np.testing.assert_array_equal(h.numpy(), h_c)
        ga, gb = torch_loop_bwd(alpha, h, dout)
        ga_c, gb_c = oracle.scan_bwd_bf16_f32out(bits(alpha), h_c, bits(dout))
        np.testing.assert_array_equal(gb.numpy(), gb_c)
        np.testing.assert_array_equal(ga.numpy(), ga_c)
