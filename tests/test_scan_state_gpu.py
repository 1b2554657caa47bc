"""GPU tests of the scans with a state entering and leaving the sequence
(fss_scan_fwd_state / fss_scan_bwd_state, scan_with_state).

The oracle is the already pinned plain scan on a sequence one step longer: with
beta'[0] = h_before, alpha'[1:] = alpha and beta'[1:] = beta, the plain scan gives
h'[1:] = h and h'[-1] = h_last; its backward with dout'[0] = 0 and grad_h_last added
to dout'[-1] gives grad_beta'[0] = grad_h_before and grad_alpha'[1] = grad_alpha[0].
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import scan_cu, scan_with_state  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402
from fast_sequential_scan_amd.workloads import make_inputs  # noqa: E402

DEV = "cuda:0"


def _extended_oracle(oracle, alpha, beta, dout, h0, g_last):
    """All in fp32 numpy; alpha/beta/dout already hold the storage dtype's values."""
    bs, seq, d = alpha.shape
    a_ext = np.concatenate([np.zeros((bs, 1, d), np.float32), alpha], axis=1)
    b_ext = np.concatenate([h0[:, None, :], beta], axis=1)
    h_ext = oracle.scan_fwd_f32(a_ext, b_ext)
    d_ext = np.concatenate([np.zeros((bs, 1, d), np.float32), dout], axis=1)
    d_ext[:, -1, :] += g_last
    ga_ext, gb_ext = oracle.scan_bwd_f32(a_ext, h_ext, d_ext)
    return h_ext[:, 1:], h_ext[:, -1], ga_ext[:, 1:], gb_ext[:, 1:], gb_ext[:, 0]


def _close(got, want, rtol, atol, what):
    got = got.detach().float().cpu().numpy()
    bad = ~(np.abs(got - want) <= atol + rtol * np.abs(want))
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} off, worst {np.abs(got - want).max():.4g}"


@pytest.mark.parametrize("dtype,rtol,atol", [(torch.bfloat16, 1e-2, 1e-2), (torch.float32, 1e-4, 1e-5)])
@pytest.mark.parametrize(
    "shape,config",
    [((2, 1, 5), None), ((3, 7, 64), (1, 8, 1)), ((2, 200, 130), None), ((2, 777, 328), (2, 8, 3)),
     ((4, 2000, 256), None), ((2, 1531, 200), (2, 16, 8, 3))],
)
def test_state_scan_matches_extended_oracle(oracle, dtype, rtol, atol, shape, config):
    alpha, beta, dout = make_inputs("sigmoid", *shape, dtype=dtype, seed=91)
    g = torch.Generator().manual_seed(92)
    h0 = torch.randn(shape[0], shape[2], generator=g)
    g_last = torch.randn(shape[0], shape[2], generator=g)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h, h_last = ext.scan_forward_state(a, b, h0.to(DEV), config)
    ga, gb, gh0 = ext.scan_backward_state(a, h, do, h0.to(DEV), g_last.to(DEV), config)
    ext.workspace_status()
    # the backward is fed the stored (rounded) h, as the product path does; the oracle its own fp32 h
    want = _extended_oracle(oracle, alpha.float().numpy(), beta.float().numpy(), dout.float().numpy(),
                            h0.numpy(), g_last.numpy())
    for name, got, ref in zip(("h", "h_last", "grad_alpha", "grad_beta", "grad_h_before"),
                              (h, h_last, ga, gb, gh0), want):
        _close(got, ref, rtol, atol, name)


@pytest.mark.parametrize("shape,recipe", [((3, 900, 192), "hawk"), ((8, 4096, 1024), "near_one")], ids=["small", "two_round_forward"])
def test_without_state_equals_plain_scan(shape, recipe):
    """Bit for bit: the scan with states cuts the sequence where the plain scan does - also where the
    library gives the forward two column tiles per workgroup (the second shape; alphas near 1 there,
    so that a different tiling would show)."""
    alpha, beta, dout = make_inputs(recipe, *shape, seed=93)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h, h_last = ext.scan_forward_state(a, b, None)
    h_plain = ext.scan_forward_half(a, b)
    assert torch.equal(h, h_plain)
    # h_last is the un-rounded last state: it rounds to the last row of h
    assert torch.equal(h_last.to(torch.bfloat16), h_plain[:, -1, :])
    ga, gb, gh0 = ext.scan_backward_state(a, h, do)
    ga_p, gb_p = ext.scan_backward_half(a, h, do)
    assert gh0 is None and torch.equal(ga, ga_p) and torch.equal(gb, gb_p)
    # NaN in alpha[:, 0] still does not matter without an incoming state
    a2 = a.clone()
    a2[:, 0, :] = float("nan")
    assert torch.equal(ext.scan_forward_state(a2, b, None)[0], h_plain)


@pytest.mark.parametrize("cut", [1, 257, 1000, 2999])
def test_two_segments_equal_the_whole_sequence(cut):
    """Forward: h_last of the first segment as h_before of the second.  Backward: grad_h_before of
    the second as grad_h_last of the first.  fp32, so only carry re-association separates the two."""
    alpha, beta, dout = make_inputs("sigmoid", 2, 3000, 192, dtype=torch.float32, seed=94)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext.scan_forward(a, b)
    ga, gb = ext.scan_backward(a, h, do)
    h1, last1 = ext.scan_forward_state(a[:, :cut].contiguous(), b[:, :cut].contiguous(), None)
    h2, last2 = ext.scan_forward_state(a[:, cut:].contiguous(), b[:, cut:].contiguous(), last1)
    torch.testing.assert_close(torch.cat([h1, h2], 1), h, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(last2, h[:, -1, :], rtol=1e-5, atol=1e-5)
    ga2, gb2, gh = ext.scan_backward_state(a[:, cut:].contiguous(), h2, do[:, cut:].contiguous(), last1, None)
    ga1, gb1, none = ext.scan_backward_state(a[:, :cut].contiguous(), h1, do[:, :cut].contiguous(), None, gh)
    assert none is None
    torch.testing.assert_close(torch.cat([gb1, gb2], 1), gb, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(torch.cat([ga1, ga2], 1), ga, rtol=1e-4, atol=1e-5)
    ext.workspace_status()


def test_scan_with_state_autograd():
    """Gradients through both outputs and into all three inputs, against autograd through a loop."""
    g = torch.Generator().manual_seed(95)
    bs, seq, d = 2, 70, 48
    alpha = torch.sigmoid(torch.randn(bs, seq, d, generator=g))
    beta = torch.randn(bs, seq, d, generator=g)
    h0 = torch.randn(bs, d, generator=g)
    w_h = torch.randn(bs, seq, d, generator=g)
    w_last = torch.randn(bs, d, generator=g)

    def loss_ref(a, b, s):
        hs, cur = [], s
        for t in range(seq):
            cur = a[:, t] * cur + b[:, t]
            hs.append(cur)
        return (torch.stack(hs, 1) * w_h).sum() + (cur * w_last).sum()

    ar, br, sr = (x.clone().double().requires_grad_(True) for x in (alpha, beta, h0))
    loss_ref(ar, br, sr).backward()

    ad, bd, sd = (x.clone().to(DEV).requires_grad_(True) for x in (alpha, beta, h0))
    h, h_last = scan_with_state(ad, bd, sd)
    ((h * w_h.to(DEV)).sum() + (h_last * w_last.to(DEV)).sum()).backward()
    torch.testing.assert_close(ad.grad.cpu().double(), ar.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(bd.grad.cpu().double(), br.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(sd.grad.cpu().double(), sr.grad, rtol=1e-4, atol=1e-5)
    # and the plain entry point is untouched by all this
    out = scan_cu(alpha.to(torch.bfloat16).to(DEV), beta.to(torch.bfloat16).to(DEV))
    assert out.shape == (bs, seq, d)


@pytest.mark.parametrize("shape", [(4, 1000, 512), (8, 4096, 1024)], ids=["small_output", "headline_shape"])
def test_cache_policies_give_identical_results_with_states(shape):
    """The scans with states follow the cache policy in the kernels large shapes run (hints on loads
    and stores only): every output bit stays, on both sides of the sizes at which the automatic
    policy switches its hints, with alphas near 1 so that the carried states matter."""
    import fast_sequential_scan_amd as pkg

    alpha, beta, dout = make_inputs("near_one", *shape, seed=21)
    g = torch.Generator().manual_seed(22)
    h0 = torch.randn(shape[0], shape[2], generator=g).to(DEV)
    g_last = torch.randn(shape[0], shape[2], generator=g).to(DEV)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    results = {}
    for policy in ("auto", "streaming"):
        previous = pkg.set_cache_policy(policy)
        try:
            h, h_last = ext.scan_forward_state(a, b, h0)
            results[policy] = (h, h_last, *ext.scan_backward_state(a, h, do, h0, g_last))
        finally:
            pkg.set_cache_policy(previous)
    ext.workspace_status()
    for x, y in zip(results["auto"], results["streaming"]):
        assert torch.equal(x, y)
