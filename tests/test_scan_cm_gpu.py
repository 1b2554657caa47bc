"""GPU tests of the channel-major scans (fss_scan_fwd_cm / fss_scan_bwd_cm, scan_cm):
tensors (bs, d_model, seq), time contiguous.  Not in the reference; the oracle is the
pinned scan on the transposed tensors.  Bars as for the row-major kernels: rtol = atol =
1e-2 (bf16), 2e-3 (fp16), 1e-4/1e-5 (fp32) against the fp32 oracle, and for the 16-bit
types at most 2 ulps from the oracle's output rounded the same way (time runs across
the lanes here, so carries are re-associated everywhere: never bit-exact by design).
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import _native, scan_cm, scan_cu  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402

DEV = "cuda:0"
TOL = {torch.bfloat16: (1e-2, 1e-2), torch.float16: (2e-3, 2e-3), torch.float32: (1e-4, 1e-5)}


def _inputs(bs, d, seq, dtype, seed, recipe="sigmoid"):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(bs, d, seq, generator=g)
    alpha = (torch.sigmoid(x) if recipe == "sigmoid" else x).to(dtype)
    beta = torch.randn(bs, d, seq, generator=g).to(dtype)
    dout = torch.randn(bs, d, seq, generator=g).to(dtype)
    return alpha, beta, dout


def _t(a: torch.Tensor) -> np.ndarray:  # (bs, d, seq) tensor -> (bs, seq, d) float32 array
    return np.ascontiguousarray(a.detach().float().cpu().numpy().transpose(0, 2, 1))


def _ordered16(x16: np.ndarray) -> np.ndarray:
    u = x16.view(np.uint16).astype(np.int32)
    return np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)


def _check(got: torch.Tensor, want_rm: np.ndarray, dtype, what):
    rtol, atol = TOL[dtype]
    got32 = _t(got)
    bad = ~(np.abs(got32 - want_rm) <= atol + rtol * np.abs(want_rm))
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} outside tolerance, worst {np.abs(got32 - want_rm).max():.4g}"
    if dtype != torch.float32:
        same = torch.from_numpy(want_rm).to(dtype)
        got_rm = got.detach().cpu().transpose(1, 2).contiguous()
        dist = np.abs(_ordered16(got_rm.view(torch.int16).numpy().view(np.uint16)) -
                      _ordered16(same.view(torch.int16).numpy().view(np.uint16)))
        close = np.abs(got32 - want_rm) <= (1e-3 if dtype == torch.bfloat16 else 2e-4)
        finite = np.isfinite(want_rm)
        assert ((dist <= 2) | close | ~finite).all(), f"{what}: max ulp distance {dist[finite].max()}"


def _run(oracle, bs, d, seq, dtype, config=None, seed=0, recipe="sigmoid"):
    alpha, beta, dout = _inputs(bs, d, seq, dtype, seed, recipe)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext.scan_forward_cm(a, b, config)
    ga, gb = ext.scan_backward_cm(a, h, do, config)
    ext.workspace_status()
    assert h.shape == (bs, d, seq) and h.dtype == dtype
    _check(h, oracle.scan_fwd_f32(_t(alpha), _t(beta), fused=True), dtype, "h")
    ga_or, gb_or = oracle.scan_bwd_f32(_t(alpha), _t(h), _t(dout), fused=True)  # fed the stored h
    _check(gb, gb_or, dtype, "grad_beta")
    _check(ga, ga_or, dtype, "grad_alpha")
    return h, ga, gb


SHAPES = [(1, 1, 1), (2, 3, 7), (2, 5, 64), (3, 4, 510), (2, 9, 512), (2, 7, 1000), (1, 13, 4096),
          (2, 6, 5000), (2, 3, 8200), (1, 8, 65536), (1, 5, 40001), (16, 24, 2048)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_cm_default_config(oracle, shape, dtype):
    _run(oracle, *shape, dtype, seed=sum(shape))


@pytest.mark.parametrize("config", [(1, 0, 1), (1, 0, 3), (2, 0, 2), (2, 0, 16), (8, 0, 1), (8, 0, 2), (8, 0, 5),
                                    (8, 0, 16), (8, 0, 8, 3), (2, 0, 4, 1)], ids=str)
def test_cm_result_does_not_depend_on_config_bf16(oracle, config):
    _run(oracle, 2, 11, 6000, torch.bfloat16, config=config, seed=1)


@pytest.mark.parametrize("config", [(1, 0, 2), (4, 0, 1), (4, 0, 3), (4, 0, 16), (4, 0, 8, 2)], ids=str)
def test_cm_result_does_not_depend_on_config_f32(oracle, config):
    _run(oracle, 2, 6, 6000, torch.float32, config=config, seed=2)
    _run(oracle, 2, 6, 600, torch.float32, config=config, seed=2, recipe="normal")


def test_cm_headline_size_and_row_major_agreement(oracle):
    """bs8 d1024 seq4096 bf16 against the oracle, and against the row-major kernels on the
    permuted tensors (two different decompositions of the same recurrence)."""
    bs, d, seq = 8, 1024, 4096
    h, ga, gb = _run(oracle, bs, d, seq, torch.bfloat16, seed=3)
    alpha, beta, dout = (t.to(DEV) for t in _inputs(bs, d, seq, torch.bfloat16, 3))
    a_rm, b_rm, do_rm = (t.transpose(1, 2).contiguous() for t in (alpha, beta, dout))
    h_rm = ext.scan_forward_half(a_rm, b_rm)
    torch.testing.assert_close(h.transpose(1, 2).float(), h_rm.float(), rtol=1e-2, atol=1e-2)
    ga_rm, gb_rm = ext.scan_backward_half(a_rm, h.transpose(1, 2).contiguous(), do_rm)
    torch.testing.assert_close(gb.transpose(1, 2).float(), gb_rm.float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(ga.transpose(1, 2).float(), ga_rm.float(), rtol=1e-2, atol=1e-2)
    # size-independent: beta scaled by a power of two scales h exactly
    assert torch.equal(ext.scan_forward_cm(alpha, 2 * beta), 2 * h)


def test_cm_first_alpha_is_never_used_and_closed_forms():
    alpha, beta, dout = (t.to(DEV) for t in _inputs(2, 5, 1536, torch.float32, 4))
    h = ext.scan_forward_cm(alpha, beta)
    a2 = alpha.clone()
    a2[..., 0] = float("nan")
    assert torch.equal(ext.scan_forward_cm(a2, beta), h)
    ga, gb = ext.scan_backward_cm(alpha, h, dout)
    ga2, gb2 = ext.scan_backward_cm(a2, h, dout)
    assert torch.equal(gb2, gb) and torch.equal(ga2, ga) and (ga[..., 0] == 0).all()
    # alpha = 1: cumulative sum; alpha = 0: h = beta
    ones = torch.ones_like(beta)
    torch.testing.assert_close(ext.scan_forward_cm(ones, beta), torch.cumsum(beta, -1), rtol=1e-4, atol=1e-3)
    assert torch.equal(ext.scan_forward_cm(torch.zeros_like(beta), beta), beta)


def test_cm_autograd_and_unaligned_views(oracle):
    alpha, beta, dout = _inputs(2, 6, 1024, torch.bfloat16, 5)
    a, b = alpha.to(DEV).requires_grad_(True), beta.to(DEV).requires_grad_(True)
    h = scan_cm(a, b)
    h.backward(dout.to(DEV))
    ga_or, gb_or = oracle.scan_bwd_f32(_t(alpha), _t(h), _t(dout))
    _check(a.grad, ga_or, torch.bfloat16, "grad_alpha")
    _check(b.grad, gb_or, torch.bfloat16, "grad_beta")
    # a row-major user: permuted views are made contiguous by the wrapper
    a_rm = alpha.to(DEV).transpose(1, 2).contiguous()
    b_rm = beta.to(DEV).transpose(1, 2).contiguous()
    assert torch.equal(scan_cm(a_rm.transpose(1, 2), b_rm.transpose(1, 2)), h.detach())
    torch.testing.assert_close(scan_cu(a_rm, b_rm).transpose(1, 2).float(), h.detach().float(), rtol=1e-2, atol=1e-2)
    # storage offset of one element: 2-byte alignment -> one timestep per lane
    big_a = torch.zeros(2 * 6 * 1024 + 1, dtype=torch.bfloat16, device=DEV)
    big_b = torch.zeros_like(big_a)
    va, vb = big_a[1:].view(2, 6, 1024), big_b[1:].view(2, 6, 1024)
    va.copy_(alpha)
    vb.copy_(beta)
    torch.testing.assert_close(ext.scan_forward_cm(va, vb).float(), h.detach().float(), rtol=1e-2, atol=1e-2)
    assert scan_cm(va[:, :, :0], vb[:, :, :0]).shape == (2, 6, 0)


def test_cm_c_abi_rejects_bad_arguments():
    lib = _native.lib()
    t = torch.zeros(2, 8, 512, dtype=torch.bfloat16, device=DEV)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    sp = torch.cuda.current_stream().cuda_stream
    p = t.data_ptr()
    tail = (ws.data_ptr(), ws.numel(), sp)

    def cfg(*v):
        return ctypes.byref(_native.FssConfig(*v))

    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, p, p, 2, 8, 512, *tail, cfg(4, 0, 0, 0)) == 5   # vec 4 not built for 16 bit
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, p, p, 2, 8, 512, *tail, cfg(0, 16, 0, 0)) == 5  # steps has no meaning here
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, p, p, 2, 8, 511, *tail, cfg(2, 0, 0, 0)) == 5   # seq % vec
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p + 2, p, p, 2, 8, 504, *tail, cfg(8, 0, 0, 0)) == 3
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, None, p, 2, 8, 512, *tail, None) == 1
    assert lib.fss_scan_bwd_cm(_native.FSS_BF16, p, p, p, p, None, 2, 8, 512, *tail, None) == 1
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, p, p, -1, 8, 512, *tail, None) == 2
    assert lib.fss_scan_fwd_cm(9, p, p, p, 2, 8, 512, *tail, None) == 5
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, p, p, 2, 0, 512, *tail, None) == 0
    # chained sequence without a workspace
    assert lib.fss_scan_fwd_cm(_native.FSS_BF16, p, p, p, 1, 1, 8192, None, 0, sp, None) == 4


def test_cm_growing_recurrence_with_zero_state_stays_zero():
    """alpha == 2 along 9000 contiguous steps: the products the lanes exchange overflow fp32; a
    state of exactly 0 must stay 0, as in the sequential order, and one impulse grows in exact
    powers of two until it overflows to inf - never NaN."""
    for dtype in (torch.bfloat16, torch.float32):
        alpha = torch.full((2, 6, 9000), 2.0, dtype=dtype, device=DEV)
        zeros = torch.zeros_like(alpha)
        h = ext.scan_forward_cm(alpha, zeros)
        ga, gb = ext.scan_backward_cm(alpha, zeros, zeros)
        ext.workspace_status()
        assert not h.any() and not ga.any() and not gb.any()
        e0 = zeros.clone()
        e0[..., 0] = 1.0
        h = ext.scan_forward_cm(alpha, e0).float()
        ext.workspace_status()
        assert not torch.isnan(h).any()
        want = torch.pow(2.0, torch.arange(9000, device=DEV, dtype=torch.float64)).to(torch.float32).to(dtype).float()
        assert torch.equal(h, want.expand_as(h))
