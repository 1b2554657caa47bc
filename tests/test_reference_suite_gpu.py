"""The reference's own test recipe (sequential_scan/test_scan_cuda.py:26-124) against the
drop-in package: inputs from ``make_tensors*`` (N(0,1), also for alpha), the expectation from
``torch_ref`` evaluated on the GPU in the tensors' dtype and differentiated by torch's autograd,
the verdict from ``check_relative_error(relative_error(...), tolerance)`` with the reference's
tolerances: 7 digits in fp32, 2 in bf16.  Everything is imported under the reference's module
names, so the reference's test file itself runs unchanged against ``sequential_scan/``.
"""
import itertools
import os
import re

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from sequential_scan.common import (  # noqa: E402
    BFLOAT16_TOL, SINGLE_TOL, check_relative_error, make_tensors, make_tensors_single, relative_error, torch_ref,
)
from sequential_scan.scan_cuda import scan, scan_single  # noqa: E402

# The reference's whole grid (test_scan_cuda.py:27-29,44-46 fp32; :80-82,97-99 bf16): bs {9,10,12,2}
# (fp32) or five sizes drawn from 1..15 (bf16: the reference draws them unseeded at collection time,
# here from a fixed seed), sq {128,256,512,1024}, d {512,768,1024}; plus two shapes its kernels
# refuse (odd lengths, widths outside its switch).
_SQ, _D = (128, 256, 512, 1024), (512, 768, 1024)
FP32_SHAPES = list(itertools.product((9, 10, 12, 2), _SQ, _D)) + [(3, 300, 200)]
_BF16_BS = [int(b) for b in np.random.default_rng(0).integers(1, 16, size=5)]
BF16_SHAPES = list(itertools.product(_BF16_BS, _SQ, _D)) + [(5, 333, 96)]


def _passes(got, want, digits):
    err = relative_error(got, want)
    assert check_relative_error(err, digits), err


@pytest.mark.parametrize("bs,sq,d", FP32_SHAPES)
def test_fwd_single(bs, sq, d):
    torch.manual_seed(0)
    alpha, beta = make_tensors_single(bs, sq, d)
    with torch.no_grad():
        _passes(scan_single(alpha, beta), torch_ref(alpha, beta), SINGLE_TOL)


@pytest.mark.parametrize("bs,sq,d", FP32_SHAPES)
def test_bwd_single(bs, sq, d):
    torch.manual_seed(0)
    alpha, beta = make_tensors_single(bs, sq, d)
    expected = torch_ref(alpha, beta)
    dy = torch.randn_like(expected)
    expected.backward(dy)
    want = [t.grad.clone() for t in (alpha, beta)]
    alpha.grad = beta.grad = None
    scan_single(alpha, beta).backward(dy)
    _passes(alpha.grad, want[0], SINGLE_TOL)
    _passes(beta.grad, want[1], SINGLE_TOL)


@pytest.mark.parametrize("bs,sq,d", BF16_SHAPES)
def test_fwd_half(bs, sq, d):
    torch.manual_seed(0)
    alpha, beta = make_tensors(bs, sq, d)
    with torch.no_grad():
        _passes(scan(alpha, beta), torch_ref(alpha, beta), BFLOAT16_TOL)


@pytest.mark.parametrize("bs,sq,d", BF16_SHAPES)
def test_bwd_half(bs, sq, d):
    torch.manual_seed(0)
    alpha, beta = make_tensors(bs, sq, d)
    expected = torch_ref(alpha, beta)
    dy = torch.randn_like(expected)
    expected.backward(dy)
    want = [t.grad.clone() for t in (alpha, beta)]
    alpha.grad = beta.grad = None
    scan(alpha, beta).backward(dy)
    _passes(alpha.grad, want[0], BFLOAT16_TOL)
    _passes(beta.grad, want[1], BFLOAT16_TOL)


# ---- the binding a maintainer of the reference would drop in, exactly as the integration notes print it ----


def _option_b_module():
    """Executes the python block of the integration notes' "Option B" (the replacement for the
    compiled module that sequential_scan/scan_cuda.py:4-9 imports) as written.  The block opens
    the library by its bare name; the built library is loaded by path first, so that name
    resolves to it (the library carries that name as its soname)."""
    import ctypes
    import types

    from fast_sequential_scan_amd import _native

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    section = text[text.index("## Option B"):]
    block = re.search(r"```python\n(.*?)```", section, flags=re.S).group(1)
    ctypes.CDLL(_native.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    mod = types.ModuleType("sequential_scan_cuda")
    exec(compile(block, "INTEGRATION.md (Option B)", "exec"), mod.__dict__)
    return mod


def test_option_b_binding_as_printed_drives_an_autograd_shell():
    """The four callees of the printed binding behind two autograd Functions of the shape the
    reference's scan_cuda.py has (forward saves (alpha, h); backward returns the two gradients),
    written here; checked with the reference's recipe and tolerances, on aligned tensors and on
    a view that starts 2 bytes into its storage (which needs the larger workspace)."""
    ext_b = _option_b_module()

    class Half(torch.autograd.Function):
        @staticmethod
        def forward(ctx, alpha, beta):
            h = ext_b.scan_forward_half(alpha, beta)
            ctx.save_for_backward(alpha, h)
            return h

        @staticmethod
        def backward(ctx, grad_output):
            alpha, h = ctx.saved_tensors
            grad_alpha, grad_beta = ext_b.scan_backward_half(alpha, h, grad_output)
            return grad_alpha, grad_beta

    class Single(torch.autograd.Function):
        @staticmethod
        def forward(ctx, alpha, beta):
            h = ext_b.scan_forward(alpha, beta)
            ctx.save_for_backward(alpha, h)
            return h

        @staticmethod
        def backward(ctx, grad_output):
            alpha, h = ctx.saved_tensors
            grad_alpha, grad_beta = ext_b.scan_backward(alpha, h, grad_output)
            return grad_alpha, grad_beta

    torch.manual_seed(0)
    for fn, make, digits, shape in ((Half.apply, make_tensors, BFLOAT16_TOL, (7, 1024, 768)),
                                    (Single.apply, make_tensors_single, SINGLE_TOL, (2, 512, 1024)),
                                    (Half.apply, make_tensors, BFLOAT16_TOL, (1, 4096, 2048))):
        alpha, beta = make(*shape)
        expected = torch_ref(alpha, beta)
        dy = torch.randn_like(expected)
        expected.backward(dy)
        want = [t.grad.clone() for t in (alpha, beta)]
        alpha.grad = beta.grad = None
        out = fn(alpha, beta)
        out.backward(dy)
        _passes(out.detach(), expected.detach(), digits)
        _passes(alpha.grad, want[0], digits)
        _passes(beta.grad, want[1], digits)
    # a 2-byte offset view of the last shape through the printed binding
    flat = torch.empty(alpha.numel() + 1, dtype=alpha.dtype, device=alpha.device)
    a_off = flat[1:].view(alpha.shape)
    a_off.copy_(alpha.detach())
    assert a_off.data_ptr() % 4 == 2
    h_off = ext_b.scan_forward_half(a_off, beta.detach())
    ga_off, gb_off = ext_b.scan_backward_half(a_off, h_off, dy)
    torch.cuda.synchronize()
    _passes(h_off, expected.detach(), digits)
    _passes(ga_off, want[0], digits)
    _passes(gb_off, want[1], digits)
