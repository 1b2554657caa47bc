"""The reference's own test recipe (sequential_scan/test_scan_cuda.py:26-124) against the
drop-in package: inputs from ``make_tensors*`` (N(0,1), also for alpha), the expectation from
``torch_ref`` evaluated on the GPU in the tensors' dtype and differentiated by torch's autograd,
the verdict from ``check_relative_error(relative_error(...), tolerance)`` with the reference's
tolerances: 7 digits in fp32, 2 in bf16.  Everything is imported under the reference's module
names, so the reference's test file itself runs unchanged against ``sequential_scan/``.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu

from sequential_scan.common import (  # noqa: E402
    BFLOAT16_TOL, SINGLE_TOL, check_relative_error, make_tensors, make_tensors_single, relative_error, torch_ref,
)
from sequential_scan.scan_cuda import scan, scan_single  # noqa: E402

# the reference's grid is bs {9,10,12,2} (fp32) / five random sizes below 16 (bf16),
# sq {128,256,512,1024}, d {512,768,1024}; a spread of it, plus shapes its kernels refuse
FP32_SHAPES = [(9, 128, 512), (10, 256, 768), (12, 512, 1024), (2, 1024, 768), (2, 1024, 1024), (3, 300, 200)]
BF16_SHAPES = [(1, 128, 512), (7, 256, 768), (15, 512, 1024), (4, 1024, 512), (11, 1024, 1024), (5, 333, 96)]


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
