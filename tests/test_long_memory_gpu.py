"""Full-size parity in the long-memory regime: alpha = sigmoid(N(0,1)+6), median 0.9975.

In the measured workloads (alpha = sigmoid(N(0,1)), N(0,1), sigmoid(N(0,1)+2)) the product of a
chunk's few hundred alphas is 0 or all but 0 in fp32, so the state a chunk receives is just what
the chunk before it produced by itself and the composed carries are never exercised at full size.
Here that product is 0.1-0.6 over a chunk, as in a trained Hawk / Griffin block, and every output
depends on carries composed across many chunks.  Same oracle (the sequential loop of
sequential_scan/common.py:46-59 restated in oracle/scan_oracle.c) and same bars as the measured
workloads: rtol = atol = 1e-2 against the fp32-accumulated scan, at most 2 bf16 ulps against the
oracle that rounds where the kernel does.  Plain scan at the three shapes with the longest chains;
the gated scan, the scan with states and the channel-major scan at the headline shape (and the
shape of the 65521-step workload where the oracle's cost allows).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402
from fast_sequential_scan_amd.workloads import LONG_MEMORY_CASES, make_inputs  # noqa: E402

from test_scan_gpu import bits, check_bf16  # noqa: E402
from test_scan_cm_gpu import _check as check_cm, _t  # noqa: E402
from test_scan_gated_gpu import _check_all as check_gated  # noqa: E402
from test_scan_state_gpu import _close, _extended_oracle  # noqa: E402

DEV = "cuda:0"


def _chunk_product(alpha, steps=512):
    return float(np.prod(alpha[0, 1:1 + steps, 0].double().numpy()))


@pytest.mark.parametrize("case", list(LONG_MEMORY_CASES), ids=list(LONG_MEMORY_CASES))
def test_plain_scan_full_size(oracle, case):
    recipe, bs, seq, d = LONG_MEMORY_CASES[case]
    alpha, beta, dout = make_inputs(recipe, bs, seq, d)
    assert 1e-3 < _chunk_product(alpha) < 0.9  # a chunk's coefficient is far from 0 and from 1
    h, ga, gb = check_bf16(oracle, alpha, beta, dout, what=case)
    ext.workspace_status()
    # the states really do carry far: h is not what the last chunk alone produces
    assert float(h.float().abs().mean()) > 0.3


def test_fp32_full_size(oracle):
    alpha, beta, dout = make_inputs("near_one", 8, 4096, 1024, dtype=torch.float32, seed=7)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext.scan_forward(a, b)
    ga, gb = ext.scan_backward(a, h, do)
    ext.workspace_status()
    h_ref = oracle.scan_fwd_f32(alpha.numpy(), beta.numpy())
    ga_ref, gb_ref = oracle.scan_bwd_f32(alpha.numpy(), h_ref, dout.numpy())
    for name, got, want in (("h", h, h_ref), ("grad_alpha", ga, ga_ref), ("grad_beta", gb, gb_ref)):
        got = got.cpu().numpy()
        rel = float(np.linalg.norm((got - want).ravel()) / np.linalg.norm(want.ravel()))
        assert rel < 1e-6, (name, rel)  # the reference's fp32 bar (sequential_scan/common.py:6,14-17)
        # elementwise: sums of ~400 terms of size 1 carried in fp32
        assert np.allclose(got, want, rtol=1e-4, atol=2e-4 * max(1.0, float(np.abs(want).max()) / 8)), name


@pytest.mark.parametrize("shape", [(8, 4096, 1024), (1, 65521, 256)], ids=["C3_4096_shape", "C5_shape"])
def test_scan_with_states_full_size(oracle, shape):
    alpha, beta, dout = make_inputs("near_one", *shape, seed=11)
    g = torch.Generator().manual_seed(12)
    h0 = torch.randn(shape[0], shape[2], generator=g)
    g_last = torch.randn(shape[0], shape[2], generator=g)
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h, h_last = ext.scan_forward_state(a, b, h0.to(DEV))
    ga, gb, gh0 = ext.scan_backward_state(a, h, do, h0.to(DEV), g_last.to(DEV))
    ext.workspace_status()
    want = _extended_oracle(oracle, alpha.float().numpy(), beta.float().numpy(), dout.float().numpy(),
                            h0.numpy(), g_last.numpy())
    for name, got, ref in zip(("h", "h_last", "grad_alpha", "grad_beta", "grad_h_before"), (h, h_last, ga, gb, gh0), want):
        _close(got, ref, 1e-2, 1e-2, name)
    # the incoming state is still felt hundreds of steps in: the scan without it differs there
    h_plain = ext.scan_forward_half(a, b)
    assert float((h[:, 300].float() - h_plain[:, 300].float()).abs().mean()) > 0.05


@pytest.mark.parametrize("shape", [(8, 1024, 4096), (1, 256, 65521)], ids=["C3_4096_shape", "C5_shape"])
def test_channel_major_full_size(oracle, shape):
    bs, d, seq = shape
    alpha, beta, dout = (t.transpose(1, 2).contiguous() for t in make_inputs("near_one", bs, seq, d, seed=13))
    a, b, do = alpha.to(DEV), beta.to(DEV), dout.to(DEV)
    h = ext.scan_forward_cm(a, b)
    ga, gb = ext.scan_backward_cm(a, h, do)
    ext.workspace_status()
    check_cm(h, oracle.scan_fwd_f32(_t(alpha), _t(beta), fused=True), torch.bfloat16, "h")
    ga_or, gb_or = oracle.scan_bwd_f32(_t(alpha), _t(h), _t(dout), fused=True)
    check_cm(gb, gb_or, torch.bfloat16, "grad_beta")
    check_cm(ga, ga_or, torch.bfloat16, "grad_alpha")


@pytest.mark.parametrize("shape", [(8, 4096, 1024), (1, 65521, 256)], ids=["C3_4096_shape", "C5_shape"])
def test_gated_scan_full_size(oracle, shape):
    """gate = N(0,1)+6, so that alpha = sigmoid(gate) is the long-memory recipe's; x ~ N(0,1)."""
    g = torch.Generator().manual_seed(17)
    gate = (torch.randn(shape, generator=g) + 6.0).to(torch.bfloat16)
    x = torch.randn(shape, generator=g).to(torch.bfloat16)
    dout = torch.randn(shape, generator=g).to(torch.bfloat16)
    gd, xd, dd = gate.to(DEV), x.to(DEV), dout.to(DEV)
    h = ext.gated_scan_forward(gd, xd)
    grad_gate, grad_x = ext.gated_scan_backward(gd, xd, h, dd)
    ext.workspace_status()
    check_gated(oracle, "bf16", 1e-2, 1e-2, gate, x, dout, h, grad_gate, grad_x)
