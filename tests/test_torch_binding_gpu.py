"""GPU tests of the C++ dispatch of the plain scan (csrc/fss_torch_binding.cpp): that the public
``scan_cu`` / ``scan_cu_single`` / ``scan_fp16`` go through it in the common case, that its results are
those of the Python wrappers bit for bit (same kernels, same launch configuration), and that everything
it does not cover still works through them."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import scan_cu, scan_cu_single  # noqa: E402
from fast_sequential_scan_amd import scan_cu_fp16 as scan_fp16  # noqa: E402
from fast_sequential_scan_amd import scan_cm, scan_gated, scan_with_state  # noqa: E402
from fast_sequential_scan_amd import scan_cuda  # noqa: E402
from fast_sequential_scan_amd import sequential_scan_cuda as ext  # noqa: E402
from fast_sequential_scan_amd.workloads import make_inputs  # noqa: E402

DEV = "cuda:0"
APIS = [(scan_cu, scan_cuda.SequentialScan, torch.bfloat16), (scan_cu_single, scan_cuda.SequentialScanSingle, torch.float32),
        (scan_fp16, scan_cuda.SequentialScanFp16, torch.float16)]


def _tensors(shape, dtype, seed):
    alpha, beta, dout = make_inputs("sigmoid", *shape, dtype=torch.float32, seed=seed)
    return tuple(t.to(dtype).to(DEV) for t in (alpha, beta, dout))


def _node_name(t):
    return t.grad_fn.name() if t.grad_fn is not None else ""


@pytest.mark.parametrize("api,function,dtype", APIS, ids=["bf16", "f32", "f16"])
@pytest.mark.parametrize("shape", [(2, 1000, 768), (3, 37, 64), (1, 5000, 130)])
def test_same_bits_as_the_python_functions(api, function, dtype, shape):
    assert ext.fast_dispatch() is not None, "the C++ dispatch was not loaded"
    alpha, beta, dout = _tensors(shape, dtype, seed=sum(shape))
    a1, b1 = alpha.clone().requires_grad_(True), beta.clone().requires_grad_(True)
    want = function.apply(a1, b1)  # the Python Function (also makes sure a workspace exists)
    want.backward(dout)
    a2, b2 = alpha.clone().requires_grad_(True), beta.clone().requires_grad_(True)
    got = api(a2, b2)
    assert "ScanNode" in _node_name(got), _node_name(got)
    got.backward(dout)
    ext.workspace_status()
    assert torch.equal(got, want) and torch.equal(a2.grad, a1.grad) and torch.equal(b2.grad, b1.grad)
    # without gradients: no node, same bits
    with torch.no_grad():
        plain = api(a2, b2)
    assert plain.grad_fn is None and not plain.requires_grad and torch.equal(plain, want)
    assert api(alpha, beta).grad_fn is None


def test_what_it_does_not_cover_goes_through_python():
    alpha, beta, dout = _tensors((2, 300, 256), torch.bfloat16, seed=3)
    scan_cu(alpha, beta)  # a workspace exists from here on
    want = scan_cu(alpha, beta)
    # non-contiguous inputs
    a_t = alpha.transpose(0, 1).contiguous().transpose(0, 1).requires_grad_(True)
    out = scan_cu(a_t, beta)
    assert "ScanNode" not in _node_name(out) and torch.equal(out, want)
    # under autocast fp32 inputs are cast to bf16, as the reference's custom_fwd does
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = scan_cu(alpha.float().requires_grad_(True), beta.float())
    assert out.dtype == torch.bfloat16 and "ScanNode" not in _node_name(out) and torch.equal(out, want)
    # errors keep the wrappers' wording
    with pytest.raises(RuntimeError, match="expected scalar type"):
        scan_cu(alpha.float(), beta.float())
    with pytest.raises(RuntimeError, match="has shape"):
        scan_cu(alpha, beta[:, :10])
    with pytest.raises(RuntimeError, match="must live on a GPU"):
        scan_cu(alpha.cpu(), beta.cpu())
    assert scan_cu(alpha[:, :0], beta[:, :0]).shape == (2, 0, 256)
    # a gradient that arrives non-contiguous, and one that arrives expanded from a scalar
    a = alpha.clone().requires_grad_(True)
    b = beta.clone().requires_grad_(True)
    out = scan_cu(a, b)
    assert "ScanNode" in _node_name(out)
    out.transpose(1, 2).backward(dout.transpose(1, 2).contiguous())
    ga, gb = ext.scan_backward_half(alpha, want, dout)
    assert torch.equal(a.grad, ga) and torch.equal(b.grad, gb)
    a.grad = b.grad = None
    scan_cu(a, b).sum().backward()
    ga, gb = ext.scan_backward_half(alpha, want, torch.ones_like(dout))
    assert torch.equal(a.grad, ga) and torch.equal(b.grad, gb)
    ext.workspace_status()


def test_a_second_backward_and_double_differentiation():
    alpha, beta, dout = _tensors((2, 500, 128), torch.float32, seed=4)
    scan_cu_single(alpha, beta)
    a, b = alpha.clone().requires_grad_(True), beta.clone().requires_grad_(True)
    out = scan_cu_single(a, b)
    assert "ScanNode" in _node_name(out)
    first = torch.autograd.grad(out, (a, b), dout, retain_graph=True)
    second = torch.autograd.grad(out, (a, b), dout, retain_graph=True)
    assert torch.equal(first[0], second[0]) and torch.equal(first[1], second[1])
    # create_graph with a differentiable incoming gradient: the results come back, differentiating through
    # them raises - from the C++ node as from the Python Function (once_differentiable)
    for make in (lambda: scan_cu_single(a, b), lambda: scan_cuda.SequentialScanSingle.apply(a, b)):
        out = make()
        ga, gb = torch.autograd.grad(out, (a, b), dout.clone().requires_grad_(True), create_graph=True)
        assert torch.equal(ga, first[0]) and torch.equal(gb, first[1]) and ga.requires_grad
        with pytest.raises(RuntimeError, match="differentiate twice"):
            ga.sum().backward()
        ga, gb = torch.autograd.grad(make(), (a, b), dout, create_graph=True)
        assert torch.equal(ga, first[0]) and not ga.requires_grad
    ext.workspace_status()


def test_other_streams_get_their_own_workspace_and_node():
    alpha, beta, dout = _tensors((2, 2000, 256), torch.bfloat16, seed=5)
    want = scan_cu(alpha, beta)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        first = scan_cu(alpha.clone().requires_grad_(True), beta)  # makes the stream's workspace (Python path)
        a = alpha.clone().requires_grad_(True)
        out = scan_cu(a, beta)
        assert "ScanNode" in _node_name(out)
        out.backward(dout)
    side.synchronize()
    ga, _ = ext.scan_backward_half(alpha, want, dout)
    assert torch.equal(first, want) and torch.equal(out, want) and torch.equal(a.grad, ga)
    ext.workspace_status()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("shape", [(2, 1000, 768), (3, 37, 64), (1, 5000, 130)])
def test_gated_scan_same_bits_as_the_python_function(dtype, shape):
    g = torch.Generator().manual_seed(sum(shape))
    gate = (1.5 * torch.randn(shape, generator=g)).to(dtype).to(DEV)
    x, dout = (torch.randn(shape, generator=g).to(dtype).to(DEV) for _ in range(2))
    g1, x1 = gate.clone().requires_grad_(True), x.clone().requires_grad_(True)
    want = scan_cuda.SequentialScanGated.apply(g1, x1)
    want.backward(dout)
    g2, x2 = gate.clone().requires_grad_(True), x.clone().requires_grad_(True)
    got = scan_gated(g2, x2)
    assert "ScanNode" in _node_name(got), _node_name(got)
    got.backward(dout)
    ext.workspace_status()
    assert torch.equal(got, want) and torch.equal(g2.grad, g1.grad) and torch.equal(x2.grad, x1.grad)
    with torch.no_grad():
        assert torch.equal(scan_gated(g2, x2), want)
    # what it does not cover: a non-contiguous gate, a gradient that arrives transposed
    g_t = gate.transpose(1, 2).contiguous().transpose(1, 2).requires_grad_(True)
    out = scan_gated(g_t, x)
    assert "ScanNode" not in _node_name(out) and torch.equal(out, want)
    g3, x3 = gate.clone().requires_grad_(True), x.clone().requires_grad_(True)
    scan_gated(g3, x3).transpose(1, 2).backward(dout.transpose(1, 2).contiguous())
    assert torch.equal(g3.grad, g1.grad) and torch.equal(x3.grad, x1.grad)
    with pytest.raises(RuntimeError):
        scan_gated(gate, x[:, :10])
    ext.workspace_status()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_decode_loop_through_the_state_dispatch(dtype):
    """Segments of 1, 3 and 700 steps chained through (h, h_last) without gradients - through the C++
    dispatch from the second call on - reproduce the Python Function's outputs bit for bit and, in
    fp32, the scan of the whole sequence."""
    bs, seq, d = 3, 1200, 192
    alpha, beta, _ = _tensors((bs, seq, d), dtype, seed=12)
    binding = ext.fast_dispatch()
    cuts = [0, 1, 4, 5, 500, 1200]
    with torch.no_grad():
        state = None
        pieces, states = [], []
        for lo, hi in zip(cuts[:-1], cuts[1:]):
            a, b = alpha[:, lo:hi].contiguous(), beta[:, lo:hi].contiguous()
            want_h, want_state = scan_cuda.SequentialScanState.apply(a, b, state)
            if lo > 0:
                assert binding.scan_state(a, b, state) is not None, "the C++ dispatch declined a plain call"
            h, new_state = scan_with_state(a, b, state)
            assert torch.equal(h, want_h) and torch.equal(new_state, want_state)
            pieces.append(h)
            states.append(new_state)
            state = new_state
        whole, whole_state = scan_with_state(alpha, beta)
    ext.workspace_status()
    if dtype == torch.float32:
        torch.testing.assert_close(torch.cat(pieces, dim=1), whole, rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(states[-1], whole_state, rtol=1e-5, atol=1e-6)
    # with gradients the call goes through the Python Function
    a = alpha[:, :50].contiguous().requires_grad_(True)
    h, last = scan_with_state(a, beta[:, :50].contiguous())
    assert h.grad_fn is not None and "ScanNode" not in _node_name(h)
    assert binding.scan_state(a, beta[:, :50].contiguous(), None) is None
    # what it declines: a state of the wrong type or shape (the wrappers raise)
    with pytest.raises(RuntimeError):
        scan_with_state(alpha, beta, torch.zeros(bs, d, device=DEV, dtype=torch.float64))
    with pytest.raises(RuntimeError):
        scan_with_state(alpha, beta, torch.zeros(bs, d + 1, device=DEV))


def test_captured_decode_step_replays_match_eager():
    """A decode step through the public API - ``scan_with_state`` without gradients, which the C++
    dispatch takes - captured as a HIP graph: every replay (with eager scans and synchronisations in
    between) gives what the eager call gives.  The state is carried in a tensor the graph updates in place."""
    bs, seq, d = 4, 2000, 256  # several chunks: the chaining workspace is in play
    alpha, beta, _ = _tensors((bs, seq, d), torch.bfloat16, seed=21)
    binding = ext.fast_dispatch()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        state = torch.zeros(bs, d, device=DEV)
        scan_with_state(alpha, beta, state)  # warm: the stream's workspace, device check, residency query
        assert binding.scan_state(alpha, beta, state) is not None
        side.synchronize()
        want = []
        s = state.clone()
        for _ in range(4):
            h, s = scan_with_state(alpha, beta, s)
            want.append((h.clone(), s.clone()))
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            h_out, s_out = scan_with_state(alpha, beta, state)
            state.copy_(s_out)
        state.zero_()
        for i in range(4):
            graph.replay()
            side.synchronize()
            assert torch.equal(h_out, want[i][0]) and torch.equal(state, want[i][1]), i
            scan_with_state(alpha, beta, torch.ones(bs, d, device=DEV))  # eager work between replays, same workspace
            side.synchronize()
    ext.workspace_status()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("shape", [(2, 768, 1000), (3, 64, 37), (1, 130, 5000), (2, 96, 9000)])
def test_channel_major_scan_same_bits_as_the_python_function(dtype, shape):
    """(bs, d_model, seq) tensors: the C++ dispatch against the Python Function, forward and backward."""
    alpha, beta, dout = _tensors(shape, dtype, seed=sum(shape))
    a1, b1 = alpha.clone().requires_grad_(True), beta.clone().requires_grad_(True)
    want = scan_cuda.SequentialScanChannelMajor.apply(a1, b1)
    want.backward(dout)
    a2, b2 = alpha.clone().requires_grad_(True), beta.clone().requires_grad_(True)
    got = scan_cm(a2, b2)
    assert "ScanNode" in _node_name(got), _node_name(got)
    got.backward(dout)
    ext.workspace_status()
    assert torch.equal(got, want) and torch.equal(a2.grad, a1.grad) and torch.equal(b2.grad, b1.grad)
    with torch.no_grad():
        assert torch.equal(scan_cm(a2, b2), want)
    a_t = alpha.transpose(1, 2).contiguous().transpose(1, 2).requires_grad_(True)
    out = scan_cm(a_t, beta)
    assert "ScanNode" not in _node_name(out) and torch.equal(out, want)
    with pytest.raises(RuntimeError):
        scan_cm(alpha, beta[:, :, :10])
    ext.workspace_status()
