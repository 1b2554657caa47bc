"""GPU test of fss_scan_fwd_noalloc, the entry point that allocates nothing: its chaining words
live in a static device array inside the library instead of a caller's workspace.  Called
through the C ABI and compared bit for bit with fss_scan_fwd_ex (same kernels, caller's
workspace) on calls in a row that share the array, the second on a smaller input."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

from fast_sequential_scan_amd import _native  # noqa: E402
from fast_sequential_scan_amd.workloads import make_inputs  # noqa: E402

DEV = "cuda:0"


def _reference(lib, dtype_code, a, b, sp):
    ws = torch.empty(lib.fss_workspace_bytes(*a.shape, dtype_code, _native.FSS_FWD, None), dtype=torch.uint8, device=DEV)
    _native.check(lib.fss_workspace_init(ws.data_ptr(), ws.numel(), sp))
    h = torch.empty_like(a)
    _native.check(lib.fss_scan_fwd_ex(dtype_code, a.data_ptr(), b.data_ptr(), h.data_ptr(), *a.shape,
                                      ws.data_ptr(), ws.numel(), sp, None))
    return h


def test_noalloc_forward_matches_the_workspace_entry_point():
    lib = _native.lib()
    sp = torch.cuda.current_stream().cuda_stream
    # chained shapes (several chunks per sequence), the second call smaller than the first, then a
    # larger one again, an fp32 one, and one that needs no chaining at all
    cases = [(torch.bfloat16, (8, 4096, 1024)), (torch.bfloat16, (2, 1000, 328)), (torch.bfloat16, (1, 65521, 256)),
             (torch.float32, (3, 2049, 200)), (torch.bfloat16, (2, 8, 64))]
    inputs, wanted = [], []
    for dtype, shape in cases:
        alpha, beta, _ = make_inputs("sigmoid", *shape, dtype=dtype, seed=sum(shape))
        a, b = alpha.to(DEV), beta.to(DEV)
        code = _native.FSS_BF16 if dtype == torch.bfloat16 else _native.FSS_F32
        inputs.append((code, a, b))
        wanted.append(_reference(lib, code, a, b, sp))
    outs = [torch.full_like(a, float("nan")) for _code, a, _b in inputs]
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated()
    for _ in range(2):  # every shape twice, back to back: each call finds the previous call's words
        for (code, a, b), out in zip(inputs, outs):
            _native.check(lib.fss_scan_fwd_noalloc(code, a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, sp))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == allocated
    for out, want, (dtype, shape) in zip(outs, wanted, cases):
        assert torch.equal(out, want), (dtype, shape)
    # on a side stream as well: the array is per device, not per stream
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        code, a, b = inputs[1]
        out = torch.empty_like(a)
        _native.check(lib.fss_scan_fwd_noalloc(code, a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, side.cuda_stream))
    side.synchronize()
    assert torch.equal(out, wanted[1])


def test_noalloc_forward_rejects_what_it_cannot_hold():
    lib = _native.lib()
    sp = torch.cuda.current_stream().cuda_stream
    t = torch.zeros(8, dtype=torch.bfloat16, device=DEV)
    p = t.data_ptr()
    # the chaining words of this shape exceed the static array: refused before anything is touched
    assert lib.fss_workspace_bytes(64, 8192, 4096, _native.FSS_BF16, _native.FSS_FWD, None) > _native.FSS_NOALLOC_SCRATCH_BYTES
    assert lib.fss_scan_fwd_noalloc(_native.FSS_BF16, p, p, p, 64, 8192, 4096, sp) == _native.FSS_ERR_TOO_LARGE
    assert "FSS_NOALLOC_SCRATCH_BYTES" in _native.strerror(_native.FSS_ERR_TOO_LARGE)
    assert lib.fss_scan_fwd_noalloc(_native.FSS_BF16, None, p, p, 1, 4, 2, sp) == 1
    assert lib.fss_scan_fwd_noalloc(_native.FSS_BF16, p, p, p, -1, 4, 2, sp) == 2
    assert lib.fss_scan_fwd_noalloc(7, p, p, p, 1, 4, 2, sp) == 5
    assert lib.fss_scan_fwd_noalloc(_native.FSS_BF16, p, p, p, 0, 4, 2, sp) == 0
    torch.cuda.synchronize()


def test_noalloc_array_is_zeroed_again_before_its_launch_tag_can_wrap():
    """The validity tags of the chaining words are a 32-bit launch counter kept in the array, and
    nobody but the library can reset that array: it counts the calls per device and zeroes the
    array again on the call's stream (nothing allocated) long before the counter wraps.  Here the
    limit is lowered to 3 calls, so a row of calls on a large and a small shape crosses it several
    times; alphas near 1, so that a stale or missing carry would show in every output."""
    lib = _native.lib()
    sp = torch.cuda.current_stream().cuda_stream
    cases = []
    for shape in ((8, 4096, 1024), (2, 1000, 328)):
        alpha, beta, _ = make_inputs("near_one", *shape, seed=3 + sum(shape))
        a, b = alpha.to(DEV), beta.to(DEV)
        cases.append((a, b, _reference(lib, _native.FSS_BF16, a, b, sp)))
    flag = torch.zeros(1, dtype=torch.int32).pin_memory()
    _native.check(lib.fss_workspace_attach_flag(None, flag.data_ptr(), sp))
    previous = lib.fss_debug_noalloc_reinit_after(3)
    try:
        outs = [(torch.full_like(cases[i % 2][0], float("nan")), cases[i % 2][2]) for i in range(11)]
        torch.cuda.synchronize()
        allocated = torch.cuda.memory_allocated()
        for i, (out, _want) in enumerate(outs):
            a, b, _ = cases[i % 2]
            _native.check(lib.fss_scan_fwd_noalloc(_native.FSS_BF16, a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, sp))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == allocated  # the zeroing in between allocates nothing either
        for out, want in outs:
            assert torch.equal(out, want)
        assert lib.fss_workspace_status(None, sp) == 0 and int(flag[0]) == 0
        # a chain time-out in that array is reported like one in a caller's workspace - through the
        # status call and through the attached word, which survived the zeroing above
        limit = lib.fss_debug_set_spin_limit(0)
        try:
            a, b, _want = cases[0]
            out = torch.empty_like(a)
            _native.check(lib.fss_scan_fwd_noalloc(_native.FSS_BF16, a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, sp))
            torch.cuda.synchronize()
        finally:
            lib.fss_debug_set_spin_limit(limit)
        assert int(flag[0]) == 1
        assert lib.fss_workspace_status(None, sp) == _native.FSS_ERR_CHAIN_TIMEOUT
        assert lib.fss_workspace_status(None, sp) == 0
        assert bool(torch.isnan(out.float()).any())
        flag[0] = 0
        # and the array is good again at the next call
        a, b, want = cases[1]
        out = torch.empty_like(a)
        _native.check(lib.fss_scan_fwd_noalloc(_native.FSS_BF16, a.data_ptr(), b.data_ptr(), out.data_ptr(), *a.shape, sp))
        torch.cuda.synchronize()
        assert torch.equal(out, want) and int(flag[0]) == 0
    finally:
        lib.fss_debug_noalloc_reinit_after(previous)
        _native.check(lib.fss_workspace_attach_flag(None, None, sp))
        torch.cuda.synchronize()
