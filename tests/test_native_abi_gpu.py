"""The C ABI from a host written in plain C (tests/native/abi_check.c): no Python, no torch
in the process that calls the library.  The binary is built by `make -C tests/native`
(done by __graft_entry__.build()); here it is only run."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "native", "_build", "abi_check")


def test_plain_c_host_runs_the_scans():
    if not os.path.exists(BINARY):
        pytest.skip("tests/native/_build/abi_check has not been built (make -C tests/native)")
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=100)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.startswith("abi_check ok"), done.stdout


def test_stream_mix_calibration_kernel_moves_what_it_says():
    """fss_stream_mix: writes[0] = XOR of the reads, writes[1] = its complement; read-only runs write nothing."""
    import torch

    from fast_sequential_scan_amd import _native

    dev = "cuda:0"
    n = 1 << 20
    g = torch.Generator(device=dev).manual_seed(1)
    reads = [torch.randint(-2**31, 2**31 - 1, (n,), dtype=torch.int32, device=dev, generator=g) for _ in range(3)]
    sp = torch.cuda.current_stream().cuda_stream
    # launch shapes: the default; two vectors per lane with a grid stride that leaves a ragged tail
    # (4 * 192 * 2 lanes do not divide the 2^18 vectors); 1024-thread workgroups, non-temporal loads
    shapes = (None, (4, 192, 2, 1), (64, 1024, 1, 1), (100000, 64, 2, 0))
    for r in (1, 2, 3):
        for w in (1, 2):
            for nt, shape in ((False, None), (True, None), (True, shapes[1]), (False, shapes[2]), (True, shapes[3])):
                outs = [torch.zeros(n, dtype=torch.int32, device=dev) for _ in range(w)]
                _native.stream_mix([t.data_ptr() for t in reads[:r]], [t.data_ptr() for t in outs], 4 * n, nt, sp,
                                   shape=shape)
                want = reads[0].clone()
                for t in reads[1:r]:
                    want ^= t
                torch.cuda.synchronize()
                assert torch.equal(outs[0], want)
                if w == 2:
                    assert torch.equal(outs[1], ~want)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    _native.stream_mix([t.data_ptr() for t in reads], [], 4 * n, True, sp, sink.data_ptr())
    torch.cuda.synchronize()
    assert int(sink.abs().sum()) == 0
    lib = _native.lib()
    assert lib.fss_stream_mix(None, 1, None, 0, 16, 0, None, None) != 0
    for bad in ((0, 256, 1, 0), (2048, 100, 1, 0), (2048, 2048, 1, 0), (2048, 256, 3, 0), (2048, 256, 1, 2)):
        with pytest.raises(_native.FssError):
            _native.stream_mix([reads[0].data_ptr()], [], 4 * n, True, sp, sink.data_ptr(), shape=bad)
