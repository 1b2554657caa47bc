"""CPU-side checks: the C-ABI library loads and exports what include/fss_scan.h
declares, launch planning is sane, the torch wrappers validate their arguments,
and the autograd glue behaves like the reference's (with a CPU stand-in behind
the four extension names, so no kernel runs here)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from fast_sequential_scan_amd import _native, scan_cuda
from fast_sequential_scan_amd import sequential_scan_cuda as ext

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fss_scan.h")).read()
    declared = set(re.findall(r"^(?:int|size_t|uint32_t|int32_t|uint64_t|const char \*)\s*(fss_[a-z0-9_]+)\(", header, flags=re.M))
    assert declared == set(_native.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(_native.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _native.lib().fss_abi_version() == _native.FSS_ABI_VERSION
    assert _native.strerror(0) == "ok"
    assert "workspace" in _native.strerror(4)


def plan_bytes(lib, bs, seq, d, dtype, direction, align):
    """Workspace bytes of the launch the library plans for tensors of this common alignment,
    recomputed from the configuration it reports (4 KiB header + 3 tagged 64-bit words per
    channel slot and tile when the sequence is chained)."""
    cfg = _native.FssConfig()
    assert lib.fss_choose_config(bs, seq, d, dtype, direction, align, ctypes.byref(cfg)) == 0
    chunks = -(-seq // (cfg.steps * (cfg.waves // cfg.cols)))
    tiles = bs * -(-d // (64 * cfg.vec)) * chunks
    return 4096 + (tiles * 3 * 64 * cfg.vec * 8 if chunks > 1 else 0), cfg


def test_workspace_sizing_and_config_choice():
    lib = _native.lib()
    cfg = _native.FssConfig()
    for dtype in (0, 1):
        esize = 2 if dtype == 0 else 4
        for direction in (0, 1):
            for bs, seq, d in [(8, 4096, 1024), (2, 1024, 768), (1, 65521, 256), (16, 2048, 512), (4, 8192, 2048), (3, 1, 7)]:
                assert lib.fss_choose_config(bs, seq, d, dtype, direction, 16, ctypes.byref(cfg)) == 0
                assert d % cfg.vec == 0 and cfg.steps in (8, 16, 32) and 1 <= cfg.waves <= 16
                need = lib.fss_workspace_bytes(bs, seq, d, dtype, direction, None)
                assert need >= 4096 and need % 256 == 0
                assert need <= lib.fss_workspace_bytes_max(bs, seq, d)
                # the answer covers every alignment the tensors may have; the cache policy selects
                # hints on loads and stores, never the tiling, so it cannot change the plan
                per_policy = []
                for policy in (_native.FSS_CACHE_AUTO, _native.FSS_CACHE_STREAMING):
                    previous = lib.fss_set_cache_policy(policy)
                    try:
                        per_policy.append([plan_bytes(lib, bs, seq, d, dtype, direction, a)[0] for a in (2, 4, 8, 16) if a >= esize])
                    finally:
                        lib.fss_set_cache_policy(previous)
                assert per_policy[0] == per_policy[1]
                assert need == max(per_policy[0])
    # the forward at the headline shape (512 tiles: two per CU) takes two column tiles per workgroup,
    # under either policy; the backward and launches of more rounds never do
    for policy in (_native.FSS_CACHE_STREAMING, _native.FSS_CACHE_AUTO):
        previous = lib.fss_set_cache_policy(policy)
        try:
            assert lib.fss_choose_config(8, 4096, 1024, 0, 0, 16, ctypes.byref(cfg)) == 0
            assert (cfg.vec, cfg.steps, cfg.waves, cfg.cols) == (2, 32, 16, 2)
            assert lib.fss_choose_config(8, 4096, 1024, 0, 1, 16, ctypes.byref(cfg)) == 0 and cfg.cols == 1
            assert lib.fss_choose_config(8, 8192, 1024, 0, 0, 16, ctypes.byref(cfg)) == 0 and cfg.cols == 1
        finally:
            lib.fss_set_cache_policy(previous)
    # odd d forces the scalar path; 2-byte alignment too
    assert lib.fss_choose_config(2, 100, 77, 0, 0, 16, ctypes.byref(cfg)) == 0 and cfg.vec == 1
    assert lib.fss_choose_config(2, 100, 64, 0, 0, 2, ctypes.byref(cfg)) == 0 and cfg.vec == 1
    # explicit configurations: bad ones are refused, good ones size the workspace
    bad = _native.FssConfig(3, 8, 1, 0)
    assert lib.fss_workspace_bytes(2, 100, 64, 0, 0, ctypes.byref(bad)) == 4096
    good = _native.FssConfig(2, 8, 2, 0)
    assert lib.fss_workspace_bytes(2, 100, 64, 0, 0, ctypes.byref(good)) == 4096 + 2 * 1 * 7 * 3 * 128 * 8
    assert lib.fss_choose_config(-1, 4, 4, 0, 0, 16, ctypes.byref(cfg)) == 2


def test_wrappers_size_the_workspace_for_any_alignment():
    """What the torch wrappers allocate (the library's answer for the shape, cached per shape) is at
    least what the launch planned for the tensors' real alignment needs: 4000 random shapes, storage
    types, directions and alignments.  A 2-byte aligned bf16 view takes one channel per lane and
    often smaller tiles, which doubles the chaining words against the 16-byte aligned plan."""
    rng = np.random.default_rng(77)
    lib = _native.lib()
    worst = 0.0
    for _ in range(4000):
        bs = int(rng.choice([1, 2, 3, 7, 8, 16, 64]))
        seq = int(rng.choice([1, 31, 256, 257, 1000, 2048, 3000, 4096, 8192, 20000, 65521]))
        d = int(rng.choice([1, 2, 64, 126, 128, 200, 256, 512, 768, 1024, 2048, 4096]))
        dtype = int(rng.integers(0, 3))
        direction = int(rng.integers(0, 4))
        esize = 4 if dtype == _native.FSS_F32 else 2
        align = int(rng.choice([a for a in (2, 4, 8, 16) if a >= esize]))
        allocated = ext._need("rm", dtype, direction, bs, seq, d, None)
        planned, cfg = plan_bytes(lib, bs, seq, d, dtype, direction, align)
        assert allocated >= planned, (bs, seq, d, dtype, direction, align, (cfg.vec, cfg.steps, cfg.waves))
        worst = max(worst, planned / lib.fss_workspace_bytes_max(bs, seq, d))
    assert worst <= 1.0
    # the case that used to fail: bf16 backward, bs 1, seq 4096, d 2048 at a 2-byte offset
    planned, _ = plan_bytes(lib, 1, 4096, 2048, _native.FSS_BF16, _native.FSS_BWD, 2)
    assert ext._need("rm", _native.FSS_BF16, _native.FSS_BWD, 1, 4096, 2048, None) >= planned > 1 << 20
    # channel-major: the sizing call is documented as an upper bound over alignments
    for seq in (4096, 8192, 20000, 65536):
        sizes = {lib.fss_cm_workspace_bytes(4, 256, seq, _native.FSS_BF16, d_, None) for d_ in (0, 1)}
        assert all(sz >= 4096 for sz in sizes)
        assert ext._need("cm", _native.FSS_BF16, _native.FSS_BWD, 4, 256, seq, None) == lib.fss_cm_workspace_bytes(
            4, 256, seq, _native.FSS_BF16, _native.FSS_BWD, None)


def test_entry_points_reject_bad_arguments_without_a_gpu():
    lib = _native.lib()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    assert lib.fss_scan_fwd_bf16(None, p, p, 1, 4, 8, None, 0, None) == 1
    assert lib.fss_scan_fwd_bf16(p, p, p, 1, -4, 8, None, 0, None) == 2
    assert lib.fss_scan_bwd_bf16(p, None, p, p, p, 1, 4, 8, None, 0, None) == 1
    assert lib.fss_scan_fwd_f32(p + 2, p, p, 1, 4, 8, None, 0, None) == 3
    assert lib.fss_scan_fwd_bf16(p, p, p, 0, 4, 8, None, 0, None) == 0  # empty: nothing to do
    assert lib.fss_scan_fwd_ex(7, p, p, p, 1, 4, 8, None, 0, None, None) == 5
    assert lib.fss_workspace_init(None, 1024, None) == 1
    assert lib.fss_copy_bytes(p, p + 1, 16, None) == 3
    assert lib.fss_scan_bwd_state(0, p, p, p, None, None, p, p, p, 1, 4, 8, None, 0, None, None) == 1  # grad_h_before needs h_before
    assert lib.fss_scan_fwd_state(0, p, p, p, p + 2, None, 1, 4, 8, None, 0, None, None) == 3
    two_chunks = _native.FssConfig(1, 8, 1, 0)
    assert lib.fss_scan_fwd_ex(0, p, p, p, 1, 9, 8, None, 0, None, ctypes.byref(two_chunks)) == 4


def test_calibration_kernel_checks_its_arguments_without_a_gpu():
    """fss_stream_mix: stream counts, launch shape, pointers and sizes are checked before anything is
    launched; zero bytes is a valid call that launches nothing."""
    lib = _native.lib()
    buf = (ctypes.c_char * 256)()
    p = ctypes.addressof(buf)
    p += (-p) % 16
    vp = ctypes.c_void_p
    reads, writes = (vp * 3)(p, p + 16, p + 32), (vp * 2)(p + 48, p + 64)
    shape = lambda *v: (ctypes.c_int * 4)(*v)  # noqa: E731
    assert lib.fss_stream_mix(reads, 3, writes, 2, 0, 1, None, None) == 0
    assert lib.fss_stream_mix(reads, 3, writes, 2, 0, 1, shape(512, 256, 2, 1), None) == 0
    assert lib.fss_stream_mix(reads, 0, writes, 1, 0, 1, None, None) == 5
    assert lib.fss_stream_mix(reads, 4, writes, 1, 0, 1, None, None) == 5
    assert lib.fss_stream_mix(reads, 1, writes, 3, 0, 1, None, None) == 5
    for bad in ((0, 256, 1, 0), ((1 << 20) + 1, 256, 1, 0), (2048, 32, 1, 0), (2048, 100, 1, 0), (2048, 2048, 1, 0),
                (2048, 256, 0, 0), (2048, 256, 3, 0), (2048, 256, 1, 2), (2048, 256, 1, -1)):
        assert lib.fss_stream_mix(reads, 3, writes, 2, 0, 1, shape(*bad), None) == 5, bad
    assert lib.fss_stream_mix(reads, 1, None, 0, 0, 1, None, None) == 1          # a read-only run still names a sink
    assert lib.fss_stream_mix(reads, 3, writes, 2, 24, 1, None, None) == 3        # not a multiple of 16 bytes
    assert lib.fss_stream_mix((vp * 3)(p, p + 8, p + 32), 3, writes, 2, 0, 1, None, None) == 3
    assert lib.fss_stream_mix((vp * 3)(p, None, p + 32), 3, writes, 2, 0, 1, None, None) == 1
    assert lib.fss_stream_mix(reads, 2, (vp * 2)(p + 48, None), 2, 0, 1, None, None) == 1


def test_noalloc_entry_point_refuses_oversized_shapes_before_touching_a_device():
    lib = _native.lib()
    buf = (ctypes.c_char * 64)()
    p = ctypes.addressof(buf)
    assert lib.fss_workspace_bytes(64, 8192, 4096, 0, 0, None) > _native.FSS_NOALLOC_SCRATCH_BYTES
    assert lib.fss_scan_fwd_noalloc(0, p, p, p, 64, 8192, 4096, None) == _native.FSS_ERR_TOO_LARGE
    assert lib.fss_scan_fwd_noalloc(0, p, p, p, -1, 4, 4, None) == 2
    assert lib.fss_scan_fwd_noalloc(0, p, p, p, 0, 4, 4, None) == 0
    assert "FSS_NOALLOC_SCRATCH_BYTES" in _native.strerror(_native.FSS_ERR_TOO_LARGE)
    # every measured workload fits the static array, at any alignment
    from fast_sequential_scan_amd.workloads import BASELINE_CASES
    for _recipe, bs, seq, d in BASELINE_CASES.values():
        assert lib.fss_workspace_bytes(bs, seq, d, 0, 0, None) <= _native.FSS_NOALLOC_SCRATCH_BYTES


def test_wrappers_validate_tensors():
    a = torch.zeros(2, 4, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        ext.scan_forward_half(a, a)
    with pytest.raises(TypeError):
        ext.scan_forward_half(a.numpy() if False else None, a)
    meta = torch.device("meta")
    with pytest.raises(RuntimeError):
        ext.scan_forward(torch.zeros(2, 4, 8, device=meta), torch.zeros(2, 4, 8, device=meta))


class _CudaLike:
    """Lets the validation run on CPU tensors that claim to be on a GPU."""

    def __init__(self, t):
        self.t = t


def test_validation_messages(monkeypatch):
    class Fake(torch.Tensor):
        @property
        def is_cuda(self):
            return True

    def fake(*shape, dtype=torch.bfloat16):
        return torch.zeros(*shape, dtype=dtype).as_subclass(Fake)

    with pytest.raises(RuntimeError, match="expected scalar type torch.bfloat16"):
        ext._validate(torch.bfloat16, alpha=fake(2, 4, 8, dtype=torch.float32), beta=fake(2, 4, 8))
    with pytest.raises(RuntimeError, match=r"\(bs, seq, d_model\)"):
        ext._validate(torch.bfloat16, alpha=fake(4, 8), beta=fake(4, 8))
    with pytest.raises(RuntimeError, match="has shape"):
        ext._validate(torch.bfloat16, alpha=fake(2, 4, 8), beta=fake(2, 5, 8))
    assert ext._validate(torch.bfloat16, alpha=fake(2, 4, 8), beta=fake(2, 4, 8)) == (2, 4, 8)


def _install_cpu_stand_in(monkeypatch, oracle):
    def fwd(alpha, beta):
        return torch.from_numpy(oracle.scan_fwd_f32(alpha.detach().numpy(), beta.detach().numpy()))

    def bwd(alpha, h, dout):
        ga, gb = oracle.scan_bwd_f32(alpha.detach().numpy(), h.detach().numpy(), dout.detach().numpy())
        return [torch.from_numpy(ga), torch.from_numpy(gb)]

    monkeypatch.setattr(scan_cuda._ext, "scan_forward", fwd)
    monkeypatch.setattr(scan_cuda._ext, "scan_backward", bwd)


def test_autograd_glue_with_cpu_stand_in(monkeypatch, oracle):
    """SequentialScanSingle wires (alpha, h) into the backward and returns two grads,
    as sequential_scan/scan_cuda.py:36-54 does; checked against autograd through a loop."""
    _install_cpu_stand_in(monkeypatch, oracle)
    g = torch.Generator().manual_seed(0)
    alpha = torch.randn(2, 12, 5, generator=g, requires_grad=True)
    beta = torch.randn(2, 12, 5, generator=g, requires_grad=True)
    dy = torch.randn(2, 12, 5, generator=g)
    out = scan_cuda.scan_single(alpha, beta)
    out.backward(dy)
    ga, gb = alpha.grad.clone(), beta.grad.clone()
    alpha.grad = beta.grad = None
    hs = [beta[:, 0]]
    for t in range(1, 12):
        hs.append(hs[-1] * alpha[:, t] + beta[:, t])
    ref = torch.stack(hs, 1)
    ref.backward(dy)
    np.testing.assert_allclose(out.detach().numpy(), ref.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(ga.numpy(), alpha.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gb.numpy(), beta.grad.numpy(), rtol=1e-4, atol=1e-5)


def test_public_names():
    import fast_sequential_scan_amd as pkg
    import sequential_scan

    assert sequential_scan.scan_cu is pkg.scan_cu and sequential_scan.scan_cu_single is pkg.scan_cu_single
    assert pkg.scan_cu is scan_cuda.scan and pkg.scan_cu_single is scan_cuda.scan_single
    with pytest.raises(NotImplementedError):
        pkg.scan_tr(None, None)


def test_torch_binding_loads_and_declines_what_it_does_not_cover():
    """No GPU here: the C++ dispatch loads, and answers None for tensors it does not take."""
    import torch

    from fast_sequential_scan_amd import sequential_scan_cuda as ext

    binding = ext.fast_dispatch()
    assert binding is not None
    for name in ("init", "scan", "scan_gated", "scan_cm", "scan_state", "register_workspace", "forget_workspaces"):
        assert callable(getattr(binding, name))
    x = torch.zeros(2, 3, 4, dtype=torch.bfloat16)
    assert binding.scan(x, x, 0) is None and binding.scan(x, x, 7) is None
    assert binding.scan_gated(x, x) is None and binding.scan_cm(x, x) is None and binding.scan_state(x, x, None) is None


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_native.NativeLibraryMissing):
        _native.lib()


def test_planning_of_the_gated_fp16_and_channel_major_entry_points():
    lib = _native.lib()
    cfg = _native.FssConfig()

    def choose(dtype, direction, shape=(8, 4096, 1024)):
        assert lib.fss_choose_config(*shape, dtype, direction, 16, ctypes.byref(cfg)) == 0
        return cfg.vec, cfg.steps, cfg.waves

    # gated: 4 bytes per lane; the backward holds four tensors, so never more than 16 steps
    assert choose(_native.FSS_BF16, _native.FSS_GATED_FWD) == (2, 32, 16)
    assert choose(_native.FSS_BF16, _native.FSS_GATED_BWD) == (2, 16, 16)
    assert choose(_native.FSS_F32, _native.FSS_GATED_FWD) == (1, 32, 16)
    assert choose(_native.FSS_F32, _native.FSS_GATED_BWD)[1] <= 16
    assert choose(_native.FSS_BF16, _native.FSS_GATED_BWD, (1, 65521, 256))[1] <= 16
    assert choose(_native.FSS_BF16, _native.FSS_GATED_BWD, (1, 1024, 1024)) == (1, 8, 8)
    # two 8-wave workgroups per CU: long gated forwards, many short gated backwards, ragged last rounds
    assert choose(_native.FSS_BF16, _native.FSS_GATED_FWD, (2, 8192, 1024)) == (2, 32, 8)
    assert choose(_native.FSS_BF16, _native.FSS_GATED_BWD, (2, 8192, 1024)) == (2, 16, 16)
    assert choose(_native.FSS_BF16, _native.FSS_GATED_BWD, (64, 512, 1024)) == (2, 16, 8)
    assert choose(_native.FSS_BF16, _native.FSS_GATED_BWD, (5, 2048, 1024)) == (2, 16, 8)
    assert choose(_native.FSS_BF16, _native.FSS_BWD, (5, 2048, 1024)) == (2, 16, 16)
    # two channels per lane in the forward at every sequence length
    assert choose(_native.FSS_BF16, _native.FSS_FWD, (1, 65521, 256)) == (2, 32, 16)
    assert choose(_native.FSS_BF16, _native.FSS_FWD, (1, 32768, 1024)) == (2, 32, 16)
    # fp32, very large tensors
    assert choose(_native.FSS_F32, _native.FSS_FWD) == (1, 32, 16)
    assert choose(_native.FSS_F32, _native.FSS_FWD, (16, 4096, 1024)) == (1, 16, 16)
    assert choose(_native.FSS_F32, _native.FSS_FWD, (256, 512, 512)) == (2, 16, 16)
    assert choose(_native.FSS_F32, _native.FSS_FWD, (8, 8192, 1024)) == (1, 32, 16)
    assert choose(_native.FSS_F32, _native.FSS_BWD, (16, 4096, 1024)) == (1, 16, 16)
    assert choose(_native.FSS_F32, _native.FSS_BWD, (32, 4096, 1024)) == (2, 8, 16)
    # fp16 plans like bf16
    for direction in (_native.FSS_FWD, _native.FSS_BWD):
        assert choose(_native.FSS_F16, direction) == choose(_native.FSS_BF16, direction)
    assert lib.fss_choose_config(8, 4096, 1024, 3, 0, 16, ctypes.byref(cfg)) == 5
    assert lib.fss_choose_config(8, 4096, 1024, 0, 4, 16, ctypes.byref(cfg)) == 5
    # every direction's workspace fits the documented upper bound
    for shape in [(8, 4096, 1024), (1, 65521, 256), (3, 1, 7)]:
        top = lib.fss_workspace_bytes_max(*shape)
        for dtype in (_native.FSS_BF16, _native.FSS_F32, _native.FSS_F16):
            for direction in range(4):
                assert lib.fss_workspace_bytes(*shape, dtype, direction, None) <= top
    # channel-major: one workgroup of 8 waves reaches 512 timesteps even at one timestep per lane
    assert lib.fss_cm_workspace_bytes(8, 1024, 512, _native.FSS_BF16, _native.FSS_FWD, None) == 4096
    assert lib.fss_cm_workspace_bytes(8, 1024, 8192, _native.FSS_BF16, _native.FSS_BWD, None) > 4096
    assert lib.fss_cm_workspace_bytes(-1, 4, 4, _native.FSS_BF16, _native.FSS_FWD, None) == 4096
    # bad arguments are rejected before any device call
    one = ctypes.c_void_p(256)
    assert lib.fss_gated_scan_fwd(0, None, one, one, 1, 8, 8, None, 0, None, None) == 1
    assert lib.fss_gated_scan_bwd(0, one, None, one, one, one, one, 1, 8, 8, None, 0, None, None) == 1
    assert lib.fss_gated_scan_fwd_state(0, one, one, None, None, None, 1, 8, 8, None, 0, None, None) == 1
    # the gradient with respect to h[-1] needs h[-1]
    assert lib.fss_gated_scan_bwd_state(0, one, one, one, one, None, None, one, one, one, 1, 8, 8, None, 0, None, None) == 1
    assert lib.fss_scan_fwd_cm(0, one, one, None, 1, 8, 8, None, 0, None, None) == 1
    assert lib.fss_scan_bwd_cm(0, one, one, one, None, one, 1, 8, 8, None, 0, None, None) == 1
    assert lib.fss_scan_fwd_cm(0, one, one, one, 1, -8, 8, None, 0, None, None) == 2
    assert lib.fss_scan_fwd_cm(0, ctypes.c_void_p(257), one, one, 1, 8, 8, None, 0, None, None) == 3


def test_shipped_package_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing under the package (or the drop-in shim) may
    import it, name its directory, or fall back to a CPU computation of the scan."""
    offenders = []
    for top in ("fast_sequential_scan_amd", "sequential_scan"):
        for base, _dirs, files in os.walk(os.path.join(ROOT, top)):
            for name in files:
                if not name.endswith((".py", ".hip", ".h")):
                    continue
                text = open(os.path.join(base, name)).read()
                if re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M) or "oracle/" in text:
                    offenders.append(os.path.join(base, name))
    assert not offenders, offenders


def test_common_helpers_follow_their_definitions(oracle):
    """The helper module under the reference's names: the scan's definition against the pinned
    oracle, the metric and its digit rule against hand-computed values."""
    import numpy as np

    from sequential_scan.common import BFLOAT16_TOL, SINGLE_TOL, check_relative_error, relative_error, torch_ref

    g = torch.Generator().manual_seed(5)
    alpha = torch.rand(3, 17, 6, generator=g, dtype=torch.float64).requires_grad_(True)
    beta = torch.randn(3, 17, 6, generator=g, dtype=torch.float64).requires_grad_(True)
    h = torch_ref(alpha, beta)
    np.testing.assert_allclose(h.detach().numpy(), oracle.scan_fwd_f64(alpha.detach().numpy(), beta.detach().numpy()),
                               rtol=1e-13)
    dy = torch.randn(3, 17, 6, generator=g, dtype=torch.float64)
    h.backward(dy)
    assert alpha.grad[:, 0].abs().max() == 0  # alpha[:, 0] is never used
    x, y = torch.tensor([3.0, 4.0]), torch.tensor([0.0, 4.0])
    assert relative_error(x, y) == pytest.approx(3.0 / 4.0)
    assert (SINGLE_TOL, BFLOAT16_TOL) == (7.0, 2.0)
    assert check_relative_error(0.0, 7) and check_relative_error(1e-8, 7) and check_relative_error(9e-7, 7)
    assert not check_relative_error(1.1e-6, 7)
    assert check_relative_error(0.09, 2) and not check_relative_error(0.11, 2)


def test_cache_policy_setter():
    import fast_sequential_scan_amd as pkg

    lib = _native.lib()
    assert lib.fss_set_cache_policy(7) == -1  # unknown: refused, nothing changes
    assert pkg.set_cache_policy("streaming") == "auto"
    assert pkg.set_cache_policy("auto") == "streaming"
    assert lib.fss_set_cache_policy(_native.FSS_CACHE_AUTO) == _native.FSS_CACHE_AUTO
    with pytest.raises(ValueError):
        pkg.set_cache_policy("hot")


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_chosen_configurations_are_valid_for_random_shapes():
    """Property test of the launch planning: whatever the shape, storage type, direction and
    alignment, the chosen configuration is one the kernels accept, never reaches further than the
    sequence needs, and sizes a workspace within the shape's upper bound."""
    rng = np.random.default_rng(2024)
    lib = _native.lib()
    cfg = _native.FssConfig()
    for _ in range(4000):
        bs = int(rng.choice([1, 2, 3, 7, 8, 16, 64, 250]))
        seq = int(rng.choice([1, 2, 5, 31, 64, 255, 256, 257, 1000, 2048, 3000, 4096, 8192, 40000, 65521, 300000]))
        d = int(rng.choice([1, 2, 3, 63, 64, 65, 126, 128, 200, 256, 768, 1024, 1537, 2560, 4096]))
        dtype = int(rng.integers(0, 3))
        direction = int(rng.integers(0, 4))
        align = int(rng.choice([2, 4, 8, 16])) if dtype != _native.FSS_F32 else int(rng.choice([4, 8, 16]))
        what = (bs, seq, d, dtype, direction, align)
        assert lib.fss_choose_config(bs, seq, d, dtype, direction, align, ctypes.byref(cfg)) == 0, what
        esize = 4 if dtype == _native.FSS_F32 else 2
        gated, backward = direction >= 2, direction % 2 == 1
        assert cfg.vec in (1, 2) and d % cfg.vec == 0 and align % (cfg.vec * esize) == 0, what
        assert cfg.steps in (8, 16, 32) and 1 <= cfg.waves <= 16, what
        if gated:
            assert cfg.vec <= (1 if dtype == _native.FSS_F32 else 2), what
            assert not backward or cfg.steps <= 16, what
        # the tile is no longer than the sequence needs: half of it would not cover the sequence
        assert cfg.waves == 1 or cfg.steps * (cfg.waves // 2) < seq, what
        assert cfg.steps == 8 or cfg.steps // 2 < seq, what
        need = lib.fss_workspace_bytes(bs, seq, d, dtype, direction, None)
        assert 4096 <= need <= lib.fss_workspace_bytes_max(bs, seq, d), what
        # the explicit form of the same configuration is accepted, and the workspace sized for the
        # shape (any alignment, the library's own choice) covers it
        explicit = _native.FssConfig(cfg.vec, cfg.steps, cfg.waves, 0)
        assert 4096 <= lib.fss_workspace_bytes(bs, seq, d, dtype, direction, ctypes.byref(explicit)) <= need, what


def _tile_groups(lib, n_groups, grid, n_chunks):
    n_tiles = n_groups * n_chunks
    out = (ctypes.c_int32 * n_tiles)()
    assert lib.fss_debug_tile_groups(n_groups, grid, n_tiles, out) == 0
    return np.frombuffer(out, dtype=np.int32).reshape(n_chunks, n_groups)


def test_tile_order_covers_every_group_of_every_chunk_once():
    """The order in which the kernels take their tiles (which column group a slot of a chunk
    stands for) must be one to one within every chunk, whatever the grid - a collision would
    leave a tile undone and another done twice.  Where the workgroups of an XCD (workgroup
    index modulo 8) share consecutive groups, a column's chunks must stay on one XCD, and
    a workgroup must meet different groups in successive rounds of the grid."""
    lib = _native.lib()
    rng = np.random.default_rng(11)
    cases = [(64, 256, 16), (64, 256, 8), (128, 256, 4), (32, 256, 16), (64, 64, 5), (64, 128, 7), (8, 256, 300),
             (16, 256, 128), (12, 256, 9), (64, 48, 6), (64, 255, 6), (1, 256, 40), (7, 3, 11), (256, 256, 3), (512, 256, 5)]
    cases += [(int(rng.integers(1, 300)), int(rng.integers(1, 300)), int(rng.integers(1, 20))) for _ in range(300)]
    cases += [(8 * int(rng.integers(1, 40)), 8 * int(rng.integers(1, 40)), int(rng.integers(1, 20))) for _ in range(300)]
    rotated = 0
    for n_groups, grid, n_chunks in cases:
        g = _tile_groups(lib, n_groups, grid, n_chunks)
        for c in range(n_chunks):
            assert sorted(g[c].tolist()) == list(range(n_groups)), (n_groups, grid, n_chunks, c)
        if n_groups % 8 == 0:
            # slot s belongs to XCD s % 8 when the grid is a multiple of 8 too; its group lies in that XCD's eighth
            per = n_groups // 8
            assert (g // per == np.arange(n_groups) % 8).all(), (n_groups, grid)
            in_flight = -(-grid // n_groups)
            if per > 1 and n_chunks > in_flight:
                # one round of the grid later, every slot stands for another group of its eighth
                assert (g[0] != g[in_flight]).all(), (n_groups, grid)
                rotated += 1
        else:
            assert (g == np.arange(n_groups)).all()
    assert rotated > 20
    # the headline backward: 64 groups, 256 workgroups, 16 chunks - every workgroup meets 4 different stripes
    g = _tile_groups(lib, 64, 256, 16).reshape(4, 256)
    assert all(len(set(g[:, b].tolist())) == 4 for b in range(256))
    assert lib.fss_debug_tile_groups(0, 256, 0, (ctypes.c_int32 * 1)()) != 0
    assert lib.fss_debug_tile_groups(8, 8, 8, None) != 0


def test_missing_cpp_dispatch_falls_back_to_the_python_wrappers(monkeypatch, tmp_path):
    """The C++ dispatch only shortens the host's way to the launch: when its module is missing or
    does not load, one warning is given and every call goes through the ctypes wrappers over the
    same HIP library (which itself has no stand-in: test_missing_library_raises...).  With
    FSS_TORCH_BINDING=1 the missing module is an error."""
    from fast_sequential_scan_amd import _torch_binding as tb

    monkeypatch.setattr(tb, "_module", None)
    monkeypatch.setattr(tb, "_tried", False)
    monkeypatch.setattr(tb, "PATH", str(tmp_path / "nowhere.so"))
    monkeypatch.delenv("FSS_TORCH_BINDING", raising=False)
    with pytest.warns(RuntimeWarning, match="C\\+\\+ dispatch is not available"):
        assert tb.load(lambda *a: None) is None
    assert tb.load(lambda *a: None) is None  # decided once: no second attempt, no second warning
    # a file that is no extension module: same fallback
    bad = tmp_path / "fss_torch_binding.so"
    bad.write_bytes(b"not an ELF file")
    monkeypatch.setattr(tb, "_tried", False)
    monkeypatch.setattr(tb, "PATH", str(bad))
    with pytest.warns(RuntimeWarning):
        assert tb.load(lambda *a: None) is None
    monkeypatch.setattr(tb, "_tried", False)
    monkeypatch.setenv("FSS_TORCH_BINDING", "1")
    with pytest.raises((tb.TorchBindingMissing, ImportError, OSError)):
        tb.load(lambda *a: None)
