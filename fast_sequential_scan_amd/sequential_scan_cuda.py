"""The four callees the reference's autograd Functions import from its compiled
extension (``from sequential_scan_cuda import scan_forward, scan_backward,
scan_forward_half, scan_backward_half``: sequential_scan/scan_cuda.py:4-9,
registered in csrc/sequential_scan.cpp:15-22), here as thin torch-tensor
wrappers over the C ABI of the HIP library.

Same names, argument order and return structure.  Differences, all supersets:
  * any ``d_model`` and any ``seq >= 1`` (the reference throws for d outside
    {512,768,1024,1536,2048}: csrc/sequential_scan_kernel.cu:54);
  * inputs are validated (device, dtype, rank, equal shapes) and made contiguous;
    the reference checks nothing;
  * kernels run on the current torch stream, not the legacy default stream;
  * ``scan_backward_half`` returns a fresh ``grad_beta``; the reference returns
    ``h_saved`` overwritten in place (csrc/sequential_scan_kernel.cu:197).
"""
from __future__ import annotations

import contextlib
import ctypes
from typing import Dict, List, Optional, Tuple

import torch

from . import _native, _torch_binding

__all__ = [
    "scan_forward", "scan_backward", "scan_forward_half", "scan_backward_half",
    "scan_forward_fp16", "scan_backward_fp16",
    "scan_forward_state", "scan_backward_state",
    "gated_scan_forward", "gated_scan_backward", "gated_scan_forward_state", "gated_scan_backward_state",
    "scan_forward_cm", "scan_backward_cm", "set_cache_policy",
]

_DTYPE_CODE = {torch.bfloat16: _native.FSS_BF16, torch.float32: _native.FSS_F32, torch.float16: _native.FSS_F16}
_CODE_DTYPE = {code: dtype for dtype, code in _DTYPE_CODE.items()}

# one workspace per (device, stream): calls on one stream are ordered, calls on
# different streams must not share the chaining words
_workspaces: Dict[Tuple[int, int], "_Workspace"] = {}
# workspaces replaced by larger ones: their host-side words (the pinned time-out flag, the launch
# count) stay alive for the rest of the process, because scans already enqueued may still set the
# flag and a backward on an autograd thread may have looked the old entry up just before it was
# replaced; only the device buffer goes back to the allocator (its reuse is ordered by the stream)
_retired: List["_Workspace"] = []

# the validity tags in a workspace are a 32-bit launch counter: reset long before it wraps
_REINIT_AFTER_LAUNCHES = 1 << 31

# bytes of workspace per (entry-point family, dtype code, direction, bs, seq, d, config): the
# library's answer covers every alignment of the tensors, so it is a pure function of these
_need_cache: Dict[tuple, int] = {}


class _Workspace:
    """The chaining words of one (device, stream) plus a pinned host word the kernels set when a
    chunk gives up waiting for its predecessor: read on the host, at the next call, with a plain
    memory read - no device call, no synchronisation."""

    __slots__ = ("buf", "ptr", "size", "launches", "flag", "flag_word")

    def __init__(self, buf: torch.Tensor, stream_handle: int):
        lib = _native.lib()
        self.buf = buf
        self.ptr = buf.data_ptr()
        self.size = buf.numel()
        # (a C integer: the C++ dispatch of the plain scan counts its launches into the same word)
        self.launches = ctypes.c_int64(0)
        self.flag = torch.zeros(1, dtype=torch.int32).pin_memory()
        self.flag_word = ctypes.c_uint32.from_address(self.flag.data_ptr())
        _native.check(lib.fss_workspace_init(self.ptr, self.size, stream_handle))
        _native.check(lib.fss_workspace_attach_flag(self.ptr, self.flag.data_ptr(), stream_handle))

    def reinit(self, stream_handle: int) -> None:
        lib = _native.lib()
        _native.check(lib.fss_workspace_init(self.ptr, self.size, stream_handle))
        _native.check(lib.fss_workspace_attach_flag(self.ptr, self.flag.data_ptr(), stream_handle))
        self.launches.value = 0

    def raise_if_flagged(self) -> None:
        if self.flag_word.value:
            self.flag_word.value = 0
            raise _native.FssError(
                _native.FSS_ERR_CHAIN_TIMEOUT,
                _native.strerror(_native.FSS_ERR_CHAIN_TIMEOUT)
                + ": an earlier scan on this stream was starved of compute units (another process or a "
                "concurrently replayed graph holding them); its outputs are NaN from the affected chunk on",
            )


def _validate(expected: torch.dtype, **tensors: torch.Tensor) -> Tuple[int, int, int]:
    first_name = first = None
    for name, t in tensors.items():
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
        if not t.is_cuda:
            raise RuntimeError(f"{name} must live on a GPU (got device {t.device})")
        if t.dtype != expected:
            raise RuntimeError(f"expected scalar type {expected} for {name} but found {t.dtype}")
        if t.dim() != 3:
            raise RuntimeError(f"{name} must have shape (bs, seq, d_model), got {tuple(t.shape)}")
        if first is None:
            first_name, first = name, t
            continue
        if t.device != first.device:
            raise RuntimeError(f"{name} is on {t.device} but {first_name} is on {first.device}")
        if t.shape != first.shape:
            raise RuntimeError(
                f"{name} has shape {tuple(t.shape)} but {first_name} has shape {tuple(first.shape)}"
            )
    bs, seq, d = first.shape
    return bs, seq, d


class _RawStream:
    """The current stream of the current device as the launch sites need it: its handle."""

    __slots__ = ("cuda_stream",)

    def __init__(self, handle: int):
        self.cuda_stream = handle


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_NO_SWITCH = contextlib.nullcontext()


def _current_stream() -> "_RawStream":
    # the raw handle costs a tenth of building a torch.cuda.Stream object per call
    if _raw_stream is not None:
        return _RawStream(_raw_stream(torch.cuda.current_device()))
    return _RawStream(torch.cuda.current_stream().cuda_stream)


def _on(device: torch.device):
    """Context that makes `device` current - nothing to enter when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def _need(family: str, code: int, direction: int, bs: int, seq: int, d: int, config) -> int:
    """Workspace bytes of one entry-point family ("rm": fss_workspace_bytes with (bs, seq, d);
    "cm": fss_cm_workspace_bytes with (bs, d, seq)); asked of the library once per key."""
    key = (family, code, direction, bs, seq, d, config if config is None else tuple(config))
    need = _need_cache.get(key)
    if need is None:
        lib = _native.lib()
        sizer = lib.fss_workspace_bytes if family == "rm" else lib.fss_cm_workspace_bytes
        need = int(sizer(bs, seq, d, code, direction, _native.make_config(config)))
        if len(_need_cache) > 4096:
            _need_cache.clear()
        _need_cache[key] = need
    return need


def _need_plain(code: int, bs: int, seq: int, d: int, config) -> int:
    """Workspace bytes of the plain scan, forward or backward: one workspace serves both, and the
    C++ dispatch of `scan_cu` only takes a call whose backward it can serve too."""
    return max(_need("rm", code, _native.FSS_FWD, bs, seq, d, config),
               _need("rm", code, _native.FSS_BWD, bs, seq, d, config))


def _need_gated(code: int, bs: int, seq: int, d: int, config) -> int:
    """The same for the gated scan."""
    return max(_need("rm", code, _native.FSS_GATED_FWD, bs, seq, d, config),
               _need("rm", code, _native.FSS_GATED_BWD, bs, seq, d, config))


def _need_cm(code: int, bs: int, d: int, seq: int, config) -> int:
    """The same for the channel-major scan."""
    return max(_need("cm", code, _native.FSS_FWD, bs, d, seq, config),
               _need("cm", code, _native.FSS_BWD, bs, d, seq, config))


def _workspace(device: torch.device, stream: "_RawStream", need: int) -> "_Workspace":
    """The workspace of (device, stream), grown to `need` bytes; raises if a scan launched through
    it earlier reported a chain time-out."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.size < need:
        if ws is not None:
            ws.raise_if_flagged()
        old = ws
        ws = _Workspace(torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=device), stream.cuda_stream)
        # the C++ dispatch learns of the new workspace before the old one lets go of anything
        binding = _torch_binding.loaded()
        if binding is not None:
            binding.register_workspace(
                key[0], key[1], ws.ptr, ws.size, ws.flag.data_ptr(), ctypes.addressof(ws.launches))
        _workspaces[key] = ws
        if old is not None:
            old.buf = None
            _retired.append(old)
    else:
        if ws.flag_word.value:
            ws.raise_if_flagged()
        if ws.launches.value >= _REINIT_AFTER_LAUNCHES:
            ws.reinit(stream.cuda_stream)
    ws.launches.value += 1
    return ws


def _slow_backward(kind: int, code: int, saved: List[torch.Tensor], grad_out: torch.Tensor):
    """What the C++ dispatch calls back for a backward it does not cover (kind 0: the plain scan,
    saved (alpha, h); kind 1: the gated scan, saved (gate, x, h))."""
    if kind == 1:
        return gated_scan_backward(saved[0], saved[1], saved[2], grad_out)
    if kind == 2:  # channel-major, saved (alpha, h)
        return scan_backward_cm(saved[0], saved[1], grad_out)
    return _backward(_CODE_DTYPE[code], saved[0], saved[1], grad_out)


def fast_dispatch():
    """The C++ dispatch of the plain and the gated scan (None when switched off), knowing every workspace that
    exists so far; later ones are registered as they are made."""
    binding = _torch_binding.loaded()
    if binding is None:
        binding = _torch_binding.load(_slow_backward)
        if binding is not None:
            for (device, stream), ws in _workspaces.items():
                binding.register_workspace(
                    device, stream, ws.ptr, ws.size, ws.flag.data_ptr(), ctypes.addressof(ws.launches))
    return binding


def _contiguous(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


_CACHE_POLICIES = {"auto": _native.FSS_CACHE_AUTO, "streaming": _native.FSS_CACHE_STREAMING}


def set_cache_policy(policy: str) -> str:
    """Process-wide: ``"auto"`` (default) assumes the tensors of a step are touched again soon (a
    benchmark loop, a short pipeline); ``"streaming"`` assumes nothing is found in the memory-side
    cache again (a scan inside a large model) and marks the forward's output and the backward's
    reads of ``dout`` as streaming at every size.  Results are bit-identical.  Returns the previous
    policy."""
    if policy not in _CACHE_POLICIES:
        raise ValueError(f"unknown cache policy {policy!r}: expected one of {sorted(_CACHE_POLICIES)}")
    previous = _native.lib().fss_set_cache_policy(_CACHE_POLICIES[policy])
    return next(name for name, code in _CACHE_POLICIES.items() if code == previous)


def workspace_status(device: Optional[torch.device] = None) -> None:
    """Synchronises the current stream and raises if a chained scan launched on it timed out."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    with torch.cuda.device(device):
        stream = _current_stream()
        ws = _workspaces.get((device.index, stream.cuda_stream))
        if ws is not None:
            try:
                _native.check(_native.lib().fss_workspace_status(ws.ptr, stream.cuda_stream))
            finally:
                ws.flag_word.value = 0


def _same_kind(dtype: torch.dtype, first, *others) -> bool:
    """The common case of _validate in a few attribute reads: GPU tensors of `dtype`, rank 3, one
    shape, one device.  Anything else goes through _validate, which names what is wrong."""
    try:
        if first.dtype is not dtype or not first.is_cuda or first.dim() != 3:
            return False
        shape, device = first.shape, first.device
        for t in others:
            if t.dtype is not dtype or t.shape != shape or t.device != device:
                return False
        return True
    except AttributeError:  # not a tensor
        return False


def _forward(dtype: torch.dtype, alpha: torch.Tensor, beta: torch.Tensor, config=None) -> torch.Tensor:
    if _same_kind(dtype, alpha, beta):
        bs, seq, d = alpha.shape
    else:
        bs, seq, d = _validate(dtype, alpha=alpha, beta=beta)
    alpha, beta = _contiguous(alpha), _contiguous(beta)
    out = torch.empty_like(alpha)
    if out.numel() == 0:
        return out
    code = _DTYPE_CODE[dtype]
    with _on(alpha.device):
        stream = _current_stream()
        ws = _workspace(alpha.device, stream, _need_plain(code, bs, seq, d, config))
        rc = _native.lib().fss_scan_fwd_ex(
            code, alpha.data_ptr(), beta.data_ptr(), out.data_ptr(), bs, seq, d,
            ws.ptr, ws.size, stream.cuda_stream, _native.make_config(config),
        )
        if rc:
            _native.check(rc)
    return out


def _backward(
    dtype: torch.dtype, alpha_saved: torch.Tensor, h_saved: torch.Tensor, grad_out: torch.Tensor, config=None,
    overwrite_grad_out: bool = False,
) -> List[torch.Tensor]:
    if _same_kind(dtype, alpha_saved, h_saved, grad_out):
        bs, seq, d = alpha_saved.shape
    else:
        bs, seq, d = _validate(dtype, alpha_saved=alpha_saved, h_saved=h_saved, grad_out=grad_out)
    alpha_saved, h_saved, grad_out = _contiguous(alpha_saved), _contiguous(h_saved), _contiguous(grad_out)
    grad_alpha = torch.empty_like(alpha_saved)
    # grad_beta over grad_out itself is the one overlap the kernels allow (every lane reads its rows
    # of dout before it stores them): one allocation per backward, as in the reference
    grad_beta = grad_out if overwrite_grad_out else torch.empty_like(alpha_saved)
    if grad_alpha.numel() == 0:
        return [grad_alpha, grad_beta]
    code = _DTYPE_CODE[dtype]
    with _on(alpha_saved.device):
        stream = _current_stream()
        ws = _workspace(alpha_saved.device, stream, _need_plain(code, bs, seq, d, config))
        rc = _native.lib().fss_scan_bwd_ex(
            code, alpha_saved.data_ptr(), h_saved.data_ptr(), grad_out.data_ptr(),
            grad_alpha.data_ptr(), grad_beta.data_ptr(), bs, seq, d,
            ws.ptr, ws.size, stream.cuda_stream, _native.make_config(config),
        )
        if rc:
            _native.check(rc)
    return [grad_alpha, grad_beta]


def scan_forward(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """fp32 forward: csrc/sequential_scan.cpp:15 / sequential_scan_kernel.cu:7-58."""
    return _forward(torch.float32, alpha, beta)


def scan_backward(alpha_saved: torch.Tensor, h_saved: torch.Tensor, grad_out: torch.Tensor,
                  overwrite_grad_out: bool = False) -> List[torch.Tensor]:
    """fp32 backward -> [grad_alpha, grad_beta]: csrc/sequential_scan.cpp:17 / sequential_scan_kernel.cu:60-124.
    ``overwrite_grad_out=True`` writes grad_beta over a contiguous ``grad_out`` (not for use inside
    autograd, which owns the gradients it hands to a backward)."""
    return _backward(torch.float32, alpha_saved, h_saved, grad_out, overwrite_grad_out=overwrite_grad_out)


def scan_forward_half(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """bf16 forward: csrc/sequential_scan.cpp:19 / sequential_scan_kernel.cu:126-187."""
    return _forward(torch.bfloat16, alpha, beta)


def scan_backward_half(alpha_saved: torch.Tensor, h_saved: torch.Tensor, grad_out: torch.Tensor,
                       overwrite_grad_out: bool = False) -> List[torch.Tensor]:
    """bf16 backward -> [grad_alpha, grad_beta]: csrc/sequential_scan.cpp:21 / sequential_scan_kernel.cu:189-268.
    The reference returns ``h_saved`` overwritten with grad_beta (sequential_scan_kernel.cu:197), i.e. it
    allocates one tensor; ``overwrite_grad_out=True`` gets the same footprint here by writing grad_beta
    over a contiguous ``grad_out`` (not for use inside autograd, which owns the gradients it hands out)."""
    return _backward(torch.bfloat16, alpha_saved, h_saved, grad_out, overwrite_grad_out=overwrite_grad_out)


def scan_forward_fp16(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """IEEE half forward (no counterpart in the reference; same kernels, fp32 carries)."""
    return _forward(torch.float16, alpha, beta)


def scan_backward_fp16(alpha_saved: torch.Tensor, h_saved: torch.Tensor, grad_out: torch.Tensor) -> List[torch.Tensor]:
    """IEEE half backward -> [grad_alpha, grad_beta]."""
    return _backward(torch.float16, alpha_saved, h_saved, grad_out)


# ---- scans with a state entering and leaving the sequence (no counterpart in the reference) ----


def _state(name: str, t: Optional[torch.Tensor], like: torch.Tensor) -> Optional[torch.Tensor]:
    if t is None:
        return None
    bs, _, d = like.shape
    if not t.is_cuda or t.device != like.device:
        raise RuntimeError(f"{name} must be on {like.device}")
    if t.dtype != torch.float32:
        raise RuntimeError(f"expected scalar type torch.float32 for {name} but found {t.dtype}")
    if tuple(t.shape) != (bs, d):
        raise RuntimeError(f"{name} must have shape (bs, d_model) = {(bs, d)}, got {tuple(t.shape)}")
    return t.contiguous()


def scan_forward_state(
    alpha: torch.Tensor, beta: torch.Tensor, h_before: Optional[torch.Tensor] = None, config=None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(h, h_last): the scan started from ``h[-1] = h_before`` (fp32 ``(bs, d)``, zeros when None;
    given, ``alpha[:, 0]`` is applied to it) and the un-rounded fp32 state after the last step."""
    dtype = alpha.dtype
    if dtype not in _DTYPE_CODE:
        raise RuntimeError(f"expected scalar type torch.bfloat16, torch.float16 or torch.float32 for alpha but found {dtype}")
    bs, seq, d = _validate(dtype, alpha=alpha, beta=beta)
    h_before = _state("h_before", h_before, alpha)
    alpha, beta = alpha.contiguous(), beta.contiguous()
    out = torch.empty_like(alpha, memory_format=torch.contiguous_format)
    if out.numel() == 0:
        h_last = torch.zeros((bs, d), dtype=torch.float32, device=alpha.device)
        if h_before is not None and seq == 0:
            h_last.copy_(h_before)
        return out, h_last
    # (every channel's entry is written by the wave that holds the sequence's last step)
    h_last = torch.empty((bs, d), dtype=torch.float32, device=alpha.device)
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    with _on(alpha.device):
        stream = _current_stream()
        ws = _workspace(alpha.device, stream, _need_plain(code, bs, seq, d, config))
        _native.check(
            lib.fss_scan_fwd_state(
                code, alpha.data_ptr(), beta.data_ptr(), out.data_ptr(),
                h_before.data_ptr() if h_before is not None else None, h_last.data_ptr(),
                bs, seq, d, ws.ptr, ws.size, stream.cuda_stream, _native.make_config(config),
            )
        )
    return out, h_last


def scan_backward_state(
    alpha_saved: torch.Tensor,
    h_saved: torch.Tensor,
    grad_out: torch.Tensor,
    h_before: Optional[torch.Tensor] = None,
    grad_h_last: Optional[torch.Tensor] = None,
    config=None,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """(grad_alpha, grad_beta, grad_h_before); the last is None when ``h_before`` is None."""
    dtype = alpha_saved.dtype
    if dtype not in _DTYPE_CODE:
        raise RuntimeError(f"expected scalar type torch.bfloat16, torch.float16 or torch.float32 for alpha but found {dtype}")
    bs, seq, d = _validate(dtype, alpha_saved=alpha_saved, h_saved=h_saved, grad_out=grad_out)
    h_before = _state("h_before", h_before, alpha_saved)
    grad_h_last = _state("grad_h_last", grad_h_last, alpha_saved)
    alpha_saved, h_saved, grad_out = alpha_saved.contiguous(), h_saved.contiguous(), grad_out.contiguous()
    grad_alpha = torch.empty_like(alpha_saved, memory_format=torch.contiguous_format)
    grad_beta = torch.empty_like(alpha_saved, memory_format=torch.contiguous_format)
    grad_h_before = torch.zeros((bs, d), dtype=torch.float32, device=alpha_saved.device) if h_before is not None else None
    if grad_alpha.numel() == 0:
        if grad_h_before is not None and grad_h_last is not None and seq == 0:
            grad_h_before.copy_(grad_h_last)
        return grad_alpha, grad_beta, grad_h_before
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    with _on(alpha_saved.device):
        stream = _current_stream()
        ws = _workspace(alpha_saved.device, stream, _need_plain(code, bs, seq, d, config))
        _native.check(
            lib.fss_scan_bwd_state(
                code, alpha_saved.data_ptr(), h_saved.data_ptr(), grad_out.data_ptr(),
                h_before.data_ptr() if h_before is not None else None,
                grad_h_last.data_ptr() if grad_h_last is not None else None,
                grad_alpha.data_ptr(), grad_beta.data_ptr(),
                grad_h_before.data_ptr() if grad_h_before is not None else None,
                bs, seq, d, ws.ptr, ws.size, stream.cuda_stream, _native.make_config(config),
            )
        )
    return grad_alpha, grad_beta, grad_h_before


# ---- gated scan: alpha = sigmoid(gate), beta = x*sqrt(1-alpha^2) inside the kernel (no counterpart
# in the reference, which is handed alpha and beta) ----


def _either_dtype(t: torch.Tensor, name: str) -> torch.dtype:
    if t.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"expected scalar type torch.bfloat16, torch.float16 or torch.float32 for {name} but found {t.dtype}")
    return t.dtype


def gated_scan_forward(gate: torch.Tensor, x: torch.Tensor, config=None) -> torch.Tensor:
    """h of the scan with ``alpha = sigmoid(gate)`` and ``beta = x * sqrt(1 - alpha**2)``."""
    dtype = _either_dtype(gate, "gate")
    bs, seq, d = _validate(dtype, gate=gate, x=x)
    gate, x = gate.contiguous(), x.contiguous()
    out = torch.empty_like(gate, memory_format=torch.contiguous_format)
    if out.numel() == 0:
        return out
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    cfg = _native.make_config(config)
    with _on(gate.device):
        stream = _current_stream()
        ws = _workspace(gate.device, stream, _need_gated(code, bs, seq, d, config))
        _native.check(
            lib.fss_gated_scan_fwd(
                code, gate.data_ptr(), x.data_ptr(), out.data_ptr(), bs, seq, d,
                ws.ptr, ws.size, stream.cuda_stream, cfg,
            )
        )
    return out


def gated_scan_backward(
    gate: torch.Tensor, x: torch.Tensor, h_saved: torch.Tensor, grad_out: torch.Tensor, config=None
) -> List[torch.Tensor]:
    """[grad_gate, grad_x] of :func:`gated_scan_forward`, given its inputs and stored output."""
    dtype = _either_dtype(gate, "gate")
    bs, seq, d = _validate(dtype, gate=gate, x=x, h_saved=h_saved, grad_out=grad_out)
    gate, x, h_saved, grad_out = gate.contiguous(), x.contiguous(), h_saved.contiguous(), grad_out.contiguous()
    grad_gate = torch.empty_like(gate, memory_format=torch.contiguous_format)
    grad_x = torch.empty_like(gate, memory_format=torch.contiguous_format)
    if grad_gate.numel() == 0:
        return [grad_gate, grad_x]
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    cfg = _native.make_config(config)
    with _on(gate.device):
        stream = _current_stream()
        ws = _workspace(gate.device, stream, _need_gated(code, bs, seq, d, config))
        _native.check(
            lib.fss_gated_scan_bwd(
                code, gate.data_ptr(), x.data_ptr(), h_saved.data_ptr(), grad_out.data_ptr(),
                grad_gate.data_ptr(), grad_x.data_ptr(), bs, seq, d,
                ws.ptr, ws.size, stream.cuda_stream, cfg,
            )
        )
    return [grad_gate, grad_x]


def gated_scan_forward_state(
    gate: torch.Tensor, x: torch.Tensor, h_before: Optional[torch.Tensor] = None, config=None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(h, h_last) of the gated scan started from ``h[-1] = h_before`` (fp32 ``(bs, d)``, zeros when
    None); ``h_last`` is the un-rounded fp32 state after the last step."""
    dtype = _either_dtype(gate, "gate")
    bs, seq, d = _validate(dtype, gate=gate, x=x)
    h_before = _state("h_before", h_before, gate)
    gate, x = gate.contiguous(), x.contiguous()
    out = torch.empty_like(gate, memory_format=torch.contiguous_format)
    h_last = torch.zeros((bs, d), dtype=torch.float32, device=gate.device)
    if out.numel() == 0:
        if h_before is not None and seq == 0:
            h_last.copy_(h_before)
        return out, h_last
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    cfg = _native.make_config(config)
    with _on(gate.device):
        stream = _current_stream()
        ws = _workspace(gate.device, stream, _need_gated(code, bs, seq, d, config))
        _native.check(
            lib.fss_gated_scan_fwd_state(
                code, gate.data_ptr(), x.data_ptr(), out.data_ptr(),
                h_before.data_ptr() if h_before is not None else None, h_last.data_ptr(),
                bs, seq, d, ws.ptr, ws.size, stream.cuda_stream, cfg,
            )
        )
    return out, h_last


def gated_scan_backward_state(
    gate: torch.Tensor,
    x: torch.Tensor,
    h_saved: torch.Tensor,
    grad_out: torch.Tensor,
    h_before: Optional[torch.Tensor] = None,
    grad_h_last: Optional[torch.Tensor] = None,
    config=None,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """(grad_gate, grad_x, grad_h_before); the last is None when ``h_before`` is None."""
    dtype = _either_dtype(gate, "gate")
    bs, seq, d = _validate(dtype, gate=gate, x=x, h_saved=h_saved, grad_out=grad_out)
    h_before = _state("h_before", h_before, gate)
    grad_h_last = _state("grad_h_last", grad_h_last, gate)
    gate, x, h_saved, grad_out = gate.contiguous(), x.contiguous(), h_saved.contiguous(), grad_out.contiguous()
    grad_gate = torch.empty_like(gate, memory_format=torch.contiguous_format)
    grad_x = torch.empty_like(gate, memory_format=torch.contiguous_format)
    grad_h_before = torch.zeros((bs, d), dtype=torch.float32, device=gate.device) if h_before is not None else None
    if grad_gate.numel() == 0:
        if grad_h_before is not None and grad_h_last is not None and seq == 0:
            grad_h_before.copy_(grad_h_last)
        return grad_gate, grad_x, grad_h_before
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    cfg = _native.make_config(config)
    with _on(gate.device):
        stream = _current_stream()
        ws = _workspace(gate.device, stream, _need_gated(code, bs, seq, d, config))
        _native.check(
            lib.fss_gated_scan_bwd_state(
                code, gate.data_ptr(), x.data_ptr(), h_saved.data_ptr(), grad_out.data_ptr(),
                h_before.data_ptr() if h_before is not None else None,
                grad_h_last.data_ptr() if grad_h_last is not None else None,
                grad_gate.data_ptr(), grad_x.data_ptr(),
                grad_h_before.data_ptr() if grad_h_before is not None else None,
                bs, seq, d, ws.ptr, ws.size, stream.cuda_stream, cfg,
            )
        )
    return grad_gate, grad_x, grad_h_before


# ---- channel-major layout: tensors (bs, d_model, seq), time contiguous (what the accelerated-scan
# package takes; the reference permutes to it in benchmark.py:67-72) ----


def scan_forward_cm(alpha: torch.Tensor, beta: torch.Tensor, config=None) -> torch.Tensor:
    """h for ``(bs, d_model, seq)`` tensors: the same recurrence along the last axis."""
    dtype = _either_dtype(alpha, "alpha")
    bs, d, seq = _validate(dtype, alpha=alpha, beta=beta)
    alpha, beta = alpha.contiguous(), beta.contiguous()
    out = torch.empty_like(alpha, memory_format=torch.contiguous_format)
    if out.numel() == 0:
        return out
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    cfg = _native.make_config(config)
    with _on(alpha.device):
        stream = _current_stream()
        ws = _workspace(alpha.device, stream, _need_cm(code, bs, d, seq, config))
        _native.check(
            lib.fss_scan_fwd_cm(
                code, alpha.data_ptr(), beta.data_ptr(), out.data_ptr(), bs, d, seq,
                ws.ptr, ws.size, stream.cuda_stream, cfg,
            )
        )
    return out


def scan_backward_cm(
    alpha_saved: torch.Tensor, h_saved: torch.Tensor, grad_out: torch.Tensor, config=None
) -> List[torch.Tensor]:
    """[grad_alpha, grad_beta] for ``(bs, d_model, seq)`` tensors."""
    dtype = _either_dtype(alpha_saved, "alpha_saved")
    bs, d, seq = _validate(dtype, alpha_saved=alpha_saved, h_saved=h_saved, grad_out=grad_out)
    alpha_saved, h_saved, grad_out = alpha_saved.contiguous(), h_saved.contiguous(), grad_out.contiguous()
    grad_alpha = torch.empty_like(alpha_saved, memory_format=torch.contiguous_format)
    grad_beta = torch.empty_like(alpha_saved, memory_format=torch.contiguous_format)
    if grad_alpha.numel() == 0:
        return [grad_alpha, grad_beta]
    lib = _native.lib()
    code = _DTYPE_CODE[dtype]
    cfg = _native.make_config(config)
    with _on(alpha_saved.device):
        stream = _current_stream()
        ws = _workspace(alpha_saved.device, stream, _need_cm(code, bs, d, seq, config))
        _native.check(
            lib.fss_scan_bwd_cm(
                code, alpha_saved.data_ptr(), h_saved.data_ptr(), grad_out.data_ptr(),
                grad_alpha.data_ptr(), grad_beta.data_ptr(), bs, d, seq,
                ws.ptr, ws.size, stream.cuda_stream, cfg,
            )
        )
    return [grad_alpha, grad_beta]
