"""Autograd Functions over the HIP scan, with the public surface of the
reference's sequential_scan/scan_cuda.py: ``SequentialScan`` (bf16, autocast
aware), ``SequentialScanSingle`` (fp32), ``scan`` and ``scan_single``.

Both Functions save ``(alpha, h)`` - the output itself, no extra activation
memory (reference scan_cuda.py:20,42) - and the backward returns
``(grad_alpha, grad_beta)``.
"""
from __future__ import annotations

from typing import Any, Optional, Tuple

import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import sequential_scan_cuda as _ext

__all__ = [
    "SequentialScan", "SequentialScanSingle", "SequentialScanFp16", "SequentialScanState", "SequentialScanGated",
    "SequentialScanChannelMajor", "SequentialScanGatedState", "scan", "scan_single", "scan_fp16", "scan_with_state",
    "scan_gated", "scan_gated_with_state", "scan_cm",
]


def _autocast_to_bf16(t: torch.Tensor) -> torch.Tensor:
    # what torch.amp.custom_fwd(cast_inputs=torch.bfloat16) casts: floating-point GPU tensors
    if isinstance(t, torch.Tensor) and t.is_cuda and t.is_floating_point() and t.dtype != torch.bfloat16:
        return t.to(torch.bfloat16)
    return t


class SequentialScan(Function):
    """bf16 scan.  Under ``torch.autocast('cuda')`` floating inputs are cast to
    bf16 and autocast is switched off inside, as the reference's
    ``custom_fwd(cast_inputs=torch.bfloat16)`` does (scan_cuda.py:15); outside
    autocast a non-bf16 input is an error, as it is there.

    The two decorators of the reference are spelled out here: they build an autocast context
    per call, tens of microseconds per training step for kernels that take as long, and the
    backward (``custom_bwd``, scan_cuda.py:25: "run under the forward's autocast state") calls
    nothing that autocast affects."""

    @staticmethod
    def forward(ctx: Any, input_alpha: torch.Tensor, input_beta: torch.Tensor) -> torch.Tensor:
        if torch.is_autocast_enabled("cuda"):
            with torch.autocast("cuda", enabled=False):
                input_alpha, input_beta = _autocast_to_bf16(input_alpha), _autocast_to_bf16(input_beta)
                h = _ext.scan_forward_half(input_alpha, input_beta)
        else:
            h = _ext.scan_forward_half(input_alpha, input_beta)
        ctx.save_for_backward(input_alpha, h)
        return h

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        input_alpha, h = ctx.saved_tensors
        alpha_grad, beta_grad = _ext.scan_backward_half(input_alpha, h, grad_output)
        return alpha_grad, beta_grad


class SequentialScanSingle(Function):
    """fp32 scan (reference scan_cuda.py:36-54)."""

    @staticmethod
    def forward(ctx: Any, input_alpha: torch.Tensor, input_beta: torch.Tensor) -> torch.Tensor:
        h = _ext.scan_forward(input_alpha, input_beta)
        ctx.save_for_backward(input_alpha, h)
        return h

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        input_alpha, h = ctx.saved_tensors
        alpha_grad, beta_grad = _ext.scan_backward(input_alpha, h, grad_output)
        return alpha_grad, beta_grad


# The C++ dispatch (csrc/fss_torch_binding.cpp) takes the common call - contiguous GPU tensors of
# the right type, outside autocast - from here to the launch and records a C++ autograd node; it
# answers None for anything else, which then goes through the Functions above, as do all errors.
_UNRESOLVED = object()
_fast: Any = _UNRESOLVED
_fast_gated: Any = _UNRESOLVED
_fast_state: Any = _UNRESOLVED
_fast_cm: Any = _UNRESOLVED


def _fast_scan(alpha: torch.Tensor, beta: torch.Tensor, code: int) -> Optional[torch.Tensor]:
    global _fast
    if _fast is _UNRESOLVED:
        binding = _ext.fast_dispatch()
        _fast = binding.scan if binding is not None else None
    if _fast is None or not isinstance(alpha, torch.Tensor) or not isinstance(beta, torch.Tensor):
        return None
    return _fast(alpha, beta, code)


def scan(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """h[:,0] = beta[:,0]; h[:,t] = alpha[:,t]*h[:,t-1] + beta[:,t]  (bf16, fp32 carry)."""
    h = _fast_scan(alpha, beta, 0)
    return h if h is not None else SequentialScan.apply(alpha, beta)


def scan_single(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """The same recurrence on fp32 tensors."""
    h = _fast_scan(alpha, beta, 1)
    return h if h is not None else SequentialScanSingle.apply(alpha, beta)


class SequentialScanFp16(Function):
    """The recurrence on IEEE half tensors (not in the reference, whose half type is bf16)."""

    @staticmethod
    def forward(ctx: Any, input_alpha: torch.Tensor, input_beta: torch.Tensor) -> torch.Tensor:
        out = _ext.scan_forward_fp16(input_alpha, input_beta)
        ctx.save_for_backward(input_alpha, out)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        input_alpha, out = ctx.saved_tensors
        grad_alpha, grad_beta = _ext.scan_backward_fp16(input_alpha, out, grad_output)
        return grad_alpha, grad_beta


def scan_fp16(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """The same recurrence on fp16 tensors."""
    h = _fast_scan(alpha, beta, 2)
    return h if h is not None else SequentialScanFp16.apply(alpha, beta)


class SequentialScanState(Function):
    """The scan with a state entering and leaving the sequence: ``(h, h_last) = f(alpha, beta, h_before)``.
    Not in the reference.  bf16 or fp32 tensors; the states are fp32 ``(bs, d_model)``.  Differentiable
    in all three inputs, through both outputs."""

    @staticmethod
    def forward(ctx: Any, alpha: torch.Tensor, beta: torch.Tensor, h_before: Optional[torch.Tensor]):
        h, h_last = _ext.scan_forward_state(alpha, beta, h_before)
        ctx.has_state = h_before is not None
        if ctx.has_state:
            ctx.save_for_backward(alpha, h, h_before)
        else:
            ctx.save_for_backward(alpha, h)
        return h, h_last

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_h: torch.Tensor, grad_h_last: torch.Tensor):
        if ctx.has_state:
            alpha, h, h_before = ctx.saved_tensors
        else:
            (alpha, h), h_before = ctx.saved_tensors, None
        grad_alpha, grad_beta, grad_h_before = _ext.scan_backward_state(alpha, h, grad_h, h_before, grad_h_last)
        return grad_alpha, grad_beta, grad_h_before


def scan_with_state(
    alpha: torch.Tensor, beta: torch.Tensor, h_before: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``h[t] = alpha[t]*h[t-1] + beta[t]`` from ``h[-1] = h_before`` (zeros when None; when given,
    ``alpha[:, 0]`` multiplies it).  Returns ``(h, h_last)`` with ``h_last`` the fp32 state after the
    last step, to be passed as ``h_before`` of the next segment."""
    global _fast_state
    if _fast_state is _UNRESOLVED:
        binding = _ext.fast_dispatch()
        _fast_state = binding.scan_state if binding is not None else None
    # (without gradients - the step of a decode loop - the C++ dispatch takes the common call)
    if (_fast_state is not None and isinstance(alpha, torch.Tensor) and isinstance(beta, torch.Tensor)
            and (h_before is None or isinstance(h_before, torch.Tensor))):
        pair = _fast_state(alpha, beta, h_before)
        if pair is not None:
            return pair
    return SequentialScanState.apply(alpha, beta, h_before)


class SequentialScanGated(Function):
    """``h = scan(sigmoid(gate), x * sqrt(1 - sigmoid(gate)**2))`` with the gating computed inside the
    scan kernels, forward and backward.  Not in the reference.  bf16 or fp32 tensors."""

    @staticmethod
    def forward(ctx: Any, gate: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
        h = _ext.gated_scan_forward(gate, x)
        ctx.save_for_backward(gate, x, h)
        return h

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        gate, x, h = ctx.saved_tensors
        grad_gate, grad_x = _ext.gated_scan_backward(gate, x, h, grad_output)
        return grad_gate, grad_x


def scan_gated(gate: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """The Hawk / RG-LRU style gated recurrence from its pre-activations:
    ``a = sigmoid(gate)``, ``h[t] = a[t]*h[t-1] + sqrt(1 - a[t]**2) * x[t]``."""
    global _fast_gated
    if _fast_gated is _UNRESOLVED:
        binding = _ext.fast_dispatch()
        _fast_gated = binding.scan_gated if binding is not None else None
    if _fast_gated is not None and isinstance(gate, torch.Tensor) and isinstance(x, torch.Tensor):
        h = _fast_gated(gate, x)
        if h is not None:
            return h
    return SequentialScanGated.apply(gate, x)


class SequentialScanGatedState(Function):
    """The gated scan with a state entering and leaving the sequence:
    ``(h, h_last) = f(gate, x, h_before)``.  Not in the reference.  Differentiable in all three
    inputs, through both outputs."""

    @staticmethod
    def forward(ctx: Any, gate: torch.Tensor, x: torch.Tensor, h_before: Optional[torch.Tensor]):
        h, h_last = _ext.gated_scan_forward_state(gate, x, h_before)
        ctx.has_state = h_before is not None
        if ctx.has_state:
            ctx.save_for_backward(gate, x, h, h_before)
        else:
            ctx.save_for_backward(gate, x, h)
        return h, h_last

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_h: torch.Tensor, grad_h_last: torch.Tensor):
        if ctx.has_state:
            gate, x, h, h_before = ctx.saved_tensors
        else:
            (gate, x, h), h_before = ctx.saved_tensors, None
        grad_gate, grad_x, grad_h_before = _ext.gated_scan_backward_state(gate, x, h, grad_h, h_before, grad_h_last)
        return grad_gate, grad_x, grad_h_before


def scan_gated_with_state(
    gate: torch.Tensor, x: torch.Tensor, h_before: Optional[torch.Tensor] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """:func:`scan_gated` from ``h[-1] = h_before`` (fp32 ``(bs, d_model)``, zeros when None).  Returns
    ``(h, h_last)`` with ``h_last`` the fp32 state after the last step, to be passed as ``h_before`` of
    the next segment (chunked prefill, decoding, a sequence sharded over devices)."""
    return SequentialScanGatedState.apply(gate, x, h_before)


class SequentialScanChannelMajor(Function):
    """The scan on ``(bs, d_model, seq)`` tensors (time contiguous), bf16, fp16 or fp32.  Not in the
    reference, whose kernels take ``(bs, seq, d_model)`` only."""

    @staticmethod
    def forward(ctx: Any, alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
        h = _ext.scan_forward_cm(alpha, beta)
        ctx.save_for_backward(alpha, h)
        return h

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        alpha, h = ctx.saved_tensors
        grad_alpha, grad_beta = _ext.scan_backward_cm(alpha, h, grad_output)
        return grad_alpha, grad_beta


def scan_cm(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """``h[..., t] = alpha[..., t]*h[..., t-1] + beta[..., t]`` for ``(bs, d_model, seq)`` tensors."""
    global _fast_cm
    if _fast_cm is _UNRESOLVED:
        binding = _ext.fast_dispatch()
        _fast_cm = binding.scan_cm if binding is not None else None
    if _fast_cm is not None and isinstance(alpha, torch.Tensor) and isinstance(beta, torch.Tensor):
        h = _fast_cm(alpha, beta)
        if h is not None:
            return h
    return SequentialScanChannelMajor.apply(alpha, beta)
