"""The reference's PyTorch sequential loop, restated for CPU tensors -- TEST/BASELINE
INFRASTRUCTURE ONLY (same rule as the rest of oracle/: never imported by the
shipped package).

Forward follows sequential_scan/common.py:46-59 (``h = h*alpha[:,t] + beta[:,t]``
over ``t``, one elementwise multiply and one add on a (bs, d) slice per step).
The reference obtains gradients by autograd through that loop
(sequential_scan/test_scan_cuda.py:104-113); at sequence lengths of tens of
thousands that graph is impractical, so the backward here is the explicit
reverse loop of csrc/include/sequential_scan_cpu.hpp:36-115.

Inputs of any floating dtype are upcast to fp32 first: this is the
"fp32-accumulated sequential scan" the device kernels are graded against, and
the CPU baseline timed next to them.  Pinned against oracle/scan_oracle.c in
tests/test_oracle.py.
"""
from __future__ import annotations

from typing import Tuple

import torch


def torch_loop_fwd(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    alpha, beta = alpha.float(), beta.float()
    out = torch.empty_like(alpha)
    h = beta[:, 0, :]
    out[:, 0, :] = h
    for t in range(1, alpha.shape[1]):
        h = h * alpha[:, t, :] + beta[:, t, :]
        out[:, t, :] = h
    return out


def torch_loop_bwd(alpha: torch.Tensor, h: torch.Tensor, dout: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    alpha, h, dout = alpha.float(), h.float(), dout.float()
    seq = alpha.shape[1]
    galpha = torch.empty_like(alpha)
    gbeta = torch.empty_like(alpha)
    g = dout[:, seq - 1, :]
    for t in range(seq - 1, -1, -1):
        if t != seq - 1:
            g = g * alpha[:, t + 1, :] + dout[:, t, :]
        gbeta[:, t, :] = g
        if t >= 1:
            galpha[:, t, :] = g * h[:, t - 1, :]
        else:
            galpha[:, t, :] = 0.0
    return galpha, gbeta


# ---- gated scan (not in the reference): the gating as torch elementwise ops, then the loops above ----


def torch_gated_fwd(gate: torch.Tensor, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(alpha, h): alpha and beta are rounded to the inputs' dtype, as tensors in memory would be."""
    dtype = gate.dtype
    alpha = torch.sigmoid(gate.float()).to(dtype)
    a = alpha.double()
    beta = (x.double() * torch.sqrt(1.0 - a * a)).float().to(dtype)
    return alpha, torch_loop_fwd(alpha, beta)


def torch_gated_bwd(
    alpha: torch.Tensor, x: torch.Tensor, h: torch.Tensor, dout: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(grad_gate, grad_x) from the rounded alpha of torch_gated_fwd."""
    galpha, gbeta = torch_loop_bwd(alpha, h, dout)
    a = alpha.double()
    om = 1.0 - a * a
    s = torch.sqrt(om)
    a_over_s = torch.where(om > 0, a / s, torch.zeros_like(a))
    grad_x = gbeta.double() * s
    grad_gate = (galpha.double() - gbeta.double() * x.double() * a_over_s) * a * (1.0 - a)
    return grad_gate.float(), grad_x.float()
