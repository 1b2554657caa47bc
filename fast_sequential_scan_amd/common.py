"""Helpers with the names and meaning of the reference's ``sequential_scan/common.py``
(tolerances :6-7, error metric :10-17, input makers :20-43, the definition of the scan
:46-59), so that code and tests written against that module run against this package.
Written from the definitions, not from the reference's text.
"""
from __future__ import annotations

import math
from typing import Tuple

import torch

# digits of agreement the reference's tests ask for (relative L2 error below 10^-digits,
# give or take the rounding of the ceiling below)
SINGLE_TOL = 7.0
BFLOAT16_TOL = 2.0

__all__ = [
    "SINGLE_TOL", "BFLOAT16_TOL", "relative_error", "check_relative_error",
    "make_tensors", "make_tensors_single", "torch_ref",
]


def relative_error(x: torch.Tensor, y: torch.Tensor) -> float:
    """||x - y||_2 / ||y||_2 over all elements."""
    return float(torch.linalg.vector_norm((x - y).flatten()) / torch.linalg.vector_norm(y.flatten()))


def check_relative_error(err: float, digits: float) -> bool:
    """True when ``err`` is zero or ceil(-log10(err)) reaches ``digits``."""
    return err == 0.0 or math.ceil(-math.log10(err)) >= digits


def _pair(bs: int, sq: int, d_model: int, dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    shape = (bs, sq, d_model)
    return tuple(torch.randn(shape, device="cuda:0", dtype=dtype, requires_grad=True) for _ in range(2))


def make_tensors(bs: int, sq: int, d_model: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Two N(0,1) bf16 leaf tensors ``(bs, sq, d_model)`` on the GPU."""
    return _pair(bs, sq, d_model, torch.bfloat16)


def make_tensors_single(bs: int, sq: int, d_model: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Two N(0,1) fp32 leaf tensors ``(bs, sq, d_model)`` on the GPU."""
    return _pair(bs, sq, d_model, torch.float32)


def torch_ref(alpha: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """The scan as its definition reads: ``h[:, 0] = beta[:, 0]`` and
    ``h[:, t] = alpha[:, t] * h[:, t-1] + beta[:, t]``, in the tensors' own dtype,
    differentiable through torch's autograd."""
    steps = [beta[:, 0, :]]
    for t in range(1, alpha.shape[1]):
        steps.append(alpha[:, t, :] * steps[-1] + beta[:, t, :])
    return torch.stack(steps, dim=1)
