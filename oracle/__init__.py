"""CPU oracle for the linear-recurrence scan -- TEST INFRASTRUCTURE ONLY.

Importable from ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py``; the shipped package never imports it.

Thin ``ctypes``/NumPy binding of ``oracle/scan_oracle.c`` (a restatement of
``sequential_scan/common.py:46-59`` and
``csrc/include/sequential_scan_cpu.hpp:5-115`` of the reference) and, when it
has been built, of ``oracle/_ref/libref_scan.so`` -- the reference's own C++
header compiled unchanged.

All arrays are C-contiguous ``(bs, seq, d)``.  bf16 tensors travel as
``uint16`` bit patterns.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import List, Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_scan.so")

_i64 = ctypes.c_int64
_ptr = ctypes.c_void_p


def build(with_ref: Optional[bool] = None, reference_dir: str = "/root/reference") -> None:
    """Compile the oracle; also the reference driver when the checkout exists."""
    subprocess.run(["make", "-C", _HERE, "-B", "all"], check=True, capture_output=True)
    if with_ref is None:
        with_ref = os.path.isfile(
            os.path.join(reference_dir, "csrc", "include", "sequential_scan_cpu.hpp")
        )
    if with_ref:
        subprocess.run(
            ["make", "-C", _HERE, "-B", "ref", f"REFERENCE_DIR={reference_dir}"],
            check=True,
            capture_output=True,
        )


_lib = None
_ref = None


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.isfile(_LIB_PATH):
            build(with_ref=False)
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _c(a: np.ndarray, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=dtype)
    if a.ndim != 3:
        raise ValueError(f"expected a (bs, seq, d) array, got shape {a.shape}")
    return a


def _p(a: np.ndarray) -> _ptr:
    return _ptr(a.ctypes.data)


def _dims(a: np.ndarray) -> Tuple[_i64, _i64, _i64]:
    return _i64(a.shape[0]), _i64(a.shape[1]), _i64(a.shape[2])


def _same_shape(*arrays: np.ndarray) -> None:
    s = arrays[0].shape
    for a in arrays[1:]:
        if a.shape != s:
            raise ValueError(f"shape mismatch: {s} vs {a.shape}")


# --------------------------------------------------------------- fp32 / fp64


def scan_fwd_f32(alpha, beta, fused: bool = False) -> np.ndarray:
    a, b = _c(alpha, np.float32), _c(beta, np.float32)
    _same_shape(a, b)
    h = np.empty_like(a)
    _load().oracle_scan_fwd_f32(_p(a), _p(b), _p(h), *_dims(a), ctypes.c_int(int(fused)))
    return h


def scan_bwd_f32(alpha, h, dout, fused: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    a, hh, do = _c(alpha, np.float32), _c(h, np.float32), _c(dout, np.float32)
    _same_shape(a, hh, do)
    ga, gb = np.empty_like(a), np.empty_like(a)
    _load().oracle_scan_bwd_f32(
        _p(a), _p(hh), _p(do), _p(ga), _p(gb), *_dims(a), ctypes.c_int(int(fused))
    )
    return ga, gb


def scan_fwd_f64(alpha, beta) -> np.ndarray:
    a, b = _c(alpha, np.float64), _c(beta, np.float64)
    _same_shape(a, b)
    h = np.empty_like(a)
    _load().oracle_scan_fwd_f64(_p(a), _p(b), _p(h), *_dims(a))
    return h


def scan_bwd_f64(alpha, h, dout) -> Tuple[np.ndarray, np.ndarray]:
    a, hh, do = _c(alpha, np.float64), _c(h, np.float64), _c(dout, np.float64)
    _same_shape(a, hh, do)
    ga, gb = np.empty_like(a), np.empty_like(a)
    _load().oracle_scan_bwd_f64(_p(a), _p(hh), _p(do), _p(ga), _p(gb), *_dims(a))
    return ga, gb


# ---------------------------------------------------------------------- bf16


def scan_fwd_bf16(alpha_bits, beta_bits, fused: bool = False) -> np.ndarray:
    """bf16 bits in, bf16 bits out, fp32 carry."""
    a, b = _c(alpha_bits, np.uint16), _c(beta_bits, np.uint16)
    _same_shape(a, b)
    h = np.empty_like(a)
    _load().oracle_scan_fwd_bf16(_p(a), _p(b), _p(h), *_dims(a), ctypes.c_int(int(fused)))
    return h


def scan_bwd_bf16(alpha_bits, h_bits, dout_bits, fused: bool = False):
    """bf16 bits in (h = stored forward output), bf16 bits out, fp32 carry."""
    a, hh, do = _c(alpha_bits, np.uint16), _c(h_bits, np.uint16), _c(dout_bits, np.uint16)
    _same_shape(a, hh, do)
    ga, gb = np.empty_like(a), np.empty_like(a)
    _load().oracle_scan_bwd_bf16(
        _p(a), _p(hh), _p(do), _p(ga), _p(gb), *_dims(a), ctypes.c_int(int(fused))
    )
    return ga, gb


def scan_fwd_bf16_f32out(alpha_bits, beta_bits) -> np.ndarray:
    """Grading oracle: bf16 inputs, everything after the load in fp32."""
    a, b = _c(alpha_bits, np.uint16), _c(beta_bits, np.uint16)
    _same_shape(a, b)
    h = np.empty(a.shape, dtype=np.float32)
    _load().oracle_scan_fwd_bf16_f32out(_p(a), _p(b), _p(h), *_dims(a))
    return h


def scan_bwd_bf16_f32out(alpha_bits, h_f32, dout_bits):
    a, do = _c(alpha_bits, np.uint16), _c(dout_bits, np.uint16)
    hh = _c(h_f32, np.float32)
    _same_shape(a, hh, do)
    ga = np.empty(a.shape, dtype=np.float32)
    gb = np.empty(a.shape, dtype=np.float32)
    _load().oracle_scan_bwd_bf16_f32out(_p(a), _p(hh), _p(do), _p(ga), _p(gb), *_dims(a))
    return ga, gb


def f32_to_bf16_bits(x) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    _load().oracle_f32_to_bf16(_p(x), _p(out), _i64(x.size))
    return out


def bf16_bits_to_f32(bits) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    _load().oracle_bf16_to_f32(_p(bits), _p(out), _i64(bits.size))
    return out


# ---- the HIP kernels' own composition order, restated sequentially (oracle/chained_model.c) ----


def chained_scan_fwd(alpha, beta, steps: int, waves: int, period: int, look: int, span: int) -> np.ndarray:
    """Forward scan composed exactly as the row-major HIP kernels compose it for a tiling of
    `waves` slices of `steps` timesteps per chunk and the given chain plan.  uint16 arrays are
    bf16 bit patterns (bf16 bits out), anything else is taken as float32 (float32 out)."""
    bits = np.asarray(alpha).dtype == np.uint16
    dt = np.uint16 if bits else np.float32
    a, b = _c(alpha, dt), _c(beta, dt)
    _same_shape(a, b)
    h = np.empty_like(a)
    fn = _load().chained_scan_fwd_bf16 if bits else _load().chained_scan_fwd_f32
    rc = fn(_p(a), _p(b), _p(h), *_dims(a), *(ctypes.c_int(int(v)) for v in (steps, waves, period, look, span)))
    if rc != 0:
        raise ValueError("bad chain configuration")
    return h


def chained_scan_bwd(alpha, h, dout, steps: int, waves: int, period: int, look: int, span: int):
    """(grad_alpha, grad_beta) composed as the row-major HIP backward composes them."""
    bits = np.asarray(alpha).dtype == np.uint16
    dt = np.uint16 if bits else np.float32
    a, hh, do = _c(alpha, dt), _c(h, dt), _c(dout, dt)
    _same_shape(a, hh, do)
    ga, gb = np.empty_like(a), np.empty_like(a)
    fn = _load().chained_scan_bwd_bf16 if bits else _load().chained_scan_bwd_f32
    rc = fn(_p(a), _p(hh), _p(do), _p(ga), _p(gb), *_dims(a),
            *(ctypes.c_int(int(v)) for v in (steps, waves, period, look, span)))
    if rc != 0:
        raise ValueError("bad chain configuration")
    return ga, gb


# torch <-> bit-pattern helpers (torch imported lazily: the oracle itself is NumPy)


def torch_bf16_to_bits(t) -> np.ndarray:
    import torch

    assert t.dtype == torch.bfloat16
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bits_to_torch_bf16(bits):
    import torch

    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16).copy()).view(torch.bfloat16)


# ------------------------------------------- the reference's own C++ CPU scan


def ref_available() -> bool:
    return os.path.isfile(_REF_PATH)


def _load_ref() -> ctypes.CDLL:
    global _ref
    if _ref is None:
        if not ref_available():
            raise FileNotFoundError(
                f"{_REF_PATH} is not built (make -C oracle ref needs the reference checkout)"
            )
        _ref = ctypes.CDLL(_REF_PATH)
    return _ref


def ref_shapes() -> List[Tuple[int, int, int]]:
    lib = _load_ref()
    out = []
    for i in range(lib.ref_scan_num_shapes()):
        bs, seq, d = _i64(), _i64(), _i64()
        lib.ref_scan_shape(i, ctypes.byref(bs), ctypes.byref(seq), ctypes.byref(d))
        out.append((bs.value, seq.value, d.value))
    return out


def ref_scan_fwd(alpha, beta) -> np.ndarray:
    a, b = _c(alpha, np.float32), _c(beta, np.float32)
    _same_shape(a, b)
    h = np.empty_like(a)
    rc = _load_ref().ref_scan_fwd(_p(a), _p(b), _p(h), *_dims(a))
    if rc != 0:
        raise ValueError(f"shape {a.shape} is not instantiated in oracle/ref_driver.cpp")
    return h


def ref_scan_bwd(alpha, h, dout):
    a, hh, do = _c(alpha, np.float32), _c(h, np.float32), _c(dout, np.float32)
    _same_shape(a, hh, do)
    ga, gb = np.empty_like(a), np.empty_like(a)
    rc = _load_ref().ref_scan_bwd(_p(a), _p(hh), _p(do), _p(ga), _p(gb), *_dims(a))
    if rc != 0:
        raise ValueError(f"shape {a.shape} is not instantiated in oracle/ref_driver.cpp")
    return ga, gb


# ---- gated scan (not in the reference: alpha = sigmoid(gate), beta = x*sqrt(1-alpha^2)) ----
#
# Elementwise arithmetic in float64 NumPy around the scans above.  `rounding` is where the
# storage type takes effect: "bf16" rounds alpha, beta and the outputs to bf16 (to nearest
# even), "f32" to float32.  Inputs are float32 arrays already holding storage-type values.


def _round_to(a: np.ndarray, rounding: str) -> np.ndarray:
    a32 = np.asarray(a, dtype=np.float64).astype(np.float32)
    if rounding == "f32":
        return a32
    if rounding == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(a32))
    if rounding == "f16":
        return a32.astype(np.float16).astype(np.float32)
    raise ValueError(rounding)


def _step_storage(v: np.ndarray, rounding: str, up: np.ndarray) -> np.ndarray:
    """The storage-type value next to `v` (non-negative storage-type values held in float32):
    one step up where `up`, else one step down (0 stays 0)."""
    if rounding == "bf16":
        bits = f32_to_bf16_bits(v).astype(np.int32)
        bits = np.where(up, bits + 1, np.maximum(bits - 1, 0))
        return bf16_bits_to_f32(bits.astype(np.uint16))
    if rounding == "f16":
        bits = v.astype(np.float16).view(np.uint16).astype(np.int32)
        bits = np.where(up, bits + 1, np.maximum(bits - 1, 0))
        return bits.astype(np.uint16).view(np.float16).astype(np.float32)
    raise ValueError(rounding)


def gate_alpha_variants(gate, rounding: str, fp32_ulps: float = 8.0):
    """(alpha, alpha_other, ambiguous): alpha = sigmoid(gate) rounded to the storage type to
    nearest; `ambiguous` marks the elements whose exact sigmoid lies within `fp32_ulps` fp32
    units in the last place of the midpoint between two storage values, i.e. where an fp32
    evaluation with a few ulps of error (a hardware exp2 and reciprocal) may legitimately round
    to the other neighbour; `alpha_other` holds that neighbour there and alpha elsewhere.
    fp32 storage has no such elements (its tests allow no deviation beyond their tolerance)."""
    g64 = np.asarray(gate, dtype=np.float64)
    exact = 1.0 / (1.0 + np.exp(-g64))
    alpha = _round_to(exact, rounding)
    if rounding == "f32":
        return alpha, alpha, np.zeros(alpha.shape, dtype=bool)
    up = exact > alpha.astype(np.float64)  # the exact value lies above the rounded one: the other neighbour is above
    other = _step_storage(alpha, rounding, up)
    mid = 0.5 * (alpha.astype(np.float64) + other.astype(np.float64))
    eps = fp32_ulps * 2.0 ** -24 * np.maximum(exact, 2.0 ** -126)
    ambiguous = np.abs(exact - mid) <= eps
    return alpha, np.where(ambiguous, other, alpha).astype(np.float32), ambiguous


def gate_transform(gate, x, rounding: str, other_rounding: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    """(alpha, beta) as float32 arrays of storage-type values.  `other_rounding`: alpha takes
    the other neighbour wherever its rounding is ambiguous (see gate_alpha_variants)."""
    alpha, alpha_other, _ = gate_alpha_variants(gate, rounding)
    if other_rounding:
        alpha = alpha_other
    a64 = alpha.astype(np.float64)
    beta = _round_to(np.asarray(x, dtype=np.float64) * np.sqrt(np.maximum(1.0 - a64 * a64, 0.0)), rounding)
    return alpha, beta


def gated_scan_fwd(gate, x, rounding: str, other_rounding: bool = False) -> np.ndarray:
    """Un-rounded fp32 h of the scan over the rounded alpha and beta."""
    alpha, beta = gate_transform(gate, x, rounding, other_rounding)
    return scan_fwd_f32(alpha, beta)


def gated_scan_bwd(gate, x, h, dout, rounding: str, other_rounding: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    """(grad_gate, grad_x) in float32, un-rounded: the plain backward, then the chain rule
    through beta = x*s, s = sqrt(1-alpha^2), alpha = sigmoid(gate).  Where alpha is exactly 1
    the x term of grad_gate is dropped."""
    alpha, _ = gate_transform(gate, x, rounding, other_rounding)
    grad_alpha, grad_beta = scan_bwd_f32(alpha, np.asarray(h, dtype=np.float32), np.asarray(dout, dtype=np.float32))
    a = alpha.astype(np.float64)
    om = np.maximum(1.0 - a * a, 0.0)
    s = np.sqrt(om)
    with np.errstate(divide="ignore", invalid="ignore"):
        a_over_s = np.where(om > 0.0, a / s, 0.0)
    gb = grad_beta.astype(np.float64)
    grad_x = gb * s
    grad_gate = (grad_alpha.astype(np.float64) - gb * np.asarray(x, dtype=np.float64) * a_over_s) * a * (1.0 - a)
    return grad_gate.astype(np.float32), grad_x.astype(np.float32)


def within_rounding_envelope(got, want, want_other, rtol: float, atol: float) -> np.ndarray:
    """Elementwise: `got` lies within rtol/atol of the interval spanned by the two oracle
    evaluations (alpha rounded to nearest / to the other neighbour where that is ambiguous).
    Where no ambiguous element influences a result the two agree and this is the plain
    tolerance check."""
    got = np.asarray(got, dtype=np.float64)
    lo = np.minimum(want, want_other).astype(np.float64)
    hi = np.maximum(want, want_other).astype(np.float64)
    tol = atol + rtol * np.maximum(np.abs(lo), np.abs(hi))
    return (got >= lo - tol) & (got <= hi + tol)
