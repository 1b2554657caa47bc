"""MI355X-native linear-recurrence scan  h_t = a_t * h_{t-1} + b_t.

Public names follow the reference package (sequential_scan/__init__.py:1-3):
``scan_cu`` (bf16) and ``scan_cu_single`` (fp32); ``scan_cu_fp16``, ``scan_with_state``,
``scan_gated``, ``scan_gated_with_state`` and ``scan_cm`` are additions.  ``scan_tr`` - the
reference's Triton backend - has no counterpart here and raises.
"""
from .scan_cuda import (SequentialScan, SequentialScanGated, SequentialScanGatedState, SequentialScanSingle,
                        SequentialScanState, SequentialScanChannelMajor, scan_cm, scan_gated,
                        scan_gated_with_state, scan_with_state)
from .scan_cuda import scan as scan_cu
from .sequential_scan_cuda import set_cache_policy
from .scan_cuda import scan_fp16 as scan_cu_fp16
from .scan_cuda import scan_single as scan_cu_single

__all__ = [
    "scan_cu", "scan_cu_single", "scan_cu_fp16", "scan_tr", "scan_with_state", "scan_gated", "scan_gated_with_state",
    "scan_cm", "set_cache_policy",
    "SequentialScan", "SequentialScanSingle", "SequentialScanState", "SequentialScanGated", "SequentialScanGatedState",
    "SequentialScanChannelMajor",
]


def scan_tr(*_args, **_kwargs):
    raise NotImplementedError(
        "this build has one backend, the HIP kernels behind scan_cu / scan_cu_single; "
        "there is no Triton path"
    )
