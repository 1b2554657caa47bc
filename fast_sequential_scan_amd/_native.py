"""ctypes binding of the C ABI declared in include/fss_scan.h.

The shared library is the only implementation: when it cannot be loaded every
entry point of the package raises, there is no fallback path.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional, Tuple

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# FSS_SCAN_LIBRARY points at an alternative build of the same library (tuning experiments)
LIB_PATH = os.environ.get("FSS_SCAN_LIBRARY") or os.path.join(PKG_DIR, "_lib", "libfss_scan.so")

FSS_BF16, FSS_F32, FSS_F16 = 0, 1, 2
FSS_FWD, FSS_BWD, FSS_GATED_FWD, FSS_GATED_BWD = 0, 1, 2, 3
FSS_OK = 0
FSS_CACHE_AUTO, FSS_CACHE_STREAMING = 0, 1
FSS_ERR_CHAIN_TIMEOUT = 7
FSS_ERR_TOO_LARGE = 9
FSS_ABI_VERSION = 3
FSS_NOALLOC_SCRATCH_BYTES = 16 << 20

EXPORTED_SYMBOLS = (
    "fss_abi_version",
    "fss_strerror",
    "fss_last_hip_error",
    "fss_workspace_bytes",
    "fss_workspace_bytes_max",
    "fss_workspace_init",
    "fss_workspace_status",
    "fss_workspace_attach_flag",
    "fss_debug_set_spin_limit",
    "fss_debug_tile_groups",
    "fss_debug_noalloc_reinit_after",
    "fss_debug_chain_plan",
    "fss_debug_chain_anchor",
    "fss_scan_fwd_noalloc",
    "fss_choose_config",
    "fss_scan_fwd_bf16",
    "fss_scan_bwd_bf16",
    "fss_scan_fwd_f32",
    "fss_scan_bwd_f32",
    "fss_scan_fwd_ex",
    "fss_scan_bwd_ex",
    "fss_scan_fwd_state",
    "fss_scan_bwd_state",
    "fss_gated_scan_fwd",
    "fss_gated_scan_bwd",
    "fss_set_cache_policy",
    "fss_gated_scan_fwd_state",
    "fss_gated_scan_bwd_state",
    "fss_cm_workspace_bytes",
    "fss_scan_fwd_cm",
    "fss_scan_bwd_cm",
    "fss_copy_bytes",
    "fss_stream_mix",
)


class FssConfig(ctypes.Structure):
    _fields_ = [
        ("vec", ctypes.c_int32),
        ("steps", ctypes.c_int32),
        ("waves", ctypes.c_int32),
        ("max_groups", ctypes.c_int32),
        ("cols", ctypes.c_int32),
    ]


class NativeLibraryMissing(RuntimeError):
    pass


class FssError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"fss_scan status {status}: {message}")
        self.status = status


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None

_vp, _i64, _sz, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_size_t, ctypes.c_int
_cfgp = ctypes.POINTER(FssConfig)


def _declare(lib: ctypes.CDLL) -> None:
    lib.fss_abi_version.restype = _int
    lib.fss_abi_version.argtypes = []
    lib.fss_strerror.restype = ctypes.c_char_p
    lib.fss_strerror.argtypes = [_int]
    lib.fss_last_hip_error.restype = _int
    lib.fss_last_hip_error.argtypes = []
    lib.fss_workspace_bytes.restype = _sz
    lib.fss_workspace_bytes.argtypes = [_i64, _i64, _i64, _int, _int, _cfgp]
    lib.fss_workspace_bytes_max.restype = _sz
    lib.fss_workspace_bytes_max.argtypes = [_i64, _i64, _i64]
    lib.fss_workspace_init.restype = _int
    lib.fss_workspace_init.argtypes = [_vp, _sz, _vp]
    lib.fss_workspace_status.restype = _int
    lib.fss_workspace_status.argtypes = [_vp, _vp]
    lib.fss_workspace_attach_flag.restype = _int
    lib.fss_workspace_attach_flag.argtypes = [_vp, _vp, _vp]
    lib.fss_debug_set_spin_limit.restype = ctypes.c_uint32
    lib.fss_debug_set_spin_limit.argtypes = [ctypes.c_uint32]
    lib.fss_debug_tile_groups.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_int32)]
    lib.fss_debug_noalloc_reinit_after.restype = ctypes.c_uint64
    lib.fss_debug_noalloc_reinit_after.argtypes = [ctypes.c_uint64]
    lib.fss_debug_chain_plan.restype = _int
    lib.fss_debug_chain_plan.argtypes = [_i64, _i64, _i64, _int, _int, _sz, _cfgp, ctypes.POINTER(ctypes.c_int32)]
    lib.fss_debug_chain_anchor.restype = ctypes.c_int32
    lib.fss_debug_chain_anchor.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32]
    lib.fss_scan_fwd_noalloc.restype = _int
    lib.fss_scan_fwd_noalloc.argtypes = [_int, _vp, _vp, _vp, _i64, _i64, _i64, _vp]
    lib.fss_choose_config.restype = _int
    lib.fss_choose_config.argtypes = [_i64, _i64, _i64, _int, _int, _sz, _cfgp]
    fwd = [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp]
    bwd = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp]
    for name in ("fss_scan_fwd_bf16", "fss_scan_fwd_f32"):
        getattr(lib, name).restype = _int
        getattr(lib, name).argtypes = fwd
    for name in ("fss_scan_bwd_bf16", "fss_scan_bwd_f32"):
        getattr(lib, name).restype = _int
        getattr(lib, name).argtypes = bwd
    lib.fss_scan_fwd_ex.restype = _int
    lib.fss_scan_fwd_ex.argtypes = [_int] + fwd + [_cfgp]
    lib.fss_scan_bwd_ex.restype = _int
    lib.fss_scan_bwd_ex.argtypes = [_int] + bwd + [_cfgp]
    lib.fss_scan_fwd_state.restype = _int
    lib.fss_scan_fwd_state.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_scan_bwd_state.restype = _int
    lib.fss_scan_bwd_state.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_copy_bytes.restype = _int
    lib.fss_gated_scan_fwd.restype = _int
    lib.fss_gated_scan_fwd.argtypes = [_int, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_set_cache_policy.restype = _int
    lib.fss_set_cache_policy.argtypes = [_int]
    lib.fss_gated_scan_fwd_state.restype = _int
    lib.fss_gated_scan_fwd_state.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_gated_scan_bwd_state.restype = _int
    lib.fss_gated_scan_bwd_state.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_gated_scan_bwd.restype = _int
    lib.fss_gated_scan_bwd.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_cm_workspace_bytes.restype = _sz
    lib.fss_cm_workspace_bytes.argtypes = [_i64, _i64, _i64, _int, _int, _cfgp]
    lib.fss_scan_fwd_cm.restype = _int
    lib.fss_scan_fwd_cm.argtypes = [_int, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_scan_bwd_cm.restype = _int
    lib.fss_scan_bwd_cm.argtypes = [_int, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _sz, _vp, _cfgp]
    lib.fss_copy_bytes.argtypes = [_vp, _vp, _sz, _vp]
    lib.fss_stream_mix.restype = _int
    lib.fss_stream_mix.argtypes = [ctypes.POINTER(_vp), _int, ctypes.POINTER(_vp), _int, _sz, _int, ctypes.POINTER(_int), _vp]


def lib() -> ctypes.CDLL:
    """The loaded library; raises NativeLibraryMissing when it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.isfile(LIB_PATH):
                    raise NativeLibraryMissing(
                        f"{LIB_PATH} not found: build it with `python -m fast_sequential_scan_amd.build` "
                        "(there is no non-HIP fallback)"
                    )
                loaded = ctypes.CDLL(LIB_PATH)
                _declare(loaded)
                _lib = loaded
    return _lib


def strerror(status: int) -> str:
    return lib().fss_strerror(status).decode()


def check(status: int) -> None:
    if status != FSS_OK:
        msg = strerror(status)
        hip = lib().fss_last_hip_error()
        if hip:
            msg += f" (hipError_t {hip})"
        raise FssError(status, msg)


def stream_mix(reads, writes, nbytes: int, nontemporal_writes: bool, stream_handle: int, sink: int = 0,
               shape: Optional[Tuple[int, int, int, int]] = None) -> None:
    """fss_stream_mix over lists of device addresses; `sink`: 16 writable bytes for a read-only run;
    `shape`: (workgroups, threads, vectors per lane and iteration, non-temporal loads) or None."""
    rd = (_vp * len(reads))(*reads)
    wr_list = list(writes) if writes else [sink]
    wr = (_vp * len(wr_list))(*wr_list)
    sh = (_int * 4)(*shape) if shape is not None else None
    check(lib().fss_stream_mix(rd, len(reads), wr, len(writes), nbytes, int(nontemporal_writes), sh, stream_handle))


def make_config(cfg: Optional[Tuple[int, int, int]]):
    """(vec, steps, waves[, max_groups[, cols]]) -> pointer for the *_ex entry points; None -> NULL."""
    if cfg is None:
        return None
    vec, steps, waves = cfg[:3]
    max_groups = cfg[3] if len(cfg) > 3 else 0
    cols = cfg[4] if len(cfg) > 4 else 0
    return ctypes.byref(FssConfig(int(vec), int(steps), int(waves), int(max_groups), int(cols)))
