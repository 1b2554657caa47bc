"""Loads ``_lib/fss_torch_binding.so`` (csrc/fss_torch_binding.cpp): the C++ dispatch of the plain, the gated and the channel-major scan.

The module is an accelerator of host-side dispatch only: what it launches are the kernels of
``libfss_scan.so`` through the same C ABI the ctypes wrappers use, and whatever it does not cover
goes through those wrappers.  ``FSS_TORCH_BINDING=0`` keeps every call on the Python wrappers; so
does a module that is missing or does not load (built against another torch, no host compiler at
build time), after one warning.  ``FSS_TORCH_BINDING=1`` makes that an error instead.
"""
from __future__ import annotations

import ctypes
import importlib.machinery
import importlib.util
import os
import threading
import warnings
from typing import Any, Callable, Optional

from . import _native

NAME = "fss_torch_binding"
PATH = os.path.join(_native.PKG_DIR, "_lib", NAME + ".so")

_lock = threading.Lock()
_module: Any = None
_tried = False


class TorchBindingMissing(RuntimeError):
    pass


def _address(function: Any) -> int:
    return ctypes.cast(function, ctypes.c_void_p).value


def load(slow_backward: Callable[..., Any]) -> Optional[Any]:
    """The initialised module, or None when it is switched off or cannot be loaded (the calls then
    go through the Python wrappers over the same C ABI; one warning says so).  With
    ``FSS_TORCH_BINDING=1`` a module that cannot be loaded is an error."""
    global _module, _tried
    if _tried:
        return _module
    with _lock:
        if _tried:
            return _module
        setting = os.environ.get("FSS_TORCH_BINDING", "")
        if setting == "0":
            _tried = True
            return None
        lib = _native.lib()  # raises if the HIP library is missing: that one has no stand-in
        try:
            if not os.path.exists(PATH):
                raise TorchBindingMissing(
                    f"{PATH} not found: build it with `python -m fast_sequential_scan_amd.build`")
            import torch  # noqa: F401  (the module links against torch's libraries)

            loader = importlib.machinery.ExtensionFileLoader(NAME, PATH)
            spec = importlib.util.spec_from_loader(NAME, loader)
            module = importlib.util.module_from_spec(spec)
            loader.exec_module(module)
        except (TorchBindingMissing, ImportError, OSError) as exc:
            if setting == "1":
                raise
            warnings.warn(
                f"fast_sequential_scan_amd: the C++ dispatch is not available ({exc}); calls go through the "
                "Python wrappers over the same HIP library (slower on the host, same kernels)",
                RuntimeWarning, stacklevel=2)
            _tried = True
            return None
        module.init(
            _address(lib.fss_scan_fwd_ex), _address(lib.fss_scan_bwd_ex), _address(lib.fss_gated_scan_fwd),
            _address(lib.fss_gated_scan_bwd), _address(lib.fss_scan_fwd_state), _address(lib.fss_scan_fwd_cm),
            _address(lib.fss_scan_bwd_cm), _address(lib.fss_workspace_bytes), _address(lib.fss_cm_workspace_bytes),
            _address(lib.fss_strerror), slow_backward,
        )
        _module = module
        _tried = True
    return _module


def loaded() -> Optional[Any]:
    """The module if `load` has initialised it."""
    return _module
