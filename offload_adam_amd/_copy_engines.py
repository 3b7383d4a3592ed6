"""Registration of liboffload_adam_copy_engines.so with the ROCr runtime.

The library (csrc/hsa_tool/copy_engine_pin.cpp) gives host->device and
device->host copies one fixed SDMA engine each.  The runtime loads tools
libraries named in ``HSA_TOOLS_LIB`` while it initialises, which happens at the
first HIP call of the process (for torch: the first CUDA call, not
``import torch``).  :func:`install` therefore runs when the package is imported
and only edits the environment; nothing is loaded here.

``OFFLOAD_ADAM_COPY_ENGINES=off`` keeps the environment untouched.
"""

import ctypes
import os
import sys
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "liboffload_adam_copy_engines.so"

_install_result = None


def _gpu_runtime_started():
    torch = sys.modules.get("torch")
    try:
        return bool(torch is not None and torch.cuda.is_initialized())
    except Exception:
        return False


def install():
    """Put the tools library on ``HSA_TOOLS_LIB``.  Returns one of
    ``"installed"``, ``"off"`` (disabled by the environment), ``"missing"``
    (library not built), ``"unusable_path"`` (the install path contains
    whitespace, which ``HSA_TOOLS_LIB`` cannot express) or ``"late"`` (the GPU
    runtime is already up)."""
    global _install_result
    if _install_result in ("installed", "off"):
        return _install_result
    if os.environ.get("OFFLOAD_ADAM_COPY_ENGINES", "").strip().lower() in ("off", "0", "none"):
        _install_result = "off"
    elif not LIB_PATH.exists():
        _install_result = "missing"
    elif any(ch.isspace() for ch in str(LIB_PATH)):
        # HSA_TOOLS_LIB is a whitespace-separated list: such a path cannot be named in it
        _install_result = "unusable_path"
    elif str(LIB_PATH) in os.environ.get("HSA_TOOLS_LIB", "").split():
        _install_result = "installed"
    elif _gpu_runtime_started():
        _install_result = "late"
    else:
        current = os.environ.get("HSA_TOOLS_LIB", "").strip()
        os.environ["HSA_TOOLS_LIB"] = (str(LIB_PATH) + " " + current).strip()
        _install_result = "installed"
    return _install_result


_handle = None


def _lib():
    global _handle
    if _handle is None and LIB_PATH.exists():
        lib = ctypes.CDLL(str(LIB_PATH))  # same handle the runtime holds, if it loaded it
        lib.oa_copy_engines_register_range.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        lib.oa_copy_engines_register_range.restype = ctypes.c_int
        lib.oa_copy_engines_unregister_range.argtypes = [ctypes.c_void_p]
        lib.oa_copy_engines_unregister_range.restype = ctypes.c_int
        _handle = lib
    return _handle


def register_range(ptr, nbytes):
    """Tell the tools library that ``[ptr, ptr + nbytes)`` is an optimizer buffer:
    from the first registration on, only copies to or from registered ranges are
    put on the fixed engines.  No-op when the library is not built."""
    lib = _lib()
    if lib is not None:
        lib.oa_copy_engines_register_range(ctypes.c_void_p(ptr), ctypes.c_size_t(nbytes))


def unregister_range(ptr):
    lib = _lib()
    if lib is not None:
        lib.oa_copy_engines_unregister_range(ctypes.c_void_p(ptr))


def tools_loaded():
    """True when the ROCr runtime has loaded the tools library (its OnLoad ran)."""
    if not LIB_PATH.exists():
        return False
    lib = _lib()
    lib.oa_copy_engines_loaded.restype = ctypes.c_int
    lib.oa_copy_engines_active.restype = ctypes.c_int
    return bool(lib.oa_copy_engines_loaded()) and bool(lib.oa_copy_engines_active())


def direct_status():
    """State of the kernel library's own fixed-engine copies (``oa_h2d_async`` /
    ``oa_d2h_async``) on the current GPU: ``{"direct", "direct_reason",
    "direct_h2d_engine", "direct_d2h_engine", "direct_h2d_copies", "direct_d2h_copies",
    "direct_runtime_copies"}``.  Sets them up when no copy has been made yet (a GPU
    call)."""
    from . import _lib as kernels

    lib = kernels.load()
    h2d, d2h = ctypes.c_uint(0), ctypes.c_uint(0)
    a, b, c = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    code = lib.oa_link_copy_status(ctypes.byref(h2d), ctypes.byref(d2h), ctypes.byref(a),
                                   ctypes.byref(b), ctypes.byref(c))
    return {"direct": code == 0,
            "direct_reason": None if code == 0 else kernels.error_string(code),
            "direct_h2d_engine": h2d.value, "direct_d2h_engine": d2h.value,
            "direct_h2d_copies": a.value, "direct_d2h_copies": b.value,
            "direct_runtime_copies": c.value}


def status():
    """Both ways of fixing the SDMA engine per direction.  The kernel library's own
    copies: the keys of :func:`direct_status` (only once the GPU runtime is up; before
    that ``direct`` is None).  The tools library, once the GPU runtime is up:
    ``{"install", "loaded", "active", "h2d_engine", "d2h_engine", "h2d_copies",
    "d2h_copies", "rejected", "unpinned_calls", "scoped", "passed_by"}``; ``loaded`` is
    False when the runtime started before :func:`install` ran (or the library is
    missing)."""
    out = {"install": _install_result, "loaded": False, "active": False, "direct": None,
           "direct_reason": "the GPU runtime has not started"}
    if _gpu_runtime_started():
        out.update(direct_status())
    if not LIB_PATH.exists():
        return out
    lib = _lib()
    lib.oa_copy_engines_loaded.restype = ctypes.c_int
    lib.oa_copy_engines_active.restype = ctypes.c_int
    lib.oa_copy_engines_config.restype = None
    lib.oa_copy_engines_stats.restype = None
    out["loaded"] = bool(lib.oa_copy_engines_loaded())
    out["active"] = bool(lib.oa_copy_engines_active())
    h2d, d2h = ctypes.c_uint(0), ctypes.c_uint(0)
    lib.oa_copy_engines_config(ctypes.byref(h2d), ctypes.byref(d2h))
    out["h2d_engine"], out["d2h_engine"] = h2d.value, d2h.value
    a, b, c = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    lib.oa_copy_engines_stats(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    out["h2d_copies"], out["d2h_copies"], out["rejected"] = a.value, b.value, c.value
    lib.oa_copy_engines_unpinned_calls.restype = ctypes.c_ulonglong
    out["unpinned_calls"] = lib.oa_copy_engines_unpinned_calls()
    lib.oa_copy_engines_scoped.restype = ctypes.c_int
    lib.oa_copy_engines_passed_by.restype = ctypes.c_ulonglong
    out["scoped"] = bool(lib.oa_copy_engines_scoped())
    out["passed_by"] = lib.oa_copy_engines_passed_by()
    return out
