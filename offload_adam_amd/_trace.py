"""Optional roctx ranges around the optimizer's per-parameter work, so that a
``rocprofv3 --marker-trace`` timeline shows which kernels and copies belong to
which parameter.  Off unless ``OFFLOAD_ADAM_ROCTX=1``; when off, ``range`` costs
one attribute test.
"""

import contextlib
import ctypes
import os

_lib = None
ENABLED = os.environ.get("OFFLOAD_ADAM_ROCTX", "") == "1"

if ENABLED:
    for _name in ("librocprofiler-sdk-roctx.so", "libroctx64.so"):
        try:
            _lib = ctypes.CDLL(_name)
            _lib.roctxRangePushA.argtypes = [ctypes.c_char_p]
            _lib.roctxRangePushA.restype = ctypes.c_int
            _lib.roctxRangePop.restype = ctypes.c_int
            break
        except (OSError, AttributeError):
            _lib = None
    ENABLED = _lib is not None


@contextlib.contextmanager
def _live_range(label):
    _lib.roctxRangePushA(label.encode())
    try:
        yield
    finally:
        _lib.roctxRangePop()


_NULL = contextlib.nullcontext()


def range(label):  # noqa: A001 - mirrors roctx's own name
    """Context manager: a roctx range called ``label`` (a no-op when disabled)."""
    return _live_range(label) if ENABLED else _NULL
