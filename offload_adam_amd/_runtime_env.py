"""Process environment the streaming path needs, set before the GPU runtime starts.

Two settings, both read by the ROCm runtime at its first call and never again:

* ``HSA_TOOLS_LIB`` gets the package's SDMA-engine tools library
  (:mod:`offload_adam_amd._copy_engines`).
* ``GPU_MAX_HW_QUEUES`` (HIP's default: 4) is raised to 8 unless the user has
  set it.  HIP streams share that many hardware queues; a stream created when
  all queues are taken is put on a queue another stream already uses.  The
  optimizer's host->device stream, its device->host stream and the compute
  stream must not share: the barrier packets that order one stream's copies
  would sit in the same in-order queue as the other's, and the two copy
  directions (or a copy and the backward kernels) then run strictly one after
  the other.  Measured on the 8B streaming step: 3.08 s with the two transfer
  streams on one queue, 2.12 s with a queue each.
  ``OFFLOAD_ADAM_HW_QUEUES=<n>`` picks another value, ``off`` leaves the
  variable alone.
"""

import os

from . import _copy_engines

DEFAULT_HW_QUEUES = 8

_prepared = None


def required():
    """True when ``OFFLOAD_ADAM_REQUIRE_COPY_ENGINES`` asks ``OffloadAdam`` for an error
    instead of a warning when its copies cannot be put on fixed SDMA engines."""
    return os.environ.get("OFFLOAD_ADAM_REQUIRE_COPY_ENGINES", "").strip().lower() in (
        "1", "on", "true", "yes")


def prepare():
    """Idempotent; returns ``{"copy_engines": ..., "hw_queues": ...}``."""
    global _prepared
    if _prepared is not None:
        return _prepared
    result = {"copy_engines": _copy_engines.install()}
    want = os.environ.get("OFFLOAD_ADAM_HW_QUEUES", "").strip().lower()
    if want in ("off", "0", "none"):
        result["hw_queues"] = os.environ.get("GPU_MAX_HW_QUEUES")
    elif "GPU_MAX_HW_QUEUES" in os.environ and not want:
        result["hw_queues"] = os.environ["GPU_MAX_HW_QUEUES"]  # the user's choice stands
    else:
        value = str(int(want)) if want else str(DEFAULT_HW_QUEUES)
        if _copy_engines._gpu_runtime_started():
            result["hw_queues"] = os.environ.get("GPU_MAX_HW_QUEUES")  # too late to matter
        else:
            os.environ["GPU_MAX_HW_QUEUES"] = value
            result["hw_queues"] = value
    _prepared = result
    return result
