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
    """True when ``OFFLOAD_ADAM_REQUIRE_COPY_ENGINES`` asks for an error instead of a
    warning whenever the copy-engine library cannot take effect."""
    return os.environ.get("OFFLOAD_ADAM_REQUIRE_COPY_ENGINES", "").strip().lower() in (
        "1", "on", "true", "yes")


LATE_HINT = (
    "offload_adam_amd was imported after the GPU runtime had started, so HSA_TOOLS_LIB and "
    "GPU_MAX_HW_QUEUES come too late for this process: host<->device copies keep the SDMA "
    "engine the HIP runtime picks and the streaming step runs half duplex.  Import "
    "offload_adam_amd before the first CUDA call, start the script with "
    "`python -m offload_adam_amd.launch script.py ...`, or export the variables first "
    "(`python -m offload_adam_amd.launch --print-env`)."
)


def prepare():
    """Idempotent; returns ``{"copy_engines": ..., "hw_queues": ...}``.  With
    ``OFFLOAD_ADAM_REQUIRE_COPY_ENGINES=1`` an import that comes too late raises."""
    global _prepared
    if _prepared is not None:
        return _prepared
    result = {"copy_engines": _copy_engines.install()}
    if result["copy_engines"] == "late" and required():
        raise RuntimeError("OFFLOAD_ADAM_REQUIRE_COPY_ENGINES is set: " + LATE_HINT)
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
