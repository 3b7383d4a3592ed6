"""offload_adam_amd: Adam with host-offloaded gradients and optimizer states,
with every kernel hand-written in HIP for AMD Instinct MI355X (gfx950).

Public surface mirrors the reference package ``offload_adam``: ``Adam`` and
``OffloadAdam`` (plus ``offload_adam_amd.kernels`` and
``offload_adam_amd.qweight``).
"""

from . import _runtime_env

# Must run before the first HIP call of the process: names the SDMA-engine tools
# library in HSA_TOOLS_LIB and reserves hardware queues for the transfer streams;
# the runtime reads both while it initialises.
_runtime_env.prepare()

from .adam import Adam  # noqa: E402
from .offload_adam import OffloadAdam  # noqa: E402

__version__ = "0.1.0"


class DistributedOffloadAdam(OffloadAdam):
    """Placeholder for the reference's ZeRO-1 optimizer.  This build targets one
    GPU: there are no collectives and no state sharding."""

    def __init__(self, *args, **kwargs):
        raise NotImplementedError(
            "DistributedOffloadAdam (ZeRO-1 over several GPUs) is not part of this "
            "single-GPU build; use OffloadAdam."
        )


__all__ = ["Adam", "OffloadAdam", "DistributedOffloadAdam"]
