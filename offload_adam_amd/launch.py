"""Start a training script with the streaming path's process environment in place.

    python -m offload_adam_amd.launch train.py [script arguments ...]
    python -m offload_adam_amd.launch -m package.module [arguments ...]
    eval "$(python -m offload_adam_amd.launch --print-env)"   # for a shell, a profiler, a job file

``OffloadAdam``'s host link runs at full duplex only when two settings are in the
environment before the process makes its first GPU call: ``HSA_TOOLS_LIB`` naming
the package's copy-engine library and ``GPU_MAX_HW_QUEUES`` (see
``offload_adam_amd._runtime_env``).  ``import offload_adam_amd`` puts them there,
but a script that touches the GPU first - ``model.cuda()`` above the optimizer's
import - is too late and only gets a warning.  Started through this module the
script may import and initialise things in any order: the package is imported,
and the environment edited, before the first line of the script runs, in the same
process (nothing is re-executed).

``--print-env`` writes the two ``export`` lines instead, for runs whose GPU
runtime starts before Python does (under ``rocprofv3`` the profiler's preloaded
library initialises it): ``eval`` them in the shell that starts the profiler.

``OFFLOAD_ADAM_REQUIRE_COPY_ENGINES=1`` turns the late-import warning into an
error, for jobs that would rather stop than run with a half-duplex link.
"""

import os
import runpy
import sys

from . import _copy_engines, _runtime_env


def environment():
    """The variables a fresh process needs, as ``{name: value}``."""
    env = {}
    if _copy_engines.LIB_PATH.exists():
        current = [t for t in os.environ.get("HSA_TOOLS_LIB", "").split()
                   if t != str(_copy_engines.LIB_PATH)]
        env["HSA_TOOLS_LIB"] = " ".join([str(_copy_engines.LIB_PATH)] + current)
    env["GPU_MAX_HW_QUEUES"] = os.environ.get("GPU_MAX_HW_QUEUES") or str(
        _runtime_env.DEFAULT_HW_QUEUES)
    return env


def main(argv=None):
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0 if argv else 2
    if argv[0] == "--print-env":
        for name, value in environment().items():
            print(f"export {name}='{value}'")
        return 0
    state = _runtime_env.prepare()  # ran when the package was imported; idempotent
    if state["copy_engines"] not in ("installed", "off"):
        print(f"offload_adam_amd.launch: copy-engine library not in effect "
              f"({state['copy_engines']})", file=sys.stderr)
    if argv[0] == "-m":
        if len(argv) < 2:
            print("offload_adam_amd.launch: -m needs a module name", file=sys.stderr)
            return 2
        sys.argv = argv[1:]
        runpy.run_module(argv[1], run_name="__main__", alter_sys=True)
    else:
        sys.argv = argv
        sys.path.insert(0, os.path.dirname(os.path.abspath(argv[0])))
        runpy.run_path(argv[0], run_name="__main__")
    return 0


if __name__ == "__main__":
    sys.exit(main())
