"""Exact-size pinned (page-locked) host tensors with an optional NUMA preference.

Same surface as the reference's ``pinned_alloc`` module
(src/offload_adam/pinned_alloc.py): ``zeros_pinned``, ``resolve_numa_target``,
``numa_node_free_bytes``, ``gpu_numa_node``.  The memory comes from the HIP
runtime through the library's ``oa_pinned_alloc`` (hipHostMalloc, rounded to
4 KiB pages - no power-of-two rounding as in torch's pinned allocator), bound
softly to a NUMA node with the thread memory policy, zero-filled by several
threads, and released when the last tensor that views it is collected.

``PinnedArena`` / ``alloc_pinned_states`` are this package's own: the optimizer
states of a model are carved out of a few large allocations (on 4 KiB
boundaries) instead of one runtime allocation per state.  The arenas are
obtained one after another (each zero-filled as it arrives) before any caller
data moves; when the runtime refuses one, those already held are released and
the error names what the runtime would still grant.  ``OffloadAdam`` asks
``largest_grantable_bytes`` first and keeps what does not fit in HBM.

A state carved from an arena is a view of that arena's storage: ``torch.save``
of such a tensor writes the whole arena (up to 8 GiB), and the arena's memory is
returned only when every tensor carved from it is gone.  ``detached`` gives
copies that own their storage, for saving a subset of the states.
"""

import ctypes
import os
import time
import weakref
from pathlib import Path

import torch

from . import _copy_engines, _lib

_PAGE_SIZE = 4096
_MPOL_SYSCALL_PROBED = None


def _numa_policy_available():
    """True when the kernel exposes NUMA nodes (memory policies can be applied)."""
    global _MPOL_SYSCALL_PROBED
    if _MPOL_SYSCALL_PROBED is None:
        _MPOL_SYSCALL_PROBED = Path("/sys/devices/system/node/node0").exists()
    return _MPOL_SYSCALL_PROBED


def gpu_numa_node(device=None) -> int:
    """NUMA node the given GPU hangs off, or -1 when the kernel reports none
    (typical for single-socket hosts)."""
    if device is None:
        device = torch.cuda.current_device()
    if isinstance(device, torch.device):
        device = device.index if device.index is not None else torch.cuda.current_device()
    node = ctypes.c_int(-1)
    code = _lib.load().oa_gpu_numa_node(int(device), ctypes.byref(node))
    if code != 0:
        raise RuntimeError(f"HIP runtime error {code}: {_lib.error_string(code)}")
    return node.value


def resolve_numa_target(numa_node):
    """Turn the user-facing ``numa_node`` knob into a node id or None.

    * ``"auto"`` - the current GPU's node if the kernel knows it, else None.
    * ``int``    - that node; raises when the host has no NUMA support.
    * ``None``   - no binding.
    """
    if numa_node == "auto":
        if torch.cuda.is_available() and _numa_policy_available():
            detected = gpu_numa_node()
            if detected >= 0:
                return detected
        return None
    if isinstance(numa_node, int) and not isinstance(numa_node, bool):
        if not _numa_policy_available():
            raise RuntimeError(
                "this host exposes no NUMA nodes; pass numa_node=None or 'auto'"
            )
        return numa_node
    if numa_node is None:
        return None
    raise ValueError(f"numa_node must be 'auto', an int, or None (got {numa_node!r})")


def numa_node_free_bytes(node: int):
    """``MemFree`` of a NUMA node in bytes, or None if it cannot be read."""
    try:
        text = Path(f"/sys/devices/system/node/node{node}/meminfo").read_text()
    except OSError:
        return None
    for line in text.splitlines():
        if "MemFree:" in line:
            return int(line.split()[-2]) * 1024  # "Node 1 MemFree:   64457228 kB"
    return None


def _alloc(size, numa_target):
    """Page-locked, zero-filled allocation; returns (address, cleanup)."""
    lib = _lib.load()
    out = ctypes.c_void_p()
    os_errno = ctypes.c_int(0)
    code = lib.oa_pinned_alloc(
        ctypes.c_size_t(size),
        -1 if numa_target is None else int(numa_target),
        ctypes.byref(out),
        ctypes.byref(os_errno),
    )
    if code == _lib.OA_EOS:
        err = os_errno.value
        raise OSError(err, f"set_mempolicy(node={numa_target}) failed: {os.strerror(err)}")
    if code != 0:
        raise RuntimeError(
            f"pinned allocation of {size} bytes failed with code {code}: "
            f"{_lib.error_string(code)}"
        )
    ptr = out.value
    # copies to and from this block go to the fixed SDMA engines; anybody else's do not
    _copy_engines.register_range(ptr, size)

    def cleanup():
        try:
            _copy_engines.unregister_range(ptr)
            lib.oa_pinned_free(ctypes.c_void_p(ptr))
        except Exception:
            pass

    return ptr, cleanup


def zeros_pinned(shape, dtype, numa_node="auto"):
    """Zero-initialised pinned CPU tensor of exactly ``shape`` / ``dtype``.

    ``numa_node``: ``"auto"`` (the GPU's node when known), an int node id, or
    None.  The backing pages are freed when the last reference is dropped.
    """
    if torch.cuda.is_available():
        torch.cuda.init()
    shape = torch.Size(shape)
    elem_size = torch.empty(0, dtype=dtype).element_size()
    nbytes = shape.numel() * elem_size
    size = ((nbytes + _PAGE_SIZE - 1) // _PAGE_SIZE) * _PAGE_SIZE
    if size == 0:
        size = _PAGE_SIZE

    target = resolve_numa_target(numa_node)
    ptr, cleanup = _alloc(size, target)
    try:
        buf = (ctypes.c_uint8 * size).from_address(ptr)
        flat = torch.frombuffer(buf, dtype=torch.uint8)
        weakref.finalize(flat.untyped_storage(), cleanup)
        return flat.view(dtype)[: shape.numel()].view(shape)
    except BaseException:
        cleanup()
        raise


# ------------------------------------------------------------------ arenas

ARENA_BYTES = 8 << 30  # a state larger than this gets an arena of its own


def _round_up_page(nbytes):
    return max(_PAGE_SIZE, (nbytes + _PAGE_SIZE - 1) // _PAGE_SIZE * _PAGE_SIZE)


class PinnedArena:
    """One page-locked, zero-filled allocation handed out in 4 KiB-aligned
    pieces.  The pieces are views of one storage: the memory is released when
    the arena and every tensor carved from it are gone."""

    def __init__(self, nbytes, numa_node="auto"):
        self.nbytes = _round_up_page(nbytes)
        self._flat = zeros_pinned((self.nbytes,), torch.uint8, numa_node=numa_node)
        self._used = 0

    @property
    def free_bytes(self):
        return self.nbytes - self._used

    def take(self, shape, dtype):
        shape = torch.Size(shape)
        nbytes = shape.numel() * torch.empty(0, dtype=dtype).element_size()
        if _round_up_page(nbytes) > self.free_bytes:
            raise ValueError("arena exhausted")
        piece = self._flat[self._used:self._used + nbytes]
        self._used += _round_up_page(nbytes)
        return piece.view(dtype).view(shape)


def detached(states):
    """Copies of pinned states that own their storage (plain CPU tensors).

    ``states``: a tensor, or a dict / list / tuple of them, nested as in
    ``optimizer.state_dict()``; anything that is not a tensor is passed through.
    Use it before ``torch.save`` of a subset of an ``OffloadAdam``'s states: the
    optimizer's own tensors are views into shared arenas, and serialising a view
    writes the whole arena behind it."""
    if isinstance(states, torch.Tensor):
        return states.detach().clone()
    if isinstance(states, dict):
        return {k: detached(v) for k, v in states.items()}
    if isinstance(states, (list, tuple)):
        return type(states)(detached(v) for v in states)
    return states


def largest_grantable_bytes(upper):
    """Largest single page-locked allocation the runtime grants right now, up to
    ``upper`` bytes, to 256 MiB (allocate-and-release probes that touch no page).

    A refusal by the driver's per-process limit returns at once, while a probe that
    succeeds costs about 40 ms per GiB, so the search walks down from ``upper`` while
    probes are refused and stops at the first success; should refusals turn slow (a
    host that is really out of memory) it falls back to bisection."""
    lib = _lib.load()
    step = 256 << 20
    hi = max(1, -(-upper // step))
    if lib.oa_pinned_probe(ctypes.c_size_t(hi * step)) == 0:
        return hi * step
    deadline = time.monotonic() + 2.0
    while hi > 1 and time.monotonic() < deadline:
        hi -= 1
        if lib.oa_pinned_probe(ctypes.c_size_t(hi * step)) == 0:
            return hi * step
    lo = 0
    while hi - lo > 1:
        mid = (lo + hi) // 2
        if lib.oa_pinned_probe(ctypes.c_size_t(mid * step)) == 0:
            lo = mid
        else:
            hi = mid
    return lo * step


def alloc_pinned_states(requests, numa_node="auto", arena_bytes=None):
    """Zero-filled pinned tensors for ``requests`` = [(shape, dtype), ...], carved
    from as few arenas of ``arena_bytes`` as hold them (in order, 4 KiB-aligned).

    The arenas are allocated first, all of them, before any caller data moves:
    when the runtime refuses one, those already obtained are released and a
    ``RuntimeError`` names the total that was asked for, how much had been
    granted, and the largest single allocation the runtime would still grant."""
    arena_bytes = ARENA_BYTES if arena_bytes is None else int(arena_bytes)
    sizes = [_round_up_page(torch.Size(shape).numel() * torch.empty(0, dtype=dtype).element_size())
             for shape, dtype in requests]
    plan, current = [], 0  # arena sizes, filled in request order
    for size in sizes:
        if plan and current + size <= plan[-1]:
            current += size
            continue
        if plan:
            plan[-1] = current  # close the arena at what it holds
        plan.append(max(arena_bytes, size))
        current = size
    if plan:
        plan[-1] = current
    total = sum(plan)
    arenas = []
    try:
        for nbytes in plan:
            arenas.append(PinnedArena(nbytes, numa_node))
    except RuntimeError as exc:
        granted = sum(a.nbytes for a in arenas)
        arenas.clear()
        still = largest_grantable_bytes(total)
        raise RuntimeError(
            f"pinned host memory: {total / 2**30:.1f} GiB were asked for in {len(plan)} "
            f"allocations and the runtime refused after {granted / 2**30:.1f} GiB ({exc}); the "
            f"largest single allocation it grants now is {still / 2**30:.1f} GiB. Nothing was "
            "kept. Page-locked memory is limited per process by the GPU driver, not by free "
            "RAM: offload fewer bytes per element (another mode, offload_grads=False) or raise "
            "inplace_param_threshold."
        ) from None
    out, index = [], 0
    for (shape, dtype), size in zip(requests, sizes):
        if size > arenas[index].free_bytes:
            index += 1  # the plan above closed this arena at exactly what it holds
        out.append(arenas[index].take(shape, dtype))
    return out
