"""``OffloadAdam``: Adam whose gradients and optimizer states live in pinned host
memory and visit the GPU only for the step.

Drop-in for the reference's ``offload_adam.OffloadAdam``
(src/offload_adam/offload_adam.py:39-678): same constructor knobs, mode
strings, ``ready_for_optimizer_step`` contract, per-parameter state layout and
the two execution paths selected by ``max_grad_norm``:

* ``max_grad_norm=None`` - the whole step of a parameter (H2D of its states,
  fused AdamW kernel, D2H write-back) runs inside that parameter's
  post-accumulate-grad hook on the last micro-batch, overlapping with the rest
  of backward;
* ``max_grad_norm=float`` - backward only accumulates gradients and records
  per-parameter L2 norms; ``step()`` forms the global clip coefficient on the
  GPU (no host sync) and walks the parameters, prefetching the next
  parameter's states while the current one is updated.

What runs underneath is this package's HIP library: the fused AdamW kernels
(with the clip coefficient folded into the gradient load instead of a separate
``grad.mul_`` pass), the norm / coefficient kernels, the pinned allocator and
``hipMemcpyAsync`` on two side streams fenced with events.
"""

import bisect
import collections
import operator
import os
import sys
import time
import warnings
from ctypes import c_int, c_size_t, c_uint64, c_void_p

import torch
from torch.optim.optimizer import Optimizer

from . import _copy_engines, _lib, _trace, grad_clip
from ._pretrained import stream_master_from_pretrained
from .adam import _LOSSY_MASTER_HINT, MODE_TABLE
from .kernels import adam_step_multi
from .pinned_alloc import (alloc_pinned_states, largest_grantable_bytes, numa_node_free_bytes,
                           resolve_numa_target, zeros_pinned)
from .qweight.base import QWeightBase

_BF16 = torch.bfloat16
_GIB = 1024**3


def get_leaf_modules_with_params(module):
    """Leaf modules (no children) that directly own a trainable parameter, in
    registration order.  Parameters held by a module that also has children are
    not seen (same scan as the reference, offload_adam.py:28-36)."""
    found = []
    for child in module.children():
        if any(True for _ in child.children()):
            found.extend(get_leaf_modules_with_params(child))
        elif any(p.requires_grad for p in child.parameters(recurse=False)):
            found.append(child)
    return found


# Who puts the optimizer's copies on fixed SDMA engines.  True: the kernel library's own
# copies (oa_h2d_async / oa_d2h_async / oa_link_copy_batch).  False: hipMemcpyAsync, whose
# engine the tools library rewrites when the ROCr runtime has loaded it.  None (default):
# decided at the first copy - OFFLOAD_ADAM_LINK_COPIES=direct|runtime, else hipMemcpyAsync
# when the tools library is in effect and the library's own copies when it is not (a
# late import, a profiler attached).  hipMemcpyAsync with its engine rewritten is about
# 4 % faster on an 8B step (the library's own copies are fenced in the stream by two small
# kernels per unit); the library's own copies need nothing from the process environment.
_FIXED_ENGINE_COPIES = None
_fixed_engines_unavailable = set()  # device indices on which oa_h2d_async declined


def _fixed_engine_copies():
    global _FIXED_ENGINE_COPIES
    if _FIXED_ENGINE_COPIES is None:
        want = os.environ.get("OFFLOAD_ADAM_LINK_COPIES", "auto").strip().lower()
        if want == "direct":
            _FIXED_ENGINE_COPIES = True
        elif want == "runtime":
            _FIXED_ENGINE_COPIES = False
        else:
            _FIXED_ENGINE_COPIES = not _copy_engines.tools_loaded()
    return _FIXED_ENGINE_COPIES


def _copy_async(dst, src, kind, stream):
    """Asynchronous copy of a whole contiguous tensor on ``stream`` by a DMA engine.

    Host<->device copies go through ``oa_h2d_async`` / ``oa_d2h_async``: a fixed SDMA
    engine per direction, chosen inside the library.  Where those are not available
    (``OFFLOAD_ADAM_COPY_ENGINES=off``, a runtime that hands out no signal memory)
    the copy is a ``hipMemcpyAsync`` and the HIP runtime picks the engine."""
    nbytes = src.numel() * src.element_size()
    lib = _lib.load()
    if kind != _lib.OA_COPY_D2D and _fixed_engine_copies():
        index = (dst if kind == _lib.OA_COPY_H2D else src).device.index
        if index not in _fixed_engines_unavailable:
            fn = lib.oa_h2d_async if kind == _lib.OA_COPY_H2D else lib.oa_d2h_async
            code = fn(c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), c_size_t(nbytes),
                      c_void_p(stream.cuda_stream), None, None)
            if code != _lib.OA_EUNAVAILABLE:
                _lib.check(code, "oa_h2d_async" if kind == _lib.OA_COPY_H2D else "oa_d2h_async")
                return
            _fixed_engines_unavailable.add(index)
    code = lib.oa_memcpy_async(
        c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), c_size_t(nbytes), c_int(kind),
        c_void_p(stream.cuda_stream),
    )
    _lib.check(code, "oa_memcpy_async")


_BATCH_COPIES = True  # False: one library call (and one stream round trip) per copy


def _batched(device_index):
    """Whether ``_copy_batch`` hands its copies to ``oa_link_copy_batch`` on this GPU."""
    return (_BATCH_COPIES and _fixed_engine_copies()
            and device_index not in _fixed_engines_unavailable)


def _copy_batch(pairs, kind, stream, events=None):
    """Copies ``pairs`` = [(dst, src), ...] of one direction on ``stream`` as one unit
    (``oa_link_copy_batch``): they start after the work the stream has been given so
    far and run back to back on the direction's engine.  ``events[i]``, when not None,
    is a ``torch.cuda.Event`` that has been recorded before (so that it has a handle);
    it is recorded again behind copy i.  Without the fixed-engine copies this is the
    plain loop of ``_copy_async`` calls and event records."""
    count = len(pairs)
    if count == 0:
        return
    lib = _lib.load()
    index = (pairs[0][0] if kind == _lib.OA_COPY_H2D else pairs[0][1]).device.index
    if _batched(index):
        dsts = (c_uint64 * count)(*[d.data_ptr() for d, _ in pairs])
        srcs = (c_uint64 * count)(*[s.data_ptr() for _, s in pairs])
        sizes = (c_size_t * count)(*[s.numel() * s.element_size() for _, s in pairs])
        recs = None
        if events is not None:
            recs = (c_uint64 * count)(*[0 if e is None else e.cuda_event for e in events])
        code = lib.oa_link_copy_batch(c_int(count), dsts, srcs, sizes, c_int(kind),
                                      c_void_p(stream.cuda_stream), recs)
        if code != _lib.OA_EUNAVAILABLE:
            _lib.check(code, "oa_link_copy_batch")
            return
        _fixed_engines_unavailable.add(index)
    for i, (dst, src) in enumerate(pairs):
        _copy_async(dst, src, kind, stream)
        if events is not None and events[i] is not None:
            events[i].record(stream)


def _handle_event(stream):
    """A ``torch.cuda.Event`` with a handle the library can record (torch creates the
    handle at the first record)."""
    event = torch.cuda.Event()
    event.record(stream)
    return event


_copy_engine_warned = False
_D2H_BY_KERNEL = False  # write-back engine: DMA (default) or the library's copy kernel
_D2H_WORKGROUPS = 8  # 1024-lane workgroups: enough requests in flight to fill the host link


_PROBE_TRANSFER_STREAMS = True
_PROBE_MAX_CANDIDATES = 8
_PROBE_PASS_RATIO = 0.85


def _probe_concurrency(device, h2d, d2h, bufs, rounds=6):
    """Time the optimizer's copy pattern on a candidate pair of side streams.

    Returns ``(duplex, h2d_with_compute, d2h_with_compute)``: elapsed time of two
    activities together divided by the sum of their times alone.  Measured
    values: 0.59 (both directions) and 0.72 (a direction and kernels) when they
    run side by side, 0.99-1.0 when one waits for the other.  Each copy is followed by
    an event record and preceded by a fence on the compute stream, as in the
    streaming step: those are what serialise streams that share a hardware
    queue."""
    host_in, host_out, dev_in, dev_out, x = bufs
    compute = torch.cuda.current_stream(device)

    def up():
        h2d.wait_stream(compute)
        _copy_async(dev_in, host_in, _lib.OA_COPY_H2D, h2d)
        h2d.record_event()

    def down():
        d2h.wait_stream(compute)
        _copy_async(host_out, dev_out, _lib.OA_COPY_D2H, d2h)
        d2h.record_event()

    def kernels():
        for _ in range(6):
            x.mul_(1.0)

    def timed(*activities):
        torch.cuda.synchronize(device)
        t0 = time.perf_counter()
        for _ in range(rounds):
            for act in activities:
                act()
        torch.cuda.synchronize(device)
        return time.perf_counter() - t0

    timed(up, down, kernels)  # warm
    t_up, t_down, t_k = timed(up), timed(down), timed(kernels)
    duplex = timed(up, down) / (t_up + t_down)
    # copy first: its fence covers the previous round's kernels, this round's run beside it
    up_with_compute = timed(up, kernels) / (t_k + t_up)
    down_with_compute = timed(down, kernels) / (t_k + t_down)
    return duplex, up_with_compute, down_with_compute


def pick_transfer_streams(device):
    """Two side streams on which host->device copies, device->host copies and the
    compute stream's kernels run concurrently.

    HIP streams share a small pool of hardware queues (``GPU_MAX_HW_QUEUES``, 4
    unless set before the HIP library loads); a new stream goes to the queue with
    the fewest users.  When the two transfer streams land on one queue, or one of
    them on the compute stream's, the event markers of one sit in the same
    in-order queue as the fences of the other and the link runs half duplex
    (measured on the 8B step: 3.1 s instead of 2.1 s).  Which queue a stream got
    cannot be asked, so it is measured: candidates are drawn from torch's stream
    pool until a pair passes, at most ``_PROBE_MAX_CANDIDATES`` streams.

    Returns ``(h2d_stream, d2h_stream, report)``."""
    nbytes = 32 << 20
    bufs = (
        zeros_pinned((nbytes,), torch.uint8, numa_node=None),
        zeros_pinned((nbytes,), torch.uint8, numa_node=None),
        torch.empty(nbytes, dtype=torch.uint8, device=device),
        torch.zeros(nbytes, dtype=torch.uint8, device=device),
        torch.zeros(128 << 20, dtype=torch.bfloat16, device=device),  # 0.1 ms per pass
    )
    with torch.cuda.device(device):
        h2d, d2h = torch.cuda.Stream(device), torch.cuda.Stream(device)
        tried, best = 2, None
        while True:
            duplex, up_c, down_c = _probe_concurrency(device, h2d, d2h, bufs)
            with_compute = max(up_c, down_c)
            score = max(duplex, with_compute)
            if best is None or score < best[0]:
                best = (score, h2d, d2h, duplex, with_compute)
            if score < _PROBE_PASS_RATIO or tried >= _PROBE_MAX_CANDIDATES:
                break
            # replace the stream that waited; a fresh stream from torch's pool
            # lands on the least-used hardware queue
            if up_c >= _PROBE_PASS_RATIO:
                h2d = torch.cuda.Stream(device)
            else:  # d2h shares with the compute stream or with h2d
                d2h = torch.cuda.Stream(device)
            tried += 1
        torch.cuda.synchronize(device)
    score, h2d, d2h, duplex, with_compute = best
    report = {"duplex_ratio": round(duplex, 3), "with_compute_ratio": round(with_compute, 3),
              "streams_tried": tried, "concurrent": score < _PROBE_PASS_RATIO}
    if not report["concurrent"]:
        warnings.warn(
            f"OffloadAdam: no pair of side streams ran copies concurrently ({report}); the "
            "streaming step will be slower.  Export GPU_MAX_HW_QUEUES=8 before starting Python.",
            stacklevel=3,
        )
    return h2d, d2h, report


def _copy_by_kernel(dst, src, stream, workgroups=None):
    """Copy a whole contiguous tensor with the library's copy kernel on
    ``stream``; either side may be pinned host memory."""
    nbytes = src.numel() * src.element_size()
    code = _lib.load().oa_copy_kernel_async(
        c_void_p(dst.data_ptr()), c_void_p(src.data_ptr()), c_size_t(nbytes),
        c_int(workgroups or _D2H_WORKGROUPS), c_void_p(stream.cuda_stream),
    )
    _lib.check(code, "oa_copy_kernel_async")


class OffloadAdam(Optimizer):
    """Adam with gradients and optimizer states offloaded to pinned host memory.

    Args:
        model (nn.Module): model whose leaf-module parameters are optimized.
        lr, betas, eps, weight_decay: the usual Adam hyper-parameters
            (defaults 1e-3, (0.9, 0.999), 1e-8, 0.01).
        mode (str): ``'stochastic_rounding'`` (default), ``'fp32_master'``,
            ``'fp31_master'`` or ``'fp32_master_custom_rounding'``.
        max_grad_norm (float | None): global L2-norm clipping threshold; ``None``
            (default) moves the step into the backward hooks.
        numa_node (str | int | None): NUMA placement of the pinned buffers -
            ``'auto'`` (the GPU's node), a node id, or ``None``.
        decoupled_weight_decay (bool): AdamW-style decay. Default False.
        inplace_param_threshold (int | None): parameters with fewer elements keep
            gradient and states on the GPU and never cross PCIe. Default 1M;
            ``0`` offloads everything.
        prefetch_policy (str): ``'eager'`` (default) starts a parameter's H2D at
            the first backward-pre hook that sees it; ``'lazy'`` waits for the
            module that owns it first in forward order (matters for parameters
            shared by several modules, e.g. tied embeddings).
        verbose (int): non-zero prints the pinned / in-place byte totals.
        spare_hbm (bool, keyword-only): ``False`` (default) reproduces the
            reference's memory and traffic contract - nothing but a bounded
            staging window of states lives in HBM besides the model, every
            partial gradient sum goes back to pinned host memory after its
            micro-batch and ``state[p]['grad']`` on the host is always current.
            ``True`` lets the optimizer spend HBM that is free when it is built to
            avoid crossing the host link: each of ``prefetch_bytes``,
            ``grad_cache_bytes`` and ``state_cache_bytes`` that was not given
            becomes ``'auto'`` (a tenth of the free HBM each) and
            ``grad_cache_policy`` becomes ``'write_back'``.  The HBM that may be
            held is printed once at construction.  Results are bit-identical.
        prefetch_bytes (int | 'auto', keyword-only): device staging the hook path
            may fill ahead of the gradient hooks (twice that number of bytes bounds
            the staging buffers that have been handed back while their write-back
            is still running: beyond it the host waits for the oldest write-back,
            which keeps the HBM really held close to the HBM allocated).  Default 4 GiB (and never fewer
            than the next two parameters); ``'auto'``: a tenth of the HBM that is
            free when the optimizer is built, at least 2 GiB.  The copies of a
            parameter's states start this far ahead in backward order; once a
            step completes, the first ``prefetch_bytes`` of the next step's
            states are staged straight away and wait in HBM through the
            accumulation micro-batches.
        offload_grads (bool, keyword-only): ``True`` (default) is the reference's
            behaviour - after every micro-batch the accumulated gradient goes
            back to pinned host memory and returns for the next one.  ``False``
            keeps the running gradient sum on the GPU between micro-batches
            (2 bytes per offloaded element of HBM); only optimizer states cross
            the host link, no ``state[p]['grad']`` host buffer is allocated, and
            with ``grad_accum`` micro-batches the link traffic per step drops
            from ``2*(grad_accum-1)+4`` to ``4`` bytes per element each way in
            ``stochastic_rounding`` mode.  Results are bit-identical, with one
            exception: with ``max_grad_norm`` set, a parameter that received no
            gradient since the last step sits ``step()`` out (the reference steps it
            again from the old contents of its host gradient buffer, which does not
            exist here).
        grad_cache_bytes (int | 'auto', keyword-only): with ``offload_grads=True``,
            HBM that may keep the device copy of accumulated gradients alive
            between micro-batches.  What is saved is fetching the same bytes again
            for the next micro-batch, or for ``step()`` on the clipping path (and,
            under ``grad_cache_policy='write_back'``, writing partial sums nobody
            reads).  Parameters are admitted in optimizer order until the budget
            is used.  Default ``0``: fetch every time, like the reference;
            ``'auto'``: a tenth of the HBM that is free when the optimizer is
            built.  Results are bit-identical.
        grad_cache_policy (str, keyword-only): when a gradient kept by
            ``grad_cache_bytes`` reaches the host.  ``'write_through'`` (default):
            after every micro-batch, as the reference does, so
            ``optimizer.state[p]['grad']`` is current between micro-batches.
            ``'write_back'``: when somebody asks for it - ``state_dict()`` brings
            every host gradient up to date before it returns - so partial sums
            that the next micro-batch replaces anyway do not cross the link.
        state_cache_bytes (int | 'auto', keyword-only): the same for the optimizer
            states: HBM that may keep the device copy of a parameter's states
            alive after the step has written them back to the host.  The host
            copy stays current after every step; what is saved is fetching the
            same bytes for the next step.  Parameters are admitted from the end
            of the optimizer's order (the ones backward reaches first, whose
            fetch has the least time to arrive).  Default ``0``: keep nothing,
            like the reference; ``'auto'``: a tenth of the HBM that is free when
            the optimizer is built (with ``max_grad_norm`` set and
            ``prefetch_bytes`` left alone, that budget is added: states staged
            ahead of ``step()`` would hold the same HBM at the same time).
            Results are bit-identical.
        pinned_limit_bytes (int | None, keyword-only): page-locked host memory the
            optimizer may take.  ``None`` (default): what the GPU driver grants this
            process (asked once at construction when more than 4 GiB are needed;
            64 GiB per process on some systems, whatever the free RAM).  When the
            states do not fit, the overflow stays in HBM instead of failing:
            first the gradients of as many parameters as needed, in optimizer
            order (for those, as with ``offload_grads=False``, the running sum
            never leaves the GPU and ``state[p]`` holds no ``'grad'``), then
            whole parameters (gradient and states resident, like the small ones
            below ``inplace_param_threshold``).  One notice on stderr says what
            was moved; ``RuntimeError`` only when HBM cannot take it either.
            Results are bit-identical.
        pending_writeback_bytes (int | None, keyword-only): bytes of staging buffers
            that may be handed back to the allocator while their write-back to the
            host is still running.  Such memory no longer counts as allocated but
            is not free either, and the hooks run far ahead of the host link; past
            this limit the host waits for the oldest write-back before it stages
            more.  ``None`` (default): twice the staging window (``prefetch_bytes``),
            at least 2 GiB - free of charge where micro-batches are accumulated and
            with ``max_grad_norm``, 0.6-2 % on steps of one micro-batch, which a
            limit of four windows avoids at that much more HBM held.  Results are
            bit-identical.
    """

    supported_modes = {
        mode: {
            "step": fn,
            "offload": {"grad": _BF16, "exp_avg": _BF16, "exp_avg_sq": _BF16, **extra},
        }
        for mode, (fn, extra) in MODE_TABLE.items()
    }

    _DEFAULT_INPLACE_PARAM_THRESHOLD = 1024 * 1024
    _CLIP_PREFETCH_DEPTH = 2  # parameters whose H2D runs ahead of the step loop
    # Hook path: parameters whose gradient is complete are stepped in groups - one
    # multi-tensor launch, one fence and one event for the write-back of the whole
    # group - because the host cost of a hook (about 85 us per parameter when each
    # is stepped alone, mostly stream waits and launches) is what a step of a
    # 1B-parameter model is bound by.  A group closes at this many parameters or
    # bytes of gradient, whichever comes first, and when the backward pass ends.
    _STEP_GROUP_PARAMS = 8
    _STEP_GROUP_BYTES = 256 << 20
    _NORM_GROUP_BYTES = 512 << 20  # clipping path: gradients one norm launch may keep alive
    _PREFETCH_MIN_PARAMS = 2  # hook path: H2D window ahead of the gradient hooks ...
    # ... and in bytes of device staging: the default window is this, or an eighth of
    # the offloaded bytes when that is less (a 1B-parameter model steps 3 % faster with
    # 0.75 GiB than with 4, at a third less HBM: its write-backs have the link to themselves)
    _PREFETCH_BYTES = 4 << 30
    _WRITEBACK_PENDING_BYTES = None  # None: derived from the staging window, see __init__
    _PREFETCH_BYTES_MIN = 256 << 20

    def __init__(
        self,
        model,
        lr=1e-3,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=0.01,
        mode="stochastic_rounding",
        max_grad_norm=None,
        numa_node="auto",
        decoupled_weight_decay=False,
        inplace_param_threshold=None,
        prefetch_policy="eager",
        verbose=0,
        *,
        offload_grads=True,
        prefetch_bytes=None,
        grad_cache_bytes=None,
        state_cache_bytes=None,
        grad_cache_policy=None,
        spare_hbm=False,
        pinned_limit_bytes=None,
        pending_writeback_bytes=None,
    ):
        if prefetch_policy not in ("eager", "lazy"):
            raise ValueError(f"prefetch_policy must be 'eager' or 'lazy' (got {prefetch_policy!r})")
        self._prefetch_policy = prefetch_policy
        assert mode in self.supported_modes, (
            f"Invalid mode: {mode}, available modes: {list(self.supported_modes)}"
        )
        self.mode = mode
        self.step_fn = self.supported_modes[mode]["step"]
        self.offload_config = self.supported_modes[mode]["offload"]
        self.offload_state_keys = list(self.offload_config)
        self._non_grad_keys = [k for k in self.offload_state_keys if k != "grad"]
        self.offload_grads = bool(offload_grads)
        # Budgets: an int, 'auto' (a tenth of the HBM free at construction) or None,
        # which is the reference's contract unless spare_hbm asks for 'auto'.
        def byte_count(name, value, auto_ok=True):
            """An integer number of bytes: ints, numpy integers, floats such as 2e9."""
            if value is None or (auto_ok and isinstance(value, str) and value == "auto"):
                return value
            ok = not isinstance(value, (bool, str))
            if ok and isinstance(value, float):
                ok = value.is_integer()
            if ok:
                try:
                    value = int(value) if isinstance(value, float) else operator.index(value)
                except TypeError:
                    ok = False
            if not ok or value < 0:
                kinds = "a non-negative int, 'auto' or None" if auto_ok else "a non-negative int or None"
                raise ValueError(f"{name} must be {kinds} (got {value!r})")
            return value

        prefetch_bytes = byte_count("prefetch_bytes", prefetch_bytes)
        grad_cache_bytes = byte_count("grad_cache_bytes", grad_cache_bytes)
        state_cache_bytes = byte_count("state_cache_bytes", state_cache_bytes)
        self._pinned_limit_arg = byte_count("pinned_limit_bytes", pinned_limit_bytes, auto_ok=False)
        pending_writeback_bytes = byte_count("pending_writeback_bytes", pending_writeback_bytes,
                                             auto_ok=False)
        if pending_writeback_bytes is not None:
            self._WRITEBACK_PENDING_BYTES = pending_writeback_bytes
        self.spare_hbm = bool(spare_hbm)
        if self.spare_hbm:
            prefetch_bytes = "auto" if prefetch_bytes is None else prefetch_bytes
            grad_cache_bytes = "auto" if grad_cache_bytes is None else grad_cache_bytes
            state_cache_bytes = "auto" if state_cache_bytes is None else state_cache_bytes
            grad_cache_policy = "write_back" if grad_cache_policy is None else grad_cache_policy
        else:
            grad_cache_bytes = 0 if grad_cache_bytes is None else grad_cache_bytes
            state_cache_bytes = 0 if state_cache_bytes is None else state_cache_bytes
            grad_cache_policy = "write_through" if grad_cache_policy is None else grad_cache_policy
        self._prefetch_bytes_arg = prefetch_bytes
        if isinstance(prefetch_bytes, int):
            self._PREFETCH_BYTES = prefetch_bytes
        if grad_cache_policy not in ("write_back", "write_through"):
            raise ValueError("grad_cache_policy must be 'write_back' or 'write_through' "
                             f"(got {grad_cache_policy!r})")
        self._grad_cache_write_back = grad_cache_policy == "write_back"

        self.max_grad_norm = max_grad_norm
        self._step_in_backward = max_grad_norm is None
        self.decoupled_weight_decay = decoupled_weight_decay
        self.verbose = verbose
        self.ready_for_optimizer_step = False

        modules = get_leaf_modules_with_params(model)
        params, owners = [], {}
        for m in modules:
            for p in m.parameters():
                if p.requires_grad:
                    if id(p) not in owners:
                        params.append(p)  # tied weights enter the optimizer once
                    owners[id(p)] = owners.get(id(p), 0) + 1
        shared = [p for p in params if owners[id(p)] > 1]
        if shared and prefetch_policy == "eager":
            warnings.warn(
                f"OffloadAdam: {len(shared)} parameter(s) shared across multiple leaf modules "
                f"({sum(p.numel() for p in shared):,} elements; e.g. tied embeddings). With "
                f"prefetch_policy='eager' their non-grad states sit on GPU through the whole "
                f"backward. Pass prefetch_policy='lazy' to defer prefetch to the input-side "
                f"module.",
                stacklevel=2,
            )
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))

        self._quant_params = {p for p in params if isinstance(p.data, QWeightBase)}
        if self._quant_params and mode != "fp32_master":
            raise ValueError(
                f"QAT params require mode='fp32_master'; got {mode!r} "
                f"({len(self._quant_params)} quant params detected)"
            )
        self._quant_master_warned = False

        if inplace_param_threshold is None:
            inplace_param_threshold = self._DEFAULT_INPLACE_PARAM_THRESHOLD
        self.inplace_param_threshold = inplace_param_threshold
        # quantised params always offload: their fp32 master belongs on the host
        self._inplace_params = {
            p for p in params
            if p.numel() < inplace_param_threshold and p not in self._quant_params
        }
        self._offload_params = [p for p in params if p not in self._inplace_params]
        # offloaded parameters whose running gradient sum never leaves the GPU: all of
        # them with offload_grads=False, else those the pinned-memory limit displaces
        self._grad_on_device = set() if self.offload_grads else set(self._offload_params)
        self.pinned_limit_report = None  # what _fit_pinned_limit moved to HBM, if anything
        self._fit_pinned_limit()

        def tenth_of_free_hbm():
            dev0 = self._offload_params[0].device
            return torch.cuda.mem_get_info(dev0)[0] // 10 if dev0.type == "cuda" else 0

        if self._prefetch_bytes_arg == "auto" and self._offload_params:
            # the model is already on the GPU; at least 2 GiB
            self._PREFETCH_BYTES = max(2 << 30, tenth_of_free_hbm())
        elif self._prefetch_bytes_arg is None:
            eighth = self._estimate_pinned_bytes(self._offload_params) // 8
            self._PREFETCH_BYTES = min(self._PREFETCH_BYTES, max(self._PREFETCH_BYTES_MIN, eighth))

        # parameters whose accumulated gradient stays on the GPU between micro-batches
        self._grad_cached = set()
        self._stale_host_grads = set()  # write_back policy: host copy older than the device's
        if self.offload_grads and self._offload_params:
            budget = tenth_of_free_hbm() if grad_cache_bytes == "auto" else grad_cache_bytes
            for p in self._offload_params:
                if p in self._grad_on_device:
                    continue
                nbytes = p.numel() * 2
                if nbytes > budget:
                    break
                budget -= nbytes
                self._grad_cached.add(p)

        # parameters whose states stay on the GPU after their write-back
        self._state_cached = set()
        # Clipping path: states staged for step() ahead of time occupy their HBM
        # through the last backward pass, when memory peaks, so keeping them instead
        # costs no more and saves the transfer (8B model: 21 GB per step, which
        # arrived 0.1 s late beside the backward kernels).  When both budgets are
        # 'auto', the staging budget goes to the state cache.
        fold = (not self._step_in_backward and self._prefetch_bytes_arg == "auto"
                and state_cache_bytes == "auto" and self.spare_hbm)
        self._prestage_bytes = 0 if fold else self._PREFETCH_BYTES
        if self._offload_params:
            budget = state_cache_bytes
            if budget == "auto":
                budget = tenth_of_free_hbm()
                if fold:
                    budget += self._PREFETCH_BYTES
            per_elem = sum(torch.empty(0, dtype=d).element_size()
                           for k, d in self.offload_config.items() if k != "grad")
            for p in reversed(self._offload_params):
                nbytes = p.numel() * per_elem
                if nbytes > budget:
                    break
                budget -= nbytes
                self._state_cached.add(p)

        if (self.verbose > 0 or self.spare_hbm) and self._offload_params:
            cached_g = sum(p.numel() for p in self._grad_cached) * 2
            cached_s = sum(p.numel() for p in self._state_cached) * (
                sum(torch.empty(0, dtype=d).element_size()
                    for k, d in self.offload_config.items() if k != "grad"))
            # part of the verbose report on stdout; at verbose=0 (spare_hbm) a notice on stderr
            print(f"HBM the optimizer may hold: gradient cache {cached_g / _GIB:.2f} GB "
                  f"({len(self._grad_cached)} params), state cache {cached_s / _GIB:.2f} GB "
                  f"({len(self._state_cached)} params), prefetch staging "
                  f"{self._PREFETCH_BYTES / _GIB:.2f} GB",
                  file=sys.stdout if self.verbose > 0 else sys.stderr)

        self._pending_norms = []      # clipping path: (gradient, slot) pairs waiting for their launch
        self._pending_norm_bytes = 0
        self._pending_steps = []      # offloaded parameters waiting for their group's launch
        self._pending_inplace = []    # GPU-resident ones
        self._pending_step_bytes = 0
        self._pending_writebacks = []  # cached gradients whose write-back waits for its group
        self._pending_writeback_bytes = 0
        self.device_states = {}
        # Device buffers given back to the allocator while a write-back still reads them
        # (``record_stream``): they no longer count as allocated, yet their memory is in
        # use until the copy is done.  The hooks run as fast as the host can enqueue, far
        # ahead of the link, so without a bound every staged byte of a pass ends up in
        # that state at once (8B model: 61 GiB held from the driver at 24.7 GiB
        # "allocated"; 96 GiB on the clipping path).  ``_throttle_writebacks`` makes the
        # host wait for the oldest write-back once more than this many bytes are pending.
        self._writebacks_pending = collections.deque()  # (event, bytes), write-back order
        self._writeback_pending_bytes = 0
        # Twice the staging window, at least 2 GiB: free of charge where micro-batches
        # are accumulated and on the clipping path, at most 2 % on steps of a single
        # micro-batch (link-bound from end to end, where the host's lead over the link is
        # what keeps both directions busy); the window itself costs those 5-10 %.
        self._writeback_pending_limit = (
            self._WRITEBACK_PENDING_BYTES if self._WRITEBACK_PENDING_BYTES is not None
            else max(2 * self._PREFETCH_BYTES, 2 << 30))
        self.h2d_events = {}
        self._h2d_event_objs = {}  # library-issued copies: the event object each parameter keeps
        self.d2h_events = {}
        self._compute_streams = {}  # raw stream handle -> torch.cuda.Stream
        self.transfer_stream_report = None
        if self._offload_params:
            self._check_copy_engines()
        if self._offload_params and _PROBE_TRANSFER_STREAMS:
            self.h2d_stream, self.d2h_stream, self.transfer_stream_report = pick_transfer_streams(
                self._offload_params[0].device
            )
            if self.verbose > 0:
                from . import _runtime_env

                print(f"Transfer streams: {self.transfer_stream_report}")
                print(f"Process environment set at import: {_runtime_env.prepare()} "
                      "(HSA_TOOLS_LIB gets the copy-engine library, GPU_MAX_HW_QUEUES the "
                      "number of hardware queues)")
        else:
            self.h2d_stream = torch.cuda.Stream()
            self.d2h_stream = torch.cuda.Stream()
        self._param2group = {p: g for g in self.param_groups for p in g["params"]}
        # first module in forward order that owns each offloaded param ('lazy' policy)
        self._prefetch_module = {}
        for m in modules:
            for p in m.parameters():
                if p.requires_grad and p not in self._inplace_params:
                    self._prefetch_module.setdefault(p, m)

        # order in which gradient hooks fire (learned on the first backward pass)
        self._bw_order = []
        self._bw_pos = {}
        self._bw_order_known = False
        self._bw_cursor = -1
        self._bw_prefix = [0]
        self._bw_issued_upto = 0
        self._bytes_per_elem_in_flight = sum(
            torch.empty(0, dtype=d).element_size() for d in self.offload_config.values()
        )

        # clipping: one bf16 slot per parameter, reduced by one kernel in step()
        self._norm_slots = None
        self._clip_coef = None
        if max_grad_norm is not None:
            dev = params[0].device if params else torch.device("cuda")
            self._norm_slots = torch.zeros(max(len(params), 1), dtype=_BF16, device=dev)
            self._clip_coef = torch.ones((), dtype=_BF16, device=dev)
            self._total_norm = torch.zeros((), dtype=_BF16, device=dev)

        self._register_hooks(modules, params)
        self._numa_precheck(self._offload_params, numa_node)
        self._alloc_pinned_states(self._offload_params, numa_node)
        self._alloc_inplace_states(self._inplace_params)

    # ------------------------------------------------------------------ setup

    def _register_hooks(self, modules, params):
        # offloaded parameters of each hooked module, looked up once (walking
        # module.parameters() costs ~10 us per hook call)
        self._module_params = {}
        for module in modules:
            own = tuple(p for p in module.parameters()
                        if p.requires_grad and p not in self._inplace_params)
            if own:
                self._module_params[module] = own
                module.register_full_backward_pre_hook(self._pre_backward_hook)
        for index, p in enumerate(params):
            state = self.state[p]
            state["step"] = 0
            if self.max_grad_norm is not None:
                state["grad_norm"] = self._norm_slots[index]  # 0-dim view of the shared buffer
            if p in self._inplace_params:
                p.register_post_accumulate_grad_hook(self._inplace_grad_hook)
            else:
                p.register_post_accumulate_grad_hook(self._grad_hook)
                self.device_states[p] = {}
                state["host_grad_valid"] = False

    def _host_keys(self, p):
        """Names of the states of offloaded parameter ``p`` that live in pinned host memory."""
        if p in self._grad_on_device:
            return self._non_grad_keys
        return self.offload_state_keys

    def _estimate_pinned_bytes(self, params):
        size = {k: torch.empty(0, dtype=d).element_size() for k, d in self.offload_config.items()}
        return sum(p.numel() * sum(size[k] for k in self._host_keys(p)) for p in params)

    _PINNED_PROBE_FROM = 4 << 30   # requests below this are not pre-flighted
    _PINNED_RESERVE = 1 << 30      # left to the rest of the process (loaders, staging probes)

    def _fit_pinned_limit(self):
        """Decide what stays in HBM when the pinned states exceed what the driver
        grants (or ``pinned_limit_bytes``): gradients first, in optimizer order,
        then whole parameters.  Runs before hooks, caches and buffers are set up."""
        need = self._estimate_pinned_bytes(self._offload_params)
        if not self._offload_params or self._offload_params[0].device.type != "cuda":
            return
        if self._pinned_limit_arg is not None:
            budget = self._pinned_limit_arg
        elif need < self._PINNED_PROBE_FROM:
            return
        else:
            asked = need + self._PINNED_RESERVE
            budget = largest_grantable_bytes(asked)
            if budget >= asked:
                return
            budget -= self._PINNED_RESERVE
        if need <= budget:
            return
        wanted = need
        size = {k: torch.empty(0, dtype=d).element_size() for k, d in self.offload_config.items()}
        state_b = sum(size[k] for k in self._non_grad_keys)
        moved_grads = []
        for p in self._offload_params:
            if need <= budget:
                break
            if p not in self._grad_on_device:
                self._grad_on_device.add(p)
                moved_grads.append(p)
                need -= p.numel() * size["grad"]
        moved_whole = []
        for p in self._offload_params:
            if need <= budget:
                break
            if p in self._quant_params:
                continue  # its fp32 master is re-encoded by the offloaded step only
            moved_whole.append(p)
            need -= p.numel() * state_b
        if need > budget:
            raise RuntimeError(
                f"OffloadAdam: {wanted / _GIB:.1f} GiB of page-locked host memory are needed, "
                f"{budget / _GIB:.1f} GiB may be taken, and what could move to HBM (every "
                "gradient, every parameter that is not quantised) does not close the gap. "
                "Page-locked memory is limited per process by the GPU driver, not by free RAM.")
        whole = set(moved_whole)
        hbm = (sum(p.numel() for p in moved_grads) * size["grad"]
               + sum(p.numel() for p in moved_whole) * state_b)
        free = torch.cuda.mem_get_info(self._offload_params[0].device)[0]
        if hbm > free:
            raise RuntimeError(
                f"OffloadAdam: {wanted / _GIB:.1f} GiB of page-locked host memory are needed and "
                f"{budget / _GIB:.1f} GiB may be taken; the remaining {hbm / _GIB:.1f} GiB do not "
                f"fit the {free / _GIB:.1f} GiB of HBM that are free either.")
        self._grad_on_device -= whole
        self._inplace_params |= whole
        self._offload_params = [p for p in self._offload_params if p not in whole]
        self.pinned_limit_report = {
            "needed_bytes": wanted, "limit_bytes": budget, "hbm_bytes": hbm,
            "grads_in_hbm": len([p for p in moved_grads if p not in whole]),
            "params_in_hbm": len(moved_whole),
        }
        print(f"OffloadAdam: {wanted / _GIB:.1f} GiB of page-locked host memory are needed, "
              f"{budget / _GIB:.1f} GiB may be taken; kept in HBM instead ({hbm / _GIB:.1f} GiB): "
              f"the gradients of {self.pinned_limit_report['grads_in_hbm']} parameters"
              + (f" and all states of {len(moved_whole)} parameters" if moved_whole else ""),
              file=sys.stderr)

    def _numa_precheck(self, params, numa_node):
        """Warn when the target NUMA node cannot hold the pinned budget: the soft
        node preference then spills the rest to remote nodes."""
        target = resolve_numa_target(numa_node)
        if target is None or not params:
            return
        free = numa_node_free_bytes(target)
        if free is None:
            return
        need = self._estimate_pinned_bytes(params)
        world_size = getattr(self, "_world_size", 1)
        fair_share = free // world_size
        if need > fair_share:
            warnings.warn(
                f"OffloadAdam: need {need / _GIB:.1f} GB pinned on NUMA node {target} "
                f"({world_size} rank(s) sharing) but fair share is {fair_share / _GIB:.1f} GB; "
                f"~{(need - fair_share) / _GIB:.1f} GB will spill to remote nodes (H2D may slow "
                f"~10-15%). Pass `numa_node=None` to let the kernel spread freely, or move GPUs "
                f"to separate NUMA domains.",
                stacklevel=3,
            )

    def _copy_master(self, p, tensor):
        dev = self.device_states.get(p)
        if dev is not None:
            # offloaded: let a write-back still under way land first, and a fetch
            # still under way finish reading the host buffer (states of the next
            # step are staged as soon as a step completes); then forget any device
            # copy (staged or cached) of the value being replaced
            self._flush_steps()
            for events in (self.d2h_events, self.h2d_events):
                event = events.get(p)
                if event is not None:
                    event.synchronize()
            # every staged state of p has arrived (the event covers them all), so
            # the ones that stay need no fence any more
            self.h2d_events.pop(p, None)
            dev["master_params"] = None
        self.state[p]["master_params"].copy_(tensor)

    def _alloc_pinned_states(self, params, numa_node):
        # Every state of every parameter, carved out of a few large pinned arenas; the
        # arenas are all obtained (or the request refused as a whole) before any
        # value is written.
        requests = [(p.shape, self.offload_config[name]) for p in params
                    for name in self._host_keys(p)]
        tensors = iter(alloc_pinned_states(requests, numa_node=numa_node))
        total = 0
        for p in params:
            state = self.state[p]
            for name in self._host_keys(p):
                t = next(tensors)
                if name == "master_params":
                    t.copy_(p.data)  # widens bf16 losslessly; dequantises a quantised weight
                state[name] = t
                total += t.numel() * t.element_size()
            if p in self._quant_params and "master_params" in self.offload_config:
                state["master_filled"] = False
        if self.verbose > 0 and params:
            print(f"Pinned host memory allocated: {total / _GIB:.2f} GB")

    def _alloc_inplace_states(self, params):
        """GPU-resident gradient and states of the small parameters.  The gradient
        buffer starts at zero and is zeroed after every step, so the hook can
        always ``add_`` into it."""
        total = 0
        for p in params:
            state = self.state[p]
            for name, dtype in self.offload_config.items():
                t = torch.zeros_like(p, dtype=dtype)
                if name == "master_params":
                    t.copy_(p.data)
                state[name] = t
                total += t.numel() * t.element_size()
        if self.verbose > 0 and params:
            print(f"In-place GPU states for {len(params)} small params: {total / 1024**2:.2f} MB")

    # --------------------------------------------------- transfer primitives
    # Ordering contract, per parameter p:
    #   H2D(p) starts after D2H(p) of the previous step and after everything the
    #   compute stream has enqueued so far (its destination buffers come from the
    #   compute stream's allocator pool);
    #   the compute stream waits for H2D(p) before touching p's device states;
    #   D2H(p) starts after everything the compute stream has enqueued so far;
    #   a device buffer is not recycled before the D2H that reads it is done;
    #   a device buffer that outlives its D2H (gradient / state cache) is not
    #   written again by the compute stream before that D2H is done.

    def _check_copy_engines(self):
        """Warn once when neither way of fixing the SDMA engine per direction is in
        effect - the library's own copies (``oa_h2d_async`` / ``oa_d2h_async``) nor the
        tools library that rewrites the HIP runtime's: the runtime then picks an engine
        per copy, and the streaming step runs half duplex with stretches of 10 GB/s
        write-back.  An error instead with ``OFFLOAD_ADAM_REQUIRE_COPY_ENGINES=1``."""
        global _copy_engine_warned
        st = _copy_engines.status()
        if st["direct"] or st["loaded"] or st["install"] == "off":
            return
        message = (
            "OffloadAdam: host<->device copies are not pinned to fixed SDMA engines (the "
            f"library's own copies are unavailable: {st['direct_reason']}; "
            f"{_copy_engines.LIB_PATH.name} is not in effect: {st['install']}); expect a slower "
            "streaming step.  Set OFFLOAD_ADAM_COPY_ENGINES=off to silence this.")
        from . import _runtime_env

        if _runtime_env.required():
            raise RuntimeError("OFFLOAD_ADAM_REQUIRE_COPY_ENGINES is set: " + message)
        if _copy_engine_warned:
            return
        _copy_engine_warned = True
        warnings.warn(message, stacklevel=3)

    def _host_view(self, p, name):
        return self.state[p][name]

    def _compute_stream(self):
        """The calling thread's current stream as a ``torch.cuda.Stream``; the
        objects are kept per raw handle (building one costs ~3 us per call and a
        hook needs it three times)."""
        raw = _lib.current_stream_id()
        stream = self._compute_streams.get(raw)
        if stream is None:
            stream = self._compute_streams[raw] = torch.cuda.current_stream()
        return stream

    def _issue_h2d(self, p, keys):
        self._issue_h2d_many([(p, keys)])

    def _issue_h2d_many(self, items):
        """H2D of ``keys`` of every ``(p, keys)`` in ``items`` behind ONE fence.

        A cross-stream wait that is still pending costs 15-25 us of host time, and
        the compute stream always has work queued.  All destination buffers are
        allocated first: whatever block the allocator hands out was released by
        work the compute stream had been given before that moment, so a single
        fence taken after the last allocation orders every copy below behind the
        previous users of its buffer."""
        if not items:
            return
        self._throttle_writebacks()  # before more staging is allocated
        h2d = self.h2d_stream
        staged = []
        for p, keys in items:
            event = self.d2h_events.get(p)
            if event is not None:
                h2d.wait_event(event)
            for key in keys:
                host = self._host_view(p, key)
                staged.append((p, key, host,
                               torch.empty(host.shape, dtype=host.dtype, device=p.device)))
        h2d.wait_stream(self._compute_stream())
        last = len(staged) - 1
        batched = _batched(staged[0][3].device.index)
        pairs, events = [], []
        for i, (p, key, host, buf) in enumerate(staged):
            # the buffer belongs to the compute stream's pool: if it is dropped
            # before a consumer has waited for this copy, the allocator must not
            # hand it out again while the copy still writes it
            buf.record_stream(h2d)
            self.device_states[p][key] = buf
            last_of_p = i == last or staged[i + 1][0] is not p
            if not batched:
                _copy_async(buf, host, _lib.OA_COPY_H2D, h2d)
                if last_of_p:
                    self.h2d_events[p] = h2d.record_event()
                continue
            pairs.append((buf, host))
            if last_of_p:
                # One event object per parameter for good, recorded behind p's last copy
                # by the batch below.  (It needs a handle, which torch creates at a first
                # record; doing that once instead of before every batch keeps a marker
                # per parameter and micro-batch out of the transfer stream.  A wait
                # taken earlier keeps referring to the record it saw.)
                event = self._h2d_event_objs.get(p)
                if event is None:
                    event = self._h2d_event_objs[p] = _handle_event(h2d)
                events.append(event)
                self.h2d_events[p] = event
            else:
                events.append(None)
        # one unit: the engine runs the copies back to back, the stream follows
        _copy_batch(pairs, _lib.OA_COPY_H2D, h2d, events)

    def _throttle_writebacks(self):
        """Keep the bytes that freed staging buffers still occupy below the limit: forget
        write-backs that have completed, then wait (the host, not a stream) for the
        oldest ones until the rest fits."""
        pending = self._writebacks_pending
        while pending and pending[0][0].query():
            self._writeback_pending_bytes -= pending.popleft()[1]
        while pending and self._writeback_pending_bytes > self._writeback_pending_limit:
            event, nbytes = pending.popleft()
            event.synchronize()
            self._writeback_pending_bytes -= nbytes

    def _note_writeback(self, event, nbytes):
        if nbytes:
            self._writebacks_pending.append((event, nbytes))
            self._writeback_pending_bytes += nbytes

    def _issue_d2h(self, p, keys):
        self._throttle_writebacks()
        compute = self._compute_stream()
        dev = self.device_states[p]
        self.d2h_stream.wait_stream(compute)
        pairs, released = [], 0
        for key in keys:
            buf = dev[key]
            # Both directions use the DMA engines.  A copy kernel moves the same
            # bytes at the same rate, but while it streams writes to host memory
            # every kernel boundary of the compute stream waits behind them
            # (measured: a 0.07 ms elementwise kernel took 2 ms); DMA copies do
            # not disturb the compute stream.
            if _D2H_BY_KERNEL and buf.data_ptr() % 16 == 0:
                _copy_by_kernel(self._host_view(p, key), buf, self.d2h_stream)
            else:
                pairs.append((self._host_view(p, key), buf))
            buf.record_stream(self.d2h_stream)
            if not self._stays_on_device(p, key):
                dev[key] = None
                released += buf.numel() * buf.element_size()
        _copy_batch(pairs, _lib.OA_COPY_D2H, self.d2h_stream)
        event = self.d2h_events[p] = self.d2h_stream.record_event()
        self._note_writeback(event, released)

    def _stays_on_device(self, p, key):
        """Write-through caches: the device copy outlives its write-back."""
        return p in (self._grad_cached if key == "grad" else self._state_cached)

    def _issue_d2h_many(self, items):
        """Write-back of ``keys`` of every ``(p, keys)`` behind one fence, with one
        event for the group (a later fetch of any of them waits for all)."""
        if not items:
            return
        self._throttle_writebacks()
        d2h = self.d2h_stream
        d2h.wait_stream(self._compute_stream())
        pairs, released = [], 0
        for p, keys in items:
            dev = self.device_states[p]
            for key in keys:
                buf = dev[key]
                pairs.append((self._host_view(p, key), buf))
                buf.record_stream(d2h)
                if not self._stays_on_device(p, key):
                    dev[key] = None
                    released += buf.numel() * buf.element_size()
        _copy_batch(pairs, _lib.OA_COPY_D2H, d2h)
        event = d2h.record_event()
        for p, _ in items:
            self.d2h_events[p] = event
        self._note_writeback(event, released)

    def _ensure_on_device(self, p, keys):
        dev = self.device_states[p]
        missing = [k for k in keys if dev.get(k) is None]
        if missing:
            self._issue_h2d(p, missing)
        if p in self.h2d_events:
            self._compute_stream().wait_event(self.h2d_events[p])

    # ------------------------------------------------- per-parameter operations

    def _accumulate_grad_on_device(self, p):
        """First micro-batch of a window adopts ``p.grad`` as the device gradient;
        later ones wait for the prefetched host gradient and add into it."""
        dev, state = self.device_states[p], self.state[p]
        if p in self._grad_on_device:
            # the running sum never leaves the GPU
            if dev.get("grad") is None:
                dev["grad"] = p.grad
            else:
                dev["grad"].add_(p.grad)
        elif state["host_grad_valid"]:
            kept = dev.get("grad")
            # fetches the sum when it is not here, and waits for a fetch under way
            self._ensure_on_device(p, ["grad"])
            if kept is None:
                dev["grad"].add_(p.grad)  # a fresh copy from the host: nobody else reads it
            elif kept.dtype == p.grad.dtype and p.grad.is_contiguous():
                # The device copy was kept (grad_cache_bytes) and its write-back may
                # still be reading it.  The sum goes into this micro-batch's buffer
                # instead (a + b == b + a bit for bit), so the compute stream never
                # waits for the host link; the kept buffer is released when the
                # write-back that holds it (record_stream) is done.
                p.grad.add_(kept)
                dev["grad"] = p.grad
            else:
                if p in self.d2h_events:
                    # in-place sum: the write-back must have read the kept copy first
                    self._compute_stream().wait_event(self.d2h_events[p])
                kept.add_(p.grad)
        else:
            dev["grad"] = p.grad
            state["host_grad_valid"] = True
        p.grad = None

    def _maybe_warn_quant_master(self, state):
        if self._quant_master_warned or state.get("master_filled") is not False:
            return
        warnings.warn("OffloadAdam: " + _LOSSY_MASTER_HINT, stacklevel=3)
        self._quant_master_warned = True

    def _call_step_fn(self, p, group, tensors, clip_coef=None):
        state = self.state[p]
        beta1, beta2 = group["betas"]
        quant = p in self._quant_params
        if quant:
            self._maybe_warn_quant_master(state)
        # A quantised weight cannot take the kernel's bf16 write-back.  The
        # fp32_master step function re-encodes the payload from the new master
        # itself (one fused pass); any other step function writes its bf16 copy
        # to the gradient buffer (a sink) and the payload is re-encoded after it.
        fused = quant and self.mode == "fp32_master"
        self.step_fn(
            tensors["grad"] if quant and not fused else p.data,
            tensors,
            group["lr"],
            group["weight_decay"],
            beta1,
            beta2,
            group["eps"],
            state["step"],
            decoupled_weight_decay=self.decoupled_weight_decay,
            clip_coef=clip_coef,
        )
        if quant and not fused:
            p.data.copy_(tensors["master_params"])

    def _step_offload(self, p, group, clip_coef=None):
        dev = self.device_states[p]
        self._ensure_on_device(p, self.offload_state_keys)
        if p in self._state_cached and p in self.d2h_events:
            # the kernel rewrites states whose last write-back may still be reading them
            self._compute_stream().wait_event(self.d2h_events[p])
        self._call_step_fn(p, group, dev, clip_coef)
        self._issue_d2h(p, self._non_grad_keys)
        dev["grad"] = None
        self._stale_host_grads.discard(p)

    def _step_inplace(self, p, group, clip_coef=None):
        state = self.state[p]
        self._call_step_fn(p, group, {k: state[k] for k in self.offload_state_keys}, clip_coef)
        state["grad"].zero_()

    def _step_inplace_batch(self, params, group, clip_coef=None):
        """``_step_inplace`` for a list of parameters with one multi-tensor launch."""
        beta1, beta2 = group["betas"]
        tensors, steps = [], []
        for p in params:
            state = self.state[p]
            state["step"] += 1
            steps.append(state["step"])
            tensors.append({k: state[k] for k in self.offload_state_keys})
        adam_step_multi(
            self.mode,
            [p.data for p in params],
            tensors,
            group["lr"],
            group["weight_decay"],
            beta1,
            beta2,
            group["eps"],
            steps,
            decoupled_weight_decay=self.decoupled_weight_decay,
            clip_coef=clip_coef,
        )
        torch._foreach_zero_([t["grad"] for t in tensors])

    def _flush_at_end_of_backward(self):
        """Queue ``_flush_steps`` on the autograd engine: it runs when this backward
        pass has executed its last node, so no group is ever left waiting for a
        hook that does not come.  False outside a backward pass.

        Queued once per parameter (half a microsecond; a call that finds nothing
        pending returns at once) rather than once per pass behind a flag: a pass
        that raises never runs its callbacks, and a flag it left set would keep
        the next pass from queueing its own."""
        try:
            torch.autograd.Variable._execution_engine.queue_callback(self._flush_steps)
        except (RuntimeError, AttributeError):  # no pass running / no such engine hook
            return False
        return True

    def _queue_step(self, p, inplace=False):
        """Hook path: ``p``'s gradient is complete; step it with its group."""
        if inplace:
            self._pending_inplace.append(p)
        else:
            self._pending_steps.append(p)
        self._pending_step_bytes += p.numel() * 2
        if not self._flush_at_end_of_backward():
            self._flush_steps()  # called by hand: nothing to wait for
        elif (len(self._pending_steps) + len(self._pending_inplace) >= self._STEP_GROUP_PARAMS
                or self._pending_step_bytes >= self._STEP_GROUP_BYTES):
            self._flush_steps()

    def _queue_grad_writeback(self, p):
        """An accumulated gradient that stays on the GPU (``grad_cache_bytes``) goes
        back to the host with its group: one fence and one event for all of them."""
        self._pending_writebacks.append(p)
        self._pending_writeback_bytes += p.numel() * 2
        if (not self._flush_at_end_of_backward()
                or len(self._pending_writebacks) >= self._STEP_GROUP_PARAMS
                or self._pending_writeback_bytes >= self._STEP_GROUP_BYTES):
            self._flush_writebacks()

    def _flush_writebacks(self):
        params, self._pending_writebacks, self._pending_writeback_bytes = (
            self._pending_writebacks, [], 0)
        self._issue_d2h_many([(p, ["grad"]) for p in params])

    @torch.no_grad()
    def _flush_steps(self):
        """Step every queued parameter: fetch what is missing (one fence), one
        multi-tensor launch per param group, one fenced write-back."""
        if self._pending_norms:
            self._flush_norms()
        if self._pending_writebacks:
            self._flush_writebacks()
        offloaded, inplace = self._pending_steps, self._pending_inplace
        if not offloaded and not inplace:
            return
        self._pending_steps, self._pending_inplace, self._pending_step_bytes = [], [], 0
        if inplace:
            by_group = {}
            for p in inplace:
                by_group.setdefault(id(self._param2group[p]), []).append(p)
            for members in by_group.values():
                self._step_inplace_batch(members, self._param2group[members[0]])
        if not offloaded:
            return
        if _trace.ENABLED:
            with _trace.range(f"oa.steps x{len(offloaded)}"):
                self._step_offload_group(offloaded)
        else:
            self._step_offload_group(offloaded)

    def _step_offload_group(self, params):
        missing = []
        for p in params:
            dev = self.device_states[p]
            keys = [k for k in self.offload_state_keys if dev.get(k) is None]
            if keys:
                missing.append((p, keys))
        self._issue_h2d_many(missing)
        compute = self._compute_stream()
        waited = set()
        for p in params:
            events = [self.h2d_events.get(p)]
            if p in self._state_cached:
                # the kernel rewrites states whose last write-back may still be reading them
                events.append(self.d2h_events.get(p))
            for event in events:
                if event is not None and id(event) not in waited:
                    compute.wait_event(event)
                    waited.add(id(event))
        by_group = {}
        for p in params:
            state = self.state[p]
            state["step"] += 1
            group = self._param2group[p]
            dev = self.device_states[p]
            if (p in self._quant_params or p.dtype != _BF16 or not p.data.is_contiguous()
                    or not dev["grad"].is_contiguous() or dev["grad"].dtype != _BF16):
                # its own launch: a quantised weight is re-encoded there, and anything
                # the kernels cannot take is reported by the step function's checks
                self._call_step_fn(p, group, dev)
            else:
                by_group.setdefault(id(group), (group, [], [], []))
                _, ps, tensors, steps = by_group[id(group)]
                ps.append(p.data)
                tensors.append(dev)
                steps.append(state["step"])
        for group, ps, tensors, steps in by_group.values():
            beta1, beta2 = group["betas"]
            adam_step_multi(self.mode, ps, tensors, group["lr"], group["weight_decay"], beta1,
                            beta2, group["eps"], steps,
                            decoupled_weight_decay=self.decoupled_weight_decay, validate=False)
        self._issue_d2h_many([(p, self._non_grad_keys) for p in params])
        for p in params:
            self.device_states[p]["grad"] = None
            self.state[p]["host_grad_valid"] = False
        self._stale_host_grads.difference_update(params)

    def _record_grad_norm(self, p, grad, resident=False):
        """Clipping path, last micro-batch: ``p``'s gradient is complete; its norm is
        taken with its group's (two launches for up to 36 gradients instead of one
        or two per gradient).  The group closes at 36 gradients, at
        ``_NORM_GROUP_BYTES`` of gradients that would otherwise have left the GPU
        by then (the list keeps them alive; ``resident`` ones live there anyway),
        and when the backward pass ends - so ``state[p]['grad_norm']`` is current
        once ``backward()`` has returned, as in the reference."""
        if grad.dtype != _BF16:
            raise TypeError("gradient clipping works on bfloat16 gradients")
        self._pending_norms.append((grad.reshape(-1), self.state[p]["grad_norm"]))
        if not resident:
            self._pending_norm_bytes += grad.numel() * 2
        if (not self._flush_at_end_of_backward()
                or len(self._pending_norms) >= grad_clip.NORMS_PER_LAUNCH
                or self._pending_norm_bytes >= self._NORM_GROUP_BYTES):
            self._flush_norms()

    def _flush_norms(self):
        pending, self._pending_norms, self._pending_norm_bytes = self._pending_norms, [], 0
        if pending:
            grad_clip.grad_norms_([g for g, _ in pending], [slot for _, slot in pending],
                                  validate=False)

    # ------------------------------------------------------------------ hooks

    def _wanted_keys(self, p, states_too=False):
        """States of ``p`` this backward pass will need on the device and that are
        not there yet: the host gradient when one is pending, plus every other
        state when the step runs inside this pass."""
        dev = self.device_states[p]
        keys = []
        if self.state[p]["host_grad_valid"] and dev.get("grad") is None:
            keys.append("grad")
        if self._step_in_backward and (self.ready_for_optimizer_step or states_too):
            keys += [k for k in self._non_grad_keys if dev.get(k) is None]
        return keys

    def _prefetch_ahead(self, pos, states_too=False):
        """Issue the H2D of the parameters whose gradient hooks come next.

        The order in which gradient hooks fire is learned during the first
        backward pass and is stable afterwards.  Running the copies a window
        ahead of the hooks (at least ``_PREFETCH_MIN_PARAMS`` parameters,
        ``_PREFETCH_BYTES`` of device staging) lets them overlap with the
        backward kernels of earlier modules; without it a copy can only start
        when the compute stream reaches its own module (the fence against the
        compute stream is taken when a copy is issued) and the compute stream
        then waits for it.

        The window's far end only moves forward within a pass, so each call looks
        at the parameters that newly entered it (a call with ``pos == -1`` starts
        a pass and looks at the whole first window)."""
        order = self._bw_order
        if len(self._bw_prefix) != len(order) + 1:
            # bytes of device staging of order[:j], for the bisection below
            self._bw_prefix = [0]
            state_b = self._bytes_per_elem_in_flight - 2
            for q in order:
                per_elem = ((0 if q in self._state_cached else state_b)
                            + (0 if q in self._grad_cached or q in self._grad_on_device else 2))
                self._bw_prefix.append(self._bw_prefix[-1] + q.numel() * per_elem)
        prefix = self._bw_prefix
        first = pos + 1
        # parameters j >= first are wanted while the bytes of order[first:j] stay
        # below the budget, and in any case the next _PREFETCH_MIN_PARAMS
        end = bisect.bisect_left(prefix, prefix[first] + self._PREFETCH_BYTES, lo=first)
        end = min(len(order), max(end, first + self._PREFETCH_MIN_PARAMS))
        start = first if pos < 0 else max(first, self._bw_issued_upto)
        wanted = []
        for j in range(start, end):
            q = order[j]
            keys = self._wanted_keys(q, states_too)
            if keys:
                wanted.append((q, keys))
        self._issue_h2d_many(wanted)
        self._bw_issued_upto = max(end, 0 if pos < 0 else self._bw_issued_upto)

    @property
    def ready_for_optimizer_step(self):
        return self._ready_for_optimizer_step

    @ready_for_optimizer_step.setter
    def ready_for_optimizer_step(self, value):
        """Same flag as the reference's attribute.  Raising it before the forward
        pass of the last micro-batch also starts the first window of state
        copies, so they run under that forward pass instead of waiting for the
        first backward hook."""
        self._ready_for_optimizer_step = bool(value)
        if (getattr(self, "_pending_steps", None) or getattr(self, "_pending_inplace", None)
                or getattr(self, "_pending_writebacks", None)
                or getattr(self, "_pending_norms", None)):
            self._flush_steps()
        if not self._ready_for_optimizer_step or not hasattr(self, "_bw_order"):
            return
        if self._step_in_backward:
            if self._bw_order_known and self._bw_cursor < 0:
                with torch.no_grad():
                    self._prefetch_ahead(-1)
        else:
            with torch.no_grad():
                self._prestage_for_step()

    def _prestage_for_step(self):
        """Clip path: the states do not depend on the clip coefficient, so the
        first ``prefetch_bytes`` of them (in the order ``step()`` walks the
        parameters) cross the link under the last backward pass instead of
        inside ``step()``.  Not when this pass has to fetch accumulated gradients
        from the host (none of those kept on the GPU by ``grad_cache_bytes``
        count): the host->device direction is then busy for the whole pass
        and staged states would only queue ahead of the gradients backward waits
        for (measured: 2.86 s instead of 2.71 s per 8B step)."""
        if any(
            self.state[p]["host_grad_valid"] and self.device_states[p].get("grad") is None
            for p in self._offload_params
        ):
            return
        budget = self._prestage_bytes
        per_elem = self._bytes_per_elem_in_flight - 2  # all states but the gradient
        wanted = []
        for group in self.param_groups:
            for p in group["params"]:
                if budget <= 0:
                    break
                if p in self._inplace_params:
                    continue
                dev = self.device_states[p]
                missing = [k for k in self._non_grad_keys if dev.get(k) is None]
                if missing:
                    wanted.append((p, missing))
                budget -= p.numel() * per_elem
        self._issue_h2d_many(wanted)

    def _pre_backward_hook(self, module, grad_output):
        # Idempotent across the several fires a backward can produce for one
        # parameter (shared modules, tied weights): only what is not yet on the
        # device is requested.
        lazy = self._prefetch_policy == "lazy"
        wanted = []
        for p in self._module_params[module]:
            if p not in self.device_states:
                continue
            if lazy and self._prefetch_module.get(p) is not module:
                continue
            keys = self._wanted_keys(p)
            if keys:
                wanted.append((p, keys))
        self._issue_h2d_many(wanted)
        if self._bw_order_known and self._bw_cursor < 0:
            self._prefetch_ahead(-1)  # a new pass: start the window at the first hook

    @torch.no_grad()
    def _grad_hook(self, p):
        if p.grad is None:
            return
        pos = self._bw_pos.get(p)
        if pos is None:  # not seen before: learn the firing order
            pos = self._bw_pos[p] = len(self._bw_order)
            self._bw_order.append(p)
        else:
            self._bw_order_known = True  # a second pass has begun
        if _trace.ENABLED:
            with _trace.range(f"oa.hook #{pos} {tuple(p.shape)}"):
                self._grad_hook_body(p, pos)
        else:
            self._grad_hook_body(p, pos)

    def _grad_hook_body(self, p, pos):
        if self._bw_order_known:
            self._bw_cursor = -1 if pos == len(self._bw_order) - 1 else pos
            self._prefetch_ahead(pos)
        self._accumulate_grad_on_device(p)
        state = self.state[p]
        last = self.ready_for_optimizer_step
        if self.max_grad_norm is not None and last:
            self._record_grad_norm(p, self.device_states[p]["grad"])
        if self._step_in_backward and last:
            self._queue_step(p)
            if self._bw_order_known and pos == len(self._bw_order) - 1:
                self._flush_steps()
                # The step is complete.  The host->device direction is idle until
                # the next accumulation pass needs gradients back (never, with
                # offload_grads=False): stage the states the next step touches
                # first now, up to the prefetch budget.
                self._prefetch_ahead(-1, states_too=True)
        elif p not in self._grad_on_device:
            if p not in self._grad_cached:
                self._issue_d2h(p, ["grad"])
            elif self._grad_cache_write_back:
                self._stale_host_grads.add(p)
            else:
                self._queue_grad_writeback(p)

    @torch.no_grad()
    def _inplace_grad_hook(self, p):
        if p.grad is None:
            return
        state = self.state[p]
        state["grad"].add_(p.grad)
        p.grad = None
        last = self.ready_for_optimizer_step
        if self.max_grad_norm is not None and last:
            self._record_grad_norm(p, state["grad"], resident=True)
        if self._step_in_backward and last:
            self._queue_step(p, inplace=True)

    # ------------------------------------------------------------- public API

    @torch.no_grad()
    def step(self, closure=None):
        if closure is not None:
            raise NotImplementedError(
                "OffloadAdam does not support closure-based step: gradients are consumed by "
                "backward hooks, so re-running backward inside a closure would corrupt "
                "optimizer state."
            )
        self._bw_cursor = -1  # the next backward pass starts a new prefetch window
        self._flush_steps()  # normally empty: the end of backward has flushed
        if self._step_in_backward:
            return

        # A parameter whose gradient sum lives on the GPU only (offload_grads=False, or
        # displaced by the pinned-memory limit) and that received no gradient in this
        # window has nothing to be stepped with: it sits the step out, as on the hook
        # path, and its norm does not count.  (With a host gradient buffer the reference
        # steps such a parameter again with the buffer's old contents,
        # src/offload_adam/offload_adam.py:446-454; that is kept where the buffer exists.)
        idle = {p for p in self._grad_on_device if self.device_states[p].get("grad") is None}
        clip_coef = None
        if self.max_grad_norm is not None:
            for p in idle:
                self.state[p]["grad_norm"].zero_()
            grad_clip.clip_coef_(self._norm_slots, float(self.max_grad_norm), self._clip_coef,
                                 self._total_norm)
            clip_coef = self._clip_coef

        order = [(g, p) for g in self.param_groups for p in g["params"] if p not in idle]
        offloaded = [p for _, p in order if p not in self._inplace_params]
        ahead = 0  # offloaded params whose H2D has been issued
        done = 0
        # GPU-resident small parameters: one multi-tensor launch per group
        for group in self.param_groups:
            small = [p for p in group["params"] if p in self._inplace_params]
            if small:
                self._step_inplace_batch(small, group, clip_coef)
        for group, p in order:
            if p in self._inplace_params:
                continue
            state = self.state[p]
            state["step"] += 1
            # keep the H2D engine a few parameters ahead of the kernels
            while ahead < min(done + 1 + self._CLIP_PREFETCH_DEPTH, len(offloaded)):
                q = offloaded[ahead]
                dev = self.device_states[q]
                missing = [k for k in self.offload_state_keys if dev.get(k) is None]
                if missing:
                    self._issue_h2d(q, missing)
                ahead += 1
            with _trace.range(f"oa.step #{done} {tuple(p.shape)}"):
                self._step_offload(p, group, clip_coef)
            state["host_grad_valid"] = False
            done += 1

    def zero_grad(self, set_to_none=False):
        """No-op: gradients are consumed by the hooks."""
        return

    def state_dict(self):
        """``Optimizer.state_dict()``; parameters still waiting for their group's
        launch are stepped first, and host gradients that the ``'write_back'``
        gradient cache has let fall behind are brought up to date."""
        self._flush_steps()
        self._refresh_host_grads()
        return super().state_dict()

    def _refresh_host_grads(self):
        stale = [p for p in self._stale_host_grads
                 if self.device_states[p].get("grad") is not None]
        self._stale_host_grads.clear()
        if stale:
            self._issue_d2h_many([(p, ["grad"]) for p in stale])
            self.d2h_events[stale[0]].synchronize()

    @torch.no_grad()
    def load_master_state_dict(self, state_dict, model, strict=False):
        """Overwrite ``master_params`` from a ``{param_name: tensor}`` mapping (any
        float dtype).  Returns ``(unexpected_keys,)``; ``strict=True`` raises
        ``ValueError`` for names that match no parameter of this optimizer."""
        if "master_params" not in self.offload_config:
            raise RuntimeError(
                "load_master_state_dict requires a mode that maintains master_params "
                f"(e.g. 'fp32_master'); current mode is {self.mode!r}."
            )
        by_name = {n: p for n, p in model.named_parameters() if p.requires_grad}
        unexpected = []
        for name, tensor in state_dict.items():
            p = by_name.get(name)
            if p is None or p not in self.state:
                unexpected.append(name)
                continue
            self._copy_master(p, tensor)
            if "master_filled" in self.state[p]:
                self.state[p]["master_filled"] = True
        if strict and unexpected:
            raise ValueError(
                f"load_master_state_dict(strict=True): no param matches {len(unexpected)} "
                f"key(s): {unexpected}"
            )
        return (unexpected,)

    @torch.no_grad()
    def load_master_from_pretrained(self, pretrained_name_or_path, model, *, strict=False):
        """Refill the fp32 masters of quantised parameters from the bf16/fp16
        checkpoint they were quantised from.  Returns the sorted names of
        quantised parameters the checkpoint lacks."""
        if "master_params" not in self.offload_config:
            raise RuntimeError(
                "load_master_from_pretrained requires a mode that maintains master_params "
                f"(e.g. 'fp32_master'); current mode is {self.mode!r}."
            )
        return stream_master_from_pretrained(self, pretrained_name_or_path, model, strict=strict)

    def load_state_dict(self, state_dict):
        raise NotImplementedError(
            "OffloadAdam.load_state_dict is not supported: the default "
            "Optimizer.load_state_dict would move pinned-host state to GPU and cast fp32 "
            "master to bf16, defeating the offload contract. Use load_offloaded_state_dict "
            "to resume."
        )

    @torch.no_grad()
    def load_offloaded_state_dict(self, state_dict):
        """Resume from ``state_dict()`` of an ``OffloadAdam`` over the same
        parameters (same order, shapes, mode and clipping setting).

        The reference has no resume path (``load_state_dict`` raises there as it
        does here, src/offload_adam/offload_adam.py:672-678).  This copies the saved
        values *into this optimizer's own buffers*: offloaded states stay in their
        pinned host allocations in their own dtypes (fp32 masters stay fp32), the
        states of the small GPU-resident parameters stay on the GPU, and nothing is
        re-allocated.  ``lr``, ``betas``, ``eps`` and ``weight_decay`` are taken
        from the saved param group.  Model weights are not part of it: load the
        model's own ``state_dict`` first.

        Call it at a step boundary.  Partial gradient sums of an unfinished
        accumulation window travel with the state (``grad`` / ``host_grad_valid``)
        unless the optimizer was built with ``offload_grads=False``, whose running
        sums never reach the state dict.
        """
        self._flush_steps()
        saved_groups = state_dict["param_groups"]
        saved_state = state_dict["state"]
        if len(saved_groups) != len(self.param_groups):
            raise ValueError(
                f"saved state has {len(saved_groups)} param groups, this optimizer "
                f"{len(self.param_groups)}")
        pairs = []
        for group, saved in zip(self.param_groups, saved_groups):
            if len(saved["params"]) != len(group["params"]):
                raise ValueError("a saved param group has a different number of parameters")
            pairs.extend(zip(saved["params"], group["params"]))
        # validate everything before the first byte moves
        for key, p in pairs:
            if key not in saved_state:
                raise ValueError(f"saved state has no entry for parameter {key}")
            mine, theirs = self.state[p], saved_state[key]
            if set(mine) != set(theirs):
                raise ValueError(
                    f"parameter {key}: saved keys {sorted(theirs)} do not match this "
                    f"optimizer's {sorted(mine)} (different mode, clipping or threshold?)")
            for name, value in mine.items():
                other = theirs[name]
                if isinstance(value, torch.Tensor) != isinstance(other, torch.Tensor):
                    raise ValueError(f"parameter {key}: '{name}' changes kind")
                if isinstance(value, torch.Tensor) and (
                        value.shape != other.shape or value.dtype != other.dtype):
                    raise ValueError(
                        f"parameter {key}: '{name}' is {tuple(other.shape)} {other.dtype} in the "
                        f"saved state, {tuple(value.shape)} {value.dtype} here")
        # nothing may be in flight or staged while the buffers are rewritten
        torch.cuda.synchronize()
        for dev in self.device_states.values():
            for name in dev:
                dev[name] = None
        self.h2d_events.clear()
        self.d2h_events.clear()
        self._writebacks_pending.clear()  # (after the synchronisation above)
        self._writeback_pending_bytes = 0
        self._stale_host_grads.clear()
        self._bw_cursor = -1
        self._bw_issued_upto = 0
        for key, p in pairs:
            mine, theirs = self.state[p], saved_state[key]
            for name, value in mine.items():
                if isinstance(value, torch.Tensor):
                    value.copy_(theirs[name])
                else:
                    mine[name] = theirs[name]
        for group, saved in zip(self.param_groups, saved_groups):
            for name, value in saved.items():
                if name != "params":
                    group[name] = value
        torch.cuda.synchronize()
