"""Base class of the quantised-weight tensor subclasses used for QAT.

A quantised weight looks like a plain ``(out_features, in_features)`` float
tensor from the outside (so ``nn.Linear`` and the optimizers need no special
cases) and keeps packed payload tensors inside.  The handful of operations a
training loop performs on a weight are routed here:

* ``F.linear(x, w)``      -> dequantise (HIP kernel) then matmul, with autograd;
* ``w.copy_(fp32_master)`` -> re-quantise into the existing payload (HIP kernel);
* ``plain.copy_(w)``       -> dequantise;
* ``detach`` / ``clone`` / ``to`` / ``zeros_like`` -> payload-wise.

Mirrors the role of the reference's ``QWeightBase``
(src/offload_adam/qweight/base.py:13-124): per-subclass tables of ATen-op and
torch-function handlers filled through ``implements`` decorators.  The handlers
every format shares are registered once, for each subclass, from
``__init_subclass__``; a format only supplies its payload names, its quantise /
dequantise routines and how a dtype change maps onto its payload.
"""

import torch
from torch import Tensor
from torch.utils._python_dispatch import return_and_correct_aliasing

aten = torch.ops.aten


_CACHE_DEQUANTIZED = False


def cache_dequantized_weights(enabled=True):
    """Let the linear layers keep the dequantised copy of each quantised weight
    until its payload changes, instead of decoding it again in every forward,
    every checkpoint re-computation and every backward of every micro-batch
    (12 decodes per weight per step with 4 checkpointed micro-batches, against 1).
    Costs one plain copy of every quantised weight in device memory, which is what
    quantisation saved, so it is off unless asked for; results do not change.
    Returns the previous setting."""
    global _CACHE_DEQUANTIZED
    previous, _CACHE_DEQUANTIZED = _CACHE_DEQUANTIZED, bool(enabled)
    return previous


def _dequantized(weight, dtype):
    if not _CACHE_DEQUANTIZED:
        return weight.dequantize(dtype=dtype)
    # every in-place change of a payload tensor moves its version counter: torch
    # ops by themselves, this package's kernels through _codec_ops.mark_written
    key = (dtype,) + tuple(getattr(weight, n)._version for n in weight._PAYLOAD)
    hit = weight.__dict__.get("_dequantized_cache")
    if hit is not None and hit[0] == key:
        return hit[1]
    w = weight.dequantize(dtype=dtype)
    weight.__dict__["_dequantized_cache"] = (key, w)
    return w


class _WeightOnlyLinear(torch.autograd.Function):
    """y = x @ dequant(w).T (+ b); backward dequantises again and returns a
    plain gradient for the weight (reference: qweight/int8.py:378-397)."""

    @staticmethod
    def forward(ctx, x, weight, bias=None):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        w = _dequantized(weight, x.dtype)
        out = x @ w.T
        return out if bias is None else out + bias

    @staticmethod
    def backward(ctx, grad_output):
        x, weight = ctx.saved_tensors
        w = _dequantized(weight, grad_output.dtype)
        grad_x = grad_output @ w
        go = grad_output.reshape(-1, weight.shape[0])
        grad_w = go.T @ x.reshape(-1, weight.shape[1])
        grad_b = go.sum(0) if ctx.has_bias else None
        return grad_x, grad_w, grad_b


class QWeightBase(Tensor):
    """Wrapper-subclass base.  Subclasses define:

    * ``_PAYLOAD``: names of the payload tensor attributes, in constructor order;
    * ``_meta()``: the non-tensor constructor arguments that follow them;
    * ``_requantize_(src)``: encode a plain float tensor into the payload, in place;
    * ``dequantize(dtype=None)``;
    * ``_payload_to(name, tensor, device, dtype)`` / ``_meta_to(dtype)``: effect
      of ``.to(device, dtype)`` on one payload tensor / on the meta arguments.
    """

    _PAYLOAD: tuple = ()
    _ATEN_OP_TABLE: dict
    _TORCH_FN_TABLE: dict

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        cls._ATEN_OP_TABLE = {}
        cls._TORCH_FN_TABLE = {}
        _register_shared_handlers(cls)

    # ---- registration decorators (same names as the reference's) ----------

    @classmethod
    def implements(cls, aten_ops):
        ops = aten_ops if isinstance(aten_ops, (list, tuple)) else [aten_ops]

        def decorator(fn):
            for op in ops:
                cls._ATEN_OP_TABLE[op] = fn
            return fn

        return decorator

    @classmethod
    def implements_torch_function(cls, torch_fns):
        fns = torch_fns if isinstance(torch_fns, (list, tuple)) else [torch_fns]

        def decorator(fn):
            for f in fns:
                cls._TORCH_FN_TABLE[f] = fn
            return fn

        return decorator

    # ---- dispatch -------------------------------------------------------

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs):
        handler = cls._ATEN_OP_TABLE.get(func)
        if handler is None:
            raise NotImplementedError(
                f"{cls.__name__} does not support {func}. "
                f"Register a handler via @{cls.__name__}.implements(...)."
            )
        return handler(func, types, args, kwargs)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        handler = cls._TORCH_FN_TABLE.get(func)
        if handler is not None:
            return handler(func, types, args, kwargs)
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)

    # ---- flatten protocol (payload names + meta) ------------------------------

    def __tensor_flatten__(self):
        return list(self._PAYLOAD), list(self._meta())

    @classmethod
    def __tensor_unflatten__(cls, tensors, attrs, outer_size=None, outer_stride=None):
        return cls(*[tensors[n] for n in cls._PAYLOAD], *attrs)

    # ---- per-format hooks -------------------------------------------------

    def _meta(self) -> tuple:
        return ()

    def _meta_to(self, dtype) -> tuple:
        return self._meta()

    def _payload_to(self, name, tensor, device, dtype):
        return tensor.to(device=device)

    def _requantize_(self, src: Tensor) -> None:
        raise NotImplementedError

    def dequantize(self, dtype=None) -> Tensor:
        """Plain tensor reconstruction at the requested dtype."""
        raise NotImplementedError

    # ---- advisory / serialisation surface (same names as the reference) ---

    @classmethod
    def can_quantize(cls, tensor: Tensor, **kwargs) -> bool:
        """False when this format cannot hold ``tensor`` (shape constraints)."""
        return True

    @classmethod
    def canonical_key_suffixes(cls) -> tuple:
        raise NotImplementedError

    def to_plain_state_dict(self) -> dict:
        raise NotImplementedError

    @classmethod
    def from_plain_state_dict(cls, plain: dict, reference=None) -> "QWeightBase":
        raise NotImplementedError

    @classmethod
    def build_hf_quantization_config(cls, skip_patterns=(), **weight_kwargs) -> dict:
        raise NotImplementedError

    def __repr__(self):
        extra = "".join(f", {k}={v}" for k, v in self._repr_extra().items())
        return (
            f"{type(self).__name__}(shape={tuple(self.shape)}, dtype={self.dtype}, "
            f"device={self.device}{extra}, requires_grad={self.requires_grad})"
        )

    def _repr_extra(self) -> dict:
        return {}


def _register_shared_handlers(cls):
    """Handlers that are identical for every format."""

    @cls.implements_torch_function(torch.nn.functional.linear)
    def _linear(func, types, args, kwargs):
        return _WeightOnlyLinear.apply(*args, **kwargs)

    @cls.implements([aten.detach.default, aten.clone.default])
    def _detach_clone(func, types, args, kwargs):
        src = args[0]
        out = cls(*[func(getattr(src, n), *args[1:], **kwargs) for n in cls._PAYLOAD], *src._meta())
        return return_and_correct_aliasing(func, args, kwargs, out)

    @cls.implements(aten._to_copy.default)
    def _to_copy(func, types, args, kwargs):
        src = args[0]
        device, dtype = kwargs.get("device", None), kwargs.get("dtype", None)
        out = cls(
            *[src._payload_to(n, getattr(src, n), device, dtype) for n in cls._PAYLOAD],
            *src._meta_to(dtype),
        )
        return return_and_correct_aliasing(func, args, kwargs, out)

    @cls.implements(aten.copy_.default)
    def _copy_(func, types, args, kwargs):
        dst, src = args[0], args[1]
        if isinstance(dst, cls) and isinstance(src, cls):
            for n in cls._PAYLOAD:
                getattr(dst, n).copy_(getattr(src, n))
        elif isinstance(dst, cls):
            dst._requantize_(src)  # the optimizer's `p.data.copy_(fp32_master)`
        else:
            dst.copy_(src.dequantize())
            return dst
        # in-place ops issued from inside a dispatch handler do not move the payload's
        # version counters; the dequantisation cache is keyed on them
        for n in cls._PAYLOAD:
            torch.autograd.graph.increment_version(getattr(dst, n))
        return dst

    @cls.implements(aten.zeros_like.default)
    def _zeros_like(func, types, args, kwargs):
        ref = args[0]
        return torch.zeros(
            ref.shape,
            dtype=kwargs.get("dtype", None) or ref.dtype,
            device=kwargs.get("device", None) or ref.device,
        )
