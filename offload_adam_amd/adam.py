"""``Adam``: the non-offload optimizer over the same fused HIP step kernels.

Drop-in for the reference's ``offload_adam.Adam``
(src/offload_adam/adam.py:16-302): same constructor, mode strings, lazily
created per-parameter state (``step``, ``exp_avg``, ``exp_avg_sq`` plus
``master_params`` or ``rounding_error`` by mode, ``master_filled`` for
quantised parameters), QAT re-quantisation after the step, and a
``load_state_dict`` that keeps fp32 masters in fp32.
"""

import warnings

import torch
from torch.optim.optimizer import Optimizer

from ._pretrained import stream_master_from_pretrained
from .kernels import (
    adam_step_fp31_master,
    adam_step_fp32_master,
    adam_step_fp32_master_custom_rounding,
    adam_step_multi,
    adam_step_stochastic_rounding,
)
from .qweight.base import QWeightBase

_BF16 = torch.bfloat16

# mode -> step function and the dtype of every persistent state tensor
MODE_TABLE = {
    "stochastic_rounding": (adam_step_stochastic_rounding, {}),
    "fp32_master": (adam_step_fp32_master, {"master_params": torch.float32}),
    "fp31_master": (adam_step_fp31_master, {"rounding_error": torch.int16}),
    "fp32_master_custom_rounding": (
        adam_step_fp32_master_custom_rounding,
        {"rounding_error": torch.int16},
    ),
}

_LOSSY_MASTER_HINT = (
    "quantized params running with a lossy dequant-seeded fp32 master. For higher "
    "precision, call `optim.load_master_from_pretrained(pretrained_name_or_path, model)` "
    "with the same bf16/fp16 checkpoint `from_pretrained` used before `quantize_linears` ran."
)


def _moment_states(extra):
    return {"exp_avg": _BF16, "exp_avg_sq": _BF16, **extra}


def _batchable(p, grad):
    """Eligible for the multi-tensor launch; anything else takes the
    single-tensor call, which reports what is wrong with it."""
    return (
        p.is_cuda and p.dtype == _BF16 and grad.dtype == _BF16
        and p.is_contiguous() and grad.is_contiguous() and grad.device == p.device
    )


class Adam(Optimizer):
    configs = {
        mode: {"step": fn, "states": _moment_states(extra)}
        for mode, (fn, extra) in MODE_TABLE.items()
    }

    def __init__(
        self,
        params,
        lr=1e-3,
        betas=(0.9, 0.999),
        eps=1e-8,
        weight_decay=0.01,
        mode="stochastic_rounding",
        decoupled_weight_decay=False,
    ):
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        assert mode in self.configs, f"Invalid mode: {mode}"
        self.mode = mode
        self.config = self.configs[mode]
        self.step_fn = self.config["step"]
        self.decoupled_weight_decay = decoupled_weight_decay
        # one launch per 36 parameters instead of one per parameter (same results)
        self.multi_tensor = True

        n_quant = sum(
            isinstance(p.data, QWeightBase) for g in self.param_groups for p in g["params"]
        )
        if n_quant and mode != "fp32_master":
            raise ValueError(
                f"Adam found {n_quant} quantized param(s) but mode={mode!r}; "
                f"QAT requires mode='fp32_master'."
            )
        # one-shot flag, not persisted; True when there is nothing to warn about
        self._quant_master_warned = n_quant == 0

    # ------------------------------------------------------------------ state

    def _init_state_if_empty(self, p, state):
        if state:
            return
        state["step"] = 0
        for name, dtype in self.config["states"].items():
            state[name] = torch.zeros_like(p, dtype=dtype)
        if "master_params" in state:
            # plain bf16/fp16 widens losslessly; a quantised weight dequantises
            # (lossy seed, flagged so load_master_from_pretrained can fix it)
            state["master_params"].copy_(p.data)
            if isinstance(p.data, QWeightBase):
                state["master_filled"] = False

    # ------------------------------------------------------------------- step

    @torch.no_grad()
    def step(self, closure=None):
        if not self._quant_master_warned:
            self._maybe_warn_lossy_master()

        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            batch_p, batch_st, batch_steps = [], [], []
            for p in group["params"]:
                grad = p.grad
                if grad is None:
                    continue
                if grad.is_sparse:
                    raise RuntimeError("Sparse gradient is not supported")
                state = self.state[p]
                self._init_state_if_empty(p, state)
                state["step"] += 1

                quant = isinstance(p.data, QWeightBase)
                tensors = {name: state[name] for name in self.config["states"]}
                tensors["grad"] = grad
                if self.multi_tensor and not quant and _batchable(p, grad):
                    # plain parameters of the group go to the GPU in one call
                    batch_p.append(p.data)
                    batch_st.append(tensors)
                    batch_steps.append(state["step"])
                    continue
                # The kernel writes a bf16 copy of the master through its first
                # argument.  Given a quantised weight the fp32_master step
                # function re-encodes the payload from the new master in the same
                # pass; any other step function gets the grad buffer as a sink of
                # matching shape and the payload is re-encoded below.
                fused = quant and self.mode == "fp32_master"
                self.step_fn(
                    grad if quant and not fused else p.data,
                    tensors,
                    group["lr"],
                    group["weight_decay"],
                    beta1,
                    beta2,
                    group["eps"],
                    state["step"],
                    decoupled_weight_decay=self.decoupled_weight_decay,
                )
                if quant:
                    if not fused:
                        p.data.copy_(state["master_params"])
                    p.grad = None  # as the reference leaves it (there it held the sink)
            if batch_p:
                adam_step_multi(
                    self.mode,
                    batch_p,
                    batch_st,
                    group["lr"],
                    group["weight_decay"],
                    beta1,
                    beta2,
                    group["eps"],
                    batch_steps,
                    decoupled_weight_decay=self.decoupled_weight_decay,
                )
        return loss

    def _maybe_warn_lossy_master(self):
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None or not isinstance(p.data, QWeightBase):
                    continue
                if self.state.get(p, {}).get("master_filled") is True:
                    continue
                warnings.warn("Adam: " + _LOSSY_MASTER_HINT, stacklevel=3)
                self._quant_master_warned = True
                return

    # ----------------------------------------------------------- master loads

    def _copy_master(self, p, tensor):
        self.state[p]["master_params"].copy_(tensor)

    @torch.no_grad()
    def load_master_state_dict(self, state_dict, model, strict=False):
        """Overwrite ``master_params`` from a ``{param_name: tensor}`` mapping
        (any float dtype; widening to fp32 is lossless).  Returns
        ``(unexpected_keys,)``; ``strict=True`` raises ``ValueError`` on names
        that match no trainable parameter."""
        if "master_params" not in self.config["states"]:
            raise RuntimeError(
                f"load_master_state_dict requires mode='fp32_master'; current mode is {self.mode!r}."
            )
        by_name = {n: p for n, p in model.named_parameters() if p.requires_grad}
        unexpected = []
        for name, tensor in state_dict.items():
            p = by_name.get(name)
            if p is None:
                unexpected.append(name)
                continue
            state = self.state[p]
            self._init_state_if_empty(p, state)
            self._copy_master(p, tensor)
            if "master_filled" in state:
                state["master_filled"] = True
        if strict and unexpected:
            raise ValueError(
                f"load_master_state_dict(strict=True): no param matches {len(unexpected)} "
                f"key(s): {unexpected}"
            )
        return (unexpected,)

    @torch.no_grad()
    def load_master_from_pretrained(self, pretrained_name_or_path, model, *, strict=False):
        """Refill the fp32 masters of quantised parameters from the bf16/fp16
        checkpoint they were quantised from (file, sharded directory or Hub id).
        Returns the sorted names of quantised parameters the checkpoint lacks."""
        if "master_params" not in self.config["states"]:
            raise RuntimeError(
                "load_master_from_pretrained requires mode='fp32_master'; "
                f"current mode is {self.mode!r}."
            )
        return stream_master_from_pretrained(self, pretrained_name_or_path, model, strict=strict)

    @torch.no_grad()
    def load_state_dict(self, state_dict):
        """``Optimizer.load_state_dict`` casts floating state to the parameter's
        dtype, which would demote the fp32 master of a bf16 model; the fp32
        tensors are set aside first and put back afterwards."""
        keep = {}
        for idx, entry in state_dict.get("state", {}).items():
            if isinstance(entry, dict):
                t = entry.get("master_params")
                if isinstance(t, torch.Tensor) and t.dtype == torch.float32:
                    keep[idx] = t.detach()
        super().load_state_dict(state_dict)
        if not keep:
            return
        flat = [p for g in self.param_groups for p in g["params"]]
        for idx, master in keep.items():
            p = flat[idx]
            st = self.state.get(p)
            if st is not None and "master_params" in st:
                st["master_params"] = master.to(device=p.device)
