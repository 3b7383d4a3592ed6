"""Swap ``nn.Linear`` weights for quantised-weight subclass instances and keep
``state_dict`` / ``load_state_dict`` working with plain tensors.

Host-side model surgery (no kernels of its own): the counterpart of the
reference's ``quantize_linears`` / ``save_quantized_pretrained``
(src/offload_adam/qweight/apply.py).
"""

import json
from pathlib import Path
from typing import List, NamedTuple, Optional, Tuple, Type, Union

import torch
import torch.nn as nn

from .base import QWeightBase


class QuantizeReport(NamedTuple):
    """Module names (as in ``model.named_modules()``) by outcome of a
    ``quantize_linears`` pass: replaced, rejected by ``can_quantize`` (with the
    reason), and skipped because a ``skip_patterns`` entry matched."""

    quantized: List[str]
    incompatible: List[Tuple[str, str]]
    excluded: List[str]


class _PlainTensorHooks:
    """state_dict hooks of one quantised Linear: save expands the subclass into
    its canonical plain tensors, load folds them back into a subclass instance
    (or lets a plain float ``weight`` re-quantise through ``copy_``)."""

    def __init__(self, module: nn.Module, weight_cls: Type[QWeightBase]):
        self.module = module
        self.weight_cls = weight_cls

    def on_save(self, mod, destination, prefix, local_metadata):
        w = destination.get(prefix + "weight")
        if isinstance(w, self.weight_cls):
            del destination[prefix + "weight"]
            for suffix, tensor in w.to_plain_state_dict().items():
                destination[prefix + suffix] = tensor

    def on_load(self, state_dict, prefix, local_metadata, strict, missing_keys,
                unexpected_keys, error_msgs):
        suffixes = self.weight_cls.canonical_key_suffixes()
        found = {s: state_dict.pop(prefix + s) for s in suffixes if prefix + s in state_dict}
        # a float "weight" is an ordinary checkpoint: put it back, copy_ re-quantises
        if "weight" in found and found["weight"].dtype is not torch.uint8:
            state_dict[prefix + "weight"] = found.pop("weight")
        if not found:
            return
        if len(found) != len(suffixes):
            missing_keys.extend(prefix + s for s in suffixes if s not in found)
            return
        current = self.module.weight.data
        reference = current if isinstance(current, self.weight_cls) else None
        state_dict[prefix + "weight"] = self.weight_cls.from_plain_state_dict(
            found, reference=reference
        )


def _attach_hooks(module: nn.Module, weight_cls: Type[QWeightBase]) -> None:
    hooks = _PlainTensorHooks(module, weight_cls)
    module._register_state_dict_hook(hooks.on_save)
    module._register_load_state_dict_pre_hook(hooks.on_load)


@torch.no_grad()
def quantize_linears(
    model: nn.Module,
    weight_cls: Type[QWeightBase],
    skip_patterns: Tuple[str, ...] = (),
    device: Optional[str] = None,
    strict: bool = False,
    update_hf_config: bool = False,
    **weight_kwargs,
) -> QuantizeReport:
    """Replace the weight of every eligible ``nn.Linear`` in place.

    ``skip_patterns`` are substrings of module names to leave alone (e.g.
    ``("lm_head",)``); ``device`` moves each weight there before encoding (the
    GPU path uses the HIP codec kernels); ``strict`` raises ``ValueError`` when
    ``weight_cls.can_quantize`` rejects a layer; ``update_hf_config`` writes the
    matching ``quantization_config`` into ``model.config``; ``weight_kwargs`` go
    to ``from_float`` / ``can_quantize`` (e.g. ``group_size=128``).
    """
    report = QuantizeReport([], [], [])
    for name, module in model.named_modules():
        if not isinstance(module, nn.Linear):
            continue
        if any(pattern in name for pattern in skip_patterns):
            report.excluded.append(name)
            continue
        w = module.weight
        if not weight_cls.can_quantize(w, **weight_kwargs):
            report.incompatible.append((name, f"shape={tuple(w.shape)} dtype={w.dtype}"))
            continue
        source = w.data if device is None else w.data.to(device)
        module.weight = nn.Parameter(
            weight_cls.from_float(source, **weight_kwargs), requires_grad=w.requires_grad
        )
        _attach_hooks(module, weight_cls)
        report.quantized.append(name)
    if strict and report.incompatible:
        detail = "; ".join(f"{n} ({why})" for n, why in report.incompatible)
        raise ValueError(
            f"quantize_linears(strict=True) rejected {len(report.incompatible)} layer(s): {detail}"
        )
    if update_hf_config and hasattr(model, "config"):
        model.config.quantization_config = weight_cls.build_hf_quantization_config(
            skip_patterns=skip_patterns, **weight_kwargs
        )
    return report


def save_quantized_pretrained(
    model: nn.Module,
    save_directory: Union[str, Path],
    weight_cls: Type[QWeightBase],
    skip_patterns: Tuple[str, ...] = (),
    **weight_kwargs,
) -> None:
    """``model.save_pretrained(save_directory)`` followed by merging the
    format's ``quantization_config`` into the written ``config.json``."""
    out_dir = Path(save_directory)
    model.save_pretrained(out_dir)
    config_file = out_dir / "config.json"
    config = json.loads(config_file.read_text())
    config["quantization_config"] = weight_cls.build_hf_quantization_config(
        skip_patterns=skip_patterns, **weight_kwargs
    )
    config_file.write_text(json.dumps(config, indent=2))
