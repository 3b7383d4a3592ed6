"""Int8 per-output-channel symmetric QAT weight (compressed-tensors W8A16).

Payload:
  weight : (out_f, in_f) int8, row-major
  scales : (out_f,) in the weight's float dtype; scale = row absmax / 127

Same storage and public names as the reference module
(src/offload_adam/qweight/int8.py).  GPU tensors are encoded and decoded by
the HIP kernels of the library; CPU tensors (model surgery before the move to
the GPU) use the equivalent torch arithmetic.
"""

from typing import Tuple

import torch
from torch import Tensor

from . import _codec_ops
from .base import QWeightBase


@torch.no_grad()
def quantize_int8_per_channel(tensor: Tensor, eps: float = 1e-12) -> Tuple[Tensor, Tensor]:
    """(out_f, in_f) float -> (int8 codes in [-128, 127], per-row scales in the
    input dtype).  The codes use the fp32 scale; ties round to even."""
    assert tensor.ndim == 2
    if tensor.is_cuda and eps == 1e-12:
        return _quantize_int8_hip(tensor, tensor.dtype)
    x = tensor.float()
    scale = x.abs().amax(dim=1) / 127.0
    recip = 1.0 / scale.clamp(min=eps)
    codes = (x * recip[:, None]).round().clamp(-128, 127).to(torch.int8)
    return codes, scale.to(tensor.dtype)


def dequantize_int8_per_channel(weight: Tensor, scales: Tensor) -> Tensor:
    """codes * scale, computed in the dtype of ``scales``."""
    if weight.is_cuda:
        return _dequant_int8_hip(weight, scales)
    return weight.to(scales.dtype) * scales[:, None]


def _quantize_int8_hip(tensor: Tensor, scale_dtype: torch.dtype) -> Tuple[Tensor, Tensor]:
    """Fused row-absmax + encode on the GPU.  Returns (weight, scales)."""
    out_f, in_f = tensor.shape
    weight = torch.empty((out_f, in_f), dtype=torch.int8, device=tensor.device)
    scales = torch.empty((out_f,), dtype=scale_dtype, device=tensor.device)
    _codec_ops.quantize_int8_into(tensor, weight, scales)
    return weight, scales


def _dequant_int8_hip(weight: Tensor, scales: Tensor) -> Tensor:
    return _codec_ops.dequantize_int8(weight.contiguous(), scales.contiguous())


class Int8QWeight(QWeightBase):
    """Outer shape (out_f, in_f) at ``scales.dtype``; ``copy_`` from a plain
    tensor re-quantises in place."""

    _PAYLOAD = ("weight", "scales")

    @staticmethod
    @torch._dynamo.disable
    def __new__(cls, weight: Tensor, scales: Tensor):
        return Tensor._make_wrapper_subclass(
            cls, tuple(weight.shape), dtype=scales.dtype, device=weight.device
        )

    @torch._dynamo.disable
    def __init__(self, weight: Tensor, scales: Tensor):
        assert weight.dtype is torch.int8 and weight.ndim == 2
        assert scales.ndim == 1 and scales.shape[0] == weight.shape[0]
        self.weight = weight
        self.scales = scales

    def _payload_to(self, name, tensor, device, dtype):
        if name == "scales":
            return tensor.to(device=device, dtype=dtype)
        return tensor.to(device=device)

    @classmethod
    def from_float(cls, tensor: Tensor, scale_dtype: torch.dtype = torch.bfloat16, **_):
        """``scale_dtype`` is both the stored scale dtype and the outer dtype."""
        weight, scales = quantize_int8_per_channel(tensor.detach())
        out = cls(weight, scales.to(scale_dtype))
        out.requires_grad_(tensor.requires_grad)
        return out

    @classmethod
    def can_quantize(cls, tensor: Tensor, **_) -> bool:
        # in_f % 4 == 0: four codes per int32 in the serialised form
        return tensor.dim() == 2 and tensor.shape[1] % 4 == 0

    def _requantize_(self, src: Tensor) -> None:
        if self.weight.is_cuda:
            src = src.detach().to(self.weight.device, non_blocking=True)
            _codec_ops.quantize_int8_into(src, self.weight, self.scales)
        else:
            codes, scales = quantize_int8_per_channel(src.detach().to(self.weight.device))
            self.weight.copy_(codes)
            self.scales.copy_(scales)

    def dequantize(self, dtype=None) -> Tensor:
        if dtype is None or dtype == self.scales.dtype:
            return dequantize_int8_per_channel(self.weight, self.scales)
        if self.weight.is_cuda and dtype == torch.float32:
            return _codec_ops.dequantize_int8(self.weight, self.scales, torch.float32)
        compute = torch.float32 if dtype == torch.float32 else self.scales.dtype
        return (self.weight.to(compute) * self.scales.to(compute)[:, None]).to(dtype)

    # ---- serialisation: compressed-tensors pack-quantized (plain torch) -------

    @classmethod
    def canonical_key_suffixes(cls) -> Tuple[str, ...]:
        return ("weight_packed", "weight_scale", "weight_shape")

    def to_plain_state_dict(self) -> dict:
        out_f, in_f = self.weight.shape
        assert in_f % 4 == 0, f"in_features={in_f} must be a multiple of 4 to pack int8 into int32"
        # int8 -> offset-binary bytes (zero point 128), four per int32, LSB first
        u = ((self.weight.to(torch.int32) + 128) & 0xFF).reshape(out_f, in_f // 4, 4)
        packed = torch.zeros(out_f, in_f // 4, dtype=torch.int32, device=u.device)
        for i in range(4):
            packed |= u[..., i] << (8 * i)
        return {
            "weight_packed": packed,
            "weight_scale": self.scales.unsqueeze(1),
            "weight_shape": torch.tensor([out_f, in_f], dtype=torch.int64, device=u.device),
        }

    @classmethod
    def from_plain_state_dict(cls, plain: dict, reference=None) -> "Int8QWeight":
        packed = plain["weight_packed"]
        out_f, quarter = packed.shape
        u = torch.stack([(packed >> (8 * i)) & 0xFF for i in range(4)], dim=-1)
        weight = (u.reshape(out_f, quarter * 4) - 128).to(torch.int8)
        return cls(weight, plain["weight_scale"].squeeze(-1))

    @classmethod
    def build_hf_quantization_config(cls, skip_patterns=(), **_) -> dict:
        return {
            "quant_method": "compressed-tensors",
            "format": "pack-quantized",
            "config_groups": {
                "group_0": {
                    "weights": {
                        "num_bits": 8,
                        "type": "int",
                        "symmetric": True,
                        "strategy": "channel",
                    },
                    "targets": ["Linear"],
                },
            },
            "ignore": list(skip_patterns),
        }
