"""Int4 symmetric group-wise QAT weight in GPTQ storage.

Payload:
  qweight : (in_f // 8, out_f) int32 - eight codes of one output row packed
            LSB first along in_f, each stored as code + 8 (zero point 8)
  scales  : (in_f // group, out_f)   - group absmax / 8

Same storage and public names as the reference module
(src/offload_adam/qweight/int4.py).  GPU tensors go through the HIP kernels,
which stage the transposed layout through LDS so both sides stay coalesced.
"""

from typing import Tuple

import torch
from torch import Tensor

from . import _codec_ops
from .base import QWeightBase


def pack_int4_gptq(int_data: Tensor) -> Tensor:
    """(out_f, in_f) int8 codes in [-8, 7] -> (in_f // 8, out_f) int32 with
    packed[k, n] = sum_i (int_data[n, 8k + i] + 8) << 4i."""
    out_f, in_f = int_data.shape
    assert in_f % 8 == 0, f"in_features={in_f} must be a multiple of 8"
    u = (int_data.to(torch.int32) + 8).reshape(out_f, in_f // 8, 8)
    words = torch.zeros(out_f, in_f // 8, dtype=torch.int32, device=int_data.device)
    for i in range(8):
        words |= u[..., i] << (4 * i)
    return words.T.contiguous()


def unpack_int4_gptq(packed: Tensor) -> Tensor:
    """Inverse of ``pack_int4_gptq``: (out_f, in_f) int8 in [-8, 7]."""
    k, out_f = packed.shape
    rows = packed.T.contiguous()
    nib = torch.stack([(rows >> (4 * i)) & 0xF for i in range(8)], dim=-1)
    return (nib - 8).to(torch.int8).reshape(out_f, k * 8)


@torch.no_grad()
def quantize_int4_groupwise(
    tensor: Tensor, group_size: int = 128, eps: float = 1e-12
) -> Tuple[Tensor, Tensor]:
    """(out_f, in_f) float -> (GPTQ-packed int32, scales (n_groups, out_f) in the
    input dtype)."""
    out_f, in_f = tensor.shape
    assert in_f % group_size == 0, f"in_features={in_f} not divisible by group_size={group_size}"
    assert in_f % 8 == 0, f"in_features={in_f} must be a multiple of 8"
    if tensor.is_cuda and eps == 1e-12 and group_size % 8 == 0:
        return _quantize_pack_int4_hip(tensor, group_size, tensor.dtype)
    x = tensor.float().reshape(out_f, in_f // group_size, group_size)
    scale = x.abs().amax(dim=-1) / 8
    recip = 1.0 / scale.clamp(min=eps)
    codes = (x * recip[..., None]).round().clamp(-8, 7).to(torch.int8).reshape(out_f, in_f)
    return pack_int4_gptq(codes), scale.T.contiguous().to(tensor.dtype)


def _quantize_pack_int4_hip(tensor, group_size, scale_dtype):
    out_f, in_f = tensor.shape
    qweight = torch.empty((in_f // 8, out_f), dtype=torch.int32, device=tensor.device)
    scales = torch.empty((in_f // group_size, out_f), dtype=scale_dtype, device=tensor.device)
    _codec_ops.quantize_int4_into(tensor, group_size, qweight, scales)
    return qweight, scales


def _dequant_int4_hip(qweight, scales, group_size):
    return _codec_ops.dequantize_int4(qweight.contiguous(), scales.contiguous(), group_size)


class Int4QWeight(QWeightBase):
    _PAYLOAD = ("qweight", "scales")

    @staticmethod
    @torch._dynamo.disable
    def __new__(cls, qweight: Tensor, scales: Tensor, group_size: int):
        return Tensor._make_wrapper_subclass(
            cls, (qweight.shape[1], qweight.shape[0] * 8), dtype=scales.dtype,
            device=qweight.device,
        )

    @torch._dynamo.disable
    def __init__(self, qweight: Tensor, scales: Tensor, group_size: int):
        assert qweight.dtype is torch.int32 and qweight.ndim == 2
        assert scales.ndim == 2
        self.qweight = qweight
        self.scales = scales
        self.group_size = group_size

    def _meta(self):
        return (self.group_size,)

    def _repr_extra(self):
        return {"group_size": self.group_size}

    def _payload_to(self, name, tensor, device, dtype):
        if name == "scales":
            return tensor.to(device=device, dtype=dtype)
        return tensor.to(device=device)

    @classmethod
    def from_float(cls, tensor: Tensor, group_size: int = 128,
                   scale_dtype: torch.dtype = torch.bfloat16):
        """``scale_dtype`` is both the stored scale dtype and the outer dtype."""
        qweight, scales = quantize_int4_groupwise(tensor.detach(), group_size)
        out = cls(qweight, scales.to(scale_dtype), group_size)
        out.requires_grad_(tensor.requires_grad)
        return out

    @classmethod
    def can_quantize(cls, tensor: Tensor, group_size: int = 128, **_) -> bool:
        return tensor.dim() == 2 and tensor.shape[1] % group_size == 0 and tensor.shape[1] % 8 == 0

    def _requantize_(self, src: Tensor) -> None:
        if self.qweight.is_cuda:
            src = src.detach().to(self.qweight.device, non_blocking=True)
            _codec_ops.quantize_int4_into(src, self.group_size, self.qweight, self.scales)
        else:
            qweight, scales = quantize_int4_groupwise(src.detach(), self.group_size)
            self.qweight.copy_(qweight)
            self.scales.copy_(scales)

    def dequantize(self, dtype=None) -> Tensor:
        want = self.scales.dtype if dtype is None else dtype
        if self.qweight.is_cuda and want in (self.scales.dtype, torch.float32):
            return _codec_ops.dequantize_int4(self.qweight, self.scales, self.group_size, want)
        compute = torch.float32 if want == torch.float32 else self.scales.dtype
        n_groups = self.scales.shape[0]
        codes = unpack_int4_gptq(self.qweight).reshape(self.shape[0], n_groups, self.group_size)
        vals = codes.to(compute) * self.scales.T.to(compute)[..., None]
        return vals.reshape(self.shape).to(want)

    # ---- serialisation: GPTQ (plain torch) -----------------------------------

    @classmethod
    def canonical_key_suffixes(cls) -> Tuple[str, ...]:
        return ("qweight", "scales", "qzeros")  # g_idx omitted (desc_act=False)

    def to_plain_state_dict(self) -> dict:
        n_groups, out_f = self.scales.shape
        assert out_f % 8 == 0, (
            f"out_features={out_f} must be a multiple of 8 to serialize symmetric qzeros"
        )
        # zero point 8 in every nibble: 0x88888888 as a signed int32
        qzeros = torch.full((n_groups, out_f // 8), -0x77777778, dtype=torch.int32,
                            device=self.qweight.device)
        return {"qweight": self.qweight, "scales": self.scales, "qzeros": qzeros}

    @classmethod
    def from_plain_state_dict(cls, plain: dict, reference=None) -> "Int4QWeight":
        qweight, scales = plain["qweight"], plain["scales"]
        return cls(qweight, scales, qweight.shape[0] * 8 // scales.shape[0])

    @classmethod
    def build_hf_quantization_config(cls, skip_patterns=(), group_size: int = 128, **_) -> dict:
        return {
            "quant_method": "gptq",
            "bits": 4,
            "group_size": group_size,
            "desc_act": False,
            "sym": True,
            "modules_to_not_convert": list(skip_patterns),
        }
