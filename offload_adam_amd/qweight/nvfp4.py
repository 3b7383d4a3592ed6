"""NVFP4 block-wise QAT weight (compressed-tensors W4A16 NVFP4 storage).

Payload:
  weight_packed   : (out_f, in_f // 2) uint8 - two FP4 (E2M1) codes per byte,
                    even column in the LOW nibble
  block_scale_fp8 : (out_f, in_f // 16) float8_e4m3fn - one scale per 16 values
  global_scale    : () fp32 - tensor scale; effective scale of a block =
                    float(block_scale) * global_scale

The tensor scale maps the largest block scale to 448 (the E4M3 maximum), so the
per-block scales use the FP8 range whatever the tensor's magnitude.  Same
storage and public names as the reference module
(src/offload_adam/qweight/nvfp4.py); on the GPU both directions run as HIP
kernels that build E2M1 and E4M3 values by bit arithmetic.
"""

from typing import Tuple

import torch
from torch import Tensor

from . import _codec_ops
from .base import QWeightBase

NVFP4_BLOCKSIZE = 16
FP4_E2M1_MAX = 6.0
FP8_E4M3_MAX = 448.0

# code bit 3 = sign, bits 2..1 = exponent (bias 1), bit 0 = mantissa
FP4_E2M1_LUT = (
    0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
    -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0,
)

_HIP_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
_lut_cache: dict = {}


def _fp4_lut(device, dtype: torch.dtype = torch.float32) -> Tensor:
    key = (torch.device(device), dtype)
    if key not in _lut_cache:
        _lut_cache[key] = torch.tensor(FP4_E2M1_LUT, dtype=dtype, device=device)
    return _lut_cache[key]


def pack_fp4(indices: Tensor) -> Tensor:
    """(out_f, in_f) uint8 codes -> (out_f, in_f // 2) uint8, even column LOW."""
    assert indices.dtype is torch.uint8 and indices.shape[1] % 2 == 0
    return ((indices[:, 1::2] << 4) | indices[:, 0::2]).to(torch.uint8)


def unpack_fp4(packed: Tensor) -> Tensor:
    assert packed.dtype is torch.uint8
    pairs = torch.stack([packed & 0xF, (packed >> 4) & 0xF], dim=-1)
    return pairs.reshape(packed.shape[0], packed.shape[1] * 2)


def _quantize_fp4_e2m1_rne(x: Tensor) -> Tensor:
    """fp32 -> E2M1 code, round to nearest even on the magnitudes
    {0, .5, 1, 1.5, 2, 3, 4, 6}, saturating at 6; bit 3 = IEEE sign (-0 -> 8).

    A tie goes to the neighbour with the even mantissa bit, hence the mix of
    strict and non-strict comparisons at the seven midpoints."""
    mag = x.abs()
    code = torch.zeros_like(mag, dtype=torch.uint8)
    for midpoint, up_on_tie in ((0.25, False), (0.75, True), (1.25, False), (1.75, True),
                                (2.5, False), (3.5, True), (5.0, False)):
        code += ((mag >= midpoint) if up_on_tie else (mag > midpoint)).to(torch.uint8)
    return code | (torch.signbit(x).to(torch.uint8) << 3)


@torch.no_grad()
def quantize_nvfp4_blockwise(tensor: Tensor, eps: float = 1e-12) -> Tuple[Tensor, Tensor, Tensor]:
    """(out_f, in_f) float -> (packed uint8, float8_e4m3fn block scales, fp32 ())."""
    assert tensor.ndim == 2
    out_f, in_f = tensor.shape
    assert in_f % NVFP4_BLOCKSIZE == 0
    if tensor.is_cuda and eps == 1e-12:
        return _quantize_nvfp4_hip(tensor)
    x = tensor.float()
    global_scale = x.abs().amax().clamp(min=eps) / (FP8_E4M3_MAX * FP4_E2M1_MAX)
    blocks = x.reshape(out_f, in_f // NVFP4_BLOCKSIZE, NVFP4_BLOCKSIZE)
    block_scale = blocks.abs().amax(dim=-1).clamp(min=eps) / FP4_E2M1_MAX
    block_scale_fp8 = (block_scale * (1.0 / global_scale)).to(torch.float8_e4m3fn)
    effective = block_scale_fp8.to(torch.float32) * global_scale
    normalized = blocks * (1.0 / effective.clamp(min=eps))[..., None]
    codes = _quantize_fp4_e2m1_rne(normalized).reshape(out_f, in_f)
    return pack_fp4(codes), block_scale_fp8, global_scale


def dequantize_nvfp4_blockwise(packed, block_scale_fp8, global_scale, in_f,
                               dtype=torch.float32) -> Tensor:
    out_f = packed.shape[0]
    vals = _fp4_lut(packed.device)[unpack_fp4(packed).long()]
    vals = vals.reshape(out_f, in_f // NVFP4_BLOCKSIZE, NVFP4_BLOCKSIZE)
    effective = (block_scale_fp8.to(torch.float32) * global_scale).reshape(out_f, -1)
    return (vals * effective[..., None]).reshape(out_f, in_f).to(dtype)


def _quantize_nvfp4_hip(tensor):
    out_f, in_f = tensor.shape
    dev = tensor.device
    packed = torch.empty((out_f, in_f // 2), dtype=torch.uint8, device=dev)
    scale = torch.empty((out_f, in_f // NVFP4_BLOCKSIZE), dtype=torch.float8_e4m3fn, device=dev)
    global_scale = torch.empty((), dtype=torch.float32, device=dev)
    _codec_ops.quantize_nvfp4_into(tensor, packed, scale, global_scale)
    return packed, scale, global_scale


def _dequant_nvfp4_hip(packed, block_scale_fp8, global_scale, in_f, out_dtype):
    return _codec_ops.dequantize_nvfp4(packed.contiguous(), block_scale_fp8.contiguous(),
                                       global_scale, in_f, out_dtype)


class NVFP4QWeight(QWeightBase):
    _PAYLOAD = ("weight_packed", "block_scale_fp8", "global_scale")

    @staticmethod
    @torch._dynamo.disable
    def __new__(cls, weight_packed, block_scale_fp8, global_scale, in_f, outer_dtype):
        return Tensor._make_wrapper_subclass(
            cls, (weight_packed.shape[0], in_f), dtype=outer_dtype, device=weight_packed.device
        )

    @torch._dynamo.disable
    def __init__(self, weight_packed, block_scale_fp8, global_scale, in_f, outer_dtype):
        assert weight_packed.dtype is torch.uint8 and weight_packed.ndim == 2
        assert block_scale_fp8.dtype is torch.float8_e4m3fn and block_scale_fp8.ndim == 2
        assert global_scale.dtype is torch.float32
        self.weight_packed = weight_packed
        self.block_scale_fp8 = block_scale_fp8
        self.global_scale = global_scale
        self.in_f = in_f
        self.outer_dtype = outer_dtype

    def _meta(self):
        return (self.in_f, self.outer_dtype)

    def _meta_to(self, dtype):
        return (self.in_f, dtype if dtype is not None else self.outer_dtype)

    @classmethod
    def from_float(cls, tensor: Tensor, **_):
        packed, scale, gs = quantize_nvfp4_blockwise(tensor.detach())
        out = cls(packed, scale, gs, tensor.shape[1], tensor.dtype)
        out.requires_grad_(tensor.requires_grad)
        return out

    @classmethod
    def can_quantize(cls, tensor: Tensor, **_) -> bool:
        return tensor.dim() == 2 and tensor.shape[1] % NVFP4_BLOCKSIZE == 0

    def _requantize_(self, src: Tensor) -> None:
        if self.weight_packed.is_cuda:
            src = src.detach().to(self.weight_packed.device, non_blocking=True)
            _codec_ops.quantize_nvfp4_into(src, self.weight_packed, self.block_scale_fp8,
                                           self.global_scale)
        else:
            packed, scale, gs = quantize_nvfp4_blockwise(src.detach())
            self.weight_packed.copy_(packed)
            self.block_scale_fp8.copy_(scale)
            self.global_scale.copy_(gs)

    def dequantize(self, dtype=None) -> Tensor:
        dtype = self.outer_dtype if dtype is None else dtype
        if self.weight_packed.is_cuda and dtype in _HIP_DTYPES:
            return _dequant_nvfp4_hip(self.weight_packed, self.block_scale_fp8,
                                      self.global_scale, self.in_f, dtype)
        return dequantize_nvfp4_blockwise(self.weight_packed, self.block_scale_fp8,
                                          self.global_scale, self.in_f, dtype)

    # ---- serialisation: compressed-tensors nvfp4-pack-quantized ---------------

    @classmethod
    def canonical_key_suffixes(cls) -> Tuple[str, ...]:
        return ("weight_packed", "weight_scale", "weight_global_scale")

    def to_plain_state_dict(self) -> dict:
        # compressed-tensors stores the reciprocal of this module's tensor scale
        return {
            "weight_packed": self.weight_packed,
            "weight_scale": self.block_scale_fp8,
            "weight_global_scale": (1.0 / self.global_scale).reshape(1),
        }

    @classmethod
    def from_plain_state_dict(cls, plain: dict, reference=None) -> "NVFP4QWeight":
        if reference is None:
            raise ValueError(
                "NVFP4QWeight.from_plain_state_dict requires a reference instance to "
                "resolve outer_dtype; the canonical state_dict carries no outer-dtype field."
            )
        packed = plain["weight_packed"]
        global_scale = (1.0 / plain["weight_global_scale"]).reshape(())
        return cls(packed, plain["weight_scale"], global_scale, packed.shape[1] * 2,
                   reference.outer_dtype)

    @classmethod
    def build_hf_quantization_config(cls, skip_patterns=(), **_) -> dict:
        return {
            "quant_method": "compressed-tensors",
            "format": "nvfp4-pack-quantized",
            "config_groups": {
                "group_0": {
                    "weights": {
                        "num_bits": 4,
                        "type": "float",
                        "symmetric": True,
                        "strategy": "tensor_group",
                        "group_size": NVFP4_BLOCKSIZE,
                    },
                    "targets": ["Linear"],
                },
            },
            "ignore": list(skip_patterns),
        }
