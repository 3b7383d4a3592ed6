"""NF4 block-wise QAT weight in bitsandbytes storage (no double quantisation).

Payload:
  weight_packed : (out_f, in_f // 2) uint8 - two 4-bit codebook indices per byte,
                  even column in the HIGH nibble
  absmax        : (out_f * n_blocks,) fp32 - per-block abs-max, row-major

Each block of ``blocksize`` values (default 64) is divided by its abs-max and
snapped to the nearest entry of the 16-value normal-float codebook.  Same
storage and public names as the reference module
(src/offload_adam/qweight/nf4.py).
"""

import json
from typing import Tuple

import torch
from torch import Tensor

from . import _codec_ops
from .base import QWeightBase

_DTYPE_NAMES = {torch.bfloat16: "bfloat16", torch.float16: "float16", torch.float32: "float32"}
_DTYPES_BY_NAME = {v: k for k, v in _DTYPE_NAMES.items()}

# bitsandbytes' canonical NF4 codebook (quantiles of N(0, 1) scaled to [-1, 1])
NF4_LUT = (
    -1.0,
    -0.6961928009986877,
    -0.5250730514526367,
    -0.39491748809814453,
    -0.28444138169288635,
    -0.18477343022823334,
    -0.09105003625154495,
    0.0,
    0.07958029955625534,
    0.16093020141124725,
    0.24611230194568634,
    0.33791524171829224,
    0.44070982933044434,
    0.5626170039176941,
    0.7229568362236023,
    1.0,
)

_lut_cache: dict = {}


def _nf4_lut(device, dtype: torch.dtype = torch.float32) -> Tensor:
    """The codebook as a tensor, cached per (device, dtype)."""
    key = (torch.device(device), dtype)
    if key not in _lut_cache:
        _lut_cache[key] = torch.tensor(NF4_LUT, dtype=dtype, device=device)
    return _lut_cache[key]


def pack_nf4(indices: Tensor) -> Tensor:
    """(out_f, in_f) uint8 indices -> (out_f, in_f // 2) uint8, even column high."""
    assert indices.dtype is torch.uint8 and indices.shape[1] % 2 == 0
    return ((indices[:, 0::2] << 4) | indices[:, 1::2]).to(torch.uint8)


def unpack_nf4(packed: Tensor) -> Tensor:
    assert packed.dtype is torch.uint8
    pairs = torch.stack([(packed >> 4) & 0xF, packed & 0xF], dim=-1)
    return pairs.reshape(packed.shape[0], packed.shape[1] * 2)


@torch.no_grad()
def quantize_nf4_blockwise(tensor: Tensor, blocksize: int = 64) -> Tuple[Tensor, Tensor]:
    """(out_f, in_f) float -> (packed uint8, flat fp32 absmax)."""
    assert tensor.ndim == 2
    out_f, in_f = tensor.shape
    assert in_f % blocksize == 0 and in_f % 2 == 0
    if tensor.is_cuda and blocksize % 2 == 0:
        return _quantize_nf4_hip(tensor, blocksize)
    x = tensor.float().reshape(out_f, in_f // blocksize, blocksize)
    absmax = x.abs().amax(dim=-1)
    # multiply by the reciprocal (not divide): that is what the kernels do
    normalized = x * (1.0 / absmax.clamp(min=1e-12))[..., None]
    dist = (normalized[..., None] - _nf4_lut(tensor.device)).abs()
    indices = dist.argmin(dim=-1).to(torch.uint8).reshape(out_f, in_f)
    return pack_nf4(indices), absmax.reshape(-1)


def dequantize_nf4_blockwise(packed, absmax, in_f, blocksize=64, dtype=torch.float32) -> Tensor:
    """Codebook gather and block scale, both in ``dtype`` (any torch float dtype)."""
    out_f = packed.shape[0]
    vals = _nf4_lut(packed.device, dtype)[unpack_nf4(packed).long()]
    vals = vals.reshape(out_f, in_f // blocksize, blocksize)
    return (vals * absmax.to(dtype).reshape(out_f, -1)[..., None]).reshape(out_f, in_f)


def _quantize_nf4_hip(tensor, blocksize):
    out_f, in_f = tensor.shape
    packed = torch.empty((out_f, in_f // 2), dtype=torch.uint8, device=tensor.device)
    absmax = torch.empty((out_f * (in_f // blocksize),), dtype=torch.float32, device=tensor.device)
    _codec_ops.quantize_nf4_into(tensor, blocksize, packed, absmax)
    return packed, absmax


def _dequant_nf4_hip(packed, absmax, in_f, blocksize, out_dtype):
    """fp32 codebook value times fp32 absmax, rounded once to ``out_dtype``."""
    return _codec_ops.dequantize_nf4(packed.contiguous(), absmax.contiguous(), in_f, blocksize,
                                     out_dtype)


class NF4QWeight(QWeightBase):
    _PAYLOAD = ("weight_packed", "absmax")

    @staticmethod
    @torch._dynamo.disable
    def __new__(cls, weight_packed, absmax, in_f, blocksize, outer_dtype):
        return Tensor._make_wrapper_subclass(
            cls, (weight_packed.shape[0], in_f), dtype=outer_dtype, device=weight_packed.device
        )

    @torch._dynamo.disable
    def __init__(self, weight_packed, absmax, in_f, blocksize, outer_dtype):
        assert weight_packed.dtype is torch.uint8 and weight_packed.ndim == 2
        assert absmax.dtype is torch.float32 and absmax.ndim == 1
        self.weight_packed = weight_packed
        self.absmax = absmax
        self.in_f = in_f
        self.blocksize = blocksize
        self.outer_dtype = outer_dtype

    def _meta(self):
        return (self.in_f, self.blocksize, self.outer_dtype)

    def _meta_to(self, dtype):
        return (self.in_f, self.blocksize, dtype if dtype is not None else self.outer_dtype)

    def _repr_extra(self):
        return {"blocksize": self.blocksize}

    @classmethod
    def from_float(cls, tensor: Tensor, blocksize: int = 64, **_):
        packed, absmax = quantize_nf4_blockwise(tensor.detach(), blocksize)
        out = cls(packed, absmax, tensor.shape[1], blocksize, tensor.dtype)
        out.requires_grad_(tensor.requires_grad)
        return out

    @classmethod
    def can_quantize(cls, tensor: Tensor, blocksize: int = 64, **_) -> bool:
        return tensor.dim() == 2 and tensor.shape[1] % blocksize == 0 and tensor.shape[1] % 2 == 0

    def _requantize_(self, src: Tensor) -> None:
        if self.weight_packed.is_cuda:
            src = src.detach().to(self.weight_packed.device, non_blocking=True)
            _codec_ops.quantize_nf4_into(src, self.blocksize, self.weight_packed, self.absmax)
        else:
            packed, absmax = quantize_nf4_blockwise(src.detach(), self.blocksize)
            self.weight_packed.copy_(packed)
            self.absmax.copy_(absmax)

    def dequantize(self, dtype=None) -> Tensor:
        dtype = self.outer_dtype if dtype is None else dtype
        if self.weight_packed.is_cuda and dtype in _DTYPE_NAMES:
            return _dequant_nf4_hip(self.weight_packed, self.absmax, self.in_f, self.blocksize,
                                    dtype)
        if dtype in _DTYPE_NAMES:
            return dequantize_nf4_blockwise(self.weight_packed, self.absmax, self.in_f,
                                            self.blocksize, torch.float32).to(dtype)
        return dequantize_nf4_blockwise(self.weight_packed, self.absmax, self.in_f,
                                        self.blocksize, dtype)

    # ---- serialisation: bitsandbytes QuantState keys (plain torch) ------------

    @classmethod
    def canonical_key_suffixes(cls) -> Tuple[str, ...]:
        return ("weight", "weight.absmax", "weight.quant_map",
                "weight.quant_state.bitsandbytes__nf4")

    def to_plain_state_dict(self) -> dict:
        out_f, half = self.weight_packed.shape
        device = self.weight_packed.device
        meta = {
            "quant_type": "nf4",
            "blocksize": self.blocksize,
            "dtype": _DTYPE_NAMES[self.outer_dtype],
            "shape": [out_f, half * 2],
        }
        blob = torch.tensor(list(json.dumps(meta).encode("utf-8")), dtype=torch.uint8,
                            device=device)
        return {
            "weight": self.weight_packed.reshape(-1, 1),  # bnb keeps a column vector
            "weight.absmax": self.absmax,
            "weight.quant_map": torch.tensor(NF4_LUT, dtype=torch.float32, device=device),
            "weight.quant_state.bitsandbytes__nf4": blob,
        }

    @classmethod
    def from_plain_state_dict(cls, plain: dict, reference=None) -> "NF4QWeight":
        raw = bytes(plain["weight.quant_state.bitsandbytes__nf4"].cpu().tolist())
        meta = json.loads(raw.decode("utf-8"))
        out_f, in_f = meta["shape"]
        return cls(plain["weight"].reshape(out_f, in_f // 2), plain["weight.absmax"], in_f,
                   meta["blocksize"], _DTYPES_BY_NAME[meta["dtype"]])

    @classmethod
    def build_hf_quantization_config(cls, skip_patterns=(), compute_dtype: str = "bfloat16",
                                     **_) -> dict:
        return {
            "quant_method": "bitsandbytes",
            "load_in_4bit": True,
            "bnb_4bit_quant_type": "nf4",
            "bnb_4bit_use_double_quant": False,
            "bnb_4bit_compute_dtype": compute_dtype,
            "llm_int8_skip_modules": list(skip_patterns),
        }
