"""Quantised-weight tensor subclasses for QAT, backed by HIP codec kernels.

Four storage formats (one module each) share ``QWeightBase``; ``apply`` holds
the helpers that swap them into a model's ``nn.Linear`` layers and write
checkpoints other runtimes can read.
"""

from . import apply as _apply
from . import base as _base
from . import int4 as _int4, int8 as _int8, nf4 as _nf4, nvfp4 as _nvfp4

QWeightBase = _base.QWeightBase
cache_dequantized_weights = _base.cache_dequantized_weights
Int8QWeight, Int4QWeight = _int8.Int8QWeight, _int4.Int4QWeight
NF4QWeight, NVFP4QWeight = _nf4.NF4QWeight, _nvfp4.NVFP4QWeight
quantize_linears = _apply.quantize_linears
save_quantized_pretrained = _apply.save_quantized_pretrained
QuantizeReport = _apply.QuantizeReport

FORMATS = {"int8": Int8QWeight, "int4": Int4QWeight, "nf4": NF4QWeight, "nvfp4": NVFP4QWeight}

__all__ = ["QWeightBase", *sorted(cls.__name__ for cls in FORMATS.values()),
           "quantize_linears", "save_quantized_pretrained", "QuantizeReport", "FORMATS",
           "cache_dequantized_weights"]
