"""HIP codec launches: quantise into existing payload buffers, dequantise into a
fresh (or given) tensor.  GPU tensors only; every function enqueues on the
current stream of the tensor's device and returns without synchronising.
"""

from ctypes import c_int, c_int64

import torch

from .. import _lib

_nvfp4_ws = {}


def _amax_workspace(device, stream_id):
    key = (device.index, stream_id)
    ws = _nvfp4_ws.get(key)
    if ws is None:
        ws = torch.zeros(_lib.load().oa_norm_workspace_bytes(), dtype=torch.uint8, device=device)
        _nvfp4_ws[key] = ws
    return ws


def _rows_view(t):
    """2-D float tensor -> (tensor with unit column stride, row stride in elements)."""
    if t.dim() != 2:
        raise ValueError(f"expected a 2-D weight, got shape {tuple(t.shape)}")
    if not t.is_cuda:
        raise ValueError("HIP codecs work on GPU tensors")
    if t.shape[1] > 1 and t.stride(1) != 1:
        t = t.contiguous()
    if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
        t = t.contiguous()
    stride = t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)
    return t, stride


def _payload(t, name, dtype, shape):
    if t.dtype != dtype or tuple(t.shape) != tuple(shape) or not t.is_contiguous() or not t.is_cuda:
        raise ValueError(
            f"{name}: need a contiguous GPU tensor of {dtype} with shape {tuple(shape)}, "
            f"got {t.dtype} {tuple(t.shape)}"
        )


def _call(name, device, *args):
    lib = _lib.load()
    with _lib.device_guard(device):
        code = getattr(lib, name)(*args, _lib.current_stream_ptr())
    _lib.check(code, name)


# -------------------------------------------------------------------- int8


def mark_written(*tensors):
    """The kernels write payload tensors through raw pointers, which autograd's
    version counters do not see; bump them, as an in-place torch op would, so
    that anything keyed on a payload's version (the dequantisation cache of the
    linear layers) notices."""
    for t in tensors:
        torch.autograd.graph.increment_version(t)


def quantize_int8_into(src, weight, scales):
    """Per-row symmetric int8 codes of ``src`` into ``weight`` (R,C) int8 and
    ``scales`` (R,) float."""
    src, stride = _rows_view(src)
    rows, cols = src.shape
    _payload(weight, "weight", torch.int8, (rows, cols))
    _payload(scales, "scales", scales.dtype, (rows,))
    _call("oa_quant_int8", src.device, _lib.ptr(src), c_int(_lib.dtype_code(src.dtype)),
          c_int64(stride), c_int64(rows), c_int64(cols), _lib.ptr(weight), _lib.ptr(scales),
          c_int(_lib.dtype_code(scales.dtype)))
    mark_written(weight, scales)


def dequantize_int8(weight, scales, out_dtype=None):
    rows, cols = weight.shape
    out = torch.empty((rows, cols), dtype=out_dtype or scales.dtype, device=weight.device)
    _payload(weight, "weight", torch.int8, (rows, cols))
    _payload(scales, "scales", scales.dtype, (rows,))
    _call("oa_dequant_int8", weight.device, _lib.ptr(weight), _lib.ptr(scales),
          c_int(_lib.dtype_code(scales.dtype)), c_int64(rows), c_int64(cols), _lib.ptr(out),
          c_int(_lib.dtype_code(out.dtype)), c_int64(max(cols, 1)))
    return out


# -------------------------------------------------------------------- int4


def quantize_int4_into(src, group_size, qweight, scales):
    """Group-wise symmetric int4 of ``src`` into ``qweight`` (C/8,R) int32 and
    ``scales`` (C/group,R)."""
    src, stride = _rows_view(src)
    rows, cols = src.shape
    _payload(qweight, "qweight", torch.int32, (cols // 8, rows))
    _payload(scales, "scales", scales.dtype, (cols // group_size, rows))
    _call("oa_quant_int4", src.device, _lib.ptr(src), c_int(_lib.dtype_code(src.dtype)),
          c_int64(stride), c_int64(rows), c_int64(cols), c_int64(group_size),
          _lib.ptr(qweight), _lib.ptr(scales), c_int(_lib.dtype_code(scales.dtype)))
    mark_written(qweight, scales)


def dequantize_int4(qweight, scales, group_size, out_dtype=None):
    rows = qweight.shape[1]
    cols = qweight.shape[0] * 8
    _payload(qweight, "qweight", torch.int32, (cols // 8, rows))
    _payload(scales, "scales", scales.dtype, (cols // group_size, rows))
    out = torch.empty((rows, cols), dtype=out_dtype or scales.dtype, device=qweight.device)
    _call("oa_dequant_int4", qweight.device, _lib.ptr(qweight), _lib.ptr(scales),
          c_int(_lib.dtype_code(scales.dtype)), c_int64(rows), c_int64(cols),
          c_int64(group_size), _lib.ptr(out), c_int(_lib.dtype_code(out.dtype)),
          c_int64(max(cols, 1)))
    return out


# --------------------------------------------------------------------- NF4


def quantize_nf4_into(src, blocksize, packed, absmax):
    src, stride = _rows_view(src)
    rows, cols = src.shape
    _payload(packed, "weight_packed", torch.uint8, (rows, cols // 2))
    _payload(absmax, "absmax", torch.float32, (rows * (cols // blocksize),))
    _call("oa_quant_nf4", src.device, _lib.ptr(src), c_int(_lib.dtype_code(src.dtype)),
          c_int64(stride), c_int64(rows), c_int64(cols), c_int64(blocksize), _lib.ptr(packed),
          _lib.ptr(absmax))
    mark_written(packed, absmax)


def dequantize_nf4(packed, absmax, in_f, blocksize, out_dtype):
    rows = packed.shape[0]
    _payload(packed, "weight_packed", torch.uint8, (rows, in_f // 2))
    _payload(absmax, "absmax", torch.float32, (rows * (in_f // blocksize),))
    out = torch.empty((rows, in_f), dtype=out_dtype, device=packed.device)
    _call("oa_dequant_nf4", packed.device, _lib.ptr(packed), _lib.ptr(absmax), c_int64(rows),
          c_int64(in_f), c_int64(blocksize), _lib.ptr(out), c_int(_lib.dtype_code(out_dtype)),
          c_int64(max(in_f, 1)))
    return out


# ------------------------------------------------------------------- NVFP4


def quantize_nvfp4_into(src, packed, block_scale_fp8, global_scale):
    src, stride = _rows_view(src)
    rows, cols = src.shape
    _payload(packed, "weight_packed", torch.uint8, (rows, cols // 2))
    _payload(block_scale_fp8, "block_scale_fp8", torch.float8_e4m3fn, (rows, cols // 16))
    _payload(global_scale, "global_scale", torch.float32, ())
    with _lib.device_guard(src.device):
        ws = _amax_workspace(src.device, _lib.current_stream_id())
    _call("oa_quant_nvfp4", src.device, _lib.ptr(src), c_int(_lib.dtype_code(src.dtype)),
          c_int64(stride), c_int64(rows), c_int64(cols), _lib.ptr(packed),
          _lib.ptr(block_scale_fp8), _lib.ptr(global_scale), _lib.ptr(ws))
    mark_written(packed, block_scale_fp8, global_scale)


def dequantize_nvfp4(packed, block_scale_fp8, global_scale, in_f, out_dtype):
    rows = packed.shape[0]
    _payload(packed, "weight_packed", torch.uint8, (rows, in_f // 2))
    _payload(block_scale_fp8, "block_scale_fp8", torch.float8_e4m3fn, (rows, in_f // 16))
    _payload(global_scale, "global_scale", torch.float32, ())
    out = torch.empty((rows, in_f), dtype=out_dtype, device=packed.device)
    _call("oa_dequant_nvfp4", packed.device, _lib.ptr(packed), _lib.ptr(block_scale_fp8),
          _lib.ptr(global_scale), c_int64(rows), c_int64(in_f), _lib.ptr(out),
          c_int(_lib.dtype_code(out_dtype)), c_int64(max(in_f, 1)))
    return out
