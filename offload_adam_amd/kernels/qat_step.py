"""fp32_master AdamW step of a quantised weight, fused with its re-encoding.

The reference steps a quantised parameter in two moves: the fp32_master kernel
with the gradient buffer as a throw-away bf16 sink, then ``p.data.copy_(master)``
which re-quantises the payload from the new master
(src/offload_adam/offload_adam.py:421-444, src/offload_adam/adam.py:139-151).
``oa_adam_requant_*`` does both in one pass over HBM with identical results; this
module picks the entry point for a weight subclass, or says it cannot.
"""

from ctypes import c_float, c_int, c_int64

import torch

from .. import _lib
from . import _common


def _is_pow2(v):
    return v > 0 and (v & (v - 1)) == 0


def _plan(qw):
    """(entry point, payload arguments before the stream, payload tensors the
    kernel writes) for a weight subclass, or None when the fused kernels do not
    cover its layout."""
    from ..qweight import Int4QWeight, Int8QWeight, NF4QWeight, NVFP4QWeight, _codec_ops

    rows, cols = qw.shape
    if rows == 0 or cols == 0 or cols % 8 != 0:
        return None
    if isinstance(qw, Int8QWeight):
        payload = (qw.weight, qw.scales)
        tail = [_lib.ptr(qw.weight), _lib.ptr(qw.scales), c_int(_lib.dtype_code(qw.scales.dtype))]
        name = "oa_adam_requant_int8"
    elif isinstance(qw, Int4QWeight):
        g = qw.group_size
        if not _is_pow2(g) or g < 8 or g > 512 or cols % g != 0 or rows > 65535 * 64:
            return None
        payload = (qw.qweight, qw.scales)
        tail = [c_int64(g), _lib.ptr(qw.qweight), _lib.ptr(qw.scales),
                c_int(_lib.dtype_code(qw.scales.dtype))]
        name = "oa_adam_requant_int4"
    elif isinstance(qw, NF4QWeight):
        b = qw.blocksize
        if b % 8 != 0 or not _is_pow2(b // 8) or b > 512 or cols % b != 0:
            return None
        payload = (qw.weight_packed, qw.absmax)
        tail = [c_int64(b), _lib.ptr(qw.weight_packed), _lib.ptr(qw.absmax)]
        name = "oa_adam_requant_nf4"
    elif isinstance(qw, NVFP4QWeight):
        if cols % 16 != 0:
            return None
        payload = (qw.weight_packed, qw.block_scale_fp8, qw.global_scale)
        with _lib.device_guard(qw.weight_packed.device):
            ws = _codec_ops._amax_workspace(qw.weight_packed.device, _lib.current_stream_id())
        tail = [_lib.ptr(qw.weight_packed), _lib.ptr(qw.block_scale_fp8),
                _lib.ptr(qw.global_scale), _lib.ptr(ws)]
        name = "oa_adam_requant_nvfp4"
    else:
        return None
    for t in payload:
        if not t.is_cuda or not t.is_contiguous() or t.data_ptr() % 16 != 0:
            return None
    return name, tail, payload


def adam_step_requant(qweight, states, lr, weight_decay, beta1, beta2, eps, step,
                      decoupled_weight_decay=False, clip_coef=None):
    """One fused launch: AdamW on ``states`` (grad, exp_avg, exp_avg_sq bf16,
    master_params fp32, all of ``qweight``'s logical shape) and the payload of
    ``qweight`` re-encoded from the new master.  Returns False without touching
    anything when the layout is outside what the fused kernels take; the caller
    then runs the step and ``qweight.copy_(master)`` separately."""
    master = states["master_params"]
    dev = master.device
    n = master.numel()
    if n != qweight.numel() or qweight.dim() != 2 or not master.is_cuda:
        return False
    plan = _plan(qweight)
    if plan is None:
        return False
    name, tail, payload = plan
    for key, dtype in (("grad", torch.bfloat16), ("exp_avg", torch.bfloat16),
                       ("exp_avg_sq", torch.bfloat16), ("master_params", torch.float32)):
        _common.check_tensor(states[key], f"states['{key}']", dtype, n, dev)
        if states[key].data_ptr() % 16 != 0:
            return False
    _common.check_clip(clip_coef, dev)
    rows, cols = qweight.shape
    b1h, b2h = _common.folded_betas(beta1, beta2, step)
    lib = _lib.load()
    with _lib.device_guard(dev):
        code = getattr(lib, name)(
            _lib.ptr(states["grad"]), _lib.ptr(states["exp_avg"]), _lib.ptr(states["exp_avg_sq"]),
            _lib.ptr(master), c_int64(rows), c_int64(cols), c_float(lr), c_float(weight_decay),
            c_float(b1h), c_float(b2h), c_float(eps), c_int(1 if decoupled_weight_decay else 0),
            _lib.ptr(clip_coef), *tail, _lib.current_stream_ptr())
    _lib.check(code, name)
    from ..qweight._codec_ops import mark_written

    mark_written(*payload)
    return True
