"""Argument handling shared by the four ``adam_step_*`` wrappers."""

from ctypes import c_float, c_int, c_int64

import torch

from .. import _lib


def folded_betas(beta1, beta2, step):
    """Bias correction folded into the running-average coefficients, in Python
    double exactly as the reference wrappers do (kernels/fp32_master.py:74-75)."""
    beta1_hat = (beta1**step - beta1) / (beta1**step - 1)
    beta2_hat = (beta2**step - beta2) / (beta2**step - 1)
    return beta1_hat, beta2_hat


def check_tensor(t, name, dtype, numel, device):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if t.device != device:
        raise ValueError(f"{name} is on {t.device}, expected {device}")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (no CPU path exists)")
    if t.numel() != numel:
        raise ValueError(f"{name} has {t.numel()} elements, expected {numel}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def check_clip(clip_coef, device):
    if clip_coef is None:
        return
    check_tensor(clip_coef, "clip_coef", torch.bfloat16, 1, device)


def scalar_args(params, lr, weight_decay, beta1, beta2, eps, step, decoupled):
    b1h, b2h = folded_betas(beta1, beta2, step)
    return [
        c_int64(params.numel()),
        c_float(lr),
        c_float(weight_decay),
        c_float(b1h),
        c_float(b2h),
        c_float(eps),
        c_int(1 if decoupled else 0),
    ]


def launch(fn_name, params, ptr_args, tail_args):
    """Call an entry point on ``params``' device and current stream."""
    lib = _lib.load()
    with _lib.device_guard(params.device):
        code = getattr(lib, fn_name)(*ptr_args, *tail_args, _lib.current_stream_ptr())
    _lib.check(code, fn_name)
