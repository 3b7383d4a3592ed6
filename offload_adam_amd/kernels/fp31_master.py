"""AdamW step on a 31-bit master kept as bf16 param + int16 rounding error.

The fp32 master loses its lowest mantissa bit (round to nearest even); the
remaining 31 bits are the bf16 param plus a signed 15-bit correction.  Per
element: 10 bytes read, 8 written: 18 bytes of HBM traffic.
"""

import torch

from .. import _lib
from . import _common


def _step_with_rounding_error(fn_name, params, states, scalars, clip_coef):
    n = params.numel()
    dev = params.device
    assert params.dtype == torch.bfloat16, "params must be bfloat16"
    _common.check_tensor(params, "params", torch.bfloat16, n, dev)
    _common.check_tensor(states["grad"], "states['grad']", torch.bfloat16, n, dev)
    _common.check_tensor(states["exp_avg"], "states['exp_avg']", torch.bfloat16, n, dev)
    _common.check_tensor(
        states["exp_avg_sq"], "states['exp_avg_sq']", torch.bfloat16, n, dev
    )
    _common.check_tensor(
        states["rounding_error"], "states['rounding_error']", torch.int16, n, dev
    )
    _common.check_clip(clip_coef, dev)
    if n == 0:
        return
    _common.launch(
        fn_name,
        params,
        [
            _lib.ptr(params),
            _lib.ptr(states["grad"]),
            _lib.ptr(states["exp_avg"]),
            _lib.ptr(states["exp_avg_sq"]),
            _lib.ptr(states["rounding_error"]),
        ],
        scalars + [_lib.ptr(clip_coef)],
    )


def adam_step_fp31_master(
    params,
    states,
    lr,
    weight_decay,
    beta1,
    beta2,
    eps,
    step,
    decoupled_weight_decay=False,
    BLOCK_SIZE=1024,
    *,
    clip_coef=None,
):
    """Same call as the reference's ``adam_step_fp31_master``
    (src/offload_adam/kernels/fp31_master.py:103-136); asserts bf16 params like
    it does (fp31_master.py:115)."""
    _step_with_rounding_error(
        "oa_adam_fp31_master",
        params,
        states,
        _common.scalar_args(
            params, lr, weight_decay, beta1, beta2, eps, step, decoupled_weight_decay
        ),
        clip_coef,
    )
