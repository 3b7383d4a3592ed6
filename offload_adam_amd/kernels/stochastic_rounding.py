"""AdamW step on bf16 params with stochastic rounding of the written param.

Per element: param, grad, exp_avg, exp_avg_sq read (8 bytes), param and both
moments written (6 bytes): 14 bytes of HBM traffic.
"""

import random
from ctypes import c_int, c_uint64

import torch

from .. import _lib
from . import _common

_RNG_CODES = {
    "triton": _lib.OA_RNG_TRITON,
    "x8": _lib.OA_RNG_X8,
    "buffer": _lib.OA_RNG_BUFFER,
}


def adam_step_stochastic_rounding(
    params,
    states,
    lr,
    weight_decay,
    beta1,
    beta2,
    eps,
    step,
    seed=None,
    decoupled_weight_decay=False,
    BLOCK_SIZE=1024,
    *,
    clip_coef=None,
    rng=None,
    rand16=None,
):
    """Same call as the reference's ``adam_step_stochastic_rounding``
    (src/offload_adam/kernels/stochastic_rounding.py:82-116).

    ``seed=None`` draws ``random.getrandbits(64)`` like the reference
    (stochastic_rounding.py:98-99).  ``rng`` picks where the 16 random bits of
    each element come from:

    * ``"triton"`` - element ``i`` gets the bits ``tl.randint(seed, i) & 0xFFFF``
      would give; with the same ``seed`` the result is bit-identical to the
      reference kernel.  Default when a ``seed`` is passed.
    * ``"x8"`` - one Philox4x32-10 block feeds 8 consecutive elements (an eighth
      of the integer work).  Default when ``seed`` is None, where the bits are
      fresh on every call and the layout cannot be observed.
    * ``"buffer"`` - element ``i`` uses ``rand16[i]`` (int16/uint16 GPU tensor).
    """
    n = params.numel()
    dev = params.device
    _common.check_tensor(params, "params", torch.bfloat16, n, dev)
    _common.check_tensor(states["grad"], "states['grad']", torch.bfloat16, n, dev)
    _common.check_tensor(states["exp_avg"], "states['exp_avg']", torch.bfloat16, n, dev)
    _common.check_tensor(
        states["exp_avg_sq"], "states['exp_avg_sq']", torch.bfloat16, n, dev
    )
    _common.check_clip(clip_coef, dev)
    if rng is None:
        rng = "buffer" if rand16 is not None else ("x8" if seed is None else "triton")
    if rng not in _RNG_CODES:
        raise ValueError(f"rng must be one of {sorted(_RNG_CODES)} (got {rng!r})")
    if rng == "buffer":
        if rand16 is None:
            raise ValueError("rng='buffer' needs rand16")
        if rand16.dtype not in (torch.int16, torch.uint16):
            raise TypeError(f"rand16 must be int16 or uint16, got {rand16.dtype}")
        _common.check_tensor(rand16, "rand16", rand16.dtype, n, dev)
    if seed is None:
        seed = random.getrandbits(64)
    if n == 0:
        return
    _common.launch(
        "oa_adam_stochastic_rounding",
        params,
        [
            _lib.ptr(params),
            _lib.ptr(states["grad"]),
            _lib.ptr(states["exp_avg"]),
            _lib.ptr(states["exp_avg_sq"]),
        ],
        _common.scalar_args(
            params, lr, weight_decay, beta1, beta2, eps, step, decoupled_weight_decay
        )
        + [
            c_uint64(seed & 0xFFFFFFFFFFFFFFFF),
            c_int(_RNG_CODES[rng]),
            _lib.ptr(rand16 if rng == "buffer" else None),
            _lib.ptr(clip_coef),
        ],
    )
