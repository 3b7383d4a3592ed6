"""One call that steps a whole list of parameters (multi-tensor launch).

Equivalent to calling the mode's ``adam_step_*`` once per parameter - same
arithmetic, bit-identical results - but the per-parameter Python and launch
overhead is paid once per 36 parameters, and consecutive tensors share a grid
so the GPU does not drain between them.
"""

import random
from ctypes import c_float, c_int, c_void_p

import numpy as np
import torch

from .. import _lib
from . import _common

MULTI_MAX = 36  # parameters per launch (their descriptors fit the kernel arguments)

MODE_CODES = {
    "fp32_master": 0,
    "stochastic_rounding": 1,
    "fp31_master": 2,
    "fp32_master_custom_rounding": 3,
}
_AUX_KEY = {
    "fp32_master": ("master_params", torch.float32),
    "stochastic_rounding": (None, None),
    "fp31_master": ("rounding_error", torch.int16),
    "fp32_master_custom_rounding": ("rounding_error", torch.int16),
}


def _ptr_table(tensors):
    return np.fromiter((t.data_ptr() for t in tensors), dtype=np.uint64, count=len(tensors))


def adam_step_multi(
    mode,
    params,
    states,
    lr,
    weight_decay,
    beta1,
    beta2,
    eps,
    steps,
    decoupled_weight_decay=False,
    *,
    seeds=None,
    rng=None,
    clip_coef=None,
    validate=True,
):
    """Step every ``params[i]`` with ``states[i]`` (dicts with the keys the
    single-tensor step functions use).

    ``steps`` is one int or a list with the step count of each parameter.
    ``seeds`` (stochastic rounding): list of ints, or None to draw
    ``random.getrandbits(64)`` per parameter like the reference does per call;
    ``rng`` defaults to ``"x8"`` without seeds and ``"triton"`` with seeds.
    """
    if mode not in MODE_CODES:
        raise ValueError(f"Invalid mode: {mode}")
    count = len(params)
    if count == 0:
        return
    if len(states) != count:
        raise ValueError("params and states must have the same length")
    dev = params[0].device
    aux_key, aux_dtype = _AUX_KEY[mode]
    if validate:
        for p, st in zip(params, states):
            n = p.numel()
            if mode != "fp32_master" or p is not st["grad"]:
                _common.check_tensor(p, "params", torch.bfloat16, n, dev)
            for key in ("grad", "exp_avg", "exp_avg_sq"):
                _common.check_tensor(st[key], f"states['{key}']", torch.bfloat16, n, dev)
            if aux_key is not None:
                _common.check_tensor(st[aux_key], f"states['{aux_key}']", aux_dtype, n, dev)
        _common.check_clip(clip_coef, dev)

    if isinstance(steps, int):
        b1h, b2h = _common.folded_betas(beta1, beta2, steps)
        b1 = np.full(count, b1h, dtype=np.float32)
        b2 = np.full(count, b2h, dtype=np.float32)
    else:
        pairs = [_common.folded_betas(beta1, beta2, s) for s in steps]
        b1 = np.array([a for a, _ in pairs], dtype=np.float32)
        b2 = np.array([b for _, b in pairs], dtype=np.float32)

    seed_tab = None
    rng_code = _lib.OA_RNG_X8
    if mode == "stochastic_rounding":
        if rng is None:
            rng = "x8" if seeds is None else "triton"
        if rng not in ("x8", "triton"):
            raise ValueError("rng must be 'x8' or 'triton' for the multi-tensor step")
        rng_code = _lib.OA_RNG_X8 if rng == "x8" else _lib.OA_RNG_TRITON
        if seeds is None:
            seeds = [random.getrandbits(64) for _ in range(count)]
        seed_tab = np.array([s & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64)

    p_tab = _ptr_table(params)
    g_tab = _ptr_table([st["grad"] for st in states])
    m_tab = _ptr_table([st["exp_avg"] for st in states])
    v_tab = _ptr_table([st["exp_avg_sq"] for st in states])
    a_tab = _ptr_table([st[aux_key] for st in states]) if aux_key is not None else None
    n_tab = np.fromiter((p.numel() for p in params), dtype=np.int64, count=count)

    def addr(a):
        return c_void_p(a.ctypes.data) if a is not None else c_void_p(None)

    lib = _lib.load()
    with _lib.device_guard(dev):
        code = lib.oa_adam_multi(
            c_int(MODE_CODES[mode]), c_int(count), addr(p_tab), addr(g_tab), addr(m_tab),
            addr(v_tab), addr(a_tab), addr(n_tab), addr(b1), addr(b2), addr(seed_tab),
            c_float(lr), c_float(weight_decay), c_float(eps),
            c_int(1 if decoupled_weight_decay else 0), c_int(rng_code), _lib.ptr(clip_coef),
            _lib.current_stream_ptr(),
        )
    _lib.check(code, "oa_adam_multi")
