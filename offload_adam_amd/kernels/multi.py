"""One call that steps a whole list of parameters (multi-tensor launch).

Equivalent to calling the mode's ``adam_step_*`` once per parameter - same
arithmetic, bit-identical results - but the per-parameter Python and launch
overhead is paid once per 36 parameters, and consecutive tensors share a grid
so the GPU does not drain between them.
"""

import random
from ctypes import c_float, c_int, c_int64, c_uint64

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
    """Addresses as a C array (plain ctypes: no numpy round trip per launch)."""
    return (c_uint64 * len(tensors))(*[t.data_ptr() for t in tensors])


def _float_table(values):
    return (c_float * len(values))(*values)


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
        b1 = _float_table([b1h] * count)
        b2 = _float_table([b2h] * count)
    else:
        folded = {}
        for step in steps:
            if step not in folded:
                folded[step] = _common.folded_betas(beta1, beta2, step)
        b1 = _float_table([folded[step][0] for step in steps])
        b2 = _float_table([folded[step][1] for step in steps])

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
        seed_tab = (c_uint64 * count)(*[s & 0xFFFFFFFFFFFFFFFF for s in seeds])

    p_tab = _ptr_table(params)
    g_tab = _ptr_table([st["grad"] for st in states])
    m_tab = _ptr_table([st["exp_avg"] for st in states])
    v_tab = _ptr_table([st["exp_avg_sq"] for st in states])
    a_tab = _ptr_table([st[aux_key] for st in states]) if aux_key is not None else None
    n_tab = (c_int64 * count)(*[p.numel() for p in params])

    lib = _lib.load()
    with _lib.device_guard(dev):
        code = lib.oa_adam_multi(
            c_int(MODE_CODES[mode]), c_int(count), p_tab, g_tab, m_tab,
            v_tab, a_tab, n_tab, b1, b2, seed_tab,
            c_float(lr), c_float(weight_decay), c_float(eps),
            c_int(1 if decoupled_weight_decay else 0), c_int(rng_code), _lib.ptr(clip_coef),
            _lib.current_stream_ptr(),
        )
    _lib.check(code, "oa_adam_multi")
