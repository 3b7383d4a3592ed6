"""AdamW step on a full fp32 master kept as bf16 param + int16 rounding error.

The bf16 param is the master rounded half-up in magnitude (bits + 0x8000, top
16 bits), which keeps the signed difference within int16, so the pair always
rebuilds the 32-bit master.  18 bytes of HBM traffic per element.
"""

from . import _common
from .fp31_master import _step_with_rounding_error


def adam_step_fp32_master_custom_rounding(
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
    """Same call as the reference's ``adam_step_fp32_master_custom_rounding``
    (src/offload_adam/kernels/fp32_master_custom_rounding.py:103-136).  The
    stored error is always applied on reconstruction: the reference's
    ``error_q != 0x8000`` guard (fp32_master_custom_rounding.py:48) compares an
    int16 with 32768 and can never be false."""
    _step_with_rounding_error(
        "oa_adam_fp32_master_custom_rounding",
        params,
        states,
        _common.scalar_args(
            params, lr, weight_decay, beta1, beta2, eps, step, decoupled_weight_decay
        ),
        clip_coef,
    )
