"""Fused AdamW step functions backed by hand-written HIP kernels (gfx950).

``STEP_FUNCTIONS`` maps each optimizer mode string to its step function;
``adam_step_multi`` steps many tensors with one launch per 36 of them.
"""

from . import fp31_master, fp32_master, fp32_master_custom_rounding, multi, stochastic_rounding

adam_step_fp32_master = fp32_master.adam_step_fp32_master
adam_step_stochastic_rounding = stochastic_rounding.adam_step_stochastic_rounding
adam_step_fp31_master = fp31_master.adam_step_fp31_master
adam_step_fp32_master_custom_rounding = (
    fp32_master_custom_rounding.adam_step_fp32_master_custom_rounding)
adam_step_multi = multi.adam_step_multi

STEP_FUNCTIONS = {
    "fp32_master": adam_step_fp32_master,
    "stochastic_rounding": adam_step_stochastic_rounding,
    "fp31_master": adam_step_fp31_master,
    "fp32_master_custom_rounding": adam_step_fp32_master_custom_rounding,
}

__all__ = [fn.__name__ for fn in STEP_FUNCTIONS.values()] + ["adam_step_multi", "STEP_FUNCTIONS"]
