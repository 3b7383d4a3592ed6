"""Fused AdamW step functions backed by hand-written HIP kernels (gfx950)."""

from .fp31_master import adam_step_fp31_master
from .fp32_master import adam_step_fp32_master
from .fp32_master_custom_rounding import adam_step_fp32_master_custom_rounding
from .multi import adam_step_multi
from .stochastic_rounding import adam_step_stochastic_rounding

__all__ = [
    "adam_step_fp32_master_custom_rounding",
    "adam_step_fp31_master",
    "adam_step_fp32_master",
    "adam_step_stochastic_rounding",
    "adam_step_multi",
]
