"""AdamW step on an fp32 master copy (bf16 moments, bf16 param written out).

Per element: grad 2 + exp_avg 2 + exp_avg_sq 2 + master 4 bytes read, the same
plus the bf16 param written: 20 bytes of HBM traffic.
"""

import torch

from .. import _lib
from . import _common


def adam_step_fp32_master(
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
    """Same call as the reference's ``adam_step_fp32_master``
    (src/offload_adam/kernels/fp32_master.py:62-94): mutates ``params`` (written
    only), ``states['exp_avg']``, ``states['exp_avg_sq']`` and
    ``states['master_params']`` in place on the current stream.  ``BLOCK_SIZE``
    is accepted and ignored.  Unlike the reference it does not synchronize the
    device.  ``clip_coef`` (optional 0-dim bf16 GPU tensor) scales the gradient
    inside the kernel with the rounding of ``grad.mul_(clip_coef)``.

    Two further forms of ``params``: ``None`` writes no bf16 copy at all, and a
    quantised weight (``QWeightBase``) gets its payload re-encoded from the new
    master - what the reference does with the gradient buffer as a throw-away
    sink followed by ``p.data.copy_(master)`` (offload_adam.py:427-444) - in
    the same pass when the layout allows, in a second launch otherwise.
    """
    from ..qweight.base import QWeightBase

    if isinstance(params, QWeightBase):
        from .qat_step import adam_step_requant

        if params.is_cuda and adam_step_requant(
                params, states, lr, weight_decay, beta1, beta2, eps, step,
                decoupled_weight_decay, clip_coef):
            return
        adam_step_fp32_master(None, states, lr, weight_decay, beta1, beta2, eps, step,
                              decoupled_weight_decay, clip_coef=clip_coef)
        params.copy_(states["master_params"])
        return
    master = states["master_params"]
    n = master.numel()
    dev = master.device
    if params is not None:
        _common.check_tensor(params, "params", torch.bfloat16, n, dev)
    _common.check_tensor(states["grad"], "states['grad']", torch.bfloat16, n, dev)
    _common.check_tensor(states["exp_avg"], "states['exp_avg']", torch.bfloat16, n, dev)
    _common.check_tensor(
        states["exp_avg_sq"], "states['exp_avg_sq']", torch.bfloat16, n, dev
    )
    _common.check_tensor(
        states["master_params"], "states['master_params']", torch.float32, n, dev
    )
    _common.check_clip(clip_coef, dev)
    if n == 0:
        return
    _common.launch(
        "oa_adam_fp32_master",
        master,
        [
            _lib.ptr(params),
            _lib.ptr(states["grad"]),
            _lib.ptr(states["exp_avg"]),
            _lib.ptr(states["exp_avg_sq"]),
            _lib.ptr(states["master_params"]),
        ],
        _common.scalar_args(
            master, lr, weight_decay, beta1, beta2, eps, step, decoupled_weight_decay
        )
        + [_lib.ptr(clip_coef)],
    )
