"""Per-parameter gradient L2 norms and the global clip coefficient on the GPU.

Stand-ins for the torch calls of the reference's clipping path
(src/offload_adam/offload_adam.py:504-505, 531-532, 553-561): one HIP launch
per norm (or two launches per 36 norms, ``grad_norms_``), one tiny launch for
the coefficient, no host synchronisation.
"""

from ctypes import c_float, c_int, c_int64, c_size_t, c_uint64

import torch

from . import _lib

_workspaces = {}


def _workspace(device, stream_id):
    """Zero-filled scratch for the norm kernel, one per (device, stream)."""
    key = (device.index, stream_id)
    ws = _workspaces.get(key)
    if ws is None:
        nbytes = _lib.load().oa_norm_workspace_bytes()
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def grad_norm_(grad, out):
    """Write ``bf16(||grad||_2)`` into the 0-dim (or 1-element) bf16 tensor ``out``.

    ``grad`` is a contiguous bf16 GPU tensor.  The sum of squares is accumulated
    in fp32 in a fixed order; the result is rounded to bf16 like
    ``torch.norm(grad, 2.0)`` on a bf16 tensor.
    """
    if grad.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise TypeError("grad_norm_ works on bfloat16 tensors")
    if not grad.is_cuda or out.device != grad.device:
        raise ValueError("grad and out must be on the same GPU")
    if not grad.is_contiguous() or out.numel() != 1:
        raise ValueError("grad must be contiguous and out must hold one element")
    lib = _lib.load()
    with _lib.device_guard(grad.device):
        stream = _lib.current_stream_id()
        ws = _workspace(grad.device, stream)
        code = lib.oa_grad_norm_bf16(
            _lib.ptr(grad), c_int64(grad.numel()), _lib.ptr(out), None, _lib.ptr(ws),
            _lib.c_void_p(stream),
        )
    _lib.check(code, "oa_grad_norm_bf16")
    return out


_multi_workspaces = {}
NORMS_PER_LAUNCH = 36  # gradients one pair of launches of ``grad_norms_`` takes


def grad_norms_(grads, outs, validate=True):
    """``grad_norm_(grads[i], outs[i])`` for every i, with two launches per 36
    gradients instead of one or two per gradient.  Same bits as the single calls.

    ``grads``: contiguous bf16 tensors on one GPU; ``outs``: one-element bf16
    tensors on that GPU (typically 0-dim views of one buffer of slots)."""
    count = len(grads)
    if len(outs) != count:
        raise ValueError("grads and outs must have the same length")
    if count == 0:
        return outs
    dev = grads[0].device
    for g, o in zip(grads, outs) if validate else ():
        if g.dtype != torch.bfloat16 or o.dtype != torch.bfloat16:
            raise TypeError("grad_norms_ works on bfloat16 tensors")
        if not g.is_cuda or g.device != dev or o.device != dev:
            raise ValueError("every gradient and output must be on the same GPU")
        if not g.is_contiguous() or o.numel() != 1:
            raise ValueError("gradients must be contiguous and outputs hold one element")
    lib = _lib.load()
    with _lib.device_guard(dev):
        stream = _lib.current_stream_id()
        key = (dev.index, stream)
        ws = _multi_workspaces.get(key)
        if ws is None:
            ws = torch.empty(lib.oa_norm_multi_workspace_bytes(), dtype=torch.uint8, device=dev)
            _multi_workspaces[key] = ws
        g_tab = (c_uint64 * count)(*[g.data_ptr() for g in grads])
        n_tab = (c_int64 * count)(*[g.numel() for g in grads])
        o_tab = (c_uint64 * count)(*[o.data_ptr() for o in outs])
        code = lib.oa_grad_norm_multi(c_int(count), g_tab, n_tab, o_tab, None, _lib.ptr(ws),
                                      c_size_t(ws.numel()), _lib.c_void_p(stream))
    _lib.check(code, "oa_grad_norm_multi")
    return outs


def grad_norm(grad):
    """``torch.norm(grad, 2.0)`` for a bf16 GPU tensor: a new 0-dim bf16 tensor."""
    out = torch.empty((), dtype=torch.bfloat16, device=grad.device)
    return grad_norm_(grad, out)


def clip_coef_(norms, max_grad_norm, coef_out, total_out=None):
    """``clamp(max_grad_norm / (||norms||_2 + 1e-6), max=1.0)`` as a bf16 scalar.

    ``norms`` is a contiguous 1-D bf16 GPU tensor of per-parameter norms.
    """
    if norms.dtype != torch.bfloat16 or coef_out.dtype != torch.bfloat16:
        raise TypeError("clip_coef_ works on bfloat16 tensors")
    if not norms.is_cuda or not norms.is_contiguous() or coef_out.numel() != 1:
        raise ValueError("norms must be a contiguous GPU tensor, coef_out one element")
    if total_out is not None and (total_out.dtype != torch.bfloat16 or total_out.numel() != 1):
        raise TypeError("total_out must be one bfloat16 element")
    lib = _lib.load()
    with _lib.device_guard(norms.device):
        code = lib.oa_clip_coef_bf16(
            _lib.ptr(norms), c_int64(norms.numel()), c_float(max_grad_norm),
            _lib.ptr(total_out), _lib.ptr(coef_out), _lib.current_stream_ptr(),
        )
    _lib.check(code, "oa_clip_coef_bf16")
    return coef_out
