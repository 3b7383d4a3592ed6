"""ctypes binding of liboffload_adam_hip.so (the C ABI in include/offload_adam_hip.h).

The library is loaded lazily on first use.  There is no fallback: if the
shared object has not been built, every operator raises.
"""

import contextlib
import ctypes
import os
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint64, c_void_p
from pathlib import Path

# OFFLOAD_ADAM_HIP_LIB points at another build of the same library (kernel tuning).
LIB_PATH = Path(os.environ.get("OFFLOAD_ADAM_HIP_LIB")
                or Path(__file__).resolve().parent / "liboffload_adam_hip.so")

OA_RNG_TRITON = 0
OA_RNG_X8 = 1
OA_RNG_BUFFER = 2

_ADAM_TAIL = [c_int64, c_float, c_float, c_float, c_float, c_float, c_int]

# name -> (restype, argtypes); every symbol include/offload_adam_hip.h declares.
SIGNATURES = {
    "oa_abi_version": (c_int, []),
    "oa_error_string": (c_char_p, [c_int]),
    "oa_adam_fp32_master": (
        c_int,
        [c_void_p] * 5 + _ADAM_TAIL + [c_void_p, c_void_p],
    ),
    "oa_adam_stochastic_rounding": (
        c_int,
        [c_void_p] * 4 + _ADAM_TAIL + [c_uint64, c_int, c_void_p, c_void_p, c_void_p],
    ),
    "oa_adam_fp31_master": (
        c_int,
        [c_void_p] * 5 + _ADAM_TAIL + [c_void_p, c_void_p],
    ),
    "oa_adam_fp32_master_custom_rounding": (
        c_int,
        [c_void_p] * 5 + _ADAM_TAIL + [c_void_p, c_void_p],
    ),
    # mode, count, 5 pointer tables, numels, beta1_hats, beta2_hats, seeds,
    # lr, wd, eps, decoupled, rng, clip_coef, stream
    "oa_adam_multi": (
        c_int,
        [c_int, c_int] + [c_void_p] * 9 + [c_float, c_float, c_float, c_int, c_int, c_void_p,
                                           c_void_p],
    ),
    "oa_norm_workspace_bytes": (c_size_t, []),
    "oa_grad_norm_bf16": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    # grad, n, norm_out, sumsq_out, stream
    "oa_grad_norm_bf16_static": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "oa_norm_multi_workspace_bytes": (c_size_t, []),
    # count, grads, numels, norm_outs, sumsq_outs, workspace, workspace_bytes, stream
    "oa_grad_norm_multi": (
        c_int,
        [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "oa_clip_coef_bf16": (
        c_int,
        [c_void_p, c_int64, c_float, c_void_p, c_void_p, c_void_p],
    ),
    # src, src_dtype, stride, rows, cols, q, scales, scale_dtype, stream
    "oa_quant_int8": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p],
    ),
    # q, scales, scale_dtype, rows, cols, out, out_dtype, out_stride, stream
    "oa_dequant_int8": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p],
    ),
    "oa_quant_int4": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int,
         c_void_p],
    ),
    "oa_dequant_int4": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64,
         c_void_p],
    ),
    "oa_quant_nf4": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "oa_dequant_nf4": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p],
    ),
    "oa_quant_nvfp4": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p],
    ),
    "oa_dequant_nvfp4": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p],
    ),
    "oa_adam_requant_int8": (
        c_int,
        [c_void_p] * 4 + [c_int64] + _ADAM_TAIL + [c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "oa_adam_requant_int4": (
        c_int,
        [c_void_p] * 4 + [c_int64] + _ADAM_TAIL
        + [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "oa_adam_requant_nf4": (
        c_int,
        [c_void_p] * 4 + [c_int64] + _ADAM_TAIL + [c_void_p, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "oa_adam_requant_nvfp4": (
        c_int,
        [c_void_p] * 4 + [c_int64] + _ADAM_TAIL
        + [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "oa_pinned_alloc": (
        c_int,
        [c_size_t, c_int, ctypes.POINTER(c_void_p), ctypes.POINTER(c_int)],
    ),
    "oa_pinned_free": (c_int, [c_void_p]),
    "oa_pinned_probe": (c_int, [c_size_t]),
    "oa_gpu_numa_node": (c_int, [c_int, ctypes.POINTER(c_int)]),
    "oa_memcpy_async": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "oa_copy_kernel_async": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    # dst, src, bytes, stream, wait_event, record_event
    "oa_h2d_async": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]),
    "oa_d2h_async": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]),
    # count, dsts, srcs, bytes, kind, stream, record_events
    "oa_link_copy_batch": (c_int, [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                   c_void_p]),
    "oa_link_wait_limit": (c_int, [ctypes.c_ulonglong, c_int]),
    "oa_link_copy_status": (
        c_int,
        [ctypes.POINTER(ctypes.c_uint), ctypes.POINTER(ctypes.c_uint),
         ctypes.POINTER(ctypes.c_ulonglong), ctypes.POINTER(ctypes.c_ulonglong),
         ctypes.POINTER(ctypes.c_ulonglong)],
    ),
}

OA_EOS = -5
OA_EUNAVAILABLE = -6
OA_COPY_H2D, OA_COPY_D2H, OA_COPY_D2D = 0, 1, 2
OA_F32, OA_BF16, OA_F16 = 0, 1, 2


def dtype_code(dtype):
    """torch float dtype -> OA_* element-type code of the C ABI."""
    import torch

    try:
        return {torch.float32: OA_F32, torch.bfloat16: OA_BF16, torch.float16: OA_F16}[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16")

_lib = None
_lock = threading.Lock()


class LibraryNotBuiltError(RuntimeError):
    pass


def load():
    """Return the loaded library (thread-safe; hooks call from the autograd thread)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise LibraryNotBuiltError(
                f"{LIB_PATH} is missing. Build it with "
                "`python -m offload_adam_amd._build` (needs ROCm hipcc); there is "
                "no CPU or PyTorch fallback for the optimizer kernels."
            )
        lib = ctypes.CDLL(str(LIB_PATH), mode=ctypes.RTLD_LOCAL)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        built = lib.oa_abi_version()
        if built != 1:
            raise RuntimeError(f"{LIB_PATH} has ABI version {built}, expected 1")
        _lib = lib
    return _lib


def error_string(code):
    return load().oa_error_string(code).decode()


def check(code, what):
    """Raise RuntimeError for a non-zero return code of an entry point."""
    if code != 0:
        raise RuntimeError(f"{what} failed with code {code}: {error_string(code)}")


_NO_GUARD = contextlib.nullcontext()


def device_guard(device):
    """Context that makes ``device`` the current GPU; free when it already is
    (``torch.cuda.device`` costs several microseconds per launch otherwise)."""
    import torch

    index = device.index
    if index is None or index == torch._C._cuda_getDevice():
        return _NO_GUARD
    return torch.cuda.device(device)


def current_stream_id():
    """Raw handle (an int) of the calling thread's current stream on the current
    GPU, without building a ``torch.cuda.Stream`` object."""
    import torch

    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def current_stream_ptr():
    return c_void_p(current_stream_id())


def ptr(t):
    """Device/host address of a tensor's first element, or NULL for None."""
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(None)
