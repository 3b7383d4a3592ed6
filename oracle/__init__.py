"""CPU oracle of the optimizer hot path -- TEST INFRASTRUCTURE ONLY.

``oa_oracle.c`` restates the reference's algorithms as scalar C; this module
binds it with ctypes over numpy arrays (bf16 / fp16 travel as ``uint16`` bit
patterns).  ``torch_eager.py`` holds a second, independent restatement in
PyTorch eager ops, used as the CPU baseline of the benchmark.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline
leg may import this package.  The shipped package ``offload_adam_amd`` never
does.
"""

import ctypes
import subprocess
from ctypes import (
    POINTER,
    c_double,
    c_float,
    c_int,
    c_int16,
    c_int64,
    c_uint8,
    c_uint16,
    c_uint32,
    c_uint64,
    c_void_p,
)
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "liboa_oracle.so"

_lib = None


def build(force=False):
    """Compile oa_oracle.c with gcc (oracle/Makefile)."""
    if force and LIB_PATH.exists():
        LIB_PATH.unlink()
    subprocess.run(["make", "-s", "-C", str(ORACLE_DIR)], check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        L = ctypes.CDLL(str(LIB_PATH))
        u16p, i16p, f32p = POINTER(c_uint16), POINTER(c_int16), POINTER(c_float)
        hyp = [c_int64, c_float, c_float, c_float, c_float, c_float, c_int]
        sigs = {
            "oaref_bf16_to_f32": (c_float, [c_uint16]),
            "oaref_f32_to_bf16": (c_uint16, [c_float]),
            "oaref_f32_to_f16": (c_uint16, [c_float]),
            "oaref_f16_to_f32": (c_float, [c_uint16]),
            "oaref_philox4x32_10": (None, [POINTER(c_uint32)] * 3),
            "oaref_triton_randint": (c_uint32, [c_uint64, c_int64]),
            "oaref_rand16": (c_uint32, [c_uint64, c_int64, c_int]),
            "oaref_sr_round": (c_uint16, [c_float, c_uint32]),
            "oaref_round_to_fp31": (c_uint32, [c_uint32]),
            "oaref_fp31_decompose": (None, [c_float, u16p, i16p]),
            "oaref_fp31_reconstruct": (c_float, [c_uint16, c_int16]),
            "oaref_custom_decompose": (None, [c_float, u16p, i16p]),
            "oaref_custom_reconstruct": (c_float, [c_uint16, c_int16]),
            "oaref_adam_fp32_master": (None, [c_void_p] * 5 + hyp + [c_void_p]),
            "oaref_adam_stochastic_rounding": (
                None,
                [c_void_p] * 4 + hyp + [c_uint64, c_int, c_void_p, c_void_p],
            ),
            "oaref_adam_fp31_master": (None, [c_void_p] * 5 + hyp + [c_void_p]),
            "oaref_adam_custom_rounding": (None, [c_void_p] * 5 + hyp + [c_void_p]),
            "oaref_grad_norm_bf16": (c_uint16, [c_void_p, c_int64]),
            "oaref_sumsq_f64": (c_double, [c_void_p, c_int64]),
            "oaref_total_norm_bf16": (c_uint16, [c_void_p, c_int64]),
            "oaref_clip_coef_bf16": (c_uint16, [c_uint16, c_float]),
            "oaref_quant_int8": (None, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
            "oaref_dequant_int8": (
                None,
                [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int],
            ),
            "oaref_quant_int4": (
                None,
                [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p],
            ),
            "oaref_dequant_int4": (
                None,
                [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int],
            ),
            "oaref_nf4_lut": (c_float, [c_int]),
            "oaref_quant_nf4": (
                None,
                [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p],
            ),
            "oaref_dequant_nf4": (
                None,
                [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int],
            ),
            "oaref_fp4_lut": (c_float, [c_int]),
            "oaref_f32_to_e4m3fn": (c_uint8, [c_float]),
            "oaref_e4m3fn_to_f32": (c_float, [c_uint8]),
            "oaref_fp4_e2m1_code": (c_uint8, [c_float]),
            "oaref_nvfp4_global_scale": (c_float, [c_void_p, c_int64]),
            "oaref_quant_nvfp4": (
                c_float,
                [c_void_p, c_int64, c_int64, c_void_p, c_void_p],
            ),
            "oaref_sr_round_array": (None, [c_void_p, c_void_p, c_int64, c_void_p]),
            "oaref_split_array": (
                None,
                [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p],
            ),
            "oaref_narrow_array": (None, [c_void_p, c_int64, c_int, c_void_p]),
            "oaref_fp4_code_array": (None, [c_void_p, c_int64, c_void_p]),
            "oaref_rand16_array": (None, [c_uint64, c_int64, c_int64, c_int, c_void_p]),
            "oaref_dequant_nvfp4": (
                None,
                [c_void_p, c_void_p, c_float, c_int64, c_int64, c_void_p, c_int],
            ),
        }
        for name, (res, args) in sigs.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


# ----------------------------------------------------------------- helpers

OUT_DTYPES = {"float32": 0, "bfloat16": 1, "float16": 2}


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(c_void_p)


def _req(a, dtype):
    assert a.dtype == dtype, f"expected {dtype}, got {a.dtype}"
    assert a.flags["C_CONTIGUOUS"]
    return a


def to_bits(t):
    """torch bf16/fp16 tensor -> numpy uint16 bit patterns (copy)."""
    import torch

    assert t.dtype in (torch.bfloat16, torch.float16)
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def from_bits(a, dtype):
    """numpy uint16 bit patterns -> torch tensor of ``dtype`` (bf16 / fp16)."""
    import torch

    return torch.from_numpy(a.view(np.int16).copy()).view(dtype)


def folded_betas(beta1, beta2, step):
    """(beta^t - beta)/(beta^t - 1) in double (kernels/fp32_master.py:74-75)."""
    b1 = (beta1**step - beta1) / (beta1**step - 1)
    b2 = (beta2**step - beta2) / (beta2**step - 1)
    return b1, b2


def _clip_arr(clip):
    if clip is None:
        return None
    return np.array([clip], dtype=np.uint16)


# -------------------------------------------------------------------- Adam


def adam_fp32_master(p_out, g, m, v, master, lr, wd, b1h, b2h, eps, decoupled, clip=None):
    """In place on numpy arrays; ``clip`` = bf16 bits of the clip coefficient."""
    n = g.size
    c = _clip_arr(clip)
    lib().oaref_adam_fp32_master(
        _p(_req(p_out, np.uint16)), _p(_req(g, np.uint16)), _p(_req(m, np.uint16)),
        _p(_req(v, np.uint16)), _p(_req(master, np.float32)), n, lr, wd, b1h, b2h, eps,
        int(decoupled), _p(c),
    )


def adam_stochastic_rounding(p, g, m, v, lr, wd, b1h, b2h, eps, decoupled, seed=0,
                             layout=0, rand16=None, clip=None):
    n = g.size
    c = _clip_arr(clip)
    if layout == 2:
        _req(rand16, np.uint16)
    lib().oaref_adam_stochastic_rounding(
        _p(_req(p, np.uint16)), _p(_req(g, np.uint16)), _p(_req(m, np.uint16)),
        _p(_req(v, np.uint16)), n, lr, wd, b1h, b2h, eps, int(decoupled),
        seed & 0xFFFFFFFFFFFFFFFF, layout, _p(rand16), _p(c),
    )


def adam_fp31_master(p, g, m, v, err, lr, wd, b1h, b2h, eps, decoupled, clip=None):
    n = g.size
    c = _clip_arr(clip)
    lib().oaref_adam_fp31_master(
        _p(_req(p, np.uint16)), _p(_req(g, np.uint16)), _p(_req(m, np.uint16)),
        _p(_req(v, np.uint16)), _p(_req(err, np.int16)), n, lr, wd, b1h, b2h, eps,
        int(decoupled), _p(c),
    )


def adam_custom_rounding(p, g, m, v, err, lr, wd, b1h, b2h, eps, decoupled, clip=None):
    n = g.size
    c = _clip_arr(clip)
    lib().oaref_adam_custom_rounding(
        _p(_req(p, np.uint16)), _p(_req(g, np.uint16)), _p(_req(m, np.uint16)),
        _p(_req(v, np.uint16)), _p(_req(err, np.int16)), n, lr, wd, b1h, b2h, eps,
        int(decoupled), _p(c),
    )


def philox(ctr, key):
    c = (c_uint32 * 4)(*ctr)
    k = (c_uint32 * 2)(*key)
    o = (c_uint32 * 4)()
    lib().oaref_philox4x32_10(c, k, o)
    return tuple(o)


def rand16_array(seed, n, layout, start=0):
    out = np.empty(n, dtype=np.uint16)
    lib().oaref_rand16_array(seed & 0xFFFFFFFFFFFFFFFF, start, n, layout, _p(out))
    return out


def sr_round_array(x_f32, r16):
    out = np.empty(x_f32.size, dtype=np.uint16)
    lib().oaref_sr_round_array(_p(_req(x_f32, np.float32)), _p(_req(r16, np.uint16)),
                               x_f32.size, _p(out))
    return out


def split_array(xbits, which):
    """which: 'fp31' or 'custom' -> (bf16 bits, int16 err, reconstructed fp32 bits)."""
    n = xbits.size
    p = np.empty(n, dtype=np.uint16)
    e = np.empty(n, dtype=np.int16)
    r = np.empty(n, dtype=np.uint32)
    lib().oaref_split_array(_p(_req(xbits, np.uint32)), n, 0 if which == "fp31" else 1,
                            _p(p), _p(e), _p(r))
    return p, e, r


def narrow_array(x_f32, kind):
    """kind: 'bfloat16' | 'float16' (uint16 bits) or 'e4m3fn' (uint8 bits)."""
    k = {"bfloat16": 0, "float16": 1, "e4m3fn": 2}[kind]
    out = np.empty(x_f32.size, dtype=np.uint8 if k == 2 else np.uint16)
    lib().oaref_narrow_array(_p(_req(x_f32, np.float32)), x_f32.size, k, _p(out))
    return out


def fp4_code_array(x_f32):
    out = np.empty(x_f32.size, dtype=np.uint8)
    lib().oaref_fp4_code_array(_p(_req(x_f32, np.float32)), x_f32.size, _p(out))
    return out


# ------------------------------------------------------------- norm / clip


def grad_norm_bf16(g):
    return lib().oaref_grad_norm_bf16(_p(_req(g, np.uint16)), g.size)


def sumsq_f64(g):
    return lib().oaref_sumsq_f64(_p(_req(g, np.uint16)), g.size)


def clip_coef_bf16(total_bits, max_norm):
    return lib().oaref_clip_coef_bf16(int(total_bits), float(max_norm))


# ------------------------------------------------------------------ codecs


def _out_buf(shape, out_dtype):
    return np.empty(shape, dtype=np.float32 if out_dtype == "float32" else np.uint16)


def quant_int8(x):
    x = _req(np.ascontiguousarray(x, dtype=np.float32), np.float32)
    rows, cols = x.shape
    q = np.empty((rows, cols), dtype=np.int8)
    s = np.empty((rows,), dtype=np.float32)
    lib().oaref_quant_int8(_p(x), rows, cols, _p(q), _p(s))
    return q, s


def dequant_int8(q, scale_f32, out_dtype="bfloat16"):
    rows, cols = q.shape
    out = _out_buf((rows, cols), out_dtype)
    lib().oaref_dequant_int8(_p(_req(q, np.int8)), _p(_req(scale_f32, np.float32)), rows,
                             cols, _p(out), OUT_DTYPES[out_dtype])
    return out


def quant_int4(x, group=128):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    assert cols % group == 0 and cols % 8 == 0 and group % 8 == 0
    qw = np.empty((cols // 8, rows), dtype=np.int32)
    s = np.empty((cols // group, rows), dtype=np.float32)
    lib().oaref_quant_int4(_p(x), rows, cols, group, _p(qw), _p(s))
    return qw, s


def dequant_int4(qw, scale_f32, group=128, out_dtype="bfloat16"):
    rows = qw.shape[1]
    cols = qw.shape[0] * 8
    out = _out_buf((rows, cols), out_dtype)
    lib().oaref_dequant_int4(_p(_req(qw, np.int32)), _p(_req(scale_f32, np.float32)), rows,
                             cols, group, _p(out), OUT_DTYPES[out_dtype])
    return out


def quant_nf4(x, block=64):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    assert cols % block == 0 and block % 2 == 0
    packed = np.empty((rows, cols // 2), dtype=np.uint8)
    absmax = np.empty((rows * (cols // block),), dtype=np.float32)
    lib().oaref_quant_nf4(_p(x), rows, cols, block, _p(packed), _p(absmax))
    return packed, absmax


def dequant_nf4(packed, absmax, block=64, out_dtype="bfloat16"):
    rows = packed.shape[0]
    cols = packed.shape[1] * 2
    out = _out_buf((rows, cols), out_dtype)
    lib().oaref_dequant_nf4(_p(_req(packed, np.uint8)), _p(_req(absmax, np.float32)), rows,
                            cols, block, _p(out), OUT_DTYPES[out_dtype])
    return out


def quant_nvfp4(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, cols = x.shape
    assert cols % 16 == 0
    packed = np.empty((rows, cols // 2), dtype=np.uint8)
    scale8 = np.empty((rows, cols // 16), dtype=np.uint8)
    gs = lib().oaref_quant_nvfp4(_p(x), rows, cols, _p(packed), _p(scale8))
    return packed, scale8, np.float32(gs)


def dequant_nvfp4(packed, scale8, gs, out_dtype="bfloat16"):
    rows = packed.shape[0]
    cols = packed.shape[1] * 2
    out = _out_buf((rows, cols), out_dtype)
    lib().oaref_dequant_nvfp4(_p(_req(packed, np.uint8)), _p(_req(scale8, np.uint8)),
                              float(gs), rows, cols, _p(out), OUT_DTYPES[out_dtype])
    return out
