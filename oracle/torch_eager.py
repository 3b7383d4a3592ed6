"""Second CPU restatement of the hot path, in PyTorch eager ops -- TEST
INFRASTRUCTURE ONLY (see oracle/__init__.py for who may import it).

Every fp32 expression is one eager op per arithmetic operation with 0-dim fp32
tensors for the scalars, so each step rounds once in binary32, as the
reference's Triton kernels do.  The tests require this module and the C oracle
to agree bit for bit; the benchmark times it as "the same update math in
PyTorch eager on the host cores".
"""

import torch

_F32 = torch.float32
_BF16 = torch.bfloat16


def _s(x):
    """Python float -> 0-dim fp32 tensor (the fp32 scalar a Triton kernel receives)."""
    return torch.tensor(float(x), dtype=_F32)


# -------------------------------------------------------------------- Adam


def _sqrt_rn(x):
    """Correctly rounded fp32 square root.  torch.sqrt on CPU goes through a
    vector math library that is allowed to be off by one ulp (measured: ~0.6 %
    of random inputs), numpy's maps to the IEEE sqrt instruction."""
    import numpy as np

    return torch.from_numpy(np.sqrt(x.numpy()))


def adam_core(M, g, m, v, lr, wd, b1h, b2h, eps, decoupled, exact_sqrt=True):
    """fp32 tensors -> (M', m', v').  kernels/fp32_master.py:46-53.
    ``exact_sqrt=False`` stays inside torch ops (benchmark timing only)."""
    lr_t, wd_t, eps_t, one = _s(lr), _s(wd), _s(eps), _s(1.0)
    if decoupled:
        M = M - (lr_t * wd_t) * M
    else:
        g = g + wd_t * M
    m = m + (one - _s(b1h)) * (g - m)
    v = v + (one - _s(b2h)) * (g * g - v)
    denom = (_sqrt_rn(v) if exact_sqrt else torch.sqrt(v)) + eps_t
    M = M - (lr_t * m) / denom
    return M, m, v


def _clipped(g_bf16, clip_coef):
    if clip_coef is None:
        return g_bf16.float()
    # grad.mul_(clip_coef) on bf16 tensors, offload_adam.py:450-451
    return (g_bf16 * clip_coef).float()


def adam_step_fp32_master(p, states, lr, wd, b1h, b2h, eps, decoupled, clip_coef=None):
    """In place on CPU tensors (bf16 p/grad/moments, fp32 master)."""
    M, m, v = adam_core(
        states["master_params"], _clipped(states["grad"], clip_coef),
        states["exp_avg"].float(), states["exp_avg_sq"].float(),
        lr, wd, b1h, b2h, eps, decoupled,
    )
    p.copy_(M.to(_BF16))
    states["exp_avg"].copy_(m.to(_BF16))
    states["exp_avg_sq"].copy_(v.to(_BF16))
    states["master_params"].copy_(M)


def sr_round(x_f32, rand16_i32):
    """kernels/stochastic_rounding.py:25-34 on an fp32 tensor and int32 draws."""
    bits = x_f32.view(torch.int32)
    frac = bits & 0xFFFF
    trunc = bits & -0x10000
    out = torch.where(rand16_i32 < frac, trunc + 0x10000, trunc)
    return out.view(_F32).to(_BF16)


def adam_step_stochastic_rounding(p, states, lr, wd, b1h, b2h, eps, decoupled, rand16,
                                  clip_coef=None):
    """``rand16``: int32 tensor of values in [0, 65535], one per element."""
    M, m, v = adam_core(
        p.float(), _clipped(states["grad"], clip_coef), states["exp_avg"].float(),
        states["exp_avg_sq"].float(), lr, wd, b1h, b2h, eps, decoupled,
    )
    states["exp_avg"].copy_(m.to(_BF16))
    states["exp_avg_sq"].copy_(v.to(_BF16))
    p.copy_(sr_round(M, rand16))


def fp31_round(x_f32):
    """kernels/fp31_master.py:26-34"""
    xi = x_f32.view(torch.int32)
    up = (xi & 1) & ((xi >> 1) & 1)
    return (((xi >> 1) + up) << 1).view(_F32)


def fp31_decompose(x_f32):
    """kernels/fp31_master.py:37-45 -> (bf16, int16)"""
    x31 = fp31_round(x_f32)
    b = x31.to(_BF16)
    err32 = x31.view(torch.int32) - b.float().view(torch.int32)
    return b, (err32 >> 1).to(torch.int16)


def fp31_reconstruct(p_bf16, err_i16):
    """kernels/fp31_master.py:48-54"""
    return (p_bf16.float().view(torch.int32) + (err_i16.to(torch.int32) << 1)).view(_F32)


def custom_decompose(x_f32):
    """kernels/fp32_master_custom_rounding.py:33-43"""
    xi = x_f32.view(torch.int32)
    b = ((xi + 0x8000) >> 16).to(torch.int16).view(_BF16)
    err = (xi - b.float().view(torch.int32)).to(torch.int16)
    return b, err


def custom_reconstruct(p_bf16, err_i16):
    """kernels/fp32_master_custom_rounding.py:46-54, error always applied."""
    return (p_bf16.float().view(torch.int32) + err_i16.to(torch.int32)).view(_F32)


def adam_step_fp31_master(p, states, lr, wd, b1h, b2h, eps, decoupled, clip_coef=None):
    M, m, v = adam_core(
        fp31_reconstruct(p, states["rounding_error"]), _clipped(states["grad"], clip_coef),
        states["exp_avg"].float(), states["exp_avg_sq"].float(), lr, wd, b1h, b2h, eps,
        decoupled,
    )
    states["exp_avg"].copy_(m.to(_BF16))
    states["exp_avg_sq"].copy_(v.to(_BF16))
    b, e = fp31_decompose(M)
    p.copy_(b)
    states["rounding_error"].copy_(e)


def adam_step_custom_rounding(p, states, lr, wd, b1h, b2h, eps, decoupled, clip_coef=None):
    M, m, v = adam_core(
        custom_reconstruct(p, states["rounding_error"]), _clipped(states["grad"], clip_coef),
        states["exp_avg"].float(), states["exp_avg_sq"].float(), lr, wd, b1h, b2h, eps,
        decoupled,
    )
    states["exp_avg"].copy_(m.to(_BF16))
    states["exp_avg_sq"].copy_(v.to(_BF16))
    b, e = custom_decompose(M)
    p.copy_(b)
    states["rounding_error"].copy_(e)


# ------------------------------------------------------------- norm / clip


def grad_norm(g_bf16):
    """offload_adam.py:504-505"""
    return torch.norm(g_bf16, 2.0)


def clip_coef(norms_bf16, max_grad_norm):
    """offload_adam.py:560-561 on a 1-D bf16 tensor of per-param norms."""
    total = torch.linalg.vector_norm(norms_bf16, 2.0)
    return torch.clamp(max_grad_norm / (total + 1e-6), max=1.0), total


# ------------------------------------------------------------------ codecs

NF4_CODEBOOK = (
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634,
    0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
    0.7229568362236023, 1.0,
)
E2M1_CODEBOOK = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
                 -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)


def quant_int8(x):
    """qweight/int8.py:30-49 -> (int8 (R,C), fp32 scale (R,))"""
    t = x.float()
    scale = t.abs().amax(dim=1) / 127.0
    inv = 1.0 / scale.clamp(min=1e-12)
    q = (t * inv[:, None]).round().clamp(-128, 127).to(torch.int8)
    return q, scale


def dequant_int8(q, scales):
    """qweight/int8.py:52-57: computed in the dtype of ``scales``"""
    return q.to(scales.dtype) * scales[:, None]


def quant_int4(x, group=128):
    """qweight/int4.py:30-48,61-92 -> (int32 (C/8,R), fp32 scale (C/group,R))"""
    R, C = x.shape
    t = x.float().reshape(R, C // group, group)
    scale = t.abs().amax(dim=-1) / 8
    inv = 1.0 / scale.clamp(min=1e-12)
    q = (t * inv[..., None]).round().clamp(-8, 7).to(torch.int32).reshape(R, C // 8, 8)
    word = torch.zeros(R, C // 8, dtype=torch.int32)
    for i in range(8):
        word |= (q[..., i] + 8) << (4 * i)
    return word.T.contiguous(), scale.T.contiguous()


def dequant_int4(qw, scales, group=128):
    """tests/test_int4.py:28-38: computed in the dtype of ``scales`` (G,R)"""
    K, R = qw.shape
    nib = torch.stack([(qw >> (4 * i)) & 0xF for i in range(8)], dim=-1)  # (K,R,8)
    sv = (nib - 8).permute(1, 0, 2).reshape(R, K * 8).to(scales.dtype)
    return (sv.reshape(R, -1, group) * scales.T[..., None]).reshape(R, K * 8)


def quant_nf4(x, block=64):
    """qweight/nf4.py:74-83,102-135 -> (uint8 (R,C/2), fp32 absmax (R*C/block,))"""
    R, C = x.shape
    t = x.float().reshape(R, C // block, block)
    absmax = t.abs().amax(dim=-1)
    nrm = t * (1.0 / absmax.clamp(min=1e-12))[..., None]
    book = torch.tensor(NF4_CODEBOOK, dtype=_F32)
    code = (nrm[..., None] - book).abs().argmin(dim=-1).to(torch.uint8).reshape(R, C)
    packed = (code[:, 0::2] << 4) | code[:, 1::2]
    return packed, absmax.reshape(-1)


def dequant_nf4(packed, absmax, block=64, dtype=_BF16):
    """tests/test_nf4.py:104-112 (fp32 gather and multiply, cast last)"""
    R, H = packed.shape
    code = torch.stack([(packed >> 4) & 0xF, packed & 0xF], dim=-1).reshape(R, 2 * H).long()
    vals = torch.tensor(NF4_CODEBOOK, dtype=_F32)[code].reshape(R, -1, block)
    return (vals * absmax.reshape(R, -1)[..., None]).reshape(R, 2 * H).to(dtype)


def e2m1_code(x):
    """qweight/nvfp4.py:100-130"""
    ax = x.abs()
    code = torch.zeros_like(ax, dtype=torch.uint8)
    for thr, strict, val in ((0.25, True, 1), (0.75, False, 2), (1.25, True, 3),
                             (1.75, False, 4), (2.5, True, 5), (3.5, False, 6),
                             (5.0, True, 7)):
        hit = (ax > thr) if strict else (ax >= thr)
        code = torch.where(hit, torch.tensor(val, dtype=torch.uint8), code)
    return code | (torch.signbit(x).to(torch.uint8) << 3)


def quant_nvfp4(x):
    """qweight/nvfp4.py:72-81,133-173 -> (uint8 (R,C/2), e4m3fn (R,C/16), fp32 ())"""
    R, C = x.shape
    t = x.float()
    gs = t.abs().amax().clamp(min=1e-12) / (448.0 * 6.0)
    tb = t.reshape(R, C // 16, 16)
    bs32 = tb.abs().amax(dim=-1).clamp(min=1e-12) / 6.0
    s8 = (bs32 * (1.0 / gs)).to(torch.float8_e4m3fn)
    eff = s8.float() * gs
    code = e2m1_code(tb * (1.0 / eff.clamp(min=1e-12))[..., None]).reshape(R, C)
    packed = (code[:, 1::2] << 4) | code[:, 0::2]
    return packed, s8, gs


def dequant_nvfp4(packed, s8, gs, dtype=_BF16):
    """qweight/nvfp4.py:176-191"""
    R, H = packed.shape
    code = torch.stack([packed & 0xF, (packed >> 4) & 0xF], dim=-1).reshape(R, 2 * H).long()
    vals = torch.tensor(E2M1_CODEBOOK, dtype=_F32)[code].reshape(R, -1, 16)
    eff = (s8.float() * gs).reshape(R, -1)
    return (vals * eff[..., None]).reshape(R, 2 * H).to(dtype)
