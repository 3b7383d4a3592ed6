"""Shared input builders for the parity tests (seeded, synthetic)."""

import numpy as np
import torch

BF16 = torch.bfloat16

HYP = dict(lr=1e-4, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, step=10)


def adam_inputs(n, seed, mode, device="cpu"):
    """bf16 param ~N(0,0.02), grad ~N(0,1e-3), exp_avg ~N(0,1e-4),
    exp_avg_sq = N(0,1e-3)^2, all stored bf16; fp32 master = param upcast;
    rounding_error random int16 in the range of its mode."""
    g = torch.Generator().manual_seed(seed)
    p = (torch.randn(n, generator=g) * 0.02).to(BF16)
    t = {
        "grad": (torch.randn(n, generator=g) * 1e-3).to(BF16),
        "exp_avg": (torch.randn(n, generator=g) * 1e-4).to(BF16),
        "exp_avg_sq": ((torch.randn(n, generator=g) * 1e-3) ** 2).to(BF16),
    }
    if mode == "fp32_master":
        # a master that is not exactly representable in bf16
        t["master_params"] = p.float() * (1 + torch.randn(n, generator=g) * 1e-3)
    elif mode == "fp31_master":
        t["rounding_error"] = torch.randint(-16384, 16385, (n,), generator=g).to(torch.int16)
    elif mode == "fp32_master_custom_rounding":
        t["rounding_error"] = torch.randint(-32768, 32768, (n,), generator=g).to(torch.int16)
    t = {k: v.to(device) for k, v in t.items()}
    return p.to(device), t


def special_values(n, seed):
    """bf16 bit patterns that stress the arithmetic: zeros, signed zeros,
    denormals, tiny/huge normals, mixed with ordinary values."""
    rng = np.random.default_rng(seed)
    pool = np.array(
        [0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x3F80, 0xBF80, 0x7F7F, 0xFF7F,
         0x3C00, 0x0100, 0x7000, 0x1000, 0x2000, 0x4000, 0x3A83, 0xBA83],
        dtype=np.uint16,
    )
    return pool[rng.integers(0, len(pool), size=n)]


def bits(t):
    """bf16/fp16/int16 tensor -> numpy uint16 copy of the bit patterns."""
    if t.dtype in (torch.bfloat16, torch.float16):
        t = t.view(torch.int16)
    return t.detach().cpu().contiguous().numpy().view(np.uint16).copy()


def from_bf16_bits(a, device="cpu"):
    return torch.from_numpy(a.view(np.int16).copy()).view(BF16).to(device)
