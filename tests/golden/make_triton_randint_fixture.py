"""Writes tests/golden/triton_randint.npz from Triton's own ``tl.randint``.

The reference draws the random bits of its stochastic rounding with
``tl.randint(seed, offsets)`` (src/offload_adam/kernels/stochastic_rounding.py:77);
the arithmetic lives in Triton 3.6.0 (``triton/language/random.py:13-105``), the
version the reference pins.  That library is installed in the build container and
its interpreter (``TRITON_INTERPRET=1``) runs ``@triton.jit`` functions on the CPU
with numpy, so the words below come from the third-party implementation itself,
not from a restatement.  Nothing of the reference is imported.  Usage::

    python tests/golden/make_triton_randint_fixture.py

Stored per seed: the 32-bit words for offsets 0..4095 (int32 offsets, as the
reference's ``block_start + tl.arange(0, BLOCK_SIZE)`` produces), and for a set
of far offsets up to 2^31 - 1.
"""

import os

os.environ["TRITON_INTERPRET"] = "1"

from pathlib import Path  # noqa: E402

import numpy as np  # noqa: E402
import torch  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402

OUT = Path(__file__).resolve().parent / "triton_randint.npz"
SEEDS = [0, 1, 0x0123456789ABCDEF, 0xFFFFFFFFFFFFFFFF, 0x9E3779B97F4A7C15, 0x00000001_00000000]
FAR = [4096, 65535, 65536, 1 << 20, (1 << 24) - 1, 1 << 24, 16777215 + 2, (1 << 30) + 12345,
       (1 << 31) - 1024, (1 << 31) - 1]
BLOCK = 1024


@triton.jit
def randint_block(out_ptr, seed, start, BLOCK: tl.constexpr):
    offs = start + tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)  # int32, as in the reference
    tl.store(out_ptr + tl.program_id(0) * BLOCK + tl.arange(0, BLOCK), tl.randint(seed, offs))


@triton.jit
def randint_at(out_ptr, offs_ptr, seed, BLOCK: tl.constexpr):
    lane = tl.arange(0, BLOCK)
    offs = tl.load(offs_ptr + lane)  # int32 offsets
    tl.store(out_ptr + lane, tl.randint(seed, offs))


def main():
    assert triton.__version__.startswith("3.6."), triton.__version__
    arrays = {"seeds": np.array(SEEDS, dtype=np.uint64), "far_offsets": np.array(FAR, dtype=np.int64)}
    far = torch.zeros(16, dtype=torch.int32)
    far[: len(FAR)] = torch.tensor(FAR, dtype=torch.int64).to(torch.int32)
    for i, seed in enumerate(SEEDS):
        out = torch.zeros(4096, dtype=torch.int32)
        randint_block[(4096 // BLOCK,)](out, seed, 0, BLOCK=BLOCK)
        arrays[f"seed{i}_first4096"] = out.numpy().view(np.uint32).copy()
        out = torch.zeros(16, dtype=torch.int32)
        randint_at[(1,)](out, far, seed, BLOCK=16)
        arrays[f"seed{i}_far"] = out.numpy().view(np.uint32)[: len(FAR)].copy()
    np.savez_compressed(OUT, **arrays)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes), triton {triton.__version__}")


if __name__ == "__main__":
    main()
