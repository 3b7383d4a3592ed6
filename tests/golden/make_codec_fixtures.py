"""Writes tests/golden/codec_fixtures.npz from the reference's pure-torch codec
functions, on the CPU.

Runs only where the reference checkout is present (``/root/reference`` or the
path in ``OFFLOAD_ADAM_REFERENCE``); the tests read the committed ``.npz`` and
never this script.  Usage::

    python tests/golden/make_codec_fixtures.py

What is called, all CPU / pure torch (no Triton kernel is launched):

* ``qweight/int8.py:30-57``   quantize_int8_per_channel, dequantize_int8_per_channel
* ``qweight/int4.py:30-92``   quantize_int4_groupwise, unpack_int4_gptq
* ``qweight/nf4.py:74-152``   quantize_nf4_blockwise, dequantize_nf4_blockwise, unpack_nf4
* ``qweight/nvfp4.py:72-191`` quantize_nvfp4_blockwise, dequantize_nvfp4_blockwise, unpack_fp4

Inputs: the seed-0 parity shapes of the reference's own tests
(``tests/test_int8.py:70-84``: ``manual_seed(0)``, ``randn * 0.05``), in bf16,
fp16 and fp32; the same with 1 % of the entries multiplied by 10; an all-zero
block; and, per format, a small tensor built so that scaled values fall exactly
on rounding ties and threshold boundaries.

Every array is stored as raw bits (uint16 for bf16/fp16, uint32 for fp32, uint8
for e4m3) so that no cast happens on load.
"""

import os
import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
OUT = HERE / "codec_fixtures.npz"
REFERENCE = Path(os.environ.get("OFFLOAD_ADAM_REFERENCE", "/root/reference"))

DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def bits(t):
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy().view(np.uint32)
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    return t.numpy()


def seeded(rows, cols, dtype, outliers=False):
    torch.manual_seed(0)
    w = torch.randn(rows, cols) * 0.05
    if outliers:
        mask = torch.rand(rows, cols) < 0.01
        w = torch.where(mask, w * 10, w)
        w[0] = 0.0            # an all-zero row: every block scale hits its floor
    return w.to(dtype)


def int8_ties():
    # row maximum 127 -> scale 1: the other entries are the codes' half-way points
    k = torch.arange(-128, 127, dtype=torch.float32) + 0.5
    row = torch.cat([k, torch.tensor([127.0])])
    return torch.stack([row, -row, row * 0.5, row * 2.0])


def int4_ties(group):
    # group maximum 8 -> scale 1: half-way points of the 16 codes, both clamps
    vals = torch.tensor([-8.0, -7.5, -6.5, -5.5, -4.5, -3.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5,
                         3.5, 4.5, 5.5, 6.5, 7.5, 8.0, 7.0, -0.0, 0.0, 0.25, -0.25, 7.49])
    row = torch.zeros(group)
    row[: len(vals)] = vals
    flipped = -row
    flipped[0] = 8.0  # +8 clamps to 7, and the group maximum stays 8
    return torch.stack([row, flipped, row * 0.125, row * 3.0])


def nf4_ties(lut, block):
    # block maximum 1 -> values are compared with the table directly; midpoints of
    # neighbouring entries and their fp32 neighbours on either side
    mids = (lut[:-1] + lut[1:]) * 0.5
    cand = torch.cat([mids, torch.nextafter(mids, torch.tensor(2.0)),
                      torch.nextafter(mids, torch.tensor(-2.0)), lut])
    rows = []
    for start in range(0, len(cand), block - 1):
        chunk = cand[start:start + block - 1]
        row = torch.zeros(block)
        row[: len(chunk)] = chunk
        row[-1] = 1.0
        rows.append(row)
    return torch.stack(rows)


def nvfp4_ties():
    # tensor maximum 448*6 and a 6.0 in every block -> every scale is exactly 1
    edges = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    cand = torch.cat([edges, torch.nextafter(edges, torch.tensor(9.0)),
                      torch.nextafter(edges, torch.tensor(-9.0)),
                      torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, 7.0])])
    cand = torch.cat([cand, -cand])
    rows = []
    for start in range(0, len(cand), 15):
        chunk = cand[start:start + 15]
        row = torch.zeros(16)
        row[0] = 6.0
        row[1: 1 + len(chunk)] = chunk
        rows.append(row)
    top = torch.zeros(16)
    top[0] = 448.0 * 6.0
    rows.append(top)
    return torch.stack(rows)


def main():
    sys.dont_write_bytecode = True  # nothing is written beside the reference's files
    sys.path.insert(0, str(REFERENCE / "src"))
    from offload_adam.qweight import int4 as r4
    from offload_adam.qweight import int8 as r8
    from offload_adam.qweight import nf4 as rn
    from offload_adam.qweight import nvfp4 as rf

    out = {}

    def put(case, **arrays):
        for key, val in arrays.items():
            out[f"{case}.{key}"] = bits(val) if isinstance(val, torch.Tensor) else np.asarray(val)

    def int8_case(case, x):
        q, s = r8.quantize_int8_per_channel(x)
        put(case, x=x, codes=q, scales=s,
            dequant=r8.dequantize_int8_per_channel(q, s),
            dequant_f32=r8.dequantize_int8_per_channel(q, s.float()))

    def int4_case(case, x, group):
        qw, s = r4.quantize_int4_groupwise(x, group)
        put(case, x=x, group=group, qweight=qw, scales=s, unpacked=r4.unpack_int4_gptq(qw))

    def nf4_case(case, x, block):
        packed, absmax = rn.quantize_nf4_blockwise(x, block)
        put(case, x=x, block=block, packed=packed, absmax=absmax,
            unpacked=rn.unpack_nf4(packed),
            dequant_f32=rn.dequantize_nf4_blockwise(packed, absmax, x.shape[1], block,
                                                    torch.float32))

    def nvfp4_case(case, x):
        packed, s8, gs = rf.quantize_nvfp4_blockwise(x)
        arrays = dict(x=x, packed=packed, block_scale=s8, global_scale=gs.reshape(1),
                      unpacked=rf.unpack_fp4(packed))
        for name, dt in DTYPES.items():
            arrays[f"dequant_{name}"] = rf.dequantize_nvfp4_blockwise(packed, s8, gs,
                                                                      x.shape[1], dt)
        put(case, **arrays)

    for dname, dt in DTYPES.items():
        for rows, cols in ((128, 256), (35, 256), (64, 37)):
            int8_case(f"int8.r{rows}c{cols}.{dname}", seeded(rows, cols, dt))
        int8_case(f"int8.outliers.{dname}", seeded(48, 256, dt, outliers=True))
        for rows, cols, group in ((128, 256, 128), (35, 256, 128), (64, 128, 32)):
            int4_case(f"int4.r{rows}c{cols}g{group}.{dname}", seeded(rows, cols, dt), group)
        int4_case(f"int4.outliers.{dname}", seeded(48, 256, dt, outliers=True), 128)
        for rows, cols, block in ((128, 256, 64), (35, 256, 64), (64, 128, 32)):
            nf4_case(f"nf4.r{rows}c{cols}b{block}.{dname}", seeded(rows, cols, dt), block)
        nf4_case(f"nf4.outliers.{dname}", seeded(48, 256, dt, outliers=True), 64)
        for rows, cols in ((128, 256), (35, 256), (64, 128)):
            nvfp4_case(f"nvfp4.r{rows}c{cols}.{dname}", seeded(rows, cols, dt))
        nvfp4_case(f"nvfp4.outliers.{dname}", seeded(48, 256, dt, outliers=True))

    int8_case("int8.ties.fp32", int8_ties())
    int4_case("int4.ties.fp32", int4_ties(32), 32)
    lut = rn._nf4_lut(torch.device("cpu"))
    nf4_case("nf4.ties.fp32", nf4_ties(lut, 64), 64)
    nvfp4_case("nvfp4.ties.fp32", nvfp4_ties())
    put("nf4", lut=lut)
    put("nvfp4", lut=rf._fp4_lut(torch.device("cpu")))

    np.savez_compressed(OUT, **out)
    print(f"{OUT}: {len(out)} arrays, {OUT.stat().st_size} bytes")


if __name__ == "__main__":
    main()
