"""Pins the CPU oracle of the four weight codecs (row C of the hot path) on CPU:
the layout anchors and known answers held by the reference's own tests, torch's
own narrow-float casts, exhaustive code tables, and a second restatement in
torch ops that must agree bit for bit on the reference's parity shapes.
"""

import numpy as np
import pytest
import torch

BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32


def _bits16(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _w(rows, cols, dtype, seed=0):
    """Reference parity input: torch.manual_seed(0); randn * 0.05 (tests/test_int8.py:81-82)."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, cols, generator=g) * 0.05).to(dtype)


# ----------------------------------------------------- narrow float casts


def test_bf16_and_f16_casts_match_torch(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200_000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 200_000).astype(np.float32),
        rng.integers(0, 2**32, 200_000, dtype=np.uint32).view(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-08,
                  6.1e-5, 6.0975552e-05, np.inf, -np.inf], dtype=np.float32),
    ])
    x = x[~np.isnan(x)]
    t = torch.from_numpy(x.copy())
    assert np.array_equal(oracle.narrow_array(x, "bfloat16"), _bits16(t.to(BF16)))
    assert np.array_equal(oracle.narrow_array(x, "float16"), _bits16(t.to(F16)))
    # all 65536 fp16 patterns widen like torch
    allh = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(F16)
    want = allh.float().numpy()
    got = np.array([oracle.lib().oaref_f16_to_f32(i) for i in range(65536)], dtype=np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert np.all(np.isnan(got[~ok]))


def test_e4m3fn_decode_all_256_codes(oracle):
    """tests/test_nvfp4.py:470-498: bit synthesis must equal torch's cast."""
    allb = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = allb.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([oracle.lib().oaref_e4m3fn_to_f32(i) for i in range(256)], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_e4m3fn_encode_matches_torch_cast(oracle):
    """Every representable value, every midpoint between neighbours, one fp32
    ulp either side of each, plus random values in the range the path uses."""
    codes = np.arange(0, 0x7F, dtype=np.uint8)  # positive finite codes
    vals = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    mids = (vals[:-1] + vals[1:]) / 2
    pts = np.concatenate([vals, mids, [448.0, 464.0, 479.99, 1e-4, 9.765625e-4, 0.0]]).astype(np.float32)
    pts = np.concatenate([pts, np.nextafter(pts, np.float32(1e9)), np.nextafter(pts, np.float32(-1))])
    rng = np.random.default_rng(1)
    pts = np.concatenate([pts, (rng.random(200_000) * 448).astype(np.float32),
                          (rng.random(50_000) * 0.02).astype(np.float32)])
    pts = np.concatenate([pts, -pts])
    want = torch.from_numpy(pts.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = oracle.narrow_array(np.ascontiguousarray(pts), "e4m3fn")
    assert np.array_equal(got, want)


# -------------------------------------------------------------------- int8


def test_int8_reference_anchor(oracle):
    """tests/test_int8.py:43-63: row [0, 0.5, -2, 1] -> scale 2/127, q[2] = -127,
    q[1] = round_half_even(31.75) = 32."""
    q, s = oracle.quant_int8(np.array([[0.0, 0.5, -2.0, 1.0]], dtype=np.float32))
    assert q.shape == (1, 4) and q.dtype == np.int8
    assert s[0] == np.float32(2.0) / np.float32(127.0)
    assert q[0, 2] == -127 and q[0, 1] == 32 and q[0, 0] == 0 and q[0, 3] == 64  # 63.5 -> even
    # per construction every row hits +-127 (tests/test_int8.py:39-41)
    q2, _ = oracle.quant_int8(_w(64, 256, F32).numpy())
    assert (np.abs(q2.astype(np.int32)).max(axis=1) == 127).all()
    # all-zero row: scale 0, codes 0 (eps clamp keeps the reciprocal finite)
    q3, s3 = oracle.quant_int8(np.zeros((1, 8), dtype=np.float32))
    assert s3[0] == 0 and not q3.any()


@pytest.mark.parametrize("shape", [(128, 256), (35, 256), (64, 37)])
@pytest.mark.parametrize("dtype", [BF16, F16, F32])
def test_int8_c_equals_torch(oracle, shape, dtype):
    from oracle import torch_eager as te

    w = _w(*shape, dtype)
    q, s = oracle.quant_int8(w.float().numpy())
    tq, ts = te.quant_int8(w)
    assert np.array_equal(q, tq.numpy())
    assert np.array_equal(s.view(np.uint32), ts.numpy().view(np.uint32))
    sdt = BF16 if dtype == F32 else dtype
    scales = ts.to(sdt)
    want = te.dequant_int8(tq, scales)
    got = oracle.dequant_int8(q, scales.float().numpy(), str(sdt).split(".")[1])
    assert np.array_equal(got, _bits16(want))
    # quantisation error bound: |x - q*scale| <= scale/2 (+ the scale's own rounding)
    err = (w.float() - tq.float() * ts[:, None]).abs()
    assert bool((err <= ts[:, None] * 0.5001 + 1e-12).all())


# -------------------------------------------------------------------- int4


def test_int4_reference_anchor(oracle):
    """tests/test_int4.py:52-69: codes -8..-1 of one row pack LSB-first as
    sum(i << 4i) = 0x76543210 in a (1, 1) int32."""
    row = np.array([[-8, -7, -6, -5, -4, -3, -2, -1]], dtype=np.float32)
    qw, s = oracle.quant_int4(row, group=8)
    assert qw.shape == (1, 1) and qw.dtype == np.int32
    assert s[0, 0] == 1.0  # absmax 8 / 8
    assert int(qw[0, 0]) == sum(i << (4 * i) for i in range(8)) == 0x76543210
    # layout: value at column c of row n sits at bits 4*(c%8) of word [c//8, n]
    x = np.zeros((3, 16), dtype=np.float32)
    x[:, 0] = 7.0  # makes the scale 7/8
    x[2, 11] = -7.0
    qw, s = oracle.quant_int4(x, group=16)
    assert qw.shape == (2, 3)
    assert (int(qw[1, 2]) >> (4 * 3)) & 0xF == 0  # rint(-8) + 8
    assert (int(qw[0, 2]) & 0xF) == 15 and (int(qw[0, 2]) >> 4) & 0xF == 8  # clamp(8)->7, zero->8


@pytest.mark.parametrize("shape,group", [((128, 256), 128), ((35, 256), 128), ((64, 256), 32)])
@pytest.mark.parametrize("dtype", [BF16, F16, F32])
def test_int4_c_equals_torch(oracle, shape, group, dtype):
    from oracle import torch_eager as te

    w = _w(*shape, dtype, seed=1)
    qw, s = oracle.quant_int4(w.float().numpy(), group)
    tq, ts = te.quant_int4(w, group)
    assert np.array_equal(qw, tq.numpy())
    assert np.array_equal(s.view(np.uint32), ts.numpy().view(np.uint32))
    sdt = BF16 if dtype == F32 else dtype
    scales = ts.to(sdt)
    want = te.dequant_int4(tq, scales, group)
    got = oracle.dequant_int4(qw, scales.float().numpy(), group, str(sdt).split(".")[1])
    assert np.array_equal(got, _bits16(want))
    # unpacked codes are in [-8, 7]
    nib = np.stack([(qw >> (4 * i)) & 0xF for i in range(8)])
    assert nib.min() >= 0 and nib.max() <= 15


# --------------------------------------------------------------------- NF4


def test_nf4_reference_anchors(oracle):
    """tests/test_nf4.py:42-64: codes 0..7 across 8 columns pack as 0x01 0x23 0x45
    0x67 (even column in the high nibble); the codebook is sorted, holds 0, and
    runs from -1 to 1 (qweight/nf4.py:35-52)."""
    lut = np.array([oracle.lib().oaref_nf4_lut(i) for i in range(16)], dtype=np.float32)
    assert lut[0] == -1.0 and lut[15] == 1.0 and lut[7] == 0.0
    assert np.all(np.diff(lut) > 0)
    assert lut[1] == np.float32(-0.6961928009986877) and lut[14] == np.float32(0.7229568362236023)
    packed, absmax = oracle.quant_nf4(lut[None, :8].copy(), block=8)
    assert packed.tolist() == [[0x01, 0x23, 0x45, 0x67]]
    assert absmax.tolist() == [1.0]
    # every codebook entry encodes to its own index and decodes to itself
    packed, absmax = oracle.quant_nf4(lut[None, :].copy(), block=16)
    assert packed.tolist() == [[0x01, 0x23, 0x45, 0x67, 0x89, 0xAB, 0xCD, 0xEF]]
    back = oracle.dequant_nf4(packed, absmax, 16, "float32")
    assert np.array_equal(back[0], lut)
    # ties go to the lower index: the exact midpoint of codes 7 (0.0) and 8
    mid = np.float32(lut[8] / 2)
    x = np.array([[mid, 1.0]], dtype=np.float32)
    p, _ = oracle.quant_nf4(x, block=2)
    d7, d8 = abs(np.float32(mid - lut[7])), abs(np.float32(mid - lut[8]))
    assert (p[0, 0] >> 4) == (7 if d7 <= d8 else 8)


@pytest.mark.parametrize("shape,block", [((128, 256), 64), ((35, 256), 64), ((64, 128), 32)])
@pytest.mark.parametrize("dtype", [BF16, F16, F32])
def test_nf4_c_equals_torch(oracle, shape, block, dtype):
    from oracle import torch_eager as te

    w = _w(*shape, dtype, seed=2)
    packed, absmax = oracle.quant_nf4(w.float().numpy(), block)
    tp, ta = te.quant_nf4(w, block)
    assert np.array_equal(absmax.view(np.uint32), ta.numpy().view(np.uint32))
    assert np.array_equal(packed, tp.numpy())
    for odt in (BF16, F16):
        want = te.dequant_nf4(tp, ta, block, odt)
        got = oracle.dequant_nf4(packed, absmax, block, str(odt).split(".")[1])
        assert np.array_equal(got, _bits16(want))


# ------------------------------------------------------------------- NVFP4

# tests/test_nvfp4.py:306-337: (magnitude, expected e2m1 value), eps = 1e-3
_EPS = 1e-3
RNE_CASES = [
    (0.0, 0.0), (0.1, 0.0), (0.25, 0.0), (0.25 + _EPS, 0.5), (0.5, 0.5), (0.75 - _EPS, 0.5),
    (0.75, 1.0), (0.75 + _EPS, 1.0), (1.0, 1.0), (1.25 - _EPS, 1.0), (1.25, 1.0),
    (1.25 + _EPS, 1.5), (1.5, 1.5), (1.75 - _EPS, 1.5), (1.75, 2.0), (1.75 + _EPS, 2.0),
    (2.0, 2.0), (2.5 - _EPS, 2.0), (2.5, 2.0), (2.5 + _EPS, 3.0), (3.0, 3.0), (3.5 - _EPS, 3.0),
    (3.5, 4.0), (3.5 + _EPS, 4.0), (4.0, 4.0), (5.0 - _EPS, 4.0), (5.0, 4.0), (5.0 + _EPS, 6.0),
    (6.0, 6.0), (1e6, 6.0),
]


def test_fp4_reference_anchors(oracle):
    L = oracle.lib()
    lut = [L.oaref_fp4_lut(i) for i in range(16)]
    # tests/test_nvfp4.py:66-74
    assert lut[:8] == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert lut[8:] == [-v for v in lut[:8]]
    assert np.signbit(np.float32(lut[8]))  # code 8 is -0 (tests/test_nvfp4.py:264-269)
    # tests/test_nvfp4.py:289-359: 30 round-to-nearest-even boundary cases x 2 signs
    for sign in (1.0, -1.0):
        mags = np.array([m for m, _ in RNE_CASES], dtype=np.float32) * np.float32(sign)
        codes = oracle.fp4_code_array(mags)
        got = np.array([lut[c] for c in codes], dtype=np.float32)
        want = np.array([e for _, e in RNE_CASES], dtype=np.float32)
        assert np.array_equal(np.abs(got), want)
        if sign < 0:
            assert np.all(codes >= 8)
    # tests/test_nvfp4.py:273-286: +0 -> code 0, -0 -> code 8
    assert oracle.fp4_code_array(np.array([0.0, -0.0], dtype=np.float32)).tolist() == [0, 8]


def test_nvfp4_layout_anchor_and_all_codes(oracle):
    """tests/test_nvfp4.py:51-63: codes 0..7 pack as 0x10 0x32 0x54 0x76 (even
    column in the LOW nibble); tests/test_nvfp4.py:233-270: every code decodes
    to its table value when the effective scale is 1."""
    L = oracle.lib()
    lut = np.array([L.oaref_fp4_lut(i) for i in range(16)], dtype=np.float32)
    x = np.zeros((1, 16), dtype=np.float32)
    x[0, :8] = lut[:8]
    packed, s8, gs = oracle.quant_nvfp4(x)
    assert packed[0, :4].tolist() == [0x10, 0x32, 0x54, 0x76]
    assert s8[0, 0] == 0x7E  # block amax == tensor amax -> scale 448
    assert gs == np.float32(6.0) / np.float32(2688.0)
    # decode: byte (j << 4) | j in 16 blocks, block scale 1.0 (0x38), global 1.0
    pk = np.array([[(j << 4) | j for j in range(16) for _ in range(8)]], dtype=np.uint8)
    sc = np.full((1, 16), 0x38, dtype=np.uint8)
    out = oracle.dequant_nvfp4(pk, sc, np.float32(1.0), "float32")[0]
    for j in range(16):
        blk = out[16 * j:16 * j + 16]
        assert np.array_equal(blk.view(np.uint32), np.full(16, lut[j], np.float32).view(np.uint32))


@pytest.mark.parametrize("shape", [(128, 256), (35, 256), (64, 64)])
@pytest.mark.parametrize("dtype", [BF16, F16, F32])
def test_nvfp4_c_equals_torch(oracle, shape, dtype):
    from oracle import torch_eager as te

    w = _w(*shape, dtype, seed=3)
    packed, s8, gs = oracle.quant_nvfp4(w.float().numpy())
    tp, ts, tgs = te.quant_nvfp4(w)
    assert np.float32(gs).view(np.uint32) == tgs.numpy().view(np.uint32)
    assert np.array_equal(s8, ts.view(torch.uint8).numpy())
    assert np.array_equal(packed, tp.numpy())
    for odt in (BF16, F16):
        want = te.dequant_nvfp4(tp, ts, tgs, odt)
        got = oracle.dequant_nvfp4(packed, s8, gs, str(odt).split(".")[1])
        assert np.array_equal(got, _bits16(want))
    # the largest block scale is exactly 448 (the block holding the tensor amax)
    assert s8.max() == 0x7E
    # relative reconstruction error of e2m1 with a per-16 scale stays below 1/3
    back = oracle.dequant_nvfp4(packed, s8, gs, "float32")
    blk_amax = np.abs(w.float().numpy()).reshape(shape[0], -1, 16).max(-1, keepdims=True)
    err = np.abs(back - w.float().numpy()).reshape(shape[0], -1, 16)
    assert np.all(err <= blk_amax / 6.0 * 1.1 + 1e-12)
