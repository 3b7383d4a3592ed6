"""GPU parity of the eight codec kernels against the C oracle: BIT-EXACT on the
packed codes, the scales and the dequantised values.

Shapes follow the reference's own parity tests (tests/test_int8.py:70-84 and
the other three files): seeded ``randn * 0.05`` in bf16 / fp16, plus fp32
masters, misaligned row counts, column counts off the 8-element fast path,
strided and unaligned sources, and benchmark config 3 (4096 x 14336 with 1 %
outliers x10).
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DT = {torch.float32: "float32", torch.bfloat16: "bfloat16", torch.float16: "float16"}


def _weight(rows, cols, dtype, seed=0, outliers=False):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(rows, cols, generator=g) * (0.02 if outliers else 0.05)
    if outliers:
        mask = torch.rand(rows, cols, generator=g) < 0.01
        w = torch.where(mask, w * 10, w)
    return w.to(dtype)


def _np_bits(t):
    """float tensor -> numpy array of raw bits (uint16 for 16-bit, uint32 for fp32)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy().view(np.uint32)
    return t.view(torch.int16).numpy().view(np.uint16)


def _oracle_out_bits(a, out_dtype):
    return a.view(np.uint32) if out_dtype == torch.float32 else a


def _cast_scales(s_f32, dtype):
    """fp32 oracle scales -> bits after torch's own cast to the scale dtype."""
    return _np_bits(torch.from_numpy(s_f32.copy()).to(dtype))


SHAPES = [(128, 256), (35, 256), (4096, 4096), (64, 2048)]


@pytest.mark.parametrize("rows,cols", SHAPES + [(64, 37), (3, 8), (1, 1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_int8(oracle, rows, cols, dtype):
    from offload_adam_amd.qweight import _codec_ops as ops

    w = _weight(rows, cols, dtype)
    sdt = torch.bfloat16 if dtype == torch.float32 else dtype
    q = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
    s = torch.empty(rows, dtype=sdt, device="cuda")
    ops.quantize_int8_into(w.cuda(), q, s)
    rq, rs = oracle.quant_int8(w.float().numpy())
    assert np.array_equal(q.cpu().numpy(), rq)
    assert np.array_equal(_np_bits(s), _cast_scales(rs, sdt))
    for odt in (sdt, torch.float32):
        got = ops.dequantize_int8(q, s, odt)
        want = oracle.dequant_int8(rq, s.float().cpu().numpy(), DT[odt])
        assert np.array_equal(_np_bits(got), _oracle_out_bits(want, odt)), odt


@pytest.mark.parametrize("rows,cols,group", [(128, 256, 128), (35, 256, 128), (4096, 4096, 128),
                                             (64, 2048, 64), (40, 96, 32), (8, 48, 24),
                                             (5, 1024, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_int4(oracle, rows, cols, group, dtype):
    from offload_adam_amd.qweight import _codec_ops as ops

    w = _weight(rows, cols, dtype, seed=1)
    sdt = torch.bfloat16 if dtype == torch.float32 else dtype
    qw = torch.empty(cols // 8, rows, dtype=torch.int32, device="cuda")
    s = torch.empty(cols // group, rows, dtype=sdt, device="cuda")
    ops.quantize_int4_into(w.cuda(), group, qw, s)
    rq, rs = oracle.quant_int4(w.float().numpy(), group)
    assert np.array_equal(qw.cpu().numpy(), rq)
    assert np.array_equal(_np_bits(s), _cast_scales(rs, sdt))
    for odt in (sdt, torch.float32):
        got = ops.dequantize_int4(qw, s, group, odt)
        want = oracle.dequant_int4(rq, s.float().cpu().numpy(), group, DT[odt])
        assert np.array_equal(_np_bits(got), _oracle_out_bits(want, odt)), odt


@pytest.mark.parametrize("rows,cols,block", [(128, 256, 64), (35, 256, 64), (4096, 4096, 64),
                                             (64, 128, 32), (16, 60, 6), (7, 1024, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_nf4(oracle, rows, cols, block, dtype):
    from offload_adam_amd.qweight import _codec_ops as ops

    w = _weight(rows, cols, dtype, seed=2)
    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(rows * (cols // block), dtype=torch.float32, device="cuda")
    ops.quantize_nf4_into(w.cuda(), block, packed, absmax)
    rp, ra = oracle.quant_nf4(w.float().numpy(), block)
    assert np.array_equal(absmax.cpu().numpy().view(np.uint32), ra.view(np.uint32))
    assert np.array_equal(packed.cpu().numpy(), rp)
    for odt in (torch.bfloat16, torch.float16, torch.float32):
        got = ops.dequantize_nf4(packed, absmax, cols, block, odt)
        want = oracle.dequant_nf4(rp, ra, block, DT[odt])
        assert np.array_equal(_np_bits(got), _oracle_out_bits(want, odt)), odt


@pytest.mark.parametrize("rows,cols", SHAPES + [(35, 16), (3, 48)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_nvfp4(oracle, rows, cols, dtype):
    from offload_adam_amd.qweight import _codec_ops as ops

    w = _weight(rows, cols, dtype, seed=3)
    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    s8 = torch.empty(rows, cols // 16, dtype=torch.float8_e4m3fn, device="cuda")
    gs = torch.empty((), dtype=torch.float32, device="cuda")
    ops.quantize_nvfp4_into(w.cuda(), packed, s8, gs)
    rp, rs, rgs = oracle.quant_nvfp4(w.float().numpy())
    assert gs.cpu().numpy().view(np.uint32) == np.float32(rgs).view(np.uint32)
    assert np.array_equal(s8.view(torch.uint8).cpu().numpy(), rs)
    assert np.array_equal(packed.cpu().numpy(), rp)
    for odt in (torch.bfloat16, torch.float16, torch.float32):
        got = ops.dequantize_nvfp4(packed, s8, gs, cols, odt)
        want = oracle.dequant_nvfp4(rp, rs, rgs, DT[odt])
        assert np.array_equal(_np_bits(got), _oracle_out_bits(want, odt)), odt


@pytest.mark.parametrize("rows,cols", [(12288, 4096), (4096, 11008)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_large_shapes_of_the_reference_parity_tests(oracle, rows, cols, dtype):
    """The two large shapes of the reference's parity lists (tests/test_int8.py:70-84,
    tests/test_int4.py:91-116, tests/test_nf4.py:86-123, tests/test_nvfp4.py:98-134),
    all four formats: codes, scales and the bf16 decode, bit for bit."""
    from offload_adam_amd.qweight import _codec_ops as ops

    w = _weight(rows, cols, dtype, seed=11)
    src = w.float().numpy()
    dev = w.cuda()
    sdt = torch.bfloat16

    q = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
    s = torch.empty(rows, dtype=sdt, device="cuda")
    ops.quantize_int8_into(dev, q, s)
    rq, rs = oracle.quant_int8(src)
    assert np.array_equal(q.cpu().numpy(), rq)
    assert np.array_equal(_np_bits(s), _cast_scales(rs, sdt))
    want = oracle.dequant_int8(rq, s.float().cpu().numpy(), "bfloat16")
    assert np.array_equal(_np_bits(ops.dequantize_int8(q, s, sdt)), want)

    qw = torch.empty(cols // 8, rows, dtype=torch.int32, device="cuda")
    s4 = torch.empty(cols // 128, rows, dtype=sdt, device="cuda")
    ops.quantize_int4_into(dev, 128, qw, s4)
    rq, rs = oracle.quant_int4(src, 128)
    assert np.array_equal(qw.cpu().numpy(), rq)
    assert np.array_equal(_np_bits(s4), _cast_scales(rs, sdt))
    want = oracle.dequant_int4(rq, s4.float().cpu().numpy(), 128, "bfloat16")
    assert np.array_equal(_np_bits(ops.dequantize_int4(qw, s4, 128, sdt)), want)

    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(rows * (cols // 64), dtype=torch.float32, device="cuda")
    ops.quantize_nf4_into(dev, 64, packed, absmax)
    rp, ra = oracle.quant_nf4(src, 64)
    assert np.array_equal(absmax.cpu().numpy().view(np.uint32), ra.view(np.uint32))
    assert np.array_equal(packed.cpu().numpy(), rp)
    want = oracle.dequant_nf4(rp, ra, 64, "bfloat16")
    assert np.array_equal(_np_bits(ops.dequantize_nf4(packed, absmax, cols, 64, sdt)), want)

    pk4 = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    s8 = torch.empty(rows, cols // 16, dtype=torch.float8_e4m3fn, device="cuda")
    gs = torch.empty((), dtype=torch.float32, device="cuda")
    ops.quantize_nvfp4_into(dev, pk4, s8, gs)
    rp, rs, rgs = oracle.quant_nvfp4(src)
    assert gs.cpu().numpy().view(np.uint32) == np.float32(rgs).view(np.uint32)
    assert np.array_equal(s8.view(torch.uint8).cpu().numpy(), rs)
    assert np.array_equal(pk4.cpu().numpy(), rp)
    want = oracle.dequant_nvfp4(rp, rs, rgs, "bfloat16")
    assert np.array_equal(_np_bits(ops.dequantize_nvfp4(pk4, s8, gs, cols, sdt)), want)


def test_strided_and_unaligned_sources(oracle):
    """Column slices (row stride > cols) and views starting off a 16-byte
    boundary give the same codes as the contiguous copy."""
    from offload_adam_amd.qweight import _codec_ops as ops

    big = _weight(64, 512 + 8, torch.float32, seed=4).cuda()
    for view in (big[:, :512], big[:, 8:520], big[:, 3:515]):
        rows, cols = view.shape
        ref = view.contiguous().cpu().numpy()
        q = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
        s = torch.empty(rows, dtype=torch.bfloat16, device="cuda")
        ops.quantize_int8_into(view, q, s)
        assert np.array_equal(q.cpu().numpy(), oracle.quant_int8(ref)[0])
        qw = torch.empty(cols // 8, rows, dtype=torch.int32, device="cuda")
        s4 = torch.empty(cols // 128, rows, dtype=torch.bfloat16, device="cuda")
        ops.quantize_int4_into(view, 128, qw, s4)
        assert np.array_equal(qw.cpu().numpy(), oracle.quant_int4(ref, 128)[0])
        pk = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
        am = torch.empty(rows * (cols // 64), dtype=torch.float32, device="cuda")
        ops.quantize_nf4_into(view, 64, pk, am)
        assert np.array_equal(pk.cpu().numpy(), oracle.quant_nf4(ref, 64)[0])
        pk4 = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
        s8 = torch.empty(rows, cols // 16, dtype=torch.float8_e4m3fn, device="cuda")
        gs = torch.empty((), dtype=torch.float32, device="cuda")
        ops.quantize_nvfp4_into(view, pk4, s8, gs)
        rp, rs, _ = oracle.quant_nvfp4(ref)
        assert np.array_equal(pk4.cpu().numpy(), rp)
        assert np.array_equal(s8.view(torch.uint8).cpu().numpy(), rs)


def test_int4_payload_that_is_only_4_byte_aligned(oracle):
    """A payload view 4, 8 or 12 bytes off a 16-byte boundary (row count a multiple of
    four, whole tiles: the shape that otherwise takes the 16-byte transposed store) gets
    the same words, from the plain encoder and from the fused step + re-encode."""
    from offload_adam_amd import _lib
    from offload_adam_amd.kernels import _common
    from offload_adam_amd.qweight import _codec_ops as ops
    from helpers import HYP, adam_inputs

    rows, cols, group = 128, 512, 128
    w = _weight(rows, cols, torch.float32, seed=6)
    want_q, want_s = oracle.quant_int4(w.numpy(), group)
    for off in (1, 2, 3):
        buf = torch.zeros((cols // 8) * rows + 4, dtype=torch.int32, device="cuda")
        qw = buf[off:off + (cols // 8) * rows].view(cols // 8, rows)
        assert qw.data_ptr() % 16 == 4 * off
        s = torch.empty(cols // group, rows, dtype=torch.bfloat16, device="cuda")
        ops.quantize_int4_into(w.cuda(), group, qw, s)
        assert np.array_equal(qw.cpu().numpy(), want_q), off
        assert np.array_equal(_np_bits(s), _cast_scales(want_s, torch.bfloat16))
        assert int(buf[:off].abs().sum()) == 0 and int(buf[off + (cols // 8) * rows:].abs().sum()) == 0
    # fused step + re-encode through the C ABI into the same kind of view
    _, st = adam_inputs(rows * cols, seed=8, mode="fp32_master", device="cuda")
    ref = {k: v.clone() for k, v in st.items()}
    b1h, b2h = _common.folded_betas(HYP["beta1"], HYP["beta2"], HYP["step"])
    lib = _lib.load()

    def fused(state, qw, s):
        rc = lib.oa_adam_requant_int4(
            _lib.ptr(state["grad"]), _lib.ptr(state["exp_avg"]), _lib.ptr(state["exp_avg_sq"]),
            _lib.ptr(state["master_params"]), rows, cols, HYP["lr"], HYP["weight_decay"], b1h, b2h,
            HYP["eps"], 1, None, group, _lib.ptr(qw), _lib.ptr(s), _lib.OA_BF16,
            _lib.current_stream_ptr())
        assert rc == 0

    aligned = torch.empty(cols // 8, rows, dtype=torch.int32, device="cuda")
    s0 = torch.empty(cols // group, rows, dtype=torch.bfloat16, device="cuda")
    fused(ref, aligned, s0)
    buf = torch.zeros((cols // 8) * rows + 4, dtype=torch.int32, device="cuda")
    shifted = buf[1:1 + (cols // 8) * rows].view(cols // 8, rows)
    s1 = torch.empty_like(s0)
    fused(st, shifted, s1)
    torch.cuda.synchronize()
    assert torch.equal(shifted, aligned) and torch.equal(s1.view(torch.int16), s0.view(torch.int16))
    assert torch.equal(st["master_params"], ref["master_params"])
    master = ref["master_params"].cpu().numpy().reshape(rows, cols)
    assert np.array_equal(aligned.cpu().numpy(), oracle.quant_int4(master, group)[0])


def test_nf4_thresholds_match_brute_force(oracle):
    """The kernel's threshold count (bucket table) must equal the 16-way fp32
    distance search for every input: all floats within 64 ulps of each decision
    point, within 8 ulps of every bucket edge k/128 - 1 (where the table index
    changes), the codebook itself, and a dense sweep of [-1, 1]."""
    from offload_adam_amd.qweight import _codec_ops as ops

    lut = np.array([oracle.lib().oaref_nf4_lut(i) for i in range(16)], dtype=np.float32)
    mids = ((lut[:-1].astype(np.float64) + lut[1:]) / 2).astype(np.float32)
    pts = [lut, np.linspace(-1, 1, 200_001, dtype=np.float32)]
    for m in mids:
        b = int(m.view(np.uint32))
        pts.append(np.arange(b - 64, b + 65, dtype=np.uint32).view(np.float32))
    for k in range(257):
        e = np.float32(k / 128.0 - 1.0)
        if e == 0:
            pts.append(np.array([0.0, -0.0, 1e-45, -1e-45, 1e-38, -1e-38], dtype=np.float32))
            continue
        b = int(e.view(np.uint32))
        pts.append(np.arange(b - 8, b + 9, dtype=np.uint32).view(np.float32))
    x = np.concatenate(pts)
    x = x[np.abs(x) <= 1.0]  # each row's absmax must stay exactly 1
    pad = (-len(x)) % 64
    x = np.concatenate([x, np.zeros(pad, dtype=np.float32)])
    # one row per 64-block whose absmax is exactly 1, so normalised == input
    x = x.reshape(-1, 64)
    x = np.concatenate([x, np.ones((x.shape[0], 64), dtype=np.float32)], axis=1)
    t = torch.from_numpy(x).cuda()
    rows, cols = t.shape
    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(rows, dtype=torch.float32, device="cuda")
    # block = 128 covers the data half and the all-ones half: absmax == 1
    ops.quantize_nf4_into(t, 128, packed, absmax)
    rp, _ = oracle.quant_nf4(x, 128)
    assert np.array_equal(packed.cpu().numpy(), rp)


def test_nvfp4_e2m1_boundaries_match_bit_level_definition(oracle):
    """The vector kernel encodes with the GPU's FP4 conversion instruction; it must
    agree with the bit-level e2m1 rounding (oracle) on every float within 64 ulps
    of each grid point and rounding boundary, and on a dense sweep of [-6, 6].
    Scales are forced to exactly 1: the tensor maximum is 448*6 (global scale 1)
    and every 16-element block carries one 6.0 (block scale 1)."""
    from offload_adam_amd.qweight import _codec_ops as ops

    pts = [np.linspace(-6, 6, 120_001, dtype=np.float32)]
    for v in (0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 3.5, 4.0, 5.0, 6.0):
        for sgn in (1.0, -1.0):
            b = int(np.float32(sgn * v).view(np.uint32))
            pts.append(np.arange(b - 64, b + 65, dtype=np.uint32).view(np.float32))
    pts.append(np.array([0.0, -0.0, 1e-45, -1e-45, 1e-38, -1e-38, 1e-20], dtype=np.float32))
    x = np.concatenate(pts)
    x = x[np.abs(x) <= 6.0]
    x = np.concatenate([x, np.zeros((-len(x)) % 15, dtype=np.float32)]).reshape(-1, 15)
    blocks = np.concatenate([np.full((x.shape[0], 1), 6.0, dtype=np.float32), x], axis=1)
    per_row = 8  # blocks per row -> 128 columns
    pad = (-blocks.shape[0]) % per_row
    blocks = np.concatenate([blocks, np.tile(blocks[:1], (pad, 1))])
    mat = blocks.reshape(-1, per_row * 16)
    top = np.zeros((1, per_row * 16), dtype=np.float32)
    top[0, 0] = 448.0 * 6.0  # sets the tensor scale to exactly 1
    mat = np.concatenate([top, mat])
    t = torch.from_numpy(mat).cuda()
    rows, cols = t.shape
    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    scales = torch.empty(rows, cols // 16, dtype=torch.float8_e4m3fn, device="cuda")
    gs = torch.zeros((), dtype=torch.float32, device="cuda")
    ops.quantize_nvfp4_into(t, packed, scales, gs)
    assert float(gs) == 1.0
    assert (scales[1:].view(torch.uint8) == 0x38).all()  # e4m3fn 1.0
    rp, rs, rg = oracle.quant_nvfp4(mat)
    assert np.array_equal(packed.cpu().numpy(), rp)
    assert np.array_equal(scales.view(torch.uint8).cpu().numpy(), rs)
    back = ops.dequantize_nvfp4(packed, scales, gs, cols, torch.float32)
    assert np.array_equal(back.cpu().numpy().view(np.uint32),
                          oracle.dequant_nvfp4(rp, rs, rg, "float32").view(np.uint32))


def test_config3_weight(oracle):
    """benchmark config 3: 4096 x 14336 bf16 weight ~N(0, 0.02) with 1 % outliers
    x10; requantise from its fp32 master, every format, then dequantise."""
    from offload_adam_amd.qweight import _codec_ops as ops

    rows, cols = 4096, 14336
    w = _weight(rows, cols, torch.bfloat16, seed=5, outliers=True)
    master = w.float()
    m_gpu = master.cuda()
    m_np = master.numpy()

    q = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
    s = torch.empty(rows, dtype=torch.bfloat16, device="cuda")
    ops.quantize_int8_into(m_gpu, q, s)
    rq, rs = oracle.quant_int8(m_np)
    assert np.array_equal(q.cpu().numpy(), rq)
    assert np.array_equal(_np_bits(s), _cast_scales(rs, torch.bfloat16))
    assert np.array_equal(_np_bits(ops.dequantize_int8(q, s)),
                          oracle.dequant_int8(rq, s.float().cpu().numpy(), "bfloat16"))

    qw = torch.empty(cols // 8, rows, dtype=torch.int32, device="cuda")
    s4 = torch.empty(cols // 128, rows, dtype=torch.bfloat16, device="cuda")
    ops.quantize_int4_into(m_gpu, 128, qw, s4)
    rq4, rs4 = oracle.quant_int4(m_np, 128)
    assert np.array_equal(qw.cpu().numpy(), rq4)
    assert np.array_equal(_np_bits(s4), _cast_scales(rs4, torch.bfloat16))
    assert np.array_equal(_np_bits(ops.dequantize_int4(qw, s4, 128)),
                          oracle.dequant_int4(rq4, s4.float().cpu().numpy(), 128, "bfloat16"))

    pk = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    am = torch.empty(rows * (cols // 64), dtype=torch.float32, device="cuda")
    ops.quantize_nf4_into(m_gpu, 64, pk, am)
    rp, ra = oracle.quant_nf4(m_np, 64)
    assert np.array_equal(pk.cpu().numpy(), rp)
    assert np.array_equal(am.cpu().numpy().view(np.uint32), ra.view(np.uint32))
    assert np.array_equal(_np_bits(ops.dequantize_nf4(pk, am, cols, 64, torch.bfloat16)),
                          oracle.dequant_nf4(rp, ra, 64, "bfloat16"))

    pk4 = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    s8 = torch.empty(rows, cols // 16, dtype=torch.float8_e4m3fn, device="cuda")
    gs = torch.empty((), dtype=torch.float32, device="cuda")
    ops.quantize_nvfp4_into(m_gpu, pk4, s8, gs)
    rp4, rs8, rgs = oracle.quant_nvfp4(m_np)
    assert gs.cpu().numpy().view(np.uint32) == np.float32(rgs).view(np.uint32)
    assert np.array_equal(pk4.cpu().numpy(), rp4)
    assert np.array_equal(s8.view(torch.uint8).cpu().numpy(), rs8)
    assert np.array_equal(_np_bits(ops.dequantize_nvfp4(pk4, s8, gs, cols, torch.bfloat16)),
                          oracle.dequant_nvfp4(rp4, rs8, rgs, "bfloat16"))
