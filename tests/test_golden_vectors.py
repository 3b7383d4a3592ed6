"""The data in tests/golden/known_answers.json against the CPU oracle, and - for
the codec entries - against the HIP kernels through the C ABI (``gpu`` tests)."""

import json
from pathlib import Path

import numpy as np
import pytest
import torch

GOLDEN = json.loads((Path(__file__).parent / "golden" / "known_answers.json").read_text())


def h(x):
    return int(x, 16)


# ------------------------------------------------------------------ oracle


def test_oracle_philox_and_triton_layout(oracle):
    for kat in GOLDEN["philox4x32_10"]:
        got = oracle.philox(tuple(map(h, kat["counter"])), tuple(map(h, kat["key"])))
        assert got == tuple(map(h, kat["output"]))
    seed = h(GOLDEN["triton_randint"]["seed"])
    for offset, word in GOLDEN["triton_randint"]["words"].items():
        assert oracle.lib().oaref_triton_randint(seed, int(offset)) == h(word)
        assert oracle.lib().oaref_rand16(seed, int(offset), 0) == h(word) & 0xFFFF


def test_oracle_folded_betas(oracle):
    g = GOLDEN["folded_betas"]
    b1, b2 = oracle.folded_betas(g["beta1"], g["beta2"], g["step"])
    assert b1 == pytest.approx(g["beta1_hat"], rel=1e-15)
    assert b2 == pytest.approx(g["beta2_hat"], rel=1e-15)


def test_oracle_codec_anchors(oracle):
    a = GOLDEN["int8_anchor"]
    q, s = oracle.quant_int8(np.array([a["row"]], dtype=np.float32))
    assert q[0].tolist() == a["codes"]
    assert s[0] == np.float32(np.float32(a["scale_numerator"]) / np.float32(a["scale_denominator"]))
    a = GOLDEN["int4_anchor"]
    qw, s = oracle.quant_int4(np.array([a["row"]], dtype=np.float32), group=a["group"])
    assert int(qw[0, 0]) & 0xFFFFFFFF == h(a["packed_word"]) and s[0, 0] == a["scale"]
    lut = [oracle.lib().oaref_nf4_lut(i) for i in range(16)]
    assert lut == [float(np.float32(v)) for v in GOLDEN["nf4_lut"]]
    assert lut == sorted(lut) and lut[0] == -1.0 and lut[7] == 0.0 and lut[15] == 1.0


def fp4_cases():
    mags = np.array([c["magnitude"] for c in GOLDEN["fp4_rne_boundaries"]], dtype=np.float32)
    want = np.array([c["expected_magnitude"] for c in GOLDEN["fp4_rne_boundaries"]],
                    dtype=np.float32)
    return mags, want


def test_oracle_fp4_boundaries_and_signed_zero(oracle):
    lut = np.array(GOLDEN["fp4_e2m1_lut"], dtype=np.float32)
    mags, want = fp4_cases()
    assert len(mags) == 30
    for sign in (1.0, -1.0):
        codes = oracle.fp4_code_array((mags * np.float32(sign)).astype(np.float32))
        assert np.array_equal(np.abs(lut[codes]), want)
        assert np.array_equal(codes >> 3, np.signbit(mags * np.float32(sign)).astype(codes.dtype))
    z = oracle.fp4_code_array(np.array([0.0, -0.0], dtype=np.float32))
    assert z.tolist() == [GOLDEN["fp4_signed_zero"]["+0.0"], GOLDEN["fp4_signed_zero"]["-0.0"]]


# --------------------------------------------------------------- HIP kernels


@pytest.mark.gpu
def test_hip_int8_and_int4_anchors():
    from offload_adam_amd.qweight import Int4QWeight, Int8QWeight

    a = GOLDEN["int8_anchor"]
    q = Int8QWeight.from_float(torch.tensor([a["row"]], device="cuda"), scale_dtype=torch.float32)
    assert q.weight.cpu()[0].tolist() == a["codes"]
    assert float(q.scales[0]) == float(np.float32(a["scale_numerator"]) /
                                       np.float32(a["scale_denominator"]))
    a = GOLDEN["int4_anchor"]
    q = Int4QWeight.from_float(torch.tensor([a["row"]], dtype=torch.float32, device="cuda"),
                               group_size=a["group"], scale_dtype=torch.float32)
    assert int(q.qweight[0, 0]) & 0xFFFFFFFF == h(a["packed_word"])
    assert float(q.scales[0, 0]) == a["scale"]


@pytest.mark.gpu
def test_hip_nf4_anchor_and_lut():
    from offload_adam_amd.qweight import NF4QWeight

    lut = torch.tensor(GOLDEN["nf4_lut"], dtype=torch.float32)
    row = torch.zeros(1, 64)
    row[0, :8] = lut[:8]      # codes 0..7 once the block's absmax is 1
    row[0, 63] = 1.0
    q = NF4QWeight.from_float(row.cuda(), blocksize=64)
    assert q.weight_packed.cpu()[0, :4].tolist() == [h(b) for b in GOLDEN["nf4_anchor"]["packed_bytes"]]
    back = q.dequantize(torch.float32).cpu()
    assert torch.equal(back[0, :8], lut[:8]) and float(back[0, 63]) == 1.0
    # every code decodes to its table entry
    full = torch.cat([lut, torch.zeros(48)]).reshape(1, 64).cuda()
    assert torch.equal(NF4QWeight.from_float(full, blocksize=64).dequantize(torch.float32).cpu()[0, :16], lut)


@pytest.mark.gpu
def test_hip_fp4_anchor_boundaries_and_signed_zero():
    """Scales forced to exactly 1 (tensor maximum 448*6, one 6.0 opening every
    16-element block), so the stored codes are the e2m1 codes of the inputs."""
    from offload_adam_amd.qweight import NVFP4QWeight

    lut = np.array(GOLDEN["fp4_e2m1_lut"], dtype=np.float32)
    mags, want = fp4_cases()
    keep = mags <= 6.0  # the 1e6 case owns the tensor scale: checked separately below
    mags, want = mags[keep], want[keep]
    assert len(mags) == 29

    def block(vals):
        return np.concatenate([[6.0], vals, np.zeros(15 - len(vals))]).astype(np.float32)

    top = np.zeros(16, dtype=np.float32)
    top[0] = 448.0 * 6.0
    rows = [top,
            block(mags[:15]), block(mags[15:]),          # rows 1, 2: positive
            block(-mags[:15]), block(-mags[15:]),        # rows 3, 4: negative
            block(np.concatenate([lut[:8], [0.0, -0.0]]).astype(np.float32))]  # row 5
    q = NVFP4QWeight.from_float(torch.from_numpy(np.stack(rows)).cuda())
    assert float(q.global_scale) == 1.0
    assert (q.block_scale_fp8[1:].view(torch.uint8) == 0x38).all()  # e4m3fn 1.0
    packed = q.weight_packed.cpu().numpy()
    codes = np.stack([packed & 0xF, packed >> 4], axis=-1).reshape(packed.shape[0], 16)

    for first, negative in ((1, 0), (3, 1)):
        got = np.concatenate([codes[first, 1:16], codes[first + 1, 1:15]])
        assert np.array_equal(np.abs(lut[got]), want), (negative, got)
        assert np.array_equal(got >> 3, np.full(29, negative, dtype=got.dtype))

    a = GOLDEN["fp4_anchor"]
    assert codes[5, 1:9].tolist() == a["codes"]
    assert codes[5, 9:11].tolist() == [GOLDEN["fp4_signed_zero"]["+0.0"],
                                       GOLDEN["fp4_signed_zero"]["-0.0"]]
    # the anchor bytes themselves: codes 0..7 starting at an even column
    row = np.concatenate([lut[:8], [6.0], np.zeros(7)]).astype(np.float32)
    qa = NVFP4QWeight.from_float(torch.from_numpy(np.stack([top, row])).cuda())
    assert qa.weight_packed.cpu().numpy()[1, :4].tolist() == [h(b) for b in a["packed_bytes"]]

    # far above the grid: saturates at +-6
    sat = np.zeros((1, 16), dtype=np.float32)
    sat[0, 0], sat[0, 1] = 1e6, -1e6
    byte = int(NVFP4QWeight.from_float(torch.from_numpy(sat).cuda()).weight_packed[0, 0])
    assert (byte & 0xF, byte >> 4) == (7, 15)


# ------------------------------------------------- reference-made codec fixtures
#
# tests/golden/codec_fixtures.npz holds inputs and the outputs of the reference's
# pure-torch quantisers on them (written by tests/golden/make_codec_fixtures.py
# on the CPU).  The oracle is checked against them here; the HIP kernels are
# checked against them, through the C ABI, in the ``gpu`` test below.

FIXTURES = np.load(Path(__file__).parent / "golden" / "codec_fixtures.npz")
TORCH_DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}
ORACLE_DT = {"bf16": "bfloat16", "fp16": "float16", "fp32": "float32"}


def fixture_cases(fmt):
    return sorted({k.rsplit(".", 1)[0] for k in FIXTURES.files
                   if k.startswith(fmt + ".") and k.count(".") == 3})


def fx(case, key):
    return FIXTURES[f"{case}.{key}"]


def fixture_input(case):
    """(torch tensor in the case's dtype, the same values as fp32 numpy)."""
    dt = TORCH_DT[case.rsplit(".", 1)[1]]
    raw = fx(case, "x")
    if dt == torch.float32:
        t = torch.from_numpy(raw.view(np.float32).copy())
    else:
        t = torch.from_numpy(raw.view(np.int16).copy()).view(dt)
    return t, t.float().numpy()


def raw_bits(t):
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy().view(np.uint32)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def cast_bits(a_f32, dt):
    """fp32 numpy -> bits after torch's cast to ``dt``."""
    return raw_bits(torch.from_numpy(np.ascontiguousarray(a_f32, dtype=np.float32)).to(dt))


def test_fixture_file_covers_every_format_and_dtype():
    for fmt, n in (("int8", 13), ("int4", 13), ("nf4", 13), ("nvfp4", 13)):
        assert len(fixture_cases(fmt)) == n, (fmt, fixture_cases(fmt))
    assert np.array_equal(FIXTURES["nf4.lut"].view(np.float32),
                          np.array(GOLDEN["nf4_lut"], dtype=np.float32))
    assert np.array_equal(FIXTURES["nvfp4.lut"].view(np.float32),
                          np.array(GOLDEN["fp4_e2m1_lut"], dtype=np.float32))


@pytest.mark.parametrize("case", fixture_cases("int8"))
def test_oracle_int8_equals_reference_fixture(oracle, case):
    t, x = fixture_input(case)
    q, s = oracle.quant_int8(x)
    assert np.array_equal(q, fx(case, "codes"))
    assert np.array_equal(cast_bits(s, t.dtype), fx(case, "scales"))
    stored = torch.from_numpy(s.copy()).to(t.dtype).float().numpy()
    name = ORACLE_DT[case.rsplit(".", 1)[1]]
    got = oracle.dequant_int8(q, stored, name)
    assert np.array_equal(got.view(fx(case, "dequant").dtype), fx(case, "dequant"))
    assert np.array_equal(oracle.dequant_int8(q, stored, "float32").view(np.uint32),
                          fx(case, "dequant_f32"))


@pytest.mark.parametrize("case", fixture_cases("int4"))
def test_oracle_int4_equals_reference_fixture(oracle, case):
    t, x = fixture_input(case)
    group = int(fx(case, "group"))
    qw, s = oracle.quant_int4(x, group)
    assert np.array_equal(qw, fx(case, "qweight"))
    assert np.array_equal(cast_bits(s, t.dtype), fx(case, "scales"))
    # the reference's own unpacking of its words: (out_f, in_f) signed codes -8..7
    unpacked = fx(case, "unpacked").astype(np.int64)
    k = np.arange(x.shape[1])
    mine = ((qw.T.astype(np.int64)[:, k // 8] >> (4 * (k % 8))) & 0xF) - 8
    assert np.array_equal(mine, unpacked)
    # decoding multiplies those codes by the stored scale of their group
    stored = torch.from_numpy(s.copy()).to(t.dtype).float().numpy()
    want = unpacked.astype(np.float32) * np.repeat(stored.T, group, axis=1)
    assert np.array_equal(oracle.dequant_int4(qw, stored, group, "float32"), want)


@pytest.mark.parametrize("case", fixture_cases("nf4"))
def test_oracle_nf4_equals_reference_fixture(oracle, case):
    t, x = fixture_input(case)
    block = int(fx(case, "block"))
    packed, absmax = oracle.quant_nf4(x, block)
    assert np.array_equal(absmax.view(np.uint32), fx(case, "absmax"))
    assert np.array_equal(packed, fx(case, "packed"))
    assert np.array_equal(oracle.dequant_nf4(packed, absmax, block, "float32").view(np.uint32),
                          fx(case, "dequant_f32"))
    # 16-bit outputs are the fp32 product cast once (qweight/nf4.py:161-227)
    want = fx(case, "dequant_f32").view(np.float32)
    for dt, name in ((torch.bfloat16, "bfloat16"), (torch.float16, "float16")):
        assert np.array_equal(oracle.dequant_nf4(packed, absmax, block, name), cast_bits(want, dt))


@pytest.mark.parametrize("case", fixture_cases("nvfp4"))
def test_oracle_nvfp4_equals_reference_fixture(oracle, case):
    t, x = fixture_input(case)
    packed, s8, gs = oracle.quant_nvfp4(x)
    assert np.float32(gs).view(np.uint32) == fx(case, "global_scale")[0]
    assert np.array_equal(s8, fx(case, "block_scale"))
    assert np.array_equal(packed, fx(case, "packed"))
    for short, name in ORACLE_DT.items():
        want = fx(case, f"dequant_{short}")
        assert np.array_equal(oracle.dequant_nvfp4(packed, s8, gs, name).view(want.dtype), want)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["int8", "int4", "nf4", "nvfp4"])
def test_hip_codecs_equal_reference_fixtures(fmt):
    """The eight codec kernels, through the C ABI, on the fixtures' inputs."""
    from offload_adam_amd.qweight import _codec_ops as ops

    for case in fixture_cases(fmt):
        t, _ = fixture_input(case)
        rows, cols = t.shape
        src = t.cuda()
        sdt = torch.bfloat16 if t.dtype == torch.float32 else t.dtype
        if fmt == "int8":
            q = torch.empty(rows, cols, dtype=torch.int8, device="cuda")
            # the reference keeps the scales in the input's dtype (qweight/int8.py:49)
            s = torch.empty(rows, dtype=t.dtype, device="cuda")
            ops.quantize_int8_into(src, q, s)
            assert np.array_equal(q.cpu().numpy(), fx(case, "codes")), case
            assert np.array_equal(raw_bits(s), fx(case, "scales")), case
            assert np.array_equal(raw_bits(ops.dequantize_int8(q, s, t.dtype)),
                                  fx(case, "dequant")), case
            assert np.array_equal(raw_bits(ops.dequantize_int8(q, s, torch.float32)),
                                  fx(case, "dequant_f32")), case
        elif fmt == "int4":
            group = int(fx(case, "group"))
            qw = torch.empty(cols // 8, rows, dtype=torch.int32, device="cuda")
            s = torch.empty(cols // group, rows, dtype=t.dtype, device="cuda")
            ops.quantize_int4_into(src, group, qw, s)
            assert np.array_equal(qw.cpu().numpy(), fx(case, "qweight")), case
            assert np.array_equal(raw_bits(s), fx(case, "scales")), case
        elif fmt == "nf4":
            block = int(fx(case, "block"))
            packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
            absmax = torch.empty(rows * (cols // block), dtype=torch.float32, device="cuda")
            ops.quantize_nf4_into(src, block, packed, absmax)
            assert np.array_equal(raw_bits(absmax), fx(case, "absmax")), case
            assert np.array_equal(packed.cpu().numpy(), fx(case, "packed")), case
            assert np.array_equal(
                raw_bits(ops.dequantize_nf4(packed, absmax, cols, block, torch.float32)),
                fx(case, "dequant_f32")), case
        else:
            packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
            s8 = torch.empty(rows, cols // 16, dtype=torch.float8_e4m3fn, device="cuda")
            gs = torch.empty((), dtype=torch.float32, device="cuda")
            ops.quantize_nvfp4_into(src, packed, s8, gs)
            assert raw_bits(gs.reshape(1))[0] == fx(case, "global_scale")[0], case
            assert np.array_equal(raw_bits(s8), fx(case, "block_scale")), case
            assert np.array_equal(packed.cpu().numpy(), fx(case, "packed")), case
            for short, dt in TORCH_DT.items():
                assert np.array_equal(raw_bits(ops.dequantize_nvfp4(packed, s8, gs, cols, dt)),
                                      fx(case, f"dequant_{short}")), (case, short)
        del sdt


# ----------------------------------------------- Triton's own tl.randint words
#
# tests/golden/triton_randint.npz was written by Triton 3.6.0's interpreter on
# the CPU (tests/golden/make_triton_randint_fixture.py): the third-party code the
# reference calls at src/offload_adam/kernels/stochastic_rounding.py:77, not a
# restatement of it.

TRITON_WORDS = np.load(Path(__file__).parent / "golden" / "triton_randint.npz")


def test_oracle_randint_equals_tritons_own(oracle):
    lib = oracle.lib()
    seeds = [int(s) for s in TRITON_WORDS["seeds"]]
    far = [int(o) for o in TRITON_WORDS["far_offsets"]]
    assert len(seeds) == 6 and max(far) == (1 << 31) - 1
    for i, seed in enumerate(seeds):
        want = TRITON_WORDS[f"seed{i}_first4096"]
        got = np.array([lib.oaref_triton_randint(seed, o) for o in range(4096)], dtype=np.uint32)
        assert np.array_equal(got, want), hex(seed)
        # the 16 bits the update uses, through the array form the parity tests call
        assert np.array_equal(oracle.rand16_array(seed, 4096, 0), (want & 0xFFFF).astype(np.uint16))
        got_far = np.array([lib.oaref_triton_randint(seed, o) for o in far], dtype=np.uint32)
        assert np.array_equal(got_far, TRITON_WORDS[f"seed{i}_far"]), hex(seed)


@pytest.mark.gpu
def test_hip_reference_layout_uses_tritons_words():
    """The kernel's reference bit layout against the same kernel fed Triton's words
    as a buffer: identical parameters for every seed of the fixture."""
    from offload_adam_amd.kernels import adam_step_stochastic_rounding

    n = 4096
    g = torch.Generator().manual_seed(11)
    p0 = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16).cuda()
    st0 = {"grad": (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16).cuda(),
           "exp_avg": (torch.randn(n, generator=g) * 1e-4).to(torch.bfloat16).cuda(),
           "exp_avg_sq": (torch.randn(n, generator=g) * 1e-3).square().to(torch.bfloat16).cuda()}
    hyp = (1e-2, 0.01, 0.9, 0.999, 1e-8, 3)
    for i, seed in enumerate(int(s) for s in TRITON_WORDS["seeds"]):
        bits = (TRITON_WORDS[f"seed{i}_first4096"] & 0xFFFF).astype(np.uint16).view(np.int16)
        rand16 = torch.from_numpy(bits.copy()).cuda()
        pa, pb = p0.clone(), p0.clone()
        sa = {k: v.clone() for k, v in st0.items()}
        sb = {k: v.clone() for k, v in st0.items()}
        adam_step_stochastic_rounding(pa, sa, *hyp, seed=seed, rng="triton")
        adam_step_stochastic_rounding(pb, sb, *hyp, seed=0, rng="buffer", rand16=rand16)
        assert torch.equal(pa.view(torch.int16), pb.view(torch.int16)), hex(seed)
        assert not torch.equal(pa.view(torch.int16), p0.view(torch.int16))
