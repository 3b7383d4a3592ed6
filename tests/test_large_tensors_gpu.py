"""Tensors of more than 2^31 elements: every index in the kernels is 64-bit, and
nothing but a run at that size shows it.  A 288 GB part holds such tensors easily
(a 131072 x 16400 embedding is one).

An elementwise update of the whole tensor must equal the same update of its two
halves (each below 2^31 elements); the counter-based random bits, which depend on
the global element index, are checked against the oracle on windows at the start,
across the 2^31 boundary and at the ragged end; reductions and codecs are checked
against the oracle / fp64 on windows and by row blocks.
"""

import sys
from pathlib import Path

import numpy as np
import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16
N = (1 << 31) + 4099          # ragged: the scalar tail path runs too
HALF = 1 << 30                # a 16-byte aligned split for every array
HYP = (1e-2, 0.01, 0.9, 0.999, 1e-8, 3)


def u16(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy()


def fill_normal(t, std, gen):
    """In place and in pieces: randn of 2^31 elements in fp32 would take 8.6 GB more."""
    step = 1 << 28
    for s in range(0, t.numel(), step):
        piece = t[s:s + step]
        piece.copy_(torch.randn(piece.numel(), device="cuda", generator=gen) * std)


@pytest.fixture(scope="module")
def operands():
    if torch.cuda.mem_get_info()[0] < 80 << 30:
        pytest.skip("needs 80 GB of free HBM")
    gen = torch.Generator(device="cuda").manual_seed(0)
    out = {}
    for name, std in (("p", 0.02), ("grad", 1e-3), ("exp_avg", 1e-4), ("exp_avg_sq", 1e-3)):
        t = torch.empty(N, dtype=BF16, device="cuda")
        fill_normal(t, std, gen)
        out[name] = t
    out["exp_avg_sq"].abs_()
    yield out
    out.clear()
    torch.cuda.empty_cache()


def clones(operands, extra=None):
    p = operands["p"].clone()
    st = {k: operands[k].clone() for k in ("grad", "exp_avg", "exp_avg_sq")}
    if extra is not None:
        st.update(extra)
    return p, st


def sliced(p, st, lo, hi):
    return p[lo:hi], {k: v[lo:hi] for k, v in st.items()}


@pytest.mark.parametrize("mode", ["fp32_master", "fp31_master", "fp32_master_custom_rounding"])
def test_update_of_the_whole_equals_the_update_of_its_halves(operands, mode):
    from offload_adam_amd import kernels

    fn = {"fp32_master": kernels.adam_step_fp32_master,
          "fp31_master": kernels.adam_step_fp31_master,
          "fp32_master_custom_rounding": kernels.adam_step_fp32_master_custom_rounding}[mode]

    def extra():
        if mode == "fp32_master":
            return {"master_params": operands["p"].float()}
        gen = torch.Generator(device="cuda").manual_seed(5)
        return {"rounding_error": torch.randint(-1000, 1000, (N,), device="cuda", generator=gen,
                                                dtype=torch.int16)}

    pw, sw = clones(operands, extra())
    fn(pw, sw, *HYP, decoupled_weight_decay=True)
    ph, sh = clones(operands, extra())
    for lo, hi in ((0, HALF), (HALF, N)):
        fn(*sliced(ph, sh, lo, hi), *HYP, decoupled_weight_decay=True)
    torch.cuda.synchronize()
    assert torch.equal(pw.view(torch.int16), ph.view(torch.int16))
    for k in sw:
        if k != "grad":
            a, b = sw[k], sh[k]
            assert torch.equal(a.view(torch.int32) if a.dtype == torch.float32 else a.view(torch.int16),
                               b.view(torch.int32) if b.dtype == torch.float32 else b.view(torch.int16)), k
    # and something happened past the 2^31st element
    assert not torch.equal(pw[-4099:].view(torch.int16), operands["p"][-4099:].view(torch.int16))


@pytest.mark.parametrize("rng,layout", [("triton", 0), ("x8", 1)])
def test_random_bits_follow_the_global_element_index(oracle, operands, rng, layout):
    """Stochastic rounding of the whole tensor against the oracle on three windows:
    the start, across element 2^31 and the ragged end."""
    from offload_adam_amd.kernels import adam_step_stochastic_rounding

    seed = 0x0123456789ABCDEF
    p, st = clones(operands)
    adam_step_stochastic_rounding(p, st, *HYP, seed=seed, decoupled_weight_decay=True, rng=rng)
    torch.cuda.synchronize()
    b1h, b2h = oracle.folded_betas(HYP[2], HYP[3], HYP[5])
    for lo, hi in ((0, 4096), ((1 << 31) - 2051, (1 << 31) + 2053), (N - 4099, N)):
        want_p = u16(operands["p"][lo:hi])
        want_m = u16(operands["exp_avg"][lo:hi])
        want_v = u16(operands["exp_avg_sq"][lo:hi])
        bits = oracle.rand16_array(seed, hi - lo, layout, start=lo)
        oracle.adam_stochastic_rounding(want_p, u16(operands["grad"][lo:hi]), want_m, want_v,
                                        HYP[0], HYP[1], b1h, b2h, HYP[4], True, layout=2,
                                        rand16=bits)
        assert np.array_equal(u16(p[lo:hi]), want_p), (rng, lo)
        assert np.array_equal(u16(st["exp_avg"][lo:hi]), want_m), (rng, lo)
        assert np.array_equal(u16(st["exp_avg_sq"][lo:hi]), want_v), (rng, lo)


def test_stochastic_rounding_from_a_buffer_whole_against_halves(operands):
    from offload_adam_amd.kernels import adam_step_stochastic_rounding

    gen = torch.Generator(device="cuda").manual_seed(9)
    rand16 = torch.randint(-32768, 32767, (N,), device="cuda", generator=gen, dtype=torch.int16)
    pw, sw = clones(operands)
    adam_step_stochastic_rounding(pw, sw, *HYP, seed=0, decoupled_weight_decay=True,
                                  rng="buffer", rand16=rand16)
    ph, sh = clones(operands)
    for lo, hi in ((0, HALF), (HALF, N)):
        q, s = sliced(ph, sh, lo, hi)
        adam_step_stochastic_rounding(q, s, *HYP, seed=0, decoupled_weight_decay=True,
                                      rng="buffer", rand16=rand16[lo:hi])
    torch.cuda.synchronize()
    assert torch.equal(pw.view(torch.int16), ph.view(torch.int16))


def test_gradient_norm_of_more_than_2_31_elements(operands):
    from offload_adam_amd.grad_clip import grad_norm_

    g = operands["grad"]
    out = torch.zeros((), dtype=BF16, device="cuda")
    grad_norm_(g, out)
    exact = 0.0
    step = 1 << 28
    for s in range(0, N, step):
        exact += float(g[s:s + step].double().square().sum())
    exact = exact ** 0.5
    near = torch.tensor(exact, dtype=torch.float32).to(BF16)
    got = int(out.view(torch.int16)) & 0xFFFF
    assert abs(got - (int(near.view(torch.int16)) & 0xFFFF)) <= 1, (float(out), exact)
    # the last 4099 elements count: a huge value there must show
    g2 = g.clone()
    g2[-1] = 1000.0
    grad_norm_(g2, out)
    assert float(out) > 999.0


ROWS, COLS = 32776, 65536     # 2,148,007,936 elements; every format's blocks divide COLS


@pytest.fixture(scope="module")
def big_weight():
    if torch.cuda.mem_get_info()[0] < 80 << 30:
        pytest.skip("needs 80 GB of free HBM")
    gen = torch.Generator(device="cuda").manual_seed(3)
    w = torch.empty(ROWS * COLS, dtype=BF16, device="cuda")
    fill_normal(w, 0.02, gen)
    w = w.view(ROWS, COLS)
    w[0, 0] = 3.0  # the tensor-wide maximum sits in the first checked window (NVFP4's scale)
    yield w
    del w
    torch.cuda.empty_cache()


# rows: the first; the last, which straddle element 2^31 (row 32768); those around element 2^30
WINDOWS = ((0, 8), (32760, 32776), (16380, 16392))


def rows_f32(w, lo, hi):
    return w[lo:hi].float().cpu().numpy()


def test_int8_codec_on_more_than_2_31_elements(oracle, big_weight):
    from offload_adam_amd.qweight import _codec_ops as ops

    q = torch.empty(ROWS, COLS, dtype=torch.int8, device="cuda")
    s = torch.empty(ROWS, dtype=BF16, device="cuda")
    ops.quantize_int8_into(big_weight, q, s)
    back = ops.dequantize_int8(q, s, BF16)
    for lo, hi in WINDOWS:
        want_q, want_s = oracle.quant_int8(rows_f32(big_weight, lo, hi))
        assert np.array_equal(q[lo:hi].cpu().numpy(), want_q), lo
        s_bits = oracle.narrow_array(want_s, "bfloat16")
        assert np.array_equal(u16(s[lo:hi]), s_bits), lo
        s_f32 = (s_bits.astype(np.uint32) << 16).view(np.float32)
        assert np.array_equal(u16(back[lo:hi]), oracle.dequant_int8(want_q, s_f32).reshape(-1)), lo


def test_int4_codec_on_more_than_2_31_elements(oracle, big_weight):
    from offload_adam_amd.qweight import _codec_ops as ops

    g = 128
    qw = torch.empty(COLS // 8, ROWS, dtype=torch.int32, device="cuda")
    s = torch.empty(COLS // g, ROWS, dtype=BF16, device="cuda")
    ops.quantize_int4_into(big_weight, g, qw, s)
    back = ops.dequantize_int4(qw, s, g, BF16)
    for lo, hi in WINDOWS:
        want_qw, want_s = oracle.quant_int4(rows_f32(big_weight, lo, hi), g)
        assert np.array_equal(qw[:, lo:hi].cpu().numpy(), want_qw), lo
        s_bits = oracle.narrow_array(want_s.reshape(-1), "bfloat16").reshape(want_s.shape)
        assert np.array_equal(u16(s[:, lo:hi]).reshape(want_s.shape), s_bits), lo
        s_f32 = (s_bits.astype(np.uint32) << 16).view(np.float32)
        assert np.array_equal(u16(back[lo:hi]),
                              oracle.dequant_int4(want_qw, s_f32, g).reshape(-1)), lo


def test_nf4_codec_on_more_than_2_31_elements(oracle, big_weight):
    from offload_adam_amd.qweight import _codec_ops as ops

    bs = 64
    packed = torch.empty(ROWS, COLS // 2, dtype=torch.uint8, device="cuda")
    absmax = torch.empty(ROWS * (COLS // bs), dtype=torch.float32, device="cuda")
    ops.quantize_nf4_into(big_weight, bs, packed, absmax)
    back = ops.dequantize_nf4(packed, absmax, COLS, bs, BF16)
    per_row = COLS // bs
    for lo, hi in WINDOWS:
        want_p, want_a = oracle.quant_nf4(rows_f32(big_weight, lo, hi), bs)
        assert np.array_equal(packed[lo:hi].cpu().numpy(), want_p), lo
        got_a = absmax[lo * per_row:hi * per_row].cpu().numpy()
        assert np.array_equal(got_a.view(np.uint32), want_a.view(np.uint32)), lo
        assert np.array_equal(u16(back[lo:hi]), oracle.dequant_nf4(want_p, want_a, bs).reshape(-1)), lo


def test_nvfp4_codec_on_more_than_2_31_elements(oracle, big_weight):
    from offload_adam_amd.qweight import _codec_ops as ops

    packed = torch.empty(ROWS, COLS // 2, dtype=torch.uint8, device="cuda")
    scale8 = torch.empty(ROWS, COLS // 16, dtype=torch.float8_e4m3fn, device="cuda")
    gs = torch.empty((), dtype=torch.float32, device="cuda")
    ops.quantize_nvfp4_into(big_weight, packed, scale8, gs)
    back = ops.dequantize_nvfp4(packed, scale8, gs, COLS, BF16)
    assert float(big_weight.abs().max()) == 3.0
    first = True
    for lo, hi in WINDOWS:
        x = rows_f32(big_weight, lo, hi)
        if not first:
            x[0, 0] = 3.0  # same tensor-wide maximum as the whole (only this element differs)
        want_p, want_s, want_gs = oracle.quant_nvfp4(x)
        if first:
            assert np.float32(float(gs)).view(np.uint32) == want_gs.view(np.uint32)
        got_p = packed[lo:hi].cpu().numpy()
        got_s = scale8[lo:hi].view(torch.uint8).cpu().numpy()
        skip = 0 if first else 1  # the planted element's block: 8 bytes of codes, 1 scale
        assert np.array_equal(got_p.reshape(-1)[8 * skip:], want_p.reshape(-1)[8 * skip:]), lo
        assert np.array_equal(got_s.reshape(-1)[skip:], want_s.reshape(-1)[skip:]), lo
        want_back = oracle.dequant_nvfp4(got_p, got_s, want_gs).reshape(-1)
        assert np.array_equal(u16(back[lo:hi]), want_back), lo
        first = False


@pytest.mark.parametrize("fmt", ["int8", "int4", "nf4", "nvfp4"])
def test_fused_step_and_reencode_on_more_than_2_31_elements(big_weight, fmt):
    """``adam_step_fp32_master`` on a quantised weight (one pass: step + payload) against
    the plain step followed by ``copy_(master)``, whole tensors compared on the GPU."""
    from offload_adam_amd import qweight
    from offload_adam_amd.kernels import adam_step_fp32_master

    cls = {"int8": qweight.Int8QWeight, "int4": qweight.Int4QWeight,
           "nf4": qweight.NF4QWeight, "nvfp4": qweight.NVFP4QWeight}[fmt]
    gen = torch.Generator(device="cuda").manual_seed(21)

    def states():
        st = {}
        for name, std in (("grad", 1e-3), ("exp_avg", 1e-4), ("exp_avg_sq", 1e-3)):
            t = torch.empty(ROWS * COLS, dtype=BF16, device="cuda")
            fill_normal(t, std, gen)
            st[name] = t.view(ROWS, COLS)
        st["exp_avg_sq"].abs_()
        st["master_params"] = big_weight.float()
        return st

    fused_w, plain_w = cls.from_float(big_weight), cls.from_float(big_weight)
    fused_st = states()
    plain_st = {k: v.clone() for k, v in fused_st.items()}
    adam_step_fp32_master(fused_w, fused_st, *HYP, decoupled_weight_decay=True)
    adam_step_fp32_master(None, plain_st, *HYP, decoupled_weight_decay=True)
    plain_w.copy_(plain_st["master_params"])
    torch.cuda.synchronize()

    def same(a, b):
        if a.dtype == torch.float8_e4m3fn:
            a, b = a.view(torch.uint8), b.view(torch.uint8)
        elif a.is_floating_point():
            a = a.view(torch.int32 if a.element_size() == 4 else torch.int16)
            b = b.view(a.dtype)
        return torch.equal(a, b)

    for k in ("exp_avg", "exp_avg_sq", "master_params"):
        assert same(fused_st[k], plain_st[k]), k
    for name in cls._PAYLOAD:
        assert same(getattr(fused_w, name), getattr(plain_w, name)), name
    # the payload moved, also past element 2^31
    before = cls.from_float(big_weight[-8:].contiguous())
    first = cls._PAYLOAD[0]
    tail = getattr(cls.from_float(fused_st["master_params"][-8:].contiguous()), first)
    assert not same(getattr(before, first), tail)
