"""GPU parity of the fp32_master AdamW step fused with re-encoding of a
quantised weight (oa_adam_requant_*), through the C ABI.

Expected results come from the C oracle run as the reference runs the two
moves: the fp32_master step, then the encoder of the format on the new master
(src/offload_adam/offload_adam.py:421-444).  Everything is BIT-EXACT: moments,
master and every payload tensor.
"""

import numpy as np
import pytest
import torch

from helpers import HYP, adam_inputs, bits

pytestmark = pytest.mark.gpu

FORMATS = ["int8", "int4", "nf4", "nvfp4"]
# (rows, cols): one block per row / several tiles / ragged row counts / a row longer
# than the int8 register cache (256 lanes x 8 octets x 8 = 16384 columns)
SHAPES = [(1, 128), (5, 256), (64, 128), (67, 384), (130, 1024), (3, 16384 + 512)]


def _weight(fmt, rows, cols, seed):
    from offload_adam_amd.qweight import Int4QWeight, Int8QWeight, NF4QWeight, NVFP4QWeight

    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(rows, cols, generator=g) * 0.02).to(torch.bfloat16).cuda()
    if fmt == "int8":
        return Int8QWeight.from_float(w)
    if fmt == "int4":
        return Int4QWeight.from_float(w, group_size=128)
    if fmt == "nf4":
        return NF4QWeight.from_float(w, blocksize=64)
    return NVFP4QWeight.from_float(w)


def _payload_bits(qw):
    out = {}
    for name in qw._PAYLOAD:
        t = getattr(qw, name).detach().cpu().contiguous()
        if t.dtype in (torch.bfloat16, torch.float16):
            t = t.view(torch.int16)
        elif t.dtype is torch.float8_e4m3fn:
            t = t.view(torch.uint8)
        elif t.dtype is torch.float32:
            t = t.view(torch.int32)
        out[name] = t.numpy().copy()
    return out


def _oracle_expected(oracle, fmt, qw, st, decoupled, clip_bits, hyp=HYP):
    """Oracle step on numpy copies, then the oracle encoder on the new master."""
    rows, cols = qw.shape
    b1h, b2h = oracle.folded_betas(hyp["beta1"], hyp["beta2"], hyp["step"])
    g, m, v = bits(st["grad"]), bits(st["exp_avg"]), bits(st["exp_avg_sq"])
    sink = np.zeros_like(g)
    master = st["master_params"].cpu().numpy().reshape(-1).copy()
    oracle.adam_fp32_master(sink, g, m, v, master, hyp["lr"], hyp["weight_decay"], b1h, b2h,
                            hyp["eps"], decoupled, clip=clip_bits)
    x = master.reshape(rows, cols)
    exp = {"exp_avg": m, "exp_avg_sq": v, "master": master.view(np.uint32)}
    scale_dt = torch.bfloat16

    def cast(s):
        return torch.from_numpy(np.ascontiguousarray(s)).to(scale_dt).view(torch.int16).numpy()

    if fmt == "int8":
        q, s = oracle.quant_int8(x)
        exp["payload"] = {"weight": q, "scales": cast(s)}
    elif fmt == "int4":
        qw_, s = oracle.quant_int4(x, group=128)
        exp["payload"] = {"qweight": qw_, "scales": cast(s)}
    elif fmt == "nf4":
        pk, am = oracle.quant_nf4(x, block=64)
        exp["payload"] = {"weight_packed": pk, "absmax": am.view(np.int32)}
    else:
        pk, s8, gs = oracle.quant_nvfp4(x)
        exp["payload"] = {"weight_packed": pk, "block_scale_fp8": s8,
                          "global_scale": np.asarray(gs, dtype=np.float32).view(np.int32)}
    return exp


def _check(qw, st, exp, ctx):
    assert np.array_equal(bits(st["exp_avg"]), exp["exp_avg"]), ctx + " exp_avg"
    assert np.array_equal(bits(st["exp_avg_sq"]), exp["exp_avg_sq"]), ctx + " exp_avg_sq"
    assert np.array_equal(st["master_params"].cpu().numpy().reshape(-1).view(np.uint32),
                          exp["master"]), ctx + " master"
    got = _payload_bits(qw)
    for name, want in exp["payload"].items():
        g = got[name]
        assert np.array_equal(g.reshape(-1).view(want.dtype), want.reshape(-1)), f"{ctx} {name}"


def _states(rows, cols, seed):
    p, st = adam_inputs(rows * cols, seed=seed, mode="fp32_master", device="cuda")
    return {k: v.reshape(rows, cols) for k, v in st.items()}


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("shape", SHAPES)
def test_fused_step_matches_oracle_step_then_encode(oracle, fmt, shape):
    from offload_adam_amd.kernels.qat_step import adam_step_requant

    rows, cols = shape
    for decoupled, clip in ((True, None), (False, 0.3359375)):
        qw = _weight(fmt, rows, cols, seed=rows + cols)
        st = _states(rows, cols, seed=7 * rows + cols)
        before = bits(st["grad"])
        clip_t = None if clip is None else torch.tensor(clip, dtype=torch.bfloat16, device="cuda")
        clip_bits = None if clip is None else bits(clip_t.reshape(1))
        exp = _oracle_expected(oracle, fmt, qw, st, decoupled, clip_bits)
        done = adam_step_requant(qw, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"],
                                 HYP["beta2"], HYP["eps"], HYP["step"], decoupled, clip_t)
        torch.cuda.synchronize()
        assert done, "these layouts are inside what the fused kernels cover"
        _check(qw, st, exp, f"{fmt} {shape} decoupled={decoupled} clip={clip}")
        assert np.array_equal(bits(st["grad"]), before), "the gradient is read-only"


@pytest.mark.parametrize("fmt", FORMATS)
def test_step_function_dispatch_equals_two_moves(oracle, fmt):
    """adam_step_fp32_master given the quantised weight = the step with a sink
    followed by copy_(master), as the reference's optimizers do it."""
    from offload_adam_amd.kernels import adam_step_fp32_master

    rows, cols = 96, 512
    args = (HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"], HYP["eps"], HYP["step"])
    qa, qb = _weight(fmt, rows, cols, 3), _weight(fmt, rows, cols, 3)
    sa, sb = _states(rows, cols, 11), _states(rows, cols, 11)
    adam_step_fp32_master(qa, sa, *args, decoupled_weight_decay=True)
    sink = sb["grad"].clone()
    adam_step_fp32_master(sink, dict(sb, grad=sb["grad"]), *args, decoupled_weight_decay=True)
    qb.copy_(sb["master_params"])
    torch.cuda.synchronize()
    for k in ("exp_avg", "exp_avg_sq"):
        assert torch.equal(sa[k], sb[k])
    assert torch.equal(sa["master_params"], sb["master_params"])
    pa, pb = _payload_bits(qa), _payload_bits(qb)
    for name in pa:
        assert np.array_equal(pa[name], pb[name]), name
    assert torch.equal(qa.dequantize(torch.float32), qb.dequantize(torch.float32))


def test_no_sink_step_equals_step_with_sink(oracle):
    from offload_adam_amd.kernels import adam_step_fp32_master

    args = (HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"], HYP["eps"], HYP["step"])
    for n in (1, 7, 8, 4099, (1 << 20) + 3):
        p, sa = adam_inputs(n, seed=n, mode="fp32_master", device="cuda")
        _, sb = adam_inputs(n, seed=n, mode="fp32_master", device="cuda")
        adam_step_fp32_master(None, sa, *args, decoupled_weight_decay=True)
        adam_step_fp32_master(p, sb, *args, decoupled_weight_decay=True)
        torch.cuda.synchronize()
        for k in ("exp_avg", "exp_avg_sq", "master_params", "grad"):
            assert torch.equal(sa[k], sb[k]), (n, k)


def test_layouts_outside_the_fused_kernels_take_two_launches(oracle):
    """cols % 8 != 0 (int8 allows cols % 4 == 0): the dispatcher declines and the
    step function falls back to step + copy_; results still match the oracle."""
    from offload_adam_amd.kernels import adam_step_fp32_master
    from offload_adam_amd.kernels.qat_step import adam_step_requant
    from offload_adam_amd.qweight import Int8QWeight

    rows, cols = 9, 36
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(rows, cols, generator=g) * 0.02).to(torch.bfloat16).cuda()
    qw = Int8QWeight.from_float(w)
    st = _states(rows, cols, 13)
    snapshot = {k: v.clone() for k, v in st.items()}
    assert adam_step_requant(qw, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"],
                             HYP["eps"], HYP["step"], True, None) is False
    for k in st:
        assert torch.equal(st[k], snapshot[k]), "a declined call touches nothing"
    exp = _oracle_expected(oracle, "int8", qw, st, True, None)
    adam_step_fp32_master(qw, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"],
                          HYP["eps"], HYP["step"], decoupled_weight_decay=True)
    torch.cuda.synchronize()
    _check(qw, st, exp, "int8 9x36 fallback")


def test_entry_points_reject_bad_arguments():
    from ctypes import c_float, c_int, c_int64, c_void_p

    from offload_adam_amd import _lib

    lib = _lib.load()
    n = 64 * 128
    bufs = [torch.zeros(n, dtype=torch.bfloat16, device="cuda") for _ in range(3)]
    master = torch.zeros(n, dtype=torch.float32, device="cuda")
    q = torch.zeros(n, dtype=torch.int8, device="cuda")
    sc = torch.zeros(64, dtype=torch.bfloat16, device="cuda")

    def call(g, m, v, M, rows, cols):
        return lib.oa_adam_requant_int8(
            _lib.ptr(g), _lib.ptr(m), _lib.ptr(v), _lib.ptr(M), c_int64(rows), c_int64(cols),
            c_float(1e-3), c_float(0.0), c_float(0.9), c_float(0.99), c_float(1e-8), c_int(1),
            c_void_p(None), _lib.ptr(q), _lib.ptr(sc), c_int(_lib.dtype_code(torch.bfloat16)),
            _lib.current_stream_ptr())

    assert call(bufs[0], bufs[1], bufs[2], master, 64, 128) == 0
    assert call(bufs[0], bufs[1], bufs[1], master, 64, 128) != 0      # exp_avg aliases exp_avg_sq
    assert call(bufs[0], bufs[0], bufs[2], master, 64, 128) != 0      # grad aliases a written array
    assert call(bufs[0], bufs[1], bufs[2], master, 64, 124) != 0      # cols % 8
    assert call(None, bufs[1], bufs[2], master, 64, 128) != 0
    assert call(bufs[0], bufs[1], bufs[2], master, 0, 128) == 0       # empty: nothing to do
    torch.cuda.synchronize()
