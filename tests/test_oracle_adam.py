"""Pins the CPU oracle of the AdamW / stochastic-rounding / split-master /
norm-clip path (rows A and B of the hot path) WITHOUT the reference being
importable: known-answer vectors, exhaustive bit-level checks, closed forms,
fp64 evaluation, torch's own optimizers, and a second restatement in torch
eager that must agree bit for bit.  Runs on CPU.
"""

import math

import numpy as np
import pytest
import torch

from helpers import HYP, adam_inputs, bits, from_bf16_bits

BF16 = torch.bfloat16
MODES = ["fp32_master", "stochastic_rounding", "fp31_master", "fp32_master_custom_rounding"]


# ------------------------------------------------------------------ Philox


def test_philox_random123_known_answers(oracle):
    """Random123 kat_vectors for philox4x32-10."""
    assert oracle.philox((0, 0, 0, 0), (0, 0)) == (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)
    f = 0xFFFFFFFF
    assert oracle.philox((f, f, f, f), (f, f)) == (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)
    assert oracle.philox((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344),
                         (0xA4093822, 0x299F31D0)) == (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)


def test_triton_randint_layout(oracle):
    """counter = (offset, 0, 0, 0), key = (seed_lo, seed_hi), word 0: vectors for
    seed 0x0123456789ABCDEF derived from the KAT-verified block function."""
    seed = 0x0123456789ABCDEF
    want = {0: 0xB850222E, 1: 0xADCA1466, 2: 0xF7CE299F, 1023: 0xD4112EF7,
            1024: 0xA399E2E0, 16777215: 0xE3DB3EA0}
    L = oracle.lib()
    for off, w in want.items():
        assert L.oaref_triton_randint(seed, off) == w
        assert oracle.philox((off, 0, 0, 0), (seed & 0xFFFFFFFF, seed >> 32))[0] == w
        assert L.oaref_rand16(seed, off, 0) == w & 0xFFFF


def test_x8_layout_is_a_partition_of_philox_blocks(oracle):
    """Layout 1: element i takes 16 bits of block i//8 (counter (j,0,1,0))."""
    seed = 0xDEADBEEFCAFEF00D
    r = oracle.rand16_array(seed, 64, 1)
    for j in range(8):
        words = oracle.philox((j, 0, 1, 0), (seed & 0xFFFFFFFF, seed >> 32))
        flat = []
        for w in words:
            flat += [w & 0xFFFF, w >> 16]
        assert list(r[8 * j:8 * j + 8]) == flat
    # uniformity smoke check on many draws
    big = oracle.rand16_array(seed, 1 << 18, 1).astype(np.float64)
    assert abs(big.mean() - 32767.5) < 200


# ---------------------------------------------------- stochastic rounding


def test_sr_round_exhaustive(oracle):
    """All 65536 low halves x edge draws x both signs x exponent edges against
    the value-level definition: keep the truncated bf16 unless r < frac, then
    step the magnitude to the next bf16."""
    fracs = np.arange(65536, dtype=np.uint32)
    highs = [0x3F80, 0xBF80, 0x0000, 0x8000, 0x0080, 0x3FFF, 0x7F7E, 0x7F7F, 0x0001, 0xC2FF]
    for hi in highs:
        x = ((np.uint32(hi) << 16) | fracs).view(np.float32)
        for rsel in ("zero", "frac-1", "frac", "max"):
            r = {"zero": np.zeros(65536, np.uint32), "frac-1": np.maximum(fracs, 1) - 1,
                 "frac": fracs, "max": np.full(65536, 0xFFFF, np.uint32)}[rsel]
            got = oracle.sr_round_array(np.ascontiguousarray(x), r.astype(np.uint16))
            up = r < fracs
            want = (np.uint32(hi) + up.astype(np.uint32)).astype(np.uint16)
            assert np.array_equal(got, want), (hex(hi), rsel)
    # r = 0xFFFF never rounds up; r = 0 rounds up whenever frac != 0; frac = 0 never moves
    # (all covered by the table above).  max-finite + up -> inf is the carry case:
    assert oracle.lib().oaref_sr_round(np.float32(np.uint32(0x7F7F0001).view(np.float32)), 0) == 0x7F80


def test_sr_round_unbiased_and_within_one_ulp(oracle):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(2000) * 0.02).astype(np.float32)
    acc = np.zeros_like(x, dtype=np.float64)
    trials = 2000
    lo = (x.view(np.uint32) & 0xFFFF0000).view(np.float32).astype(np.float64)
    hi = ((x.view(np.uint32) & 0xFFFF0000) + 0x10000).astype(np.uint32).view(np.float32).astype(np.float64)
    for t in range(trials):
        r = oracle.rand16_array(1234 + t, x.size, 0)
        out = (oracle.sr_round_array(x, r).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        assert np.all((out == lo) | (out == hi))
        acc += out
    ulp = np.abs(hi - lo)
    assert np.all(np.abs(acc / trials - x) <= 6 * ulp / 2 / math.sqrt(trials))


# ------------------------------------------------------ split master forms


def _all_low_halves(highs):
    lows = np.arange(65536, dtype=np.uint32)
    return np.concatenate([(np.uint32(h) << 16) | lows for h in highs])


HIGHS = [0x3F80, 0xBF80, 0x3C23, 0xBC23, 0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080,
         0x3FFF, 0xBFFF, 0x7F00, 0xFF00, 0x4000, 0x1234, 0x9ABC]


def test_fp31_split_round_trip(oracle):
    x = _all_low_halves(HIGHS)
    p, e, recon = oracle.split_array(x, "fp31")
    L = oracle.lib()
    x31 = np.array([L.oaref_round_to_fp31(int(v)) for v in x[::97]], dtype=np.uint32)
    assert np.array_equal(recon[::97], x31)
    # independent statement of round-to-31-bits, ties to even on bit 0 (two's
    # complement integer arithmetic, as the reference does it)
    xi = x.view(np.int32).astype(np.int64)
    want = (((xi >> 1) + ((xi & 1) & ((xi >> 1) & 1))) << 1) & 0xFFFFFFFF
    assert np.array_equal(recon.astype(np.int64), want)
    assert e.min() >= -16384 and e.max() <= 16384
    assert np.all(recon & 1 == 0)
    # idempotent: splitting the reconstruction gives the same pair
    p2, e2, recon2 = oracle.split_array(recon, "fp31")
    assert np.array_equal(p2, p) and np.array_equal(e2, e) and np.array_equal(recon2, recon)
    # the bf16 half is the round-to-nearest-even of the 31-bit value (torch's cast)
    t = torch.from_numpy(recon.view(np.float32).copy()).to(BF16)
    assert np.array_equal(bits(t), p)
    # ties table on the two low bits: 00->00, 01->00, 10->10, 11->+1 (to even)
    for low, out in [(0b00, 0x3F800000), (0b01, 0x3F800000), (0b10, 0x3F800002), (0b11, 0x3F800004)]:
        assert L.oaref_round_to_fp31(0x3F800000 | low) == out
    # err = 0 reconstructs float(p)
    assert L.oaref_fp31_reconstruct(0x3F80, 0) == 1.0


def test_custom_split_round_trip(oracle):
    x = _all_low_halves(HIGHS)
    p, e, recon = oracle.split_array(x, "custom")
    assert np.array_equal(recon, x), "lossless for every bit pattern"
    assert e.min() == -32768 and e.max() == 32767
    # bf16 half = (bits + 0x8000) >> 16: round half up in magnitude
    want_p = (((x.astype(np.uint64) + 0x8000) >> 16) & 0xFFFF).astype(np.uint16)
    assert np.array_equal(p, want_p)


# ------------------------------------------------------------ Adam update


def test_folded_beta_closed_forms(oracle):
    for beta in (0.9, 0.999, 0.95):
        for t in (1, 2, 10, 1000):
            got = oracle.folded_betas(beta, beta, t)[0]
            if t == 1:
                assert got == 0.0
            else:
                assert got == pytest.approx(beta * (1 - beta ** (t - 1)) / (1 - beta**t), rel=1e-12)
    b1, b2 = oracle.folded_betas(0.9, 0.999, 10)
    assert b1 == pytest.approx(0.846466006721237, rel=1e-12)
    assert b2 == pytest.approx(0.8995491745886153, rel=1e-12)


def _run_oracle(oracle, mode, p, st, hyp, decoupled, clip_bits=None, seed=0, layout=0):
    b1h, b2h = oracle.folded_betas(hyp["beta1"], hyp["beta2"], hyp["step"])
    pb, g, m, v = bits(p), bits(st["grad"]), bits(st["exp_avg"]), bits(st["exp_avg_sq"])
    args = (hyp["lr"], hyp["weight_decay"], b1h, b2h, hyp["eps"], decoupled)
    out = {}
    if mode == "fp32_master":
        M = st["master_params"].numpy().copy()
        oracle.adam_fp32_master(pb, g, m, v, M, *args, clip=clip_bits)
        out["master_params"] = M
    elif mode == "stochastic_rounding":
        oracle.adam_stochastic_rounding(pb, g, m, v, *args, seed=seed, layout=layout, clip=clip_bits)
    else:
        e = st["rounding_error"].numpy().copy()
        (oracle.adam_fp31_master if mode == "fp31_master" else oracle.adam_custom_rounding)(
            pb, g, m, v, e, *args, clip=clip_bits)
        out["rounding_error"] = e
    out.update(param=pb, exp_avg=m, exp_avg_sq=v)
    return out


def test_first_step_closed_form(oracle):
    """t = 1 (beta_hat = 0), zero moments, wd = 0:  M' = M - lr * g / (|g| + eps)
    up to the rounding of sqrt(g*g); moments become g and g*g."""
    n = 4096
    p, st = adam_inputs(n, 1, "fp32_master")
    st["exp_avg"].zero_()
    st["exp_avg_sq"].zero_()
    hyp = dict(HYP, step=1, weight_decay=0.0)
    out = _run_oracle(oracle, "fp32_master", p, st, hyp, False)
    g = st["grad"].double()
    M0 = st["master_params"].double()
    lr32, eps32 = float(np.float32(hyp["lr"])), float(np.float32(hyp["eps"]))
    want = M0 - lr32 * g / (g.abs() + eps32)
    got = torch.from_numpy(out["master_params"]).double()
    # one ulp of the largest operand of the final subtraction (it can cancel)
    scale = np.maximum(np.abs(out["master_params"]), np.abs(st["master_params"].numpy()))
    ulp = torch.from_numpy(np.spacing(np.maximum(scale, np.float32(hyp["lr"])))).double()
    # g*g, sqrt, the product and the quotient each round once before the subtraction
    assert bool(((got - want).abs() <= 2 * ulp).all())
    assert np.array_equal(out["exp_avg"], bits(st["grad"]))
    assert np.array_equal(out["exp_avg_sq"], bits((st["grad"].float() ** 2).to(BF16)))


@pytest.mark.parametrize("decoupled", [False, True])
def test_fp64_evaluation_within_one_ulp(oracle, decoupled):
    n = 20000
    p, st = adam_inputs(n, 2, "fp32_master")
    out = _run_oracle(oracle, "fp32_master", p, st, HYP, decoupled)
    b1h, b2h = oracle.folded_betas(HYP["beta1"], HYP["beta2"], HYP["step"])
    f = lambda x: float(np.float32(x))  # the fp32 scalars the kernel receives
    lr, wd, eps, b1h, b2h = f(HYP["lr"]), f(HYP["weight_decay"]), f(HYP["eps"]), f(b1h), f(b2h)
    M, g = st["master_params"].double(), st["grad"].double()
    m, v = st["exp_avg"].double(), st["exp_avg_sq"].double()
    if decoupled:
        M = M - lr * wd * M
    else:
        g = g + wd * M
    m = m + (1 - b1h) * (g - m)
    v = v + (1 - b2h) * (g * g - v)
    upd = lr * m / (v.sqrt() + eps)
    M = M - upd
    got = torch.from_numpy(out["master_params"]).double()
    scale = np.maximum(np.abs(out["master_params"]), np.abs(st["master_params"].numpy()))
    ulp = torch.from_numpy(np.spacing(scale)).double()
    # one ulp of the master, plus the few fp32 roundings inside the update term
    # (they matter only where the master is much smaller than the update)
    assert bool(((got - M).abs() <= ulp + 4 * 2.0**-24 * upd.abs()).all())
    # moments: within one bf16 ulp of the fp64 value, and almost always exact
    olds = {"exp_avg": st["exp_avg"].double().abs() + g.abs(),
            "exp_avg_sq": st["exp_avg_sq"].double() + g * g}
    for key, ref in (("exp_avg", m), ("exp_avg_sq", v)):
        got16 = from_bf16_bits(out[key]).double()
        ulp16 = (got16.abs() * 2.0**-7).clamp(min=1e-45)
        # bf16 rounding of the result plus fp32 rounding of the (cancelling) operands
        assert bool(((got16 - ref).abs() <= ulp16 + 2.0**-22 * olds[key]).all())
    # outputs are mutually consistent: param == bf16_rne(master)
    assert np.array_equal(out["param"], bits(torch.from_numpy(out["master_params"]).to(BF16)))


def test_against_torch_adamw_and_adam(oracle):
    """One step from zero state against torch.optim in fp32 (library routine)."""
    n = 5000
    for decoupled in (True, False):
        p, st = adam_inputs(n, 3, "fp32_master")
        st["exp_avg"].zero_()
        st["exp_avg_sq"].zero_()
        hyp = dict(HYP, step=1)
        out = _run_oracle(oracle, "fp32_master", p, st, hyp, decoupled)
        w = st["master_params"].clone().requires_grad_(True)
        cls = torch.optim.AdamW if decoupled else torch.optim.Adam
        opt = cls([w], lr=hyp["lr"], betas=(hyp["beta1"], hyp["beta2"]), eps=hyp["eps"],
                  weight_decay=hyp["weight_decay"])
        w.grad = st["grad"].float()
        opt.step()
        got = torch.from_numpy(out["master_params"])
        assert torch.allclose(got, w.detach(), rtol=3e-6, atol=1e-9)


def test_multi_step_tracks_torch_adamw(oracle):
    """20 steps: the bias-corrected bf16-moment recursion stays within bf16
    resolution of torch.optim.AdamW's fp32 trajectory."""
    n = 2000
    p, st = adam_inputs(n, 4, "fp32_master")
    st["exp_avg"].zero_()
    st["exp_avg_sq"].zero_()
    w = st["master_params"].clone().requires_grad_(True)
    opt = torch.optim.AdamW([w], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    gen = torch.Generator().manual_seed(0)
    cur_p, cur = p, st
    start = st["master_params"].clone()
    for step in range(1, 21):
        g = (torch.randn(n, generator=gen) * 1e-3).to(BF16)
        cur["grad"] = g
        out = _run_oracle(oracle, "fp32_master", cur_p, cur, dict(HYP, lr=1e-3, step=step), True)
        cur = {"grad": g, "exp_avg": from_bf16_bits(out["exp_avg"]),
               "exp_avg_sq": from_bf16_bits(out["exp_avg_sq"]),
               "master_params": torch.from_numpy(out["master_params"].copy())}
        w.grad = g.float()
        opt.step()
    moved = (w.detach() - start).abs()
    err = (cur["master_params"] - w.detach()).abs()
    assert float(err.max()) <= 0.02 * float(moved.max())


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("decoupled", [False, True])
@pytest.mark.parametrize("clip", [None, 0.3359375])
def test_c_oracle_equals_torch_eager_restatement(oracle, mode, decoupled, clip):
    from oracle import torch_eager as te

    n = 30011
    p, st = adam_inputs(n, 5, mode)
    clip_t = None if clip is None else torch.tensor(clip, dtype=BF16)
    cb = None if clip is None else int(bits(clip_t.reshape(1))[0])
    out = _run_oracle(oracle, mode, p, st, HYP, decoupled, clip_bits=cb, seed=77, layout=0)
    b1h, b2h = oracle.folded_betas(HYP["beta1"], HYP["beta2"], HYP["step"])
    args = (HYP["lr"], HYP["weight_decay"], b1h, b2h, HYP["eps"], decoupled)
    p2, st2 = p.clone(), {k: v.clone() for k, v in st.items()}
    if mode == "fp32_master":
        te.adam_step_fp32_master(p2, st2, *args, clip_coef=clip_t)
        assert np.array_equal(out["master_params"].view(np.uint32),
                              st2["master_params"].numpy().view(np.uint32))
    elif mode == "stochastic_rounding":
        r = torch.from_numpy(oracle.rand16_array(77, n, 0).astype(np.int32))
        te.adam_step_stochastic_rounding(p2, st2, *args, r, clip_coef=clip_t)
    elif mode == "fp31_master":
        te.adam_step_fp31_master(p2, st2, *args, clip_coef=clip_t)
    else:
        te.adam_step_custom_rounding(p2, st2, *args, clip_coef=clip_t)
    if "rounding_error" in out:
        assert np.array_equal(out["rounding_error"], st2["rounding_error"].numpy())
    assert np.array_equal(out["param"], bits(p2))
    assert np.array_equal(out["exp_avg"], bits(st2["exp_avg"]))
    assert np.array_equal(out["exp_avg_sq"], bits(st2["exp_avg_sq"]))


def test_modes_agree_where_they_must(oracle):
    """With zero rounding error the split-master modes start from float(p), and
    the fp32 master they rebuild equals the fp32_master result rounded to 31
    bits (fp31) or exactly (custom)."""
    n = 10007
    p, st = adam_inputs(n, 6, "fp32_master")
    st["master_params"] = p.float()
    ref = _run_oracle(oracle, "fp32_master", p, st, HYP, True)
    L = oracle.lib()
    for mode in ("fp31_master", "fp32_master_custom_rounding"):
        st2 = {k: v for k, v in st.items() if k != "master_params"}
        st2["rounding_error"] = torch.zeros(n, dtype=torch.int16)
        out = _run_oracle(oracle, mode, p, st2, HYP, True)
        shift = 1 if mode == "fp31_master" else 0
        recon = (out["param"].astype(np.uint32) << 16) + (
            out["rounding_error"].astype(np.int32).astype(np.uint32) << shift)
        want = ref["master_params"].view(np.uint32)
        if mode == "fp31_master":
            want = np.array([L.oaref_round_to_fp31(int(x)) for x in want], dtype=np.uint32)
        assert np.array_equal(recon, want)
        assert np.array_equal(out["exp_avg"], ref["exp_avg"])


# -------------------------------------------------------------- norm / clip


def test_grad_norm_against_fp64_and_torch(oracle):
    gen = torch.Generator().manual_seed(0)
    for n in (1, 7, 1000, 100003):
        g = (torch.randn(n, generator=gen) * 5e-3).to(BF16)
        got = oracle.grad_norm_bf16(bits(g))
        exact = math.sqrt(float(g.double().pow(2).sum()))
        got_f = from_bf16_bits(np.array([got], dtype=np.uint16)).item()
        assert abs(got_f - exact) <= exact * 2.0**-8
        lib = bits(torch.norm(g, 2.0).reshape(1))[0]
        assert abs(int(lib) - int(got)) <= 1
    # closed form: constant tensor
    g = torch.full((1024,), 2.0**-7, dtype=BF16)
    assert from_bf16_bits(np.array([oracle.grad_norm_bf16(bits(g))], dtype=np.uint16)).item() == 0.25


def test_clip_coef_equals_the_reference_expression_in_torch(oracle):
    """clamp(max_norm / (total + 1e-6), max=1.0) on 0-dim bf16 tensors, evaluated
    by torch itself for every positive normal bf16 total in a wide range."""
    totals = np.arange(0x3000, 0x4800, dtype=np.uint16)  # ~4.7e-10 .. 131072
    for max_norm in (1.0, 0.3, 2.5):
        t = from_bf16_bits(totals)
        want = torch.stack([torch.clamp(max_norm / (x + 1e-6), max=1.0) for x in t])
        got = np.array([oracle.clip_coef_bf16(int(b), max_norm) for b in totals], dtype=np.uint16)
        assert np.array_equal(got, bits(want)), max_norm
        assert bool((from_bf16_bits(got).float() <= 1.0).all())
    # a small total gives exactly 1
    assert oracle.clip_coef_bf16(0x3C00, 1.0) == 0x3F80
