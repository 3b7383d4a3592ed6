"""GPU parity of the four fused AdamW kernels against the C oracle.

The HIP kernels are called through the C ABI (ctypes, via the Python step
functions).  Tolerance: north star allows 1 fp32 ulp on the master; these tests
assert BIT-EXACT equality of every output (param, moments, master / rounding
error), because kernel and oracle evaluate the same un-fused fp32 expression.
"""

import numpy as np
import pytest
import torch

from helpers import HYP, adam_inputs, bits, from_bf16_bits, special_values

pytestmark = pytest.mark.gpu

MODES = ["fp32_master", "stochastic_rounding", "fp31_master", "fp32_master_custom_rounding"]
SIZES = [1, 7, 8, 9, 63, 1000, 4096, 4099, 2048 * 2 * 3 + 5, (1 << 20) + 3]


def _step_fn(mode):
    from offload_adam_amd import kernels

    return getattr(kernels, "adam_step_" + mode)


def _oracle_step(oracle, mode, p, st, decoupled, clip_bits, seed=0, layout=0, rand16=None,
                 hyp=HYP):
    """Run the C oracle on numpy copies; returns dict of numpy outputs."""
    b1h, b2h = oracle.folded_betas(hyp["beta1"], hyp["beta2"], hyp["step"])
    g, m, v = bits(st["grad"]), bits(st["exp_avg"]), bits(st["exp_avg_sq"])
    pb = bits(p)
    args = (hyp["lr"], hyp["weight_decay"], b1h, b2h, hyp["eps"], decoupled)
    out = {}
    if mode == "fp32_master":
        master = st["master_params"].cpu().numpy().copy()
        oracle.adam_fp32_master(pb, g, m, v, master, *args, clip=clip_bits)
        out["master_params"] = master
    elif mode == "stochastic_rounding":
        oracle.adam_stochastic_rounding(pb, g, m, v, *args, seed=seed, layout=layout,
                                        rand16=rand16, clip=clip_bits)
    else:
        err = st["rounding_error"].cpu().numpy().copy()
        fn = oracle.adam_fp31_master if mode == "fp31_master" else oracle.adam_custom_rounding
        fn(pb, g, m, v, err, *args, clip=clip_bits)
        out["rounding_error"] = err
    out.update(param=pb, exp_avg=m, exp_avg_sq=v)
    return out


def _canon_nan(name, a):
    """NaN sign and payload are not part of parity (x86 makes 0xFFC00000 for an
    invalid operation, gfx950 0x7FC00000): map every NaN to one pattern."""
    if name == "rounding_error":
        return a
    if a.dtype == np.uint32:
        return np.where((a & 0x7FFFFFFF) > 0x7F800000, np.uint32(0x7FC00000), a)
    return np.where((a & 0x7FFF) > 0x7F80, np.uint16(0x7FC0), a)


def _nan_master_mask(mode, ref):
    """True where the oracle's new master is NaN (its split into param and
    rounding error then depends on the NaN's sign and payload)."""
    if mode not in ("fp31_master", "fp32_master_custom_rounding"):
        return None
    shift = 1 if mode == "fp31_master" else 0
    m = (ref["param"].astype(np.uint32) << 16) + (
        ref["rounding_error"].astype(np.int32).astype(np.uint32) << shift)
    return (m & 0x7FFFFFFF) > 0x7F800000


def _assert_equal(mode, p, st, ref, ctx):
    got = {"param": bits(p), "exp_avg": bits(st["exp_avg"]), "exp_avg_sq": bits(st["exp_avg_sq"])}
    if mode == "fp32_master":
        got["master_params"] = st["master_params"].cpu().numpy().view(np.uint32)
        ref = dict(ref, master_params=ref["master_params"].view(np.uint32))
    if "rounding_error" in ref:
        got["rounding_error"] = st["rounding_error"].cpu().numpy()
    nan_mask = _nan_master_mask(mode, ref)
    for k, r in ref.items():
        g_k, r = _canon_nan(k, got[k]), _canon_nan(k, r)
        got[k] = g_k
        differ = g_k != r
        if nan_mask is not None and k in ("param", "rounding_error"):
            differ &= ~nan_mask
        bad = np.nonzero(differ)[0]
        assert bad.size == 0, (
            f"{ctx}: {k} differs at {bad.size} of {r.size} elements, first index "
            f"{bad[0]}: got {got[k][bad[0]]:#x} want {r[bad[0]]:#x}"
        )


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("decoupled", [False, True])
@pytest.mark.parametrize("clip", [None, 0.3359375])
def test_adam_matches_oracle(oracle, mode, decoupled, clip):
    for n in SIZES:
        p, st = adam_inputs(n, seed=n, mode=mode, device="cuda")
        clip_t = None if clip is None else torch.tensor(clip, dtype=torch.bfloat16, device="cuda")
        clip_bits = None if clip is None else int(bits(clip_t.reshape(1))[0])
        kw = dict(seed=1234 + n) if mode == "stochastic_rounding" else {}
        ref = _oracle_step(oracle, mode, p, st, decoupled, clip_bits, seed=1234 + n, layout=0)
        g_before = bits(st["grad"])
        _step_fn(mode)(p, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"],
                       HYP["eps"], HYP["step"], decoupled_weight_decay=decoupled,
                       clip_coef=clip_t, **kw)
        torch.cuda.synchronize()
        _assert_equal(mode, p, st, ref, f"{mode} n={n} dec={decoupled} clip={clip}")
        assert np.array_equal(bits(st["grad"]), g_before), "grad must not be written"


@pytest.mark.parametrize("mode", MODES)
def test_adam_unaligned_views(oracle, mode):
    """Buffers that start 2 bytes off a 16-byte boundary take the scalar path."""
    n = 5000
    p0, st0 = adam_inputs(n + 1, seed=77, mode=mode, device="cuda")
    p = p0[1:]
    st = {k: v[1:] for k, v in st0.items()}
    assert p.data_ptr() % 16 != 0
    ref = _oracle_step(oracle, mode, p, st, True, None, seed=99, layout=0)
    kw = dict(seed=99) if mode == "stochastic_rounding" else {}
    _step_fn(mode)(p, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"],
                   HYP["eps"], HYP["step"], decoupled_weight_decay=True, **kw)
    torch.cuda.synchronize()
    _assert_equal(mode, p, st, ref, f"{mode} unaligned")


@pytest.mark.parametrize("mode", MODES)
def test_adam_special_values(oracle, mode):
    """Zeros, signed zeros, denormals, extreme normals in every operand."""
    n = 8192 + 5
    p, st = adam_inputs(n, seed=5, mode=mode, device="cuda")
    p = from_bf16_bits(special_values(n, 1), "cuda")
    st["grad"] = from_bf16_bits(special_values(n, 2), "cuda")
    st["exp_avg"] = from_bf16_bits(special_values(n, 3), "cuda")
    # exp_avg_sq is a running mean of squares: never negative
    st["exp_avg_sq"] = from_bf16_bits(special_values(n, 4) & np.uint16(0x7FFF), "cuda")
    if mode == "fp32_master":
        st["master_params"] = p.float().clone()
    hyp = dict(HYP, step=1)
    for decoupled in (False, True):
        pp, ss = p.clone(), {k: v.clone() for k, v in st.items()}
        ref = _oracle_step(oracle, mode, pp, ss, decoupled, None, seed=3, layout=0, hyp=hyp)
        kw = dict(seed=3) if mode == "stochastic_rounding" else {}
        _step_fn(mode)(pp, ss, hyp["lr"], hyp["weight_decay"], hyp["beta1"], hyp["beta2"],
                       hyp["eps"], hyp["step"], decoupled_weight_decay=decoupled, **kw)
        torch.cuda.synchronize()
        _assert_equal(mode, pp, ss, ref, f"{mode} special dec={decoupled}")


@pytest.mark.parametrize("rng,layout", [("triton", 0), ("x8", 1), ("buffer", 2)])
def test_stochastic_rounding_bit_exact_with_identical_bits(oracle, rng, layout):
    """Same random bits in -> same bf16 params out, for all three bit sources."""
    mode = "stochastic_rounding"
    for n in (9, 4099, (1 << 18) + 7):
        p, st = adam_inputs(n, seed=11, mode=mode, device="cuda")
        seed = 0x0123456789ABCDEF
        rand = None
        kw = dict(seed=seed, rng=rng)
        if rng == "buffer":
            rand = np.random.default_rng(n).integers(0, 65536, size=n, dtype=np.uint16)
            kw = dict(rand16=torch.from_numpy(rand.view(np.int16)).cuda())
        ref = _oracle_step(oracle, mode, p, st, True, None, seed=seed, layout=layout, rand16=rand)
        _step_fn(mode)(p, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"],
                       HYP["eps"], HYP["step"], decoupled_weight_decay=True, **kw)
        torch.cuda.synchronize()
        _assert_equal(mode, p, st, ref, f"sr rng={rng} n={n}")


def test_stochastic_rounding_unbiased_and_within_one_ulp(oracle):
    """Fresh seeds: the mean of the rounded params converges to the fp32 update
    and every sample is one of the two bf16 neighbours."""
    mode = "stochastic_rounding"
    n = 4096
    p0, st0 = adam_inputs(n, seed=21, mode=mode, device="cuda")
    # exact fp32 result of the update (buffer layout with r=0xFFFF truncates, so
    # compute it from the fp32_master kernel instead)
    stm = {k: v.clone() for k, v in st0.items()}
    stm["master_params"] = p0.float().clone()
    sink = torch.empty_like(p0)
    _step_fn("fp32_master")(sink, stm, HYP["lr"], 0.0, HYP["beta1"], HYP["beta2"], HYP["eps"],
                            HYP["step"])
    exact = stm["master_params"].double()
    lo = (stm["master_params"].view(torch.int32) & -0x10000).view(torch.float32).double()
    hi = ((stm["master_params"].view(torch.int32) & -0x10000) + 0x10000).view(torch.float32).double()
    acc = torch.zeros(n, dtype=torch.float64, device="cuda")
    trials = 512
    for rng in ("x8", "triton"):
        acc.zero_()
        for t in range(trials):
            p = p0.clone()
            st = {k: v.clone() for k, v in st0.items()}
            _step_fn(mode)(p, st, HYP["lr"], 0.0, HYP["beta1"], HYP["beta2"], HYP["eps"],
                           HYP["step"], seed=1000 + t, rng=rng)
            pd = p.double()
            assert bool(((pd == lo) | (pd == hi)).all()), "result is not a bf16 neighbour"
            acc += pd
        mean = acc / trials
        ulp = (hi - lo).abs()
        # standard error of a two-point distribution <= ulp/2/sqrt(trials); 6 sigma
        assert bool(((mean - exact).abs() <= 6 * ulp / 2 / trials**0.5 + 1e-30).all()), rng


def test_fp32_master_param_may_alias_grad(oracle):
    """The quantised-weight path passes the grad buffer as the bf16 sink."""
    n = 4096 + 3
    p, st = adam_inputs(n, seed=31, mode="fp32_master", device="cuda")
    ref = _oracle_step(oracle, "fp32_master", p, st, True, None)
    sink = st["grad"]
    _step_fn("fp32_master")(sink, st, HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"],
                            HYP["eps"], HYP["step"], decoupled_weight_decay=True)
    torch.cuda.synchronize()
    assert np.array_equal(bits(sink), ref["param"])
    assert np.array_equal(st["master_params"].cpu().numpy().view(np.uint32),
                          ref["master_params"].view(np.uint32))


def test_config0_full_size(oracle):
    """benchmark config 0: one flat tensor of 16,777,216 elements, fp32_master,
    lr=1e-4, betas=(0.9,0.999), eps=1e-8, wd=0.01 decoupled, step=10."""
    n = 16_777_216
    p, st = adam_inputs(n, seed=0, mode="fp32_master", device="cuda")
    st["master_params"] = p.float().clone()
    ref = _oracle_step(oracle, "fp32_master", p, st, True, None)
    _step_fn("fp32_master")(p, st, 1e-4, 0.01, 0.9, 0.999, 1e-8, 10, decoupled_weight_decay=True)
    torch.cuda.synchronize()
    _assert_equal("fp32_master", p, st, ref, "config 0")
    # size-independent property: the bf16 param is the RNE rounding of the master
    assert torch.equal(p, st["master_params"].to(torch.bfloat16))


def test_multi_step_trajectory(oracle):
    """Ten consecutive steps stay bit-identical to the oracle in every mode."""
    n = 3000
    for mode in MODES:
        p, st = adam_inputs(n, seed=41, mode=mode, device="cuda")
        pc, sc = p.cpu().clone(), {k: v.cpu().clone() for k, v in st.items()}
        for step in range(1, 11):
            hyp = dict(HYP, step=step)
            g = (torch.randn(n, generator=torch.Generator().manual_seed(step)) * 1e-3).to(torch.bfloat16)
            st["grad"] = g.cuda()
            sc["grad"] = g.clone()
            ref = _oracle_step(oracle, mode, pc, sc, True, None, seed=step, layout=0, hyp=hyp)
            kw = dict(seed=step) if mode == "stochastic_rounding" else {}
            _step_fn(mode)(p, st, hyp["lr"], hyp["weight_decay"], hyp["beta1"], hyp["beta2"],
                           hyp["eps"], step, decoupled_weight_decay=True, **kw)
            torch.cuda.synchronize()
            _assert_equal(mode, p, st, ref, f"{mode} step {step}")
            # carry the oracle state forward
            pc = from_bf16_bits(ref["param"])
            sc["exp_avg"] = from_bf16_bits(ref["exp_avg"])
            sc["exp_avg_sq"] = from_bf16_bits(ref["exp_avg_sq"])
            if "master_params" in ref:
                sc["master_params"] = torch.from_numpy(ref["master_params"].copy())
            if "rounding_error" in ref:
                sc["rounding_error"] = torch.from_numpy(ref["rounding_error"].copy())


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("clip", [None, 0.3359375])
def test_multi_tensor_equals_single_calls(oracle, mode, clip):
    """One multi-tensor call over 80 tensors (three launch chunks, sizes from 1
    element to 300k, one unaligned view, per-tensor step counts and seeds) leaves
    every tensor exactly as the oracle's per-tensor result."""
    from offload_adam_amd.kernels import adam_step_multi

    rng = np.random.default_rng(0)
    sizes = [1, 7, 8, 2048, 2049, 300_001] + [int(s) for s in rng.integers(1, 50_000, 74)]
    params, states, steps, seeds, refs = [], [], [], [], []
    clip_t = None if clip is None else torch.tensor(clip, dtype=torch.bfloat16, device="cuda")
    clip_bits = None if clip is None else int(bits(clip_t.reshape(1))[0])
    for i, n in enumerate(sizes):
        off = 1 if i == 5 else 0  # one tensor off the 16-byte boundary
        p0, st0 = adam_inputs(n + off, seed=100 + i, mode=mode, device="cuda")
        p, st = p0[off:], {k: v[off:] for k, v in st0.items()}
        step, seed = 1 + i % 7, 1000 + i
        refs.append(_oracle_step(oracle, mode, p, st, True, clip_bits, seed=seed, layout=0,
                                 hyp=dict(HYP, step=step)))
        params.append(p)
        states.append(st)
        steps.append(step)
        seeds.append(seed)
    kw = dict(seeds=seeds, rng="triton") if mode == "stochastic_rounding" else {}
    adam_step_multi(mode, params, states, HYP["lr"], HYP["weight_decay"], HYP["beta1"],
                    HYP["beta2"], HYP["eps"], steps, decoupled_weight_decay=True,
                    clip_coef=clip_t, **kw)
    torch.cuda.synchronize()
    for i, (p, st, ref) in enumerate(zip(params, states, refs)):
        _assert_equal(mode, p, st, ref, f"multi {mode} tensor {i} n={sizes[i]}")


def test_multi_tensor_rejects_before_launching():
    from offload_adam_amd import _lib
    from offload_adam_amd.kernels import adam_step_multi

    p, st = adam_inputs(64, seed=1, mode="fp31_master", device="cuda")
    before = bits(p)
    bad = dict(st, exp_avg=st["exp_avg"][:8])
    with pytest.raises(ValueError):
        adam_step_multi("fp31_master", [p, p], [st, bad], 1e-3, 0.0, 0.9, 0.999, 1e-8, 1)
    with pytest.raises(ValueError):
        adam_step_multi("fp99", [p], [st], 1e-3, 0.0, 0.9, 0.999, 1e-8, 1)
    torch.cuda.synchronize()
    assert np.array_equal(bits(p), before)
    lib = _lib.load()
    assert lib.oa_adam_multi(9, 1, None, None, None, None, None, None, None, None, None,
                             0, 0, 0, 0, 0, None, None) == -1
    assert lib.oa_adam_multi(0, 0, None, None, None, None, None, None, None, None, None,
                             0, 0, 0, 0, 0, None, None) == 0


def test_argument_errors():
    from offload_adam_amd import _lib

    fn = _step_fn("fp32_master")
    p, st = adam_inputs(16, seed=1, mode="fp32_master", device="cuda")
    with pytest.raises(TypeError):
        fn(p.float(), st, 1e-3, 0.0, 0.9, 0.999, 1e-8, 1)
    bad = dict(st, exp_avg=st["exp_avg"][:8])
    with pytest.raises(ValueError):
        fn(p, bad, 1e-3, 0.0, 0.9, 0.999, 1e-8, 1)
    with pytest.raises(ValueError):
        fn(p.cpu(), {k: v.cpu() for k, v in st.items()}, 1e-3, 0.0, 0.9, 0.999, 1e-8, 1)
    with pytest.raises(AssertionError):
        _step_fn("fp31_master")(p.float(), st, 1e-3, 0.0, 0.9, 0.999, 1e-8, 1)
    # the C ABI itself rejects bad arguments without launching
    lib = _lib.load()
    assert lib.oa_adam_fp32_master(None, None, None, None, None, 8, 0, 0, 0, 0, 0, 0, None, None) == -1
    assert lib.oa_adam_fp32_master(None, None, None, None, None, -1, 0, 0, 0, 0, 0, 0, None, None) == -1
    assert lib.oa_adam_fp32_master(None, None, None, None, None, 0, 0, 0, 0, 0, 0, 0, None, None) == 0
    m = st["exp_avg"]
    rc = lib.oa_adam_fp32_master(_lib.ptr(p), _lib.ptr(st["grad"]), _lib.ptr(m), _lib.ptr(m),
                                 _lib.ptr(st["master_params"]), 16, 0, 0, 0, 0, 0, 0, None, None)
    assert rc == -4


def _llama_1b_shapes():
    """The 201 parameter tensors of benchmark config 1 (hidden 2048, MLP 5632, 22
    layers, 32 query / 4 key-value heads of 64, vocabulary 32000, untied)."""
    h, inter, layers, kv, vocab = 2048, 5632, 22, 4 * 64, 32000
    shapes = [(vocab, h)]
    for _ in range(layers):
        shapes += [(h,), (h, h), (kv, h), (kv, h), (h, h), (h,), (inter, h), (inter, h), (h, inter)]
    shapes += [(h,), (vocab, h)]
    return shapes


def test_config1_full_set(oracle):
    """benchmark config 1 at full size: 201 tensors, 1,100,048,384 elements,
    stochastic rounding, one multi-tensor step (6 launches).

    * one tensor of every distinct size (82 M elements) is compared bit for bit
      with the C oracle;
    * every tensor is checked through size-independent properties evaluated with
      plain fp32 torch ops on the GPU: the stored moments are exactly
      bf16_rne(m + (1-b1)(g-m)) and bf16_rne(v + (1-b2)(g*g-v)); the stored
      parameter is the fp32 result M' truncated to bf16 or one step above in
      magnitude (M' taken within 1 fp32 ulp: torch's own sqrt and divide are
      not promised correctly rounded); and over the whole set the number of
      round-ups matches the sum of the round-up probabilities frac/65536
      (unbiasedness) within 6 standard deviations."""
    from offload_adam_amd.kernels import adam_step_multi

    shapes = _llama_1b_shapes()
    assert len(shapes) == 201 and sum(int(np.prod(s)) for s in shapes) == 1_100_048_384
    gen = torch.Generator(device="cuda").manual_seed(1)
    params, states, seeds = [], [], []
    for i, shape in enumerate(shapes):
        n = int(np.prod(shape))
        params.append((torch.randn(n, device="cuda", generator=gen) * 0.02).to(torch.bfloat16))
        states.append({
            "grad": (torch.randn(n, device="cuda", generator=gen) * 1e-3).to(torch.bfloat16),
            "exp_avg": (torch.randn(n, device="cuda", generator=gen) * 1e-4).to(torch.bfloat16),
            "exp_avg_sq": (torch.randn(n, device="cuda", generator=gen) * 1e-3).square()
            .to(torch.bfloat16),
        })
        seeds.append(0x5EED0000 + i)
    old = [(p.clone(), st["exp_avg"].clone(), st["exp_avg_sq"].clone())
           for p, st in zip(params, states)]
    first_of_size = {}
    for i, p in enumerate(params):
        first_of_size.setdefault(p.numel(), i)
    refs = {}
    for i in first_of_size.values():
        refs[i] = _oracle_step(oracle, "stochastic_rounding", params[i], states[i], True, None,
                               seed=seeds[i], layout=1)
    assert sum(params[i].numel() for i in refs) > 80_000_000 and len(refs) == 5

    adam_step_multi("stochastic_rounding", params, states, HYP["lr"], HYP["weight_decay"],
                    HYP["beta1"], HYP["beta2"], HYP["eps"], HYP["step"],
                    decoupled_weight_decay=True, seeds=seeds, rng="x8")
    torch.cuda.synchronize()
    for i, ref in refs.items():
        _assert_equal("stochastic_rounding", params[i], states[i], ref, f"config 1 tensor {i}")

    b1h, b2h = oracle.folded_betas(HYP["beta1"], HYP["beta2"], HYP["step"])
    f32 = np.float32
    omb1, omb2 = float(f32(1) - f32(b1h)), float(f32(1) - f32(b2h))
    lr, eps = float(f32(HYP["lr"])), float(f32(HYP["eps"]))
    lr_wd = float(f32(HYP["lr"]) * f32(HYP["weight_decay"]))
    ups = 0.0
    expected_ups = 0.0
    variance = 0.0
    for i, (p, st) in enumerate(zip(params, states)):
        p0, m0, v0 = (t.float() for t in old[i])
        g = st["grad"].float()
        m = m0 + omb1 * (g - m0)
        v = v0 + omb2 * (g * g - v0)
        assert torch.equal(st["exp_avg"], m.to(torch.bfloat16)), f"tensor {i} exp_avg"
        assert torch.equal(st["exp_avg_sq"], v.to(torch.bfloat16)), f"tensor {i} exp_avg_sq"
        M = p0 - lr_wd * p0
        M = M - (lr * m) / (torch.sqrt(v) + eps)
        mb = M.view(torch.int32)
        pb = p.view(torch.int16).to(torch.int32) << 16

        def on_grid(b):
            t = b & -0x10000
            return (pb == t) | (pb == t + 0x10000)

        ok = on_grid(mb) | on_grid(mb + 1) | on_grid(mb - 1)
        assert bool(ok.all()), f"tensor {i}: {int((~ok).sum())} params off the two bf16 neighbours"
        frac = (mb & 0xFFFF).double() / 65536.0
        ups += float((pb != (mb & -0x10000)).double().sum())
        expected_ups += float(frac.sum())
        variance += float((frac * (1 - frac)).sum())
        old[i] = None
    assert abs(ups - expected_ups) < 6.0 * variance ** 0.5 + 1e3, (ups, expected_ups, variance)
