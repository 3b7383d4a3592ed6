"""GPU parity of the gradient-norm and clip-coefficient kernels.

Tolerances: the per-parameter norm and the total are sums whose order torch
does not specify, so they are compared within ONE bf16 ulp of the fp64
evaluation (and of torch.norm itself); everything downstream of the total
(the coefficient, the clipped gradient inside the Adam kernel) is bit-exact.
"""

import pytest
import torch

from helpers import HYP, adam_inputs, bits

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def _ulp_diff(a_bits, b_bits):
    """Distance in bf16 ulps between two non-negative bf16 bit patterns."""
    return abs(int(a_bits) - int(b_bits))


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 4099, 65536, (1 << 20) + 3, 11_534_336])
def test_grad_norm_vs_oracle(oracle, n):
    from offload_adam_amd.grad_clip import grad_norm

    g = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 5e-3).to(BF16).cuda()
    got = grad_norm(g)
    assert got.dtype == BF16 and got.dim() == 0
    want = oracle.grad_norm_bf16(bits(g))
    assert _ulp_diff(bits(got.reshape(1))[0], want) <= 1
    if n:
        lib = torch.norm(g, 2.0)
        assert _ulp_diff(bits(got.reshape(1))[0], bits(lib.reshape(1))[0]) <= 1
    # run-to-run determinism (fixed reduction order)
    again = grad_norm(g)
    assert bits(again.reshape(1))[0] == bits(got.reshape(1))[0]


def test_grad_norm_closed_form():
    """Constant tensors: ||c * ones(n)|| = c * sqrt(n), exact for n = 4^k, c = 2^j."""
    from offload_adam_amd.grad_clip import grad_norm

    for n, c in [(4, 0.5), (1024, 2.0**-7), (1 << 20, 2.0**-10), (1 << 24, 2.0**-12)]:
        g = torch.full((n,), c, dtype=BF16, device="cuda")
        assert grad_norm(g).item() == c * n**0.5


def test_grad_norm_unaligned_and_reuse(oracle):
    """Views at every 2-byte offset from a 16-byte boundary; the workspace is
    reused across calls without re-zeroing."""
    from offload_adam_amd.grad_clip import grad_norm

    base = (torch.randn(70_000, generator=torch.Generator().manual_seed(1)) * 1e-2).to(BF16).cuda()
    for off in range(9):
        for n in (1, 5, 17, 60_001):
            g = base[off:off + n]
            got = bits(grad_norm(g).reshape(1))[0]
            assert _ulp_diff(got, oracle.grad_norm_bf16(bits(g))) <= 1, (off, n)


def test_multi_tensor_norms_equal_single_calls(oracle):
    """oa_grad_norm_multi: every slot holds the bits the per-gradient call writes
    (same block counts, same fold order), for empty, tiny, ragged and unaligned
    gradients, a gradient with more tiles than workgroups, and more gradients
    than one launch takes; within one bf16 ulp of the oracle."""
    from offload_adam_amd.grad_clip import grad_norm_, grad_norms_

    gen = torch.Generator().manual_seed(11)
    sizes = ([0, 1, 7, 8, 9, 4096, 4099, 16384, 16385, 65_536, (1 << 20) + 3]
             + [4096] * 40 + [524_288] * 6 + [11_534_336, 3 * (1 << 28) // 2 + 5])
    base = [(torch.randn(n + 8, generator=gen) * 5e-3).to(BF16).cuda() for n in sizes]
    # every second gradient starts off a 16-byte boundary
    grads = [b[(i % 2) * (1 + i % 7):][:n] for i, (b, n) in enumerate(zip(base, sizes))]
    assert len(grads) > 36
    single = torch.full((len(grads),), -1.0, dtype=BF16, device="cuda")
    for i, g in enumerate(grads):
        grad_norm_(g, single[i])
    multi = torch.full((len(grads),), -1.0, dtype=BF16, device="cuda")
    grad_norms_(grads, [multi[i] for i in range(len(grads))])
    torch.cuda.synchronize()
    assert bits(multi).tolist() == bits(single).tolist()
    for i, g in enumerate(grads):
        if g.numel() <= (1 << 24):
            assert _ulp_diff(bits(multi[i:i + 1])[0], oracle.grad_norm_bf16(bits(g))) <= 1, i
    # second call on the same workspace, fewer and smaller gradients
    again = torch.full((5,), -1.0, dtype=BF16, device="cuda")
    grad_norms_(grads[3:8], [again[i] for i in range(5)])
    assert bits(again).tolist() == bits(single[3:8]).tolist()


def test_multi_tensor_norm_c_abi_contract():
    """Through the C ABI: a workspace of the single-tensor size still works (more
    launches, same bits), sums of squares are optional per entry, bad arguments
    are rejected before anything is written."""
    import ctypes

    from offload_adam_amd import _lib
    from offload_adam_amd.grad_clip import grad_norm_

    lib = _lib.load()
    gen = torch.Generator().manual_seed(12)
    sizes = [58_720_256, 16_777_216, 4096, 300_000_000, 1, 65_536]
    grads = [(torch.randn(n, generator=gen) * 5e-3).to(BF16).cuda() for n in sizes]
    count = len(grads)
    want = torch.zeros(count, dtype=BF16, device="cuda")
    for i, g in enumerate(grads):
        grad_norm_(g, want[i])
    small_ws = torch.empty(lib.oa_norm_workspace_bytes(), dtype=torch.uint8, device="cuda")
    assert lib.oa_norm_multi_workspace_bytes() == 36 * lib.oa_norm_workspace_bytes()
    out = torch.full((count,), -1.0, dtype=BF16, device="cuda")
    sumsq = torch.full((count,), -1.0, dtype=torch.float32, device="cuda")
    g_tab = (ctypes.c_uint64 * count)(*[g.data_ptr() for g in grads])
    n_tab = (ctypes.c_int64 * count)(*sizes)
    o_tab = (ctypes.c_uint64 * count)(*[out[i].data_ptr() for i in range(count)])
    s_tab = (ctypes.c_uint64 * count)(*[sumsq[i].data_ptr() if i % 2 == 0 else 0
                                        for i in range(count)])
    stream = _lib.current_stream_ptr()
    rc = lib.oa_grad_norm_multi(count, g_tab, n_tab, o_tab, s_tab, small_ws.data_ptr(),
                                small_ws.numel(), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert bits(out).tolist() == bits(want).tolist()
    for i in range(count):
        if i % 2 == 0:
            assert bits(torch.sqrt(sumsq[i]).to(BF16).reshape(1))[0] == bits(out[i:i + 1])[0]
        else:
            assert sumsq[i].item() == -1.0
    # rejected: workspace smaller than one tensor needs, negative size, null output
    untouched = torch.full((count,), -1.0, dtype=BF16, device="cuda")
    u_tab = (ctypes.c_uint64 * count)(*[untouched[i].data_ptr() for i in range(count)])
    assert lib.oa_grad_norm_multi(count, g_tab, n_tab, u_tab, None, small_ws.data_ptr(),
                                  small_ws.numel() - 64, stream) == -1
    bad_n = (ctypes.c_int64 * count)(*([sizes[0], -1] + sizes[2:]))
    assert lib.oa_grad_norm_multi(count, g_tab, bad_n, u_tab, None, small_ws.data_ptr(),
                                  small_ws.numel(), stream) == -1
    bad_o = (ctypes.c_uint64 * count)(*([untouched[0].data_ptr(), 0]
                                        + [untouched[i].data_ptr() for i in range(2, count)]))
    assert lib.oa_grad_norm_multi(count, g_tab, n_tab, bad_o, None, small_ws.data_ptr(),
                                  small_ws.numel(), stream) == -1
    odd = (ctypes.c_uint64 * count)(*([grads[0].data_ptr() + 1] + [g.data_ptr() for g in grads[1:]]))
    assert lib.oa_grad_norm_multi(count, odd, n_tab, u_tab, None, small_ws.data_ptr(),
                                  small_ws.numel(), stream) == -2
    assert lib.oa_grad_norm_multi(0, None, None, None, None, None, 0, stream) == 0
    torch.cuda.synchronize()
    assert (untouched == -1.0).all()


def test_clip_coef_matches_oracle_and_torch(oracle):
    from offload_adam_amd.grad_clip import clip_coef_

    rng = torch.Generator().manual_seed(3)
    for count, scale, max_norm in [(291, 0.18, 1.0), (291, 0.01, 1.0), (1, 3.0, 1.0),
                                   (201, 0.5, 0.3), (5000, 0.05, 2.5), (2, 0.0, 1.0)]:
        norms = (torch.rand(count, generator=rng) * scale).to(BF16).cuda()
        coef = torch.empty((), dtype=BF16, device="cuda")
        total = torch.empty((), dtype=BF16, device="cuda")
        clip_coef_(norms, max_norm, coef, total)
        t_bits = bits(total.reshape(1))[0]
        assert _ulp_diff(t_bits, oracle.grad_norm_bf16(bits(norms))) <= 1
        # everything after the total is exact bf16 arithmetic
        assert bits(coef.reshape(1))[0] == oracle.clip_coef_bf16(t_bits, max_norm)
        assert coef.item() <= 1.0
        if total.item() + 1e-6 <= max_norm * 0.99:
            assert coef.item() == 1.0
        # the reference's own expression, evaluated by torch on the GPU
        ref_total = torch.linalg.vector_norm(norms, 2.0)
        ref = torch.clamp(max_norm / (ref_total + 1e-6), max=1.0)
        if bits(ref_total.reshape(1))[0] == t_bits:
            assert bits(ref.reshape(1))[0] == bits(coef.reshape(1))[0]


@pytest.mark.parametrize("mode", ["fp32_master", "stochastic_rounding", "fp31_master",
                                  "fp32_master_custom_rounding"])
def test_fused_clip_equals_separate_mul(mode):
    """Adam with clip_coef == torch's grad.mul_(clip_coef) followed by Adam without."""
    from offload_adam_amd import kernels

    fn = getattr(kernels, "adam_step_" + mode)
    n = 50_003
    p, st = adam_inputs(n, seed=9, mode=mode, device="cuda")
    coef = torch.tensor(0.3359375, dtype=BF16, device="cuda")
    p2, st2 = p.clone(), {k: v.clone() for k, v in st.items()}
    st2["grad"].mul_(coef)
    kw = dict(seed=5) if mode == "stochastic_rounding" else {}
    args = (HYP["lr"], HYP["weight_decay"], HYP["beta1"], HYP["beta2"], HYP["eps"], HYP["step"])
    fn(p, st, *args, decoupled_weight_decay=True, clip_coef=coef, **kw)
    fn(p2, st2, *args, decoupled_weight_decay=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(p.view(torch.int16), p2.view(torch.int16))
    for k in st:
        if k == "grad":
            continue
        a, b = st[k], st2[k]
        if a.dtype == BF16:
            a, b = a.view(torch.int16), b.view(torch.int16)
        assert torch.equal(a, b), k


def test_config2_norm_and_clip_flow(oracle):
    """benchmark config 2 shape of the flow at reduced tensor sizes: grads scaled
    so the global norm is ~3 with max_grad_norm=1 (coef ~ 1/3)."""
    from offload_adam_amd.grad_clip import clip_coef_, grad_norm_

    gen = torch.Generator().manual_seed(7)
    sizes = [4096] * 65 + [65_536] * 64 + [262_144] * 32
    grads = [(torch.randn(s, generator=gen) * 5e-3).to(BF16) for s in sizes]
    tot = sum(float(g.double().pow(2).sum()) for g in grads) ** 0.5
    grads = [(g.float() * (3.0 / tot)).to(BF16).cuda() for g in grads]
    norms = torch.zeros(len(grads), dtype=BF16, device="cuda")
    for i, g in enumerate(grads):
        grad_norm_(g, norms[i])
    coef = torch.empty((), dtype=BF16, device="cuda")
    total = torch.empty((), dtype=BF16, device="cuda")
    clip_coef_(norms, 1.0, coef, total)
    for i, g in enumerate(grads):
        assert _ulp_diff(bits(norms[i:i + 1])[0], oracle.grad_norm_bf16(bits(g))) <= 1
    assert abs(total.item() - 3.0) < 0.05
    assert abs(coef.item() - 1.0 / 3.0) < 0.01
    assert bits(coef.reshape(1))[0] == oracle.clip_coef_bf16(bits(total.reshape(1))[0], 1.0)


def _llama_8b_shapes():
    """The 291 parameter tensors of benchmark config 2 / 4 (hidden 4096, MLP 14336,
    32 layers, 32 query / 8 key-value heads of 128, vocabulary 128256, untied)."""
    h, inter, layers, kv, vocab = 4096, 14336, 32, 8 * 128, 128256
    shapes = [(vocab, h)]
    for _ in range(layers):
        shapes += [(h,), (h, h), (kv, h), (kv, h), (h, h), (h,), (inter, h), (inter, h), (h, inter)]
    shapes += [(h,), (vocab, h)]
    return shapes


def test_config2_full_set(oracle):
    """benchmark config 2 at full size, kernel legs on GPU-resident buffers: 291
    tensors, 8,030,261,248 elements, fp31_master, gradients with a global norm of
    about 3 clipped to max_grad_norm = 1 inside the AdamW kernel.

    * every per-tensor norm within one bf16 ulp of torch.norm, the total within
      one ulp of the fp64 value, the coefficient bit-exact given the total;
    * one tensor of every size below 60 M elements and the first 4 M elements of
      an embedding are compared bit for bit with the C oracle;
    * every tensor through size-independent properties, in plain fp32 torch ops
      on the GPU: moments exactly bf16_rne of the update computed from the
      clipped gradient bf16_rne(g * coef); the (param, rounding_error) pair
      reconstructs round_to_fp31(M') with M' taken within one fp32 ulp; the
      param is exactly bf16_rne of that master; the error stays in
      [-16384, 16384]."""
    import numpy as np

    from offload_adam_amd.grad_clip import clip_coef_, grad_norm_
    from offload_adam_amd.kernels import adam_step_multi

    shapes = _llama_8b_shapes()
    numels = [int(np.prod(s)) for s in shapes]
    total_n = sum(numels)
    assert len(shapes) == 291 and total_n == 8_030_261_248
    gen = torch.Generator(device="cuda").manual_seed(2)
    g_std = 3.0 / total_n ** 0.5

    def draw(n, std):
        return (torch.randn(n, device="cuda", generator=gen) * std).to(BF16)

    grads = [draw(n, g_std) for n in numels]
    norms = torch.zeros(len(grads), dtype=BF16, device="cuda")
    for i, g in enumerate(grads):
        grad_norm_(g, norms[i])
    coef = torch.empty((), dtype=BF16, device="cuda")
    total = torch.empty((), dtype=BF16, device="cuda")
    clip_coef_(norms, 1.0, coef, total)
    torch.cuda.synchronize()
    norm_bits = bits(norms)
    sumsq = 0.0
    for i, g in enumerate(grads):
        lib = torch.norm(g, 2.0)
        assert _ulp_diff(norm_bits[i], bits(lib.reshape(1))[0]) <= 1, f"norm of tensor {i}"
        sumsq += float(norms[i].double()) ** 2
    want_total = torch.tensor(sumsq ** 0.5, dtype=torch.float64).to(BF16)
    assert _ulp_diff(bits(total.reshape(1))[0], bits(want_total.reshape(1))[0]) <= 1
    assert abs(total.item() - 3.0) < 0.05 and abs(coef.item() - 1.0 / 3.0) < 0.01
    coef_bits = bits(coef.reshape(1))[0]
    assert coef_bits == oracle.clip_coef_bf16(bits(total.reshape(1))[0], 1.0)

    b1h, b2h = oracle.folded_betas(HYP["beta1"], HYP["beta2"], HYP["step"])
    f32 = np.float32
    omb1, omb2 = float(f32(1) - f32(b1h)), float(f32(1) - f32(b2h))
    lr, eps = float(f32(HYP["lr"])), float(f32(HYP["eps"]))
    lr_wd = float(f32(HYP["lr"]) * f32(HYP["weight_decay"]))
    oracle_args = (HYP["lr"], HYP["weight_decay"], b1h, b2h, HYP["eps"], True)
    sizes_checked = set()
    chunk = 36  # tensors per launch of the multi-tensor kernel
    for c0 in range(0, len(shapes), chunk):
        idx = range(c0, min(c0 + chunk, len(shapes)))
        params = [draw(numels[i], 0.02) for i in idx]
        states = [{"grad": grads[i], "exp_avg": draw(numels[i], 1e-4),
                   "exp_avg_sq": draw(numels[i], 1e-3).float().square().to(BF16),
                   "rounding_error": torch.randint(-16384, 16385, (numels[i],), device="cuda",
                                                   generator=gen, dtype=torch.int16)}
                  for i in idx]
        old = [(p.clone(), st["exp_avg"].clone(), st["exp_avg_sq"].clone(),
                st["rounding_error"].clone()) for p, st in zip(params, states)]
        # oracle on CPU copies taken before the step
        refs = {}
        for j, i in enumerate(idx):
            n = numels[i]
            take = n if n < 60_000_000 else 4_000_000
            if (n, take) in sizes_checked:
                continue
            sizes_checked.add((n, take))
            pb, gb = bits(params[j][:take]), bits(states[j]["grad"][:take])
            mb, vb = bits(states[j]["exp_avg"][:take]), bits(states[j]["exp_avg_sq"][:take])
            err = states[j]["rounding_error"][:take].cpu().numpy().copy()
            oracle.adam_fp31_master(pb, gb, mb, vb, err, *oracle_args,
                                    clip=np.array([coef_bits], dtype=np.uint16))
            refs[j] = (take, pb, mb, vb, err)
        adam_step_multi("fp31_master", params, states, HYP["lr"], HYP["weight_decay"],
                        HYP["beta1"], HYP["beta2"], HYP["eps"], HYP["step"],
                        decoupled_weight_decay=True, clip_coef=coef)
        torch.cuda.synchronize()
        for j, (take, pb, mb, vb, err) in refs.items():
            ctx = f"config 2 tensor {c0 + j}"
            assert np.array_equal(bits(params[j][:take]), pb), ctx + " param"
            assert np.array_equal(bits(states[j]["exp_avg"][:take]), mb), ctx + " exp_avg"
            assert np.array_equal(bits(states[j]["exp_avg_sq"][:take]), vb), ctx + " exp_avg_sq"
            assert np.array_equal(states[j]["rounding_error"][:take].cpu().numpy(), err), ctx
        for j, (p, st) in enumerate(zip(params, states)):
            ctx = f"config 2 tensor {c0 + j}"
            p0, m0, v0, e0 = old[j]
            g = (st["grad"] * coef).float()
            m0, v0 = m0.float(), v0.float()
            m = m0 + omb1 * (g - m0)
            v = v0 + omb2 * (g * g - v0)
            assert torch.equal(st["exp_avg"], m.to(BF16)), ctx + " exp_avg"
            assert torch.equal(st["exp_avg_sq"], v.to(BF16)), ctx + " exp_avg_sq"
            M = ((p0.view(torch.int16).to(torch.int32) << 16) + (e0.to(torch.int32) << 1)
                 ).view(torch.float32)
            M = M - lr_wd * M
            M = M - (lr * m) / (torch.sqrt(v) + eps)
            # A random rounding error next to a param of exactly +-0 reconstructs to
            # NaN bits, a state no run produces: those elements are left out.
            fin = torch.isfinite(M)
            assert int((~fin).sum()) <= 1 + p.numel() // 1_000_000, ctx + " non-finite masters"
            b = M.view(torch.int32)
            want = ((b >> 1) + (b & (b >> 1) & 1)) << 1
            e1 = st["rounding_error"].to(torch.int32)
            got = (p.view(torch.int16).to(torch.int32) << 16) + (e1 << 1)
            assert int(((got - want).abs() * fin).max()) <= 2, ctx + " master"
            same = p.view(torch.int16) == got.view(torch.float32).to(BF16).view(torch.int16)
            assert bool((same | ~fin).all()), ctx + " param = bf16(master)"
            assert int((e1.abs() * fin).max()) <= 16384, ctx + " error range"
            old[j] = None
        del params, states, old
    assert len(sizes_checked) == 5
