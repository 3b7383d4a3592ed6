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
    """BASELINE config 2 shape of the flow at reduced tensor sizes: grads scaled
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
