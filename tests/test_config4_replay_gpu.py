"""Benchmark config 4 in the small: the hook path of ``OffloadAdam`` (stochastic
rounding, four micro-batches per step, eager prefetch, a threshold that splits
the parameter set into offloaded and GPU-resident ones) on the Llama-shaped,
activation-checkpointed decoder of ``bench_e2e.py``, replayed on the CPU by the
oracle.

What is compared is the optimizer *class* against the oracle, not one HIP path
against another: every micro-batch's gradient is captured before the optimizer's
hook consumes it, the bf16 accumulation (src/offload_adam/offload_adam.py:398,
528) is redone with CPU tensors, ``oracle.adam_stochastic_rounding`` is applied
with the seeds the optimizer drew, and parameters and both moments must be
bit-equal after each of three steps.  ``Adam`` (states in HBM, plain ``step()``)
is checked the same way, and so are the other three modes on the hook path and
benchmark config 2 in the small: the clipping path (gradient norms recorded in the
hooks, global coefficient and fused clip in ``step()``).
"""

import ctypes
import sys
import warnings
from pathlib import Path

import numpy as np
import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16
HYP = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
GA, STEPS, SEQ = 4, 3, 48
THRESHOLD = 100_000  # embeddings, lm_head and the MLP weights stream; the rest stay in HBM
LAYOUT = {"triton": 0, "x8": 1}


def u16(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy()


def tiny_decoder():
    import bench_e2e

    return bench_e2e.build_model(bench_e2e.MODELS["tiny"], torch.device("cuda:0"))


def token_batches(vocab):
    g = torch.Generator().manual_seed(5)
    return [torch.randint(0, vocab, (2, SEQ), generator=g).cuda() for _ in range(GA * STEPS)]


class SeedLog:
    """Stands in for ``adam_step_multi`` in a module: draws the seeds itself from
    a counter, remembers which parameter buffer got which seed, and passes them
    on with the chosen bit layout.  Everything else reaches the real function."""

    def __init__(self, real, rng):
        self.real, self.rng, self.counter, self.by_ptr = real, rng, 0, {}

    def __call__(self, mode, params, states, *args, **kw):
        assert mode == "stochastic_rounding" and kw.get("seeds") is None
        seeds = []
        for p in params:
            self.counter += 1
            seed = (0x9E3779B97F4A7C15 * self.counter + 0x1234567) & 0xFFFFFFFFFFFFFFFF
            assert p.data_ptr() not in self.by_ptr, "a parameter stepped twice in one step"
            self.by_ptr[p.data_ptr()] = seed
            seeds.append(seed)
        kw.update(seeds=seeds, rng=self.rng)
        return self.real(mode, params, states, *args, **kw)


AUX_KEY = {"stochastic_rounding": None, "fp32_master": "master_params",
           "fp31_master": "rounding_error", "fp32_master_custom_rounding": "rounding_error"}


class OracleReplica:
    """CPU copy of parameters, moments and the mode's extra state, advanced by the oracle."""

    def __init__(self, oracle, model, decoupled, mode="stochastic_rounding"):
        self.oracle, self.decoupled, self.mode = oracle, decoupled, mode
        self.names = [n for n, _ in model.named_parameters()]
        self.p = {n: u16(p) for n, p in model.named_parameters()}
        self.m = {n: np.zeros_like(b) for n, b in self.p.items()}
        self.v = {n: np.zeros_like(b) for n, b in self.p.items()}
        if mode == "fp32_master":  # the master starts as the widened parameter
            self.aux = {n: p.detach().float().cpu().numpy().reshape(-1).copy()
                        for n, p in model.named_parameters()}
        elif AUX_KEY[mode]:
            self.aux = {n: np.zeros(b.size, dtype=np.int16) for n, b in self.p.items()}
        self.step = 0

    def total_gradient(self, grads, n):
        total = grads[n][0].clone()
        for g in grads[n][1:]:
            total.add_(g)  # bf16 += bf16: fp32 sum, one rounding, as on the GPU
        return u16(total)

    def advance(self, grads, seeds=None, layout=0, clip=None):
        """``grads[name]``: the micro-batch gradients in firing order (CPU bf16);
        ``clip``: bf16 bits of the clip coefficient or None."""
        self.step += 1
        b1h, b2h = self.oracle.folded_betas(*HYP["betas"], self.step)
        hyp = (HYP["lr"], HYP["weight_decay"], b1h, b2h, HYP["eps"], self.decoupled)
        for n in self.names:
            g = self.total_gradient(grads, n)
            if self.mode == "stochastic_rounding":
                self.oracle.adam_stochastic_rounding(self.p[n], g, self.m[n], self.v[n], *hyp,
                                                     seed=seeds[n], layout=layout, clip=clip)
            else:
                fn = {"fp32_master": self.oracle.adam_fp32_master,
                      "fp31_master": self.oracle.adam_fp31_master,
                      "fp32_master_custom_rounding": self.oracle.adam_custom_rounding}[self.mode]
                fn(self.p[n], g, self.m[n], self.v[n], self.aux[n], *hyp, clip=clip)

    def assert_equal(self, model, state_of, step):
        for n, p in model.named_parameters():
            st = state_of(p)
            assert np.array_equal(u16(p), self.p[n]), f"step {step}: param {n}"
            assert np.array_equal(u16(st["exp_avg"]), self.m[n]), f"step {step}: exp_avg {n}"
            assert np.array_equal(u16(st["exp_avg_sq"]), self.v[n]), f"step {step}: exp_avg_sq {n}"
            key = AUX_KEY[self.mode]
            if key == "master_params":
                got = st[key].detach().cpu().numpy().reshape(-1)
                assert np.array_equal(got.view(np.uint32), self.aux[n].view(np.uint32)), \
                    f"step {step}: master {n}"
            elif key:
                got = st[key].detach().cpu().numpy().reshape(-1)
                assert np.array_equal(got, self.aux[n]), f"step {step}: rounding_error {n}"


def capture_hooks(model, sink):
    """Registered before the optimizer's own hooks, so they see ``p.grad`` first."""
    names = {p: n for n, p in model.named_parameters()}

    def hook(p):
        sink.setdefault(names[p], []).append(p.grad.detach().to("cpu", copy=True))

    for p in model.parameters():
        p.register_post_accumulate_grad_hook(hook)


CACHES = {
    "reference_traffic": dict(grad_cache_bytes=0, state_cache_bytes=0,
                              grad_cache_policy="write_through", prefetch_bytes=1 << 20),
    "caches_on": dict(grad_cache_bytes=1 << 20, state_cache_bytes=3 << 20,
                      grad_cache_policy="write_back", prefetch_bytes=2 << 20),
}


@pytest.mark.parametrize("rng", ["triton", "x8"])
@pytest.mark.parametrize("caches", sorted(CACHES))
@pytest.mark.parametrize("decoupled", [True, False])
def test_offload_adam_hook_path_equals_the_oracle(oracle, monkeypatch, rng, caches, decoupled):
    from offload_adam_amd import OffloadAdam
    from offload_adam_amd import offload_adam as oa_mod

    log = SeedLog(oa_mod.adam_step_multi, rng)
    monkeypatch.setattr(oa_mod, "adam_step_multi", log)
    model = tiny_decoder()
    replica = OracleReplica(oracle, model, decoupled)
    grads = {}
    capture_hooks(model, grads)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="stochastic_rounding", prefetch_policy="eager",
                          inplace_param_threshold=THRESHOLD, decoupled_weight_decay=decoupled,
                          **HYP, **CACHES[caches])
    assert opt._offload_params and opt._inplace_params, "the threshold must split the set"
    data = token_batches(model.c["vocab"])
    ptr_name = {p.data_ptr(): n for n, p in model.named_parameters()}
    for s in range(STEPS):
        grads.clear()
        log.by_ptr.clear()
        for mb in range(GA):
            opt.ready_for_optimizer_step = mb == GA - 1
            model(data[s * GA + mb]).backward()
        opt.step()
        opt.zero_grad()
        torch.cuda.synchronize()
        assert all(len(g) == GA for g in grads.values()) and len(grads) == len(ptr_name)
        seeds = {ptr_name[ptr]: seed for ptr, seed in log.by_ptr.items()}
        assert len(seeds) == len(ptr_name), "every parameter is stepped exactly once per step"
        replica.advance(grads, seeds, LAYOUT[rng])
        replica.assert_equal(model, lambda p: opt.state[p], s + 1)
    # the pinned host copies are what a checkpoint would hold
    for p in opt._offload_params:
        assert not opt.state[p]["exp_avg"].is_cuda and opt.state[p]["exp_avg"].is_pinned()


@pytest.mark.parametrize("rng", ["triton", "x8"])
def test_resident_adam_equals_the_oracle(oracle, monkeypatch, rng):
    from offload_adam_amd import Adam
    from offload_adam_amd import adam as adam_mod

    log = SeedLog(adam_mod.adam_step_multi, rng)
    monkeypatch.setattr(adam_mod, "adam_step_multi", log)
    model = tiny_decoder()
    replica = OracleReplica(oracle, model, True)
    opt = Adam(model.parameters(), mode="stochastic_rounding", decoupled_weight_decay=True, **HYP)
    data = token_batches(model.c["vocab"])
    ptr_name = {p.data_ptr(): n for n, p in model.named_parameters()}
    for s in range(STEPS):
        log.by_ptr.clear()
        per_mb = {n: [] for n in ptr_name.values()}
        for mb in range(GA):
            # autograd sums into p.grad in bf16; each micro-batch's own gradient is the
            # input of the replay, so it is taken from a pass that starts without one
            saved = {n: p.grad for n, p in model.named_parameters()}
            for p in model.parameters():
                p.grad = None
            model(data[s * GA + mb]).backward()
            for n, p in model.named_parameters():
                per_mb[n].append(p.grad.detach().to("cpu", copy=True))
                if saved[n] is not None:
                    p.grad = saved[n].add_(p.grad)
        opt.step()
        opt.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        seeds = {ptr_name[ptr]: seed for ptr, seed in log.by_ptr.items()}
        assert len(seeds) == len(ptr_name)
        replica.advance(per_mb, seeds, LAYOUT[rng])
        replica.assert_equal(model, lambda p: opt.state[p], s + 1)


@pytest.mark.parametrize("mode", ["fp32_master", "fp31_master", "fp32_master_custom_rounding"])
@pytest.mark.parametrize("caches", sorted(CACHES))
def test_offload_adam_other_modes_equal_the_oracle(oracle, mode, caches):
    from offload_adam_amd import OffloadAdam

    model = tiny_decoder()
    replica = OracleReplica(oracle, model, True, mode)
    grads = {}
    capture_hooks(model, grads)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode=mode, inplace_param_threshold=THRESHOLD,
                          decoupled_weight_decay=True, **HYP, **CACHES[caches])
    data = token_batches(model.c["vocab"])
    for s in range(STEPS):
        grads.clear()
        for mb in range(GA):
            opt.ready_for_optimizer_step = mb == GA - 1
            model(data[s * GA + mb]).backward()
        opt.step()
        opt.zero_grad()
        torch.cuda.synchronize()
        replica.advance(grads)
        replica.assert_equal(model, lambda p: opt.state[p], s + 1)


@pytest.mark.parametrize("mode", ["fp31_master", "stochastic_rounding"])
@pytest.mark.parametrize("caches", sorted(CACHES))
def test_clipping_path_equals_the_oracle(oracle, monkeypatch, mode, caches):
    """Benchmark config 2 in the small (src/offload_adam/offload_adam.py:504-505,
    542-571): per-parameter norms from the hooks within one bf16 ulp of the oracle's,
    the global norm and the coefficient bit-equal given those norms, and the clipped
    update bit-equal."""
    from offload_adam_amd import OffloadAdam
    from offload_adam_amd import offload_adam as oa_mod
    from offload_adam_amd.kernels import stochastic_rounding as sr_mod

    max_norm = 0.25
    seeds_by_ptr = {}
    if mode == "stochastic_rounding":
        # the clipping path steps parameter by parameter through the single-tensor entry
        real = sr_mod.adam_step_stochastic_rounding
        counter = [0]

        def logged(params, states, *args, **kw):
            counter[0] += 1
            seed = (0x9E3779B97F4A7C15 * counter[0] + 99) & 0xFFFFFFFFFFFFFFFF
            seeds_by_ptr[params.data_ptr()] = seed
            kw.update(seed=seed, rng="triton")
            return real(params, states, *args, **kw)

        monkeypatch.setitem(oa_mod.OffloadAdam.supported_modes[mode], "step", logged)
        log = SeedLog(oa_mod.adam_step_multi, "triton")  # the GPU-resident small parameters
        monkeypatch.setattr(oa_mod, "adam_step_multi", log)
    model = tiny_decoder()
    replica = OracleReplica(oracle, model, True, mode)
    grads = {}
    capture_hooks(model, grads)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode=mode, max_grad_norm=max_norm,
                          inplace_param_threshold=THRESHOLD, decoupled_weight_decay=True,
                          **HYP, **CACHES[caches])
    names = {p: n for n, p in model.named_parameters()}
    order = [names[p] for g in opt.param_groups for p in g["params"]]
    ptr_name = {p.data_ptr(): n for n, p in model.named_parameters()}
    data = token_batches(model.c["vocab"])
    for s in range(STEPS):
        grads.clear()
        seeds_by_ptr.clear()
        if mode == "stochastic_rounding":
            log.by_ptr.clear()
        for mb in range(GA):
            opt.ready_for_optimizer_step = mb == GA - 1
            model(data[s * GA + mb]).backward()
        opt.step()
        opt.zero_grad()
        torch.cuda.synchronize()
        gpu_norms = u16(opt._norm_slots)
        for i, n in enumerate(order):
            want = int(oracle.grad_norm_bf16(replica.total_gradient(grads, n)))
            assert abs(int(gpu_norms[i]) - want) <= 1, (s, n, gpu_norms[i], want)
        total = oracle.lib().oaref_total_norm_bf16(
            gpu_norms.ctypes.data_as(ctypes.c_void_p), len(order))
        assert int(u16(opt._total_norm.reshape(1))[0]) == total
        coef = oracle.clip_coef_bf16(total, max_norm)
        assert int(u16(opt._clip_coef.reshape(1))[0]) == coef
        assert coef < 0x3F80, "the threshold must clip"
        seeds = None
        if mode == "stochastic_rounding":
            merged = dict(seeds_by_ptr)
            merged.update(log.by_ptr)
            seeds = {ptr_name[ptr]: seed for ptr, seed in merged.items()}
            assert len(seeds) == len(ptr_name)
        replica.advance(grads, seeds, LAYOUT["triton"], clip=coef)
        replica.assert_equal(model, lambda p: opt.state[p], s + 1)


@pytest.mark.parametrize("mode,max_norm", [("stochastic_rounding", None), ("fp31_master", None),
                                           ("fp31_master", 0.25)])
def test_the_benchmarks_own_step_check_passes_and_can_fail(mode, max_norm):
    """``bench_e2e.py --check`` (what vouches for the 8B runs of the bench line) on the
    tiny decoder: it passes on an honest step and fails when one moment is off by a bit."""
    import bench_e2e
    from offload_adam_amd import OffloadAdam

    results = []
    for tamper in (False, True):
        torch.manual_seed(0)
        model = tiny_decoder()
        check = bench_e2e.StepCheck(torch, model)  # its hooks precede the optimizer's
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, mode=mode, max_grad_norm=max_norm, lr=1e-3, weight_decay=0.1,
                              decoupled_weight_decay=True, inplace_param_threshold=THRESHOLD)
        data = token_batches(model.c["vocab"])

        def one_step(s):
            for mb in range(GA):
                opt.ready_for_optimizer_step = mb == GA - 1
                model(data[s * GA + mb]).backward()
            opt.step()
            opt.zero_grad()

        one_step(0)
        check.before(opt)
        one_step(1)
        torch.cuda.synchronize()
        if tamper:
            p = next(iter(check.sample))
            st = opt.state[p]["exp_avg"]
            st.view(torch.int16).reshape(-1)[7] ^= 1
        results.append(check.after(opt, decoupled=True))
    honest, tampered = results
    assert honest["passed"] and honest["failed"] == [], honest
    assert honest["elements"] > 500_000
    if max_norm is not None:
        assert honest["clip_coef"] < 1.0 and honest["norms_within_1_bf16_ulp_and_coef_exact"]
    assert not tampered["passed"] and not tampered["moments_exact"], tampered
