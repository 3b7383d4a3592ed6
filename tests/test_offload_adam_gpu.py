"""GPU tests of the host driver: pinned allocator, H2D/D2H streaming with event
fencing, hook-driven and one-shot (clipping) steps, state layout, QAT.

The reference has no test of this part; what pins it here is equivalence:
``OffloadAdam`` (states on the host, step inside backward hooks, transfers on
side streams) must leave parameters and states BIT-IDENTICAL to ``Adam`` (states
on the GPU, plain ``step()``), which itself is checked against the oracle in
test_adam_kernels_gpu.py.  Any missing fence or stale buffer breaks equality.
"""

import gc
import random
import warnings

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16
MODES = ["stochastic_rounding", "fp32_master", "fp31_master", "fp32_master_custom_rounding"]


class TinyNet(nn.Module):
    """A few Linear / norm layers; sizes straddle the in-place threshold used below."""

    def __init__(self, d=96, h=160, tied=False):
        super().__init__()
        self.emb = nn.Embedding(50, d)
        self.blocks = nn.ModuleList(
            [nn.ModuleDict({"norm": nn.LayerNorm(d), "up": nn.Linear(d, h), "down": nn.Linear(h, d)})
             for _ in range(3)]
        )
        self.head = nn.Linear(d, 50, bias=False)
        if tied:
            self.head.weight = self.emb.weight

    def forward(self, ids):
        x = self.emb(ids)
        for b in self.blocks:
            x = x + b["down"](F.gelu(b["up"](b["norm"](x))))
        return self.head(x)


def make_model(seed=0, tied=False):
    torch.manual_seed(seed)
    return TinyNet(tied=tied).to(device="cuda", dtype=BF16)


def batches(n, seed=1):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, 50, (4, 16), generator=g).cuda() for _ in range(n)]


def loss_of(model, ids):
    return F.cross_entropy(model(ids).float().reshape(-1, 50), ids.reshape(-1))


@pytest.fixture
def fixed_seed(monkeypatch):
    """Both optimizers draw the stochastic-rounding seed from random.getrandbits;
    a constant makes their random bits identical whatever the parameter order."""
    monkeypatch.setattr(random, "getrandbits", lambda k: 0x1234_5678_9ABC_DEF0)


def run_reference_adam(mode, steps, ga, seed=0, tied=False, **kw):
    from offload_adam_amd import Adam

    model = make_model(seed, tied)
    opt = Adam(model.parameters(), mode=mode, lr=1e-2, weight_decay=0.01, **kw)
    data = batches(steps * ga)
    for s in range(steps):
        for mb in range(ga):
            loss_of(model, data[s * ga + mb]).backward()  # grads accumulate in bf16
        opt.step()
        opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    return model, opt


def run_offload_adam(mode, steps, ga, seed=0, tied=False, threshold=5000, **kw):
    from offload_adam_amd import OffloadAdam

    model = make_model(seed, tied)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode=mode, lr=1e-2, weight_decay=0.01,
                          inplace_param_threshold=threshold, **kw)
    data = batches(steps * ga)
    for s in range(steps):
        for mb in range(ga):
            opt.ready_for_optimizer_step = mb == ga - 1
            loss_of(model, data[s * ga + mb]).backward()
        opt.step()
        opt.zero_grad()
    torch.cuda.synchronize()
    return model, opt


def assert_same_params(a, b):
    for (n1, p1), (n2, p2) in zip(a.named_parameters(), b.named_parameters()):
        assert n1 == n2
        assert torch.equal(p1.view(torch.int16), p2.view(torch.int16)), n1


# ------------------------------------------------------------- pinned memory


def test_zeros_pinned_invariants():
    from offload_adam_amd.pinned_alloc import (gpu_numa_node, numa_node_free_bytes,
                                               resolve_numa_target, zeros_pinned)

    for shape, dtype in [((3, 5), torch.float32), ((1000, 1000), BF16), ((0,), torch.int16),
                         ((4097,), torch.int16)]:
        t = zeros_pinned(shape, dtype, numa_node="auto")
        assert t.shape == torch.Size(shape) and t.dtype == dtype and t.device.type == "cpu"
        assert t.data_ptr() % 4096 == 0
        assert t.is_pinned()
        assert not t.any()
        t.fill_(1)  # writable
    node = gpu_numa_node()
    assert isinstance(node, int) and node >= -1
    assert resolve_numa_target(None) is None
    assert resolve_numa_target("auto") in (None, node)
    with pytest.raises(ValueError):
        resolve_numa_target("nearest")
    with pytest.raises(ValueError):
        zeros_pinned((4,), BF16, numa_node=1.5)
    free0 = numa_node_free_bytes(0)
    if free0 is not None:  # the host exposes NUMA nodes: an explicit node works
        assert free0 > 0
        t = zeros_pinned((1 << 20,), torch.float32, numa_node=0)
        assert not t.any() and t.is_pinned()
        # a node the host does not have: the memory-policy call fails, nothing is allocated
        with pytest.raises(OSError) as info:
            zeros_pinned((4,), BF16, numa_node=1000)
        assert info.value.errno > 0
        # beyond what the node mask can name at all
        with pytest.raises(RuntimeError):
            zeros_pinned((4,), BF16, numa_node=5000)
    assert numa_node_free_bytes(10_000) is None


def test_pinned_memory_is_released():
    from offload_adam_amd import _lib, pinned_alloc

    lib = _lib.load()
    real = lib.oa_pinned_free
    freed = []

    def spy(ptr):
        freed.append(ptr.value if hasattr(ptr, "value") else ptr)
        return real(ptr)

    gc.collect()  # buffers other tests left behind go now, not while this one watches
    lib.oa_pinned_free = spy
    try:
        t = pinned_alloc.zeros_pinned((1 << 20,), torch.float32, numa_node=None)
        ptr = t.data_ptr()
        view = t[10:20]
        del t
        gc.collect()
        assert ptr not in freed  # a surviving view keeps the pages alive
        view.fill_(3.0)
        assert view.sum().item() == 30.0
        del view
        gc.collect()
        assert freed.count(ptr) == 1  # released exactly once, when the last view died
    finally:
        lib.oa_pinned_free = real


def test_states_are_carved_from_arenas_and_released_together():
    """States come out of a few large pinned allocations on 4 KiB boundaries, in
    request order, zero-filled and of the exact shape and dtype; an arena goes back
    to the runtime when its last piece dies."""
    from offload_adam_amd import _lib, pinned_alloc

    lib = _lib.load()
    real_alloc, real_free = lib.oa_pinned_alloc, lib.oa_pinned_free
    calls, freed = [], []

    def spy_alloc(size, *rest):
        calls.append(size.value if hasattr(size, "value") else size)
        return real_alloc(size, *rest)

    def spy_free(ptr):
        freed.append(ptr.value if hasattr(ptr, "value") else ptr)
        return real_free(ptr)

    requests = [((300, 70), BF16), ((5000,), torch.float32), ((1,), torch.int16),
                ((40_000,), BF16), ((0,), BF16), ((33_000,), torch.float32)]
    gc.collect()
    lib.oa_pinned_alloc, lib.oa_pinned_free = spy_alloc, spy_free
    try:
        pieces = pinned_alloc.alloc_pinned_states(requests, numa_node=None, arena_bytes=128 << 10)
        # 45056 + 20480 + 4096 | 81920 + 4096 | 135168 (its own arena): three allocations
        assert calls == [69632, 86016, 135168]
        for (shape, dtype), t in zip(requests, pieces):
            assert t.shape == torch.Size(shape) and t.dtype == dtype and t.is_contiguous()
            assert t.data_ptr() % 4096 == 0 and not t.any()
            assert t.numel() == 0 or t.is_pinned()
        bases = [pieces[0].data_ptr(), pieces[3].data_ptr(), pieces[5].data_ptr()]
        assert pieces[1].data_ptr() == bases[0] + 45056
        assert pieces[2].data_ptr() == bases[0] + 45056 + 20480
        for t in pieces:
            t.fill_(1)  # writable, and no piece overlaps another
        assert all(int(t.double().sum()) == t.numel() for t in pieces)
        keep = pieces[1]
        del pieces, t
        gc.collect()
        assert set(freed) == {bases[1], bases[2]}  # the first arena still has a live piece
        assert int(keep.double().sum()) == 5000
        del keep
        gc.collect()
        assert sorted(freed) == sorted(bases)
    finally:
        lib.oa_pinned_alloc, lib.oa_pinned_free = real_alloc, real_free


def test_a_request_the_runtime_cannot_grant_fails_before_anything_is_kept():
    """The reference meets a refusal one mapping at a time, mid-construction
    (src/offload_adam/pinned_alloc.py:204-221).  Here the arenas are obtained first:
    a refusal releases them all and reports the total, what had been granted and the
    largest block the runtime would still give."""
    from offload_adam_amd import pinned_alloc

    with pytest.raises(RuntimeError) as info:
        pinned_alloc.alloc_pinned_states([((1 << 40,), torch.uint8)] * 64, numa_node=None)
    text = str(info.value)
    assert "65536.0 GiB were asked for in 64 allocations" in text
    assert "refused after 0.0 GiB" in text and "largest single allocation" in text
    # the probe behind that figure: grants are granted, refusals refused, nothing is left over
    lib = pinned_alloc._lib.load()
    assert lib.oa_pinned_probe(1 << 20) == 0
    assert lib.oa_pinned_probe(1 << 46) != 0
    t = pinned_alloc.zeros_pinned((1 << 20,), torch.uint8, numa_node=None)  # still works
    assert t.is_pinned() and not t.any()


def test_numa_preference_is_applied_and_the_thread_policy_restored():
    """numa_node=k: the allocation runs under MPOL_PREFERRED(k) and the calling
    thread is back on the default policy afterwards.  Where the kernel tells on
    which node the pages of the mapping sit (/proc/self/numa_maps ``N<k>=`` counts,
    or move_pages(2) with a NULL node list), they must sit on node k; a page-locked
    block that is a mapping of the GPU's device file exposes neither, which the test
    then states instead."""
    import ctypes
    import re

    from offload_adam_amd.pinned_alloc import numa_node_free_bytes, zeros_pinned

    if numa_node_free_bytes(0) is None:
        pytest.skip("this host exposes no NUMA nodes")
    libc = ctypes.CDLL(None, use_errno=True)
    SYS_get_mempolicy, SYS_move_pages = 239, 279  # x86-64
    node = 0
    t = zeros_pinned((8 << 20,), torch.uint8, numa_node=node)
    mode = ctypes.c_int(-1)
    assert libc.syscall(SYS_get_mempolicy, ctypes.byref(mode), None, 0, None, 0) == 0
    assert mode.value == 0  # MPOL_DEFAULT again
    t[::4096] = 1  # the CPU has touched every page
    n = 64
    pages = (ctypes.c_void_p * n)(*[t.data_ptr() + i * 32 * 4096 for i in range(n)])
    status = (ctypes.c_int * n)(*([-99] * n))
    rc = libc.syscall(SYS_move_pages, 0, ctypes.c_ulong(n), pages, None, status, 0)
    assert rc == 0
    placed = [s for s in status if s >= 0]
    line = next((ln for ln in open("/proc/self/numa_maps")
                 if ln.split()[0] == format(t.data_ptr(), "x")), "")
    counts = {int(k): int(v) for k, v in re.findall(r"N(\d+)=(\d+)", line)}
    if placed or counts:
        assert all(s == node for s in placed), list(status)
        assert set(counts) <= {node}, line
    else:
        # -ENOENT for every page and no per-node counts: not ordinary process memory
        assert all(s == -2 for s in status), list(status)
        assert "file=/dev/" in line, line


def test_async_copy_round_trip_with_event_fencing():
    """H2D on one side stream, kernel on the compute stream, D2H on another."""
    from offload_adam_amd import _lib
    from offload_adam_amd.offload_adam import _copy_async
    from offload_adam_amd.pinned_alloc import zeros_pinned

    n = 8_000_000
    host_in = zeros_pinned((n,), torch.float32, numa_node=None)
    host_out = zeros_pinned((n,), torch.float32, numa_node=None)
    host_in.copy_(torch.arange(n, dtype=torch.float32))
    h2d, d2h = torch.cuda.Stream(), torch.cuda.Stream()
    compute = torch.cuda.current_stream()
    for rep in range(3):
        dev = torch.empty(n, dtype=torch.float32, device="cuda")
        h2d.wait_stream(compute)
        _copy_async(dev, host_in, _lib.OA_COPY_H2D, h2d)
        ev = h2d.record_event()
        compute.wait_event(ev)
        dev.mul_(2.0)
        d2h.wait_stream(compute)
        _copy_async(host_out, dev, _lib.OA_COPY_D2H, d2h)
        dev.record_stream(d2h)
        d2h.synchronize()
        assert torch.equal(host_out, host_in * 2.0), rep


@pytest.mark.parametrize("nbytes", [16, 4096 + 7, 3 * (1 << 20) + 5, 64 << 20])
@pytest.mark.parametrize("workgroups", [1, 8])
def test_copy_kernel_moves_exact_bytes(nbytes, workgroups):
    """oa_copy_kernel_async: host->device and device->host, byte tail included."""
    from offload_adam_amd import _lib
    from offload_adam_amd.pinned_alloc import zeros_pinned

    lib = _lib.load()
    g = torch.Generator().manual_seed(nbytes)
    host_in = zeros_pinned((nbytes + 16,), torch.uint8, numa_node=None)
    host_out = zeros_pinned((nbytes + 16,), torch.uint8, numa_node=None)
    host_in.copy_(torch.randint(0, 256, (nbytes + 16,), dtype=torch.uint8, generator=g))
    dev = torch.full((nbytes + 16,), 0xAA, dtype=torch.uint8, device="cuda")
    s = _lib.current_stream_ptr()
    _lib.check(lib.oa_copy_kernel_async(_lib.ptr(dev), _lib.ptr(host_in), nbytes, workgroups, s),
               "h2d")
    _lib.check(lib.oa_copy_kernel_async(_lib.ptr(host_out), _lib.ptr(dev), nbytes, workgroups, s),
               "d2h")
    torch.cuda.synchronize()
    assert torch.equal(dev[:nbytes].cpu(), host_in[:nbytes])
    assert (dev[nbytes:] == 0xAA).all()  # nothing written past the byte count
    assert torch.equal(host_out[:nbytes], host_in[:nbytes])
    assert (host_out[nbytes:] == 0).all()
    # argument checks
    assert lib.oa_copy_kernel_async(_lib.ptr(dev), _lib.ptr(host_in), nbytes, 0, s) == -1
    assert lib.oa_copy_kernel_async(dev.data_ptr() + 4, _lib.ptr(host_in), nbytes, 1, s) == -2
    assert lib.oa_copy_kernel_async(None, None, 0, 1, s) == 0


def test_d2h_by_kernel_switch_gives_identical_results(fixed_seed, monkeypatch):
    """The write-back path by copy kernel is a transport choice only."""
    from offload_adam_amd import offload_adam as oa_mod

    ref_model, _ = run_offload_adam("stochastic_rounding", steps=3, ga=2)
    monkeypatch.setattr(oa_mod, "_D2H_BY_KERNEL", True)
    model, _ = run_offload_adam("stochastic_rounding", steps=3, ga=2)
    assert_same_params(ref_model, model)


# ------------------------------------------------------- optimizer equivalence


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("ga", [1, 3])
@pytest.mark.parametrize("spare_hbm", [False, True])
def test_hook_path_equals_adam(fixed_seed, mode, ga, spare_hbm):
    ref_model, ref_opt = run_reference_adam(mode, steps=4, ga=ga, decoupled_weight_decay=True)
    model, opt = run_offload_adam(mode, steps=4, ga=ga, decoupled_weight_decay=True,
                                  spare_hbm=spare_hbm)
    assert len(opt._offload_params) > 0 and len(opt._inplace_params) > 0
    assert_same_params(ref_model, model)
    # states agree too (host-resident vs GPU-resident)
    for (pr, p) in zip(ref_model.parameters(), model.parameters()):
        for key in ref_opt.config["states"]:
            a, b = ref_opt.state[pr][key].cpu(), opt.state[p][key].cpu()
            if a.dtype == BF16:
                a, b = a.view(torch.int16), b.view(torch.int16)
            assert torch.equal(a, b), key
        assert opt.state[p]["step"] == 4


@pytest.mark.parametrize("policy", ["eager", "lazy"])
def test_tied_weights_and_prefetch_policies(fixed_seed, policy):
    ref_model, _ = run_reference_adam("fp32_master", steps=3, ga=2, tied=True)
    model, opt = run_offload_adam("fp32_master", steps=3, ga=2, tied=True, prefetch_policy=policy)
    assert_same_params(ref_model, model)
    assert sum(1 for _ in opt.param_groups[0]["params"]) == len(list(model.parameters()))


def test_everything_offloaded_and_everything_inplace(fixed_seed):
    ref_model, _ = run_reference_adam("stochastic_rounding", steps=3, ga=2)
    m0, o0 = run_offload_adam("stochastic_rounding", steps=3, ga=2, threshold=0)
    m1, o1 = run_offload_adam("stochastic_rounding", steps=3, ga=2, threshold=10**9)
    assert not o0._inplace_params and not o1._offload_params
    assert_same_params(ref_model, m0)
    assert_same_params(ref_model, m1)


@pytest.mark.parametrize("mode", ["fp31_master", "stochastic_rounding", "fp32_master"])
@pytest.mark.parametrize("ga", [1, 2])
def test_clip_path_equals_manual_clip_then_adam(fixed_seed, mode, ga):
    """max_grad_norm path == per-parameter bf16 norms -> global bf16 coefficient
    -> grad.mul_(coef) (torch) -> Adam.step(), the sequence the reference runs."""
    from offload_adam_amd import Adam
    from offload_adam_amd.grad_clip import clip_coef_, grad_norm_

    max_norm = 0.05  # small enough to clip on every step
    steps = 3
    model, opt = run_offload_adam(mode, steps=steps, ga=ga, max_grad_norm=max_norm)
    assert float(opt._clip_coef) < 1.0

    ref = make_model(0)
    ref_opt = Adam(ref.parameters(), mode=mode, lr=1e-2, weight_decay=0.01)
    params = list(ref.parameters())
    norms = torch.zeros(len(params), dtype=BF16, device="cuda")
    coef = torch.ones((), dtype=BF16, device="cuda")
    data = batches(steps * ga)
    for s in range(steps):
        for mb in range(ga):
            loss_of(ref, data[s * ga + mb]).backward()
        for i, p in enumerate(params):
            grad_norm_(p.grad.reshape(-1), norms[i])
        clip_coef_(norms, max_norm, coef)
        for p in params:
            p.grad.mul_(coef)
        ref_opt.step()
        ref_opt.zero_grad(set_to_none=True)
    torch.cuda.synchronize()
    assert_same_params(ref, model)
    assert torch.equal(norms.view(torch.int16), opt._norm_slots.view(torch.int16))


def test_clip_not_triggered_is_identity(fixed_seed):
    ref_model, _ = run_reference_adam("fp31_master", steps=2, ga=1)
    model, opt = run_offload_adam("fp31_master", steps=2, ga=1, max_grad_norm=1e6)
    assert float(opt._clip_coef) == 1.0
    assert_same_params(ref_model, model)


# ------------------------------------------------------------ layout, errors


def test_state_layout_and_api_surface():
    from offload_adam_amd import OffloadAdam

    model = make_model()
    opt = OffloadAdam(model, mode="fp32_master", max_grad_norm=1.0, inplace_param_threshold=5000,
                      verbose=0)
    assert opt.mode == "fp32_master" and opt.ready_for_optimizer_step is False
    assert opt.offload_state_keys == ["grad", "exp_avg", "exp_avg_sq", "master_params"]
    group = opt.param_groups[0]
    assert {"lr", "betas", "eps", "weight_decay", "params"} <= set(group)
    for p in group["params"]:
        st = opt.state[p]
        assert st["step"] == 0
        assert st["grad_norm"].dim() == 0 and st["grad_norm"].is_cuda
        if p in opt._inplace_params:
            assert "host_grad_valid" not in st
            assert all(st[k].is_cuda for k in opt.offload_state_keys)
        else:
            assert st["host_grad_valid"] is False
            for k, dt in opt.offload_config.items():
                assert st[k].device.type == "cpu" and st[k].is_pinned()
                assert st[k].dtype == dt and st[k].shape == p.shape
            assert torch.equal(st["master_params"], p.detach().float().cpu())
    sd = opt.state_dict()
    assert set(sd) == {"state", "param_groups"} and len(sd["state"]) == len(group["params"])
    with pytest.raises(NotImplementedError):
        opt.load_state_dict(sd)
    with pytest.raises(NotImplementedError):
        opt.step(closure=lambda: None)
    assert opt.zero_grad() is None
    with pytest.raises(ValueError):
        OffloadAdam(make_model(), prefetch_policy="sometimes")
    with pytest.raises(AssertionError):
        OffloadAdam(make_model(), mode="fp64_master")
    with pytest.raises(RuntimeError):
        OffloadAdam(make_model(), mode="stochastic_rounding").load_master_state_dict({}, model)


def test_step_is_noop_in_hook_mode_and_returns_none():
    from offload_adam_amd import OffloadAdam

    model = make_model()
    opt = OffloadAdam(model, inplace_param_threshold=5000)
    before = [p.detach().clone() for p in model.parameters()]
    assert opt.step() is None
    for a, p in zip(before, model.parameters()):
        assert torch.equal(a, p)


# ----------------------------------------------------------------------- QAT


@pytest.mark.parametrize("fmt", ["int8", "int4", "nf4", "nvfp4"])
def test_qat_offload_equals_adam(fmt):
    from offload_adam_amd import Adam, OffloadAdam
    from offload_adam_amd.qweight import (Int4QWeight, Int8QWeight, NF4QWeight, NVFP4QWeight,
                                          QWeightBase, quantize_linears)

    cls, kw = {"int8": (Int8QWeight, {}), "int4": (Int4QWeight, {"group_size": 32}),
               "nf4": (NF4QWeight, {"blocksize": 32}), "nvfp4": (NVFP4QWeight, {})}[fmt]

    def build():
        m = make_model()
        report = quantize_linears(m, cls, skip_patterns=("head",), **kw)
        assert len(report.quantized) == 6 and report.excluded == ["head"]
        return m

    data = batches(6)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        ref = build()
        ref_opt = Adam(ref.parameters(), mode="fp32_master", lr=1e-2)
        model = build()
        opt = OffloadAdam(model, mode="fp32_master", lr=1e-2, inplace_param_threshold=5000)
        assert len(opt._quant_params) == 6
        for s in range(3):
            for mb in range(2):
                loss_of(ref, data[2 * s + mb]).backward()
                opt.ready_for_optimizer_step = mb == 1
                loss_of(model, data[2 * s + mb]).backward()
            ref_opt.step()
            ref_opt.zero_grad(set_to_none=True)
            opt.step()
    torch.cuda.synchronize()
    for (n, pr), (_, p) in zip(ref.named_parameters(), model.named_parameters()):
        if isinstance(p.data, QWeightBase):
            for name in type(p.data)._PAYLOAD:
                a, b = getattr(pr.data, name), getattr(p.data, name)
                assert torch.equal(a.reshape(-1).view(torch.uint8),
                                   b.reshape(-1).view(torch.uint8)), (n, name)
            assert torch.equal(ref_opt.state[pr]["master_params"].cpu(),
                               opt.state[p]["master_params"])
            assert opt.state[p]["master_filled"] is False
        else:
            assert torch.equal(pr.view(torch.int16), p.view(torch.int16)), n
    with pytest.raises(ValueError):
        OffloadAdam(build(), mode="stochastic_rounding")


def test_quant_master_warning_and_master_loading(tmp_path):
    from safetensors.torch import save_file

    from offload_adam_amd import OffloadAdam
    from offload_adam_amd.qweight import Int8QWeight, quantize_linears

    plain = make_model()
    originals = {n: p.detach().clone() for n, p in plain.named_parameters()}
    quantize_linears(plain, Int8QWeight, skip_patterns=("head",))
    opt = OffloadAdam(plain, mode="fp32_master", inplace_param_threshold=5000)
    q_names = [n for n, p in plain.named_parameters() if p in opt._quant_params]
    # lossy seed: master == dequantised weight, flagged
    p0 = dict(plain.named_parameters())[q_names[0]]
    assert opt.state[p0]["master_filled"] is False
    assert torch.equal(opt.state[p0]["master_params"], p0.data.dequantize().float().cpu())
    opt.ready_for_optimizer_step = True
    with pytest.warns(UserWarning, match="lossy dequant-seeded"):
        loss_of(plain, batches(1)[0]).backward()
    # lossless refill from a checkpoint of the original bf16 weights
    ckpt = tmp_path / "model.safetensors"
    save_file({n: t.cpu().contiguous() for n, t in originals.items()}, str(ckpt))
    missing = opt.load_master_from_pretrained(str(ckpt), plain, strict=True)
    assert missing == []
    for n in q_names[1:]:
        p = dict(plain.named_parameters())[n]
        assert opt.state[p]["master_filled"] is True
    unexpected, = opt.load_master_state_dict({"nope": torch.zeros(1)}, plain)
    assert unexpected == ["nope"]
    with pytest.raises(ValueError):
        opt.load_master_state_dict({"nope": torch.zeros(1)}, plain, strict=True)


def test_adam_state_dict_round_trip_keeps_fp32_master():
    from offload_adam_amd import Adam

    model = make_model()
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-2)
    loss_of(model, batches(1)[0]).backward()
    opt.step()
    sd = opt.state_dict()
    opt2 = Adam(make_model().parameters(), mode="fp32_master", lr=1e-2)
    opt2.load_state_dict(sd)
    for p, p2 in zip(opt.param_groups[0]["params"], opt2.param_groups[0]["params"]):
        assert opt2.state[p2]["master_params"].dtype == torch.float32
        assert torch.equal(opt.state[p]["master_params"], opt2.state[p2]["master_params"])
        assert opt2.state[p2]["step"] == 1


@pytest.mark.parametrize("mode", ["fp32_master", "fp31_master", "stochastic_rounding"])
@pytest.mark.parametrize("ga,save_after_microbatches", [(1, 2), (3, 6), (3, 7)])
def test_resume_continues_bit_identically(fixed_seed, mode, ga, save_after_microbatches):
    """Four steps in one go against: stop after some micro-batches (at a step
    boundary, or one micro-batch into an accumulation window), save, build a new
    model and optimizer, load both, and finish.  Parameters and every state
    tensor end up identical."""
    import copy

    from offload_adam_amd import OffloadAdam

    steps = 4
    data = batches(steps * ga)
    kw = dict(mode=mode, lr=1e-2, weight_decay=0.01, inplace_param_threshold=5000,
              max_grad_norm=None)

    def build(seed):
        model = make_model(seed)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            return model, OffloadAdam(model, **kw)

    def run(model, opt, first, last):
        for i in range(first, last):
            opt.ready_for_optimizer_step = i % ga == ga - 1
            loss_of(model, data[i]).backward()
            if i % ga == ga - 1:
                opt.step()
                opt.zero_grad()
        torch.cuda.synchronize()

    ref_model, ref_opt = build(0)
    run(ref_model, ref_opt, 0, steps * ga)

    model, opt = build(0)
    run(model, opt, 0, save_after_microbatches)
    saved_opt = copy.deepcopy(opt.state_dict())
    saved_model = copy.deepcopy(model.state_dict())
    del model, opt

    model2, opt2 = build(123)  # different initial weights: everything must come from the files
    model2.load_state_dict(saved_model)
    with pytest.raises(NotImplementedError):
        opt2.load_state_dict(saved_opt)
    opt2.load_offloaded_state_dict(saved_opt)
    for st in opt2.state.values():  # still this optimizer's own kind of buffers
        if "host_grad_valid" in st:
            assert st["exp_avg"].is_pinned() and st["grad"].is_pinned()
    run(model2, opt2, save_after_microbatches, steps * ga)

    assert_same_params(ref_model, model2)
    for pr, p2 in zip(ref_model.parameters(), model2.parameters()):
        a, b = ref_opt.state[pr], opt2.state[p2]
        assert set(a) == set(b)
        for k in a:
            if k == "grad" and a.get("host_grad_valid") is False:
                continue  # no window is open: the host gradient holds no information
            if isinstance(a[k], torch.Tensor):
                assert torch.equal(a[k].cpu(), b[k].cpu()), k
            else:
                assert a[k] == b[k], k


def test_resume_rejects_a_state_that_does_not_fit(fixed_seed):
    import copy

    _, opt31 = run_offload_adam("fp31_master", 1, 1)
    _, opt32 = run_offload_adam("fp32_master", 1, 1)
    before = {k: v.clone() for k, v in next(iter(opt32.state.values())).items()
              if isinstance(v, torch.Tensor)}
    with pytest.raises(ValueError):
        opt32.load_offloaded_state_dict(opt31.state_dict())
    sd = copy.deepcopy(opt32.state_dict())
    first = sd["state"][0]
    first["exp_avg"] = first["exp_avg"][:1]
    with pytest.raises(ValueError):
        opt32.load_offloaded_state_dict(sd)
    sd = copy.deepcopy(opt32.state_dict())
    sd["param_groups"][0]["params"] = sd["param_groups"][0]["params"][:-1]
    with pytest.raises(ValueError):
        opt32.load_offloaded_state_dict(sd)
    after = next(iter(opt32.state.values()))
    for k, v in before.items():
        assert torch.equal(after[k], v), "a rejected load changes nothing"


class BranchyNet(TinyNet):
    """TinyNet whose middle block is skipped for odd ``route`` and whose head is
    one of two: some parameters get no gradient in some passes."""

    def __init__(self):
        super().__init__()
        self.head2 = nn.Linear(96, 50, bias=False)

    def forward(self, ids, route=0):
        x = self.emb(ids)
        for i, b in enumerate(self.blocks):
            if i == 1 and route % 2:
                continue
            x = x + b["down"](F.gelu(b["up"](b["norm"](x))))
        return (self.head2 if route % 3 == 2 else self.head)(x)


@pytest.mark.parametrize("mode", ["fp31_master", "stochastic_rounding"])
@pytest.mark.parametrize("kw", [dict(), dict(spare_hbm=True), dict(prefetch_bytes=0),
                                dict(offload_grads=False)])
def test_parameters_without_a_gradient_in_some_passes(fixed_seed, mode, kw):
    """The order of gradient hooks is learned, and prefetch runs along it; passes
    that skip modules (their hooks never fire, their prefetched states are not
    consumed) must neither stall nor change a result.  Every step uses one route
    for all its micro-batches, so the optimizer without offloading sees the same
    set of gradients."""
    from offload_adam_amd import Adam, OffloadAdam

    steps, ga = 7, 2
    data = batches(steps * ga)

    def train(make_opt, offloaded):
        torch.manual_seed(0)
        model = BranchyNet().to(device="cuda", dtype=BF16)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = make_opt(model)
        for s in range(steps):
            for mb in range(ga):
                if offloaded:
                    opt.ready_for_optimizer_step = mb == ga - 1
                out = model(data[s * ga + mb], route=s)
                F.cross_entropy(out.float().reshape(-1, 50), data[s * ga + mb].reshape(-1)).backward()
            opt.step()
            opt.zero_grad(*([] if offloaded else [True]))
        torch.cuda.synchronize()
        return model, opt

    ref, _ = train(lambda m: Adam(m.parameters(), mode=mode, lr=1e-2, weight_decay=0.01), False)
    got, opt = train(lambda m: OffloadAdam(m, mode=mode, lr=1e-2, weight_decay=0.01,
                                           inplace_param_threshold=5000, **kw), True)
    assert_same_params(ref, got)
    used = [opt.state[p]["step"] for p in got.parameters()]
    assert min(used) < steps and max(used) == steps  # some parameters did skip steps


@pytest.mark.parametrize("mode,clip", [("stochastic_rounding", None), ("fp31_master", 0.05),
                                       ("fp32_master", None)])
def test_bound_on_pending_write_backs_changes_no_result(fixed_seed, mode, clip):
    """Staging buffers handed back while their write-back still runs are bounded in bytes;
    past the bound the host waits for the oldest write-back.  With a bound of one byte
    (a wait at every issue) and with none, on the hook path and the clipping path: the
    same bits, and the books are back at zero once everything has completed."""
    from offload_adam_amd import OffloadAdam

    results = []
    _, default = run_offload_adam(mode, steps=1, ga=1, max_grad_norm=clip)
    assert default._writeback_pending_limit == max(2 * default._PREFETCH_BYTES, 2 << 30)
    for limit in (1, 1 << 60):
        model, opt = run_offload_adam(mode, steps=3, ga=3, max_grad_norm=clip,
                                      pending_writeback_bytes=limit)
        assert opt._writeback_pending_limit == limit
        if limit == 1:
            # nothing older than the newest write-back is ever left pending
            assert len(opt._writebacks_pending) <= 1
        torch.cuda.synchronize()
        opt._throttle_writebacks()
        assert opt._writeback_pending_bytes == 0 and not opt._writebacks_pending
        results.append(model)
    assert_same_params(results[0], results[1])
    if clip is None:
        ref, _ = run_reference_adam(mode, steps=3, ga=3)
        assert_same_params(ref, results[0])


@pytest.mark.parametrize("kw", [dict(offload_grads=False), dict(pinned_limit_bytes=620_000)])
def test_clip_path_leaves_out_parameters_whose_device_gradient_never_came(fixed_seed, kw):
    """Clipping path, gradient sums kept on the GPU only: a parameter that got no gradient
    in a window has no buffer to be stepped from; it sits the step out and its norm does
    not count.  With weight_decay = 0 and modules that never run, the default optimizer
    (host gradient buffers, all zero for those parameters: a step that changes nothing)
    must give the same bits."""
    from offload_adam_amd import OffloadAdam

    steps, ga = 4, 2
    data = batches(steps * ga)

    def train(**extra):
        torch.manual_seed(0)
        model = BranchyNet().to(device="cuda", dtype=BF16)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, mode="fp31_master", lr=1e-2, weight_decay=0.0,
                              max_grad_norm=0.05, inplace_param_threshold=5000, **extra)
        for s in range(steps):
            for mb in range(ga):
                opt.ready_for_optimizer_step = mb == ga - 1
                out = model(data[s * ga + mb], route=1)  # block 1 and head2 never run
                F.cross_entropy(out.float().reshape(-1, 50), data[s * ga + mb].reshape(-1)).backward()
            opt.step()
            opt.zero_grad()
        torch.cuda.synchronize()
        return model, opt

    ref, _ = train()
    got, opt = train(**kw)
    assert_same_params(ref, got)
    idle = [p for p in opt._grad_on_device if opt.state[p]["step"] == 0]
    assert idle, "the case needs a parameter with its gradient on the GPU and no gradient"
    assert any(opt.state[p]["step"] == steps for p in opt._grad_on_device)
    torch.manual_seed(0)
    fresh = BranchyNet().to(device="cuda", dtype=BF16)
    names = {id(p): n for n, p in got.named_parameters()}
    init = dict(fresh.named_parameters())
    for p in idle:
        assert torch.equal(p, init[names[id(p)]]), names[id(p)]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("cache,policy", [(0, "write_back"), (40_000, "write_back"),
                                          (40_000, "write_through"), ("auto", "write_back"),
                                          ("auto", "write_through")])
@pytest.mark.parametrize("clip", [None, 0.05])
def test_gradient_cache_does_not_change_results(fixed_seed, mode, cache, clip, policy):
    """grad_cache_bytes = 0 (every accumulated gradient is fetched back, as in the
    reference and by default), a budget that admits only some parameters, and 'auto', under
    either write policy: same bits as the optimizer without offloading, on the
    hook path and the clip path."""
    if clip is None:
        ref_model, _ = run_reference_adam(mode, steps=3, ga=3)
    else:
        ref_model, _ = run_offload_adam(mode, steps=3, ga=3, max_grad_norm=clip,
                                        grad_cache_bytes=0)
    model, opt = run_offload_adam(mode, steps=3, ga=3, max_grad_norm=clip, grad_cache_bytes=cache,
                                  grad_cache_policy=policy)
    assert_same_params(ref_model, model)
    n_cached = len(opt._grad_cached)
    if cache == 0:
        assert n_cached == 0
    elif cache == "auto":
        assert n_cached == len(opt._offload_params)
    else:
        assert 0 < n_cached < len(opt._offload_params)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("cache", [0, 200_000, "auto"])
@pytest.mark.parametrize("clip", [None, 0.05])
def test_state_cache_does_not_change_results(fixed_seed, mode, cache, clip):
    """state_cache_bytes = 0 (every state is fetched for every step, as in the
    reference and by default), a budget that admits only some parameters, and 'auto': same
    bits; the host copies are current after every step."""
    ref_model, ref_opt = run_offload_adam(mode, steps=4, ga=2, max_grad_norm=clip,
                                          state_cache_bytes=0, grad_cache_bytes=0)
    model, opt = run_offload_adam(mode, steps=4, ga=2, max_grad_norm=clip,
                                  state_cache_bytes=cache)
    assert_same_params(ref_model, model)
    n_cached = len(opt._state_cached)
    if cache == 0:
        assert n_cached == 0
    elif cache == "auto":
        assert n_cached == len(opt._offload_params)
    else:
        assert 0 < n_cached < len(opt._offload_params)
    for pr, p in zip(ref_model.parameters(), model.parameters()):
        a, b = ref_opt.state[pr], opt.state[p]
        for k in opt._non_grad_keys:
            assert torch.equal(a[k], b[k]), k  # pinned host copies (GPU ones for small params)
            if p in opt._state_cached:
                assert torch.equal(opt.device_states[p][k].cpu(), b[k].cpu()), k


def test_loading_masters_replaces_cached_device_copies(fixed_seed):
    """load_master_state_dict after some steps: the next step starts from the
    loaded masters, not from a device copy kept from the previous step."""
    from offload_adam_amd import OffloadAdam

    results = []
    for cache in (0, "auto"):
        model = make_model(0)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, mode="fp32_master", lr=1e-2, inplace_param_threshold=5000,
                              state_cache_bytes=cache)
        data = batches(3)
        for i in range(2):
            opt.ready_for_optimizer_step = True
            loss_of(model, data[i]).backward()
            opt.step()
        new_masters = {n: torch.full_like(p, 0.25, dtype=torch.float32)
                       for n, p in model.named_parameters()}
        opt.load_master_state_dict(new_masters, model)
        opt.ready_for_optimizer_step = True
        loss_of(model, data[2]).backward()
        opt.step()
        torch.cuda.synchronize()
        results.append([p.detach().clone() for p in model.parameters()])
        big = opt._offload_params[0]
        assert abs(opt.state[big]["master_params"].mean().item() - 0.25) < 0.05
    for a, b in zip(*results):
        assert torch.equal(a, b)


def test_loading_masters_while_the_next_step_is_prestaged(fixed_seed):
    """Once a hook-path step completes, the states the next step touches first are
    fetched straight away.  Loading masters at that moment must wait for that
    fetch (it reads the host buffer about to be overwritten, and writes a device
    buffer about to be dropped) and the next step must start from the loaded
    values: two 134 MB masters make the fetch long enough to be under way."""
    from offload_adam_amd import Adam, OffloadAdam

    def net():
        torch.manual_seed(0)
        return nn.Sequential(nn.Linear(4096, 8192, bias=False), nn.GELU(),
                             nn.Linear(8192, 4096, bias=False)).to(device="cuda", dtype=BF16)

    g = torch.Generator().manual_seed(3)
    xs = [torch.randn(8, 4096, generator=g).to(BF16).cuda() for _ in range(3)]
    results = []
    for offload in (False, True):
        model = net()
        if offload:
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")
                opt = OffloadAdam(model, mode="fp32_master", lr=1e-2, inplace_param_threshold=0)
        else:
            opt = Adam(model.parameters(), mode="fp32_master", lr=1e-2)
        for i in range(2):
            opt.ready_for_optimizer_step = True
            model(xs[i]).float().square().mean().backward()
            opt.step()
            opt.zero_grad(set_to_none=True) if not offload else opt.zero_grad()
        if offload:  # the next step's states are on their way
            assert any(d.get("master_params") is not None for d in opt.device_states.values())
        new = {n: torch.full_like(p, 0.01 * (i + 1), dtype=torch.float32)
               for i, (n, p) in enumerate(model.named_parameters())}
        opt.load_master_state_dict(new, model)
        opt.ready_for_optimizer_step = True
        model(xs[2]).float().square().mean().backward()
        opt.step()
        torch.cuda.synchronize()
        results.append(([p.detach().clone() for p in model.parameters()],
                        [opt.state[p]["master_params"].cpu().clone() for p in model.parameters()]))
    for a, b in zip(results[0][0], results[1][0]):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for a, b in zip(results[0][1], results[1][1]):
        assert torch.equal(a, b)


def test_cached_gradient_reaches_the_host(fixed_seed):
    """Two micro-batches into a window, the pinned ``state['grad']`` holds the same
    sum whether or not the device copy was kept: at once under 'write_through',
    and in what ``state_dict()`` returns under 'write_back' (where nothing crossed
    the link before that call)."""
    from offload_adam_amd import OffloadAdam

    sums = []
    for cache, policy in ((0, "write_back"), ("auto", "write_through"), ("auto", "write_back")):
        model = make_model(0)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, mode="fp31_master", lr=1e-2, inplace_param_threshold=5000,
                              grad_cache_bytes=cache, grad_cache_policy=policy)
        data = batches(2)
        for mb in range(2):
            opt.ready_for_optimizer_step = False
            loss_of(model, data[mb]).backward()
        torch.cuda.synchronize()
        lazy = cache == "auto" and policy == "write_back"
        if lazy:
            assert len(opt._stale_host_grads) == len(opt._offload_params)
            assert all(opt.state[p]["grad"].abs().sum() == 0 for p in opt._offload_params)
            saved = opt.state_dict()["state"]
            assert not opt._stale_host_grads
            index = {id(q): i for i, q in enumerate(opt.param_groups[0]["params"])}
            sums.append([saved[index[id(p)]]["grad"].clone() for p in opt._offload_params])
        else:
            sums.append([opt.state[p]["grad"].clone() for p in opt._offload_params])
        kept = [opt.device_states[p].get("grad") is not None for p in opt._offload_params]
        assert all(kept) if cache == "auto" else not any(kept)
    for a, b, c in zip(*sums):
        assert torch.equal(a, b) and torch.equal(a, c) and a.abs().sum() > 0


def test_default_contract_is_the_reference_one(fixed_seed, capsys):
    """Without ``spare_hbm`` nothing but the bounded staging window is kept in HBM and
    the pinned ``state[p]['grad']`` holds the running bf16 sum after every
    micro-batch (src/offload_adam/offload_adam.py:360-372, 513-514); with it, the HBM
    that may be held is printed even at verbose=0 and the host gradient is current
    in what ``state_dict()`` returns."""
    from offload_adam_amd import OffloadAdam

    def build(**kw):
        model = make_model(0)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            return model, OffloadAdam(model, mode="stochastic_rounding", lr=1e-2,
                                      inplace_param_threshold=5000, **kw)

    model, opt = build()
    assert capsys.readouterr().out == ""
    assert not opt._grad_cached and not opt._state_cached and not opt._grad_cache_write_back
    # a bounded staging window: 4 GiB, or an eighth of what is offloaded (at least 256 MiB)
    assert opt._PREFETCH_BYTES == 256 << 20 and opt._prestage_bytes == 256 << 20
    assert OffloadAdam._PREFETCH_BYTES == 4 << 30
    names = {p: n for n, p in model.named_parameters()}
    sums = {}

    def capture(p):
        g = p.grad.detach().to("cpu", copy=True)
        sums[names[p]] = g if names[p] not in sums else sums[names[p]].add_(g)

    # (hooks registered after the optimizer's would find p.grad already consumed)
    model, sums = make_model(0), {}
    names = {p: n for n, p in model.named_parameters()}
    for p in model.parameters():
        p.register_post_accumulate_grad_hook(capture)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="stochastic_rounding", lr=1e-2, inplace_param_threshold=5000)
    for mb, ids in enumerate(batches(3)):
        opt.ready_for_optimizer_step = False
        loss_of(model, ids).backward()
        torch.cuda.synchronize()
        for p in opt._offload_params:
            host = opt.state[p]["grad"]
            assert not host.is_cuda
            assert torch.equal(host.view(torch.int16), sums[names[p]].view(torch.int16)), (mb, names[p])
            assert opt.device_states[p].get("grad") is None  # nothing kept in HBM

    model, opt = build(spare_hbm=True)
    captured = capsys.readouterr()
    assert captured.out == "" and "HBM the optimizer may hold" in captured.err
    assert opt._grad_cache_write_back and len(opt._grad_cached) == len(opt._offload_params)
    assert len(opt._state_cached) == len(opt._offload_params)
    with pytest.raises(ValueError, match="prefetch_bytes"):
        build(prefetch_bytes=-1)
    with pytest.raises(ValueError, match="state_cache_bytes"):
        build(state_cache_bytes="lots")


def test_grad_cache_policy_is_validated():
    from offload_adam_amd import OffloadAdam

    with pytest.raises(ValueError, match="grad_cache_policy"):
        OffloadAdam(make_model(0), grad_cache_policy="sometimes")


@pytest.mark.parametrize("group_params,group_bytes", [(1, 1 << 30), (3, 1 << 30), (100, 1 << 30),
                                                      (100, 40_000)])
def test_step_groups_of_any_size_give_the_same_result(fixed_seed, monkeypatch, group_params,
                                                      group_bytes):
    from offload_adam_amd import offload_adam as oa_mod

    monkeypatch.setattr(oa_mod.OffloadAdam, "_STEP_GROUP_PARAMS", group_params)
    monkeypatch.setattr(oa_mod.OffloadAdam, "_STEP_GROUP_BYTES", group_bytes)
    for mode in ("stochastic_rounding", "fp31_master"):
        ref_model, _ = run_reference_adam(mode, steps=3, ga=2)
        model, _ = run_offload_adam(mode, steps=3, ga=2)
        assert_same_params(ref_model, model)


def test_backward_alone_completes_the_step(fixed_seed):
    """Hook mode: the step happens inside backward().  A loop that never calls
    step(), zero_grad() or touches ready_for_optimizer_step again still has every
    parameter stepped when backward() returns (the last group is closed by a
    callback on the autograd engine, not by the next call into the optimizer)."""
    from offload_adam_amd import Adam, OffloadAdam

    data = batches(4)
    ref = make_model(0)
    ref_opt = Adam(ref.parameters(), mode="fp31_master", lr=1e-2, weight_decay=0.01)
    for ids in data:
        loss_of(ref, ids).backward()
        ref_opt.step()
        ref_opt.zero_grad(set_to_none=True)
    model = make_model(0)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="fp31_master", lr=1e-2, weight_decay=0.01,
                          inplace_param_threshold=5000)
    opt.ready_for_optimizer_step = True
    for ids in data:
        loss_of(model, ids).backward()
        assert not opt._pending_steps and not opt._pending_inplace
        assert all(st["step"] > 0 for st in opt.state.values())
    torch.cuda.synchronize()
    assert_same_params(ref, model)


@pytest.mark.parametrize("reentrant", [False, True])
def test_activation_checkpointing_of_either_kind(fixed_seed, reentrant):
    """Re-entrant checkpointing runs nested backward passes (each with its own
    end-of-pass callbacks); the result is the same as without checkpointing."""
    from torch.utils.checkpoint import checkpoint

    from offload_adam_amd import OffloadAdam

    class Checkpointed(TinyNet):
        def forward(self, ids):
            x = self.emb(ids)
            for b in self.blocks:
                x = x + checkpoint(lambda y, b=b: b["down"](F.gelu(b["up"](b["norm"](y)))), x,
                                   use_reentrant=reentrant)
            return self.head(x)

    ref_model, _ = run_offload_adam("fp31_master", steps=3, ga=2)
    torch.manual_seed(0)
    model = Checkpointed().to(device="cuda", dtype=BF16)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="fp31_master", lr=1e-2, weight_decay=0.01,
                          inplace_param_threshold=5000)
    data = batches(6)
    for s_ in range(3):
        for mb in range(2):
            opt.ready_for_optimizer_step = mb == 1
            loss_of(model, data[s_ * 2 + mb]).backward()
        opt.step()
        opt.zero_grad()
    torch.cuda.synchronize()
    assert_same_params(ref_model, model)


def test_verbose_reports_pinned_memory_and_budgets(capsys):
    from offload_adam_amd import OffloadAdam

    model = make_model(0)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        OffloadAdam(model, mode="fp32_master", inplace_param_threshold=5000, verbose=1,
                    grad_cache_bytes=40_000)
    out = capsys.readouterr().out
    assert "Pinned host memory allocated" in out
    assert "In-place GPU states" in out
    assert "gradient cache" in out and "(1 params)" in out and "state cache" in out


def test_hooks_called_outside_backward_step_at_once(fixed_seed):
    """A gradient hook invoked by hand (no backward pass is running, so there is no
    engine to call back): the parameter is stepped before the hook returns."""
    from offload_adam_amd import OffloadAdam

    model = make_model(0)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="stochastic_rounding", lr=1e-2, inplace_param_threshold=5000)
    opt.ready_for_optimizer_step = True
    p = opt._offload_params[0]
    before = p.detach().clone()
    p.grad = torch.full_like(p, 0.01)
    opt._grad_hook(p)
    torch.cuda.synchronize()
    assert opt.state[p]["step"] == 1 and not opt._pending_steps
    assert not torch.equal(before, p.detach())


def test_transfer_streams_are_picked_by_measured_concurrency():
    """With more live streams than hardware queues, the optimizer still ends up
    with side streams whose copies run beside each other and beside kernels."""
    from offload_adam_amd.offload_adam import pick_transfer_streams

    crowd = [torch.cuda.Stream() for _ in range(5)]
    for s in crowd:
        with torch.cuda.stream(s):
            torch.zeros(16, device="cuda")
    torch.cuda.synchronize()
    with warnings.catch_warnings():
        warnings.simplefilter("error")  # a failed search warns
        h2d, d2h, report = pick_transfer_streams(torch.device("cuda:0"))
    assert h2d.cuda_stream != d2h.cuda_stream
    # serialised work measures 1.0; copies that overlap measure 0.6 (two directions)
    # and 0.72 (beside a kernel) on an idle MI355X
    assert report["concurrent"] and report["duplex_ratio"] < 0.9, report
    assert report["with_compute_ratio"] < 0.9, report
    _, opt = run_offload_adam("stochastic_rounding", steps=1, ga=1)
    assert opt.transfer_stream_report["concurrent"], opt.transfer_stream_report


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("ga", [1, 3])
def test_grads_on_device_gives_identical_results(fixed_seed, mode, ga):
    """offload_grads=False changes where the gradient sum waits, nothing else."""
    ref_model, ref_opt = run_offload_adam(mode, steps=4, ga=ga, decoupled_weight_decay=True)
    model, opt = run_offload_adam(mode, steps=4, ga=ga, decoupled_weight_decay=True,
                                  offload_grads=False)
    assert_same_params(ref_model, model)
    for pr, p in zip(ref_model.parameters(), model.parameters()):
        if p in opt._inplace_params:
            continue
        assert "grad" in ref_opt.state[pr] and ref_opt.state[pr]["grad"].is_pinned()
        assert "grad" not in opt.state[p]  # no host gradient buffer at all
        for key in opt._non_grad_keys:
            a, b = ref_opt.state[pr][key], opt.state[p][key]
            assert b.is_pinned() and torch.equal(a.view(torch.uint8), b.view(torch.uint8)), key
    per_elem = {"stochastic_rounding": 4, "fp32_master": 8, "fp31_master": 6,
                "fp32_master_custom_rounding": 6}[mode]
    n = sum(p.numel() for p in opt._offload_params)
    assert opt._estimate_pinned_bytes(opt._offload_params) == n * per_elem
    assert ref_opt._estimate_pinned_bytes(ref_opt._offload_params) == n * (per_elem + 2)


@pytest.mark.parametrize("ga", [1, 2])
def test_grads_on_device_with_clipping(fixed_seed, ga):
    ref_model, _ = run_offload_adam("fp31_master", steps=3, ga=ga, max_grad_norm=0.05)
    model, opt = run_offload_adam("fp31_master", steps=3, ga=ga, max_grad_norm=0.05,
                                  offload_grads=False)
    assert float(opt._clip_coef) < 1.0
    assert_same_params(ref_model, model)


@pytest.mark.parametrize("prefetch_bytes", [0, 200_000, 1 << 30])
def test_prefetch_budget_does_not_change_results(fixed_seed, prefetch_bytes):
    """Window sizes from 'minimum two parameters' to 'everything staged after
    the previous step' give the same bits."""
    ref_model, _ = run_reference_adam("stochastic_rounding", steps=4, ga=3)
    model, opt = run_offload_adam("stochastic_rounding", steps=4, ga=3,
                                  prefetch_bytes=prefetch_bytes)
    assert opt._PREFETCH_BYTES == prefetch_bytes
    assert_same_params(ref_model, model)
    model2, _ = run_offload_adam("stochastic_rounding", steps=4, ga=3,
                                 prefetch_bytes=prefetch_bytes, offload_grads=False)
    assert_same_params(ref_model, model2)


@pytest.mark.parametrize("kw", [dict(), dict(max_grad_norm=0.05), dict(offload_grads=False),
                                dict(spare_hbm=True), dict(spare_hbm=True, max_grad_norm=0.05),
                                dict(prefetch_bytes=0), dict(grad_cache_bytes=0),
                                dict(grad_cache_bytes=0, max_grad_norm=0.05),
                                dict(grad_cache_bytes=40_000), dict(state_cache_bytes="auto"),
                                dict(grad_cache_bytes="auto", grad_cache_policy="write_back"),
                                dict(spare_hbm=True, grad_cache_policy="write_through",
                                     max_grad_norm=0.05),
                                dict(grad_cache_policy="write_back", grad_cache_bytes=40_000),
                                dict(state_cache_bytes=200_000, grad_cache_bytes=0),
                                dict(state_cache_bytes=0, grad_cache_bytes=0, prefetch_bytes=0)])
def test_transfer_issue_order_respects_the_happens_before_edges(fixed_seed, monkeypatch, kw):
    """Log every H2D / kernel / D2H the optimizer issues and check, per parameter
    and state key: a key is on the device (H2D issued, not yet written back) when
    the kernel runs; it is written back after the kernel and before it is fetched
    again; nothing is fetched twice without a write-back in between; each
    offloaded parameter is stepped exactly once per optimizer step."""
    from offload_adam_amd import offload_adam as oa_mod

    log = []
    real = {n: getattr(oa_mod.OffloadAdam, n)
            for n in ("_issue_h2d_many", "_issue_d2h", "_issue_d2h_many", "_call_step_fn")}
    real_multi = oa_mod.adam_step_multi

    def h2d(self, items):  # every fetch goes through the batched form
        for p, keys in items:
            log.append(("h2d", p, tuple(keys)))
        return real["_issue_h2d_many"](self, items)

    def d2h(self, p, keys):
        log.append(("d2h", p, tuple(keys)))
        return real["_issue_d2h"](self, p, keys)

    def d2h_many(self, items):
        for p, keys in items:
            log.append(("d2h", p, tuple(keys)))
        return real["_issue_d2h_many"](self, items)

    def step(self, p, group, tensors, clip_coef=None):
        log.append(("step", p, tuple(tensors)))
        return real["_call_step_fn"](self, p, group, tensors, clip_coef)

    by_address = {}

    def multi(mode, params, states, *args, **kwargs):  # the grouped launch of the hook path
        for data, tensors in zip(params, states):
            log.append(("step", by_address[data.data_ptr()], tuple(tensors)))
        return real_multi(mode, params, states, *args, **kwargs)

    monkeypatch.setattr(oa_mod.OffloadAdam, "_issue_h2d_many", h2d)
    monkeypatch.setattr(oa_mod.OffloadAdam, "_issue_d2h", d2h)
    monkeypatch.setattr(oa_mod.OffloadAdam, "_issue_d2h_many", d2h_many)
    monkeypatch.setattr(oa_mod.OffloadAdam, "_call_step_fn", step)
    monkeypatch.setattr(oa_mod, "adam_step_multi", multi)
    real_init = oa_mod.OffloadAdam.__init__

    def init(self, model, *a, **k):
        by_address.update({q.data_ptr(): q for q in model.parameters()})
        return real_init(self, model, *a, **k)

    monkeypatch.setattr(oa_mod.OffloadAdam, "__init__", init)
    steps, ga = 3, 3
    model, opt = run_offload_adam("fp31_master", steps=steps, ga=ga, **kw)
    offloaded = set(opt._offload_params)
    on_device = {}  # (param, key) -> True while a fetched copy is live
    stepped = {p: 0 for p in offloaded}
    for op, p, keys in log:
        if p not in offloaded:
            assert op == "step"  # GPU-resident parameters never cross the link
            continue
        if op == "h2d":
            for k in keys:
                assert not on_device.get((p, k)), f"{k} fetched while a copy is on the device"
                on_device[(p, k)] = True
        elif op == "d2h":
            for k in keys:
                if k == "grad" and not opt.offload_grads:
                    continue
                # a cached gradient or state is written back and stays on the GPU as well
                on_device[(p, k)] = p in (opt._grad_cached if k == "grad" else opt._state_cached)
        else:
            stepped[p] += 1
            for k in opt._non_grad_keys:
                assert on_device.get((p, k)), f"kernel ran without {k} on the device"
            if opt.offload_grads and ga > 1:
                # under 'write_back' a cached gradient never left the GPU
                assert on_device.get((p, "grad")) or (
                    p in opt._grad_cached and opt._grad_cache_write_back
                ), "kernel ran without the accumulated gradient"
    assert set(stepped.values()) == {steps}
    # at the end of a step nothing but staged states of the next step is live, and
    # every state written by a kernel went back to the host
    last_step_index = max(i for i, e in enumerate(log) if e[0] == "step" and e[1] in offloaded)
    written_back = {(p, k) for op, p, keys in log[last_step_index:] if op == "d2h" for k in keys}
    p_last = log[last_step_index][1]
    assert {(p_last, k) for k in opt._non_grad_keys} <= written_back


def test_parameters_the_kernels_cannot_take_are_reported():
    """fp32 parameters: the step function's checks raise instead of the grouped
    launch reading them as bf16."""
    from offload_adam_amd import OffloadAdam

    for threshold in (0, 10**9):  # everything offloaded / everything GPU-resident
        torch.manual_seed(0)
        model = TinyNet().to(device="cuda", dtype=torch.float32)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, mode="stochastic_rounding", inplace_param_threshold=threshold)
        opt.ready_for_optimizer_step = True
        ids = batches(1)[0]
        with pytest.raises((TypeError, RuntimeError)):
            F.cross_entropy(model(ids).reshape(-1, 50), ids.reshape(-1)).backward()
            opt.step()
        opt._pending_steps.clear()
        opt._pending_inplace.clear()


def test_a_backward_pass_that_raises_does_not_stall_later_ones(fixed_seed):
    """A pass that raises midway never reaches its end-of-pass callbacks.  The passes
    after it still close their last group by themselves (no step(), no flag
    toggling in between)."""
    from offload_adam_amd import OffloadAdam

    class Boom(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            return x.clone()

        @staticmethod
        def backward(ctx, g):
            raise RuntimeError("boom")

    model = make_model(0)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="fp31_master", lr=1e-2, inplace_param_threshold=5000)
    opt.ready_for_optimizer_step = True
    ids = batches(1)[0]
    x = model.emb(ids)
    for i, b in enumerate(model.blocks):
        if i == 1:
            x = Boom.apply(x)  # head and the last block get their gradients, then it raises
        x = x + b["down"](F.gelu(b["up"](b["norm"](x))))
    with pytest.raises(RuntimeError, match="boom"):
        F.cross_entropy(model.head(x).float().reshape(-1, 50), ids.reshape(-1)).backward()
    for ids in batches(3, seed=2):
        loss_of(model, ids).backward()
        assert not opt._pending_steps and not opt._pending_inplace
    torch.cuda.synchronize()
    steps = {st["step"] for st in opt.state.values()}
    assert min(steps) >= 3


LARGE_CASES = [
    ("fp31_master", dict(grad_cache_bytes=0, state_cache_bytes=0)),
    ("fp31_master", dict()),
    ("fp31_master", dict(spare_hbm=True)),
    ("fp31_master", dict(spare_hbm=True, grad_cache_policy="write_through")),
    ("fp31_master", dict(spare_hbm=True, state_cache_bytes=0)),
    ("fp31_master", dict(prefetch_bytes=0, grad_cache_bytes=0)),
    ("fp31_master", dict(offload_grads=False)),
    ("fp31_master", dict(prefetch_policy="lazy", grad_cache_bytes=0)),
    ("fp31_master", dict(max_grad_norm=1e-3)),
    ("fp31_master", dict(max_grad_norm=1e-3, spare_hbm=True)),
    ("fp31_master", dict(max_grad_norm=1e-3, spare_hbm=True, grad_cache_policy="write_through")),
    ("fp31_master", dict(max_grad_norm=1e-3, offload_grads=False)),
    ("stochastic_rounding", dict()),
    ("stochastic_rounding", dict(spare_hbm=True)),
    ("fp32_master", dict()),
    ("fp32_master", dict(spare_hbm=True)),
]


@pytest.mark.parametrize("mode,kw", LARGE_CASES)
def test_large_parameters_equal_adam(fixed_seed, mode, kw):
    """Two 134 MB weights: each of their transfers takes over 2 ms, far longer than
    the kernels around it, so a kernel that does not wait for a fetch under way, or
    that overwrites a buffer under its write-back, gives different bits than the
    optimizer without offloading (tiny tensors cross the link before anything can
    overtake them and would hide it).  Hook path and clipping path, every cache
    setting."""
    from offload_adam_amd import Adam, OffloadAdam
    from offload_adam_amd.grad_clip import clip_coef_, grad_norm_

    def build():
        torch.manual_seed(0)
        return nn.Sequential(nn.Linear(8192, 8192, bias=False), nn.LayerNorm(8192),
                             nn.Linear(8192, 8192, bias=False)).to(device="cuda", dtype=BF16)

    g = torch.Generator().manual_seed(3)
    steps, ga = 3, 3
    data = [torch.randn(4, 8192, generator=g).to(device="cuda", dtype=BF16)
            for _ in range(steps * ga)]

    def loss(model, x):
        return model(x).float().pow(2).mean()

    max_norm = kw.get("max_grad_norm")
    ref = build()
    ref_opt = Adam(ref.parameters(), mode=mode, lr=1e-2)
    ref_params = list(ref.parameters())
    norms = torch.zeros(len(ref_params), dtype=BF16, device="cuda")
    coef = torch.ones((), dtype=BF16, device="cuda")
    model = build()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode=mode, lr=1e-2, **kw)
    assert len(opt._offload_params) == 2
    for step in range(steps):
        for mb in range(ga):
            x = data[step * ga + mb]
            loss(ref, x).backward()
            opt.ready_for_optimizer_step = mb == ga - 1
            loss(model, x).backward()
        if max_norm is not None:
            for i, p in enumerate(ref_params):
                grad_norm_(p.grad.reshape(-1), norms[i])
            clip_coef_(norms, max_norm, coef)
            for p in ref_params:
                p.grad.mul_(coef)
        ref_opt.step()
        ref_opt.zero_grad(set_to_none=True)
        opt.step()
    torch.cuda.synchronize()
    if max_norm is not None:
        assert float(coef) < 1.0
    assert_same_params(ref, model)


@pytest.mark.parametrize("fmt", ["int8", "int4", "nf4", "nvfp4"])
@pytest.mark.parametrize("kw", [dict(), dict(spare_hbm=True)])
def test_large_quantised_parameters_equal_adam(fmt, kw):
    """The same with two quantised 8192 x 8192 weights (268 MB of fp32 master each):
    payloads and masters end up bit-identical to the optimizer without offloading."""
    from offload_adam_amd import Adam, OffloadAdam
    from offload_adam_amd.qweight import FORMATS, QWeightBase, quantize_linears

    def build():
        torch.manual_seed(0)
        m = nn.Sequential(nn.Linear(8192, 8192, bias=False), nn.LayerNorm(8192),
                          nn.Linear(8192, 8192, bias=False)).to(device="cuda", dtype=BF16)
        assert len(quantize_linears(m, FORMATS[fmt]).quantized) == 2
        return m

    g = torch.Generator().manual_seed(3)
    data = [torch.randn(4, 8192, generator=g).to(device="cuda", dtype=BF16) for _ in range(6)]
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        ref = build()
        ref_opt = Adam(ref.parameters(), mode="fp32_master", lr=1e-3)
        model = build()
        opt = OffloadAdam(model, mode="fp32_master", lr=1e-3, **kw)
        for step in range(3):
            for mb in range(2):
                x = data[step * 2 + mb]
                ref(x).float().pow(2).mean().backward()
                opt.ready_for_optimizer_step = mb == 1
                model(x).float().pow(2).mean().backward()
            ref_opt.step()
            ref_opt.zero_grad(set_to_none=True)
            opt.step()
    torch.cuda.synchronize()
    for (n, pr), (_, p) in zip(ref.named_parameters(), model.named_parameters()):
        if isinstance(p.data, QWeightBase):
            for name in type(p.data)._PAYLOAD:
                a, b = getattr(pr.data, name), getattr(p.data, name)
                assert torch.equal(a.reshape(-1).view(torch.uint8),
                                   b.reshape(-1).view(torch.uint8)), (n, name)
            assert torch.equal(ref_opt.state[pr]["master_params"].cpu(),
                               opt.state[p]["master_params"]), n
        else:
            assert torch.equal(pr.view(torch.int16), p.view(torch.int16)), n


def test_clipping_path_gives_its_spare_staging_budget_to_the_state_cache():
    """States staged ahead of step() would hold HBM through the last backward pass;
    with spare_hbm, unless the caller sizes a budget, the optimizer keeps them instead."""
    from offload_adam_amd import OffloadAdam

    def build(**kw):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            return OffloadAdam(make_model(0), mode="fp31_master", inplace_param_threshold=5000,
                               **kw)

    hook = build(spare_hbm=True)
    assert hook._prestage_bytes == hook._PREFETCH_BYTES > 0
    clip = build(max_grad_norm=1.0, spare_hbm=True)
    assert clip._prestage_bytes == 0 and len(clip._state_cached) == len(clip._offload_params)
    sized = build(max_grad_norm=1.0, spare_hbm=True, prefetch_bytes=123_456)
    assert sized._prestage_bytes == 123_456
    sized = build(max_grad_norm=1.0, spare_hbm=True, state_cache_bytes=0)
    assert sized._prestage_bytes == sized._PREFETCH_BYTES and not sized._state_cached
    plain = build(max_grad_norm=1.0)
    assert plain._prestage_bytes == plain._PREFETCH_BYTES and not plain._state_cached


# ----------------------------------------------- pinned memory beyond the limit


def _pinned_need(mode, **kw):
    model, opt = run_offload_adam(mode, steps=0, ga=1, **kw)
    return opt._estimate_pinned_bytes(opt._offload_params), opt


@pytest.mark.parametrize("mode,kw", [
    ("stochastic_rounding", dict()),
    ("fp32_master", dict()),
    ("fp31_master", dict(max_grad_norm=0.05)),
])
@pytest.mark.parametrize("ga", [1, 3])
@pytest.mark.parametrize("fraction", [0.9, 0.55])
def test_states_beyond_the_pinned_limit_stay_in_hbm(fixed_seed, capsys, mode, kw, ga, fraction):
    """A limit below what the states need is a placement decision, not an error:
    gradients stay in HBM first (0.9 of the need), then whole parameters (0.55: less
    than the states without any gradient); one notice; results bit-identical to the
    unconstrained run; the host never holds more than the limit."""
    need, free_opt = _pinned_need(mode, **kw)
    assert free_opt.pinned_limit_report is None and not free_opt._grad_on_device
    n_offloaded = len(free_opt._offload_params)
    ref_model, ref_opt = run_offload_adam(mode, steps=3, ga=ga, decoupled_weight_decay=True, **kw)
    capsys.readouterr()
    limit = int(need * fraction)
    model, opt = run_offload_adam(mode, steps=3, ga=ga, decoupled_weight_decay=True,
                                  pinned_limit_bytes=limit, **kw)
    err = capsys.readouterr().err
    assert err.count("page-locked host memory are needed") == 1 and "kept in HBM instead" in err
    report = opt.pinned_limit_report
    assert report["needed_bytes"] == need and report["limit_bytes"] == limit
    assert opt._estimate_pinned_bytes(opt._offload_params) <= limit
    pinned = sum(t.numel() * t.element_size() for p in opt._offload_params
                 for t in opt.state[p].values() if torch.is_tensor(t) and t.is_pinned())
    assert pinned == opt._estimate_pinned_bytes(opt._offload_params)
    assert report["grads_in_hbm"] + report["params_in_hbm"] > 0
    if fraction < 0.6:
        assert report["params_in_hbm"] > 0 and len(opt._offload_params) < n_offloaded
        assert all(p in opt._grad_on_device for p in opt._offload_params)
    else:
        assert report["params_in_hbm"] == 0 and 0 < len(opt._grad_on_device) < n_offloaded
    assert_same_params(ref_model, model)
    for pr, p in zip(ref_model.parameters(), model.parameters()):
        for key in opt._non_grad_keys:
            a, b = ref_opt.state[pr][key], opt.state[p][key]
            assert torch.equal(a.cpu().view(torch.uint8), b.cpu().view(torch.uint8)), key
        if p in opt._grad_on_device:
            assert "grad" not in opt.state[p]


def test_quantised_weights_keep_their_masters_on_the_host_under_a_limit(capsys):
    """Quantised parameters are never made resident; when nothing else can move,
    the constructor raises and says why."""
    from offload_adam_amd import OffloadAdam
    from offload_adam_amd.qweight import Int8QWeight, quantize_linears

    def build(limit):
        model = make_model(0)
        quantize_linears(model, Int8QWeight)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            return OffloadAdam(model, mode="fp32_master", inplace_param_threshold=0,
                               pinned_limit_bytes=limit)

    free = build(None)
    need = free._estimate_pinned_bytes(free._offload_params)
    quant_states = sum(p.numel() for p in free._quant_params) * 8
    opt = build(quant_states + 4096)
    offloaded = {id(p) for p in opt._offload_params}  # (== is not defined for quantised weights)
    assert all(id(p) in offloaded for p in opt._quant_params)
    assert opt.pinned_limit_report["params_in_hbm"] > 0
    with pytest.raises(RuntimeError, match="does not close the gap"):
        build(quant_states - 4096)
    assert need > quant_states


@pytest.mark.parametrize("value,ok", [(2 ** 20, True), (2e6, True), (2.5, False), (-1, False),
                                      ("auto", False), (True, False)])
def test_byte_budgets_accept_any_integral_number(value, ok):
    """numpy integers and integral floats are byte counts too; 'auto' only where it means something."""
    import numpy as np

    from offload_adam_amd import OffloadAdam

    def build(**kw):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            return OffloadAdam(make_model(0), inplace_param_threshold=5000, **kw)

    if ok:
        assert build(pinned_limit_bytes=value)._pinned_limit_arg == int(value)
        assert build(prefetch_bytes=np.int64(value))._PREFETCH_BYTES == int(value)
        assert build(grad_cache_bytes=value, state_cache_bytes=np.int32(4096)) is not None
        assert build(pending_writeback_bytes=value)._writeback_pending_limit == int(value)
    else:
        with pytest.raises(ValueError, match="pinned_limit_bytes"):
            build(pinned_limit_bytes=value)
        with pytest.raises(ValueError, match="pending_writeback_bytes"):
            build(pending_writeback_bytes=value)
        if value != "auto":
            with pytest.raises(ValueError, match="prefetch_bytes"):
                build(prefetch_bytes=value)


def test_saving_one_carved_state_writes_its_arena_and_detached_does_not(tmp_path):
    """States carved from one arena share its storage: ``torch.save`` of one of them
    serialises the arena; ``pinned_alloc.detached`` gives copies that stand alone."""
    from offload_adam_amd.pinned_alloc import alloc_pinned_states, detached

    a, b, c = alloc_pinned_states([((1000,), torch.float32), ((300_000,), BF16),
                                   ((70_000,), torch.int16)], numa_node=None)
    a.fill_(1.5)
    arena_bytes = a.untyped_storage().nbytes()
    assert arena_bytes >= 4096 + 600_064 + 140_000
    assert b.untyped_storage().data_ptr() == a.untyped_storage().data_ptr()
    torch.save(a, tmp_path / "view.pt")
    assert (tmp_path / "view.pt").stat().st_size >= arena_bytes
    own = detached({"state": {0: {"exp_avg": a, "step": 3}}, "list": [c]})
    assert own["state"][0]["step"] == 3 and torch.equal(own["state"][0]["exp_avg"], a)
    assert own["state"][0]["exp_avg"].untyped_storage().nbytes() == 4000
    torch.save(own["state"][0]["exp_avg"], tmp_path / "own.pt")
    assert (tmp_path / "own.pt").stat().st_size < 4000 + 4096
    loaded = torch.load(tmp_path / "own.pt", weights_only=True)
    assert torch.equal(loaded, a)
