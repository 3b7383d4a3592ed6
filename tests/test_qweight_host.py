"""Host-side contracts of the quantised-weight subclasses and of the model
surgery around them: what ``state_dict`` holds, that it survives safetensors and
``torch.load(weights_only=True)``, that a reloaded model dequantises to the same
bits, the checkpoint-config dictionaries, and the error behaviour of the
optimizers' constructors.

The bodies run wherever the tensors live: on the CPU the subclasses use their
torch specification functions, on a GPU (second parametrisation, marked ``gpu``)
the HIP codec kernels - both must agree with the oracle and with each other.
Areas follow the reference's tests/test_state_dict_roundtrip.py,
tests/test_hf_config.py and the CPU parts of tests/test_int8.py / test_int4.py /
test_nf4.py / test_nvfp4.py.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn

from offload_adam_amd.qweight import (Int4QWeight, Int8QWeight, NF4QWeight, NVFP4QWeight,
                                      QWeightBase, quantize_linears)

FORMATS = [
    pytest.param(Int4QWeight, {"group_size": 128}, id="int4"),
    pytest.param(Int8QWeight, {}, id="int8"),
    pytest.param(NF4QWeight, {"blocksize": 64}, id="nf4"),
    pytest.param(NVFP4QWeight, {}, id="nvfp4"),
]
DEVICES = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]


class TwoLinears(nn.Module):
    def __init__(self, in_f=256, mid_f=256, out_f=128):
        super().__init__()
        self.l1 = nn.Linear(in_f, mid_f, bias=False)
        self.ln = nn.LayerNorm(mid_f)
        self.l2 = nn.Linear(mid_f, out_f, bias=True)

    def forward(self, x):
        return self.l2(self.ln(self.l1(x)))


def build(weight_cls, kw, device, seed=0):
    torch.manual_seed(seed)
    model = TwoLinears().to(torch.bfloat16).to(device)
    report = quantize_linears(model, weight_cls, **kw)
    assert report.quantized == ["l1", "l2"] and not report.incompatible and not report.excluded
    return model


# ----------------------------------------------------------------- state_dict


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_state_dict_holds_plain_tensors_under_canonical_keys(weight_cls, kw, device):
    model = build(weight_cls, kw, device)
    assert isinstance(model.l1.weight.data, weight_cls)
    sd = model.state_dict()
    for key, value in sd.items():
        assert type(value) is torch.Tensor, (key, type(value))
    for name in ("l1", "l2"):
        for suffix in weight_cls.canonical_key_suffixes():
            assert f"{name}.{suffix}" in sd
    assert {"ln.weight", "ln.bias", "l2.bias"} <= set(sd)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_round_trip_through_safetensors_and_weights_only_load(weight_cls, kw, device, tmp_path):
    from safetensors.torch import load_file, save_file

    model = build(weight_cls, kw, device)
    sd = {k: v.contiguous() for k, v in model.state_dict().items()}
    save_file(sd, str(tmp_path / "m.safetensors"))
    torch.save(sd, tmp_path / "m.pt")
    for loaded in (load_file(str(tmp_path / "m.safetensors")),
                   torch.load(tmp_path / "m.pt", weights_only=True)):
        assert set(loaded) == set(sd)
        for key in sd:
            a, b = sd[key].cpu(), loaded[key].cpu()
            assert a.dtype == b.dtype and torch.equal(a.view(torch.uint8), b.view(torch.uint8)), key


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_reloaded_model_dequantises_to_the_same_bits(weight_cls, kw, device):
    src = build(weight_cls, kw, device, seed=0)
    dst = build(weight_cls, kw, device, seed=1)  # different weights before the load
    before = dst.l1.weight.data.dequantize().clone()
    missing, unexpected = dst.load_state_dict(src.state_dict())
    assert not missing and not unexpected
    for name in ("l1", "l2"):
        a = getattr(src, name).weight.data.dequantize()
        b = getattr(dst, name).weight.data.dequantize()
        assert isinstance(getattr(dst, name).weight.data, weight_cls)
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), name
    assert not torch.equal(before, dst.l1.weight.data.dequantize())
    x = torch.randn(4, 256, dtype=torch.bfloat16, device=device)
    assert torch.equal(src(x), dst(x))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_plain_float_checkpoint_requantises_on_load(weight_cls, kw, device):
    """A checkpoint of the unquantised model loads into the quantised one: the
    float ``weight`` goes through ``copy_`` and is encoded on the way in."""
    torch.manual_seed(3)
    plain = TwoLinears().to(torch.bfloat16).to(device)
    model = build(weight_cls, kw, device, seed=4)
    model.load_state_dict(plain.state_dict())
    expect = weight_cls.from_float(plain.l1.weight.data, **kw).dequantize()
    got = model.l1.weight.data.dequantize()
    assert isinstance(model.l1.weight.data, weight_cls)
    assert torch.equal(expect.view(torch.int16), got.view(torch.int16))


@pytest.mark.gpu
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_cpu_and_gpu_encoders_agree(weight_cls, kw):
    """torch specification (CPU tensors) == HIP kernels (GPU tensors), payload by payload."""
    torch.manual_seed(7)
    w = (torch.randn(96, 512) * 0.05).to(torch.bfloat16)
    on_cpu = weight_cls.from_float(w, **kw).to_plain_state_dict()
    on_gpu = weight_cls.from_float(w.cuda(), **kw).to_plain_state_dict()
    assert set(on_cpu) == set(on_gpu)
    for key in on_cpu:
        a, b = on_cpu[key].contiguous(), on_gpu[key].cpu().contiguous()
        assert a.dtype == b.dtype and a.shape == b.shape, key
        assert torch.equal(a.reshape(-1).view(torch.uint8), b.reshape(-1).view(torch.uint8)), key


# ------------------------------------------------ layout anchors (class API)


def test_int8_anchor_through_the_class():
    w = torch.tensor([[0.0, 0.5, -2.0, 1.0]])
    q = Int8QWeight.from_float(w, scale_dtype=torch.float32)
    assert q.weight.tolist() == [[0, 32, -127, 64]]
    assert float(q.scales[0]) == pytest.approx(2.0 / 127.0, rel=1e-7)


def test_int4_anchor_through_the_class():
    w = torch.arange(-8, 0, dtype=torch.float32).reshape(1, 8)
    q = Int4QWeight.from_float(w, group_size=8, scale_dtype=torch.float32)
    assert q.qweight.shape == (1, 1) and q.scales.shape == (1, 1)
    assert int(q.qweight[0, 0]) & 0xFFFFFFFF == 0x76543210
    assert float(q.scales[0, 0]) == 1.0


def test_nf4_and_nvfp4_nibble_order(oracle):
    lut = np.array([oracle.lib().oaref_nf4_lut(i) for i in range(16)], dtype=np.float32)
    row = torch.from_numpy(np.concatenate([lut[:8], np.full(56, 0.0, np.float32)])).reshape(1, 64)
    row[0, 63] = 1.0  # absmax 1 so the codes of the first eight are 0..7
    row[0, 62] = -1.0
    q = NF4QWeight.from_float(row, blocksize=64)
    assert q.weight_packed[0, :4].tolist() == [0x01, 0x23, 0x45, 0x67]  # even column high
    vals = torch.tensor([[0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0] + [0.0] * 8])
    big = torch.zeros(1, 16)
    big[0, 0] = 448.0 * 6.0
    f = NVFP4QWeight.from_float(torch.cat([vals, big], dim=1))
    assert float(f.global_scale) == 1.0
    assert f.weight_packed[0, :4].tolist() == [0x10, 0x32, 0x54, 0x76]  # even column low


@pytest.mark.parametrize("weight_cls,kw,bad_shape", [
    (Int4QWeight, {"group_size": 128}, (64, 100)),
    (NF4QWeight, {"blocksize": 64}, (64, 100)),
    (NVFP4QWeight, {}, (64, 24)),
])
def test_can_quantize_rejects_what_the_layout_cannot_hold(weight_cls, kw, bad_shape):
    assert weight_cls.can_quantize(torch.zeros(64, 256), **kw)
    assert not weight_cls.can_quantize(torch.zeros(*bad_shape), **kw)
    assert not weight_cls.can_quantize(torch.zeros(256), **kw)
    model = nn.Sequential(nn.Linear(bad_shape[1], bad_shape[0], bias=False))
    report = quantize_linears(model, weight_cls, **kw)
    assert report.quantized == [] and len(report.incompatible) == 1
    with pytest.raises(ValueError):
        quantize_linears(model, weight_cls, strict=True, **kw)


def test_skip_patterns_leave_modules_alone():
    model = nn.ModuleDict({"body": nn.Linear(128, 128), "lm_head": nn.Linear(128, 64)})
    report = quantize_linears(model, Int8QWeight, skip_patterns=("lm_head",))
    assert report.quantized == ["body"] and report.excluded == ["lm_head"]
    assert not isinstance(model["lm_head"].weight.data, QWeightBase)


# -------------------------------------------------------- checkpoint configs


def test_checkpoint_config_dictionaries():
    c = Int4QWeight.build_hf_quantization_config(skip_patterns=("lm_head",), group_size=128)
    assert (c["quant_method"], c["bits"], c["group_size"], c["sym"], c["desc_act"]) == (
        "gptq", 4, 128, True, False)
    assert c["modules_to_not_convert"] == ["lm_head"]
    c = Int8QWeight.build_hf_quantization_config(skip_patterns=("lm_head",))
    w = c["config_groups"]["group_0"]["weights"]
    assert (c["quant_method"], c["format"]) == ("compressed-tensors", "pack-quantized")
    assert (w["num_bits"], w["type"], w["strategy"], w["symmetric"]) == (8, "int", "channel", True)
    assert c["ignore"] == ["lm_head"]
    c = NF4QWeight.build_hf_quantization_config(skip_patterns=("lm_head",))
    assert (c["quant_method"], c["load_in_4bit"], c["bnb_4bit_quant_type"]) == (
        "bitsandbytes", True, "nf4")
    assert c["bnb_4bit_use_double_quant"] is False and c["bnb_4bit_compute_dtype"] == "bfloat16"
    assert c["llm_int8_skip_modules"] == ["lm_head"]
    assert NF4QWeight.build_hf_quantization_config(
        compute_dtype="float16")["bnb_4bit_compute_dtype"] == "float16"
    c = NVFP4QWeight.build_hf_quantization_config(skip_patterns=("lm_head",))
    w = c["config_groups"]["group_0"]["weights"]
    assert (c["quant_method"], c["format"]) == ("compressed-tensors", "nvfp4-pack-quantized")
    assert (w["num_bits"], w["type"], w["group_size"]) == (4, "float", 16)
    assert c["ignore"] == ["lm_head"]


def test_update_hf_config_writes_the_model_config():
    from types import SimpleNamespace

    model = TwoLinears()
    model.config = SimpleNamespace()
    quantize_linears(model, Int4QWeight, skip_patterns=("l2",), update_hf_config=True,
                     group_size=128)
    assert model.config.quantization_config["quant_method"] == "gptq"
    assert model.config.quantization_config["modules_to_not_convert"] == ["l2"]


# ------------------------------------------- optimizer argument validation


def test_constructor_errors_come_before_any_allocation():
    """Bad arguments raise on a machine with no GPU: nothing is allocated first."""
    from offload_adam_amd import Adam, DistributedOffloadAdam, OffloadAdam
    from offload_adam_amd.pinned_alloc import resolve_numa_target

    model = TwoLinears()
    with pytest.raises(ValueError, match="prefetch_policy"):
        OffloadAdam(model, prefetch_policy="sometimes")
    with pytest.raises(AssertionError, match="Invalid mode"):
        OffloadAdam(model, mode="fp64_master")
    with pytest.raises(AssertionError):
        Adam(model.parameters(), mode="fp64_master")
    with pytest.raises(NotImplementedError):
        DistributedOffloadAdam(model)
    with pytest.raises(ValueError):
        resolve_numa_target(1.5)
    assert resolve_numa_target(None) is None
    qmodel = TwoLinears()
    quantize_linears(qmodel, Int8QWeight)
    with pytest.raises(ValueError, match="fp32_master"):
        OffloadAdam(qmodel, mode="stochastic_rounding")


def test_folded_betas_closed_form():
    from offload_adam_amd.kernels._common import folded_betas

    assert folded_betas(0.9, 0.999, 1) == (0.0, 0.0)
    b1, b2 = folded_betas(0.9, 0.999, 10)
    assert b1 == pytest.approx(0.846466006721237, rel=1e-15)
    assert b2 == pytest.approx(0.8995491745886153, rel=1e-15)
    for t in (2, 7, 1000):
        b1, _ = folded_betas(0.9, 0.999, t)
        assert b1 == pytest.approx(0.9 * (1 - 0.9 ** (t - 1)) / (1 - 0.9 ** t), rel=1e-12)


def test_leaf_module_scan():
    from offload_adam_amd.offload_adam import get_leaf_modules_with_params

    class Holder(nn.Module):
        def __init__(self):
            super().__init__()
            self.own = nn.Parameter(torch.zeros(3))  # held beside a child: not seen
            self.child = nn.Linear(2, 2)
            self.frozen = nn.Linear(2, 2)
            self.frozen.requires_grad_(False)

    found = get_leaf_modules_with_params(nn.Sequential(Holder(), nn.LayerNorm(2)))
    assert [type(m).__name__ for m in found] == ["Linear", "LayerNorm"]


# ------------------------------------------------- F.linear, copy_, partial loads


def payload_of(qw):
    return {k: v for k, v in qw.to_plain_state_dict().items()}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_linear_forward_and_backward_equal_the_dequantised_layer(weight_cls, kw, device):
    """``F.linear`` on a quantised weight (reference: int8.py:378-407 and the same
    in the other formats) gives what a plain layer holding the dequantised weight
    gives; the weight's gradient is a plain tensor of the full shape."""
    import torch.nn.functional as F

    torch.manual_seed(0)
    out_f, in_f, batch = 64, 256, 8
    dtype = torch.bfloat16 if device == "cuda" else torch.float32
    w = (torch.randn(out_f, in_f) * 0.05).to(device=device, dtype=dtype)
    b = (torch.randn(out_f) * 0.05).to(device=device, dtype=dtype).requires_grad_(True)
    x = torch.randn(batch, in_f).to(device=device, dtype=dtype).requires_grad_(True)
    qw = weight_cls.from_float(w, **kw).requires_grad_(True)
    F.linear(x, qw, b).sum().backward()

    x2 = x.detach().clone().requires_grad_(True)
    b2 = b.detach().clone().requires_grad_(True)
    w2 = qw.dequantize(dtype).detach().clone().requires_grad_(True)
    y2 = F.linear(x2, w2, b2)
    y2.sum().backward()
    y = F.linear(x.detach(), qw.detach(), b.detach())
    tol = dict(atol=1e-2, rtol=1e-2)
    assert torch.allclose(y, y2, **tol)
    assert torch.allclose(x.grad, x2.grad, **tol)
    assert torch.allclose(b.grad, b2.grad, **tol)
    assert torch.allclose(qw.grad.float(), w2.grad.float(), **tol)  # stored in the weight's dtype
    assert type(qw.grad) is torch.Tensor and qw.grad.shape == (out_f, in_f)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_copy_of_a_float_tensor_re_encodes_like_a_fresh_quantisation(weight_cls, kw, device):
    """``qw.copy_(fp32)`` - what both optimizers do with the new master - leaves the
    payload that ``from_float`` of the same values builds, bit for bit."""
    torch.manual_seed(0)
    old = (torch.randn(64, 256) * 0.05).to(device=device, dtype=torch.bfloat16)
    new = torch.randn(64, 256, dtype=torch.float32, device=device)
    qw = weight_cls.from_float(old, **kw)
    qw.copy_(new)
    fresh = weight_cls.from_float(new, **kw)
    a, b = payload_of(qw), payload_of(fresh)
    assert a.keys() == b.keys()
    for key in a:
        if "quant_state" in key:
            continue  # serialised metadata; it names the dtype the weight was built from
        if a[key].dtype == b[key].dtype:
            assert torch.equal(a[key], b[key]), key
        else:  # from_float of an fp32 tensor may keep wider scales than the stored ones
            assert torch.equal(a[key].float(), b[key].to(a[key].dtype).float()), key


@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_partial_checkpoint_reports_the_keys_it_lacks(weight_cls, kw):
    src, dst = build(weight_cls, kw, "cpu", seed=0), build(weight_cls, kw, "cpu", seed=1)
    full = src.state_dict()
    dropped = "l2." + weight_cls.canonical_key_suffixes()[0]
    assert dropped in full
    partial = {k: v for k, v in full.items() if k != dropped}
    missing, unexpected = dst.load_state_dict(partial, strict=False)
    assert not unexpected
    assert missing and all(k.startswith("l2.") for k in missing)


def test_update_hf_config_is_opt_in_and_needs_a_config():
    from types import SimpleNamespace

    model = TwoLinears().to(torch.bfloat16)
    model.config = SimpleNamespace()
    quantize_linears(model, Int8QWeight)  # update_hf_config defaults to False
    assert not hasattr(model.config, "quantization_config")
    bare = TwoLinears().to(torch.bfloat16)
    quantize_linears(bare, Int8QWeight, update_hf_config=True)  # no .config: nothing to patch
    assert not hasattr(bare, "config")


def test_save_quantized_pretrained_merges_the_config(tmp_path):
    import json

    from offload_adam_amd.qweight import save_quantized_pretrained

    class Saves(TwoLinears):
        def save_pretrained(self, directory):
            directory.mkdir(parents=True, exist_ok=True)
            (directory / "config.json").write_text(json.dumps({"model_type": "toy"}))

    model = Saves().to(torch.bfloat16)
    quantize_linears(model, Int4QWeight, group_size=128, skip_patterns=("l2",))
    save_quantized_pretrained(model, tmp_path / "out", Int4QWeight, skip_patterns=("l2",),
                              group_size=128)
    written = json.loads((tmp_path / "out" / "config.json").read_text())
    assert written["model_type"] == "toy"
    assert written["quantization_config"] == Int4QWeight.build_hf_quantization_config(
        skip_patterns=("l2",), group_size=128)


# ------------------------------------------------------- dequantisation cache


@pytest.fixture
def dequant_cache():
    from offload_adam_amd.qweight import cache_dequantized_weights

    previous = cache_dequantized_weights(True)
    yield
    cache_dequantized_weights(previous)


def count_dequantize_calls(monkeypatch, weight_cls):
    calls = []
    real = weight_cls.dequantize

    def counting(self, dtype=None):
        calls.append(dtype)
        return real(self, dtype)

    monkeypatch.setattr(weight_cls, "dequantize", counting)
    return calls


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_dequantised_weights_are_decoded_once_until_the_payload_changes(
        weight_cls, kw, device, dequant_cache, monkeypatch):
    """With ``cache_dequantized_weights(True)`` forward and backward of several
    micro-batches share one decode; ``copy_`` of new values (what the optimizers do),
    loading a state dict and a payload written by hand each bring a new one; outputs
    equal those without the cache."""
    from offload_adam_amd.qweight import cache_dequantized_weights

    model = build(weight_cls, kw, device)
    dtype = torch.bfloat16
    torch.manual_seed(2)
    xs = [torch.randn(4, 256).to(device=device, dtype=dtype) for _ in range(3)]
    calls = count_dequantize_calls(monkeypatch, weight_cls)
    outs = []
    for x in xs:
        y = model(x)
        y.float().sum().backward()
        outs.append(y.detach().clone())
    assert len(calls) == 2  # two quantised layers, three forward and backward passes each
    grads = [p.grad.clone() for p in model.parameters()]

    cache_dequantized_weights(False)
    model.zero_grad(set_to_none=True)
    for x, y_cached in zip(xs, outs):
        y = model(x)
        y.float().sum().backward()
        assert torch.equal(y, y_cached)
    for p, g in zip(model.parameters(), grads):
        assert torch.equal(p.grad, g)
    assert len(calls) == 2 + 2 * 2 * 3
    cache_dequantized_weights(True)

    # new values through copy_: decoded again, and the output follows
    new = torch.randn(256, 256, dtype=torch.float32, device=device) * 0.05
    model.l1.weight.data.copy_(new)
    before = len(calls)
    y_new = model(xs[0])
    assert len(calls) == before + 1 and not torch.equal(y_new, outs[0])
    cache_dequantized_weights(False)
    assert torch.equal(model(xs[0]), y_new)
    cache_dequantized_weights(True)

    # a state dict from another model
    other = build(weight_cls, kw, device, seed=5)
    model.load_state_dict(other.state_dict())
    assert torch.equal(model(xs[1]), other(xs[1]))


@pytest.mark.gpu
@pytest.mark.parametrize("weight_cls,kw", FORMATS)
def test_the_fused_step_invalidates_the_dequantisation_cache(weight_cls, kw, dequant_cache):
    """The fused step + re-encode writes the payload through raw pointers; the
    cached decode must not survive it."""
    from offload_adam_amd.kernels import adam_step_fp32_master

    torch.manual_seed(0)
    layer = nn.Linear(256, 128, bias=False).to(device="cuda", dtype=torch.bfloat16)
    quantize_linears(layer, weight_cls, **kw)
    p = layer.weight
    x = torch.randn(4, 256, device="cuda", dtype=torch.bfloat16)
    y0 = layer(x).detach().clone()
    versions = [getattr(p, n)._version for n in weight_cls._PAYLOAD]
    states = {"grad": torch.randn(128, 256, device="cuda").to(torch.bfloat16),
              "exp_avg": torch.zeros(128, 256, device="cuda", dtype=torch.bfloat16),
              "exp_avg_sq": torch.zeros(128, 256, device="cuda", dtype=torch.bfloat16),
              "master_params": p.data.dequantize(torch.float32).contiguous()}
    adam_step_fp32_master(p.data, states, 0.05, 0.0, 0.9, 0.999, 1e-8, 1)
    assert all(getattr(p, n)._version > v for n, v in zip(weight_cls._PAYLOAD, versions))
    y1 = layer(x)
    assert not torch.equal(y0, y1)
    assert torch.equal(y1, x @ p.data.dequantize(torch.bfloat16).T)
