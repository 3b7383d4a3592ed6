"""The optimizer side of quantisation-aware training, as a user of the reference
drives it: ``quantize_linears(model, ...)`` then ``Adam(model.parameters(),
mode='fp32_master')`` or ``OffloadAdam(model, mode='fp32_master')``.

Behaviour checked here is the contract the reference's tests/test_qat_optimizer.py
pins (:84-426): what ``quantize_linears`` reports, how the fp32 master is seeded
and flagged, when the lossy-master warning fires, how
``load_master_from_pretrained`` / ``load_master_state_dict`` refill it, and what
survives a ``state_dict`` round trip.  Every step runs this package's HIP kernels.
"""

import json
import warnings

import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16
FEATURES = 128  # one int4 group of 128 per row


class OneLinear(nn.Module):
    def __init__(self):
        super().__init__()
        self.l1 = nn.Linear(FEATURES, FEATURES, bias=False)

    def forward(self, x):
        return self.l1(x)


class TwoLinears(nn.Module):
    def __init__(self):
        super().__init__()
        self.l1 = nn.Linear(FEATURES, FEATURES, bias=False)
        self.l2 = nn.Linear(FEATURES, FEATURES, bias=False)

    def forward(self, x):
        return self.l2(self.l1(x))


class LinearAndNorm(nn.Module):
    def __init__(self):
        super().__init__()
        self.l1 = nn.Linear(FEATURES, FEATURES, bias=False)
        self.ln = nn.LayerNorm(FEATURES)

    def forward(self, x):
        return self.ln(self.l1(x))


def fresh(cls=OneLinear, quantized=False):
    from offload_adam_amd.qweight import Int4QWeight, quantize_linears

    torch.manual_seed(0)
    model = cls().to(device="cuda", dtype=BF16)
    if quantized:
        quantize_linears(model, Int4QWeight, group_size=128)
    return model


def quantize(model):
    from offload_adam_amd.qweight import Int4QWeight, quantize_linears

    return quantize_linears(model, Int4QWeight, group_size=128)


def one_backward(model):
    torch.manual_seed(1)
    x = torch.randn(4, FEATURES, dtype=BF16, device="cuda")
    model(x).sum().backward()


def lossy_master_warnings(fn):
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        fn()
    return sum("lossy dequant-seeded" in str(w.message) for w in caught)


def write_checkpoint(model, path, only=None):
    from safetensors.torch import save_file

    save_file({n: p.detach().cpu().contiguous() for n, p in model.named_parameters()
               if only is None or n in only}, str(path))


# ---------------------------------------------------------------- quantize_linears


def test_report_lists_quantized_excluded_and_incompatible():
    from offload_adam_amd.qweight import Int4QWeight, QuantizeReport, quantize_linears

    model = fresh(TwoLinears)
    report = quantize_linears(model, Int4QWeight, group_size=128, skip_patterns=("l2",))
    assert isinstance(report, QuantizeReport)
    assert (report.quantized, report.excluded, report.incompatible) == (["l1"], ["l2"], [])
    assert isinstance(model.l1.weight.data, Int4QWeight)
    assert not isinstance(model.l2.weight.data, Int4QWeight)


def test_strict_refuses_a_layer_the_layout_cannot_hold():
    from offload_adam_amd.qweight import Int4QWeight, quantize_linears

    layer = nn.Linear(100, 128, bias=False).to(device="cuda", dtype=BF16)  # 100 % 128 != 0
    with pytest.raises(ValueError, match="strict=True"):
        quantize_linears(layer, Int4QWeight, group_size=128, strict=True)
    report = quantize_linears(layer, Int4QWeight, group_size=128)
    assert report.quantized == [] and len(report.incompatible) == 1


def test_a_bare_linear_keeps_its_parameter_name():
    layer = nn.Linear(FEATURES, FEATURES, bias=False).to(device="cuda", dtype=BF16)
    quantize(layer)
    assert "weight" in dict(layer.named_parameters())


# ------------------------------------------------------------------ master seeding


def test_adam_seeds_the_master_of_a_quantised_weight_from_its_dequantisation():
    from offload_adam_amd import Adam

    model = fresh(quantized=True)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    state = opt.state[model.l1.weight]
    opt._init_state_if_empty(model.l1.weight, state)
    assert state["master_filled"] is False
    assert state["master_params"].dtype == torch.float32
    assert torch.equal(state["master_params"], model.l1.weight.data.dequantize().float())


def test_adam_seeds_the_master_of_a_plain_weight_losslessly():
    from offload_adam_amd import Adam

    model = fresh()
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    state = opt.state[model.l1.weight]
    opt._init_state_if_empty(model.l1.weight, state)
    assert torch.equal(state["master_params"], model.l1.weight.data.float())
    assert "master_filled" not in state


def test_offload_adam_allocates_an_unfilled_fp32_master():
    from offload_adam_amd import OffloadAdam

    model = fresh(quantized=True)
    opt = OffloadAdam(model, mode="fp32_master", lr=1e-3)
    state = opt.state[model.l1.weight]
    assert state["master_filled"] is False
    assert state["master_params"].dtype == torch.float32 and state["master_params"].is_pinned()
    assert torch.equal(state["master_params"], model.l1.weight.data.dequantize().float().cpu())


# ------------------------------------------------------------------------- warning


def test_lossy_master_warning_fires_on_the_first_real_step_only():
    from offload_adam_amd import Adam

    model = fresh(quantized=True)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    assert lossy_master_warnings(opt.step) == 0  # no gradient yet: nothing stepped, nothing said
    one_backward(model)
    assert lossy_master_warnings(opt.step) == 1
    model.zero_grad(set_to_none=True)
    one_backward(model)
    assert lossy_master_warnings(opt.step) == 0


def test_plain_weights_never_warn():
    from offload_adam_amd import Adam

    model = fresh()
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    one_backward(model)
    assert lossy_master_warnings(opt.step) == 0


# ------------------------------------------------------ load_master_from_pretrained


def test_refill_from_a_single_file(tmp_path):
    from offload_adam_amd import Adam

    model = fresh()
    original = model.l1.weight.data.float().clone()
    path = tmp_path / "model.safetensors"
    write_checkpoint(model, path)
    quantize(model)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    assert opt.load_master_from_pretrained(path, model) == []
    state = opt.state[model.l1.weight]
    assert state["master_filled"] is True
    assert torch.equal(state["master_params"], original)
    one_backward(model)
    assert lossy_master_warnings(opt.step) == 0  # the master is lossless now


def test_refill_leaves_plain_parameters_alone(tmp_path):
    from offload_adam_amd import Adam

    model = fresh(LinearAndNorm)
    path = tmp_path / "model.safetensors"
    write_checkpoint(model, path)
    norm_weight = model.ln.weight.data.float().clone()
    quantize(model)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    assert opt.load_master_from_pretrained(path, model) == []
    assert opt.state[model.l1.weight]["master_filled"] is True
    state = opt.state[model.ln.weight]
    opt._init_state_if_empty(model.ln.weight, state)  # created lazily, from the parameter itself
    assert torch.equal(state["master_params"], norm_weight)
    assert "master_filled" not in state


def test_missing_names_are_returned_or_raised(tmp_path):
    from offload_adam_amd import Adam

    model = fresh(TwoLinears)
    path = tmp_path / "model.safetensors"
    write_checkpoint(model, path, only={"l1.weight"})
    quantize(model)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    with pytest.raises(ValueError, match="strict=True"):
        opt.load_master_from_pretrained(path, model, strict=True)
    assert opt.load_master_from_pretrained(path, model) == ["l2.weight"]


def test_refill_from_a_sharded_directory(tmp_path):
    from safetensors.torch import save_file

    from offload_adam_amd import Adam

    model = fresh(TwoLinears)
    originals = {n: p.data.float().clone() for n, p in model.named_parameters()}
    shards = {"l1.weight": "model-00001-of-00002.safetensors",
              "l2.weight": "model-00002-of-00002.safetensors"}
    for name, filename in shards.items():
        save_file({name: dict(model.named_parameters())[name].detach().cpu().contiguous()},
                  str(tmp_path / filename))
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"metadata": {"total_size": 0}, "weight_map": shards}))
    quantize(model)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    assert opt.load_master_from_pretrained(tmp_path, model, strict=True) == []
    for name, p in model.named_parameters():
        assert torch.equal(opt.state[p]["master_params"], originals[name]), name


def test_offload_adam_refills_its_pinned_master(tmp_path):
    from offload_adam_amd import OffloadAdam

    model = fresh()
    original = model.l1.weight.data.float().cpu()
    path = tmp_path / "model.safetensors"
    write_checkpoint(model, path)
    quantize(model)
    opt = OffloadAdam(model, mode="fp32_master", lr=1e-3)
    assert opt.load_master_from_pretrained(path, model, strict=True) == []
    state = opt.state[model.l1.weight]
    assert state["master_filled"] is True and state["master_params"].is_pinned()
    assert torch.equal(state["master_params"].cpu(), original)


# ---------------------------------------------------------- load_master_state_dict


def test_load_master_state_dict_reports_names_it_cannot_place():
    from offload_adam_amd import Adam

    model = fresh(quantized=True)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    with pytest.raises(ValueError, match="strict=True"):
        opt.load_master_state_dict({"l1.weigth": torch.zeros(FEATURES, FEATURES)}, model,
                                   strict=True)
    (unexpected,) = opt.load_master_state_dict(
        {"l1.weight": torch.zeros(FEATURES, FEATURES), "ghost.weight": torch.zeros(4)}, model)
    assert unexpected == ["ghost.weight"]
    assert opt.state[model.l1.weight]["master_params"].abs().sum() == 0


# -------------------------------------------------------------------------- resume


def test_adam_state_dict_round_trip_keeps_fp32_master_and_flag(tmp_path):
    from offload_adam_amd import Adam

    path = tmp_path / "model.safetensors"
    write_checkpoint(fresh(), path)
    model = fresh(quantized=True)
    opt = Adam(model.parameters(), mode="fp32_master", lr=1e-3)
    opt.load_master_from_pretrained(path, model, strict=True)
    one_backward(model)
    opt.step()
    master = opt.state[model.l1.weight]["master_params"].clone()
    saved = opt.state_dict()

    model2 = fresh(quantized=True)
    opt2 = Adam(model2.parameters(), mode="fp32_master", lr=1e-3)
    opt2.load_state_dict(saved)
    state = opt2.state[model2.l1.weight]
    assert state["master_filled"] is True
    assert state["master_params"].dtype == torch.float32
    assert torch.equal(state["master_params"], master)
    one_backward(model2)
    assert lossy_master_warnings(opt2.step) == 0


def test_offload_adam_load_state_dict_is_refused():
    from offload_adam_amd import OffloadAdam

    model = fresh(quantized=True)
    opt = OffloadAdam(model, mode="fp32_master", lr=1e-3)
    with pytest.raises(NotImplementedError, match="not supported"):
        opt.load_state_dict(opt.state_dict())
