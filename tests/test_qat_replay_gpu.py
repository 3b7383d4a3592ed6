"""Quantisation-aware training through the optimizer classes, replayed by the oracle.

``OffloadAdam`` (hook path, four micro-batches per step, a threshold that splits
the parameters into streamed and GPU-resident ones) and ``Adam`` train the
Llama-shaped tiny decoder of ``bench_e2e.py`` whose ``nn.Linear`` weights were
swapped for int8 / int4 / NF4 / NVFP4 weights (``quantize_linears``; layers whose
width the format cannot group stay plain bf16, so both kinds of parameter are in
every run).  The per-step contract of a quantised parameter in the reference
(src/offload_adam/offload_adam.py:421-444, src/offload_adam/adam.py:131-151):
``fp32_master`` step on the master, then ``p.data.copy_(master)`` re-encodes the
payload.  Here every micro-batch's gradient is captured before the optimizer's
hook, the bf16 accumulation is redone on the CPU, ``oracle.adam_fp32_master``
advances a CPU master and ``oracle.quant_*`` encodes it: moments, masters and
every payload tensor must be bit-equal after each of three steps.  The seed of
the master (``master.copy_(p.data)``: decode to bf16, widen) is checked against
``oracle.dequant_*`` before the first step.
"""

import sys
import warnings
from pathlib import Path

import numpy as np
import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[1]))

pytestmark = pytest.mark.gpu

HYP = dict(lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
GA, STEPS, SEQ = 4, 3, 48
THRESHOLD = 100_000
FORMATS = ["int8", "int4", "nf4", "nvfp4"]


def u16(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1).copy()


def widen(bf16_bits):
    return (bf16_bits.astype(np.uint32) << 16).view(np.float32)


def quantised_tiny_decoder(fmt):
    import bench_e2e
    from offload_adam_amd import qweight

    model = bench_e2e.build_model(bench_e2e.MODELS["tiny"], torch.device("cuda:0"))
    cls = {"int8": qweight.Int8QWeight, "int4": qweight.Int4QWeight, "nf4": qweight.NF4QWeight,
           "nvfp4": qweight.NVFP4QWeight}[fmt]
    report = qweight.quantize_linears(model, cls, skip_patterns=("lm_head",))
    assert report.quantized, "nothing was quantised"
    return model, cls


def payload_bits(qw):
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


def bf16_scale_bits(scale_f32):
    return torch.from_numpy(np.ascontiguousarray(scale_f32)).to(torch.bfloat16) \
        .view(torch.int16).numpy()


class Codec:
    """The oracle's encoder / decoder of one format, on this package's payload names."""

    def __init__(self, oracle, fmt):
        self.o, self.fmt = oracle, fmt

    def encode(self, master_2d):
        o = self.o
        if self.fmt == "int8":
            q, s = o.quant_int8(master_2d)
            return {"weight": q, "scales": bf16_scale_bits(s)}
        if self.fmt == "int4":
            qw, s = o.quant_int4(master_2d, group=128)
            return {"qweight": qw, "scales": bf16_scale_bits(s)}
        if self.fmt == "nf4":
            pk, am = o.quant_nf4(master_2d, block=64)
            return {"weight_packed": pk, "absmax": am.view(np.int32)}
        pk, s8, gs = o.quant_nvfp4(master_2d)
        return {"weight_packed": pk, "block_scale_fp8": s8,
                "global_scale": np.asarray(gs, dtype=np.float32).view(np.int32)}

    def decode_bf16(self, payload, shape):
        """bf16 bits of ``dequantize()`` in the weight's own dtype."""
        o = self.o
        if self.fmt == "int8":
            out = o.dequant_int8(payload["weight"].reshape(shape),
                                 widen(payload["scales"].view(np.uint16).reshape(-1)))
        elif self.fmt == "int4":
            out = o.dequant_int4(payload["qweight"], widen(
                payload["scales"].view(np.uint16).reshape(-1)).reshape(payload["scales"].shape),
                group=128)
        elif self.fmt == "nf4":
            out = o.dequant_nf4(payload["weight_packed"], payload["absmax"].view(np.float32),
                                block=64)
        else:
            out = o.dequant_nvfp4(payload["weight_packed"], payload["block_scale_fp8"],
                                  payload["global_scale"].view(np.float32).reshape(-1)[0])
        return out.reshape(-1)


class QatReplica:
    """CPU copy of every parameter's fp32 master, moments and (for quantised ones)
    payload, advanced by the oracle."""

    def __init__(self, oracle, model, codec):
        from offload_adam_amd.qweight.base import QWeightBase

        self.oracle, self.codec = oracle, codec
        self.names = [n for n, _ in model.named_parameters()]
        self.shape = {n: tuple(p.shape) for n, p in model.named_parameters()}
        self.quant = {n for n, p in model.named_parameters() if isinstance(p.data, QWeightBase)}
        self.payload, self.p, self.master = {}, {}, {}
        for n, p in model.named_parameters():
            if n in self.quant:
                self.payload[n] = payload_bits(p.data)
                # master.copy_(p.data): decoded to bf16, then widened
                self.master[n] = widen(codec.decode_bf16(self.payload[n], self.shape[n])).copy()
            else:
                self.p[n] = u16(p)
                self.master[n] = widen(self.p[n]).copy()
        self.m = {n: np.zeros(self.master[n].size, dtype=np.uint16) for n in self.names}
        self.v = {n: np.zeros(self.master[n].size, dtype=np.uint16) for n in self.names}
        self.step = 0

    @staticmethod
    def total_gradient(per_mb):
        total = per_mb[0].clone()
        for g in per_mb[1:]:
            total.add_(g)  # bf16 += bf16: fp32 sum, one rounding, as on the GPU
        return u16(total)

    def advance(self, grads):
        self.step += 1
        b1h, b2h = self.oracle.folded_betas(*HYP["betas"], self.step)
        for n in self.names:
            g = self.total_gradient(grads[n])
            sink = np.zeros_like(g)
            self.oracle.adam_fp32_master(sink, g, self.m[n], self.v[n], self.master[n], HYP["lr"],
                                         HYP["weight_decay"], b1h, b2h, HYP["eps"], True)
            if n in self.quant:
                self.payload[n] = self.codec.encode(self.master[n].reshape(self.shape[n]))
            else:
                self.p[n] = sink

    def assert_equal(self, model, state_of, step):
        for n, p in model.named_parameters():
            st = state_of(p)
            ctx = f"step {step}: {n}"
            if step:
                assert np.array_equal(u16(st["exp_avg"]), self.m[n]), ctx + " exp_avg"
                assert np.array_equal(u16(st["exp_avg_sq"]), self.v[n]), ctx + " exp_avg_sq"
            got = st["master_params"].detach().cpu().numpy().reshape(-1)
            assert np.array_equal(got.view(np.uint32), self.master[n].view(np.uint32)), \
                ctx + " master"
            if n in self.quant:
                have = payload_bits(p.data)
                for key, want in self.payload[n].items():
                    assert np.array_equal(have[key].reshape(-1).view(want.dtype),
                                          want.reshape(-1)), f"{ctx} payload {key}"
            else:
                assert np.array_equal(u16(p), self.p[n]), ctx + " param"


def token_batches(vocab):
    g = torch.Generator().manual_seed(5)
    return [torch.randint(0, vocab, (2, SEQ), generator=g).cuda() for _ in range(GA * STEPS)]


@pytest.mark.parametrize("fmt", FORMATS)
def test_offload_adam_qat_equals_the_oracle(oracle, fmt):
    from offload_adam_amd import OffloadAdam

    model, _ = quantised_tiny_decoder(fmt)
    replica = QatReplica(oracle, model, Codec(oracle, fmt))
    assert replica.quant and len(replica.quant) < len(replica.names)
    grads = {}
    names = {p: n for n, p in model.named_parameters()}

    def capture(p):  # registered before the optimizer's hooks: sees p.grad first
        grads.setdefault(names[p], []).append(p.grad.detach().to("cpu", copy=True))

    for p in model.parameters():
        p.register_post_accumulate_grad_hook(capture)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, mode="fp32_master", inplace_param_threshold=THRESHOLD,
                          decoupled_weight_decay=True, prefetch_bytes=1 << 20, **HYP)
        assert opt._offload_params and opt._inplace_params, "the threshold must split the set"
        offloaded = {id(p) for p in opt._offload_params}  # (no == for quantised weights)
        assert opt._quant_params and all(id(p) in offloaded for p in opt._quant_params)
        torch.cuda.synchronize()
        replica.assert_equal(model, lambda p: opt.state[p], 0)  # the seeded masters
        data = token_batches(model.c["vocab"])
        for s in range(STEPS):
            grads.clear()
            for mb in range(GA):
                opt.ready_for_optimizer_step = mb == GA - 1
                model(data[s * GA + mb]).backward()
            opt.step()
            opt.zero_grad()
            torch.cuda.synchronize()
            assert all(len(g) == GA for g in grads.values()) and len(grads) == len(names)
            replica.advance(grads)
            replica.assert_equal(model, lambda p: opt.state[p], s + 1)
    for p in opt._quant_params:
        assert opt.state[p]["master_params"].is_pinned() and not opt.state[p]["master_params"].is_cuda


@pytest.mark.parametrize("fmt", FORMATS)
def test_resident_adam_qat_equals_the_oracle(oracle, fmt):
    from offload_adam_amd import Adam

    model, _ = quantised_tiny_decoder(fmt)
    replica = QatReplica(oracle, model, Codec(oracle, fmt))
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = Adam(model.parameters(), mode="fp32_master", decoupled_weight_decay=True, **HYP)
        data = token_batches(model.c["vocab"])
        for s in range(STEPS):
            per_mb = {n: [] for n in replica.names}
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
            replica.advance(per_mb)
            replica.assert_equal(model, lambda p: opt.state[p], s + 1)


@pytest.mark.parametrize("fmt", FORMATS + [None])
def test_the_benchmarks_fp32_master_check_passes_and_can_fail(fmt):
    """``bench_e2e.py --check`` in ``fp32_master`` mode (what vouches for the QAT and
    mode-comparison rows of the bench line) on the tiny decoder, with quantised and
    with plain weights: it passes on an honest step, and fails when a payload byte, a
    master or a moment is off."""
    import bench_e2e
    from offload_adam_amd import OffloadAdam
    from offload_adam_amd.qweight.base import QWeightBase

    outcomes = {}
    for tamper in (None, "payload", "master", "moment"):
        if tamper == "payload" and fmt is None:
            continue
        torch.manual_seed(0)
        if fmt is None:
            model = bench_e2e.build_model(bench_e2e.MODELS["tiny"], torch.device("cuda:0"))
        else:
            model, _ = quantised_tiny_decoder(fmt)
        check = bench_e2e.StepCheck(torch, model)  # its hooks precede the optimizer's
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            opt = OffloadAdam(model, mode="fp32_master", lr=1e-3, weight_decay=0.1,
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
        quant = [p for p in check.sample if isinstance(p.data, QWeightBase)]
        assert bool(quant) == (fmt is not None)
        if tamper == "payload":
            t = getattr(quant[0].data, quant[0].data._PAYLOAD[0])
            t.view(torch.uint8).reshape(-1)[5] ^= 1
        elif tamper == "master":
            p = quant[0] if quant else next(iter(check.sample))
            opt.state[p]["master_params"].view(torch.int32).reshape(-1)[3] += 4
        elif tamper == "moment":
            p = next(iter(check.sample))
            opt.state[p]["exp_avg"].view(torch.int16).reshape(-1)[7] ^= 1
        outcomes[tamper] = check.after(opt, decoupled=True)
    honest = outcomes[None]
    assert honest["passed"] and honest["failed"] == [], honest
    assert honest["elements"] > 400_000
    assert (honest["quantised_tensors"] > 0) == (fmt is not None)
    if fmt is not None:
        assert not outcomes["payload"]["passed"]
        assert not outcomes["payload"]["payload_is_the_encoding_of_the_master"]
    assert not outcomes["master"]["passed"] and not outcomes["master"]["master_is_the_fp32_result"]
    assert not outcomes["moment"]["passed"] and not outcomes["moment"]["moments_exact"]
