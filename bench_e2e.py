#!/usr/bin/env python3
"""End-to-end synthetic training step with OffloadAdam on one MI355X
(benchmark config 4) and the host-link measurements that go with it.

    python bench_e2e.py [--model llama8b|llama1b|tiny] [--steps K] [--warmup W]
                        [--grad-accum 4] [--seq 4096] [--mode stochastic_rounding]

Model: a Llama-style decoder written here in plain PyTorch (RMSNorm, rotary
embeddings, grouped-query SDPA attention, SwiGLU MLP, untied embeddings), bf16,
random init, per-layer activation checkpointing.  Data: uniform random token
ids.  The loop has the shape of the reference's example
(examples/e2e_train/train.py:183-213): for each micro-batch set
``optimizer.ready_for_optimizer_step``, forward, backward; then
``optimizer.step()``.

Reported: step time, tokens/s, the same loop with no optimizer (pure
forward/backward) to expose the optimizer's non-overlapped cost, bytes moved
over the host link per step and the achieved H2D / D2H rates against the pinned
``hipMemcpyAsync`` peak measured in the same run.  Prints ONE JSON line.
"""

import argparse
import json
import os
import math
import sys
import time
import warnings
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

MODELS = {
    # benchmark config 4 / config 2 shapes
    "llama8b": dict(hidden=4096, inter=14336, layers=32, q_heads=32, kv_heads=8, head_dim=128,
                    vocab=128256),
    # benchmark config 1 shapes
    "llama1b": dict(hidden=2048, inter=5632, layers=22, q_heads=32, kv_heads=4, head_dim=64,
                    vocab=32000),
    "tiny": dict(hidden=256, inter=688, layers=2, q_heads=4, kv_heads=2, head_dim=64, vocab=1024),
}


def build_model(cfg, device):
    import torch
    import torch.nn as nn
    import torch.nn.functional as F
    from torch.utils.checkpoint import checkpoint

    class RMSNorm(nn.Module):
        def __init__(self, dim, eps=1e-5):
            super().__init__()
            self.weight = nn.Parameter(torch.ones(dim))
            self.eps = eps

        def forward(self, x):
            v = x.float()
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
            return (v * self.weight.float()).to(x.dtype)

    def rotary(x, cos, sin):
        x1, x2 = x[..., ::2], x[..., 1::2]
        return torch.stack((x1 * cos - x2 * sin, x1 * sin + x2 * cos), dim=-1).flatten(-2)

    class Block(nn.Module):
        def __init__(self, c):
            super().__init__()
            h, hd = c["hidden"], c["head_dim"]
            self.nq, self.nkv, self.hd = c["q_heads"], c["kv_heads"], hd
            self.input_layernorm = RMSNorm(h)
            self.q_proj = nn.Linear(h, self.nq * hd, bias=False)
            self.k_proj = nn.Linear(h, self.nkv * hd, bias=False)
            self.v_proj = nn.Linear(h, self.nkv * hd, bias=False)
            self.o_proj = nn.Linear(self.nq * hd, h, bias=False)
            self.post_attention_layernorm = RMSNorm(h)
            self.gate_proj = nn.Linear(h, c["inter"], bias=False)
            self.up_proj = nn.Linear(h, c["inter"], bias=False)
            self.down_proj = nn.Linear(c["inter"], h, bias=False)

        def forward(self, x, cos, sin):
            b, s, _ = x.shape
            y = self.input_layernorm(x)
            q = self.q_proj(y).view(b, s, self.nq, self.hd).transpose(1, 2)
            k = self.k_proj(y).view(b, s, self.nkv, self.hd).transpose(1, 2)
            v = self.v_proj(y).view(b, s, self.nkv, self.hd).transpose(1, 2)
            q, k = rotary(q, cos, sin), rotary(k, cos, sin)
            rep = self.nq // self.nkv
            if rep > 1:
                k = k.repeat_interleave(rep, dim=1)
                v = v.repeat_interleave(rep, dim=1)
            a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
            x = x + self.o_proj(a.transpose(1, 2).reshape(b, s, self.nq * self.hd))
            y = self.post_attention_layernorm(x)
            return x + self.down_proj(F.silu(self.gate_proj(y)) * self.up_proj(y))

    class Decoder(nn.Module):
        def __init__(self, c):
            super().__init__()
            self.c = c
            self.embed_tokens = nn.Embedding(c["vocab"], c["hidden"])
            self.layers = nn.ModuleList([Block(c) for _ in range(c["layers"])])
            self.norm = RMSNorm(c["hidden"])
            self.lm_head = nn.Linear(c["hidden"], c["vocab"], bias=False)

        def forward(self, ids):
            s = ids.shape[1]
            hd = self.c["head_dim"]
            inv = 1.0 / (500000.0 ** (torch.arange(0, hd, 2, device=ids.device).float() / hd))
            ang = torch.arange(s, device=ids.device).float()[:, None] * inv[None, :]
            cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
            x = self.embed_tokens(ids)
            for layer in self.layers:
                x = checkpoint(layer, x, cos, sin, use_reentrant=False)
            x = self.norm(x)
            # cross-entropy in sequence chunks: the fp32 logits of 4096 x 128256 stay bounded
            loss = x.new_zeros((), dtype=torch.float32)
            chunk = 1024
            tgt = torch.roll(ids, -1, dims=1)
            for i in range(0, s, chunk):
                logits = self.lm_head(x[:, i:i + chunk]).float()
                loss = loss + F.cross_entropy(logits.reshape(-1, logits.shape[-1]),
                                              tgt[:, i:i + chunk].reshape(-1), reduction="sum")
            return loss / ids.numel()

    with torch.device(device):
        model = Decoder(cfg).to(torch.bfloat16)
    g = torch.Generator(device=device).manual_seed(0)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() > 1:
                p.normal_(0.0, 0.02, generator=g)
    return model


def measure_link(nbytes=1 << 30, reps=5):
    """Pinned hipMemcpyAsync rates of this box: H2D alone, D2H alone, both at once."""
    import torch

    from offload_adam_amd import _lib
    from offload_adam_amd.offload_adam import _copy_async
    from offload_adam_amd.pinned_alloc import zeros_pinned

    host_a = zeros_pinned((nbytes,), torch.uint8)
    host_b = zeros_pinned((nbytes,), torch.uint8)
    dev_a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dev_b = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()

    def run(h2d, d2h):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            if h2d:
                _copy_async(dev_a, host_a, _lib.OA_COPY_H2D, s1)
            if d2h:
                _copy_async(host_b, dev_b, _lib.OA_COPY_D2H, s2)
        s1.synchronize()
        s2.synchronize()
        return nbytes * reps / (time.perf_counter() - t0) / 1e9

    def run_mixed(wg):
        """H2D on the DMA engine while the copy kernel writes back (the pairing
        the optimizer uses)."""
        from offload_adam_amd.offload_adam import _copy_by_kernel

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            _copy_async(dev_a, host_a, _lib.OA_COPY_H2D, s1)
            _copy_by_kernel(host_b, dev_b, s2, wg)
        s1.synchronize()
        s2.synchronize()
        return nbytes * reps / (time.perf_counter() - t0) / 1e9

    run(True, True)  # warm-up

    def best(*what):
        # The best of up to five, with pauses: a process started right after one
        # that held tens of GiB of pinned memory measures D2H at 30 GB/s instead
        # of 57 for its first seconds (the driver is still releasing those pages).
        rates = []
        for _ in range(5):
            rates.append(run(*what))
            if rates[-1] > 45.0:
                break
            time.sleep(1.0)
        return round(max(rates), 2)

    return {
        "h2d_GBps": best(True, False),
        "d2h_GBps": best(False, True),
        "bidir_each_GBps": best(True, True),
        "dma_h2d_plus_kernel_d2h_each_GBps": {wg: round(run_mixed(wg), 2) for wg in (4, 8, 16)},
    }


def link_bytes_per_step(opt, grad_accum):
    """Bytes the hook path moves per optimizer step for the offloaded parameters."""
    import torch

    n = sum(p.numel() for p in opt._offload_params)
    state_b = sum(torch.empty(0, dtype=d).element_size()
                  for k, d in opt.offload_config.items() if k != "grad")
    # states and gradients kept on the GPU after their write-back are not fetched again
    states_in = state_b * sum(p.numel() for p in opt._offload_params
                              if p not in opt._state_cached)
    # gradients that cross the link at all (not with offload_grads=False, nor those the
    # pinned-memory limit keeps in HBM)
    streamed = [p for p in opt._offload_params if p not in opt._grad_on_device]
    if not streamed:
        return states_in, n * state_b
    fetched = sum(p.numel() for p in streamed if p not in opt._grad_cached)
    # partial sums written to the host: all of them, or (write-back gradient cache)
    # only those that do not stay on the GPU
    written = fetched if opt._grad_cache_write_back else sum(p.numel() for p in streamed)
    passes = grad_accum - 1 if opt._step_in_backward else grad_accum
    h2d = states_in + fetched * 2 * passes
    d2h = n * state_b + written * 2 * passes
    return h2d, d2h


class CopyTimeline:
    """Times every copy the optimizer issues with a pair of events on the copy's own
    stream (the profiler cannot be used for this: under rocprofv3 the copy-engine
    tools library is not loaded).  ``summary()`` covers the copies of the last
    ``steps`` optimizer steps."""

    def __init__(self, torch, oa_mod):
        self.torch, self.oa_mod, self.log = torch, oa_mod, []
        self._orig = oa_mod._copy_async
        oa_mod._copy_async = self._timed_copy
        # every copy its own library call, so that each can be bracketed by events (a
        # stream round trip per copy: about 5 % slower than the batched default; under
        # rocprofv3 --memory-copy-trace the default path itself is visible)
        self._batched = oa_mod._BATCH_COPIES
        oa_mod._BATCH_COPIES = False

    def _timed_copy(self, dst, src, kind, stream):
        e0 = self.torch.cuda.Event(enable_timing=True)
        e1 = self.torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        self._orig(dst, src, kind, stream)
        e1.record(stream)
        self.log.append((kind, src.numel() * src.element_size(), e0, e1))

    def mark(self):
        self.first = len(self.log)

    def close(self):
        self.oa_mod._copy_async = self._orig
        self.oa_mod._BATCH_COPIES = self._batched

    @staticmethod
    def _union(iv):
        out = []
        for s, e in sorted(iv):
            if out and s <= out[-1][1]:
                out[-1][1] = max(out[-1][1], e)
            else:
                out.append([s, e])
        return out

    def summary(self, steps):
        rows = self.log[self.first:]
        if not rows:
            return None
        base = rows[0][2]
        iv = {0: [], 1: []}
        big = {0: [], 1: []}
        for kind, nbytes, e0, e1 in rows:
            s, e = base.elapsed_time(e0), base.elapsed_time(e1)
            iv[kind].append((s, e))
            if nbytes >= 100e6 and e > s:
                big[kind].append(nbytes / (e - s) / 1e6)
        uh, ud = self._union(iv[0]), self._union(iv[1])
        both, i, j = 0.0, 0, 0
        while i < len(uh) and j < len(ud):
            lo, hi = max(uh[i][0], ud[j][0]), min(uh[i][1], ud[j][1])
            both += max(0.0, hi - lo)
            if uh[i][1] < ud[j][1]:
                i += 1
            else:
                j += 1
        med = lambda v: round(sorted(v)[len(v) // 2], 1) if v else None  # noqa: E731
        return {
            "copies_per_step": len(rows) // steps,
            "h2d_busy_s_per_step": round(sum(e - s for s, e in uh) / 1e3 / steps, 3),
            "d2h_busy_s_per_step": round(sum(e - s for s, e in ud) / 1e3 / steps, 3),
            "both_busy_s_per_step": round(both / 1e3 / steps, 3),
            "h2d_GBps_median_large_copy": med(big[0]),
            "d2h_GBps_median_large_copy": med(big[1]),
            "h2d_GBps_min_large_copy": round(min(big[0]), 1) if big[0] else None,
            "d2h_GBps_min_large_copy": round(min(big[1]), 1) if big[1] else None,
        }


class StepCheck:
    """Numerical check of one optimizer step of the 8B-style run (``--check``).

    A sample of parameters (the first of every distinct shape) is followed
    through one extra step after the timed ones: hooks registered BEFORE the
    optimizer's capture each micro-batch's gradient, parameters and moments are
    copied before the step, and afterwards plain fp32 torch ops on the GPU must
    reproduce what the optimizer left behind - both moments bit for bit
    (bf16_rne(m + (1-b1)(g-m)), bf16_rne(v + (1-b2)(g*g-v)) with g the bf16 sum
    of the micro-batch gradients), every parameter on one of the two bf16
    neighbours of the fp32 result (taken within 1 fp32 ulp: torch's sqrt and
    divide are not promised correctly rounded), and the number of round-ups equal
    to the sum of the round-up probabilities within 6 standard deviations.

    With ``fp31_master`` (benchmark config 2 as a training step, with or without
    the clipping path) the gradient is first scaled as ``grad.mul_(clip_coef)``
    would, the moments are again exact, and the master the optimizer left behind
    - the parameter's bf16 bits plus twice its int16 rounding error - must be the
    31-bit rounding of the fp32 result (same 1-ulp allowance), with the parameter
    its bf16 rounding.  Every sampled per-parameter norm must lie within one bf16
    ulp of the fp64 norm of the summed gradient, the total within one of the
    norm of all the slots, and the coefficient must equal the reference's bf16
    expression ``clamp(max_norm / (total + 1e-6), max=1.0)`` bit for bit.

    With ``fp32_master`` (the mode comparison of the reference's example, and every
    ``--qat`` run) the moments are exact again, the fp32 master the optimizer left
    behind must be the fp32 result of the update (same 1-ulp allowance), a plain
    bf16 parameter must be the bf16 rounding of its master, and a quantised
    parameter's payload must be, bit for bit, what the library's stand-alone encoder
    (``copy_(master)`` into a clone) makes of that master, with its decoded value
    within one quantisation step of the master."""

    # decoded value against master, as a fraction of the largest magnitude of the
    # element's row / group / block: the format's largest code error (int8 half of
    # 1/127; int4 one step of 1/8, its largest value is clamped to code 7; NF4 half of
    # the codebook's widest gap, 0.152; NVFP4 half of the 4..6 gap under an e4m3 scale
    # that may be 1/16 off) plus 2^-8 each for a bf16 scale and the bf16 output
    QAT_STEP_BOUND = {"Int8QWeight": 0.0125, "Int4QWeight": 0.134, "NF4QWeight": 0.157,
                      "NVFP4QWeight": 0.19}

    def __init__(self, torch, model):
        self.torch, self.armed, self.grads, self.sample = torch, False, {}, {}
        seen = set()
        for name, p in model.named_parameters():
            if tuple(p.shape) not in seen:
                seen.add(tuple(p.shape))
                self.sample[p] = name
                p.register_post_accumulate_grad_hook(self._capture)

    def _capture(self, p):
        if self.armed and p.grad is not None:
            self.grads.setdefault(p, []).append(p.grad.detach().clone())

    def before(self, opt):
        torch = self.torch
        torch.cuda.synchronize()
        self.old = {p: (p.detach().clone(), opt.state[p]["exp_avg"].to(p.device, copy=True),
                        opt.state[p]["exp_avg_sq"].to(p.device, copy=True))
                    for p in self.sample}
        self.old_err = {p: opt.state[p]["rounding_error"].to(p.device, copy=True)
                        for p in self.sample if "rounding_error" in opt.state[p]}
        self.old_master = {p: opt.state[p]["master_params"].to(p.device, copy=True)
                           for p in self.sample if "master_params" in opt.state[p]}
        self.grads.clear()
        self.armed = True

    @staticmethod
    def _bf16_neighbours(torch, got_bf16, exact_f64):
        """True where the bf16 value is the exact one rounded down or up."""
        near = exact_f64.to(torch.float32).to(torch.bfloat16)
        bits = near.view(torch.int16).to(torch.int32)
        got = got_bf16.view(torch.int16).to(torch.int32)
        return (got - bits).abs() <= 1

    def _check_clipping(self, opt, totals, report):
        """Norm slots, total norm and coefficient of the clipping path."""
        torch = self.torch
        ok = True
        for p, name in self.sample.items():
            exact = totals[p].double().square().sum().sqrt()
            if not bool(self._bf16_neighbours(torch, opt.state[p]["grad_norm"].reshape(1),
                                              exact.reshape(1)).all()):
                ok = False
                report["failed"].append(name + ": gradient norm")
        exact_total = opt._norm_slots.double().square().sum().sqrt()
        if not bool(self._bf16_neighbours(torch, opt._total_norm.reshape(1),
                                          exact_total.reshape(1)).all()):
            ok = False
            report["failed"].append("total norm")
        want = torch.clamp(float(opt.max_grad_norm) / (opt._total_norm + 1e-6), max=1.0)
        if not torch.equal(want.view(torch.int16), opt._clip_coef.view(torch.int16)):
            ok = False
            report["failed"].append("clip coefficient")
        report["norms_within_1_bf16_ulp_and_coef_exact"] = ok
        report["total_norm"] = float(opt._total_norm)
        report["clip_coef"] = float(opt._clip_coef)
        return ok

    def after(self, opt, decoupled):
        import numpy as np

        if not decoupled:
            raise SystemExit("--check covers decoupled weight decay only")
        torch = self.torch
        self.armed = False
        torch.cuda.synchronize()
        if opt.mode == "fp31_master":
            return self._after_fp31(opt)
        if opt.mode == "fp32_master":
            return self._after_fp32_master(opt)
        f32 = np.float32
        group = opt.param_groups[0]
        lr, eps, wd = float(f32(group["lr"])), float(f32(group["eps"])), group["weight_decay"]
        lr_wd = float(f32(group["lr"]) * f32(wd))
        beta1, beta2 = group["betas"]
        report = {"tensors": len(self.sample), "elements": 0, "moments_exact": True,
                  "params_on_bf16_neighbours": True, "failed": []}
        ups = expected = variance = 0.0
        for p, name in self.sample.items():
            step = opt.state[p]["step"]
            b1h = (beta1**step - beta1) / (beta1**step - 1)
            b2h = (beta2**step - beta2) / (beta2**step - 1)
            omb1, omb2 = float(f32(1) - f32(b1h)), float(f32(1) - f32(b2h))
            p0, m0, v0 = (t.float() for t in self.old.pop(p))
            total = self.grads[p][0]
            for g in self.grads[p][1:]:
                total.add_(g)  # bf16 += bf16, as the optimizer accumulates
            g = total.float()
            m = m0 + omb1 * (g - m0)
            v = v0 + omb2 * (g * g - v0)
            m_now = opt.state[p]["exp_avg"].to(p.device)
            v_now = opt.state[p]["exp_avg_sq"].to(p.device)
            if not (torch.equal(m_now, m.to(torch.bfloat16))
                    and torch.equal(v_now, v.to(torch.bfloat16))):
                report["moments_exact"] = False
                report["failed"].append(name + ": moments")
            M = p0 - lr_wd * p0
            M = M - (lr * m) / (torch.sqrt(v) + eps)
            mb = M.view(torch.int32)
            pb = p.detach().view(torch.int16).to(torch.int32) << 16

            def on_grid(b):
                t = b & -0x10000
                return (pb == t) | (pb == t + 0x10000)

            ok = on_grid(mb) | on_grid(mb + 1) | on_grid(mb - 1)
            if not bool(ok.all()):
                report["params_on_bf16_neighbours"] = False
                report["failed"].append(f"{name}: {int((~ok).sum())} params off the grid")
            frac = (mb & 0xFFFF).double() / 65536.0
            ups += float((pb != (mb & -0x10000)).double().sum())
            expected += float(frac.sum())
            variance += float((frac * (1 - frac)).sum())
            report["elements"] += p.numel()
            del p0, m0, v0, g, m, v, M, mb, pb, ok, frac
        self.grads.clear()
        report["round_ups"] = int(ups)
        report["expected_round_ups"] = round(expected, 1)
        report["round_up_sigma"] = round(variance ** 0.5, 1)
        # the fp32 result is known within one ulp per element, i.e. each round-up
        # probability within 2^-16: that much systematic offset is allowed on top
        report["unbiased_within_6_sigma"] = (abs(ups - expected)
                                             < 6.0 * variance ** 0.5 + report["elements"] / 65536.0)
        report["passed"] = (report["moments_exact"] and report["params_on_bf16_neighbours"]
                            and report["unbiased_within_6_sigma"])
        return report

    def _after_fp32_master(self, opt):
        import numpy as np

        from offload_adam_amd.qweight.base import QWeightBase

        torch = self.torch
        f32 = np.float32
        group = opt.param_groups[0]
        lr, eps, wd = float(f32(group["lr"])), float(f32(group["eps"])), group["weight_decay"]
        lr_wd = float(f32(group["lr"]) * f32(wd))
        beta1, beta2 = group["betas"]
        report = {"tensors": len(self.sample), "quantised_tensors": 0, "elements": 0,
                  "moments_exact": True, "master_is_the_fp32_result": True,
                  "param_is_bf16_of_the_master": True,
                  "payload_is_the_encoding_of_the_master": True,
                  "decoded_payload_within_one_step": True, "failed": []}
        for p, name in self.sample.items():
            step = opt.state[p]["step"]
            b1h = (beta1**step - beta1) / (beta1**step - 1)
            b2h = (beta2**step - beta2) / (beta2**step - 1)
            omb1, omb2 = float(f32(1) - f32(b1h)), float(f32(1) - f32(b2h))
            _, m0, v0 = self.old.pop(p)
            m0, v0 = m0.float(), v0.float()
            total = self.grads[p][0]
            for g in self.grads[p][1:]:
                total.add_(g)  # bf16 += bf16, as the optimizer accumulates
            g = total.float()
            m = m0 + omb1 * (g - m0)
            v = v0 + omb2 * (g * g - v0)
            m_now = opt.state[p]["exp_avg"].to(p.device)
            v_now = opt.state[p]["exp_avg_sq"].to(p.device)
            if not (torch.equal(m_now, m.to(torch.bfloat16))
                    and torch.equal(v_now, v.to(torch.bfloat16))):
                report["moments_exact"] = False
                report["failed"].append(name + ": moments")
            M0 = self.old_master.pop(p)
            M = M0 - lr_wd * M0
            M = M - (lr * m) / (torch.sqrt(v) + eps)
            master = opt.state[p]["master_params"].to(p.device)
            off = (master.view(torch.int32) - M.view(torch.int32)).abs() > 1
            if bool((off & (master != M)).any()):
                report["master_is_the_fp32_result"] = False
                report["failed"].append(f"{name}: {int(off.sum())} masters off")
            if isinstance(p.data, QWeightBase):
                report["quantised_tensors"] += 1
                q = p.data
                again = q.detach().clone()
                again.copy_(master)  # the stand-alone encoder on the master the step left
                for key in q._PAYLOAD:
                    a, b = getattr(q, key), getattr(again, key)
                    if not torch.equal(a.reshape(-1).view(torch.uint8),
                                       b.reshape(-1).view(torch.uint8)):
                        report["payload_is_the_encoding_of_the_master"] = False
                        report["failed"].append(f"{name}: payload {key}")
                span = {"Int8QWeight": master.shape[1], "Int4QWeight": getattr(q, "group_size", 0),
                        "NF4QWeight": getattr(q, "blocksize", 0), "NVFP4QWeight": 16}[type(q).__name__]
                grouped = master.reshape(master.shape[0], -1, span)
                err = (q.dequantize().float().reshape(grouped.shape) - grouped).abs()
                bound = grouped.abs().amax(dim=-1, keepdim=True) * self.QAT_STEP_BOUND[type(q).__name__]
                if bool((err > bound + 1e-30).any()):
                    report["decoded_payload_within_one_step"] = False
                    report["failed"].append(f"{name}: decoded payload off by more than a step")
                del again, grouped, err, bound
            elif not torch.equal(master.to(torch.bfloat16).view(torch.int16),
                                 p.detach().view(torch.int16)):
                report["param_is_bf16_of_the_master"] = False
                report["failed"].append(name + ": param is not the bf16 rounding of its master")
            report["elements"] += p.numel()
            del m0, v0, g, m, v, M0, M, master, off
        self.grads.clear()
        report["passed"] = not report["failed"]
        return report

    def _after_fp31(self, opt):
        import numpy as np

        torch = self.torch
        f32 = np.float32
        group = opt.param_groups[0]
        lr, eps, wd = float(f32(group["lr"])), float(f32(group["eps"])), group["weight_decay"]
        lr_wd = float(f32(group["lr"]) * f32(wd))
        beta1, beta2 = group["betas"]
        report = {"tensors": len(self.sample), "elements": 0, "moments_exact": True,
                  "master_is_fp31_of_the_fp32_result": True, "param_is_bf16_of_the_master": True,
                  "failed": []}
        totals = {}
        for p in self.sample:
            total = self.grads[p][0]
            for g in self.grads[p][1:]:
                total.add_(g)  # bf16 += bf16, as the optimizer accumulates
            totals[p] = total
        clipped_ok = True
        coef = None
        if opt.max_grad_norm is not None:
            clipped_ok = self._check_clipping(opt, totals, report)
            coef = opt._clip_coef.float()

        def round31(bits):
            up = bits & (bits >> 1) & 1
            return ((bits >> 1) + up) << 1

        for p, name in self.sample.items():
            step = opt.state[p]["step"]
            b1h = (beta1**step - beta1) / (beta1**step - 1)
            b2h = (beta2**step - beta2) / (beta2**step - 1)
            omb1, omb2 = float(f32(1) - f32(b1h)), float(f32(1) - f32(b2h))
            p0, m0, v0 = self.old.pop(p)
            err0 = self.old_err.pop(p).to(torch.int32)
            g = totals.pop(p).float()
            if coef is not None:
                g = (g * coef).to(torch.bfloat16).float()  # grad.mul_(clip_coef) in bf16
            m0, v0 = m0.float(), v0.float()
            m = m0 + omb1 * (g - m0)
            v = v0 + omb2 * (g * g - v0)
            m_now = opt.state[p]["exp_avg"].to(p.device)
            v_now = opt.state[p]["exp_avg_sq"].to(p.device)
            if not (torch.equal(m_now, m.to(torch.bfloat16))
                    and torch.equal(v_now, v.to(torch.bfloat16))):
                report["moments_exact"] = False
                report["failed"].append(name + ": moments")
            M0 = ((p0.view(torch.int16).to(torch.int32) << 16) + (err0 << 1)).view(torch.float32)
            M = M0 - lr_wd * M0
            M = M - (lr * m) / (torch.sqrt(v) + eps)
            mb = M.view(torch.int32)
            err_now = opt.state[p]["rounding_error"].to(p.device).to(torch.int32)
            pb = p.detach().view(torch.int16).to(torch.int32) << 16
            master_now = pb + (err_now << 1)
            ok = ((master_now == round31(mb)) | (master_now == round31(mb + 1))
                  | (master_now == round31(mb - 1)))
            if not bool(ok.all()) or int(err_now.abs().max()) > 16384:
                report["master_is_fp31_of_the_fp32_result"] = False
                report["failed"].append(f"{name}: {int((~ok).sum())} masters off")
            if not torch.equal(master_now.view(torch.float32).to(torch.bfloat16).view(torch.int16),
                               p.detach().view(torch.int16)):
                report["param_is_bf16_of_the_master"] = False
                report["failed"].append(name + ": param is not the bf16 rounding of its master")
            report["elements"] += p.numel()
            del p0, m0, v0, err0, g, m, v, M0, M, mb, err_now, pb, master_now, ok
        self.grads.clear()
        report["passed"] = (report["moments_exact"] and report["master_is_fp31_of_the_fp32_result"]
                            and report["param_is_bf16_of_the_master"] and clipped_ok)
        return report


def run(args):
    import torch

    from offload_adam_amd import OffloadAdam, _copy_engines, _lib  # before any CUDA call

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = MODELS[args.model]
    out = {"model": args.model, "mode": args.mode, "seq": args.seq, "batch": 1,
           "grad_accum": args.grad_accum, "max_grad_norm": args.max_grad_norm,
           "offload_grads": not args.grads_on_device}

    out["link_peak"] = measure_link()

    model = build_model(cfg, dev)
    if args.qat:
        from offload_adam_amd import qweight

        cls = {"int8": qweight.Int8QWeight, "int4": qweight.Int4QWeight,
               "nf4": qweight.NF4QWeight, "nvfp4": qweight.NVFP4QWeight}[args.qat]
        report = qweight.quantize_linears(model, cls, skip_patterns=("lm_head",))
        out["qat"] = {"format": args.qat, "quantized_linears": len(report.quantized),
                      "incompatible": len(report.incompatible),
                      "cache_dequantized": args.cache_dequantized}
        qweight.cache_dequantized_weights(args.cache_dequantized)
        torch.cuda.empty_cache()
        out["model_gpu_GiB"] = round(torch.cuda.memory_allocated() / 1024**3, 2)
    n_params = sum(p.numel() for p in model.parameters())
    out["params"] = n_params
    ids = [torch.randint(0, cfg["vocab"], (1, args.seq), device=dev,
                         generator=torch.Generator(device=dev).manual_seed(i))
           for i in range(args.grad_accum)]

    check = None
    if args.check:
        if not ((args.mode == "stochastic_rounding" and args.max_grad_norm is None)
                or args.mode == "fp31_master"
                or (args.mode == "fp32_master" and args.max_grad_norm is None)):
            raise SystemExit("--check covers the stochastic-rounding hook path (config 4), "
                             "fp31_master with or without clipping (config 2) and the "
                             "fp32_master hook path with plain or quantised (--qat) weights")
        check = StepCheck(torch, model)  # its hooks must precede the optimizer's

    compute_done = {}

    def loop(opt, steps):
        torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record()
        t0 = time.perf_counter()
        for _ in range(steps):
            for mb in range(args.grad_accum):
                if opt is not None:
                    opt.ready_for_optimizer_step = mb == args.grad_accum - 1
                loss = model(ids[mb])
                loss.backward()
                if opt is None:
                    model.zero_grad(set_to_none=True)
            if opt is not None:
                opt.step()
                opt.zero_grad()
        last.record()  # compute stream: the write-backs still under way are on another
        torch.cuda.synchronize()
        elapsed = (time.perf_counter() - t0) / steps
        compute_done["s"] = first.elapsed_time(last) / 1e3 / steps
        return elapsed

    # 1) forward/backward only: what a step costs with a free optimizer
    loop(None, 1)
    torch.cuda.reset_peak_memory_stats()
    out["fwd_bwd_only_s"] = round(loop(None, args.steps), 4)
    out["fwd_bwd_only_peak_GiB"] = round(torch.cuda.max_memory_allocated() / 1024**3, 2)
    out["fwd_bwd_only_reserved_GiB"] = round(torch.cuda.max_memory_reserved() / 1024**3, 2)

    if args.optimizer == "adam":
        return run_resident_adam(args, out, model, loop, torch)

    # 2) the offloaded optimizer
    t0 = time.perf_counter()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = OffloadAdam(model, lr=1e-5, mode=args.mode, max_grad_norm=args.max_grad_norm,
                          inplace_param_threshold=1024 * 1024, prefetch_policy="eager",
                          decoupled_weight_decay=True, offload_grads=not args.grads_on_device,
                          prefetch_bytes=int(args.prefetch_gib * 2**30) if args.prefetch_gib else None,
                          grad_cache_bytes=(None if args.grad_cache_gib is None
                                            else int(args.grad_cache_gib * 2**30)),
                          state_cache_bytes=(None if args.state_cache_gib is None
                                             else int(args.state_cache_gib * 2**30)),
                          grad_cache_policy=args.grad_cache_policy, spare_hbm=args.spare_hbm)
    torch.cuda.synchronize()
    out["optimizer_init_s"] = round(time.perf_counter() - t0, 2)
    out["offloaded_params"] = len(opt._offload_params)
    out["inplace_params"] = len(opt._inplace_params)
    out["prefetch_GiB"] = round(opt._PREFETCH_BYTES / 1024**3, 2)
    out["grad_cache_GiB"] = round(sum(p.numel() for p in opt._grad_cached) * 2 / 1024**3, 2)
    out["grad_cache_policy"] = "write_back" if opt._grad_cache_write_back else "write_through"
    out["spare_hbm"] = bool(args.spare_hbm)
    out["state_cache_GiB"] = round(
        sum(p.numel() for p in opt._state_cached) * (opt._bytes_per_elem_in_flight - 2) / 1024**3, 2)
    out["pinned_GiB"] = round(opt._estimate_pinned_bytes(opt._offload_params) / 1024**3, 2)
    if opt.pinned_limit_report:
        out["pinned_limit"] = {k: (round(v / 1024**3, 2) if k.endswith("_bytes") else v)
                               for k, v in opt.pinned_limit_report.items()}

    timeline = None
    if args.copy_timeline:
        from offload_adam_amd import offload_adam as oa_mod

        timeline = CopyTimeline(torch, oa_mod)
    model.zero_grad(set_to_none=True)
    torch.cuda.empty_cache()  # so that the reserved figure below is this phase's own
    torch.cuda.reset_peak_memory_stats()
    loop(opt, args.warmup)
    if timeline:
        timeline.mark()
    step_s = loop(opt, args.steps)
    if timeline:
        timeline.close()
        out["copy_timeline"] = timeline.summary(args.steps)
    out["step_s"] = round(step_s, 4)
    # the same steps up to the last kernel, i.e. without the write-back that trails the last
    # step (a training run pays that once, this measurement once per `steps`)
    out["step_s_to_last_kernel"] = round(compute_done["s"], 4)
    out["tokens_per_s"] = round(args.grad_accum * args.seq / step_s, 1)
    out["exposed_optimizer_s"] = round(step_s - out["fwd_bwd_only_s"], 4)
    out["peak_gpu_GiB"] = round(torch.cuda.max_memory_allocated() / 1024**3, 2)
    # what the caching allocator holds from the driver: includes blocks that were freed
    # but wait for a copy on another stream (record_stream) before they can be reused
    out["peak_reserved_GiB"] = round(torch.cuda.max_memory_reserved() / 1024**3, 2)
    stats = torch.cuda.memory_stats()
    out["allocator"] = {"device_allocs": stats.get("num_device_alloc"),
                        "device_frees": stats.get("num_device_free"),
                        "alloc_retries": stats.get("num_alloc_retries")}
    h2d, d2h = link_bytes_per_step(opt, args.grad_accum)
    out["h2d_GB_per_step"] = round(h2d / 1e9, 2)
    out["d2h_GB_per_step"] = round(d2h / 1e9, 2)
    out["h2d_GBps_over_step"] = round(h2d / step_s / 1e9, 2)
    out["d2h_GBps_over_step"] = round(d2h / step_s / 1e9, 2)
    # no schedule can beat: each direction at its solo rate, both together at twice
    # the rate each reaches while the other is busy
    peaks = out["link_peak"]
    out["link_floor_s"] = round(max(h2d / 1e9 / peaks["h2d_GBps"], d2h / 1e9 / peaks["d2h_GBps"],
                                    (h2d + d2h) / 1e9 / (2 * peaks["bidir_each_GBps"])), 4)
    out["transfer_streams"] = opt.transfer_stream_report
    st = _copy_engines.status()
    from offload_adam_amd import offload_adam as _oa_mod

    out["link_copies"] = "direct" if _oa_mod._fixed_engine_copies() else "runtime"
    out["copy_engines"] = {k: st.get(k) for k in (
        "direct", "direct_reason", "direct_h2d_engine", "direct_d2h_engine", "direct_h2d_copies",
        "direct_d2h_copies", "direct_runtime_copies", "loaded", "active", "h2d_copies",
        "d2h_copies", "rejected")}
    if check is not None:
        check.before(opt)
        loop(opt, 1)
        out["check"] = check.after(opt, decoupled=True)
    out["loss_finite"] = bool(math.isfinite(float(model(ids[0]))))
    return out


def run_resident_adam(args, out, model, loop, torch):
    """Same loop with ``Adam``: gradients accumulate in ``p.grad``, states stay in HBM."""
    from offload_adam_amd import Adam

    class Stepper:
        def __init__(self, opt):
            self.opt, self.ready_for_optimizer_step = opt, False

        def step(self):
            self.opt.step()

        def zero_grad(self):
            self.opt.zero_grad(set_to_none=True)

    opt = Stepper(Adam(model.parameters(), lr=1e-5, mode=args.mode, decoupled_weight_decay=True))
    torch.cuda.reset_peak_memory_stats()
    loop(opt, args.warmup)
    step_s = loop(opt, args.steps)
    out.update(optimizer="adam", step_s=round(step_s, 4),
               tokens_per_s=round(args.grad_accum * args.seq / step_s, 1),
               exposed_optimizer_s=round(step_s - out["fwd_bwd_only_s"], 4),
               peak_gpu_GiB=round(torch.cuda.max_memory_allocated() / 1024**3, 2))
    return out


def copy_trace_summary(directory, window_s=None):
    """Per-direction figures of a ``rocprofv3 --memory-copy-trace --output-format csv``
    run of this program: copies, busy time (union of the copies' intervals), the sum
    of their durations (equal to the union when one engine serves the direction) and
    the time both directions were busy at once - over the last ``window_s`` seconds of
    the trace (the timed steps: steps x step_s of the run's own output), or all of it.
    The trace carries time stamps per copy and no byte counts; bytes per step are in
    this program's output (``h2d_GB_per_step``)."""
    import csv
    import glob

    files = glob.glob(os.path.join(directory, "**", "*memory_copy_trace.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no *memory_copy_trace.csv under {directory}")
    per = {}
    with open(files[0]) as fh:
        for row in csv.DictReader(fh):
            per.setdefault(row["Direction"], []).append(
                (int(row["Start_Timestamp"]), int(row["End_Timestamp"])))
    end = max(e for v in per.values() for _, e in v)
    start = end - int(window_s * 1e9) if window_s else min(s for v in per.values() for s, _ in v)

    def merged(intervals):
        out = []
        for s, e in sorted(intervals):
            if out and s <= out[-1][1]:
                out[-1][1] = max(out[-1][1], e)
            else:
                out.append([s, e])
        return out

    report, unions = {"window_s": round((end - start) / 1e9, 4)}, {}
    for name, intervals in sorted(per.items()):
        inside = [(s, e) for s, e in intervals if s >= start]
        unions[name] = merged(inside)
        report[name] = {"copies": len(inside),
                        "busy_s": round(sum(e - s for s, e in unions[name]) / 1e9, 4),
                        "sum_of_durations_s": round(sum(e - s for s, e in inside) / 1e9, 4)}
    up = [v for k, v in unions.items() if "HOST_TO_DEVICE" in k]
    down = [v for k, v in unions.items() if "DEVICE_TO_HOST" in k]
    if up and down:
        a, b, i, j, both = up[0], down[0], 0, 0, 0
        while i < len(a) and j < len(b):
            both += max(0, min(a[i][1], b[j][1]) - max(a[i][0], b[j][0]))
            if a[i][1] < b[j][1]:
                i += 1
            else:
                j += 1
        report["both_directions_busy_s"] = round(both / 1e9, 4)
    return report


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--copy-trace-summary", metavar="DIR", default=None,
                    help="no run: summarise the *memory_copy_trace.csv that rocprofv3 "
                         "--memory-copy-trace wrote under DIR (see --trace-window-s)")
    ap.add_argument("--trace-window-s", type=float, default=None,
                    help="with --copy-trace-summary: only the last so many seconds of the trace")
    ap.add_argument("--model", default="llama8b", choices=sorted(MODELS))
    ap.add_argument("--mode", default="stochastic_rounding")
    ap.add_argument("--seq", type=int, default=4096)
    ap.add_argument("--grad-accum", type=int, default=4)
    ap.add_argument("--max-grad-norm", type=float, default=None)
    ap.add_argument("--steps", type=int, default=2)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--d2h-workgroups", type=int, default=None,
                    help="workgroups of the write-back copy kernel (default: the optimizer's)")
    ap.add_argument("--writeback-pending-gib", type=float, default=None,
                    help="bytes of freed staging buffers that write-backs may still be reading "
                         "before the host waits (default: the optimizer's, = its staging window)")
    ap.add_argument("--prefetch-gib", type=float, default=None,
                    help="device staging budget of the H2D prefetch window")
    ap.add_argument("--optimizer", default="offload", choices=["offload", "adam"],
                    help="'adam': the GPU-resident Adam of this package (states in HBM, "
                         "multi-tensor launches in step()) instead of OffloadAdam")
    ap.add_argument("--qat", default=None, choices=["int8", "int4", "nf4", "nvfp4"],
                    help="quantise every decoder Linear weight (lm_head excluded) and train "
                         "against fp32 masters: implies --mode fp32_master")
    ap.add_argument("--grad-cache-gib", type=float, default=None,
                    help="OffloadAdam(grad_cache_bytes=...): HBM for gradients kept on the GPU "
                         "after their write-back (default: the optimizer's; 0 = fetch every time "
                         "like the reference)")
    ap.add_argument("--state-cache-gib", type=float, default=None,
                    help="OffloadAdam(state_cache_bytes=...): HBM for optimizer states kept on the "
                         "GPU after their write-back (default: the optimizer's; 0 = none, like "
                         "the reference)")
    ap.add_argument("--cache-dequantized", action="store_true",
                    help="with --qat: qweight.cache_dequantized_weights(True), one decode per "
                         "weight per step instead of one per forward / re-computation / backward")
    ap.add_argument("--grad-cache-policy", default=None,
                    choices=["write_back", "write_through"],
                    help="OffloadAdam(grad_cache_policy=...): 'write_through' (the default "
                         "without --spare-hbm) sends every partial gradient sum to the host "
                         "after its micro-batch, like the reference")
    ap.add_argument("--spare-hbm", action="store_true",
                    help="OffloadAdam(spare_hbm=True): budgets not given become a tenth of the "
                         "free HBM each and gradients are written back lazily; without it the "
                         "run has the reference's traffic (80.3 GB each way at 8B, ga=4)")
    ap.add_argument("--check", action="store_true",
                    help="after the timed steps, follow one more step numerically on a sample "
                         "of parameters (see StepCheck); the result is in 'check'")
    ap.add_argument("--grads-on-device", action="store_true",
                    help="OffloadAdam(offload_grads=False): the gradient sum stays in HBM")
    ap.add_argument("--copy-timeline", action="store_true",
                    help="time every optimizer copy with events on its stream and report link "
                         "occupancy per direction (adds two event records per copy)")
    ap.add_argument("--runtime-copy-engines", action="store_true",
                    help="leave the SDMA engine of each copy to the HIP runtime "
                         "(OFFLOAD_ADAM_COPY_ENGINES=off: neither the library's fixed-engine "
                         "copies nor the tools library)")
    ap.add_argument("--link-copies", default=None, choices=["direct", "runtime"],
                    help="'direct': the kernel library issues the copies on its fixed engines "
                         "(oa_link_copy_batch); 'runtime': hipMemcpyAsync, engine rewritten by "
                         "the HSA tools library when it is loaded.  Default: 'runtime' when the "
                         "tools library is in effect, else 'direct'")
    args = ap.parse_args()
    if args.copy_trace_summary:
        print(json.dumps(copy_trace_summary(args.copy_trace_summary, args.trace_window_s)))
        return
    if args.qat:
        args.mode = "fp32_master"
    if args.runtime_copy_engines:
        import os

        os.environ["OFFLOAD_ADAM_COPY_ENGINES"] = "off"  # before the package is imported
    if args.link_copies:
        import os

        os.environ["OFFLOAD_ADAM_LINK_COPIES"] = args.link_copies
    if args.d2h_workgroups:
        from offload_adam_amd import offload_adam as _oa_mod

        _oa_mod._D2H_BY_KERNEL = True
        _oa_mod._D2H_WORKGROUPS = args.d2h_workgroups
    if args.writeback_pending_gib is not None:
        from offload_adam_amd import OffloadAdam as _OffloadAdam

        _OffloadAdam._WRITEBACK_PENDING_BYTES = int(args.writeback_pending_gib * 2**30)
    print(json.dumps(run(args)))


if __name__ == "__main__":
    main()
