#!/usr/bin/env python3
"""Benchmark of the optimizer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A "step" is one pass of the fused AdamW kernel over every tensor of the
workload, with all operands already resident in HBM.  The default workload is
benchmark config 1: stochastic_rounding mode over the Llama-style 1.1B
parameter set (201 tensors, 1,100,048,384 elements, 14 algorithmic bytes per
element).  Prints ONE JSON line.

After the timed region of the default workload the same line also carries

* ``cpu_baseline``: benchmark config 0 exactly (fp32_master, 16,777,216
  elements) in PyTorch eager on this host's cores;
* ``other_configs``: config 0, the two kernel legs of config 2 (gradient norms,
  fp31_master with the clip coefficient folded in, Llama-3-8B shapes) and the
  codec kernels of config 3, each with its own ``roofline`` from HIP events and
  a small ``cpu_baseline``;
* ``offloaded_step_8b``: config 4 as a training step through ``OffloadAdam``
  (child processes running bench_e2e.py): at the reference's traffic, with the
  HBM caches, the same model with the GPU-resident ``Adam``, and config 2 as a
  training step (fp31_master with the clipping path);
* ``offloaded_step_1b``: config 1 as a training step (the 1.1B set streamed, one
  micro-batch per step);
* ``mode_comparison_8b`` and ``qat_step``: the reference's rounding-mode and QAT
  tables as training steps through ``OffloadAdam``, each with a numerical check;
* ``summary`` (the LAST key): roofline fraction per config and, per streamed step,
  time, exposed optimizer time, link use, peak HBM and the check's verdict.

``--only-main`` stops after the timed region.  Only one GPU is used;
``--gpus N`` with N > 1 exits with a message.
"""

import argparse
import gc
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE and
# WRITE_SIZE counter runs of this script, each scaled by what the same counter
# read for a 1 GiB device copy (factors 2.000 and 1.000).  Counters cannot be
# read from inside the run, so the figure is carried over from that profile and
# the line says so (``traffic_source``).  Keyed by (workload, launch form).
TRAFFIC_FROM_PROFILE = {
    ("c1_sr_llama1b", "multi_tensor"): (
        2_566_900_000, "profiles/adam_multi_kernel_sr_c1_llama1b_hbm_traffic.txt"),
}

BYTES_PER_ELEM = {
    "stochastic_rounding": 14,
    "fp32_master": 20,
    "fp31_master": 18,
    "fp32_master_custom_rounding": 18,
}
HYP = dict(lr=1e-4, wd=0.01, beta1=0.9, beta2=0.999, eps=1e-8)  # config 0's, step 10 on the CPU


def llama_shapes(hidden, inter, layers, q_heads, kv_heads, head_dim, vocab):
    """Parameter shapes of an untied Llama-style decoder, in module order."""
    shapes = [("embed_tokens", (vocab, hidden))]
    for i in range(layers):
        shapes += [
            (f"l{i}.input_norm", (hidden,)),
            (f"l{i}.q_proj", (q_heads * head_dim, hidden)),
            (f"l{i}.k_proj", (kv_heads * head_dim, hidden)),
            (f"l{i}.v_proj", (kv_heads * head_dim, hidden)),
            (f"l{i}.o_proj", (hidden, q_heads * head_dim)),
            (f"l{i}.post_norm", (hidden,)),
            (f"l{i}.gate_proj", (inter, hidden)),
            (f"l{i}.up_proj", (inter, hidden)),
            (f"l{i}.down_proj", (hidden, inter)),
        ]
    shapes += [("final_norm", (hidden,)), ("lm_head", (vocab, hidden))]
    return shapes


WORKLOADS = {
    # benchmark config 1
    "c1_sr_llama1b": dict(
        mode="stochastic_rounding",
        shapes=llama_shapes(2048, 5632, 22, 32, 4, 64, 32000),
        clip=False,
    ),
    # benchmark config 0 (one flat tensor)
    "c0_fp32_master_16m": dict(mode="fp32_master", shapes=[("flat", (16_777_216,))], clip=False),
    # benchmark config 2 kernel leg: fp31_master + fused clip on Llama-3-8B shapes
    "c2_fp31_clip_llama8b": dict(
        mode="fp31_master",
        shapes=llama_shapes(4096, 14336, 32, 32, 8, 128, 128256),
        clip=True,
    ),
}


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


def make_tensors(mode, shapes, device, seed=0):
    import torch

    g = torch.Generator(device=device).manual_seed(seed)
    out = []
    for _, shape in shapes:
        n = numel(shape)
        p = (torch.randn(n, device=device, generator=g) * 0.02).to(torch.bfloat16)
        st = {
            "grad": (torch.randn(n, device=device, generator=g) * 1e-3).to(torch.bfloat16),
            "exp_avg": (torch.randn(n, device=device, generator=g) * 1e-4).to(torch.bfloat16),
            "exp_avg_sq": ((torch.randn(n, device=device, generator=g) * 1e-3) ** 2).to(
                torch.bfloat16
            ),
        }
        if mode == "fp32_master":
            st["master_params"] = p.float()
        elif mode in ("fp31_master", "fp32_master_custom_rounding"):
            st["rounding_error"] = torch.zeros(n, dtype=torch.int16, device=device)
        out.append((p, st))
    return out


# ------------------------------------------------------------------ CPU side


def host_description():
    """What the CPU figures ran on: core counts as the OS, the scheduler and
    torch see them, CPU model, NUMA nodes."""
    import torch

    model = None
    try:
        with open("/proc/cpuinfo") as fh:
            for ln in fh:
                if ln.startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        nodes = len([d for d in os.listdir("/sys/devices/system/node") if d[4:].isdigit()
                     and d.startswith("node")])
    except OSError:
        nodes = None
    try:
        affinity = len(os.sched_getaffinity(0))
    except AttributeError:
        affinity = None
    return {"os_cpu_count": os.cpu_count(), "sched_affinity": affinity,
            "omp_num_threads_env": os.environ.get("OMP_NUM_THREADS"),
            "torch_num_threads": torch.get_num_threads(), "cpu_model": model,
            "numa_nodes": nodes}


def cpu_adam_inputs(mode, n, seed=0):
    import torch

    g = torch.Generator().manual_seed(seed)
    p = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16)
    st = {
        "grad": (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16),
        "exp_avg": (torch.randn(n, generator=g) * 1e-4).to(torch.bfloat16),
        "exp_avg_sq": ((torch.randn(n, generator=g) * 1e-3) ** 2).to(torch.bfloat16),
    }
    if mode == "fp32_master":
        st["master_params"] = p.float()
    elif mode in ("fp31_master", "fp32_master_custom_rounding"):
        st["rounding_error"] = torch.zeros(n, dtype=torch.int16)
    return p, st


def cpu_baseline(mode="fp32_master", n=16_777_216, budget_s=12.0, min_iters=5, clip=False):
    """The same update math in PyTorch eager (the oracle's torch restatement, fp32
    compute, one rounding per op) on this host's cores.  Default = benchmark
    config 0 exactly: fp32_master, one flat tensor of 16,777,216 elements, lr 1e-4,
    betas (0.9, 0.999), eps 1e-8, weight decay 0.01 decoupled, step 10.  Two
    warm-up passes, then timed passes until ``budget_s`` is spent (at least
    ``min_iters``); median and minimum reported.  Random bits of the
    stochastic-rounding variant are drawn before the timed passes."""
    import torch

    from oracle import folded_betas, torch_eager

    p, st = cpu_adam_inputs(mode, n)
    b1h, b2h = folded_betas(HYP["beta1"], HYP["beta2"], 10)
    args = (HYP["lr"], HYP["wd"], b1h, b2h, HYP["eps"], True)
    coef = torch.tensor(0.3359375, dtype=torch.bfloat16) if clip else None
    if mode == "stochastic_rounding":
        bits = torch.randint(0, 65536, (n,), dtype=torch.int32,
                             generator=torch.Generator().manual_seed(1))

        def run():
            torch_eager.adam_step_stochastic_rounding(p, st, *args, bits)
    elif mode == "fp32_master":
        def run():
            torch_eager.adam_step_fp32_master(p, st, *args)
    else:
        fn = (torch_eager.adam_step_fp31_master if mode == "fp31_master"
              else torch_eager.adam_step_custom_rounding)

        def run():
            fn(p, st, *args, clip_coef=coef)
    run()
    run()
    times, spent = [], 0.0
    while len(times) < min_iters or (spent < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
        spent += times[-1]
    med = sorted(times)[len(times) // 2]
    alg = n * BYTES_PER_ELEM[mode]
    return {
        "value": round(alg / med / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{mode}{' + clip' if clip else ''}, one flat tensor of {n} elements, torch eager "
                  f"fp32 on the host CPU, {len(times)} timed passes after 2 warm-up: median "
                  f"{med * 1e3:.1f} ms, min {min(times) * 1e3:.1f} ms",
        "median_ms": round(med * 1e3, 2),
        "min_ms": round(min(times) * 1e3, 2),
        "best_GBps": round(alg / min(times) / 1e9, 3),
        "passes": len(times),
    }


def cpu_baselines_of_the_other_kernels(rows=512, cols=14336):
    """The C restatement (one thread) of every kernel besides the AdamW update,
    on a bounded sample: ``rows`` x ``cols`` of the codec workload's weight and as
    many elements of gradient.  GB/s of the same algorithmic bytes the GPU figures
    use (bf16 source and output)."""
    import numpy as np

    import oracle

    rng = np.random.default_rng(0)
    x = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    x[rng.random((rows, cols)) < 0.01] *= 10
    # the values a bf16 weight holds
    x = (oracle.narrow_array(x, "bfloat16").astype(np.uint32) << 16).view(np.float32)
    x = np.ascontiguousarray(x.reshape(rows, cols))
    n = rows * cols
    g_bits = oracle.narrow_array((rng.standard_normal(n) * 5e-3).astype(np.float32), "bfloat16")
    out = {}

    def timed(name, alg_bytes, fn):
        fn()
        t0 = time.perf_counter()
        res = fn()
        dt = time.perf_counter() - t0
        out[name] = round(alg_bytes / dt / 1e9, 3)
        return res

    timed("grad_norm", 2 * n, lambda: oracle.grad_norm_bf16(g_bits))
    q8 = timed("quant_int8", 3 * n, lambda: oracle.quant_int8(x))
    timed("dequant_int8", 3 * n, lambda: oracle.dequant_int8(*q8))
    q4 = timed("quant_int4", n * (2 + 0.5 + 2 / 128), lambda: oracle.quant_int4(x, 128))
    timed("dequant_int4", n * (2 + 0.5 + 2 / 128), lambda: oracle.dequant_int4(*q4, 128))
    qn = timed("quant_nf4", n * (2 + 0.5 + 4 / 64), lambda: oracle.quant_nf4(x, 64))
    timed("dequant_nf4", n * (2 + 0.5 + 4 / 64), lambda: oracle.dequant_nf4(*qn, 64))
    qf = timed("quant_nvfp4", n * (4 + 0.5 + 1 / 16), lambda: oracle.quant_nvfp4(x))
    timed("dequant_nvfp4", n * (2 + 0.5 + 1 / 16), lambda: oracle.dequant_nvfp4(*qf))
    return {"unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{rows} x {cols} elements per kernel, C restatement, one pass timed",
            "value": out}


# ------------------------------------------------------------------ GPU side


def time_adam_workload(name, steps, warmup, *, rng=None, per_tensor=False, use_events=True,
                       sets=1):
    """``steps`` timed passes of the fused AdamW kernel over every tensor of
    workload ``name`` between two device synchronisations, after ``warmup``
    passes.  ``sets`` > 1 rotates through that many copies of the operands (one
    per pass), so a workload smaller than the 256 MiB memory-side cache is read
    from HBM.  Returns the figures of the bench line."""
    import torch

    from offload_adam_amd import kernels
    from offload_adam_amd.kernels import adam_step_multi
    from offload_adam_amd.kernels.multi import MULTI_MAX

    dev = torch.device("cuda:0")
    wl = WORKLOADS[name]
    mode = wl["mode"]
    operand_sets = [make_tensors(mode, wl["shapes"], dev, seed=s) for s in range(sets)]
    tensors = operand_sets[0]
    step_fn = getattr(kernels, "adam_step_" + mode)
    clip = torch.tensor(0.3359375, dtype=torch.bfloat16, device=dev) if wl["clip"] else None
    total_elems = sum(p.numel() for p, _ in tensors)
    bytes_per_step = total_elems * BYTES_PER_ELEM[mode]
    kw, multi_kw = {}, {}
    if mode == "stochastic_rounding" and rng is not None:
        kw["rng"] = rng
        kw["seed"] = 1
        multi_kw["rng"] = rng
        multi_kw["seeds"] = list(range(1, len(tensors) + 1))

    multi = not per_tensor
    lists = [([p for p, _ in ts], [st for _, st in ts]) for ts in operand_sets]
    launches_per_step = -(-len(tensors) // MULTI_MAX) if multi else len(tensors)

    def one_step(step_no, events=None):
        """One pass of the fused AdamW kernel over every tensor of the workload."""
        which = step_no % sets
        if multi:
            p_list, st_list = lists[which]
            if events is not None:
                events[0][0].record()
            adam_step_multi(mode, p_list, st_list, HYP["lr"], HYP["wd"], HYP["beta1"],
                            HYP["beta2"], HYP["eps"], step_no, decoupled_weight_decay=True,
                            clip_coef=clip, validate=False, **multi_kw)
            if events is not None:
                events[0][1].record()
            return
        for i, (p, st) in enumerate(operand_sets[which]):
            if events is not None:
                events[i][0].record()
            step_fn(p, st, HYP["lr"], HYP["wd"], HYP["beta1"], HYP["beta2"], HYP["eps"], step_no,
                    decoupled_weight_decay=True, clip_coef=clip, **kw)
            if events is not None:
                events[i][1].record()

    for w in range(warmup):
        one_step(w + 1)
    torch.cuda.synchronize()

    # Timed region: exactly ``steps`` steps, bracketed by device synchronisation.
    # Events are recorded on the stream the kernels run on (torch's current
    # stream) and read back after the closing synchronisation.
    # The collector is off inside it, as in timeit: a full collection of this process's
    # heap takes about 80 ms, and one that falls between a start event and its launch
    # turns a 20 ms measurement of 50 us launches into a quarter of its rate.  (Switched
    # off only, not run first: collecting here would leave the GPU idle for those 80 ms
    # between warm-up and measurement, and the clock-sensitive kernels then start slow.)
    pairs_per_step = 1 if multi else len(tensors)
    all_events = []
    gc.disable()
    try:
        t0 = time.perf_counter()
        for s in range(steps):
            ev = None
            if use_events:
                ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                      for _ in range(pairs_per_step)]
                all_events.append(ev)
            one_step(warmup + s + 1, ev)
        enqueue = time.perf_counter() - t0
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    finally:
        gc.enable()
    kernel_ms = sum(a.elapsed_time(b) for ev in all_events for a, b in ev)
    launches = launches_per_step * len(all_events)

    roofline = None
    if use_events and launches:
        avg_launch_s = kernel_ms / launches / 1e3
        alg_bytes_per_launch = bytes_per_step / launches_per_step
        achieved = alg_bytes_per_launch / avg_launch_s / 1e9
        traffic, source = TRAFFIC_FROM_PROFILE.get(
            (name, "multi_tensor" if multi else "per_tensor"), (None, None))
        roofline = {
            "bound": "hbm",
            "kernel": f"{'adam_multi_kernel' if multi else 'adam_vec_kernel'}<{mode}>",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": (source + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                               "command; carried over, not measured in this run)") if source else None,
            "alg_bytes_per_launch": int(alg_bytes_per_launch),
            "avg_launch_us": round(avg_launch_s * 1e6, 2),
            "launches": launches,
        }
    return {
        "mode": mode, "tensors": len(tensors), "elements": total_elems,
        "bytes_per_step": bytes_per_step, "elapsed_s": elapsed, "roofline": roofline,
        "host_enqueue_us_per_step": round(enqueue / steps * 1e6, 1),
        "launch": "multi_tensor" if multi else "per_tensor",
        "rng": (rng or "x8") if mode == "stochastic_rounding" else None,
    }


def config0_row(steps=400, warmup=20):
    """Benchmark config 0 on the GPU.  The row's ``roofline`` is the HBM figure:
    six operand sets in rotation, so that the 256 MiB memory-side cache cannot serve
    any of the 335 MB a step touches.  ``cache_assisted`` is the same kernel on the
    same operands every step (what the config literally describes), part of which
    that cache serves: not an HBM bandwidth."""
    import torch

    row = {"workload": "fp32_master, one flat tensor of 16,777,216 elements, 20 B/elem",
           "floor_us_at_8TBps": 41.94}
    for label, sets in (("same_operands", 1), ("rotating_6_sets", 6)):
        r = time_adam_workload("c0_fp32_master_16m", steps, warmup, sets=sets)
        entry = {"ms_per_step": round(r["elapsed_s"] / steps * 1e3, 4),
                 "GBps_wall": round(r["bytes_per_step"] * steps / r["elapsed_s"] / 1e9, 1),
                 "host_enqueue_us_per_step": r["host_enqueue_us_per_step"],
                 "roofline": r["roofline"]}
        if sets > 1:
            row["roofline"] = r["roofline"]
            row["hbm_cold"] = entry
        else:
            entry["note"] = ("335 MB of operands reused every step; the 256 MiB memory-side "
                             "cache serves part of them")
            row["cache_assisted"] = entry
    return row


def config2_row(steps=5, warmup=2):
    """Kernel legs of benchmark config 2 on GPU-resident buffers at the real
    shapes (291 tensors, 8,030,261,248 elements): per-parameter gradient norms,
    the clip coefficient, and the fp31_master step with the coefficient folded
    into the gradient load."""
    import torch

    from offload_adam_amd import grad_clip

    r = time_adam_workload("c2_fp31_clip_llama8b", steps, warmup)
    row = {"adam_leg": {"ms_per_step": round(r["elapsed_s"] / steps * 1e3, 3),
                        "GBps_wall": round(r["bytes_per_step"] * steps / r["elapsed_s"] / 1e9, 1),
                        "roofline": r["roofline"], "floor_ms_at_8TBps": 18.07}}
    # norm leg: 291 gradients scaled so that the global norm is about 3
    dev = torch.device("cuda:0")
    shapes = WORKLOADS["c2_fp31_clip_llama8b"]["shapes"]
    g = torch.Generator(device=dev).manual_seed(2)
    grads = [(torch.randn(numel(s), device=dev, generator=g) * 3.35e-5).to(torch.bfloat16)
             for _, s in shapes]
    slots = torch.zeros(len(grads), dtype=torch.bfloat16, device=dev)
    coef = torch.ones((), dtype=torch.bfloat16, device=dev)
    total = torch.zeros((), dtype=torch.bfloat16, device=dev)

    # Groups as OffloadAdam's gradient hooks form them on the clipping path: a group
    # closes at 36 gradients or 512 MB of gradients (two launches per group).
    from offload_adam_amd.offload_adam import OffloadAdam

    groups, cur, cur_bytes = [], [], 0
    for i, t in enumerate(grads):
        cur.append(i)
        cur_bytes += t.numel() * 2
        if len(cur) >= grad_clip.NORMS_PER_LAUNCH or cur_bytes >= OffloadAdam._NORM_GROUP_BYTES:
            groups.append(cur)
            cur, cur_bytes = [], 0
    if cur:
        groups.append(cur)
    slot_views = [slots[i] for i in range(len(grads))]

    def norms_grouped():
        for idx in groups:
            grad_clip.grad_norms_([grads[i] for i in idx], [slot_views[i] for i in idx],
                                  validate=False)
        grad_clip.clip_coef_(slots, 1.0, coef, total)

    def norms_one_call():
        grad_clip.grad_norms_(grads, slot_views, validate=False)
        grad_clip.clip_coef_(slots, 1.0, coef, total)

    def norms_per_tensor():
        for i, t in enumerate(grads):
            grad_clip.grad_norm_(t, slot_views[i])
        grad_clip.clip_coef_(slots, 1.0, coef, total)

    def timed_pass(fn, reps=5):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    nbytes = 2 * sum(t.numel() for t in grads)
    ms = timed_pass(norms_grouped)
    ms_one = timed_pass(norms_one_call)
    ms_each = timed_pass(norms_per_tensor)
    row["norm_leg"] = {
        "ms_per_pass": round(ms, 3),
        "launches_per_pass": 2 * len(groups) + 1,
        "global_norm": float(total), "clip_coef": float(coef),
        "roofline": {"bound": "hbm", "kernel": "grad_norm_multi_partial_kernel + "
                     f"grad_norm_multi_final_kernel (x{len(groups)} groups) + clip_coef_kernel",
                     "achieved": round(nbytes / ms / 1e6, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                     "alg_bytes_per_pass": nbytes, "traffic": None},
        "floor_ms_at_8TBps": 2.01,
        "one_call_for_all_291": {"ms_per_pass": round(ms_one, 3),
                                 "frac": round(nbytes / ms_one / 1e6 / HBM_PEAK_GBS, 4)},
        "one_call_per_gradient": {"ms_per_pass": round(ms_each, 3),
                                  "frac": round(nbytes / ms_each / 1e6 / HBM_PEAK_GBS, 4),
                                  "launches_per_pass":
                                      sum(1 if t.numel() <= 16384 else 2 for t in grads) + 1},
        "note": "one pass = every per-parameter norm plus the coefficient; the headline groups "
                "the gradients as OffloadAdam's hooks do on the clipping path (36 gradients or "
                "512 MB per pair of launches); one call per gradient is what the reference's "
                "torch.norm per parameter amounts to and is bound by the host's launch rate",
    }
    del grads
    row["workload"] = ("fp31_master + clip, Llama-3-8B shapes: 291 tensors, 8,030,261,248 "
                       "elements, norm 2 B/elem, step 18 B/elem")
    return row


def config3_row(reps=40):
    """Benchmark config 3: the eight codec kernels and the fused fp32_master step
    + re-encode on one 4096 x 14336 weight (rotating buffers), through
    bench_kernels.py's routines."""
    import torch

    import bench_kernels

    args = argparse.Namespace(reps=reps)
    bench_kernels.SINK = rows = []
    try:
        bench_kernels.bench_codecs(args, torch)
        bench_kernels.bench_qat_step(args, torch)
    finally:
        bench_kernels.SINK = None
    keep = ("kernel", "alg_bytes_per_launch", "avg_launch_us", "achieved_GBps", "frac",
            "fused_speedup")
    return {"workload": "one 4096 x 14336 bf16 weight ~N(0, 0.02), 1 % of the entries x10",
            "kernels": [{k: r[k] for k in keep if k in r} for r in rows]}


def other_configs(cpu=True):
    out = {}
    for name, fn in (("c0_fp32_master_16m", config0_row), ("c2_fp31_clip_llama8b", config2_row),
                     ("c3_codecs", config3_row)):
        progress(f"other config {name}")
        try:
            out[name] = fn()
        except Exception as exc:  # a failed side measurement must not lose the main line
            out[name] = {"error": repr(exc)[:300]}
    if cpu:
        try:
            out["c2_fp31_clip_llama8b"]["cpu_baseline"] = cpu_baseline(
                "fp31_master", n=16_777_216, budget_s=4.0, clip=True)
            out["c3_codecs"]["cpu_baseline"] = cpu_baselines_of_the_other_kernels()
        except Exception as exc:
            out["cpu_baseline_error"] = repr(exc)[:300]
    return out


_T0 = time.time()


def progress(what):
    """One line on stderr per finished section: a run of several minutes must not
    look hung to whoever watches its output (stdout carries the JSON line only)."""
    print(f"[bench.py +{time.time() - _T0:5.0f} s] {what}", file=sys.stderr, flush=True)


def run_e2e(extra, steps, warmup, timeout_s, model="llama8b"):
    import subprocess

    progress(f"bench_e2e.py --model {model} {' '.join(extra)}")
    cmd = [sys.executable, str(ROOT / "bench_e2e.py"), "--model", model, "--steps", str(steps),
           "--warmup", str(warmup)] + extra
    try:
        res = subprocess.run(cmd, capture_output=True, text=True, timeout=timeout_s, cwd=str(ROOT))
        if res.returncode != 0:
            return {"error": f"bench_e2e.py exited with {res.returncode}",
                    "stderr_tail": res.stderr[-300:]}
        full = json.loads(res.stdout.strip().splitlines()[-1])
    except Exception as exc:  # a failed side measurement must not lose the main line
        return {"error": repr(exc)[:300]}
    full["steps"], full["warmup"] = steps, warmup
    keep = ("optimizer", "mode", "steps", "warmup", "seq", "grad_accum", "spare_hbm",
            "offload_grads", "params", "step_s", "step_s_to_last_kernel", "tokens_per_s",
            "fwd_bwd_only_s", "exposed_optimizer_s", "h2d_GB_per_step", "d2h_GB_per_step",
            "h2d_GBps_over_step", "d2h_GBps_over_step", "link_peak", "link_floor_s", "pinned_GiB",
            "prefetch_GiB", "grad_cache_GiB", "grad_cache_policy", "state_cache_GiB",
            "peak_gpu_GiB", "peak_reserved_GiB", "fwd_bwd_only_reserved_GiB", "optimizer_init_s", "link_copies", "copy_engines", "transfer_streams",
            "check",
            "max_grad_norm", "qat", "model_gpu_GiB", "pinned_limit",
            "loss_finite")
    row = {k: full[k] for k in keep if k in full}
    peak = (full.get("link_peak") or {}).get("bidir_each_GBps")
    if peak and "h2d_GBps_over_step" in full:
        row["h2d_frac_of_bidir_peak"] = round(full["h2d_GBps_over_step"] / peak, 3)
        row["d2h_frac_of_bidir_peak"] = round(full["d2h_GBps_over_step"] / peak, 3)
    return row


def offloaded_step_8b():
    """The second half of the metric: a synthetic Llama-3-8B-shaped training step
    (benchmark config 4: stochastic rounding, 4 micro-batches of 4096 tokens,
    hook path), measured by bench_e2e.py in child processes.  PCIe-inclusive;
    never part of ``value``.

    * ``reference_traffic``: OffloadAdam as constructed by default - caches off,
      every partial gradient sum written through: 80.3 GB each way per step, the
      reference's traffic and memory contract - followed by a numerical check of
      one more step;
    * ``spare_hbm``: ``OffloadAdam(spare_hbm=True)``;
    * ``resident_adam``: the same loop with the GPU-resident ``Adam`` for scale;
    * ``clip_path_fp31``: benchmark config 2 as a training step on the same model -
      ``fp31_master``, ``max_grad_norm=1.0`` (norms in the hooks, one-shot ``step()``),
      default memory contract - with the numerical check of one more step."""
    return {
        "model": "llama8b (32 layers, hidden 4096, vocab 128256), bf16, 1 x 4096 tokens x 4 "
                 "micro-batches, activation checkpointing",
        "reference_traffic": run_e2e(["--check"], steps=4, warmup=2, timeout_s=300),
        "spare_hbm": run_e2e(["--spare-hbm"], steps=4, warmup=2, timeout_s=300),
        "resident_adam": run_e2e(["--optimizer", "adam"], steps=3, warmup=1, timeout_s=300),
        "clip_path_fp31": run_e2e(["--mode", "fp31_master", "--max-grad-norm", "1.0", "--check"],
                                  steps=3, warmup=1, timeout_s=300),
    }


def mode_comparison_8b():
    """The reference's rounding-mode table (examples/e2e_train/README.md:99-109: one
    micro-batch of 4096 tokens per step, offloading on) on the same 8B-shaped model,
    both rows with ``OffloadAdam`` as constructed by default.  ``fp32_master`` needs
    74.8 GiB of pinned host memory at this size; where the driver grants less, the
    optimizer keeps the overflow (gradients first) in HBM and says so in
    ``pinned_limit``."""
    common = ["--grad-accum", "1"]
    return {
        "stochastic_rounding": run_e2e(common, steps=4, warmup=2, timeout_s=300),
        "fp32_master": run_e2e(common + ["--mode", "fp32_master", "--check"], steps=3, warmup=1,
                               timeout_s=300),
    }


def qat_steps():
    """The reference's QAT table (examples/qat/README.md:121-130: ``fp32_master``,
    one micro-batch of 8192 tokens per step, every attention / MLP projection
    quantised, lm_head in bf16) through ``OffloadAdam`` as constructed by default,
    each followed by the numerical check of one more step: the four formats and the
    unquantised row on the 1.1B-shaped model, and int4 (the example's own command)
    on the 8B-shaped one; then the same five 1.1B rows with the GPU-resident ``Adam``
    (no check there: tests/test_qat_replay_gpu.py replays that optimizer against the
    oracle)."""
    common = ["--grad-accum", "1", "--seq", "8192", "--check"]
    rows = {"llama1b": {"none": run_e2e(common + ["--mode", "fp32_master"], steps=5, warmup=2,
                                        timeout_s=200, model="llama1b")}}
    for fmt in ("int8", "int4", "nf4", "nvfp4"):
        rows["llama1b"][fmt] = run_e2e(common + ["--qat", fmt], steps=5, warmup=2, timeout_s=200,
                                       model="llama1b")
    rows["llama8b"] = {"int4": run_e2e(common + ["--qat", "int4"], steps=3, warmup=1,
                                       timeout_s=300)}
    # the table's other half: the GPU-resident Adam of this package on the same rows
    resident = ["--grad-accum", "1", "--seq", "8192", "--optimizer", "adam"]
    rows["llama1b_adam"] = {"none": run_e2e(resident + ["--mode", "fp32_master"], steps=5,
                                            warmup=2, timeout_s=200, model="llama1b")}
    for fmt in ("int8", "int4", "nf4", "nvfp4"):
        rows["llama1b_adam"][fmt] = run_e2e(resident + ["--qat", fmt], steps=5, warmup=2,
                                            timeout_s=200, model="llama1b")
    return rows


def _step_summary(row, reserved=False):
    """One streamed-step row boiled down for the summary at the end of the line
    (``GiB``: peak HBM allocated, the reference's measure; ``res``: peak HBM the caching
    allocator held from the driver)."""
    if not isinstance(row, dict) or "step_s" not in row:
        return {"error": (row or {}).get("error", "missing")[:60]} if isinstance(row, dict) else None
    out = {"s": row["step_s"], "exposed": row.get("exposed_optimizer_s"),
           "GiB": row.get("peak_gpu_GiB")}
    if reserved and "peak_reserved_GiB" in row:
        out["res"] = row["peak_reserved_GiB"]
    if "h2d_frac_of_bidir_peak" in row:
        out["h2d"], out["d2h"] = row["h2d_frac_of_bidir_peak"], row["d2h_frac_of_bidir_peak"]
    if "check" in row:
        out["ok"] = bool(row["check"].get("passed"))
    return out


def summary_of(out):
    """The figures a reader wants first, small enough to survive a log that keeps
    only the end of the line: roofline fraction per config, and per streamed step
    its time, exposed optimizer time, link use against the bidirectional peak, peak
    HBM and whether its numerical check passed."""
    def frac(d):
        return (d or {}).get("frac") if isinstance(d, dict) else None

    other = out.get("other_configs", {})
    c0, c2, c3 = (other.get(k, {}) for k in ("c0_fp32_master_16m", "c2_fp31_clip_llama8b",
                                             "c3_codecs"))
    kernels = c3.get("kernels", []) if isinstance(c3, dict) else []

    def least(pred):
        vals = [k["frac"] for k in kernels if pred(k["kernel"]) and "frac" in k]
        return min(vals) if vals else None

    fr = {"c1": frac(out.get("roofline")),
          "c1_ref_bits": frac(out.get("roofline_reference_layout")),
          "c0_cold": frac(c0.get("roofline")),
          "c0_cached": frac((c0.get("cache_assisted") or {}).get("roofline")),
          "c2_step": frac((c2.get("adam_leg") or {}).get("roofline")),
          "c2_norm": frac((c2.get("norm_leg") or {}).get("roofline")),
          "c3_enc_min": least(lambda k: k.startswith("quant_") or k.startswith("nvfp4_amax")),
          "c3_dec_min": least(lambda k: k.startswith("dequant_")),
          "c3_fused_min": least(lambda k: k.endswith(", fused"))}
    steps = {}
    e8 = out.get("offloaded_step_8b", {})
    for key, name in (("reference_traffic", "8b_ref"), ("spare_hbm", "8b_spare"),
                      ("resident_adam", "8b_adam"), ("clip_path_fp31", "8b_clip")):
        if key in e8:
            steps[name] = _step_summary(e8[key], reserved=True)
    if "offloaded_step_1b" in out:
        steps["1b"] = _step_summary(out["offloaded_step_1b"])
    for key, row in out.get("mode_comparison_8b", {}).items():
        steps["8b_ga1_" + ("sr" if key == "stochastic_rounding" else "fp32m")] = _step_summary(row)
    for model, rows in out.get("qat_step", {}).items():
        for fmt, row in rows.items():
            steps[f"qat_{model[5:]}_{fmt}"] = _step_summary(row)
    return {"frac": fr, "steps": steps}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c1_sr_llama1b", choices=sorted(WORKLOADS))
    ap.add_argument("--rng", default=None, choices=[None, "triton", "x8"],
                    help="stochastic_rounding bit layout (default: the optimizer's own, x8)")
    ap.add_argument("--per-tensor", action="store_true",
                    help="one launch per tensor (the hook-path call pattern) instead of the "
                         "multi-tensor launch")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run three 1 GiB device copies first (reference for counter runs)")
    ap.add_argument("--only-main", action="store_true",
                    help="the timed region only: no CPU baseline, other configs or 8B step "
                         "(profiler runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip configs 0, 2 and 3 (about half a minute)")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the training steps (bench_e2e.py in child processes after the timed "
                         "region; about four minutes)")
    ap.add_argument("--no-events", action="store_true",
                    help="skip per-launch HIP events (used for profiler runs)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from offload_adam_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    _lib.load()  # fails loudly when the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        # A plain device copy of known size (1 GiB read + 1 GiB written), so a
        # counter run can scale FETCH_SIZE / WRITE_SIZE to bytes.
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    r = time_adam_workload(args.workload, args.steps, args.warmup, rng=args.rng,
                           per_tensor=args.per_tensor, use_events=not args.no_events)
    ms_per_step = r["elapsed_s"] / args.steps * 1e3
    value = r["bytes_per_step"] * args.steps / r["elapsed_s"] / 1e9

    out = {
        "metric": "fused Adam GB/s & % HBM peak; 8B offloaded step time (s), 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "mode": r["mode"],
            "tensors": r["tensors"],
            "elements": r["elements"],
            "alg_bytes_per_elem": BYTES_PER_ELEM[r["mode"]],
            "resident": "HBM",
            "launch": r["launch"],
            "rng": r["rng"],
        },
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": r["roofline"],
    }
    side = not args.only_main
    if side and args.workload == "c1_sr_llama1b" and args.rng != "triton":
        # the same workload with the reference's random-bit layout (one Philox block per
        # element, tl.randint's), which is what a like-for-like reading of the kernel asks for
        ref = time_adam_workload(args.workload, max(5, args.steps // 2), args.warmup, rng="triton")
        out["roofline_reference_layout"] = dict(ref["roofline"], rng="triton")
    progress(f"timed region done: {out['value']} GB/s, frac {out['roofline']['frac'] if out['roofline'] else None}")
    if side and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        out["cpu_baseline"]["host"] = host_description()
        if args.workload == "c1_sr_llama1b":
            out["cpu_baseline_c1_sample"] = cpu_baseline("stochastic_rounding", n=64 << 20,
                                                         budget_s=4.0, min_iters=3)
    if side and args.workload == "c1_sr_llama1b":
        if not args.no_other_configs:
            out["other_configs"] = other_configs(cpu=not args.no_cpu_baseline)
        if not args.no_e2e:
            torch.cuda.empty_cache()  # the child processes below need the HBM
            out["offloaded_step_8b"] = offloaded_step_8b()
            # benchmark config 1 as a training step: the 1.1B set streamed through the
            # default OffloadAdam, one micro-batch of 4096 tokens per step, with the check
            out["offloaded_step_1b"] = run_e2e(["--grad-accum", "1", "--check"], steps=10,
                                               warmup=3, timeout_s=200, model="llama1b")
            out["mode_comparison_8b"] = mode_comparison_8b()
            out["qat_step"] = qat_steps()
    progress("done")
    if side:
        out["summary"] = summary_of(out)  # last key: it survives a log that keeps the tail
    print(json.dumps(out))


if __name__ == "__main__":
    main()
