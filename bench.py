#!/usr/bin/env python3
"""Benchmark of the optimizer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A "step" is one pass of the fused AdamW kernel over every tensor of the
workload, with all operands already resident in HBM.  The default workload is
benchmark config 1: stochastic_rounding mode over the Llama-style 1.1B
parameter set (201 tensors, 1,100,048,384 elements, 14 algorithmic bytes per
element).  Prints ONE JSON line.

Only one GPU is used; ``--gpus N`` with N > 1 exits with a message.
"""

import argparse
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
# read for a 1 GiB device copy (factors 2.000 and 1.000).  Keyed by
# (workload, launch form); the summary with the commands is
# profiles/adam_multi_kernel_sr_c1_llama1b_hbm_traffic.txt.
MEASURED_TRAFFIC_BYTES = {
    ("c1_sr_llama1b", "multi_tensor"): 2_566_900_000,
}

BYTES_PER_ELEM = {
    "stochastic_rounding": 14,
    "fp32_master": 20,
    "fp31_master": 18,
    "fp32_master_custom_rounding": 18,
}


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


def cpu_baseline(mode, target_elems=256 * 1024 * 1024, iters=5):
    """The same update math in PyTorch eager on this host's cores, on a bounded
    sample of the workload: one flat tensor of ``target_elems`` elements (a
    quarter of config 1), ``iters`` timed passes of about 2 s each."""
    import torch

    from oracle import folded_betas, torch_eager

    n = target_elems
    g = torch.Generator().manual_seed(0)
    p = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16)
    st = {
        "grad": (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16),
        "exp_avg": (torch.randn(n, generator=g) * 1e-4).to(torch.bfloat16),
        "exp_avg_sq": ((torch.randn(n, generator=g) * 1e-3) ** 2).to(torch.bfloat16),
    }
    b1h, b2h = folded_betas(0.9, 0.999, 10)
    args = (1e-4, 0.01, b1h, b2h, 1e-8, True)
    if mode == "stochastic_rounding":
        def run():
            r = torch.randint(0, 65536, (n,), dtype=torch.int32)
            torch_eager.adam_step_stochastic_rounding(p, st, *args, r)
    elif mode == "fp32_master":
        st["master_params"] = p.float()
        def run():
            torch_eager.adam_step_fp32_master(p, st, *args)
    else:
        st["rounding_error"] = torch.zeros(n, dtype=torch.int16)
        fn = (torch_eager.adam_step_fp31_master if mode == "fp31_master"
              else torch_eager.adam_step_custom_rounding)
        def run():
            fn(p, st, *args)
    run()  # warm-up
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    best = sorted(times)[len(times) // 2]
    return {
        "value": round(n * BYTES_PER_ELEM[mode] / best / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"one flat tensor of {n} elements, {mode}, torch eager fp32 on CPU, "
                  f"median of {iters} passes ({best:.3f} s per pass)",
    }


def cpu_baselines_of_the_other_kernels(rows=512, cols=14336):
    """The C restatement (one thread) of every kernel besides the AdamW update,
    on a bounded sample: ``rows`` x ``cols`` of the codec workload's weight and as
    many elements of gradient.  GB/s of the same algorithmic bytes the GPU figures
    of bench_kernels.py use (bf16 source and output)."""
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


def offloaded_step_8b(timeout_s=420):
    """The second half of the metric: step time of a synthetic Llama-3-8B-shaped
    training step through OffloadAdam (benchmark config 4), measured by
    bench_e2e.py in a child process.  PCIe-inclusive; never part of ``value``."""
    import subprocess

    # 12 steps: the write-back that trails the last step (0.5 s) is timed with them
    cmd = [sys.executable, str(ROOT / "bench_e2e.py"), "--model", "llama8b", "--steps", "12",
           "--warmup", "2"]
    try:
        res = subprocess.run(cmd, capture_output=True, text=True, timeout=timeout_s, cwd=str(ROOT))
        if res.returncode != 0:
            return {"error": f"bench_e2e.py exited with {res.returncode}",
                    "stderr_tail": res.stderr[-300:]}
        full = json.loads(res.stdout.strip().splitlines()[-1])
    except Exception as exc:  # a failed side measurement must not lose the main line
        return {"error": repr(exc)[:300]}
    full["steps"], full["warmup"] = 12, 2
    keep = ("model", "mode", "steps", "warmup", "seq", "grad_accum", "offload_grads", "params", "step_s",
            "step_s_to_last_kernel",
            "tokens_per_s", "fwd_bwd_only_s", "exposed_optimizer_s", "h2d_GB_per_step",
            "d2h_GB_per_step", "h2d_GBps_over_step", "d2h_GBps_over_step", "link_peak",
            "link_floor_s", "pinned_GiB", "prefetch_GiB", "grad_cache_GiB", "grad_cache_policy", "state_cache_GiB", "peak_gpu_GiB", "optimizer_init_s", "copy_engines",
            "transfer_streams")
    return {k: full[k] for k in keep if k in full}


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
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-baseline-other-kernels", action="store_true",
                    help="also time the CPU restatement of the norm and codec kernels "
                         "(bounded sample, a few seconds) and add it to the line")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the 8B offloaded training step (bench_e2e.py, run as a child "
                         "process after the timed region; about a minute)")
    ap.add_argument("--no-events", action="store_true",
                    help="skip per-launch HIP events (used for profiler runs)")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from offload_adam_amd import _lib, kernels
    from offload_adam_amd.kernels import adam_step_multi
    from offload_adam_amd.kernels.multi import MULTI_MAX

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    _lib.load()  # fails loudly when the HIP library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    wl = WORKLOADS[args.workload]
    mode = wl["mode"]
    tensors = make_tensors(mode, wl["shapes"], dev)
    step_fn = getattr(kernels, "adam_step_" + mode)
    clip = torch.tensor(0.3359375, dtype=torch.bfloat16, device=dev) if wl["clip"] else None
    total_elems = sum(p.numel() for p, _ in tensors)
    bytes_per_step = total_elems * BYTES_PER_ELEM[mode]
    kw, multi_kw = {}, {}
    if mode == "stochastic_rounding" and args.rng is not None:
        kw["rng"] = args.rng
        kw["seed"] = 1
        multi_kw["rng"] = args.rng
        multi_kw["seeds"] = list(range(1, len(tensors) + 1))

    multi = not args.per_tensor
    p_list = [p for p, _ in tensors]
    st_list = [st for _, st in tensors]
    launches_per_step = -(-len(tensors) // MULTI_MAX) if multi else len(tensors)

    def one_step(step_no, events=None):
        """One pass of the fused AdamW kernel over every tensor of the workload."""
        if multi:
            if events is not None:
                events[0][0].record()
            adam_step_multi(mode, p_list, st_list, 1e-4, 0.01, 0.9, 0.999, 1e-8, step_no,
                            decoupled_weight_decay=True, clip_coef=clip, validate=False,
                            **multi_kw)
            if events is not None:
                events[0][1].record()
            return
        for i, (p, st) in enumerate(tensors):
            if events is not None:
                events[i][0].record()
            step_fn(p, st, 1e-4, 0.01, 0.9, 0.999, 1e-8, step_no,
                    decoupled_weight_decay=True, clip_coef=clip, **kw)
            if events is not None:
                events[i][1].record()

    if args.copy_calibration:
        # A plain device copy of known size (1 GiB read + 1 GiB written), so a
        # counter run can scale FETCH_SIZE / WRITE_SIZE to bytes.
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for w in range(args.warmup):
        one_step(w + 1)
    torch.cuda.synchronize()

    # Timed region: exactly --steps steps, bracketed by device synchronisation.
    # Events are recorded on the stream the kernels run on (torch's current
    # stream) and read back after the closing synchronisation.
    use_events = not args.no_events
    pairs_per_step = 1 if multi else len(tensors)
    all_events = []
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev = None
        if use_events:
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                  for _ in range(pairs_per_step)]
            all_events.append(ev)
        one_step(args.warmup + s + 1, ev)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_ms = sum(a.elapsed_time(b) for ev in all_events for a, b in ev)
    launches = launches_per_step * len(all_events)

    ms_per_step = elapsed / args.steps * 1e3
    value = bytes_per_step * args.steps / elapsed / 1e9

    roofline = None
    if use_events and launches:
        avg_launch_s = kernel_ms / launches / 1e3
        alg_bytes_per_launch = bytes_per_step / launches_per_step
        achieved = alg_bytes_per_launch / avg_launch_s / 1e9
        roofline = {
            "bound": "hbm",
            "kernel": f"{'adam_multi_kernel' if multi else 'adam_vec_kernel'}<{mode}>",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(
                (args.workload, "multi_tensor" if multi else "per_tensor")),
            "alg_bytes_per_launch": int(alg_bytes_per_launch),
            "avg_launch_us": round(avg_launch_s * 1e6, 2),
            "launches": launches,
        }

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
            "mode": mode,
            "tensors": len(tensors),
            "elements": total_elems,
            "alg_bytes_per_elem": BYTES_PER_ELEM[mode],
            "resident": "HBM",
            "launch": "multi_tensor" if multi else "per_tensor",
            "rng": kw.get("rng", "x8") if mode == "stochastic_rounding" else None,
        },
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(mode)
    if args.cpu_baseline_other_kernels:
        out["cpu_baseline_other_kernels"] = cpu_baselines_of_the_other_kernels()
    if not args.no_e2e and args.workload == "c1_sr_llama1b":
        del tensors, p_list, st_list
        torch.cuda.empty_cache()
        out["offloaded_step_8b"] = offloaded_step_8b()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
