#!/usr/bin/env python3
"""Clock and power of the GPU while each streaming loop of the optimizer path runs.

    python bench_telemetry.py [--seconds 2.5] [--loops idle,c1_x8,c1_triton,c2_fp31_clip,
                               c0_rotating6,c0_same,norm_1gib,fill_1gib]

Every loop launches one kernel back to back for at least ``--seconds`` while a
child process (which never touches HIP) samples the GPU's own telemetry through
the ``amdsmi`` Python package about every 5 ms: the graphics clock of each of the
8 XCDs, socket power, the power cap, the memory clock, memory-controller
activity, and the firmware's residency counters (milliseconds the part spent
throttled by the socket power limit "ppt", by temperature, by the voltage
regulators, by HBM temperature).  One JSON line per loop: the loop's own HBM
throughput (algorithmic bytes over the HIP-event time) next to the medians of
the samples taken in the last 70 % of its window, and the residency deltas over
the whole window.

The loops are the multi-tensor AdamW launches of bench.py's workloads
(stochastic rounding with the package's random-bit layout and with the
reference's, fp31_master with the clip folded in, fp32_master on one 16.8 M
element tensor with rotating and with fixed operands), a read-only pass (the
gradient-norm kernel over 1 GiB) and a write-only pass (``fill_`` of 1 GiB).

``OFFLOAD_ADAM_HIP_LIB`` selects another build of the library, e.g. one compiled
with ``-DOA_ADAM_APPROX_DIV_SQRT=1`` to see what the exact divide and square root
cost in clock and power.
"""

import argparse
import json
import os
import subprocess
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

KEEP = ("gfxclk", "uclk", "power", "residency", "accumulation", "gfx_activity", "umc_activity",
        "temperature_hotspot", "temperature_mem")


def _plain(x):
    if isinstance(x, dict):
        return {str(k): _plain(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_plain(v) for v in x]
    return x if isinstance(x, (int, float, str, bool)) or x is None else str(x)


def sampler(bdf, samples_path, stop_path, period_s):
    """Child process: amdsmi only (sysfs and drm ioctls), no HIP."""
    import amdsmi

    amdsmi.amdsmi_init()
    handles = amdsmi.amdsmi_get_processor_handles()
    handle = None
    for h in handles:
        if str(amdsmi.amdsmi_get_gpu_device_bdf(h)).lower() == bdf.lower():
            handle = h
    if handle is None:
        if len(handles) != 1:
            raise SystemExit(f"bench_telemetry: no amdsmi device with PCI address {bdf}")
        handle = handles[0]
    info = {"bdf": bdf}
    for name in ("amdsmi_get_power_cap_info", "amdsmi_get_gpu_metrics_header_info"):
        try:
            info[name] = _plain(getattr(amdsmi, name)(handle))
        except Exception as exc:  # noqa: BLE001 - telemetry is best effort per field
            info[name] = repr(exc)
    with open(samples_path, "w") as out:
        out.write(json.dumps({"info": info}) + "\n")
        while not os.path.exists(stop_path):
            m = amdsmi.amdsmi_get_gpu_metrics_info(handle)
            rec = {"t": time.time(),
                   "m": _plain({k: v for k, v in m.items() if any(s in k for s in KEEP)})}
            out.write(json.dumps(rec) + "\n")
            time.sleep(period_s)


def _num(x):
    try:
        return float(x)
    except (TypeError, ValueError):
        return None


def _median(xs):
    xs = sorted(x for x in xs if x is not None)
    return xs[len(xs) // 2] if xs else None


def summarise(mark, recs, alg_bytes):
    """Medians over the steady part of one loop's window, residency over all of it."""
    t0, t1 = mark["t0"], mark["t1"]
    steady = [r["m"] for r in recs if t0 + 0.3 * (t1 - t0) <= r["t"] <= t1]
    whole = [r["m"] for r in recs if t0 <= r["t"] <= t1]
    row = {"loop": mark["name"], "launches": mark["reps"],
           "ms_per_launch": round(mark["gpu_ms_per_rep"], 4), "samples": len(whole)}
    if alg_bytes and mark["gpu_ms_per_rep"]:
        gbps = alg_bytes / mark["gpu_ms_per_rep"] / 1e6
        row["achieved_GBps"] = round(gbps, 1)
        row["frac_of_8TBps"] = round(gbps / 8000.0, 4)
    clocks = []
    for m in steady:
        per_xcd = [_num(v) for v in (m.get("current_gfxclks") or [])]
        per_xcd = [v for v in per_xcd if v is not None and v < 60000]
        if per_xcd:
            clocks.append(sum(per_xcd) / len(per_xcd))
    row["gfxclk_MHz"] = _median(clocks)
    row["gfxclk_MHz_min"] = min(clocks) if clocks else None
    row["socket_power_W"] = _median([_num(m.get("current_socket_power")) for m in steady])
    row["uclk_MHz"] = _median([_num(m.get("current_uclk")) for m in steady])
    row["gfx_activity_pct"] = _median([_num(m.get("average_gfx_activity")) for m in steady])
    row["umc_activity_pct"] = _median([_num(m.get("average_umc_activity")) for m in steady])
    row["temperature_hotspot_C"] = _median([_num(m.get("temperature_hotspot")) for m in steady])
    row["temperature_mem_C"] = _median([_num(m.get("temperature_mem")) for m in steady])
    if len(whole) >= 2:
        first, last = whole[0], whole[-1]
        ticks = (_num(last.get("accumulation_counter")) or 0) - (_num(first.get("accumulation_counter")) or 0)
        row["firmware_ticks"] = ticks
        for key in ("ppt", "prochot", "socket_thm", "vr_thm", "hbm_thm"):
            k = key + "_residency_acc"
            a, b = _num(first.get(k)), _num(last.get(k))
            if a is not None and b is not None:
                row[key + "_throttled_frac"] = round((b - a) / ticks, 3) if ticks else None
    return row


def run_loops(args):
    import torch

    import bench
    from offload_adam_amd import _lib, grad_clip
    from offload_adam_amd.kernels import adam_step_multi

    if not torch.cuda.is_available():
        raise SystemExit("bench_telemetry.py: no GPU visible")
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    pr = torch.cuda.get_device_properties(0)
    bdf = f"{pr.pci_domain_id:04x}:{pr.pci_bus_id:02x}:{pr.pci_device_id:02x}.0"
    tmp = tempfile.mkdtemp(prefix="oa_telemetry_")
    samples, stop = os.path.join(tmp, "samples.jsonl"), os.path.join(tmp, "stop")
    child = subprocess.Popen([sys.executable, str(Path(__file__).resolve()), "--sampler", bdf,
                              samples, stop, str(args.period_ms / 1e3)])
    time.sleep(1.0)
    marks, alg = [], {}

    def timed_loop(name, launch, min_s):
        """``launch(k)`` issues k launches; run it for at least min_s between two events."""
        launch(3)
        torch.cuda.synchronize()
        t0 = time.time()
        launch(10)
        torch.cuda.synchronize()
        reps = max(10, int(min_s / ((time.time() - t0) / 10)))
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        time.sleep(0.5)  # back to idle, so that the ramp lies inside the window
        t0 = time.time()
        a.record()
        launch(reps)
        b.record()
        torch.cuda.synchronize()
        marks.append({"name": name, "t0": t0, "t1": time.time(), "reps": reps,
                      "gpu_ms_per_rep": a.elapsed_time(b) / reps})

    def adam_loop(workload, rng, sets):
        wl = bench.WORKLOADS[workload]
        mode = wl["mode"]
        operands = [bench.make_tensors(mode, wl["shapes"], dev, seed=s) for s in range(sets)]
        lists = [([p for p, _ in ts], [st for _, st in ts]) for ts in operands]
        clip = torch.tensor(0.3359375, dtype=torch.bfloat16, device=dev) if wl["clip"] else None
        kw = {}
        if mode == "stochastic_rounding" and rng is not None:
            kw = {"rng": rng, "seeds": list(range(1, len(operands[0]) + 1))}
        hyp = bench.HYP
        turn = [0]

        def launch(k):
            for _ in range(k):
                turn[0] += 1
                params, states = lists[turn[0] % sets]
                adam_step_multi(mode, params, states, hyp["lr"], hyp["wd"], hyp["beta1"],
                                hyp["beta2"], hyp["eps"], 10, decoupled_weight_decay=True,
                                clip_coef=clip, validate=False, **kw)
        elems = sum(p.numel() for p, _ in operands[0])
        return launch, elems * bench.BYTES_PER_ELEM[mode]

    want = args.loops.split(",")
    if "idle" in want:
        torch.cuda.synchronize()
        t0 = time.time()
        time.sleep(args.seconds)
        marks.append({"name": "idle", "t0": t0, "t1": time.time(), "reps": 0, "gpu_ms_per_rep": 0})
    for name, workload, rng, sets in (("c1_x8", "c1_sr_llama1b", None, 1),
                                      ("c1_triton", "c1_sr_llama1b", "triton", 1),
                                      ("c2_fp31_clip", "c2_fp31_clip_llama8b", None, 1),
                                      ("c0_rotating6", "c0_fp32_master_16m", None, 6),
                                      ("c0_same", "c0_fp32_master_16m", None, 1)):
        if name in want:
            launch, alg[name] = adam_loop(workload, rng, sets)
            timed_loop(name, launch, args.seconds)
            del launch
            torch.cuda.empty_cache()
    if "norm_1gib" in want:
        g = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_(0, 1e-3)
        slot = torch.zeros(1, dtype=torch.bfloat16, device=dev)
        alg["norm_1gib"] = 2 * g.numel()
        timed_loop("norm_1gib", lambda k: [grad_clip.grad_norm_(g, slot[0]) for _ in range(k)],
                   args.seconds)
        del g
        torch.cuda.empty_cache()
    if "fill_1gib" in want:
        g = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        alg["fill_1gib"] = g.numel()
        timed_loop("fill_1gib", lambda k: [g.fill_(1) for _ in range(k)], args.seconds)
        del g
        torch.cuda.empty_cache()

    time.sleep(0.3)
    open(stop, "w").close()
    child.wait(timeout=30)
    with open(samples) as fh:
        recs = [json.loads(ln) for ln in fh]
    info, recs = recs[0]["info"], recs[1:]
    cap = (info.get("amdsmi_get_power_cap_info") or {})
    print(json.dumps({"library": os.environ.get("OFFLOAD_ADAM_HIP_LIB") or "as shipped",
                      "power_cap_W": (_num(cap.get("power_cap")) or 0) / 1e6 if isinstance(cap, dict) else None,
                      "gpu_metrics_revision": info.get("amdsmi_get_gpu_metrics_header_info"),
                      "samples": len(recs), "device": pr.name}), flush=True)
    for mk in marks:
        print(json.dumps(summarise(mk, recs, alg.get(mk["name"]))), flush=True)
    for p in (samples, stop):
        os.remove(p)
    os.rmdir(tmp)


def main():
    if len(sys.argv) > 1 and sys.argv[1] == "--sampler":
        sampler(sys.argv[2], sys.argv[3], sys.argv[4], float(sys.argv[5]))
        return
    ap = argparse.ArgumentParser()
    ap.add_argument("--seconds", type=float, default=2.5, help="minimum length of each loop")
    ap.add_argument("--period-ms", type=float, default=4.0, help="pause between samples")
    ap.add_argument("--loops", default="idle,c1_x8,c1_triton,c2_fp31_clip,c0_rotating6,c0_same,"
                                       "norm_1gib,fill_1gib")
    run_loops(ap.parse_args())


if __name__ == "__main__":
    main()
