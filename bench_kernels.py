#!/usr/bin/env python3
"""Per-kernel throughput of everything on the optimizer path besides the fused
AdamW launch that ``bench.py`` measures: gradient L2 norm, clip coefficient,
the fused AdamW kernel with the clip coefficient folded in (fp31_master), and
the eight weight codecs, and the fp32_master step of a quantised weight (fused
with its re-encoding, and as the reference's two moves).  One JSON line per kernel.

    python bench_kernels.py [--reps 20] [--only norm_large,norm_small,norm_multi,clip,adam,codecs,qat,stream]

Shapes: the offloaded parameters of a Llama-3-8B-shaped decoder for the norm
and AdamW kernels, one 4096 x 14336 bf16 weight ~N(0, 0.02) with 1 % outliers
x10 for the codecs.  Every launch works on buffers that were not touched by the
previous launches of the same kernel (the inputs rotate through more distinct
buffers than the 256 MiB memory-side cache holds), so the figures are HBM
figures.  ``achieved`` = algorithmic bytes of one launch / (time between two HIP
events around ``--reps`` back-to-back launches on the launch stream / reps);
``frac`` is against 8 TB/s.
"""

import argparse
import gc
import json
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
ROWS, COLS = 4096, 14336


def timed(fn, reps, torch):
    """fn(i) launches once on rotation slot i; returns microseconds per launch.

    The launches are issued back to back between ONE pair of events: while the
    host keeps ahead of the GPU (true for every kernel here longer than the
    ~15 us a Python launch costs) the interval is GPU time, launch gaps included;
    for shorter kernels it is the host's launch rate, and says so in the
    profiler summary under profiles/."""
    for i in range(3):
        fn(i)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    gc.disable()  # as timeit does: a full collection (about 80 ms here) would land in the interval
    try:
        a.record()
        for i in range(reps):
            fn(i)
        b.record()
        torch.cuda.synchronize()
    finally:
        gc.enable()
    return a.elapsed_time(b) / reps * 1e3


SINK = None  # a list here collects the lines instead of printing them (bench.py does that)


def line(kernel, workload, alg_bytes, us, **extra):
    gbs = alg_bytes / us / 1e3
    out = {"kernel": kernel, "workload": workload, "alg_bytes_per_launch": int(alg_bytes),
           "avg_launch_us": round(us, 2), "achieved_GBps": round(gbs, 1),
           "peak_GBps": HBM_PEAK_GBS, "frac": round(gbs / HBM_PEAK_GBS, 4), "bound": "hbm"}
    out.update(extra)
    if SINK is not None:
        SINK.append(out)
    else:
        print(json.dumps(out), flush=True)


def outlier_weight(torch, seed, dtype):
    g = torch.Generator(device="cuda").manual_seed(seed)
    w = torch.randn(ROWS, COLS, device="cuda", generator=g) * 0.02
    mask = torch.rand(ROWS, COLS, device="cuda", generator=g) < 0.01
    return torch.where(mask, w * 10, w).to(dtype)


def bench_norm_and_clip(args, torch, todo):
    from offload_adam_amd import grad_clip

    if "norm_large" in todo:
        bench_norm_large(args, torch, grad_clip)
    if "norm_small" in todo:
        norms = torch.zeros(1, dtype=torch.bfloat16, device="cuda")
        small = torch.randn(4096 * 1024, device="cuda", dtype=torch.bfloat16)
        us = timed(lambda i: grad_clip.grad_norm_(small, norms[0]), args.reps, torch)
        line("grad_norm_partial_kernel + grad_norm_final_kernel",
             "bf16 gradient 1024x4096 (cache resident)", 2 * small.numel(), us)
    if "clip" in todo:
        per_param = torch.rand(291, device="cuda").to(torch.bfloat16)
        coef = torch.ones((), dtype=torch.bfloat16, device="cuda")
        us = timed(lambda i: grad_clip.clip_coef_(per_param, 1.0, coef), args.reps, torch)
        line("clip_coef_kernel", "291 per-parameter norms", 2 * 291, us, bound="latency")


def bench_norm_multi(args, torch):
    """The 291 per-parameter norms of a Llama-3-8B-shaped model (16.06 GB of bf16
    gradients) through the multi-tensor entry point: all in one call (9 pairs of
    launches), grouped as OffloadAdam's hooks group them (36 gradients or 512 MB per
    pair), and one call per gradient for comparison."""
    import bench
    from offload_adam_amd import grad_clip
    from offload_adam_amd.offload_adam import OffloadAdam

    shapes = bench.WORKLOADS["c2_fp31_clip_llama8b"]["shapes"]
    g = torch.Generator(device="cuda").manual_seed(2)
    grads = [(torch.randn(bench.numel(s), device="cuda", generator=g) * 3.35e-5).to(torch.bfloat16)
             for _, s in shapes]
    slots = torch.zeros(len(grads), dtype=torch.bfloat16, device="cuda")
    views = [slots[i] for i in range(len(grads))]
    nbytes = 2 * sum(t.numel() for t in grads)
    groups, cur, cur_bytes = [], [], 0
    for i, t in enumerate(grads):
        cur.append(i)
        cur_bytes += t.numel() * 2
        if len(cur) >= grad_clip.NORMS_PER_LAUNCH or cur_bytes >= OffloadAdam._NORM_GROUP_BYTES:
            groups.append(cur)
            cur, cur_bytes = [], 0
    if cur:
        groups.append(cur)

    def grouped(_):
        for idx in groups:
            grad_clip.grad_norms_([grads[i] for i in idx], [views[i] for i in idx], validate=False)

    reps = max(3, args.reps // 8)
    wl = "291 bf16 gradients of a Llama-3-8B-shaped model"
    us = timed(lambda i: grad_clip.grad_norms_(grads, views, validate=False), reps, torch)
    line("grad_norm_multi_partial_kernel + grad_norm_multi_final_kernel", wl + ", one call",
         nbytes, us, launches=2 * -(-len(grads) // grad_clip.NORMS_PER_LAUNCH))
    us = timed(grouped, reps, torch)
    line("grad_norm_multi_partial_kernel + grad_norm_multi_final_kernel",
         wl + f", {len(groups)} groups of up to 36 gradients or 512 MB", nbytes, us,
         launches=2 * len(groups))
    us = timed(lambda i: [grad_clip.grad_norm_(t, views[j]) for j, t in enumerate(grads)], reps,
               torch)
    line("grad_norm_partial_kernel + grad_norm_final_kernel", wl + ", one call per gradient",
         nbytes, us, launches=sum(1 if t.numel() <= 16384 else 2 for t in grads),
         note="host-bound: the launch rate of the Python loop")


def bench_norm_large(args, torch, grad_clip):
    n_big = COLS * 4096
    slots = 8  # 8 x 117 MB = 0.94 GB rotation
    grads = [torch.randn(n_big, device="cuda", dtype=torch.bfloat16) * 5e-3 for _ in range(slots)]
    norms = torch.zeros(slots, dtype=torch.bfloat16, device="cuda")
    us = timed(lambda i: grad_clip.grad_norm_(grads[i % slots], norms[i % slots]), args.reps, torch)
    line("grad_norm_partial_kernel + grad_norm_final_kernel", "bf16 gradient 14336x4096", 2 * n_big, us)


def bench_adam_clip(args, torch):
    from offload_adam_amd.kernels import adam_step_fp31_master, adam_step_stochastic_rounding

    n = COLS * 4096
    slots = 4
    clip = torch.tensor(0.3359375, dtype=torch.bfloat16, device="cuda")

    def states(extra):
        st = {"grad": torch.randn(n, device="cuda", dtype=torch.bfloat16) * 5e-3,
              "exp_avg": torch.randn(n, device="cuda", dtype=torch.bfloat16) * 1e-4,
              "exp_avg_sq": (torch.randn(n, device="cuda") * 1e-3).square().to(torch.bfloat16)}
        if extra:
            st["rounding_error"] = torch.zeros(n, dtype=torch.int16, device="cuda")
        return st

    ps = [torch.randn(n, device="cuda", dtype=torch.bfloat16) * 0.02 for _ in range(slots)]
    st31 = [states(True) for _ in range(slots)]
    us = timed(lambda i: adam_step_fp31_master(ps[i % slots], st31[i % slots], 1e-4, 0.01, 0.9,
                                               0.999, 1e-8, 10, decoupled_weight_decay=True,
                                               clip_coef=clip), args.reps, torch)
    line("adam_vec_kernel<fp31_master, clip>", "one 14336x4096 parameter (hook-path launch)",
         18 * n, us)
    us = timed(lambda i: adam_step_stochastic_rounding(ps[i % slots], st31[i % slots], 1e-4, 0.01,
                                                       0.9, 0.999, 1e-8, 10,
                                                       decoupled_weight_decay=True),
               args.reps, torch)
    line("adam_vec_kernel<stochastic_rounding>", "one 14336x4096 parameter (hook-path launch)",
         14 * n, us)


def bench_codecs(args, torch):
    from offload_adam_amd.qweight import _codec_ops as ops

    n = ROWS * COLS
    slots = 6
    bf16 = torch.bfloat16
    ws = [outlier_weight(torch, s, bf16) for s in range(slots)]
    wl = "4096x14336 bf16 weight"

    q8 = [torch.empty(ROWS, COLS, dtype=torch.int8, device="cuda") for _ in range(slots)]
    s8 = [torch.empty(ROWS, dtype=bf16, device="cuda") for _ in range(slots)]
    us = timed(lambda i: ops.quantize_int8_into(ws[i % slots], q8[i % slots], s8[i % slots]),
               args.reps, torch)
    line("quant_int8_kernel", wl, n * 3 + ROWS * 2, us)
    us = timed(lambda i: ops.dequantize_int8(q8[i % slots], s8[i % slots], bf16), args.reps, torch)
    line("dequant_int8_kernel", wl, n * 3 + ROWS * 2, us)

    g = 128
    q4 = [torch.empty(COLS // 8, ROWS, dtype=torch.int32, device="cuda") for _ in range(slots)]
    s4 = [torch.empty(COLS // g, ROWS, dtype=bf16, device="cuda") for _ in range(slots)]
    us = timed(lambda i: ops.quantize_int4_into(ws[i % slots], g, q4[i % slots], s4[i % slots]),
               args.reps, torch)
    line("quant_int4_kernel", wl + ", group 128", n * 2.5 + n // g * 2, us)
    us = timed(lambda i: ops.dequantize_int4(q4[i % slots], s4[i % slots], g, bf16),
               args.reps, torch)
    line("dequant_int4_kernel", wl + ", group 128", n * 2.5 + n // g * 2, us)

    b = 64
    qn = [torch.empty(ROWS, COLS // 2, dtype=torch.uint8, device="cuda") for _ in range(slots)]
    an = [torch.empty(ROWS * (COLS // b), dtype=torch.float32, device="cuda")
          for _ in range(slots)]
    us = timed(lambda i: ops.quantize_nf4_into(ws[i % slots], b, qn[i % slots], an[i % slots]),
               args.reps, torch)
    line("quant_nf4_kernel", wl + ", block 64", n * 2.5 + n // b * 4, us)
    us = timed(lambda i: ops.dequantize_nf4(qn[i % slots], an[i % slots], COLS, b, bf16),
               args.reps, torch)
    line("dequant_nf4_kernel", wl + ", block 64", n * 2.5 + n // b * 4, us)

    qf = [torch.empty(ROWS, COLS // 2, dtype=torch.uint8, device="cuda") for _ in range(slots)]
    sf = [torch.empty(ROWS, COLS // 16, dtype=torch.float8_e4m3fn, device="cuda")
          for _ in range(slots)]
    gf = [torch.zeros((), dtype=torch.float32, device="cuda") for _ in range(slots)]
    us = timed(lambda i: ops.quantize_nvfp4_into(ws[i % slots], qf[i % slots], sf[i % slots],
                                                 gf[i % slots]), args.reps, torch)
    line("nvfp4_amax_partial_kernel + nvfp4_global_scale_kernel + quant_nvfp4_kernel", wl + ", group 16",
         n * 2 + n * 2.5 + n // 16, us,
         note="three launches: per-block amax (reads the weight), global scale, encode (reads it again)")
    us = timed(lambda i: ops.dequantize_nvfp4(qf[i % slots], sf[i % slots], gf[i % slots], COLS,
                                              bf16), args.reps, torch)
    line("dequant_nvfp4_kernel", wl + ", group 16", n * 2.5 + n // 16, us)


def bench_stream_ceiling(args, torch):
    """What a plain device-to-device copy reaches on this part: the runtime's own
    copy kernel (``Tensor.copy_`` between two HBM buffers), reads + writes counted,
    on buffers that rotate like the other sections'.  The yardstick the AdamW
    kernels' 14-20 bytes per element are held against besides the 8 TB/s nameplate."""
    from offload_adam_amd import grad_clip
    from offload_adam_amd.offload_adam import _copy_by_kernel

    # read-only: the gradient-norm kernel over 1 GiB
    n = 512 << 20
    gs = [torch.empty(n, dtype=torch.bfloat16, device="cuda").normal_(0, 1e-3) for _ in range(3)]
    out = torch.zeros((), dtype=torch.bfloat16, device="cuda")
    us = timed(lambda i: grad_clip.grad_norm_(gs[i % 3], out), args.reps, torch)
    line("grad_norm_partial_kernel + grad_norm_final_kernel (read only)", "1024 MiB read", 2 * n, us)
    del gs
    for mib in (392, 1024):
        n = mib << 20
        slots = max(2, (3 << 30) // (2 * n) + 1)
        src = [torch.empty(n, dtype=torch.uint8, device="cuda").random_() for _ in range(slots)]
        dst = [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(slots)]
        wl = f"{mib} MiB read + {mib} MiB written"
        us = timed(lambda i: dst[i % slots].copy_(src[i % slots]), args.reps, torch)
        line("runtime device-to-device copy", wl, 2 * n, us)
        stream = torch.cuda.current_stream()
        for wgs in (1024, 4096):
            us = timed(lambda i: _copy_by_kernel(dst[i % slots], src[i % slots], stream, wgs),
                       args.reps, torch)
            line(f"link_copy_kernel between HBM buffers, {wgs} workgroups", wl, 2 * n, us)
        del src, dst


def bench_qat_step(args, torch):
    """fp32_master AdamW on a quantised 4096 x 14336 weight, then its payload
    re-encoded from the new master: one fused launch (oa_adam_requant_*) against
    the two moves of the reference (step with the gradient buffer as bf16 sink,
    then copy_(master))."""
    from offload_adam_amd.kernels import adam_step_fp32_master
    from offload_adam_amd.qweight import Int4QWeight, Int8QWeight, NF4QWeight, NVFP4QWeight

    n = ROWS * COLS
    slots = 4
    bf16 = torch.bfloat16
    hyp = (1e-4, 0.01, 0.9, 0.999, 1e-8, 10)

    def states():
        w = outlier_weight(torch, 0, bf16)
        return {"grad": (torch.randn(ROWS, COLS, device="cuda") * 5e-3).to(bf16),
                "exp_avg": (torch.randn(ROWS, COLS, device="cuda") * 1e-4).to(bf16),
                "exp_avg_sq": (torch.randn(ROWS, COLS, device="cuda") * 1e-3).square().to(bf16),
                "master_params": w.float()}

    sts = [states() for _ in range(slots)]
    formats = (("int8", Int8QWeight, {}, 1 + 2 / COLS),
               ("int4", Int4QWeight, {"group_size": 128}, 0.5 + 2 / 128),
               ("nf4", NF4QWeight, {"blocksize": 64}, 0.5 + 4 / 64),
               ("nvfp4", NVFP4QWeight, {}, 0.5 + 1 / 16))
    for name, cls, kw, payload_bpe in formats:
        qws = [cls.from_float(outlier_weight(torch, s, bf16), **kw) for s in range(slots)]
        wl = f"4096x14336 {name} weight, fp32 master, bf16 moments"
        us = timed(lambda i: adam_step_fp32_master(qws[i % slots], sts[i % slots], *hyp,
                                                   decoupled_weight_decay=True),
                   args.reps, torch)
        # NVFP4 reads the stored master once more for the encode launch
        extra = 4 if name == "nvfp4" else 0
        line(f"adam fp32_master + requant {name}, fused", wl, n * (18 + extra + payload_bpe), us)

        def two_moves(i):
            st = sts[i % slots]
            adam_step_fp32_master(st["grad"], st, *hyp, decoupled_weight_decay=True)
            qws[i % slots].copy_(st["master_params"])

        us2 = timed(two_moves, args.reps, torch)
        line(f"adam fp32_master + requant {name}, two moves", wl,
             n * (20 + 4 + extra + payload_bpe), us2, fused_speedup=round(us2 / us, 3))
        del qws


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=40)
    ap.add_argument("--only", default="norm_large,norm_small,norm_multi,clip,adam,codecs,qat,stream",
                    help="comma-separated subset of: norm_large, norm_small, norm_multi, clip, adam, "
                         "codecs, qat, stream")
    args = ap.parse_args()

    import torch

    from offload_adam_amd import _lib

    if not torch.cuda.is_available():
        print("bench_kernels.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    _lib.load()
    torch.cuda.set_device(0)
    todo = set(args.only.split(","))
    if todo & {"norm_large", "norm_small", "clip"}:
        bench_norm_and_clip(args, torch, todo)
    if "norm_multi" in todo:
        bench_norm_multi(args, torch)
    if "adam" in todo:
        bench_adam_clip(args, torch)
    if "codecs" in todo:
        bench_codecs(args, torch)
    if "qat" in todo:
        bench_qat_step(args, torch)
    if "stream" in todo:
        bench_stream_ceiling(args, torch)


if __name__ == "__main__":
    main()
