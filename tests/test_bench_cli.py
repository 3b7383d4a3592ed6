"""The benchmark program's own contract, as far as it can be checked without a GPU:
one GPU only, the workload tables hold the benchmark configs' tensor sets, and the
CPU baseline leg reports the fields the bench line carries."""

import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_a_rank_of_a_larger_world_is_refused(monkeypatch):
    import os

    env = dict(os.environ, WORLD_SIZE="4", RANK="1", LOCAL_RANK="1")
    r = subprocess.run([sys.executable, str(ROOT / "bench.py")], env=env,
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr


def test_workload_tables_hold_the_benchmark_tensor_sets():
    import bench

    def total(name):
        return sum(bench.numel(s) for _, s in bench.WORKLOADS[name]["shapes"])

    # Llama-1.1B: 201 tensors, 1,100,048,384 elements; Llama-3-8B: 291 tensors, 8,030,261,248
    c1, c2 = bench.WORKLOADS["c1_sr_llama1b"], bench.WORKLOADS["c2_fp31_clip_llama8b"]
    assert len(c1["shapes"]) == 201 and total("c1_sr_llama1b") == 1_100_048_384
    assert len(c2["shapes"]) == 291 and total("c2_fp31_clip_llama8b") == 8_030_261_248
    assert total("c0_fp32_master_16m") == 16_777_216
    assert c1["mode"] == "stochastic_rounding" and c2["mode"] == "fp31_master" and c2["clip"]
    # algorithmic bytes per element of the four modes (param + grad + two moments + extra state)
    assert bench.BYTES_PER_ELEM == {"fp32_master": 20, "stochastic_rounding": 14,
                                    "fp31_master": 18, "fp32_master_custom_rounding": 18}


def test_cpu_baseline_fields_on_a_small_sample():
    import bench

    row = bench.cpu_baseline(mode="fp32_master", n=1 << 16, budget_s=0.05, min_iters=3)
    assert row["unit"] == "GB/s" and row["kind"] == "port" and row["value"] > 0
    assert row["cores"] >= 1 and row["passes"] >= 3
    assert "65536 elements" in row["sample"]
    host = bench.host_description()  # travels with the baseline in the bench line
    assert host["os_cpu_count"] >= 1 and host["numa_nodes"] >= 1 and host["torch_num_threads"] >= 1


def test_summary_is_the_last_key_material_and_stays_small():
    """``summary_of`` boils a full line down to what must survive a log that keeps
    only the last 2000 characters."""
    import json

    import bench

    roof = lambda f: {"frac": f, "achieved": 8000 * f}  # noqa: E731
    step = {"step_s": 2.0123, "exposed_optimizer_s": 0.6123, "peak_gpu_GiB": 24.71,
            "peak_reserved_GiB": 39.81,
            "h2d_frac_of_bidir_peak": 0.831, "d2h_frac_of_bidir_peak": 0.829,
            "check": {"passed": True}}
    line = {
        "roofline": roof(0.78), "roofline_reference_layout": roof(0.72),
        "other_configs": {
            "c0_fp32_master_16m": {"roofline": roof(0.73), "cache_assisted": {"roofline": roof(0.84)}},
            "c2_fp31_clip_llama8b": {"adam_leg": {"roofline": roof(0.776)},
                                     "norm_leg": {"roofline": roof(0.82)}},
            "c3_codecs": {"kernels": [{"kernel": "quant_int8_kernel", "frac": 0.75},
                                      {"kernel": "quant_int4_kernel", "frac": 0.67},
                                      {"kernel": "dequant_nf4_kernel", "frac": 0.81},
                                      {"kernel": "adam fp32_master + requant int8, fused", "frac": 0.66},
                                      {"kernel": "adam fp32_master + requant int8, two moves",
                                       "frac": 0.5}]},
        },
        "offloaded_step_8b": {"model": "x", "reference_traffic": step, "spare_hbm": step,
                              "resident_adam": {"step_s": 1.47, "exposed_optimizer_s": 0.03,
                                                "peak_gpu_GiB": 65.1},
                              "clip_path_fp31": step},
        "offloaded_step_1b": step,
        "mode_comparison_8b": {"stochastic_rounding": step, "fp32_master": step},
        "qat_step": {"llama1b": {k: step for k in ("none", "int8", "int4", "nf4", "nvfp4")},
                     "llama8b": {"int4": {"error": "bench_e2e.py exited with 1"}},
                     "llama1b_adam": {k: {"step_s": 0.2123, "exposed_optimizer_s": 0.0123,
                                          "peak_gpu_GiB": 12.34}
                                      for k in ("none", "int8", "int4", "nf4", "nvfp4")}},
    }
    s = bench.summary_of(line)
    assert s["frac"] == {"c1": 0.78, "c1_ref_bits": 0.72, "c0_cold": 0.73, "c0_cached": 0.84,
                         "c2_step": 0.776, "c2_norm": 0.82, "c3_enc_min": 0.67,
                         "c3_dec_min": 0.81, "c3_fused_min": 0.66}
    assert s["steps"]["8b_ref"] == {"s": 2.0123, "exposed": 0.6123, "GiB": 24.71, "res": 39.81,
                                    "h2d": 0.831, "d2h": 0.829, "ok": True}
    assert "res" not in s["steps"]["1b"]
    assert "ok" not in s["steps"]["8b_adam"]
    assert set(s["steps"]) == {"8b_ref", "8b_spare", "8b_adam", "8b_clip", "1b", "8b_ga1_sr",
                               "8b_ga1_fp32m", "qat_1b_none", "qat_1b_int8", "qat_1b_int4",
                               "qat_1b_nf4", "qat_1b_nvfp4", "qat_8b_int4", "qat_1b_adam_none",
                               "qat_1b_adam_int8", "qat_1b_adam_int4", "qat_1b_adam_nf4",
                               "qat_1b_adam_nvfp4"}
    assert "error" in s["steps"]["qat_8b_int4"]
    assert len(json.dumps({"summary": s})) < 1950
    assert bench.summary_of({})["steps"] == {}


def test_copy_trace_summary_on_a_synthetic_trace(tmp_path):
    """bench_e2e.copy_trace_summary: union of intervals per direction, overlap of the two
    directions, and the trailing window, on a hand-made rocprofv3 memory-copy trace."""
    import bench_e2e

    rows = [("MEMORY_COPY_HOST_TO_DEVICE", 0, 100), ("MEMORY_COPY_HOST_TO_DEVICE", 50, 150),
            ("MEMORY_COPY_HOST_TO_DEVICE", 1_000_000_000, 1_400_000_000),
            ("MEMORY_COPY_DEVICE_TO_HOST", 1_200_000_000, 1_500_000_000),
            ("MEMORY_COPY_DEVICE_TO_HOST", 1_600_000_000, 2_000_000_000)]
    sub = tmp_path / "host" / "pid"
    sub.mkdir(parents=True)
    with open(sub / "t_memory_copy_trace.csv", "w") as fh:
        fh.write('"Kind","Direction","Stream_Id","Start_Timestamp","End_Timestamp"\n')
        for d, s, e in rows:
            fh.write(f'"MEMORY_COPY","{d}",1,{s},{e}\n')
    whole = bench_e2e.copy_trace_summary(str(tmp_path))
    assert whole["MEMORY_COPY_HOST_TO_DEVICE"] == {"copies": 3, "busy_s": 0.4, "sum_of_durations_s": 0.4}
    assert whole["MEMORY_COPY_DEVICE_TO_HOST"]["busy_s"] == 0.7
    assert whole["both_directions_busy_s"] == 0.2
    tail = bench_e2e.copy_trace_summary(str(tmp_path), window_s=1.0)  # from t = 1.0 s on
    assert tail["MEMORY_COPY_HOST_TO_DEVICE"]["copies"] == 1 and tail["window_s"] == 1.0
    with pytest.raises(SystemExit):
        bench_e2e.copy_trace_summary(str(tmp_path / "nothing_here"))
