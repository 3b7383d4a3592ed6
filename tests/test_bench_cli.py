"""The benchmark program's own contract, as far as it can be checked without a GPU:
one GPU only, the workload tables hold the benchmark configs' tensor sets, and the
CPU baseline leg reports the fields the bench line carries."""

import subprocess
import sys
from pathlib import Path

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
