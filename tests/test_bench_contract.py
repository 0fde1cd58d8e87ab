"""bench.py's command-line contract that can be checked without a GPU, and the workload tables
behind its byte counts."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import workloads  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and r.stdout.strip() == ""
    assert "--gpus 1" in r.stderr


def test_workload_sizes_match_the_published_configuration_table():
    base = json.load(open(os.path.join(ROOT, "BASELINE.json")))
    assert len(base["configs"]) == 5
    # chunks and algorithmic bytes of the two benchmarked configurations (1B set, k = 32)
    cfg = workloads.CONFIGS["cfg3_llama1b"]
    assert cfg["k"] == 32 and workloads.chunks_2d(cfg["shapes"]) == 294144
    assert workloads.encode_bytes(cfg["shapes"], 32) == 4871480832
    n = workloads.chunks_2d(cfg["shapes"])
    assert n * (15 * 176 + 16384) == 5595795456
    cfg5 = workloads.CONFIGS["cfg5_72b_block"] if "cfg5_72b_block" in workloads.CONFIGS else None
    if cfg5 is not None:
        assert cfg5["k"] == 64 and workloads.chunks_2d(cfg5["shapes"]) == 214272
