"""bench.py's command-line contract that can be checked without a GPU: more than one GPU is refused with a message,
the workload names exist, and the algorithmic figures of the headline configuration are what the documentation quotes."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)


def test_algorithmic_figures_of_the_headline_configuration():
    sys.path.insert(0, str(ROOT))
    import bench

    fl = bench.algorithmic_flops(bench.CFG)
    routes = 4096 * 8
    assert fl["gate_up"] == 2 * routes * 1024 * 2048 and fl["down"] == 2 * routes * 2048 * 512
    assert fl["base_total"] == 2 * (fl["gate_up"] + fl["down"])
    assert abs(fl["total"] / 1e9 - 430.0) < 0.5                      # GFLOP per step
    assert bench.packed_weight_bytes(bench.CFG) == 256 * (1024 * 2048 + 2048 * 512) * 144 // 256
    ap_help = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--help"], capture_output=True, text=True, timeout=300).stdout
    for name in ("moe_q4k", "dense_q4k", "lmhead_q6k", "moe_iq2xxs", "moe_q4k_separated"):
        assert name in ap_help
