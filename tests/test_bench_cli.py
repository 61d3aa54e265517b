"""CPU checks of bench.py's command line: the workloads it knows and what it says to a request for several GPUs."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       cwd=ROOT, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_workloads_and_their_algorithmic_counts():
    sys.path.insert(0, ROOT)
    import bench
    cfg = bench.configs()
    for name in ("C1", "C2", "C3", "C4", "C5"):
        assert name in cfg
    # the counts the configurations are defined by: visible pairs only for FLOPs, K/V once per KV head for bytes
    assert bench.algorithmic(cfg["C1"]) == (1_075_838_976, 10_485_760)
    assert bench.algorithmic(cfg["C2"]) == (1_073_741_824, 268_697_600)
    assert bench.algorithmic(cfg["C3"]) == (549_822_922_752, 167_772_160)
    assert bench.algorithmic(cfg["C4"]) == (128_865_796_096, 100_663_296)
    assert bench.algorithmic(cfg["C4B"])[0] == 137_438_953_472
    assert bench.visible_pairs(cfg["C4"]) == 4 * 1_966_336
