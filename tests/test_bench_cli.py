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


def _fake_result(bench, name, with_cpu=True):
    """A record shaped like bench.run_config's, with long numbers and the longest texts the real ones carry."""
    if name in bench.LAYER_STEPS:
        ls = bench.LAYER_STEPS[name]
        c = dict(kind=ls["kind"], B=ls["B"], H=ls["H"], Hkv=ls["Hkv"], Sq=ls["n"], Skv=ls["start"] + ls["n"], D=ls["D"],
                 dtype=ls["dtype"], causal=True)
    else:
        c = bench.configs()[name]
    decode = c["kind"] in ("decode", "layer_decode", "layer_prompt")
    roof = dict(bound="hbm" if decode else "mfma", achieved=5912.123456789, peak=8000.0, unit="GB/s" if decode else "TFLOP/s",
                frac=0.7390154320987, traffic=270342052.36343193,
                traffic_note="FETCH_SIZE 2.692e+08 B + WRITE_SIZE 1.114e+06 B per launch", kernel="decode_splitkv",
                kernel_ms_mean=0.045456789012, kernel_ms_median=0.0454123456, kernel_ms_min=0.0441234567)
    res = dict(value=5517.123456789012, unit=roof["unit"], ms_per_step=0.04870123456789, roofline=roof,
               config=dict(workload=name, kind=c["kind"], batch=c["B"], q_heads=c["H"], kv_heads=c["Hkv"], q_len=c["Sq"],
                           kv_len=c["Skv"], head_dim=c["D"], causal=c["causal"], q_pos_offset=c.get("q_pos_offset"),
                           window=c.get("window"), ragged_lens=c.get("ragged"), kv_sets_rotated=5,
                           algorithmic_flops=549_822_922_752, algorithmic_bytes=5_967_384_576),
               dtype=c["dtype"], frac_of_roofline=0.689640432098765, spot_check_max_abs_err=0.0001220703125)
    if with_cpu:
        res["cpu_baseline"] = dict(value=10.123456789012, unit=roof["unit"], cores=16, kind="port",
                                   sample="the full step (all 16 sequences), f16 upcast to f32 first, median of 3 passes after "
                                          "one warm-up pass, and some more words that a sample description might carry")
    return res


def test_the_last_line_stays_short_enough_for_a_log_tail_and_keeps_the_prefill_half():
    """The driver's record keeps the tail of stdout: the final line carries both halves of the metric (C2 decode, C3
    prefill under "prefill") with roofline and cpu_baseline each, and one short entry per other workload, in under 4 KB."""
    import json
    sys.path.insert(0, ROOT)
    import bench
    main = _fake_result(bench, "C2")
    pre = _fake_result(bench, "C3")
    others = {name: _fake_result(bench, name, cpu) for name, (_, _, cpu) in bench.EXTRA_WORKLOADS.items()}
    cal = [dict(dtype="f16", operands="random", duty_percent=100, tflops=1571.123456789, ms=160.123456, sclk_ghz_median=1.58123456,
                sclk_ghz_min=1.5012345, sclk_ghz_max=1.73123456)]
    read_cal = dict(mib_per_launch=256, slices_rotated=5, launches=60, us_per_launch=40.3123456, gbps=6658.123456, frac_of_peak=0.83226)
    line = bench.final_line(main, 100, 10, read_cal, pre, cal, others)
    text = json.dumps(line)
    assert len(text) < 4096, len(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "prefill", "configs"):
        assert key in line, key
    for half in (line, line["prefill"]):
        assert {"bound", "achieved", "peak", "unit", "frac", "traffic"} <= set(half["roofline"])
        assert {"value", "unit", "cores", "kind", "sample"} <= set(half["cpu_baseline"])
    assert line["config"]["workload"] == "C2" and line["prefill"]["config"]["workload"] == "C3"
    assert line["prefill"]["mfma_calibration"]["duty_percent"] == 100
    assert set(line["configs"]) == set(bench.EXTRA_WORKLOADS)
