"""bench.py's command line and the one JSON line it prints (the fields a driver reads), on the default workload and on
the prefill workload; more than one GPU is refused with a message."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")
COMMON = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
          "vs_baseline", "dtype", "data", "config", "roofline")
ROOFLINE = ("bound", "achieved", "peak", "unit", "frac", "traffic")


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr + r.stdout


def run(args):
    r = subprocess.run([sys.executable, BENCH] + args, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "bench.py prints exactly one line"
    return json.loads(lines[0])


@pytest.mark.gpu
def test_decode_line_has_the_fields_a_driver_reads():
    d = run(["--steps", "3", "--warmup", "1"])
    for k in COMMON + ("cpu_baseline",):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["unit"] == "GB/s" and d["dtype"] == "u8" and d["vs_baseline"] is None
    assert d["config"]["workload"] == "ragged_b64_q8_0" and "model" not in d["config"]
    for k in ROOFLINE:
        assert k in d["roofline"], k
    assert d["roofline"]["bound"] == "hbm" and d["roofline"]["peak"] == 8000.0
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / d["roofline"]["peak"]) < 1e-3
    # whole-step throughput = algorithmic bytes / step time
    assert abs(d["value"] - d["kv_bytes_per_step"] / (d["ms_per_step"] * 1e-3) / 1e9) < 0.01 * d["value"]
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in d["cpu_baseline"], k
    assert d["cpu_baseline"]["kind"] in ("port", "reference") and d["cpu_baseline"]["cores"] >= 1
    assert d["parity_max_rel_err"] < 2e-3
    # the other configurations that fill a GPU are timed by the same run, into one object of the same line
    assert sorted(d["also"]) == ["b16_ctx128k_q4_0", "b1_ctx32k_q8_0", "prefill_b8_ctx16k_chunk2k_q4_0",
                                 "prefill_b8_ctx16k_chunk2k_q8_0", "ragged_b64_f16", "ragged_b64_kv4a16", "ragged_b64_kv8a16"]
    for name, r in d["also"].items():
        assert r["value"] > 0 and r["ms_per_step"] > 0 and r["parity_max_rel_err"] < 2e-3, name
        assert 0.0 < r["roofline"]["frac"] < 1.0 and r["roofline"]["bound"] == ("mfma" if "prefill" in name else "hbm")
    # the decode workloads also say what their steps cost right after an idle period (an extra figure)
    assert d["after_idle"]["ms_per_step"] > 0 and d["also"]["b16_ctx128k_q4_0"]["after_idle"]["ms_per_step"] > 0
    assert "config1_tiny" in d["cpu_baseline"]["configs"] and "config2_b1_ctx32k" in d["cpu_baseline"]["configs"]


@pytest.mark.gpu
def test_prefill_line():
    d = run(["--workload", "prefill_b8_ctx16k_chunk2k_q8_0", "--steps", "2", "--warmup", "1", "--no-cpu-baseline"])
    for k in COMMON + ("append",):
        assert k in d, k
    assert d["unit"] == "TFLOP/s" and d["roofline"]["bound"] == "mfma" and d["roofline"]["peak"] == 2500.0
    assert d["dtype"] == "f16" and d["parity_max_rel_err"] < 2e-3
    assert 0.0 < d["roofline"]["frac"] < 1.0 and 0.0 < d["append"]["frac_of_hbm_peak"] < 1.0


@pytest.mark.gpu
def test_clock_trace_and_step_options():
    """--clock-trace adds the launch-by-launch durations with the shader clock after each and the clock under load; the
    step's other forms (--separate-append, --graph-replay) give a line of the same shape."""
    d = run(["--workload", "b1_ctx32k_q8_0", "--steps", "4", "--warmup", "1", "--no-cpu-baseline", "--clock-trace",
             "--graph-replay", "--separate-append"])
    ct = d["clock_trace"]
    assert len(ct["kernel_ms"]) == len(ct["shader_mhz"]) == 60
    assert all(300 < m < 3500 for m in ct["shader_mhz"]) and 300 < ct["under_load"]["shader_mhz_median"] < 3500
    assert d["graph_replay"]["ms_per_step"] > 0 and "append, part, reduce" in d["config"]["step"]
    assert d["roofline"]["kernel"] == "DattnPartWhole"   # a batch of one: whole tiles, one partial per workgroup
