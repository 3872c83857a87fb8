"""The measurement script's contract: one JSON line with the agreed keys; more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=timeout)


def test_more_than_one_gpu_is_refused():
    proc = run_bench("--gpus", "2")
    assert proc.returncode == 2
    assert len(proc.stdout.strip().splitlines()) == 1 and "one GPU" in proc.stdout


@pytest.mark.gpu
def test_decode_record_has_the_agreed_keys():
    proc = run_bench("--layers", "2", "--steps", "4", "--warmup", "2", "--context", "256", "--batch", "2")
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "points", "prefill"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 4 and rec["warmup"] == 2 and rec["value"] > 0
    config = rec["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 2 and config["layers_of_model"] == 36 and config["global_batch"] == 2
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["peak"] == 8000.0
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / 8000.0) < 1e-3
    assert {"decode_b1", "decode_b64", "decode_b16", "decode_b32", "decode_b2_ctx1024", "prefill_8192", "prefill_128",
            "prefill_512", "f32_decode_b2_layers2", "f32_prefill_2048_layers2"} <= set(rec["points"])
    # eager steps: the wall time beside the kernels' own
    for step in rec["eager_steps"].values():
        assert step["wall_ms"] > 0 and step["graph_ms"] > 0 and step["kernel_calls"] > 0 and 0 <= step["host_frac"] < 1
    assert all(isinstance(v, (int, float)) and v > 0 for v in rec["points"].values())
    # (every decode point has its share of the memory's peak under its own name, every prompt its share of the matrix peak)
    assert set(rec["points"]) <= set(rec["points_hbm_frac"]) | {"prefill_8192", "prefill_128", "prefill_512", "f32_prefill_2048_layers2",
                                                                  "shape0.6B_prefill_128", "shape0.6B_prefill_512"}
    assert {"shape0.6B_decode_b1_ctx2048", "shape0.6B_decode_b8_ctx2048", "shape0.6B_prefill_128_mfma"} <= set(rec["points_hbm_frac"])
    assert rec["prefill"]["tokens"] == 2048 and rec["prefill"]["value"] > 0 and 0 < rec["prefill"]["frac"] < 1
    # mean and deviation over five repetitions, for decode and prefill
    assert rec["decode_runs"]["runs"] == 5 and rec["decode_runs"]["ms_per_step_mean"] > 0 and rec["decode_runs"]["ms_per_step_std"] >= 0
    assert rec["prefill"]["runs"] == 5 and rec["prefill"]["ms_std"] >= 0 and rec["prefill"]["ms_best"] <= rec["prefill"]["ms"]
    assert rec["prefill"]["first_token_ms"] > 0
    # fractions of the measured roofs beside those of the published peaks
    roof = rec["roofline"]
    assert 1000 < roof["measured_peak"] < 8000.0 and abs(roof["frac_of_measured"] - roof["achieved"] / roof["measured_peak"]) < 1e-3
    assert 100 < rec["prefill"]["measured_peak_tflops"] < 2500 and rec["prefill"]["frac_of_measured"] > rec["prefill"]["frac"]
    # microseconds by kernel for one decode step and one prefill
    for phase in ("decode", "prefill"):
        table = rec["kernels"][phase]
        assert table and all(v["calls"] > 0 and v["us"] > 0 for v in table.values())
    assert "gemm_skinny_stream" in rec["kernels"]["decode"] and "attention_mfma" in rec["kernels"]["prefill"]


@pytest.mark.gpu
def test_workload_record():
    proc = run_bench("--workload", "mixed16", "--shape", "8B", "--layers", "1", "--decode-tokens", "4", "--steps", "1")
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().splitlines()[-1])
    assert rec["config"]["requests"] == 16 and rec["config"]["decode_tokens"] == 4 and rec["value"] > 0
    assert rec["first_token_s"]["max"] >= rec["first_token_s"]["mean"] > 0
    assert rec["prompt_phase"]["prompt_tok_s"] > 0 and rec["decode_phase"]["tok_s"] > 0
