"""bench.py's contract: one GPU only (any other count is said in one line, exit code 2), one JSON line
with the fields the record needs, a flat `config` of at most 20 keys, and byte and flop counts that
are those of the model's sizes."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_more_than_one_gpu_is_refused_in_one_line():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    lines = [line for line in run.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0] and "--gpus 2" in lines[0]


def test_bytes_and_flops_of_the_record_are_the_models():
    import bench
    cfg = dict(bench.TINYLLAMA)
    h, i, v, layers = 2048, 5632, 32000, 22
    per_layer = (2048 + 2 * 256) * h + h * 2048 + 2 * i * h + h * i + 2 * h          # q/k/v, output, gate and up, down, two norms
    assert bench.weight_bytes_per_step(cfg, 2) == 2 * (layers * per_layer + h + v * h)
    assert bench.kv_bytes_per_token(cfg, 2) == 2 * 4 * 64 * layers * 2                    # keys and values of 4 heads of 64
    # a prompt of T tokens: 2 flops a weight and token (the output head for the one wanted row only), and
    # the causal attention's 4 T^2 d a head over two
    tokens = 2048
    products = 2 * tokens * layers * (per_layer - 2 * h) + 2 * v * h
    attention = layers * 32 * 4 * 64 * tokens * tokens // 2
    got = bench.prefill_flops(cfg, tokens)
    assert abs(got - (products + attention)) <= 0.02 * got, (got, products + attention)


@pytest.mark.gpu
def test_the_record_is_one_flat_json_line():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "4", "--warmup", "2", "--layers", "2",
                          "--context", "256", "--no-points", "--repeats", "1"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [line for line in run.stdout.splitlines() if line.strip()]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 4 and record["warmup"] == 2 and record["higher_is_better"] is True
    assert record["unit"] == "tokens/s" and record["dtype"] == "bf16" and "synthetic" in record["data"]
    assert abs(record["value"] - 8 * 1e3 / record["ms_per_step"]) <= 1e-6 * record["value"]
    config = record["config"]
    assert len(config) <= 20 and all(not isinstance(value, (dict, list)) for value in config.values())
    assert config["layers"] == 2 and config["layers_of_model"] == 22 and config["global_batch"] == 8 and config["seq_len"] == 256
    roofline = record["roofline"]
    assert roofline["bound"] == "hbm" and roofline["unit"] == "GB/s" and roofline["peak"] == 8000.0
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-9
    assert record["library_fallbacks"] == 0
