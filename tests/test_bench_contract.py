"""The measuring program's contract with whoever runs it: one JSON line with fixed keys on one GPU,
one plain line and exit code 2 for more than one."""
import json
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def run_bench(*args, env=None):
    return subprocess.run([sys.executable, str(ROOT / "bench.py"), *args], capture_output=True, text=True,
                          env={**os.environ, **(env or {})}, cwd=ROOT, timeout=600)


@pytest.mark.parametrize("args,env", [(["--gpus", "2"], {}), ([], {"WORLD_SIZE": "4"})])
def test_more_than_one_gpu_is_refused_in_one_line(args, env):
    p = run_bench(*args, env=env)
    assert p.returncode == 2
    lines = [line for line in p.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


@pytest.mark.gpu
def test_the_line_of_a_short_run_has_every_key():
    p = run_bench("--layers", "2", "--steps", "6", "--warmup", "2")
    assert p.returncode == 0, p.stderr[-2000:]
    line = json.loads(p.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 6 and line["warmup"] == 2 and line["higher_is_better"] is True
    assert line["metric"] == "decode_tokens_per_s" and line["dtype"] == "bf16" and line["value"] > 0
    cfg = line["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 2 and cfg["layers_full"] == 36 and cfg["global_batch"] == 8
    assert set(line["prefill"]) == {"value", "tokens", "ms", "frac"} and line["prefill"]["tokens"] == 2048
    assert line["roofline"]["bound"] == "hbm" and line["roofline"]["peak"] == 8000.0 and line["roofline"]["unit"] == "GB/s"
    assert abs(line["roofline"]["frac"] - line["roofline"]["achieved"] / 8000.0) < 1e-3
    assert set(line["points"]) == {"decode_b1", "decode_b64", "decode_b8_ctx8k"}
    assert all(isinstance(v, float) and v > 0 for v in line["points"].values())
    for name, d in line["points_detail"].items():
        assert set(d) == {"tok_s", "ms_per_step", "batch", "mean_context", "gb_read", "frac"} and d["tok_s"] == line["points"][name]
        assert abs(d["frac"] - d["gb_read"] / (d["ms_per_step"] * 1e-3) / 8000.0) < 2e-3
    assert line["points_detail"]["decode_b8_ctx8k"]["mean_context"] > 7900
    assert "median of 3" in line["data"]
    cal = line["calibration"]
    assert 0 < cal["hbm_read_gbs"] < 8000 and 0 < cal["mfma_bf16_tflops"] < 2500       # what the box reaches lies below the published peaks
    for phase in ("decode", "prefill"):
        shares = line["kernel_share"][phase]
        assert abs(sum(shares.values()) - 1.0) < 0.01 and shares.get("attention", 0) > 0
        assert shares.get("products_own", 0) + shares.get("products_library", 0) > 0.4
    assert abs(line["value"] - 8 / (line["ms_per_step"] * 1e-3)) < 0.01 * line["value"]
