"""bench.py's one line, from a short run on two layers: the keys the contract names, flat configuration, and
figures that follow from one another."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_line_that_bench_prints():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "2", "--steps", "6", "--warmup", "2",
                          "--batch", "3", "--prompt", "200", "--context", "512", "--no-other-models"],
                         capture_output=True, text=True, cwd=ROOT, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [ln for ln in run.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 6 and d["warmup"] == 2 and d["dtype"] == "bf16" and d["higher_is_better"] is True
    cfg = d["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 2 and cfg["layers_full"] == 36 and cfg["global_batch"] == 3 and cfg["seq_len"] == 512
    assert abs(d["value"] - 3 * 1e3 / d["ms_per_step"]) / d["value"] < 0.01          # tokens a second from the step's time
    assert set(d["prefill"]) == {"value", "tokens", "ms", "frac"} and d["prefill"]["tokens"] == 200
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s" and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert {"decode_b1", "decode_b64"} <= set(d["points"])
    assert cfg["launches_per_step"] == 2 * 6 + 4                                      # six kernels a layer and four around them
