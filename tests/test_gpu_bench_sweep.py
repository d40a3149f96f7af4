"""bench_sweep.py, the counterpart of the reference's benchmark harness
(simplicial/test_performance.py:409-594): a short run of two of its sweeps must print one JSON line
per point, with times and rates for every shape the library takes and an error record (not a
crash) for the one it rejects, head_dim 512."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_precision_and_head_dim_sweeps_emit_json_lines():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench_sweep.py"), "--sweeps", "precision,head_dim",
                          "--iters", "2"], capture_output=True, text=True, timeout=240)
    assert res.returncode == 0, res.stderr[-2000:]
    points = [json.loads(line) for line in res.stdout.splitlines() if line.strip()]
    assert [p["sweep"] for p in points] == ["head_dim"] * 5 + ["precision"] * 3
    assert [p["D"] for p in points[:5]] == [32, 64, 128, 256, 512]
    assert [p["dtype"] for p in points[5:]] == ["fp16", "bf16", "fp32"]
    for p in points:
        if p["D"] == 512:
            assert "error" in p and "bad shape" in p["error"]          # D <= 256 is the library's limit
            continue
        assert "error" not in p, p
        assert p["fwd_ms"] > 0 and p["bwd_ms"] > 0 and p["fwd_tflops"] > 0 and p["bwd_tflops"] > 0
        assert p["tokens_per_s"] > 0 and p["peak_mem_mb"] > 0
        # every shape of these two sweeps has matrix-pipe kernels: 16-bit head_dim 32 ... 256, fp32 head_dim 64
        assert p["mfma"] is True
