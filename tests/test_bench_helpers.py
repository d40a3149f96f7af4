"""CPU-side checks of bench.py's bookkeeping: the triple count behind every TFLOP/s figure, the
counter values it reads from the tracked rocprofv3 summaries, the literal-loop CPU leg, and its
refusal to run on more than one GPU."""
import os
import subprocess
import sys

import torch

from oracle import simplicial_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_triple_counts_match_the_oracle_and_the_published_figures():
    for name, (B, N, H, D, w1, w2, seed, std) in bench.WORKLOADS.items():
        if N <= 8192:
            assert bench.count_triples(B, N, H, w1, w2) == orc.count_triples(B, N, H, w1, w2), name
    assert bench.count_triples(1, 8192, 16, 512, 32) == 2149480960            # 4*D*T = 1.1005e12 at D = 128
    assert bench.count_triples(2, 2048, 8, 512, 32) == 485292544
    assert bench.count_triples(1, 32768, 8, 1024, 64) == 17192081920


def test_profile_keys_come_from_the_tracked_summaries():
    keys, sources = bench.profile_keys()
    for wl in ("c4", "c2", "c5"):
        assert sources[wl] == "profiles/pmc_counters_%s.md" % wl
        for group in ("forward", "backward_k_side", "backward_kprime_side"):
            busy = keys[(wl, group, "mfma_busy")]
            traffic = keys[(wl, group, "traffic_bytes")]
            assert 0.05 < busy < 1.0, (wl, group, busy)
            assert traffic > 1e7, (wl, group, traffic)
    # HBM traffic is never below the algorithmic bytes of the workload (c4 forward: 201.9 MB)
    assert keys[("c4", "forward", "traffic_bytes")] > 201.9e6
    assert bench.profile_keys()[0].get(("c9", "forward", "mfma_busy")) is None


def test_literal_cpu_leg_reports_iterations_and_extrapolation():
    torch.set_num_threads(min(4, torch.get_num_threads()))
    leg = bench.cpu_reference_literal(134342560, "c4 forward")
    assert leg["iterations"] == 62016 == orc.count_triples(1, 128, 1, 32, 16)     # (B, H) is vectorised
    assert leg["kind"] == "port" and leg["ms"] > 0
    assert abs(leg["us_per_iteration"] * leg["iterations"] / 1e3 - leg["ms"]) < 1e-6 * leg["ms"] + 1e-9
    hours = leg["extrapolated"]["hours_forward"]
    assert abs(hours - leg["us_per_iteration"] * 134342560 / 3.6e9) < 1e-9 * hours + 1e-12
    assert "extrapolation" in leg["extrapolated"]["note"]


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode == 2
    assert "one GPU" in res.stderr and not res.stdout.strip()


def test_board_power_reads_a_number_or_nothing():
    w = bench.board_power_w()
    assert w is None or 0 < w < 5000
    cap = bench.board_power_cap_w()
    assert cap is None or cap > 0
    if w is None:
        assert bench.power_under(lambda: None) is None
