#!/usr/bin/env python3
"""Benchmark of the 2-simplicial attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c2|c5|c1|c2f32]

A step is one forward + backward pass of the operator over one batch of
synthetic input that is already resident in HBM (iid normal, seeded, bf16).
The default workload is the headline configuration: bf16, B=1 H=16 N=8192 D=128,
w1=512 w2=32.  Workloads c1 (fp32 B=1 H=2 N=128 D=64 w 32/16, the forward-only plumbing
configuration) and c2f32 (fp32 tensors at the shape of c2) run on the fp32 MFMA kernels and are
priced against the fp32 matrix peak.  Prints ONE JSON line:

  metric/value   forward+backward algorithmic TFLOP/s: 16*D*T flops per step,
                 T = number of valid (i,j,k) triples (matmul flops only, 2 per
                 MAC: 4*D*T forward, 12*D*T backward)
  roofline       the kernel group that takes the longest in the step (whichever of the
                 forward, the K-side and the K'-side backward measures longest in this
                 run), against the bf16 dense MFMA peak (achieved = that group's
                 algorithmic flops / its duration, measured here with events on the
                 launch stream); `groups` lists all three; `mfma_busy` and
                 `traffic` are rocprofv3 counter results read from profiles/
                 (measured in separate profiler runs of this same script)
  kernels        the same for every kernel group of the step, plus HBM GB/s
  clock          shader clock observed while the kernels run (a spin kernel on a
                 second stream counts device cycles between two events) and the
                 peak recomputed from it: CUs x 4096 flop/clk x clock
  cpu_baseline   the CPU oracle (a port of the reference's PyTorch loop) timed on
                 this host on a bounded sample of the same workload
  cpu_reference_literal   the literal triple loop of the reference (reference.py:39-74,
                 restated in oracle/) timed at configuration c1, with its cost per
                 loop iteration and the extrapolation to this workload
"""
import argparse
import glob
import json
import math
import os
import re
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6     # published: 256 CU x 2.4 GHz x 4096 flop/clk/CU, dense
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
BF16_FLOP_PER_CLK_PER_CU = 4096

WORKLOADS = {
    # name: (B, N, H, D, w1, w2, seed, qk_std)
    "c1": (1, 128, 2, 64, 32, 16, 0, 1.0),
    "c2": (2, 2048, 8, 64, 512, 32, 1, 1.0),
    "c4": (1, 8192, 16, 128, 512, 32, 3, 1.0),
    "c5": (1, 32768, 8, 128, 1024, 64, 4, 0.5),
    "c2f32": (2, 2048, 8, 64, 512, 32, 1, 1.0),
}
FP32_WORKLOADS = ("c1", "c2f32")


def profile_keys():
    """Counter results of the tracked rocprofv3 summaries: every line of profiles/*.md of the form
    `<workload>.<kernel group>.<quantity> = <number>` (HBM bytes per launch from FETCH_SIZE and
    WRITE_SIZE scaled by a copy kernel; matrix-pipe busy fraction from SQ_VALU_MFMA_BUSY_CYCLES).
    They are measured under the profiler, not in this run: a key that is missing reads as None."""
    keys, sources = {}, {}
    pat = re.compile(r"^([a-z0-9]+)\.([a-z_]+)\.([a-z_]+) = ([-+0-9.eE]+)\s*$")
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        for line in open(path):
            m = pat.match(line.strip())
            if m:
                keys[(m.group(1), m.group(2), m.group(3))] = float(m.group(4))
                sources[m.group(1)] = os.path.relpath(path, ROOT)
    return keys, sources


def count_triples(B, N, H, w1, w2):
    return B * H * sum((min(i, w1) + 1) * (min(i, w2) + 1) for i in range(N))


def make_inputs(B, N, H, D, seed, qk_std, device, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    out = []
    for t in range(6):
        x = torch.randn(B, N, H, D, generator=g, dtype=torch.float32)
        if t < 3:
            x = x * qk_std
        out.append(x.to(dtype).to(device))
    return out


def time_gpu(fn, steps, warmup):
    """Average milliseconds per call, events on the current (launch) stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def observed_clock_mhz(fn, ms_per_call, spin_ms=60.0):
    """Shader clock while `fn` keeps the GPU busy: a one-thread spin kernel on a second stream
    waits for a given number of ticks of the device's cycle counter between two events, and
    calls of `fn` queued right behind it on the launch stream run for its whole duration.  The
    spin is launched on an idle (but just warmed) GPU so that it starts at once and the events
    bracket exactly its ticks.  (The spinning wavefront takes one CU's slot for its duration;
    this is a measurement of its own, outside the timed region.)"""
    side = torch.cuda.Stream()
    cycles = int(2.4e6 * spin_ms)                      # lasts about `spin_ms` at 2.4 GHz
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        e0.record()
        torch.cuda._sleep(cycles)
        e1.record()
    for _ in range(int(math.ceil(1.4 * spin_ms / ms_per_call)) + 2):
        fn()
    torch.cuda.synchronize()
    return cycles / e0.elapsed_time(e1) / 1e3


def library_gemm_tflops(device, m=8192, iters=20):
    """What the vendor's bf16 GEMM (torch.matmul -> hipBLASLt) reaches on this device on N(0,1) operands and
    on zeros, m x m x m: the matrix pipes draw more power on random operands than on quiet ones and the chip
    slows down, so the published peak is out of reach for any kernel on the bench's data.  Context for the
    roofline fractions, not a target and not part of the timed step."""
    res = {}
    c = torch.empty(m, m, device=device, dtype=torch.bfloat16)
    for kind in ("zeros", "n01"):
        a = torch.zeros(m, m, device=device, dtype=torch.bfloat16)
        b = torch.zeros(m, m, device=device, dtype=torch.bfloat16)
        if kind == "n01":
            a.normal_()
            b.normal_()
        ms = time_gpu(lambda: torch.matmul(a, b.t(), out=c), iters, 5)
        res[kind] = 2.0 * m ** 3 / ms / 1e9
        pw = power_under(lambda: torch.matmul(a, b.t(), out=c), 0.6)
        if pw is not None:
            pw["pj_per_flop"] = pw["joules_per_call"] / (2.0 * m ** 3) * 1e12
        res[kind + "_power"] = pw
    return res


POWER_GLOB = "/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"


def board_power_w():
    """Board power in watts from the amdgpu hwmon node of the first card (None where it cannot be read)."""
    import glob
    for path in sorted(glob.glob(POWER_GLOB)):
        try:
            with open(path) as f:
                return int(f.read()) / 1e6
        except (OSError, ValueError):
            continue
    return None


def board_power_cap_w():
    import glob
    for path in sorted(glob.glob(POWER_GLOB.replace("power1_input", "power1_cap"))):
        try:
            with open(path) as f:
                return int(f.read()) / 1e6
        except (OSError, ValueError):
            continue
    return None


def power_under(fn, seconds=0.8):
    """Average board power while `fn` runs back to back for `seconds` (sampled between batches of
    calls during the second half), with the average duration of a call in that loop."""
    if board_power_w() is None:
        return None
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    calls, samples = 0, []
    while True:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        calls += 10
        elapsed = time.perf_counter() - t0
        if elapsed > 0.5 * seconds:
            samples.append(board_power_w())
        if elapsed > seconds:
            break
    watts = sum(samples) / len(samples)
    ms = elapsed / calls * 1e3
    return {"watts": watts, "ms_per_call": ms, "joules_per_call": watts * ms * 1e-3}


def cpu_reference_literal(target_iterations, target_name):
    """The reference's literal triple loop (queries x K keys x K' keys, one weight at a time;
    simplicial/reference.py:39-74 as restated in oracle/) at configuration c1, the only one it
    finishes in seconds, and its per-iteration cost extrapolated by iteration count."""
    from oracle import simplicial_oracle as orc
    B, N, H, D, w1, w2 = 1, 128, 2, 64, 32, 16
    g = torch.Generator().manual_seed(0)
    tens = [torch.randn(B, N, H, D, generator=g, dtype=torch.float32) for _ in range(5)]
    iterations = sum((min(i, w1) + 1) * (min(i, w2) + 1) for i in range(N))     # (B, H) is vectorised
    t0 = time.perf_counter()
    orc.literal_loop(*tens, w1, w2)
    dt = time.perf_counter() - t0
    return {
        "workload": "c1: fp32 forward B=1 H=2 N=128 D=64 w1=32 w2=16", "kind": "port", "ms": dt * 1e3,
        "iterations": iterations, "us_per_iteration": dt / iterations * 1e6, "cores": torch.get_num_threads(),
        "extrapolated": {"workload": target_name, "iterations": target_iterations,
                         "hours_forward": dt / iterations * target_iterations / 3600.0,
                         "note": "per-iteration cost at c1 x iteration count; an extrapolation, not a measurement "
                                 "(the loop's tensors grow with B*H*D, so this is a lower bound)"},
    }


def cpu_baseline(name, cfg, budget_rows, fp32=False):
    """Times the CPU oracle forward + autograd on `budget_rows` steady-state
    query rows of the workload (all batches and heads) and scales by the triple
    count.  Returns the JSON object."""
    from oracle import simplicial_oracle as orc
    B, N, H, D, w1, w2, seed, qk_std = cfg
    g = torch.Generator().manual_seed(seed)
    tens = []
    for t in range(6):
        x = torch.randn(B, N, H, D, generator=g, dtype=torch.float32)
        if t < 3:
            x = x * qk_std
        tens.append(x if fp32 else x.to(torch.bfloat16).float())
    budget_rows = min(budget_rows, N)
    r0 = min(N - budget_rows, max(w1, w2) + 64)
    r0 = max(r0, 0)
    r1 = min(N, r0 + budget_rows)
    t0 = time.perf_counter()
    orc.grads_windowed(*tens[:5], tens[5][:, r0:r1], w1, w2, rows=(r0, r1), chunk=16, compute_dtype=torch.float32)
    dt = time.perf_counter() - t0
    t_rows = B * H * sum((min(i, w1) + 1) * (min(i, w2) + 1) for i in range(r0, r1))
    flops = 16.0 * D * t_rows
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": "oracle forward+autograd (fp32, vectorised restatement of reference.py) on query rows "
                  "[%d,%d) of workload %s, all %d heads; %.1f s; scaled by triple count" % (r0, r1, name, B * H, dt),
        "seconds": dt, "host_cpus": os.cpu_count(),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=2560)
    ap.add_argument("--counters-only", action="store_true",
                    help="for rocprofv3 --pmc runs: one 1 GiB device copy (the counter calibration), then two "
                         "forward and two backward calls of the workload; prints no JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (heads are independent and would "
              "shard with no communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    import simplical_attn_amd as sa
    from simplical_attn_amd import _lib
    lib = _lib.load()

    cfg = WORKLOADS[args.workload]
    B, N, H, D, w1, w2, seed, qk_std = cfg
    fp32 = args.workload in FP32_WORKLOADS
    dtype_name, code = ("fp32", _lib.SA2_F32) if fp32 else ("bf16", _lib.SA2_BF16)
    # published dense matrix peak of the arithmetic type the kernels compute in
    PEAK_TFLOPS = PEAK_FP32_TFLOPS if fp32 else PEAK_BF16_TFLOPS
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(0)
    q, k1, k2, v1, v2, dout = make_inputs(B, N, H, D, seed, qk_std, dev, torch.float32 if fp32 else torch.bfloat16)
    T = count_triples(B, N, H, w1, w2)
    fwd_flops, bwd_flops = 4.0 * D * T, 12.0 * D * T
    E = B * N * H * D
    esz = 4 if fp32 else 2
    fwd_bytes = 6 * E * esz + 4 * B * H * N                # read q,k1,k2,v1,v2; write O, LSE
    bwd_bytes = 12 * E * esz + 12 * B * H * N              # read 5 inputs, O, dO; write 5 grads; LSE, D

    if args.counters_only:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)                                   # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        for _ in range(2):
            out, lse = sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2)
            sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2)
        torch.cuda.synchronize()
        return

    leaves = [t.clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    attn = sa.TwoSimplicialAttention(D, w1, w2)

    def step():
        for t in leaves:
            t.grad = None
        out = attn(*leaves)
        out.backward(dout)

    # ---- the timed region: K full steps --------------------------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = e0.elapsed_time(e1) / args.steps

    # ---- the forward's and the backward's share of a step (events inside further steps) ----
    # Back-to-back forwards draw more power than the step's mix; on some boxes the forward runs up
    # to 5 % faster between two backwards than in a loop of its own.  Both figures are reported.
    marks = []
    for _ in range(max(5, args.steps)):
        for t in leaves:
            t.grad = None
        m = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        m[0].record()
        o = attn(*leaves)
        m[1].record()
        o.backward(dout)
        m[2].record()
        marks.append(m)
    torch.cuda.synchronize()
    fwd_in_step_ms = sum(m[0].elapsed_time(m[1]) for m in marks) / len(marks)
    bwd_in_step_ms = sum(m[1].elapsed_time(m[2]) for m in marks) / len(marks)

    # ---- per-kernel-group durations (same stream, events) -------------------
    out, lse = sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2)
    ksteps = max(5, args.steps)
    fwd_ms = time_gpu(lambda: sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2), ksteps, 2)
    rowdot_ms = time_gpu(lambda: sa.simplicial_rowdot(dout, out), ksteps, 2)
    bwd_all_ms = time_gpu(lambda: sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2), ksteps, 2)
    bwd_k1_ms = time_gpu(lambda: sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2,
                                                        needs=(False, True, False, True, False)), ksteps, 2) - rowdot_ms
    bwd_rest_ms = time_gpu(lambda: sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2,
                                                          needs=(True, False, True, False, True)), ksteps, 2) - rowdot_ms
    mfma = bool(lib.sa2_uses_mfma(B, N, H, D, w1, w2, code))
    # Algorithmic flops per launch: forward 4*D*T; the backward's 12*D*T split evenly between its
    # two MFMA kernels (each owns two output contractions, 4*D*T, and half of the S / dP
    # recomputation that the pair shares, 2*D*T).
    half_bwd = bwd_flops / 2
    keys, key_sources = profile_keys()
    wl = args.workload
    if fp32:
        labels = ("f32_fwd_kernel<%d> (v_mfma_f32_32x32x2_f32)" % D, 1, "f32_bwd_kv_kernel<%d> (dK, dV)" % D, 1,
                  "f32_bwd_kp_kernel<%d> + f32_dq_sum_kernel (dQ, dK', dV')" % D, 2)
    else:
        labels = ("mfma_fwd_kernel<%d> (pre-pass + fast kernel + repair launch)" % D, 3, "mfma_bwd_kv_kernel<%d> (dK, dV)" % D, 1,
                  "mfma_bwd_kp_kernel<%d> (pre-pass + main) + dq_sum (dQ, dK', dV')" % D, 3)
    kernels = {
        "forward": {"kernel": labels[0], "ms": fwd_ms, "flops": fwd_flops, "launches": labels[1]},
        "backward_k_side": {"kernel": labels[2], "ms": bwd_k1_ms, "flops": half_bwd, "launches": labels[3]},
        "backward_kprime_side": {"kernel": labels[4], "ms": bwd_rest_ms, "flops": half_bwd, "launches": labels[5]},
    }
    for name, k in kernels.items():
        k["tflops"] = k["flops"] / k["ms"] / 1e9
        k["frac_bf16_peak"] = k["tflops"] / PEAK_TFLOPS              # (of the fp32 matrix peak for the fp32 workloads)
        k["mfma_busy"] = keys.get((wl, name, "mfma_busy"))          # rocprofv3, from profiles/
        k["traffic"] = keys.get((wl, name, "traffic_bytes"))
    kernels["forward"]["hbm_gbs"] = fwd_bytes / fwd_ms / 1e6
    kernels["forward"]["ms_in_step"] = fwd_in_step_ms
    kernels["forward"]["frac_bf16_peak_in_step"] = fwd_flops / fwd_in_step_ms / 1e9 / PEAK_TFLOPS
    kernels["backward"] = {"ms": bwd_all_ms, "tflops": bwd_flops / bwd_all_ms / 1e9, "hbm_gbs": bwd_bytes / bwd_all_ms / 1e6,
                           "frac_bf16_peak": bwd_flops / bwd_all_ms / 1e9 / PEAK_TFLOPS}
    kernels["backward"]["ms_in_step"] = bwd_in_step_ms
    kernels["rowdot"] = {"ms": rowdot_ms, "hbm_gbs": (4 * E + 4 * B * H * N) / rowdot_ms / 1e6}

    # ---- shader clock while the kernels run, and the peak it implies -------------------
    bwd_call = lambda: sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2)
    fwd_call = lambda: sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2)
    clocks = {}
    for cname, call, ms_call in (("forward", fwd_call, fwd_ms), ("backward", bwd_call, bwd_all_ms), ("step", step, ms_per_step)):
        clocks[cname] = observed_clock_mhz(call, ms_call)
    cus = props.multi_processor_count
    flop_per_clk_per_cu = int(round(BF16_FLOP_PER_CLK_PER_CU * PEAK_TFLOPS / PEAK_BF16_TFLOPS))      # 4096 bf16, 256 fp32
    peak_at = lambda mhz: cus * flop_per_clk_per_cu * mhz * 1e6 / 1e12
    clock = {"mhz": clocks, "method": "device cycle counter (60 ms spin kernel on a second stream) / event time",
             "peak_bf16_tflops_at_observed_clock": {k: peak_at(v) for k, v in clocks.items()},
             "published_peak_bf16_tflops": PEAK_TFLOPS,
             "published_peak_is": "%d CU x 2400 MHz x %d flop/clk/CU (%s matrix)" % (cus, flop_per_clk_per_cu, dtype_name)}
    kernels["forward"]["frac_at_observed_clock"] = kernels["forward"]["tflops"] / peak_at(clocks["forward"])
    for name in ("backward_k_side", "backward_kprime_side", "backward"):
        kernels[name]["frac_at_observed_clock"] = kernels[name]["tflops"] / peak_at(clocks["backward"])

    # The dominant kernel group: the one that takes the longest in the step.  The K-side kernel is a
    # single launch (its duration here: the call that requests only dK and dV, minus the row-dot
    # kernel); the forward and the K'-side group hold three launches each (a pre-pass and a short
    # epilogue kernel beside the main one), of which the main kernel is more than nine tenths.
    dominant = max(("forward", "backward_k_side", "backward_kprime_side"), key=lambda k: kernels[k]["ms"])
    roofline = {
        "bound": "mfma", "kernel": kernels[dominant]["kernel"], "group": dominant,
        "launches": kernels[dominant]["launches"],
        "achieved": kernels[dominant]["tflops"], "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": kernels[dominant]["frac_bf16_peak"],
        "traffic": kernels[dominant]["traffic"],
        "algorithmic_flops_per_launch": kernels[dominant]["flops"],
        "avg_ms": kernels[dominant]["ms"],
        "mfma_busy": kernels[dominant]["mfma_busy"],
        "frac_at_observed_clock": kernels[dominant]["frac_at_observed_clock"],
        "counters_from": key_sources.get(wl),
        "groups": {k: {"ms": kernels[k]["ms"], "frac": kernels[k]["frac_bf16_peak"]}
                   for k in ("forward", "backward_k_side", "backward_kprime_side")},
    }
    roofline_fwd = {
        "bound": "mfma", "kernel": kernels["forward"]["kernel"], "achieved": kernels["forward"]["tflops"],
        "peak": PEAK_TFLOPS, "unit": "TFLOP/s", "frac": kernels["forward"]["frac_bf16_peak"],
        "frac_at_observed_clock": kernels["forward"]["frac_at_observed_clock"],
        "mfma_busy": kernels["forward"]["mfma_busy"], "traffic": kernels["forward"]["traffic"],
        "counters_from": key_sources.get(wl),
        "hbm_gbs": kernels["forward"]["hbm_gbs"], "hbm_frac": kernels["forward"]["hbm_gbs"] / PEAK_HBM_GBS,
        "avg_ms": fwd_ms, "ms_in_step": fwd_in_step_ms,
        "frac_in_step": kernels["forward"]["frac_bf16_peak_in_step"],
    }

    # ---- board power: these kernels run at the board's power limit on N(0,1) data ----------
    idle_w = board_power_w()
    power = None
    if idle_w is not None:
        power = {"source": POWER_GLOB, "cap_w": board_power_cap_w(),
                 "step": power_under(step), "forward": power_under(fwd_call), "backward": power_under(bwd_call)}
        power["forward"]["pj_per_algorithmic_flop"] = power["forward"]["joules_per_call"] / fwd_flops * 1e12
        power["backward"]["pj_per_algorithmic_flop"] = power["backward"]["joules_per_call"] / bwd_flops * 1e12
        power["step"]["pj_per_algorithmic_flop"] = power["step"]["joules_per_call"] / (fwd_flops + bwd_flops) * 1e12
    gemm = library_gemm_tflops(dev)
    clock["library_gemm_bf16_tflops"] = {
        "shape": "8192^3, torch.matmul", "n01_operands": gemm["n01"], "zero_operands": gemm["zeros"],
        "n01_frac_of_published_peak": gemm["n01"] / PEAK_BF16_TFLOPS,
        "n01_power": gemm["n01_power"], "zero_power": gemm["zeros_power"]}
    roofline["frac_of_library_gemm_on_n01"] = roofline["achieved"] / gemm["n01"]
    roofline_fwd["frac_of_library_gemm_on_n01"] = roofline_fwd["achieved"] / gemm["n01"]

    line = {
        "metric": "fwd+bwd TFLOP/s & %% %s MFMA peak, N=%d D=%d w1=%d w2=%d" % (dtype_name, N, D, w1, w2),
        "value": (fwd_flops + bwd_flops) / ms_per_step / 1e9,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "wall_ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype_name, "data": "synthetic",
        "config": {"workload": "%s: %s fwd+bwd B=%d H=%d N=%d D=%d w1=%d w2=%d scale=1/sqrt(D)" % (
                       args.workload, dtype_name, B, H, N, D, w1, w2),
                   "triples": T, "flops_fwd": fwd_flops, "flops_bwd": bwd_flops,
                   "mfma_kernels": mfma, "device": props.name, "cus": cus,
                   "clock_mhz": clocks["step"]},
        "frac_bf16_peak": (fwd_flops + bwd_flops) / ms_per_step / 1e9 / PEAK_TFLOPS,
        "peak_tflops": PEAK_TFLOPS,
        "frac_bf16_peak_at_observed_clock": (fwd_flops + bwd_flops) / ms_per_step / 1e9 / peak_at(clocks["step"]),
        "clock": clock,
        "power": power,
        "roofline": roofline,
        "roofline_forward": roofline_fwd,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.workload, cfg, args.cpu_rows, fp32)
        line["cpu_reference_literal"] = cpu_reference_literal(T // (B * H), "%s forward" % args.workload)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
