#!/usr/bin/env python3
"""Scaling sweeps of the 2-simplicial attention operator on one MI355X.

    python bench_sweep.py [--sweeps seq,batch,heads,head_dim,window,precision,memory,sdpa,long] [--iters K]

Counterpart of the reference's benchmark harness (simplicial/test_performance.py:
scaling sweeps 409-482, precision 484-500, memory 502-542, comparison with ordinary
attention 544-594), with the same base shapes, plus a `long` sweep at production
shapes (bf16, H=16, D=128, w1=512, w2=32, N up to 65536).  Forward and backward are
timed separately with events on the launch stream (the reference's harness times the
backward as forward+backward and then adds the forward again; that is not
reproduced).  One JSON line per measured point:

  {"sweep": ..., "B": ..., "N": ..., "H": ..., "D": ..., "w1": ..., "w2": ..., "dtype": ...,
   "mfma": true|false, "fwd_ms": ..., "bwd_ms": ..., "fwd_tflops": ..., "bwd_tflops": ...,
   "tokens_per_s": ..., "peak_mem_mb": ...}

TFLOP/s count matmul flops of valid (i,j,k) triples only: 4*D*T forward, 12*D*T
backward.  A shape the library rejects is reported as {"error": ...} and the sweep
goes on.  `sdpa` lines add torch's causal scaled_dot_product_attention at the same
shape (full causal attention, not windowed: a different amount of work, shown for
orientation as the reference's harness does).
"""
import argparse
import json
import math
import os
import sys

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def count_triples(B, N, H, w1, w2):
    w1, w2 = min(w1, N - 1), min(w2, N - 1)
    head = sum((min(i, w1) + 1) * (min(i, w2) + 1) for i in range(min(N, max(w1, w2))))
    return B * H * (head + max(0, N - max(w1, w2)) * (w1 + 1) * (w2 + 1))


def time_gpu(fn, iters, warmup=3):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def measure(sa, lib, sweep, B, N, H, D, w1, w2, dtype="bf16", iters=20, sdpa=False):
    from simplical_attn_amd import _lib
    point = {"sweep": sweep, "B": B, "N": N, "H": H, "D": D, "w1": w1, "w2": w2, "dtype": dtype}
    try:
        dev = torch.device("cuda:0")
        g = torch.Generator(device=dev).manual_seed(B * 1000003 + N * 101 + H * 7 + D)
        td = DTYPES[dtype]
        q, k1, k2, v1, v2, dout = (torch.randn(B, N, H, D, generator=g, device=dev, dtype=torch.float32).to(td)
                                   for _ in range(6))
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        out, lse = sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2)
        sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2)
        torch.cuda.synchronize()
        point["peak_mem_mb"] = (torch.cuda.max_memory_allocated() - base) / 2**20
        point["mfma"] = bool(lib.sa2_uses_mfma(B, N, H, D, w1, w2, {"fp32": _lib.SA2_F32, "bf16": _lib.SA2_BF16,
                                                                    "fp16": _lib.SA2_F16}[dtype]))
        fwd_ms = time_gpu(lambda: sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2), iters)
        bwd_ms = time_gpu(lambda: sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2), iters)
        T = count_triples(B, N, H, w1, w2)
        point.update(fwd_ms=fwd_ms, bwd_ms=bwd_ms, fwd_tflops=4.0 * D * T / fwd_ms / 1e9,
                     bwd_tflops=12.0 * D * T / bwd_ms / 1e9, tokens_per_s=B * N / ((fwd_ms + bwd_ms) * 1e-3))
        if sdpa:
            import torch.nn.functional as F
            qs, ks, vs = (t.transpose(1, 2).contiguous().requires_grad_(True) for t in (q, k1, v1))
            gs = dout.transpose(1, 2).contiguous()
            o = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True)
            point["sdpa_fwd_ms"] = time_gpu(lambda: F.scaled_dot_product_attention(qs, ks, vs, is_causal=True), iters)
            point["sdpa_bwd_ms"] = time_gpu(lambda: torch.autograd.grad(o, (qs, ks, vs), gs, retain_graph=True), iters)
    except Exception as e:  # a rejected shape or an out-of-memory point ends the point, not the sweep
        point["error"] = "%s: %s" % (type(e).__name__, e)
    print(json.dumps(point), flush=True)
    return point


def main():
    all_sweeps = ["seq", "batch", "heads", "head_dim", "window", "precision", "memory", "sdpa", "long"]
    ap = argparse.ArgumentParser()
    ap.add_argument("--sweeps", default=",".join(all_sweeps))
    ap.add_argument("--iters", type=int, default=20)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("bench_sweep.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    import simplical_attn_amd as sa
    from simplical_attn_amd import _lib
    lib = _lib.load()
    wanted = [s for s in args.sweeps.split(",") if s]
    for s in wanted:
        if s not in all_sweeps:
            ap.error("unknown sweep %r (choose from %s)" % (s, ", ".join(all_sweeps)))

    def m(sweep, **kw):
        return measure(sa, lib, sweep, iters=args.iters, **kw)

    # base shapes and ranges of the reference's harness (test_performance.py:424-480)
    if "seq" in wanted:
        for n in (64, 128, 256, 512, 1024, 2048):
            m("seq", B=2, N=n, H=4, D=64, w1=32, w2=32)
    if "batch" in wanted:
        for b in (1, 2, 4, 8, 16, 32):
            m("batch", B=b, N=256, H=4, D=64, w1=32, w2=32)
    if "heads" in wanted:
        for h in (1, 2, 4, 8, 16, 32):
            m("heads", B=2, N=256, H=h, D=64, w1=32, w2=32)
    if "head_dim" in wanted:
        for d in (32, 64, 128, 256, 512):
            m("head_dim", B=2, N=256, H=4, D=d, w1=32, w2=32)
    if "window" in wanted:
        for w in (8, 16, 32, 64, 128, 256):
            m("window", B=2, N=512, H=4, D=64, w1=w, w2=w)
    if "precision" in wanted:                       # test_performance.py:488-491
        for dt in ("fp16", "bf16", "fp32"):
            m("precision", B=4, N=256, H=8, D=64, w1=32, w2=32, dtype=dt)
    if "memory" in wanted:                          # test_performance.py:507-516
        for b, n in ((1, 512), (4, 512), (1, 1024), (2, 1024), (1, 2048)):
            m("memory", B=b, N=n, H=4, D=64, w1=32, w2=32)
    if "sdpa" in wanted:                            # test_performance.py:549-551
        for n in (64, 128, 256, 512, 1024, 2048):
            m("sdpa", B=2, N=n, H=4, D=64, w1=32, w2=32, sdpa=True)
    if "long" in wanted:
        for n in (2048, 4096, 8192, 16384, 32768, 65536):
            m("long", B=1, N=n, H=16, D=128, w1=512, w2=32, sdpa=True)
        for w1, w2 in ((256, 16), (512, 32), (1024, 64), (2048, 32), (512, 64)):
            m("long_window", B=1, N=16384, H=16, D=128, w1=w1, w2=w2)
        for d in (64, 128):
            m("long_head_dim", B=1, N=16384, H=16, D=d, w1=512, w2=32)


if __name__ == "__main__":
    main()
