"""Writes the golden vectors of the parity tests (tests/golden/*.npz).

The reference's own tests hold no stored vectors for this path (they draw random
inputs at run time), so these are produced by the CPU oracle, which
tests/test_oracle.py pins against brute force, library routines and closed
forms.  Outputs: O from the literal triple loop in the reference's summation
order (simplicial/reference.py:39-74) in the case's dtype, LSE and the five
gradients from the fp64 windowed form.  Inputs come from a seeded CPU generator;
small cases store them, the larger one stores per-tensor sums as a guard.

    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import simplicial_oracle as orc  # noqa: E402
from util import make_inputs  # noqa: E402

CASES = {
    # name: (B, N, H, D, w1, w2, scale, k2_bias, v2_bias, seed, store_inputs)
    "c1_fp32": (1, 128, 2, 64, 32, 16, 0.125, 0.0, 0.0, 0, False),
    "tiny_biased": (2, 20, 2, 16, 5, 3, None, 0.3, -0.2, 11, True),
    "tiny_wide_windows": (1, 12, 1, 8, 64, 64, 0.5, 0.0, 0.0, 12, True),
    "tiny_unit_windows": (1, 9, 2, 32, 1, 0, None, 0.1, 0.0, 13, True),
}


def build(name):
    B, N, H, D, w1, w2, scale, kb, vb, seed, store = CASES[name]
    ins = make_inputs(B, N, H, D, seed, torch.float32)
    q, k1, k2, v1, v2, dout = ins
    out = orc.literal_loop(q, k1, k2, v1, v2, w1, w2, scale, kb, vb)
    d = [x.double() for x in ins]
    res = orc.grads_windowed(*d, w1, w2, scale, kb, vb, compute_dtype=torch.float64)
    rec = {"out_literal": out.numpy(), "out": res[0].numpy(), "lse": res[1].numpy()}
    for key, g in zip(("dq", "dk1", "dk2", "dv1", "dv2"), res[2:]):
        rec[key] = g.float().numpy()
    rec["out"] = rec["out"].astype(np.float32)
    rec["lse"] = rec["lse"].astype(np.float32)
    rec["input_sums"] = np.array([x.double().sum().item() for x in ins])
    if store:
        for key, x in zip(("q", "k1", "k2", "v1", "v2", "dout"), ins):
            rec[key] = x.numpy()
    return rec


if __name__ == "__main__":
    for name in CASES:
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **build(name))
        print("wrote", name)
