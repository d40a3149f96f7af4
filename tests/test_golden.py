"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_vectors.py):
the oracle must keep reproducing them on CPU, the HIP kernels must match them on
the GPU through the C ABI."""
import os
import sys

import numpy as np
import pytest
import torch

from oracle import simplicial_oracle as orc
from util import make_inputs, run_device

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLDEN)
from make_vectors import CASES  # noqa: E402

GRADS = ("dq", "dk1", "dk2", "dv1", "dv2")


def load(name):
    rec = dict(np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False))
    B, N, H, D, w1, w2, scale, kb, vb, seed, stored = CASES[name]
    ins = make_inputs(B, N, H, D, seed, torch.float32)
    # the seeded generator must still give the inputs the vectors were made from
    np.testing.assert_allclose([x.double().sum().item() for x in ins], rec["input_sums"], rtol=0, atol=1e-9)
    if stored:
        for key, x in zip(("q", "k1", "k2", "v1", "v2", "dout"), ins):
            assert np.array_equal(x.numpy(), rec[key])
    return rec, ins, (w1, w2, scale, kb, vb)


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_the_vectors(name):
    rec, ins, (w1, w2, scale, kb, vb) = load(name)
    out, lse = orc.forward_windowed(*ins[:5], w1, w2, scale, kb, vb)
    # the literal loop adds one weight at a time in fp32; the windowed form sums
    # in blocks: they agree to fp32 rounding of a few thousand terms
    np.testing.assert_allclose(out.numpy(), rec["out_literal"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(out.numpy(), rec["out"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(lse.numpy(), rec["lse"], rtol=1e-5, atol=1e-5)
    res = orc.grads_windowed(*[x.double() for x in ins], w1, w2, scale, kb, vb, compute_dtype=torch.float64)
    for key, g in zip(GRADS, res[2:]):
        np.testing.assert_allclose(g.float().numpy(), rec[key], rtol=1e-6, atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_fp32_kernels_match_the_vectors(name):
    rec, ins, (w1, w2, scale, kb, vb) = load(name)
    got = run_device(ins, w1, w2, scale, kb, vb)
    for key in ("out", "lse") + GRADS:
        np.testing.assert_allclose(got[key].float().cpu().numpy(), rec[key], rtol=1e-5, atol=1e-5, err_msg=key)
    np.testing.assert_allclose(got["out"].cpu().numpy(), rec["out_literal"], rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
def test_bf16_kernels_match_the_c1_vectors_within_bf16_bounds():
    # D=64 bf16 goes through the MFMA kernels; inputs are rounded to bf16, so the
    # comparison carries the input rounding as well: 3e-2 of max|ref| per tensor.
    rec, ins, (w1, w2, scale, kb, vb) = load("c1_fp32")
    got = run_device([x.bfloat16() for x in ins], w1, w2, scale, kb, vb)
    for key in ("out", "lse") + GRADS:
        ref = rec[key]
        diff = np.abs(got[key].float().cpu().numpy() - ref).max()
        assert diff <= 3e-2 * np.abs(ref).max(), (key, diff, np.abs(ref).max())
