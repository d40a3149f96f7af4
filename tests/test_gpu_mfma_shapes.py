"""MFMA kernels against the CPU oracle over a seeded spread of shapes: sequence lengths around the
32-row tile and the 8-block / 4-block groups of the pre-pass kernels, K' windows that are and are
not multiples of 4 and 8, windows longer than the sequence, the three head dims, both 16-bit
element types, biases, and both window conventions (closed [i-w, i] as simplicial/reference.py:41-45,
half-open (i-w, i] as simplicial/kernels.py:133-136).  Every tensor (out, LSE, five gradients) of
the forced-MFMA run and of the default dispatch is compared with the fp64 oracle on the same
rounded inputs; the fp32 FMA kernels are compared as well (to a tighter bar), and the MFMA result
with them as a second, kernel-against-kernel check."""
import random

import pytest
import torch

from tests.util import (assert_close_rel, assert_within, cancellation_bounds, make_inputs, oracle_all, record,
                        single_triple)

pytestmark = pytest.mark.gpu
AUTO, GENERIC, MFMA = 0, 1, 2
NAMES = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")


def _cases():
    rng = random.Random(20240607)
    lens = [1, 31, 32, 33, 63, 64, 65, 95, 127, 128, 129, 255, 256, 257, 289, 320, 511, 513, 700]
    w2s = [0, 1, 3, 4, 7, 8, 9, 15, 16, 24, 31, 32, 33, 40, 48, 64]
    out = []
    for n in range(72):
        N = rng.choice(lens)
        D = rng.choice([32, 64, 128])
        w2 = rng.choice(w2s)
        if D == 128 and w2 > 64:
            w2 = 64
        w1 = rng.choice([0, 5, 31, 32, 33, 64, 100, 255, 256, 1000])
        B, H = rng.choice([(1, 1), (1, 3), (2, 2)])
        dtype = torch.float16 if n % 4 == 3 else torch.bfloat16
        bias = rng.choice([(0.0, 0.0), (0.0, 0.0), (0.25, -0.5)])
        out.append((B, N, H, D, w1, w2, bias, dtype, True))
    # the half-open convention of the reference's device kernels: window w holds w keys, so the
    # pre-pass kernels are taken at w2 = 9, 17, 33, 65 (reach 8, 16, 32, 64)
    for n in range(24):
        N = rng.choice(lens)
        D = rng.choice([32, 64, 128])
        w2 = rng.choice([1, 2, 4, 5, 8, 9, 16, 17, 32, 33, 41, 65])
        w1 = rng.choice([1, 6, 32, 33, 65, 101, 256, 257, 1000])
        B, H = rng.choice([(1, 1), (1, 3), (2, 2)])
        dtype = torch.float16 if n % 4 == 3 else torch.bfloat16
        bias = rng.choice([(0.0, 0.0), (0.25, -0.5)])
        out.append((B, N, H, D, w1, w2, bias, dtype, False))
    return out


def _id(case):
    B, N, H, D, w1, w2, bias, dtype, inclusive = case
    return "B%dN%dH%dD%d-w%d_%d-%s%s%s" % (B, N, H, D, w1, w2, "bf16" if dtype == torch.bfloat16 else "fp16",
                                           "-bias" if bias != (0.0, 0.0) else "", "" if inclusive else "-halfopen")


@pytest.mark.parametrize("case", _cases(), ids=_id)
def test_mfma_matches_oracle(case):
    import simplical_attn_amd as sa
    B, N, H, D, w1, w2, (kb, vb), dtype, inclusive = case
    dev = torch.device("cuda:0")
    host = make_inputs(B, N, H, D, seed=N * 131 + w1 * 7 + w2, dtype=dtype)
    inp = [x.to(dev) for x in host]
    res = {}
    for flags in (GENERIC, MFMA, AUTO):
        out, lse = sa.simplicial_forward(*inp[:5], w1, w2, None, kb, vb, flags=flags, window_inclusive=inclusive)
        grads = sa.simplicial_backward(*inp[:5], out, lse, inp[5], w1, w2, None, kb, vb, flags=flags,
                                       window_inclusive=inclusive)
        res[flags] = dict(zip(NAMES, (out, lse, *grads)))
    want = oracle_all(host, w1, w2, None, kb, vb, inclusive=inclusive)
    bf16 = dtype == torch.bfloat16
    # parity bars: the 16-bit MFMA path 2e-2 (bf16) / 1e-2 (fp16) of max|ref| per tensor.  The fp32
    # kernels compute in fp32 but store 16-bit results, and their backward starts from the rounded
    # output: the row term D = sum dO*O inherits its half-ulp errors, which on short sequences
    # (little averaging) reach 1e-2 of max|ref| in bf16.  They get the same bar for bf16, half for fp16.
    tol_mfma = 2e-2 if bf16 else 1e-2
    tol_exact = 2e-2 if bf16 else 5e-3
    lone = single_triple(N, w1, w2, inclusive)
    noise = cancellation_bounds(host, want["out"], None, kb, vb) if lone else None
    label = "shapes %s%s" % ("bf16" if bf16 else "fp16", "" if inclusive else " half-open")
    for which, tol in ((MFMA, tol_mfma), (AUTO, tol_mfma), (GENERIC, tol_exact)):
        for name in NAMES:
            got = res[which][name]
            assert torch.isfinite(got).all(), name
            if lone and name in noise:
                assert_within(got, noise[name], "%s (%d) %s" % (name, which, _id(case)))
                continue
            assert_close_rel(got, want[name], tol, "%s (flags %d) %s" % (name, which, _id(case)), atol=1e-5,
                             label=label if which == MFMA else None)
    # second check, kernel against kernel: both sides carry their own rounding
    for name in NAMES:
        if lone and name in noise:
            continue
        assert_close_rel(res[MFMA][name], res[GENERIC][name].float().cpu(), 3e-2 if bf16 else 1e-2,
                         "%s mfma vs fp32 kernels %s" % (name, _id(case)), atol=1e-5)
