"""MFMA kernels against the fp32 FMA kernels (which tests/test_gpu_generic.py ties to the oracle)
over a seeded spread of shapes: sequence lengths around the 32-row tile and the 8-block /
4-block groups of the pre-pass kernels, K' windows that are and are not multiples of 4 and 8,
windows longer than the sequence, the three head dims and both 16-bit element types."""
import random

import pytest
import torch

from tests.util import assert_close_rel, make_inputs

pytestmark = pytest.mark.gpu
AUTO, GENERIC, MFMA = 0, 1, 2


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
        out.append((B, N, H, D, w1, w2, bias, dtype))
    return out


@pytest.mark.parametrize("case", _cases())
def test_mfma_matches_exact_kernels(case):
    import simplical_attn_amd as sa
    B, N, H, D, w1, w2, (kb, vb), dtype = case
    dev = torch.device("cuda:0")
    inp = [x.to(dev) for x in make_inputs(B, N, H, D, seed=N * 131 + w1 * 7 + w2, dtype=dtype)]
    res = {}
    for flags in (GENERIC, MFMA, AUTO):
        out, lse = sa.simplicial_forward(*inp[:5], w1, w2, None, kb, vb, flags=flags)
        grads = sa.simplicial_backward(*inp[:5], out, lse, inp[5], w1, w2, None, kb, vb, flags=flags)
        res[flags] = (out, lse, *grads)
    # The two sides are both rounded results (the parity bar against the oracle, 2e-2 for bf16, is
    # held in test_gpu_mfma_fwd.py / test_gpu_mfma_bwd.py), so their difference gets a little more.
    tol = 3e-2 if dtype == torch.bfloat16 else 1e-2
    # gradients that vanish by cancellation (one-triple windows) are held to an absolute floor
    floor = 0.1 if (min(w1, N - 1) == 0 and min(w2, N - 1) == 0) else 1e-5
    # MFMA forces the pre-pass kernels where the window allows; AUTO leaves them out at these sizes
    for which in (MFMA, AUTO):
        for name, a, b in zip(("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2"), res[which], res[GENERIC]):
            assert torch.isfinite(a).all(), name
            assert_close_rel(a, b.float().cpu(), tol, "%s %s" % (name, case),
                             atol=floor if name in ("dq", "dk1", "dk2") else 1e-5)
