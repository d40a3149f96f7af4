"""GPU parity of the head_dim 256 MFMA kernels (bf16 and fp16) against the CPU oracle, through the
C ABI: simplicial/test_correctness.py:33 lists head_dim 256 among the reference's test sizes.  Every
tensor (out, LSE, five gradients) of the forced-MFMA run and of the default dispatch (which must pick
the same kernels: same bits) is compared with the fp64 oracle on the same rounded inputs at the 16-bit
bars (bf16 2e-2, fp16 1e-2 of max|ref| per tensor), and with the fp32 FMA kernels as a second,
kernel-against-kernel check."""
import random

import pytest
import torch

from simplical_attn_amd import _lib
from tests.util import (assert_close_rel, assert_within, cancellation_bounds, make_inputs, oracle_all,
                        single_triple)

pytestmark = pytest.mark.gpu
AUTO, GENERIC, MFMA = 0, 1, 2
NAMES = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")
D = 256


def _cases():
    rng = random.Random(256)
    lens = [1, 31, 32, 33, 64, 65, 127, 129, 200, 257, 320]
    out = []
    for n in range(20):
        N = rng.choice(lens)
        w2 = rng.choice([0, 1, 3, 4, 7, 8, 9, 16, 31, 32, 33, 64, 82])
        w1 = rng.choice([0, 5, 31, 32, 33, 64, 100, 255, 1000])
        B, H = rng.choice([(1, 1), (1, 3), (2, 2)])
        dtype = torch.float16 if n % 4 == 3 else torch.bfloat16
        bias = rng.choice([(0.0, 0.0), (0.0, 0.0), (0.25, -0.5)])
        out.append((B, N, H, w1, w2, bias, dtype, True))
    for n in range(6):
        N = rng.choice(lens)
        w2 = rng.choice([1, 2, 5, 9, 17, 33])
        w1 = rng.choice([1, 6, 33, 65, 257, 1000])
        B, H = rng.choice([(1, 1), (1, 3), (2, 2)])
        dtype = torch.float16 if n % 3 == 2 else torch.bfloat16
        out.append((B, N, H, w1, w2, rng.choice([(0.0, 0.0), (0.25, -0.5)]), dtype, False))
    return out


def _id(case):
    B, N, H, w1, w2, bias, dtype, inclusive = case
    return "B%dN%dH%d-w%d_%d-%s%s%s" % (B, N, H, w1, w2, "bf16" if dtype == torch.bfloat16 else "fp16",
                                        "-bias" if bias != (0.0, 0.0) else "", "" if inclusive else "-halfopen")


def _run(sa, inp, w1, w2, kb, vb, flags, inclusive=True, needs=(True,) * 5):
    out, lse = sa.simplicial_forward(*inp[:5], w1, w2, None, kb, vb, flags=flags, window_inclusive=inclusive)
    grads = sa.simplicial_backward(*inp[:5], out, lse, inp[5], w1, w2, None, kb, vb, needs=needs, flags=flags,
                                   window_inclusive=inclusive)
    return dict(zip(NAMES, (out, lse, *grads)))


def test_dispatch_picks_the_mfma_kernels_for_head_dim_256():
    lib = _lib.load()
    assert lib.sa2_uses_mfma(1, 256, 2, 256, 32, 16, _lib.SA2_BF16) == 1
    assert lib.sa2_uses_mfma(1, 256, 2, 256, 32, 16, _lib.SA2_F16) == 1
    assert lib.sa2_uses_mfma(1, 256, 2, 256, 32, 16, _lib.SA2_F32) == 0
    assert lib.sa2_uses_mfma(1, 256, 2, 192, 32, 16, _lib.SA2_BF16) == 0


@pytest.mark.parametrize("case", _cases(), ids=_id)
def test_head_dim_256_matches_oracle(case):
    import simplical_attn_amd as sa
    B, N, H, w1, w2, (kb, vb), dtype, inclusive = case
    dev = torch.device("cuda:0")
    host = make_inputs(B, N, H, D, seed=N * 131 + w1 * 7 + w2, dtype=dtype, mag=0.7)
    inp = [x.to(dev) for x in host]
    res = {flags: _run(sa, inp, w1, w2, kb, vb, flags, inclusive) for flags in (GENERIC, MFMA, AUTO)}
    want = oracle_all(host, w1, w2, None, kb, vb, inclusive=inclusive)
    bf16 = dtype == torch.bfloat16
    tol = 2e-2 if bf16 else 1e-2
    lone = single_triple(N, w1, w2, inclusive)
    noise = cancellation_bounds(host, want["out"], None, kb, vb) if lone else None
    label = "head_dim 256 %s" % ("bf16" if bf16 else "fp16")
    for name in NAMES:
        assert torch.equal(res[MFMA][name], res[AUTO][name]), name          # the default dispatch takes these kernels
        got = res[MFMA][name]
        assert torch.isfinite(got).all(), name
        if lone and name in noise:
            assert_within(got, noise[name], "%s %s" % (name, _id(case)))
            continue
        assert_close_rel(got, want[name], tol, "%s %s" % (name, _id(case)), atol=1e-5, label=label)
        assert_close_rel(got, res[GENERIC][name].float().cpu(), 3e-2 if bf16 else 1e-2,
                         "%s mfma vs fp32 kernels %s" % (name, _id(case)), atol=1e-5)


def test_reference_matrix_shape_with_head_dim_256():
    """simplicial/test_correctness.py:148-177 with its input scale (0.1) and tolerance (1e-2), at head_dim 256,
    plus the relative bar."""
    import simplical_attn_amd as sa
    from oracle import simplicial_oracle as orc
    for dtype, rel in ((torch.bfloat16, 2e-2), (torch.float16, 1e-2)):
        g = torch.Generator().manual_seed(256)
        inp = [(torch.randn(1, 64, 2, D, generator=g) * 0.1).to(dtype) for _ in range(5)]
        out = sa.TwoSimplicialAttention(D, 16, 16)(*[x.cuda() for x in inp])
        want, _ = orc.forward_windowed(*[x.float() for x in inp], 16, 16, compute_dtype=torch.float32)
        assert out.dtype == dtype and torch.allclose(out.cpu().float(), want, atol=1e-2, rtol=1e-2)
        assert (out.cpu().float() - want).abs().max() <= rel * want.abs().max()


def test_deterministic_and_needs_subsets():
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    host = make_inputs(2, 150, 2, D, seed=3, dtype=torch.bfloat16)
    inp = [x.to(dev) for x in host]
    a = _run(sa, inp, 40, 9, 0.0, 0.0, MFMA)
    b = _run(sa, inp, 40, 9, 0.0, 0.0, MFMA)
    for name in NAMES:
        assert torch.equal(a[name], b[name]), name
    for subset in ((0,), (1, 3), (2, 4)):
        needs = tuple(t in subset for t in range(5))
        c = _run(sa, inp, 40, 9, 0.0, 0.0, MFMA, needs=needs)
        for t, name in enumerate(NAMES[2:]):
            if t in subset:
                assert torch.equal(c[name], a[name]), name
            else:
                assert c[name] is None


def test_longer_sequence_against_oracle_row_ranges_and_the_fp32_kernels():
    """bf16 B1 H2 N1024 D256 w 256/32: the oracle on three row ranges, the fp32 FMA kernels over whole tensors."""
    import simplical_attn_amd as sa
    from oracle import simplicial_oracle as orc
    dev = torch.device("cuda:0")
    N, w1, w2 = 1024, 256, 32
    host = make_inputs(1, N, 2, D, seed=9, dtype=torch.bfloat16, mag=0.7)
    inp = [x.to(dev) for x in host]
    got = _run(sa, inp, w1, w2, 0.0, 0.0, MFMA)
    exact = _run(sa, inp, w1, w2, 0.0, 0.0, GENERIC)
    for name in NAMES:
        assert_close_rel(got[name], exact[name].float().cpu(), 3e-2, name + " vs fp32 kernels")
    for rows in ((0, 96), (224, 320), (N - 64, N)):
        want_out, want_lse = orc.forward_windowed(*[x.double() for x in host[:5]], w1, w2, rows=rows)
        assert_close_rel(got["out"][:, rows[0]:rows[1]], want_out, 2e-2, "out rows %s" % (rows,))
        assert_close_rel(got["lse"][:, :, rows[0]:rows[1]], want_lse, 2e-2, "lse rows %s" % (rows,))


def test_wide_k2_windows_in_segments_and_unaligned_rows():
    """K' windows beyond the K'-side kernel's dQ accumulator in LDS (w2 > 82) are walked in segments of 80 deltas
    (two and four segments here), forced and under the default dispatch (same bits), against the oracle.
    Rows off the 16-byte grid: everything on the fp32 kernels."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    for N, w1, w2, kb in ((160, 8, 120, 0.0), (290, 12, 250, 0.1)):
        host = make_inputs(1, N, 1, D, seed=12, dtype=torch.bfloat16, mag=0.5)
        x = [t.to(dev) for t in host]
        a = _run(sa, x, w1, w2, kb, 0.0, MFMA)
        b = _run(sa, x, w1, w2, kb, 0.0, AUTO)
        want = oracle_all(host, w1, w2, None, kb, 0.0)
        for name in NAMES:
            assert torch.equal(a[name], b[name]), name
            assert_close_rel(a[name], want[name], 2e-2, "%s w2=%d" % (name, w2))
    host = make_inputs(1, 160, 1, D, seed=12, dtype=torch.bfloat16, mag=0.5)
    wide = [torch.zeros(1, 160, 1, D + 8, dtype=torch.bfloat16, device=dev) for _ in host]
    views = [w[..., 4:4 + D] for w in wide]
    for v, t in zip(views, host):
        v.copy_(t)
    with pytest.raises(_lib.Sa2Error):
        sa.simplicial_forward(*views[:5], 8, 8, flags=MFMA)
    a = _run(sa, views, 8, 8, 0.0, 0.0, AUTO)
    b = _run(sa, views, 8, 8, 0.0, 0.0, GENERIC)
    for name in NAMES:
        assert torch.equal(a[name], b[name]), name
