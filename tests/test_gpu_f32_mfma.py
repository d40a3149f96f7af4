"""GPU parity of the fp32 MFMA kernels (v_mfma_f32_32x32x2_f32: fp32 products and sums; head_dim 32,
64, 128) against the CPU oracle, through the C ABI: the fp32 contract, rtol = atol = 1e-5, on
configuration c1 (fp32 B1 H2 N128 D64 w 32/16, seed 0) and on the reference's own test matrix
(simplicial/test_correctness.py:33, 37, 148-226, 256-288, 324-396), forced and under the default
dispatch (which must pick them: same bits)."""
import math

import pytest
import torch

from oracle import simplicial_oracle as orc
from simplical_attn_amd import _lib
from tests.util import assert_close_rel, make_inputs, oracle_all, record, run_device

pytestmark = pytest.mark.gpu
AUTO, GENERIC, MFMA = 0, 1, 2
NAMES = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")
LABEL = "c1 fp32 (fp32 MFMA kernels)"


def test_dispatch_picks_the_fp32_mfma_kernels():
    lib = _lib.load()
    for D in (32, 64, 128):
        assert lib.sa2_uses_mfma(1, 128, 2, D, 32, 16, _lib.SA2_F32) == 1
    for D in (16, 48, 256):
        assert lib.sa2_uses_mfma(1, 128, 2, D, 32, 16, _lib.SA2_F32) == 0


def test_config1_fp32_forward_matches_literal_oracle():
    inp = make_inputs(1, 128, 2, 64, seed=0)
    got = run_device(inp, 32, 16, flags=MFMA, backward=False)
    lit = orc.literal_loop(*inp[:5], 32, 16)
    assert torch.allclose(got["out"].cpu(), lit, rtol=1e-5, atol=1e-5)
    o64, lse64 = orc.forward_windowed(*[x.double() for x in inp[:5]], 32, 16)
    assert torch.allclose(got["out"].cpu().double(), o64, rtol=1e-5, atol=1e-5)
    assert torch.allclose(got["lse"].cpu().double(), lse64, rtol=1e-5, atol=1e-5)
    record(LABEL, "out", got["out"], o64)
    record(LABEL, "lse", got["lse"], lse64)
    auto = run_device(inp, 32, 16, flags=AUTO, backward=False)
    assert torch.equal(auto["out"], got["out"]) and torch.equal(auto["lse"], got["lse"])
    exact = run_device(inp, 32, 16, flags=GENERIC, backward=False)
    assert not torch.equal(exact["out"], got["out"])               # (another kernel: another summation order)


def test_config1_fp32_gradients():
    inp = make_inputs(1, 128, 2, 64, seed=0)
    got = run_device(inp, 32, 16, flags=MFMA)
    auto = run_device(inp, 32, 16, flags=AUTO)
    want = oracle_all(inp, 32, 16)
    for name in ("dq", "dk1", "dk2", "dv1", "dv2"):
        assert torch.allclose(got[name].cpu().double(), want[name], rtol=1e-5, atol=1e-5), name
        assert torch.equal(got[name], auto[name]), name
        record(LABEL, name, got[name], want[name])


@pytest.mark.parametrize("shape", [(2, 64, 2, 32), (4, 128, 4, 64), (1, 256, 8, 128), (2, 37, 3, 64), (1, 1, 1, 32),
                                   (1, 33, 2, 128), (3, 100, 1, 32)])
def test_forward_backward_vs_oracle(shape):
    """simplicial/test_correctness.py:148-177 (fp32 rows, w1 = w2 = 16), plus gradients and LSE."""
    B, N, H, D = shape
    inp = make_inputs(B, N, H, D, seed=N + D, mag=0.5)
    got = run_device(inp, 16, 16, flags=MFMA)
    want = oracle_all(inp, 16, 16)
    for name in NAMES:
        # (N = 1: dq, dk1, dk2 vanish by cancellation, a relative error of noise says nothing)
        assert_close_rel(got[name], want[name], 1e-5, name, label="fp32 MFMA shapes" if N > 1 else None)


@pytest.mark.parametrize("w", [(1, 1), (4, 4), (8, 3), (0, 5), (5, 0), (0, 0), (64, 64), (100, 7), (70, 200), (31, 32),
                               (32, 33)])
@pytest.mark.parametrize("inclusive", [True, False])
def test_window_sizes_both_conventions(w, inclusive):
    """simplicial/test_correctness.py:179-198, the w = 1 / w > N edge cases (324-354) and the half-open
    windows of the reference's device kernels (simplicial/kernels.py:133-136)."""
    if not inclusive and 0 in w:
        pytest.skip("a half-open window of 0 keys is empty")
    inp = make_inputs(2, 96, 2, 32, seed=7)
    got = run_device(inp, w[0], w[1], flags=MFMA, inclusive=inclusive)
    want = oracle_all(inp, w[0], w[1], inclusive=inclusive)
    # single-triple windows: dq, dk, dk' vanish by cancellation; what comes back is rounding noise
    lone = (w == (0, 0)) if inclusive else (w == (1, 1))
    for name in NAMES:
        assert_close_rel(got[name], want[name], 2e-5, name, atol=1e-5 if lone else 1e-6)


@pytest.mark.parametrize("bias", [(0.0, 0.0), (0.1, 0.2), (-0.1, -0.2), (1.0, 0.5)])
@pytest.mark.parametrize("D", [32, 128])
def test_bias_values(bias, D):
    """simplicial/test_correctness.py:200-226."""
    inp = make_inputs(2, 70, 2, D, seed=11)
    got = run_device(inp, 16, 8, None, bias[0], bias[1], flags=MFMA)
    want = oracle_all(inp, 16, 8, None, bias[0], bias[1])
    for name in NAMES:
        assert_close_rel(got[name], want[name], 2e-5, name)


def test_zero_and_extreme_inputs():
    """simplicial/test_correctness.py:356-396: all-zero inputs, and all-10.0 inputs (logits of 4000 at
    head_dim 32... here 8000 at scale 1/sqrt(32)) stay finite and equal the analytic answer."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    z = torch.zeros(1, 40, 2, 32, device=dev)
    out, lse = sa.simplicial_forward(z, z, z, z, z, 8, 8, flags=MFMA)
    assert torch.equal(out, torch.zeros_like(out))
    want = torch.tensor([math.log((min(i, 8) + 1) ** 2 + 1e-8) for i in range(40)])
    assert torch.allclose(lse[0, 0].cpu(), want.float(), rtol=1e-6)
    t = torch.full((1, 40, 2, 32), 10.0, device=dev)
    out, lse = sa.simplicial_forward(t, t, t, t, t, 8, 8, flags=MFMA)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.allclose(out, torch.full_like(out, 100.0), rtol=1e-5)


def test_epsilon_dominates_for_very_negative_logits():
    """Row 0 with one very negative logit: O -> 0 and LSE -> log(1e-8) (simplicial/reference.py:74)."""
    inp = make_inputs(1, 8, 1, 32, seed=3, mag=3.0)
    q, k1, k2 = inp[0], inp[1], inp[2]
    sign = torch.sign((q[:, 0] * k1[:, 0] * k2[:, 0]).sum(-1, keepdim=True))
    inp[0][:, 0] = -q[:, 0] * sign * 50.0
    got = run_device(inp, 4, 4, 1.0, flags=MFMA, backward=False)
    o64, lse64 = orc.forward_windowed(*[x.double() for x in inp[:5]], 4, 4, 1.0)
    assert torch.allclose(got["out"].cpu().double(), o64, rtol=1e-4, atol=1e-6)
    assert torch.allclose(got["lse"].cpu().double(), lse64, rtol=1e-5, atol=1e-5)
    assert abs(got["lse"][0, 0, 0].item() - math.log(1e-8)) < 1e-3


def test_deterministic_needs_subsets_and_accumulation():
    """simplicial/test_correctness.py:290-318, 402-421: two runs give identical bits, a second backward
    doubles .grad; gradients that are not needed are not computed and the others do not change."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    inp = make_inputs(2, 200, 2, 64, seed=42)
    a = run_device(inp, 40, 9, flags=MFMA)
    b = run_device(inp, 40, 9, flags=MFMA)
    for name in a:
        assert torch.equal(a[name], b[name]), name
    for subset in ((0,), (1, 3), (2, 4)):
        leaves = [x.to(dev).requires_grad_(t in subset) for t, x in enumerate(inp[:5])]
        sa.TwoSimplicialAttentionFunction.apply(*leaves, 40, 9, None, 0.0, 0.0, True, MFMA).backward(inp[5].to(dev))
        for t, name in enumerate(NAMES[2:]):
            if t in subset:
                assert torch.equal(leaves[t].grad, a[name]), name
            else:
                assert leaves[t].grad is None
    leaves = [x.to(dev).requires_grad_(True) for x in inp[:5]]
    attn = sa.TwoSimplicialAttention(64, 40, 9)
    attn(*leaves).sum().backward()
    first = [t.grad.clone() for t in leaves]
    attn(*leaves).sum().backward()
    for t, g in zip(leaves, first):
        assert torch.allclose(t.grad, 2 * g, rtol=1e-6, atol=1e-6)


def test_longer_sequence_against_the_oracle_on_row_ranges_and_the_fma_kernels():
    """fp32 B1 H2 N1024 D128 w 256/32: the oracle on three row ranges (first rows, rows straddling
    i = w1, last rows), the fp32 FMA kernels over whole tensors."""
    B, N, H, D, w1, w2 = 1, 1024, 2, 128, 256, 32
    inp = make_inputs(B, N, H, D, seed=9, mag=0.7)
    got = run_device(inp, w1, w2, flags=MFMA)
    exact = run_device(inp, w1, w2, flags=GENERIC)
    for name in NAMES:
        assert_close_rel(got[name], exact[name].cpu(), 2e-5, name + " vs FMA kernels")
    for rows in ((0, 96), (224, 320), (N - 64, N)):
        want_out, want_lse = orc.forward_windowed(*[x.double() for x in inp[:5]], w1, w2, rows=rows)
        assert_close_rel(got["out"][:, rows[0]:rows[1]], want_out, 1e-5, "out rows %s" % (rows,))
        assert_close_rel(got["lse"][:, :, rows[0]:rows[1]], want_lse, 1e-5, "lse rows %s" % (rows,))


def test_unaligned_fp32_rows_take_the_fma_kernels():
    """fp32 rows that are not 16-byte aligned (the MFMA kernels move float4): default dispatch equals the
    forced FMA kernels bit for bit, a forced MFMA call is refused."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2 = 1, 96, 2, 64, 20, 6
    host = make_inputs(B, N, H, D, seed=4)
    wide = [torch.zeros(B, N, H, D + 2, device=dev) for _ in host]
    views = [w[..., 1:1 + D] for w in wide]
    for v, x in zip(views, host):
        v.copy_(x)
    with pytest.raises(_lib.Sa2Error) as err:
        sa.simplicial_forward(*views[:5], w1, w2, flags=MFMA)
    assert err.value.status == -8
    res = {}
    for flags in (AUTO, GENERIC):
        out, lse = sa.simplicial_forward(*views[:5], w1, w2, flags=flags)
        grads = sa.simplicial_backward(*views[:5], out, lse, views[5], w1, w2, flags=flags)
        res[flags] = (out, lse, *grads)
    want = oracle_all(host, w1, w2)
    for name, a, b in zip(NAMES, res[AUTO], res[GENERIC]):
        assert torch.equal(a, b), name
        assert_close_rel(a, want[name], 1e-5, name)


@pytest.mark.parametrize("case", [(1, 160, 1, 128, 8, 120, 0.0), (1, 300, 2, 128, 20, 260, 0.2), (1, 500, 1, 64, 6, 450, 0.0),
                                  (1, 100, 1, 128, 8, 200, 0.0)],
                         ids=lambda c: "N%d-D%d-w%d_%d" % (c[1], c[3], c[4], c[5]))
def test_wide_k2_windows_are_walked_in_segments(case):
    """K' windows beyond what the K'-side kernel's dQ accumulator holds in LDS (86 deltas at head_dim 128, 378 at 64):
    the kernel walks them in segments of 84 / 376 deltas (two, four and two segments here; in the last case the
    window is wider than the sequence).  Forced and under the default dispatch (same bits), against the oracle."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2, kb = case
    host = make_inputs(B, N, H, D, seed=12, mag=0.5)
    x = [t.to(dev) for t in host]
    res = {}
    for flags in (MFMA, AUTO):
        out, lse = sa.simplicial_forward(*x[:5], w1, w2, None, kb, 0.0, flags=flags)
        grads = sa.simplicial_backward(*x[:5], out, lse, x[5], w1, w2, None, kb, 0.0, flags=flags)
        res[flags] = (out, lse, *grads)
    want = oracle_all(host, w1, w2, None, kb, 0.0)
    for name, a, b in zip(NAMES, res[MFMA], res[AUTO]):
        assert torch.equal(a, b), name
        assert_close_rel(a, want[name], 1e-5, name)
