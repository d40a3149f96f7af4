"""GPU parity of the MFMA forward kernel (bf16 and fp16 elements), through the C ABI.

Tolerance (bf16 path): max|diff| <= 2e-2 * max|ref| per tensor against the
fp64 oracle evaluated on the same bf16-rounded inputs.  Large shapes are
checked against the oracle on row ranges (the oracle is O(T) on the CPU) and,
over the whole tensor, against the generic fp32 kernels, which the small-shape
tests tie to the oracle."""
import math

import pytest
import torch

from oracle import simplicial_oracle as orc
from tests.util import assert_close_rel, make_inputs

pytestmark = pytest.mark.gpu
GENERIC, MFMA = 1, 2
BF16_TOL = 2e-2


def fwd(inp, w1, w2, scale=None, kb=0.0, vb=0.0, flags=MFMA):
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    return sa.simplicial_forward(*[x.to(dev) for x in inp[:5]], w1, w2, scale, kb, vb, flags=flags)


def sa_forward_half_open(inp, w1, w2):
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    return sa.simplicial_forward(*[x.to(dev) for x in inp[:5]], w1, w2, flags=MFMA, window_inclusive=False)


def oracle_rows(inp, w1, w2, rows, scale=None, kb=0.0, vb=0.0, dtype=torch.float64):
    return orc.forward_windowed(*[x.to(dtype) for x in inp[:5]], w1, w2, scale, kb, vb, rows=rows,
                                compute_dtype=dtype)


SMALL = [  # B, N, H, D, w1, w2, k2_bias, v2_bias
    (1, 64, 1, 64, 16, 8, 0.0, 0.0),
    (2, 100, 2, 128, 40, 5, 0.0, 0.0),        # N not a multiple of the tile
    (1, 256, 2, 64, 512, 32, 0.0, 0.0),       # windows wider than the sequence
    (1, 200, 1, 128, 0, 0, 0.0, 0.0),         # single-triple windows
    (1, 130, 2, 64, 33, 1, 0.1, 0.2),
    (1, 96, 1, 128, 7, 64, -0.1, -0.2),       # K' window wider than the K window
    (2, 160, 3, 128, 64, 32, 1.0, 0.5),
    (1, 33, 1, 64, 31, 32, 0.0, 0.0),
    (1, 1, 1, 64, 4, 4, 0.0, 0.0),
    (2, 130, 2, 32, 33, 8, 0.1, 0.2),         # head_dim 32
    (1, 200, 1, 32, 64, 32, 0.0, 0.0),
]


@pytest.mark.parametrize("case", SMALL)
def test_small_shapes_vs_oracle(case):
    B, N, H, D, w1, w2, kb, vb = case
    inp = make_inputs(B, N, H, D, seed=N + D + w1, dtype=torch.bfloat16, with_dout=False)
    out, lse = fwd(inp, w1, w2, None, kb, vb)
    want, want_lse = oracle_rows(inp, w1, w2, None, None, kb, vb)
    assert_close_rel(out, want, BF16_TOL, "out", label="small shapes bf16 (fwd)")
    assert_close_rel(lse, want_lse, BF16_TOL, "lse", label="small shapes bf16 (fwd)")


FP16_CASES = [SMALL[1], SMALL[4], SMALL[6], SMALL[7]]


@pytest.mark.parametrize("case", FP16_CASES)
def test_small_shapes_fp16_vs_oracle(case):
    """fp16 elements on the same kernels (fp16 MFMA); the tolerance of the bf16 path is kept."""
    B, N, H, D, w1, w2, kb, vb = case
    inp = make_inputs(B, N, H, D, seed=N + D + w1, dtype=torch.float16, with_dout=False)
    out, lse = fwd(inp, w1, w2, None, kb, vb)
    assert out.dtype == torch.float16
    want, want_lse = oracle_rows(inp, w1, w2, None, None, kb, vb)
    assert_close_rel(out, want, 4e-3, "out")
    assert_close_rel(lse, want_lse, 4e-3, "lse")


def test_fp16_weights_beyond_half_range_go_to_the_repair_kernel():
    """Logits that grow along the window push softmax weights (relative to the reference point
    fixed at the first tile) past 65504: the block is recomputed with running maxima."""
    B, N, H, D = 1, 192, 1, 64
    g = torch.Generator().manual_seed(11)
    q = torch.ones(B, N, H, D)
    k2 = torch.ones(B, N, H, D)
    ramp = torch.linspace(-1.0, 1.0, N).view(1, N, 1, 1)
    k1 = (ramp * 4.0).expand(B, N, H, D).contiguous()           # s_ij grows with j: 64 * 4 * ramp / 8
    v1 = torch.randn(B, N, H, D, generator=g)
    v2 = torch.randn(B, N, H, D, generator=g)
    inp = [t.to(torch.float16) for t in (q, k1, k2, v1, v2)]
    out, lse = fwd(inp, 160, 8)
    want, want_lse = oracle_rows(inp, 160, 8, None)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert_close_rel(out, want, 4e-3, "out")
    assert_close_rel(lse, want_lse, 4e-3, "lse")


def test_auto_dispatch_takes_mfma_for_bf16_d64_d128():
    from simplical_attn_amd import _lib
    lib = _lib.load()
    assert lib.sa2_uses_mfma(2, 2048, 8, 64, 512, 32, _lib.SA2_BF16) == 1
    assert lib.sa2_uses_mfma(1, 8192, 16, 128, 512, 32, _lib.SA2_BF16) == 1
    assert lib.sa2_uses_mfma(1, 8192, 16, 128, 512, 32, _lib.SA2_F16) == 1
    assert lib.sa2_uses_mfma(1, 128, 2, 64, 32, 16, _lib.SA2_F32) == 1      # (the fp32 MFMA kernels)
    assert lib.sa2_uses_mfma(1, 128, 2, 256, 32, 16, _lib.SA2_F32) == 0
    assert lib.sa2_uses_mfma(1, 128, 2, 32, 32, 16, _lib.SA2_BF16) == 1
    assert lib.sa2_uses_mfma(1, 128, 2, 48, 32, 16, _lib.SA2_BF16) == 0
    inp = make_inputs(1, 96, 2, 64, seed=1, dtype=torch.bfloat16, with_dout=False)
    a = fwd(inp, 20, 6, flags=0)
    b = fwd(inp, 20, 6, flags=MFMA)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_config2_forward():
    """Benchmark configuration 2: bf16, B2 H8 N2048 D64, w 512/32, seed 1."""
    inp = make_inputs(2, 2048, 8, 64, seed=1, dtype=torch.bfloat16, with_dout=False)
    out, lse = fwd(inp, 512, 32)
    for rows in ((0, 96), (480, 576), (1990, 2048)):
        want, want_lse = oracle_rows(inp, 512, 32, rows, dtype=torch.float32)
        assert_close_rel(out[:, rows[0]:rows[1]], want, BF16_TOL, "out rows %s" % (rows,), label="c2 bf16 B2 H8 N2048 D64 w512/32")
        assert_close_rel(lse[:, :, rows[0]:rows[1]], want_lse, BF16_TOL, "lse rows %s" % (rows,), label="c2 bf16 B2 H8 N2048 D64 w512/32")
    ref, ref_lse = fwd(inp, 512, 32, flags=GENERIC)
    assert_close_rel(out, ref.float().cpu(), BF16_TOL, "out vs generic kernel")
    assert_close_rel(lse, ref_lse.cpu(), BF16_TOL, "lse vs generic kernel")


def test_config4_forward_headline_shape():
    """Benchmark configuration 4: bf16, B1 H16 N8192 D128, w 512/32, seed 3; oracle on
    row ranges (start, the block straddling i = w1, end), generic kernel on all rows."""
    inp = make_inputs(1, 8192, 16, 128, seed=3, dtype=torch.bfloat16, with_dout=False)
    out, lse = fwd(inp, 512, 32)
    for rows in ((0, 40), (500, 540), (8160, 8192)):
        want, want_lse = oracle_rows(inp, 512, 32, rows, dtype=torch.float32)
        assert_close_rel(out[:, rows[0]:rows[1]], want, BF16_TOL, "out rows %s" % (rows,))
        assert_close_rel(lse[:, :, rows[0]:rows[1]], want_lse, BF16_TOL, "lse rows %s" % (rows,))
    # the half-open windows of the reference's device kernels at the same shape (w 512/32 then
    # reach 511/31: no pre-pass, a partial last round), oracle with its own half-open masks
    out_h, lse_h = sa_forward_half_open(inp, 512, 32)
    for rows in ((0, 40), (500, 540), (8160, 8192)):
        want, want_lse = orc.forward_windowed(*[x.float() for x in inp[:5]], 512, 32, rows=rows,
                                              compute_dtype=torch.float32, inclusive=False)
        assert_close_rel(out_h[:, rows[0]:rows[1]], want, BF16_TOL, "half-open out rows %s" % (rows,))
        assert_close_rel(lse_h[:, :, rows[0]:rows[1]], want_lse, BF16_TOL, "half-open lse rows %s" % (rows,))
    ref, ref_lse = fwd(inp, 512, 32, flags=GENERIC)
    assert_close_rel(out, ref.float().cpu(), BF16_TOL, "out vs generic kernel")
    assert_close_rel(lse, ref_lse.cpu(), BF16_TOL, "lse vs generic kernel")


def test_extreme_and_zero_inputs():
    dev = torch.device("cuda:0")
    import simplical_attn_amd as sa
    t = torch.full((1, 64, 2, 64), 10.0, device=dev, dtype=torch.bfloat16)
    out, lse = sa.simplicial_forward(t, t, t, t, t, 8, 8, flags=MFMA)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.allclose(out.float(), torch.full_like(out, 100.0).float(), rtol=1e-2)
    z = torch.zeros_like(t)
    out, lse = sa.simplicial_forward(z, z, z, z, z, 8, 8, flags=MFMA)
    assert torch.equal(out, torch.zeros_like(out))
    want = torch.tensor([math.log((min(i, 8) + 1) ** 2 + 1e-8) for i in range(64)])
    assert torch.allclose(lse[0, 0].cpu(), want.float(), rtol=1e-5)


def test_repair_pass_when_logits_outgrow_the_first_reference_point():
    """The fast kernel fixes a unit's softmax reference at its first tile; logits that
    later grow by hundreds of octaves overflow its weights, the block is marked and the
    repair kernel redoes it with a moving reference.  The result must still match."""
    B, N, H, D, w1, w2 = 1, 160, 2, 64, 100, 5
    q = torch.full((B, N, H, D), 0.5)
    k2 = torch.full((B, N, H, D), 0.5)
    ramp = torch.zeros(N)
    ramp[40:] = 200.0                  # logit 0 on the first keys, 200 (288 octaves) later
    ramp[120:] = 900.0
    k1 = ramp[None, :, None, None].expand(B, N, H, D).contiguous()
    g = torch.Generator().manual_seed(0)
    v1 = torch.randn(B, N, H, D, generator=g)
    v2 = torch.randn(B, N, H, D, generator=g)
    inp = [t.to(torch.bfloat16) for t in (q, k1, k2, v1, v2)]
    scale = 1.0 / (D * 0.25)           # s[i,j,k] = ramp[j]
    out, lse = fwd(inp, w1, w2, scale)
    want, want_lse = oracle_rows(inp, w1, w2, None, scale)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert_close_rel(out, want, BF16_TOL, "out")
    assert_close_rel(lse, want_lse, BF16_TOL, "lse")


def test_deterministic():
    inp = make_inputs(2, 300, 2, 128, seed=42, dtype=torch.bfloat16, with_dout=False)
    a = fwd(inp, 100, 20)
    b = fwd(inp, 100, 20)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
