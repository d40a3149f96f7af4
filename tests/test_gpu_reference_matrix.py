"""The reference's own correctness tests (simplicial/test_correctness.py) re-expressed against this
build under its default kernel choice: same shapes, dtypes, window sizes, bias values, input scales
and tolerances (test_correctness.py:28-49), with the CPU oracle in the place of the reference's
PyTorch loop."""
import pytest
import torch

from oracle import simplicial_oracle as orc

pytestmark = pytest.mark.gpu
TOL = {torch.float16: 1e-2, torch.bfloat16: 1e-2, torch.float32: 1e-4}     # atol = rtol (test_correctness.py:45-49)
# The reference's inputs are scaled by 0.1, so its outputs are ~1e-3 and its absolute bars pass for almost
# any output.  Beside them every comparison here also holds max|diff| to a fraction of max|ref|: the
# 16-bit parity bars, and 1e-5 for fp32 (the fp32 contract of this build).
REL = {torch.float16: 1e-2, torch.bfloat16: 2e-2, torch.float32: 1e-5}


def _close(out, want, dtype):
    """The reference's own allclose bar and, beside it, the relative one."""
    got, ref = out.cpu().float(), want.float()
    assert torch.allclose(got, ref, atol=TOL[dtype], rtol=TOL[dtype])
    diff, scale = (got - ref).abs().max().item(), ref.abs().max().item()
    assert diff <= REL[dtype] * scale, "max|diff| %.3e > %.1e * max|ref| %.3e" % (diff, REL[dtype], scale)


def _inputs(B, N, H, D, dtype, seed, std=0.1):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(B, N, H, D, generator=g) * std).to(dtype) for _ in range(5)]


def _module(D, w1, w2, **kw):
    import simplical_attn_amd as sa
    return sa.TwoSimplicialAttention(D, w1, w2, **kw)


def _oracle(inp, w1, w2, k2_bias=0.0, v2_bias=0.0):
    out, _ = orc.forward_windowed(*[x.float() for x in inp], w1, w2, None, k2_bias, v2_bias,
                                  compute_dtype=torch.float32)
    return out


@pytest.mark.parametrize("shape", [(1, 32, 1, 16), (2, 64, 2, 32), (4, 128, 4, 64), (1, 256, 8, 128)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_forward_vs_reference(shape, dtype):
    """test_correctness.py:148-177."""
    B, N, H, D = shape
    inp = _inputs(B, N, H, D, dtype, seed=N + D)
    out = _module(D, 16, 16)(*[x.cuda() for x in inp])
    assert out.dtype == dtype and out.shape == (B, N, H, D)
    _close(out, _oracle(inp, 16, 16), dtype)


@pytest.mark.parametrize("w", [(4, 4), (8, 8), (16, 16), (32, 32), (64, 64)])
def test_window_sizes(w):
    """test_correctness.py:179-198."""
    inp = _inputs(2, 128, 4, 64, torch.bfloat16, seed=5)
    out = _module(64, *w)(*[x.cuda() for x in inp])
    _close(out, _oracle(inp, *w), torch.bfloat16)


@pytest.mark.parametrize("bias", [(0.0, 0.0), (0.1, 0.2), (-0.1, -0.2), (1.0, 0.5)])
def test_bias_values(bias):
    """test_correctness.py:200-226."""
    inp = _inputs(2, 64, 2, 32, torch.bfloat16, seed=6)
    out = _module(32, 16, 16, k2_bias=bias[0], v2_bias=bias[1])(*[x.cuda() for x in inp])
    _close(out, _oracle(inp, 16, 16, *bias), torch.bfloat16)


def test_backward_pass_basic_and_accumulation():
    """test_correctness.py:232-254 (every gradient exists, is finite and non-zero) and 290-318 (a
    second backward pass doubles .grad)."""
    leaves = [x.cuda().requires_grad_(True) for x in _inputs(1, 32, 1, 16, torch.float32, seed=7, std=1.0)]
    attn = _module(16, 8, 8)
    attn(*leaves).sum().backward()
    first = [t.grad.clone() for t in leaves]
    for g in first:
        assert torch.isfinite(g).all() and g.abs().sum() > 0
    attn(*leaves).sum().backward()
    for t, g in zip(leaves, first):
        assert torch.allclose(t.grad, 2 * g, atol=1e-4)


def test_edge_cases():
    """test_correctness.py:321-396: tiny problem with w = 1, windows longer than the sequence,
    all-zero inputs, all-ten inputs (logits of 4000)."""
    for (N, D, w) in ((16, 16, 1), (32, 32, 100)):
        inp = [x.cuda() for x in _inputs(1, N, 1, D, torch.bfloat16, seed=8)]
        out = _module(D, w, w)(*inp)
        assert torch.isfinite(out).all()
    z = torch.zeros(1, 32, 2, 64, dtype=torch.bfloat16, device="cuda")
    assert torch.equal(_module(64, 8, 8)(z, z, z, z, z), z)
    t = torch.full((1, 32, 2, 64), 10.0, dtype=torch.bfloat16, device="cuda")
    out = _module(64, 8, 8)(t, t, t, t, t)
    assert torch.isfinite(out).all()
    assert torch.allclose(out.float(), torch.full_like(out, 100.0).float(), rtol=1e-2)


def test_deterministic_output_and_precision_consistency():
    """test_correctness.py:402-421 (same inputs, same bits) and 423-455 (fp32 inputs against their
    bf16 rounding: max difference < 0.1, mean < 0.01)."""
    inp = _inputs(2, 64, 2, 64, torch.float32, seed=42, std=1.0)
    attn = _module(64, 16, 16)
    a = attn(*[x.cuda() for x in inp])
    b = attn(*[x.cuda() for x in inp])
    assert torch.equal(a, b)
    low = attn(*[x.to(torch.bfloat16).cuda() for x in inp])
    diff = (a - low.float()).abs()
    assert diff.max().item() < 0.1 and diff.mean().item() < 0.01
