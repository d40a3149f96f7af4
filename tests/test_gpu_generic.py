"""GPU parity of the generic fp32-FMA kernels against the CPU oracle, through
the C ABI.  Shapes, dtypes, windows, biases and edge cases re-express the
reference's own correctness suite (simplicial/test_correctness.py:148-455) with
N(0,1)-sized inputs where the reference used 0.1*N(0,1)."""
import math

import pytest
import torch

from oracle import simplicial_oracle as orc
from tests.util import assert_close_rel, make_inputs, oracle_all, record, rel_err, run_device

pytestmark = pytest.mark.gpu
GENERIC = 1


def test_config1_fp32_forward_matches_literal_oracle():
    """Benchmark configuration 1: fp32, B1 H2 N128 D64, w 32/16, seed 0, rtol = atol = 1e-5
    against the literal-order fp32 loop and against the fp64 truth."""
    inp = make_inputs(1, 128, 2, 64, seed=0)
    got = run_device(inp, 32, 16, flags=GENERIC, backward=False)
    lit = orc.literal_loop(*inp[:5], 32, 16)
    assert torch.allclose(got["out"].cpu(), lit, rtol=1e-5, atol=1e-5)
    o64, lse64 = orc.forward_windowed(*[x.double() for x in inp[:5]], 32, 16)
    assert torch.allclose(got["out"].cpu().double(), o64, rtol=1e-5, atol=1e-5)
    assert torch.allclose(got["lse"].cpu().double(), lse64, rtol=1e-5, atol=1e-5)
    record("c1 fp32 B1 H2 N128 D64 w32/16", "out", got["out"], o64)
    record("c1 fp32 B1 H2 N128 D64 w32/16", "lse", got["lse"], lse64)


def test_config1_fp32_gradients():
    inp = make_inputs(1, 128, 2, 64, seed=0)
    got = run_device(inp, 32, 16, flags=GENERIC)
    want = oracle_all(inp, 32, 16)
    for name in ("dq", "dk1", "dk2", "dv1", "dv2"):
        assert torch.allclose(got[name].cpu().double(), want[name], rtol=1e-5, atol=1e-5), name
        record("c1 fp32 B1 H2 N128 D64 w32/16", name, got[name], want[name])


@pytest.mark.parametrize("shape", [(1, 32, 1, 16), (2, 64, 2, 32), (4, 128, 4, 64), (1, 256, 8, 128), (1, 40, 2, 256),
                                   (2, 37, 3, 20)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_forward_backward_vs_oracle(shape, dtype):
    """simplicial/test_correctness.py:148-177 (w1 = w2 = 16), plus gradients."""
    B, N, H, D = shape
    inp = make_inputs(B, N, H, D, seed=N + D, dtype=dtype, mag=0.5)
    got = run_device(inp, 16, 16, flags=GENERIC)
    want = oracle_all(inp, 16, 16)
    tol = 1e-5 if dtype == torch.float32 else (1e-2 if dtype == torch.bfloat16 else 2e-3)
    for name in ("out", "dq", "dk1", "dk2", "dv1", "dv2"):
        assert_close_rel(got[name], want[name], tol, name)
    assert_close_rel(got["lse"], want["lse"], 1e-5, "lse")


@pytest.mark.parametrize("w", [(1, 1), (4, 4), (8, 3), (0, 5), (5, 0), (0, 0), (64, 64), (100, 7), (70, 200)])
def test_window_sizes(w):
    """simplicial/test_correctness.py:179-198 and the w = 1 / w > N edge cases (324-354)."""
    inp = make_inputs(2, 96, 2, 32, seed=7)
    got = run_device(inp, w[0], w[1], flags=GENERIC)
    want = oracle_all(inp, w[0], w[1])
    # single-triple windows: dq, dk, dk' vanish by cancellation (only the 1e-8 epsilon
    # keeps them from being exactly 0); what the fp32 kernels return is rounding noise
    atol = 1e-5 if w == (0, 0) else 1e-6
    for name in ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2"):
        assert_close_rel(got[name], want[name], 2e-5, name, atol=atol)


@pytest.mark.parametrize("bias", [(0.0, 0.0), (0.1, 0.2), (-0.1, -0.2), (1.0, 0.5)])
def test_bias_values(bias):
    """simplicial/test_correctness.py:200-226."""
    inp = make_inputs(2, 64, 2, 32, seed=11)
    got = run_device(inp, 16, 8, None, bias[0], bias[1], flags=GENERIC)
    want = oracle_all(inp, 16, 8, None, bias[0], bias[1])
    for name in ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2"):
        assert_close_rel(got[name], want[name], 2e-5, name)


def test_zero_and_extreme_inputs():
    """simplicial/test_correctness.py:356-396: all-zero inputs, and all-10.0
    inputs (logits of 4000) stay finite and equal the analytic answer."""
    dev = torch.device("cuda:0")
    import simplical_attn_amd as sa
    z = torch.zeros(1, 32, 2, 16, device=dev)
    out, lse = sa.simplicial_forward(z, z, z, z, z, 8, 8, flags=GENERIC)
    assert torch.equal(out, torch.zeros_like(out))
    want = torch.tensor([math.log((min(i, 8) + 1) ** 2 + 1e-8) for i in range(32)])
    assert torch.allclose(lse[0, 0].cpu(), want.float(), rtol=1e-6)
    t = torch.full((1, 32, 2, 16), 10.0, device=dev)
    out, lse = sa.simplicial_forward(t, t, t, t, t, 8, 8, flags=GENERIC)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.allclose(out, torch.full_like(out, 100.0), rtol=1e-5)


def test_epsilon_dominates_for_very_negative_logits():
    """Row 0 with one very negative logit: O -> 0 and LSE -> log(1e-8) as the
    oracle's +1e-8 demands (simplicial/reference.py:74)."""
    inp = make_inputs(1, 8, 1, 16, seed=3, mag=3.0)
    q, k1, k2 = inp[0], inp[1], inp[2]
    sign = torch.sign((q[:, 0] * k1[:, 0] * k2[:, 0]).sum(-1, keepdim=True))
    inp[0][:, 0] = -q[:, 0] * sign * 50.0
    got = run_device(inp, 4, 4, 1.0, flags=GENERIC, backward=False)
    o64, lse64 = orc.forward_windowed(*[x.double() for x in inp[:5]], 4, 4, 1.0)
    assert torch.allclose(got["out"].cpu().double(), o64, rtol=1e-4, atol=1e-6)
    assert torch.allclose(got["lse"].cpu().double(), lse64, rtol=1e-5, atol=1e-5)
    assert abs(got["lse"][0, 0, 0].item() - math.log(1e-8)) < 1e-3


def test_deterministic_and_gradient_accumulation():
    """simplicial/test_correctness.py:290-318, 402-421: two runs give identical
    bits; a second backward doubles .grad."""
    inp = make_inputs(2, 80, 2, 32, seed=42)
    a = run_device(inp, 12, 6, flags=GENERIC)
    b = run_device(inp, 12, 6, flags=GENERIC)
    for name in a:
        assert torch.equal(a[name], b[name]), name
    from simplical_attn_amd import TwoSimplicialAttention
    dev = torch.device("cuda:0")
    leaves = [x.to(dev).requires_grad_(True) for x in inp[:5]]
    attn = TwoSimplicialAttention(32, 12, 6)
    attn(*leaves).sum().backward()
    first = [x.grad.clone() for x in leaves]
    attn(*leaves).sum().backward()
    for g, x in zip(first, leaves):
        assert torch.allclose(x.grad, 2 * g, atol=1e-4)


def test_finite_differences():
    """simplicial/test_correctness.py:256-288 re-expressed: central differences
    of sum(O*dO) on sampled elements, fp32 inputs."""
    from simplical_attn_amd import TwoSimplicialAttention
    dev = torch.device("cuda:0")
    inp = make_inputs(1, 16, 1, 8, seed=5, mag=0.7)
    dout = inp[5].to(dev)
    attn = TwoSimplicialAttention(8, 4, 4)
    got = run_device(inp, 4, 4, flags=GENERIC)
    base = [x.to(dev) for x in inp[:5]]
    g = torch.Generator().manual_seed(0)
    eps = 1e-2
    for t, name in enumerate(("dq", "dk1", "dk2", "dv1", "dv2")):
        flat_idx = torch.randperm(base[t].numel(), generator=g)[:12]
        for idx in flat_idx.tolist():
            plus = [x.clone() for x in base]
            minus = [x.clone() for x in base]
            plus[t].view(-1)[idx] += eps
            minus[t].view(-1)[idx] -= eps
            num = ((attn(*plus) * dout).sum() - (attn(*minus) * dout).sum()).item() / (2 * eps)
            ana = got[name].view(-1)[idx].item()
            assert abs(num - ana) <= 2e-2 * max(1.0, abs(ana)), (name, idx, num, ana)


def test_strided_inputs_and_needs_input_grad():
    """Per-tensor strides (a packed [B,N,5,H,D] projection sliced five ways) and
    gradients requested for a subset of the inputs (triton_impl.py:73-77)."""
    from simplical_attn_amd import TwoSimplicialAttentionFunction as Fn
    dev = torch.device("cuda:0")
    B, N, H, D = 2, 48, 2, 32
    inp = make_inputs(B, N, H, D, seed=9)
    packed = torch.stack(inp[:5], dim=2).to(dev)            # [B,N,5,H,D]
    views = [packed[:, :, t] for t in range(5)]
    assert not views[0].is_contiguous()
    leaves = [v.detach().requires_grad_(t in (0, 2, 3)) for t, v in enumerate(views)]
    out = Fn.apply(*leaves, 8, 5, None, 0.0, 0.0)
    out.backward(inp[5].to(dev))
    want = oracle_all(inp, 8, 5)
    assert_close_rel(out.detach(), want["out"], 2e-5, "out")
    assert leaves[1].grad is None and leaves[4].grad is None
    for t, name in ((0, "dq"), (2, "dk2"), (3, "dv1")):
        assert_close_rel(leaves[t].grad, want[name], 2e-5, name)


def test_half_open_window_convention():
    """window_inclusive = 0 masks (i-w, i] like the reference's device kernels
    (simplicial/kernels.py:133-136): equal to the closed window with w-1."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    inp = [x.to(dev) for x in make_inputs(1, 40, 2, 16, seed=13, with_dout=False)]
    a, la = sa.simplicial_forward(*inp, 6, 4, flags=GENERIC, window_inclusive=False)
    b, lb = sa.simplicial_forward(*inp, 5, 3, flags=GENERIC, window_inclusive=True)
    assert torch.equal(a, b) and torch.equal(la, lb)
    # and against the oracle's own half-open windows, forward and gradients, to the fp32 bar
    host = make_inputs(1, 40, 2, 16, seed=13)
    got = run_device(host, 6, 4, flags=GENERIC, inclusive=False)
    want = oracle_all(host, 6, 4, inclusive=False)
    for name in ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2"):
        assert torch.allclose(got[name].cpu().double(), want[name], rtol=1e-5, atol=1e-5), name


def test_error_codes():
    from simplical_attn_amd import _lib, simplicial_forward
    dev = torch.device("cuda:0")
    x = torch.zeros(1, 8, 1, 260, device=dev)
    with pytest.raises(_lib.Sa2Error) as e:
        simplicial_forward(x, x, x, x, x, 4, 4)
    assert e.value.status == -3
    y = torch.zeros(1, 8, 1, 16, device=dev)
    with pytest.raises(_lib.Sa2Error) as e:
        simplicial_forward(y, y, y, y, y, -1, 4)
    assert e.value.status == -5
    with pytest.raises(RuntimeError):
        simplicial_forward(y.cpu(), y.cpu(), y.cpu(), y.cpu(), y.cpu(), 4, 4)


def test_exact_entry_points_run_the_fp32_kernels():
    """two_simplicial_attention_exact / TwoSimplicialAttentionExact (argument lists of
    simplicial/reference.py:8, 79): bf16 tensors, fp32 arithmetic, differentiable; they agree with
    the oracle more closely than the bf16 parity bar and with the MFMA kernels within it."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    inp = make_inputs(1, 96, 2, 64, seed=9, dtype=torch.bfloat16)
    leaves = [x.to(dev).requires_grad_(True) for x in inp[:5]]
    out = sa.TwoSimplicialAttentionExact(64, 20, 6, k2_bias=0.1)(*leaves)
    out.backward(inp[5].to(dev))
    want = oracle_all(inp, 20, 6, None, 0.1, 0.0)
    assert_close_rel(out, want["out"], 5e-3, "out")
    for name, leaf in zip(("dq", "dk1", "dk2", "dv1", "dv2"), leaves):
        assert_close_rel(leaf.grad, want[name], 1e-2, name)
    fast = sa.TwoSimplicialAttention(64, 20, 6, k2_bias=0.1)(*[x.to(dev) for x in inp[:5]])
    assert_close_rel(fast, out.detach().float().cpu(), 2e-2, "mfma vs exact kernels")


def test_rowdot():
    from simplical_attn_amd import compute_D_kernel, simplicial_rowdot
    dev = torch.device("cuda:0")
    a = torch.randn(2, 33, 3, 40, device=dev, dtype=torch.bfloat16)
    b = torch.randn(2, 33, 3, 40, device=dev, dtype=torch.bfloat16)
    want = (a.float() * b.float()).sum(-1)                           # [B,N,H]
    assert torch.allclose(simplicial_rowdot(a, b), want.permute(0, 2, 1), rtol=1e-5, atol=1e-5)
    # the reference helper's layout and dtype (simplicial/kernels.py:569-571): [B,N,H] like dO
    got = compute_D_kernel(a, b)
    assert got.shape == (2, 33, 3) and got.dtype == torch.bfloat16
    assert torch.equal(got, want.to(torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", [16, 32, 64, 128, 256, 40])
def test_rowdot_kernels(D, dtype):
    """The 16-byte-per-lane kernel (16-bit elements, D = 8 << n, aligned rows), the element-wise one
    (everything else), and views whose rows are not 16-byte aligned."""
    from simplical_attn_amd import simplicial_rowdot
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(D)
    a = torch.randn(2, 37, 3, D, generator=g).to(dtype).to(dev)
    b = torch.randn(2, 37, 3, D, generator=g).to(dtype).to(dev)
    want = (a.double() * b.double()).sum(-1).permute(0, 2, 1)
    assert torch.allclose(simplicial_rowdot(a, b).double(), want, rtol=1e-5, atol=1e-4)
    wide = torch.randn(2, 37, 3, D + 4, generator=g).to(dtype).to(dev)        # rows 8 bytes off the 16-byte grid
    av = wide[..., 4:]
    want = (av.double() * b.double()).sum(-1).permute(0, 2, 1)
    assert torch.allclose(simplicial_rowdot(av, b).double(), want, rtol=1e-5, atol=1e-4)


def test_broadcast_views_are_accepted():
    """Losses that hand backward an expanded gradient (stride 0 along a summed axis) and keys
    expanded over heads (stride 0 on H) run, as the reference's stride-generic launch lets them
    (simplicial/triton_impl.py:38-45), and give what the materialised tensors give."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    inp = make_inputs(2, 70, 3, 64, seed=21, dtype=torch.float32)
    attn = sa.TwoSimplicialAttention(64, 12, 5)

    def grads_of(loss_of, k1_of=lambda t: t):
        leaves = [x.to(dev).requires_grad_(True) for x in inp[:5]]
        args = list(leaves)
        args[1] = k1_of(leaves[1])
        loss_of(attn(*args)).backward()
        return [t.grad for t in leaves]

    w = inp[5].to(dev)
    # sum over N: autograd expands a [B,H,D] gradient with stride 0 on N
    a = grads_of(lambda o: (o.sum(dim=1) * w[:, 0]).sum())
    b = grads_of(lambda o: (o * w[:, :1].expand_as(o).contiguous()).sum())
    for x, y in zip(a, b):
        assert torch.allclose(x, y, rtol=1e-5, atol=1e-6)
    # sum over everything but D: strides (0, 0, 0, 1)
    a = grads_of(lambda o: (o.sum(dim=(0, 1, 2)) * w[0, 0, 0]).sum())
    b = grads_of(lambda o: (o * w[:1, :1, :1].expand_as(o).contiguous()).sum())
    for x, y in zip(a, b):
        assert torch.allclose(x, y, rtol=1e-5, atol=1e-6)
    # one key head shared by all query heads (MQA): k1 expanded over H
    a = grads_of(lambda o: (o * w).sum(), k1_of=lambda t: t[:, :, :1].expand(-1, -1, 3, -1))
    b = grads_of(lambda o: (o * w).sum(), k1_of=lambda t: t[:, :, :1].expand(-1, -1, 3, -1).contiguous())
    for x, y in zip(a, b):
        assert torch.allclose(x, y, rtol=1e-5, atol=1e-6)
    want = oracle_all([inp[0], inp[1][:, :, :1].expand(-1, -1, 3, -1), *inp[2:]], 12, 5)
    out = attn(inp[0].to(dev), inp[1].to(dev)[:, :, :1].expand(-1, -1, 3, -1), *[x.to(dev) for x in inp[2:5]])
    assert torch.allclose(out.cpu().double(), want["out"], rtol=1e-5, atol=1e-5)
