"""The torch.library registration: fake-tensor shapes on CPU, tracing and gradients on the GPU."""
import pytest
import torch

import simplical_attn_amd as sa
from simplical_attn_amd.compiled_op import backward_op, forward_op
from tests.util import make_inputs


def test_fake_implementations_give_shapes_and_dtypes():
    B, N, H, D = 2, 40, 3, 64
    x = [torch.empty(B, N, H, D, dtype=torch.bfloat16, device="meta") for _ in range(6)]
    out, lse = forward_op(*x[:5], 8, 4, 0.125, 0.0, 0.0)
    assert out.shape == (B, N, H, D) and out.dtype == torch.bfloat16
    assert lse.shape == (B, H, N) and lse.dtype == torch.float32
    grads = backward_op(*x[:5], out, lse, x[5], 8, 4, 0.125, 0.0, 0.0)
    assert len(grads) == 5 and all(g.shape == (B, N, H, D) and g.dtype == torch.bfloat16 for g in grads)


def test_fake_outputs_are_contiguous_like_the_real_ones():
    """The kernels' results are freshly allocated contiguous tensors whatever the strides of the
    inputs; the fake implementations must say the same or compiled graphs mis-address them."""
    B, N, H, D = 2, 40, 3, 64
    x = [torch.empty(B, H, N, D, dtype=torch.bfloat16, device="meta").transpose(1, 2) for _ in range(6)]
    assert not x[0].is_contiguous()
    out, lse = forward_op(*x[:5], 8, 4, 0.125, 0.0, 0.0)
    want = torch.empty(B, N, H, D, device="meta").stride()
    assert out.shape == (B, N, H, D) and out.stride() == want
    assert lse.stride() == torch.empty(B, H, N, device="meta").stride()
    grads = backward_op(*x[:5], out, lse, x[5], 8, 4, 0.125, 0.0, 0.0)
    assert all(g.shape == (B, N, H, D) and g.stride() == want for g in grads)


@pytest.mark.gpu
def test_traced_op_matches_the_eager_function():
    dev = torch.device("cuda:0")
    inp = [t.to(dev) for t in make_inputs(1, 160, 2, 128, seed=5, dtype=torch.bfloat16)]
    w1, w2 = 48, 9

    def f(q, k1, k2, v1, v2):
        return sa.two_simplicial_attention(q, k1, k2, v1, v2, w1, w2, None, 0.1, -0.1) * 2.0

    eager = [t.clone().requires_grad_(True) for t in inp[:5]]
    ref = sa.TwoSimplicialAttentionFunction.apply(*eager, w1, w2, None, 0.1, -0.1) * 2.0
    ref.backward(inp[5])
    traced = [t.clone().requires_grad_(True) for t in inp[:5]]
    out = torch.compile(f, backend="aot_eager", fullgraph=True)(*traced)
    out.backward(inp[5])
    assert torch.equal(out, ref)
    for a, b in zip(traced, eager):
        assert torch.equal(a.grad, b.grad)
