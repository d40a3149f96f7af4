"""Kernel choice and argument plumbing on the GPU.

(1) The layout guards of the MFMA path: 16-bit tensors whose rows are not on the 16-byte grid the
direct global->LDS loads need must take the fp32 kernels under the default dispatch - same bits as
a forced fp32-kernel run, and within the 16-bit bar of the oracle - and a forced MFMA run must
refuse them without launching anything.  Nothing misaligned is ever given to an MFMA kernel here.
(2) The window convention is an argument of every entry point (module, autograd Function, traced
op): each must give what the direct call gives for the half-open windows of the reference's
device kernels (simplicial/kernels.py:133-136), against the oracle with inclusive=False."""
import pytest
import torch

from simplical_attn_amd import _lib
from tests.util import assert_close_rel, make_inputs, oracle_all

pytestmark = pytest.mark.gpu
AUTO, GENERIC, MFMA = 0, 1, 2
NAMES = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")


def _step(sa, x, w1, w2, flags):
    out, lse = sa.simplicial_forward(*x[:5], w1, w2, flags=flags)
    grads = sa.simplicial_backward(*x[:5], out, lse, x[5], w1, w2, flags=flags)
    return dict(zip(NAMES, (out, lse, *grads)))


@pytest.mark.parametrize("which", ["rows 8 bytes off the grid", "row stride not a multiple of 16 bytes"])
def test_unaligned_16bit_rows_take_the_fp32_kernels(which):
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2 = 1, 160, 2, 128, 48, 9
    host = make_inputs(B, N, H, D, seed=77, dtype=torch.bfloat16)
    if which.startswith("rows 8"):
        # every row starts 4 elements (8 bytes) into a wider row: base pointer off the 16-byte grid
        wide = [torch.zeros(B, N, H, D + 8, dtype=torch.bfloat16, device=dev) for _ in host]
        views = [w[..., 4:4 + D] for w in wide]
    else:
        # rows of D + 4 elements: base aligned, every second row 8 bytes off the grid
        wide = [torch.zeros(B, N, H, D + 4, dtype=torch.bfloat16, device=dev) for _ in host]
        views = [w[..., :D] for w in wide]
    for v, x in zip(views, host):
        v.copy_(x)
        assert v.stride(-1) == 1 and not v.is_contiguous()
    assert views[0].data_ptr() % 16 == (8 if which.startswith("rows 8") else 0)
    with pytest.raises(_lib.Sa2Error) as err:
        sa.simplicial_forward(*views[:5], w1, w2, flags=MFMA)
    assert err.value.status == -8
    auto = _step(sa, views, w1, w2, AUTO)
    exact = _step(sa, views, w1, w2, GENERIC)
    want = oracle_all(host, w1, w2)
    for name in NAMES:
        assert torch.equal(auto[name], exact[name]), name                    # the guard routed to the fp32 kernels
        assert_close_rel(auto[name], want[name], 2e-2, name + " " + which, atol=1e-5)
    # the same data in aligned tensors does take the MFMA kernels (and differs in its rounding)
    aligned = _step(sa, [x.to(dev) for x in host], w1, w2, AUTO)
    forced = _step(sa, [x.to(dev) for x in host], w1, w2, MFMA)
    # (AUTO leaves the pre-pass kernels out on small grids; w2 = 9 takes none either way)
    for name in NAMES:
        assert torch.equal(aligned[name], forced[name]), name
    assert not torch.equal(aligned["out"], exact["out"])


def test_window_convention_is_an_argument_of_every_entry_point():
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2 = 2, 130, 2, 64, 33, 9
    host = make_inputs(B, N, H, D, seed=5, dtype=torch.bfloat16)
    dout = host[5].to(dev)
    want = {True: oracle_all(host, w1, w2, inclusive=True), False: oracle_all(host, w1, w2, inclusive=False)}
    assert (want[True]["out"] - want[False]["out"]).abs().max() > 1e-2          # the conventions differ visibly

    def grads_of(fn):
        leaves = [x.to(dev).requires_grad_(True) for x in host[:5]]
        out = fn(*leaves)
        out.backward(dout)
        return [out.detach()] + [t.grad for t in leaves]

    for inclusive in (True, False):
        runs = {
            "module": grads_of(sa.TwoSimplicialAttention(D, w1, w2, window_inclusive=inclusive)),
            "function": grads_of(lambda *x: sa.TwoSimplicialAttentionFunction.apply(*x, w1, w2, None, 0.0, 0.0,
                                                                                    inclusive)),
            "op": grads_of(lambda *x: sa.two_simplicial_attention(*x, w1, w2, window_inclusive=inclusive)),
            "exact": grads_of(sa.TwoSimplicialAttentionExact(D, w1, w2, window_inclusive=inclusive)),
        }
        for name, got in runs.items():
            for tname, g in zip(("out", "dq", "dk1", "dk2", "dv1", "dv2"), got):
                assert_close_rel(g, want[inclusive][tname], 2e-2, "%s %s inclusive=%s" % (name, tname, inclusive))
        for a, b in zip(runs["module"], runs["function"]):
            assert torch.equal(a, b)
        for a, b in zip(runs["module"], runs["op"]):
            assert torch.equal(a, b)
    # the reference's ten-argument positional call (simplicial/triton_impl.py:183-186) is the closed window
    ten = grads_of(lambda *x: sa.TwoSimplicialAttentionFunction.apply(*x, w1, w2, None, 0.0, 0.0))
    dflt = grads_of(sa.TwoSimplicialAttention(D, w1, w2))
    for a, b in zip(ten, dflt):
        assert torch.equal(a, b)


def test_backward_rejects_mismatched_saved_tensors_on_the_device():
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    x = [t.to(dev) for t in make_inputs(1, 64, 2, 64, seed=1, dtype=torch.bfloat16)]
    out, lse = sa.simplicial_forward(*x[:5], 8, 8)
    with pytest.raises(ValueError, match="lse must be contiguous"):
        sa.simplicial_backward(*x[:5], out, lse.transpose(1, 2).contiguous(), x[5], 8, 8)
    with pytest.raises(ValueError, match="float32"):
        sa.simplicial_backward(*x[:5], out, lse.half(), x[5], 8, 8)
    with pytest.raises(ValueError, match="dout must match q"):
        sa.simplicial_backward(*x[:5], out, lse, x[5].float(), 8, 8)
    with pytest.raises(ValueError, match="out must match q"):
        sa.simplicial_backward(*x[:5], out.cpu(), lse, x[5], 8, 8)
    from simplical_attn_amd.compiled_op import backward_op
    with pytest.raises(ValueError, match="out must match q"):
        backward_op(*x[:5], out[:, :32], lse, x[5], 8, 8, 0.125, 0.0, 0.0)
