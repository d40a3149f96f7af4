"""Shared helpers of the parity tests."""
import torch

from oracle import simplicial_oracle as orc

NAMES = ("q", "k1", "k2", "v1", "v2")


def make_inputs(B, N, H, D, seed, dtype=torch.float32, mag=1.0, qk_mag=None, with_dout=True):
    """iid normal tensors from a seeded CPU generator, generated in fp32 and
    rounded to `dtype`; returns the rounded values (as `dtype`, on CPU).  Order:
    q, k1, k2, v1, v2 (, dout).  qk_mag scales q, k1, k2 only."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for t in range(6 if with_dout else 5):
        x = torch.randn(B, N, H, D, generator=g, dtype=torch.float32)
        x = x * (qk_mag if (qk_mag is not None and t < 3) else mag)
        out.append(x.to(dtype))
    return out


def rel_err(got, want):
    """max|got-want| / max|want| (the bf16 parity measure)."""
    want = want.double()
    return ((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def assert_close_rel(got, want, tol, what, atol=1e-6):
    """max|got-want| <= tol*max|want| + atol.  The small absolute floor only
    matters for tensors that are ~0 by cancellation (e.g. dq when every window
    holds a single triple and only the 1e-8 epsilon keeps it from vanishing)."""
    want = want.double()
    diff = (got.double().cpu() - want).abs().max().item()
    bound = tol * want.abs().max().item() + atol
    assert diff <= bound, "%s: max|diff| = %.3e > %.3e (max|ref| = %.3e)" % (what, diff, bound, want.abs().max().item())


def oracle_all(inputs, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, dtype=torch.float64, rows=None):
    """fp64 (default) oracle on the exact values in `inputs` (q,k1,k2,v1,v2,dout):
    returns dict with out, lse and the five gradients."""
    q, k1, k2, v1, v2, dout = [x.to(dtype) for x in inputs]
    if rows is not None:
        dout = dout[:, rows[0]:rows[1]]
    res = orc.grads_windowed(q, k1, k2, v1, v2, dout, w1, w2, scale, k2_bias, v2_bias, rows=rows,
                             compute_dtype=dtype)
    keys = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")
    return dict(zip(keys, res))


def run_device(inputs, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, flags=0, backward=True):
    """Runs the HIP path through the autograd Function on cuda:0; returns the
    same dict as oracle_all (tensors on the GPU) plus lse from a direct call."""
    import simplical_attn_amd as sa
    from simplical_attn_amd.simplicial_attn import TwoSimplicialAttentionFunction as Fn
    dev = torch.device("cuda:0")
    leaves = [x.to(dev).requires_grad_(backward) for x in inputs[:5]]
    old = Fn.kernel_flags
    Fn.kernel_flags = flags
    try:
        out = Fn.apply(*leaves, w1, w2, scale, k2_bias, v2_bias)
        res = {"out": out.detach()}
        _, res["lse"] = sa.simplicial_forward(*[x.detach() for x in leaves], w1, w2, scale, k2_bias, v2_bias,
                                              flags=flags)
        if backward:
            out.backward(inputs[5].to(dev))
            for name, leaf in zip(("dq", "dk1", "dk2", "dv1", "dv2"), leaves):
                res[name] = leaf.grad
    finally:
        Fn.kernel_flags = old
    return res
