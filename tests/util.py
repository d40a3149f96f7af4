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


# Measured parity errors, max|got-want| / max|want| per (label, tensor); the worst value seen is
# kept and the table is printed at the end of the session (tests/conftest.py).
MEASURED = {}


def record(label, name, got, want):
    err = rel_err(got, want)
    key = (label, name)
    MEASURED[key] = max(MEASURED.get(key, 0.0), err)
    return err


def rel_err(got, want):
    """max|got-want| / max|want| (the bf16 parity measure)."""
    want = want.double()
    return ((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def assert_close_rel(got, want, tol, what, atol=1e-6, label=None):
    """max|got-want| <= tol*max|want| + atol.  The small absolute floor only
    matters for tensors that are ~0 by cancellation (e.g. dq when every window
    holds a single triple and only the 1e-8 epsilon keeps it from vanishing).
    With `label` the measured relative error goes into the session's table."""
    want = want.double()
    diff = (got.double().cpu() - want).abs().max().item()
    bound = tol * want.abs().max().item() + atol
    if label is not None:
        record(label, what.split()[0], got, want)
    assert diff <= bound, "%s: max|diff| = %.3e > %.3e (max|ref| = %.3e)" % (what, diff, bound, want.abs().max().item())


def oracle_all(inputs, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, dtype=torch.float64, rows=None,
               inclusive=True):
    """fp64 (default) oracle on the exact values in `inputs` (q,k1,k2,v1,v2,dout):
    returns dict with out, lse and the five gradients."""
    q, k1, k2, v1, v2, dout = [x.to(dtype) for x in inputs]
    if rows is not None:
        dout = dout[:, rows[0]:rows[1]]
    res = orc.grads_windowed(q, k1, k2, v1, v2, dout, w1, w2, scale, k2_bias, v2_bias, rows=rows,
                             compute_dtype=dtype, inclusive=inclusive)
    keys = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")
    return dict(zip(keys, res))


def single_triple(N, w1, w2, inclusive=True):
    """Every query sees exactly one (j, k) pair, itself."""
    r1, r2 = (w1, w2) if inclusive else (w1 - 1, w2 - 1)
    return N == 1 or (r1 == 0 and r2 == 0)


def cancellation_bounds(inputs, want_out, scale=None, k2_bias=0.0, v2_bias=0.0):
    """Elementwise bounds on |dq|, |dk1|, |dk2| for problems where every query sees one triple.

    There P = 1 (up to the 1e-8 epsilon), dP_i = sum_d dO*v2~*v1 = sum_d dO*O = D_i, and
    dS = P*(dP - D) vanishes: the three gradients are exactly ~0.  A 16-bit kernel forms dP from
    rounded products dO*v2~ and D from the rounded output, each term off by at most half an ulp
    (2^-9 relative for bf16), so what it returns is rounding noise with
        |dS_i| <= 2^-8 * sum_d |dO_id * O_id|
    and dq_i = scale*dS_i*k1_i*k2~_i, dk1_i = scale*dS_i*q_i*k2~_i, dk2_i = scale*dS_i*q_i*k1_i.
    The bounds are these products, element by element (1e-6 added for the fp32 arithmetic):
    a gradient that is small but not of this shape fails them."""
    q, k1, k2, v1, v2, dout = [x.double() for x in inputs]
    D = q.shape[-1]
    if scale is None:
        scale = D ** -0.5
    ds = 2.0 ** -8 * (dout * want_out.double()).abs().sum(-1, keepdim=True)
    k2b = k2 + k2_bias
    return {"dq": scale * ds * (k1 * k2b).abs() + 1e-6,
            "dk1": scale * ds * (q * k2b).abs() + 1e-6,
            "dk2": scale * ds * (q * k1).abs() + 1e-6}


def assert_within(got, bound, what):
    excess = (got.double().cpu().abs() - bound).max().item()
    assert excess <= 0, "%s: exceeds its rounding-noise bound by %.3e" % (what, excess)


def run_device(inputs, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, flags=0, backward=True, inclusive=True):
    """Runs the HIP path through the autograd Function on cuda:0; returns the
    same dict as oracle_all (tensors on the GPU) plus lse from a direct call."""
    import simplical_attn_amd as sa
    Fn = sa.TwoSimplicialAttentionFunction
    dev = torch.device("cuda:0")
    leaves = [x.to(dev).requires_grad_(backward) for x in inputs[:5]]
    out = Fn.apply(*leaves, w1, w2, scale, k2_bias, v2_bias, inclusive, flags)
    res = {"out": out.detach()}
    _, res["lse"] = sa.simplicial_forward(*[x.detach() for x in leaves], w1, w2, scale, k2_bias, v2_bias,
                                          flags=flags, window_inclusive=inclusive)
    if backward:
        out.backward(inputs[5].to(dev))
        for name, leaf in zip(("dq", "dk1", "dk2", "dv1", "dv2"), leaves):
            res[name] = leaf.grad
    return res
