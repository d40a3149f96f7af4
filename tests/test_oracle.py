"""Pins the CPU oracle (oracle/simplicial_oracle.py) without ever running the
reference: the reference's tests hold no golden vectors for this path
(simplicial/test_correctness.py generates random inputs at run time), so the
oracle is pinned by what the mathematics fixes.  Each check is chosen so that a
plausible mistake (window off by one, dropped bias, missing epsilon, swapped
operand, wrong scale) fails at least one of them."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import simplicial_oracle as orc


def rnd(shape, seed, dtype=torch.float64, mag=1.0):
    g = torch.Generator().manual_seed(seed)
    return mag * torch.randn(*shape, generator=g, dtype=dtype)


def five(B, N, H, D, seed, dtype=torch.float64, mag=1.0):
    return [rnd((B, N, H, D), seed * 10 + t, dtype, mag) for t in range(5)]


def brute_force(q, k1, k2, v1, v2, w1, w2, scale, k2_bias=0.0, v2_bias=0.0):
    """Dense N^3 evaluation: all logits by one einsum, two band masks, exp,
    divide by (sum + 1e-8).  Shares no windowing or tiling code with the oracle."""
    B, N, H, D = q.shape
    k2b, v2b = k2 + k2_bias, v2 + v2_bias
    s = torch.einsum("bihd,bjhd,bkhd->bhijk", q, k1, k2b) * scale
    idx = torch.arange(N)
    i, j, k = idx[:, None, None], idx[None, :, None], idx[None, None, :]
    mask = (j <= i) & (j >= i - w1) & (k <= i) & (k >= i - w2)
    w = torch.exp(s) * mask
    tot = w.sum(dim=(-1, -2))
    out = torch.einsum("bhijk,bjhd,bkhd->bihd", w, v1, v2b) / (tot.permute(0, 2, 1)[..., None] + 1e-8)
    return out, torch.log(tot + 1e-8)


def band_mask(N, w):
    idx = torch.arange(N)
    return (idx[None, :] <= idx[:, None]) & (idx[None, :] >= idx[:, None] - w)


CASES = [  # B, N, H, D, w1, w2, k2_bias, v2_bias
    (1, 12, 1, 4, 3, 2, 0.0, 0.0),
    (2, 20, 2, 8, 5, 7, 0.1, -0.2),
    (1, 24, 2, 6, 30, 4, 1.0, 0.5),      # w1 >= N
    (1, 16, 1, 8, 0, 0, 0.0, 0.0),       # single (i,i,i) triple
    (1, 33, 3, 5, 1, 9, -0.1, 0.2),
]


@pytest.mark.parametrize("case", CASES)
def test_literal_and_windowed_match_brute_force(case):
    B, N, H, D, w1, w2, kb, vb = case
    t = five(B, N, H, D, seed=N)
    scale = 0.37
    ref, ref_lse = brute_force(*t, w1, w2, scale, kb, vb)
    lit = orc.literal_loop(*t, w1, w2, scale, kb, vb)
    win, lse = orc.forward_windowed(*t, w1, w2, scale, kb, vb, chunk=7)
    assert torch.allclose(lit, ref, rtol=1e-11, atol=1e-12)
    assert torch.allclose(win, ref, rtol=1e-11, atol=1e-12)
    assert torch.allclose(lse, ref_lse, rtol=1e-11, atol=1e-12)


def test_default_scale_is_rsqrt_d():
    t = five(1, 10, 1, 16, seed=3)
    a = orc.literal_loop(*t, 4, 4)
    b, _ = brute_force(*t, 4, 4, 1.0 / math.sqrt(16))
    c, _ = orc.forward_windowed(*t, 4, 4)
    assert torch.allclose(a, b, rtol=1e-11, atol=1e-12)
    assert torch.allclose(c, b, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("via_bias", [False, True])
def test_reduces_to_sdpa_when_second_pair_is_ones(via_bias):
    """k2 = v2 = 1: the weights replicate over k and cancel, so the output is
    ordinary banded softmax attention of (q, k1, v1)."""
    B, N, H, D, w1, w2 = 2, 40, 2, 8, 6, 11
    q, k1, _, v1, _ = five(B, N, H, D, seed=5)
    if via_bias:
        k2, v2, kb, vb = torch.zeros_like(q), torch.zeros_like(q), 1.0, 1.0
    else:
        k2, v2, kb, vb = torch.ones_like(q), torch.ones_like(q), 0.0, 0.0
    scale = 0.3
    sd = F.scaled_dot_product_attention(q.transpose(1, 2), k1.transpose(1, 2), v1.transpose(1, 2),
                                        attn_mask=band_mask(N, w1), scale=scale).transpose(1, 2)
    for fn in (orc.literal_loop, lambda *a: orc.forward_windowed(*a)[0]):
        out = fn(q, k1, k2, v1, v2, w1, w2, scale, kb, vb)
        assert torch.allclose(out, sd, rtol=1e-7, atol=1e-8)   # epsilon term is ~1e-8 relative


def test_reduces_to_sdpa_on_the_other_side():
    B, N, H, D, w1, w2 = 1, 36, 2, 8, 9, 4
    q, _, k2, _, v2 = five(B, N, H, D, seed=6)
    one = torch.ones_like(q)
    scale = 0.25
    sd = F.scaled_dot_product_attention(q.transpose(1, 2), k2.transpose(1, 2), v2.transpose(1, 2),
                                        attn_mask=band_mask(N, w2), scale=scale).transpose(1, 2)
    for fn in (orc.literal_loop, lambda *a: orc.forward_windowed(*a)[0]):
        out = fn(q, one, k2, one, v2, w1, w2, scale)
        assert torch.allclose(out, sd, rtol=1e-7, atol=1e-8)


def test_w2_zero_closed_form():
    """w2 = 0: k = i only, so O_i = v2_i * SDPA(q_i*k2_i, k1, v1)."""
    B, N, H, D, w1 = 1, 30, 2, 8, 5
    q, k1, k2, v1, v2 = five(B, N, H, D, seed=7)
    kb, vb, scale = 0.3, -0.4, 0.2
    sd = F.scaled_dot_product_attention((q * (k2 + kb)).transpose(1, 2), k1.transpose(1, 2),
                                        v1.transpose(1, 2), attn_mask=band_mask(N, w1),
                                        scale=scale).transpose(1, 2)
    want = sd * (v2 + vb)
    for fn in (orc.literal_loop, lambda *a: orc.forward_windowed(*a)[0]):
        out = fn(q, k1, k2, v1, v2, w1, 0, scale, kb, vb)
        assert torch.allclose(out, want, rtol=1e-7, atol=1e-8)


def test_zero_query_gives_window_means_and_counts():
    """q = 0: every weight is 1, O_i = mean_J v1 * mean_K v2 (up to epsilon) and
    LSE_i = log(|J(i)|*|K(i)| + 1e-8) with |J(i)| = min(i,w1)+1: pins the
    closed-interval window [i-w, i]."""
    B, N, H, D, w1, w2 = 1, 25, 1, 4, 6, 3
    _, k1, k2, v1, v2 = five(B, N, H, D, seed=8)
    q = torch.zeros_like(k1)
    out, lse = orc.forward_windowed(q, k1, k2, v1, v2, w1, w2, 1.0, 0.0, 0.25)
    lit = orc.literal_loop(q, k1, k2, v1, v2, w1, w2, 1.0, 0.0, 0.25)
    for i in range(N):
        nj, nk = min(i, w1) + 1, min(i, w2) + 1
        sv1 = v1[:, i - nj + 1:i + 1].sum(1)
        sv2 = (v2[:, i - nk + 1:i + 1] + 0.25).sum(1)
        want = sv1 * sv2 / (nj * nk + 1e-8)
        assert torch.allclose(out[:, i], want, rtol=1e-12, atol=1e-13)
        assert torch.allclose(lit[:, i], want, rtol=1e-12, atol=1e-13)
        assert abs(lse[0, 0, i].item() - math.log(nj * nk + 1e-8)) < 1e-12


def test_row_zero_and_epsilon():
    """Row 0 sees one triple: O_0 = v1_0*v2_0*e^s/(e^s+1e-8); with a very
    negative logit the epsilon dominates and the output collapses to 0."""
    B, N, H, D = 1, 4, 1, 4
    q, k1, k2, v1, v2 = five(B, N, H, D, seed=9)
    for scale in (0.5, -40.0, -400.0, -40000.0):
        s = (q[:, 0] * k1[:, 0] * k2[:, 0]).sum(-1, keepdim=True).abs() * scale
        q0 = q.clone()
        q0[:, 0] = q[:, 0] * torch.sign((q[:, 0] * k1[:, 0] * k2[:, 0]).sum(-1, keepdim=True))
        es = torch.exp(s)
        want = v1[:, 0] * v2[:, 0] * es / (es + 1e-8)
        out, lse = orc.forward_windowed(q0, k1, k2, v1, v2, 2, 2, scale)
        lit = orc.literal_loop(q0, k1, k2, v1, v2, 2, 2, scale)
        assert torch.allclose(out[:, 0], want, rtol=1e-10, atol=1e-300)
        assert torch.allclose(lit[:, 0], want, rtol=1e-10, atol=1e-300)
        assert torch.allclose(lse[:, :, 0], torch.log(es + 1e-8)[..., 0], rtol=1e-10)


def test_swap_symmetry_and_bias_shift():
    B, N, H, D, w1, w2 = 1, 28, 2, 6, 7, 3
    q, k1, k2, v1, v2 = five(B, N, H, D, seed=10)
    a, la = orc.forward_windowed(q, k1, k2, v1, v2, w1, w2, 0.3)
    b, lb = orc.forward_windowed(q, k2, k1, v2, v1, w2, w1, 0.3)
    assert torch.allclose(a, b, rtol=1e-11, atol=1e-12) and torch.allclose(la, lb, rtol=1e-11)
    c, _ = orc.forward_windowed(q, k1, k2, v1, v2, w1, w2, 0.3, 0.7, -0.3)
    d, _ = orc.forward_windowed(q, k1, k2 + 0.7, v1, v2 - 0.3, w1, w2, 0.3)
    assert torch.allclose(c, d, rtol=1e-11, atol=1e-12)


def test_extreme_logits_stay_finite():
    """All-10.0 inputs (logits ~4000): the windowed restatement stays finite and
    equals the analytic answer (uniform weights -> v1*v2 = 100)."""
    q = torch.full((1, 16, 1, 16), 10.0, dtype=torch.float32)
    out, lse = orc.forward_windowed(q, q, q, q, q, 4, 4)
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.allclose(out, torch.full_like(out, 100.0), rtol=1e-5)


def test_rows_subset_equals_full():
    t = five(1, 50, 2, 8, seed=11)
    full, lse = orc.forward_windowed(*t, 9, 4, 0.3)
    part, lp = orc.forward_windowed(*t, 9, 4, 0.3, rows=(13, 37), chunk=5)
    assert torch.equal(part, full[:, 13:37]) or torch.allclose(part, full[:, 13:37], rtol=1e-13, atol=1e-14)
    assert torch.allclose(lp, lse[:, :, 13:37], rtol=1e-13)


def test_gradients_match_brute_force_autograd_and_gradcheck():
    B, N, H, D, w1, w2 = 1, 14, 2, 4, 4, 3
    t = five(B, N, H, D, seed=12)
    dout = rnd((B, N, H, D), 99)
    kb, vb, scale = 0.2, -0.1, 0.4
    leaves = [x.clone().requires_grad_(True) for x in t]
    o, _ = brute_force(*leaves, w1, w2, scale, kb, vb)
    (o * dout).sum().backward()
    res = orc.grads_windowed(*t, dout, w1, w2, scale, kb, vb, chunk=5)
    assert torch.allclose(res[0], o.detach(), rtol=1e-11, atol=1e-12)
    for g, leaf in zip(res[2:], leaves):
        assert torch.allclose(g, leaf.grad, rtol=1e-9, atol=1e-11)
    small = [x[:, :8].clone().requires_grad_(True) for x in t]
    fn = lambda *a: orc.forward_windowed(*a, 3, 2, scale, kb, vb, chunk=3)[0]
    assert torch.autograd.gradcheck(fn, small, eps=1e-6, atol=1e-6, rtol=1e-5)


def test_gradient_rows_subset_complete_for_inner_keys():
    """Gradients restricted to queries [r0,r1) are complete for K rows j with
    [j, j+w1] inside the range and K' rows k with [k, k+w2] inside it."""
    B, N, H, D, w1, w2 = 1, 40, 1, 4, 6, 3
    t = five(B, N, H, D, seed=13)
    dout = rnd((B, N, H, D), 98)
    full = orc.grads_windowed(*t, dout, w1, w2, 0.3)
    r0, r1 = 10, 30
    part = orc.grads_windowed(*t, dout[:, r0:r1], w1, w2, 0.3, rows=(r0, r1))
    assert torch.allclose(part[2][:, r0:r1], full[2][:, r0:r1], rtol=1e-11, atol=1e-12)        # dq
    assert torch.allclose(part[3][:, r0:r1 - w1], full[3][:, r0:r1 - w1], rtol=1e-11, atol=1e-12)  # dk1
    assert torch.allclose(part[4][:, r0:r1 - w2], full[4][:, r0:r1 - w2], rtol=1e-11, atol=1e-12)  # dk2


def test_fp32_literal_tracks_fp64():
    """The fp32 literal loop (the reference's own precision) agrees with the
    fp64 truth to fp32 rounding on the smallest benchmark-like shape."""
    t64 = five(1, 48, 2, 16, seed=14)
    t32 = [x.float() for x in t64]
    a = orc.literal_loop(*t32, 8, 4)
    b, _ = orc.forward_windowed(*[x.double() for x in t32], 8, 4)
    assert torch.allclose(a.double(), b, rtol=2e-5, atol=2e-6)


def test_count_triples():
    assert orc.count_triples(1, 128, 2, 32, 16) == 124032
    assert orc.count_triples(1, 8192, 16, 512, 32) == 2149480960
    n = 0
    for i in range(20):
        for j in range(max(0, i - 5), i + 1):
            for k in range(max(0, i - 2), i + 1):
                n += 1
    assert orc.count_triples(2, 20, 3, 5, 2) == 6 * n


# ---- the half-open windows of the reference's device kernels (simplicial/kernels.py:133-136) ----

def brute_force_half_open(q, k1, k2, v1, v2, w1, w2, scale, k2_bias=0.0, v2_bias=0.0):
    """brute_force with the masks as the device kernels write them:
    q_idx - w < kv_idx <= q_idx on both sides."""
    B, N, H, D = q.shape
    s = torch.einsum("bihd,bjhd,bkhd->bhijk", q, k1, k2 + k2_bias) * scale
    idx = torch.arange(N)
    i, j, k = idx[:, None, None], idx[None, :, None], idx[None, None, :]
    mask = ((i - w1) < j) & (j <= i) & ((i - w2) < k) & (k <= i)
    w = torch.exp(s) * mask
    tot = w.sum(dim=(-1, -2))
    out = torch.einsum("bhijk,bjhd,bkhd->bihd", w, v1, v2 + v2_bias) / (tot.permute(0, 2, 1)[..., None] + 1e-8)
    return out, torch.log(tot + 1e-8)


@pytest.mark.parametrize("case", [
    (1, 12, 1, 4, 3, 2, 0.0, 0.0),
    (2, 20, 2, 8, 5, 7, 0.1, -0.2),
    (1, 24, 2, 6, 30, 4, 1.0, 0.5),      # w1 >= N
    (1, 16, 1, 8, 1, 1, 0.0, 0.0),       # single (i,i,i) triple
    (1, 33, 3, 5, 2, 9, -0.1, 0.2),
])
def test_half_open_windows_match_brute_force(case):
    B, N, H, D, w1, w2, kb, vb = case
    t = five(B, N, H, D, seed=N + 100)
    dout = rnd((B, N, H, D), 77)
    scale = 0.41
    leaves = [x.clone().requires_grad_(True) for x in t]
    ref, ref_lse = brute_force_half_open(*leaves, w1, w2, scale, kb, vb)
    (ref * dout).sum().backward()
    lit = orc.literal_loop(*t, w1, w2, scale, kb, vb, inclusive=False)
    res = orc.grads_windowed(*t, dout, w1, w2, scale, kb, vb, chunk=7, inclusive=False)
    assert torch.allclose(lit, ref.detach(), rtol=1e-11, atol=1e-12)
    assert torch.allclose(res[0], ref.detach(), rtol=1e-11, atol=1e-12)
    assert torch.allclose(res[1], ref_lse.detach(), rtol=1e-11, atol=1e-12)
    for g, leaf in zip(res[2:], leaves):
        assert torch.allclose(g, leaf.grad, rtol=1e-9, atol=1e-11)
    # and it differs from the closed windows of the same w (one key more per side)
    closed, _ = orc.forward_windowed(*t, w1, w2, scale, kb, vb)
    assert not torch.allclose(closed[:, 1:], ref.detach()[:, 1:], rtol=1e-3, atol=1e-3)


def test_half_open_zero_query_counts_w_keys():
    """q = 0: LSE_i = log(|J(i)|*|K(i)| + 1e-8) with |J(i)| = min(i+1, w1): w keys, not w+1."""
    B, N, H, D, w1, w2 = 1, 25, 1, 4, 6, 3
    _, k1, k2, v1, v2 = five(B, N, H, D, seed=8)
    q = torch.zeros_like(k1)
    out, lse = orc.forward_windowed(q, k1, k2, v1, v2, w1, w2, 1.0, 0.0, 0.25, inclusive=False)
    for i in range(N):
        nj, nk = min(i + 1, w1), min(i + 1, w2)
        want = v1[:, i - nj + 1:i + 1].sum(1) * (v2[:, i - nk + 1:i + 1] + 0.25).sum(1) / (nj * nk + 1e-8)
        assert torch.allclose(out[:, i], want, rtol=1e-12, atol=1e-13)
        assert abs(lse[0, 0, i].item() - math.log(nj * nk + 1e-8)) < 1e-12


def test_half_open_rejects_empty_windows_and_counts_triples():
    t = five(1, 6, 1, 4, seed=2)
    with pytest.raises(ValueError):
        orc.forward_windowed(*t, 0, 3, inclusive=False)
    with pytest.raises(ValueError):
        orc.literal_loop(*t, 3, 0, inclusive=False)
    assert orc.count_triples(1, 128, 2, 32, 16, inclusive=False) == 113840
    assert orc.count_triples(1, 8192, 16, 512, 32, inclusive=False) == 2080418560
    n = sum(1 for i in range(20) for j in range(20) for k in range(20)
            if i - 5 < j <= i and i - 2 < k <= i)
    assert orc.count_triples(2, 20, 3, 5, 2, inclusive=False) == 6 * n
