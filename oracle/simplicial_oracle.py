"""CPU oracle for causal sliding-window 2-simplicial (trilinear) attention.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file;
only the tests, the smoke check and the benchmark's CPU-baseline leg do, and
only as the checker.  The shipped path is the HIP library and fails loudly when
that library is missing.

It restates, in this build's own code, the arithmetic of the reference's
PyTorch "gold standard":

    windows      J(i) = [max(0,i-w1), i],  K(i) = [max(0,i-w2), i]
                                               (simplicial/reference.py:41-45)
    biases       k2 <- k2 + k2_bias, v2 <- v2 + v2_bias
                                               (simplicial/reference.py:33-34)
    logit        s[i,j,k] = sum_d q[i,d]*k1[j,d]*k2[k,d]*scale
                                               (simplicial/reference.py:64)
    weight       w = exp(s)   (no max subtraction)
                                               (simplicial/reference.py:65)
    output       O[i] = sum_{j,k} w*(v1[j]*v2[k]) / (sum_{j,k} w + 1e-8)
                                               (simplicial/reference.py:68-74)
    scale        defaults to 1/sqrt(D)         (simplicial/reference.py:29-30)

The reference's device kernels mask half-open windows instead, (i-w, i], w keys
(simplicial/kernels.py:133-136: ``q_idx - w < kv_idx``).  ``inclusive=False`` selects that
convention in every function below; the default is reference.py's.

The reference never returns a log-sum-exp; the only definition in the
reference is the device kernels' ``m + log(l)`` (simplicial/kernels.py:164).
Here LSE is defined so that ``exp(s - LSE)`` is exactly the oracle's normalised
weight, i.e. ``LSE = log(sum w + 1e-8)``.

How each function is pinned (tests/test_oracle.py):
  literal_loop        brute-force dense N^3 einsum (fp64), scaled-dot-product
                      attention reductions (k2 = v2 = 1 and the mirror case),
                      w2 = 0 and w1 = w2 = 0 closed forms, q = 0 closed form
                      (pins the w+1-key window convention), row-0 closed form,
                      swap symmetry, bias == shifted input.
  forward_windowed    the same checks, plus equality with literal_loop.
  inclusive=False     the same brute force with strict lower bounds (j > i-w1, k > i-w2), the
                      q = 0 closed form with min(i+1, w) keys per window, and the published
                      triple counts of the half-open convention.
  grads_windowed      torch.autograd.gradcheck (fp64) on forward_windowed, the
                      closed-form gradients of the dense brute force (autograd
                      through an independent einsum formulation), and central
                      finite differences.
"""

import math

import torch


def default_scale(head_dim):
    """1/sqrt(D) (simplicial/reference.py:29-30)."""
    return 1.0 / math.sqrt(head_dim)


def literal_loop(q, k1, k2, v1, v2, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, inclusive=True):
    """Literal-order restatement: queries, then K keys, then K' keys, one
    weight at a time, numerator accumulated in the input dtype and the
    denominator in fp32 (simplicial/reference.py:39-74; the fp32 denominator is
    simplicial/reference.py:51).  For fp64 inputs the denominator is kept in
    fp64 here, so that an fp64 run is a truth source.  Vectorised over
    (batch, head) only.  Feasible for small shapes (N*(w1+1)*(w2+1) steps)."""
    B, N, H, D = q.shape
    _check_windows(w1, w2, inclusive)
    if scale is None:
        scale = default_scale(D)
    k2b = k2 + k2_bias
    v2b = v2 + v2_bias
    out = torch.zeros_like(q)
    for i in range(N):
        if inclusive:
            j_lo, k_lo = max(0, i - w1), max(0, i - w2)              # reference.py:41-45
        else:
            j_lo, k_lo = max(0, i - w1 + 1), max(0, i - w2 + 1)      # kernels.py:133-136
        qi = q[:, i]                                   # [B,H,D]
        num = torch.zeros_like(qi)
        den = torch.zeros(B, H, 1, dtype=torch.float32 if q.dtype != torch.float64 else torch.float64)
        for j in range(j_lo, i + 1):
            qk1 = qi * k1[:, j]
            for k in range(k_lo, i + 1):
                s = (qk1 * k2b[:, k] * scale).sum(-1, keepdim=True)
                w = torch.exp(s)
                num = num + w * (v1[:, j] * v2b[:, k])
                den = den + w
        out[:, i] = num / (den + 1e-8)
    return out


def _check_windows(w1, w2, inclusive):
    if w1 < 0 or w2 < 0 or (not inclusive and (w1 < 1 or w2 < 1)):
        raise ValueError("windows must be >= 0 (>= 1 for the half-open convention, which would hold no key)")


def _band(rows, cols, w, inclusive=True):
    """mask[r,c] = (rows[r]-w <= cols[c] <= rows[r]); with inclusive=False the lower
    bound is strict (simplicial/kernels.py:133-136)."""
    r = rows[:, None]
    c = cols[None, :]
    return (c <= r) & ((c >= r - w) if inclusive else (c > r - w))


def forward_windowed(q, k1, k2, v1, v2, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0,
                     rows=None, chunk=32, compute_dtype=None, inclusive=True):
    """Vectorised restatement of the same arithmetic on a range of query rows.

    rows = (r0, r1) restricts the computation to queries r0 <= i < r1 (outputs
    have r1-r0 rows); default all rows.  Differentiable by torch autograd, so
    gradients restricted to those query rows come from ``.backward``.
    Returns (O [B,n,H,D], LSE [B,H,n]) in ``compute_dtype`` (default: the
    input dtype for fp32/fp64 inputs, fp32 for 16-bit inputs).

    Mathematically identical to literal_loop: the maximum is subtracted before
    exponentiation and the epsilon is carried as 1e-8*exp(-max), so that
    O = sum w v / (sum w + 1e-8) holds for logits of any magnitude.
    """
    B, N, H, D = q.shape
    _check_windows(w1, w2, inclusive)
    if scale is None:
        scale = default_scale(D)
    if compute_dtype is None:
        compute_dtype = q.dtype if q.dtype in (torch.float32, torch.float64) else torch.float32
    r0, r1 = (0, N) if rows is None else rows
    cast = lambda t: t.to(compute_dtype).permute(0, 2, 1, 3)      # [B,H,N,D]
    qf, k1f, v1f = cast(q), cast(k1), cast(v1)
    k2f, v2f = cast(k2) + k2_bias, cast(v2) + v2_bias
    outs, lses = [], []
    eps = 1e-8
    for c0 in range(r0, r1, chunk):
        c1 = min(r1, c0 + chunk)
        ii = torch.arange(c0, c1)
        j0, k0 = max(0, c0 - w1), max(0, c0 - w2)
        jj = torch.arange(j0, c1)
        kk = torch.arange(k0, c1)
        qk = qf[:, :, c0:c1, None, :] * k2f[:, :, None, k0:c1, :]        # [B,H,i,k,D]
        s = torch.matmul(qk, k1f[:, :, None, j0:c1, :].transpose(-1, -2)) * scale   # [B,H,i,k,j]
        mask = _band(ii, kk, w2, inclusive)[:, :, None] & _band(ii, jj, w1, inclusive)[:, None, :]      # [i,k,j]
        s = s.masked_fill(~mask, float("-inf"))
        m = s.amax(dim=(-1, -2), keepdim=True)                           # [B,H,i,1,1]
        w = torch.exp(s - m)
        den = w.sum(dim=(-1, -2)) + eps * torch.exp(-m[..., 0, 0])       # [B,H,i]
        r = torch.matmul(w, v1f[:, :, None, j0:c1, :])                   # [B,H,i,k,D]
        num = (r * v2f[:, :, None, k0:c1, :]).sum(dim=3)                 # [B,H,i,D]
        outs.append(num / den[..., None])
        # log(sum w + eps) for any m: when e^m underflows against eps, factor eps out instead
        mm, l = m[..., 0, 0], w.sum(dim=(-1, -2))
        log_eps = math.log(eps)
        hi = mm + torch.log(l + eps * torch.exp(-mm.clamp_min(log_eps)))
        lo = log_eps + torch.log1p(l * torch.exp(mm.clamp_max(log_eps) - log_eps))
        lses.append(torch.where(mm > log_eps, hi, lo))
    out = torch.cat(outs, dim=2).permute(0, 2, 1, 3)                     # [B,n,H,D]
    lse = torch.cat(lses, dim=2)                                         # [B,H,n]
    return out, lse


def grads_windowed(q, k1, k2, v1, v2, dout, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0,
                   rows=None, chunk=32, compute_dtype=None, inclusive=True):
    """Gradients of sum(O*dout) over the query rows in ``rows`` with respect to
    the five inputs, by autograd through forward_windowed, one chunk at a
    time.  ``dout`` has the same row range as the output.  Returns
    (O, LSE, dq, dk1, dk2, dv1, dv2); gradients are full [B,N,H,D] tensors in
    compute_dtype holding only the contributions of the selected queries."""
    B, N, H, D = q.shape
    if compute_dtype is None:
        compute_dtype = q.dtype if q.dtype in (torch.float32, torch.float64) else torch.float32
    r0, r1 = (0, N) if rows is None else rows
    leaves = [t.detach().to(compute_dtype).clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    outs, lses = [], []
    for c0 in range(r0, r1, chunk):
        c1 = min(r1, c0 + chunk)
        o, lse = forward_windowed(*leaves, w1, w2, scale, k2_bias, v2_bias,
                                  rows=(c0, c1), chunk=chunk, compute_dtype=compute_dtype, inclusive=inclusive)
        (o * dout[:, c0 - r0:c1 - r0].to(compute_dtype)).sum().backward()
        outs.append(o.detach())
        lses.append(lse.detach())
    grads = [t.grad if t.grad is not None else torch.zeros_like(t) for t in leaves]
    return (torch.cat(outs, dim=1), torch.cat(lses, dim=2), *grads)


def count_triples(B, N, H, w1, w2, inclusive=True):
    """Number of valid (i,j,k) triples summed over batch and heads:
    B*H*sum_i (min(i,w1)+1)*(min(i,w2)+1) (windows of simplicial/reference.py:41-45), or
    B*H*sum_i min(i+1,w1)*min(i+1,w2) for the half-open windows of simplicial/kernels.py:133-136."""
    t = 0
    for i in range(N):
        t += (min(i, w1) + 1) * (min(i, w2) + 1) if inclusive else min(i + 1, w1) * min(i + 1, w2)
    return B * H * t
