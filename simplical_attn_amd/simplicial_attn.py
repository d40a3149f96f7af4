"""Host side of the 2-simplicial attention operator on MI355X.

Same operator interface as the reference's wrapper (simplicial/triton_impl.py):
``TwoSimplicialAttentionFunction.apply(q, k1, k2, v1, v2, w1, w2, scale,
k2_bias, v2_bias)`` (triton_impl.py:15-158) and the module
``TwoSimplicialAttention(head_dim, w1, w2, scale, k2_bias, v2_bias)``
(triton_impl.py:161-186).  The kernels behind it are the HIP library's, reached
through the C ABI in include/sa2.h; torch only owns the device buffers and the
stream.  There is no CPU or eager fallback: tensors must live on the GPU and
the library must have been built.
"""
import math

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.SA2_F32, torch.bfloat16: _lib.SA2_BF16, torch.float16: _lib.SA2_F16}

# Window convention, an argument of every entry point below (``window_inclusive``):
# True = closed windows [i-w, i] as the reference's PyTorch oracle defines them
# (simplicial/reference.py:41-45); False = half-open (i-w, i] as the reference's device
# kernels mask (simplicial/kernels.py:133-136).  This is only the default of that argument;
# nothing reads it at call time.
WINDOW_INCLUSIVE = True


def _check_inputs(q, k1, k2, v1, v2):
    if q.dim() != 4:
        raise ValueError("expected [batch, seq_len, num_heads, head_dim] tensors, got shape %s" % (tuple(q.shape),))
    if q.dtype not in _DTYPES:
        raise TypeError("unsupported dtype %s (float32, bfloat16, float16)" % q.dtype)
    for name, t in (("k1", k1), ("k2", k2), ("v1", v1), ("v2", v2)):
        if t.shape != q.shape or t.dtype != q.dtype or t.device != q.device:
            raise ValueError("%s must match q in shape, dtype and device" % name)
    if not q.is_cuda:
        raise RuntimeError("TwoSimplicialAttention runs on the GPU only; got a %s tensor" % q.device)


def _check_saved(q, out, lse, dout):
    """The tensors a backward call gets beside the five inputs: their addresses go to the kernels
    as they are, so everything the kernels assume is checked here."""
    B, N, H, _ = q.shape
    for name, t in (("out", out), ("dout", dout)):
        if not isinstance(t, torch.Tensor) or t.shape != q.shape or t.dtype != q.dtype or t.device != q.device:
            raise ValueError("%s must match q in shape, dtype and device" % name)
    if not isinstance(lse, torch.Tensor) or lse.dtype != torch.float32 or lse.device != q.device:
        raise ValueError("lse must be a float32 tensor on q's device")
    if tuple(lse.shape) != (B, H, N) or not lse.is_contiguous():
        raise ValueError("lse must be contiguous [batch, num_heads, seq_len] = %s, got shape %s strides %s"
                         % ((B, H, N), tuple(lse.shape), lse.stride()))


def _rows(t):
    """Tensor usable by the kernels: unit stride along head_dim and a positive stride on every
    axis longer than 1.  Broadcast views (stride 0: a gradient expanded by ``sum`` in the loss,
    a key expanded over heads) and anything else are copied, as the reference's launch accepts
    arbitrary strides (simplicial/triton_impl.py:38-45)."""
    ok = t.stride(-1) == 1 and all(st > 0 or n == 1 for st, n in zip(t.stride()[:-1], t.shape[:-1]))
    return t if ok else t.contiguous()


def _pad_head_dim(D, dtype, flags):
    """head_dim the kernels are run with.  The MFMA kernels start at head_dim 32 (one 32-column
    value tile); tensors with head_dim 16 are zero-padded to 32 on the way in (zero columns
    add nothing to a logit and give zero output and gradient columns, which are dropped again), so
    that they take the MFMA kernels of their element type instead of the fp32 FMA kernels.  The
    softmax scale is always the caller's (1/sqrt(16) by default), not that of the padded width."""
    return 32 if (D == 16 and dtype in (torch.bfloat16, torch.float16, torch.float32) and flags == _lib.FLAG_AUTO) else D


def _padded(t, width):
    return t if t.shape[-1] == width else torch.nn.functional.pad(t, (0, width - t.shape[-1]))


def _strides(*tensors):
    return _lib.stride_array([(t.stride(0), t.stride(1), t.stride(2)) for t in tensors])


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def simplicial_forward(q, k1, k2, v1, v2, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, flags=_lib.FLAG_AUTO,
                       window_inclusive=True):
    """Runs the forward kernel; returns (output like q, LSE [B,H,N] fp32).
    Replaces the launch in triton_impl.py:23-51."""
    _check_inputs(q, k1, k2, v1, v2)
    lib = _lib.load()
    B, N, H, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    width = _pad_head_dim(D, q.dtype, flags)
    if width != D:
        out, lse = simplicial_forward(*(_padded(t, width) for t in (q, k1, k2, v1, v2)), w1, w2, scale, k2_bias,
                                      v2_bias, flags, window_inclusive)
        return out[..., :D].contiguous(), lse
    q, k1, k2, v1, v2 = (_rows(t) for t in (q, k1, k2, v1, v2))
    with torch.cuda.device(q.device):
        out = torch.empty((B, N, H, D), dtype=q.dtype, device=q.device)
        lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
        _lib.check(lib.sa2_forward(
            q.data_ptr(), k1.data_ptr(), k2.data_ptr(), v1.data_ptr(), v2.data_ptr(),
            out.data_ptr(), lse.data_ptr(), B, N, H, D, _strides(q, k1, k2, v1, v2, out),
            int(w1), int(w2), float(scale), float(k2_bias), float(v2_bias),
            _DTYPES[q.dtype], int(bool(window_inclusive)), int(flags), _stream(q)))
    return out, lse


def simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0,
                        needs=(True, True, True, True, True), flags=_lib.FLAG_AUTO, window_inclusive=True):
    """Runs the backward kernels; returns (dq, dk1, dk2, dv1, dv2) in the input
    dtype, None where ``needs`` is False.  Replaces triton_impl.py:61-158.
    ``out`` and ``lse`` are what simplicial_forward returned for the same inputs and arguments."""
    _check_inputs(q, k1, k2, v1, v2)
    _check_saved(q, out, lse, dout)
    if len(needs) != 5:
        raise ValueError("needs must have five entries (dq, dk1, dk2, dv1, dv2), got %d" % len(needs))
    lib = _lib.load()
    B, N, H, D = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    width = _pad_head_dim(D, q.dtype, flags)
    if width != D:
        grads = simplicial_backward(*(_padded(t, width) for t in (q, k1, k2, v1, v2, out)), lse, _padded(dout, width),
                                    w1, w2, scale, k2_bias, v2_bias, needs, flags, window_inclusive)
        return tuple(g[..., :D].contiguous() if g is not None else None for g in grads)
    q, k1, k2, v1, v2, out, dout = (_rows(t) for t in (q, k1, k2, v1, v2, out, dout))
    dt = _DTYPES[q.dtype]
    reach1 = int(w1) if window_inclusive else int(w1) - 1
    reach2 = int(w2) if window_inclusive else int(w2) - 1
    with torch.cuda.device(q.device):
        grads = [torch.empty((B, N, H, D), dtype=q.dtype, device=q.device) if need else None for need in needs]
        ws_bytes = lib.sa2_bwd_workspace_bytes(B, N, H, D, reach1, reach2, dt, int(flags))
        workspace = torch.empty(max(int(ws_bytes), 256), dtype=torch.uint8, device=q.device)
        like = grads[0] if grads[0] is not None else q
        stride_src = [g if g is not None else like for g in grads]
        ptr = lambda g: g.data_ptr() if g is not None else None
        _lib.check(lib.sa2_backward(
            q.data_ptr(), k1.data_ptr(), k2.data_ptr(), v1.data_ptr(), v2.data_ptr(),
            out.data_ptr(), dout.data_ptr(), lse.data_ptr(),
            ptr(grads[0]), ptr(grads[1]), ptr(grads[2]), ptr(grads[3]), ptr(grads[4]),
            workspace.data_ptr(), workspace.numel(), B, N, H, D,
            _strides(q, k1, k2, v1, v2, out, dout, *stride_src),
            int(w1), int(w2), float(scale), float(k2_bias), float(v2_bias),
            dt, int(bool(window_inclusive)), int(flags), _stream(q)))
    return tuple(grads)


def simplicial_rowdot(dO, O):
    """sum_d dO*O per (batch, head, position) in fp32, laid out [B,H,N] as the backward
    kernels index it (C entry point sa2_rowdot)."""
    lib = _lib.load()
    B, N, H, D = O.shape
    O, dO = _rows(O), _rows(dO)
    with torch.cuda.device(O.device):
        dsum = torch.empty((B, H, N), dtype=torch.float32, device=O.device)
        _lib.check(lib.sa2_rowdot(O.data_ptr(), dO.data_ptr(), dsum.data_ptr(), B, N, H, D,
                                  _strides(O, dO), _DTYPES[O.dtype], _stream(O)))
    return dsum


def compute_D_kernel(dO, O):
    """The reference helper of that name (simplicial/kernels.py:569-571): ``sum(dO * O, dim=-1)``,
    shape [B,N,H] in dO's dtype.  The sum itself is taken in fp32 by the device kernel."""
    return simplicial_rowdot(dO, O).transpose(1, 2).to(dO.dtype)


class TwoSimplicialAttentionFunction(torch.autograd.Function):
    """autograd Function with the reference's argument list
    (simplicial/triton_impl.py:19): forward saves (q, k1, k2, v1, v2, output,
    LSE) as triton_impl.py:54 does; backward returns five gradients in the
    inputs' dtype and None for every other argument (triton_impl.py:157-158).

    Two trailing arguments beyond the reference's ten, both optional so that the reference's
    positional call works unchanged: ``window_inclusive`` (True: closed windows [i-w, i] of
    simplicial/reference.py:41-45; False: the half-open (i-w, i] of the reference's device
    kernels, simplicial/kernels.py:133-136) and ``kernel_flags`` (kernel choice of the C ABI:
    0 automatic, 1 fp32 FMA kernels, 2 MFMA kernels or an error).  Both travel in ``ctx``;
    no process-wide state is read."""

    @staticmethod
    def forward(ctx, q, k1, k2, v1, v2, w1, w2, scale, k2_bias, v2_bias, window_inclusive=True,
                kernel_flags=_lib.FLAG_AUTO):
        if scale is None:
            scale = 1.0 / math.sqrt(q.shape[-1])
        window_inclusive = bool(window_inclusive)
        out, lse = simplicial_forward(q, k1, k2, v1, v2, w1, w2, scale, k2_bias, v2_bias, kernel_flags,
                                      window_inclusive)
        ctx.save_for_backward(q, k1, k2, v1, v2, out, lse)
        ctx.w1, ctx.w2, ctx.scale, ctx.k2_bias, ctx.v2_bias = w1, w2, scale, k2_bias, v2_bias
        ctx.flags = kernel_flags
        ctx.window_inclusive = window_inclusive
        return out

    @staticmethod
    def backward(ctx, grad_output):
        q, k1, k2, v1, v2, out, lse = ctx.saved_tensors
        grads = simplicial_backward(q, k1, k2, v1, v2, out, lse, grad_output, ctx.w1, ctx.w2, ctx.scale,
                                    ctx.k2_bias, ctx.v2_bias, needs=tuple(ctx.needs_input_grad[:5]),
                                    flags=ctx.flags, window_inclusive=ctx.window_inclusive)
        # (autograd drops the trailing None entries of a call that left the optional arguments out)
        return (*grads, None, None, None, None, None, None, None)


def two_simplicial_attention_exact(q, k1, k2, v1, v2, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0,
                                   window_inclusive=True):
    """Argument list of the reference's PyTorch implementation (simplicial/reference.py:8-9), run
    on the fp32 FMA kernels on the GPU (same windows, bias and epsilon as reference.py:27-76),
    differentiable.  It is a device-side yardstick for the MFMA kernels: HIP kernels of this same
    library, NOT an independent reference and not a CPU path.  Comparing the operator with it is a
    kernel-against-kernel check."""
    return TwoSimplicialAttentionFunction.apply(q, k1, k2, v1, v2, w1, w2, scale, k2_bias, v2_bias,
                                                window_inclusive, _lib.FLAG_FORCE_GENERIC)


class TwoSimplicialAttentionExact(torch.nn.Module):
    """Module wrapper of two_simplicial_attention_exact with the constructor of the reference's
    TwoSimplicialAttentionReference (simplicial/reference.py:79-103)."""

    def __init__(self, head_dim, w1=64, w2=64, scale=None, k2_bias=0.0, v2_bias=0.0, *, window_inclusive=True):
        super().__init__()
        self.head_dim = head_dim
        self.w1 = w1
        self.w2 = w2
        self.scale = scale if scale is not None else (1.0 / math.sqrt(head_dim))
        self.k2_bias = k2_bias
        self.v2_bias = v2_bias
        self.window_inclusive = bool(window_inclusive)

    def forward(self, q, k1, k2, v1, v2):
        return two_simplicial_attention_exact(q, k1, k2, v1, v2, self.w1, self.w2, self.scale,
                                              self.k2_bias, self.v2_bias, self.window_inclusive)


class TwoSimplicialAttention(torch.nn.Module):
    """Module wrapper with the reference's constructor and call signature
    (simplicial/triton_impl.py:161-186); holds no parameters.  The keyword-only
    ``window_inclusive=False`` selects the half-open windows (i-w, i] of the reference's device
    kernels (simplicial/kernels.py:133-136) for callers that migrate from them."""

    def __init__(self, head_dim, w1=64, w2=64, scale=None, k2_bias=0.0, v2_bias=0.0, *, window_inclusive=True):
        super().__init__()
        self.head_dim = head_dim
        self.w1 = w1
        self.w2 = w2
        self.scale = scale if scale is not None else (1.0 / math.sqrt(head_dim))
        self.k2_bias = k2_bias
        self.v2_bias = v2_bias
        self.window_inclusive = bool(window_inclusive)

    def forward(self, q, k1, k2, v1, v2):
        return TwoSimplicialAttentionFunction.apply(q, k1, k2, v1, v2, self.w1, self.w2, self.scale,
                                                    self.k2_bias, self.v2_bias, self.window_inclusive)
