"""The operator as a `torch.library` custom op, so that callers under `torch.compile`
(or any other fake-tensor tracing) can use it: shapes and dtypes come from the
registered fake implementations, gradients from the registered autograd formula.
The eager path is `TwoSimplicialAttentionFunction` (simplicial/triton_impl.py:18-158 in
the reference); this module calls the same two entry points of the C ABI."""
import math
from typing import Tuple

import torch

from . import simplicial_attn as _sa

Tensor = torch.Tensor


@torch.library.custom_op("simplical_attn_amd::forward", mutates_args=())
def forward_op(q: Tensor, k1: Tensor, k2: Tensor, v1: Tensor, v2: Tensor, w1: int, w2: int, scale: float,
               k2_bias: float, v2_bias: float, window_inclusive: bool = True) -> Tuple[Tensor, Tensor]:
    return _sa.simplicial_forward(q, k1, k2, v1, v2, w1, w2, scale, k2_bias, v2_bias,
                                  window_inclusive=window_inclusive)


@forward_op.register_fake
def _(q, k1, k2, v1, v2, w1, w2, scale, k2_bias, v2_bias, window_inclusive=True):
    # the real op returns freshly allocated contiguous tensors whatever the strides of q
    B, N, H, D = q.shape
    return q.new_empty((B, N, H, D)), q.new_empty((B, H, N), dtype=torch.float32)


@torch.library.custom_op("simplical_attn_amd::backward", mutates_args=())
def backward_op(q: Tensor, k1: Tensor, k2: Tensor, v1: Tensor, v2: Tensor, out: Tensor, lse: Tensor, dout: Tensor,
                w1: int, w2: int, scale: float, k2_bias: float, v2_bias: float,
                window_inclusive: bool = True) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    return tuple(_sa.simplicial_backward(q, k1, k2, v1, v2, out, lse, dout, w1, w2, scale, k2_bias, v2_bias,
                                         window_inclusive=window_inclusive))


@backward_op.register_fake
def _(q, k1, k2, v1, v2, out, lse, dout, w1, w2, scale, k2_bias, v2_bias, window_inclusive=True):
    return tuple(t.new_empty(tuple(t.shape)) for t in (q, k1, k2, v1, v2))


def _setup_context(ctx, inputs, output):
    q, k1, k2, v1, v2, w1, w2, scale, k2_bias, v2_bias, window_inclusive = inputs
    out, lse = output
    ctx.save_for_backward(q, k1, k2, v1, v2, out, lse)
    ctx.args = (w1, w2, scale, k2_bias, v2_bias, window_inclusive)


def _backward(ctx, grad_out, grad_lse):
    q, k1, k2, v1, v2, out, lse = ctx.saved_tensors
    grads = backward_op(q, k1, k2, v1, v2, out, lse, grad_out.contiguous(), *ctx.args)
    return (*grads, None, None, None, None, None, None)


forward_op.register_autograd(_backward, setup_context=_setup_context)


def two_simplicial_attention(q, k1, k2, v1, v2, w1, w2, scale=None, k2_bias=0.0, v2_bias=0.0, window_inclusive=True):
    """Output of causal sliding-window 2-simplicial attention, traceable by torch.compile.
    Same argument meaning as TwoSimplicialAttentionFunction.apply; ``window_inclusive=False``
    selects the half-open windows of the reference's device kernels (simplicial/kernels.py:133-136)."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    return forward_op(q, k1, k2, v1, v2, int(w1), int(w2), float(scale), float(k2_bias), float(v2_bias),
                      bool(window_inclusive))[0]
