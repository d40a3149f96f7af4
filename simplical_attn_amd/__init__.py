"""MI355X-native 2-simplicial attention: HIP kernels behind a C ABI, with the
reference's operator interface on top."""
from .simplicial_attn import (  # noqa: F401
    TwoSimplicialAttention,
    TwoSimplicialAttentionFunction,
    compute_D_kernel,
    simplicial_backward,
    simplicial_forward,
)

from .compiled_op import two_simplicial_attention  # noqa: F401,E402

__all__ = [
    "two_simplicial_attention",
    "TwoSimplicialAttention",
    "TwoSimplicialAttentionFunction",
    "compute_D_kernel",
    "simplicial_forward",
    "simplicial_backward",
]
