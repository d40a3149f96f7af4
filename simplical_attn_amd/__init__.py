"""MI355X-native 2-simplicial attention: HIP kernels behind a C ABI, with the
reference's operator interface on top."""
from .simplicial_attn import (  # noqa: F401
    TwoSimplicialAttention,
    TwoSimplicialAttentionFunction,
    TwoSimplicialAttentionExact,
    compute_D_kernel,
    simplicial_backward,
    simplicial_forward,
    simplicial_rowdot,
    two_simplicial_attention_exact,
)

from .compiled_op import two_simplicial_attention  # noqa: F401,E402

__all__ = [
    "two_simplicial_attention",
    "TwoSimplicialAttention",
    "TwoSimplicialAttentionFunction",
    "two_simplicial_attention_exact",
    "TwoSimplicialAttentionExact",
    "compute_D_kernel",
    "simplicial_forward",
    "simplicial_backward",
    "simplicial_rowdot",
]

# Names the reference package exports (simplicial/__init__.py:12-27) that have no
# counterpart here: its PyTorch CPU loop (simplicial/reference.py; this package has no CPU path
# and ships no second implementation to check itself with), its Triton kernel objects and its
# test runners.
_CPU_LOOP = ("the reference's own simplicial/reference.py on CPU tensors (it stays the check of this operator); "
             "two_simplicial_attention_exact / TwoSimplicialAttentionExact run the same maths on this "
             "library's fp32 kernels on the GPU, which is a kernel-against-kernel comparison")
_NOT_PROVIDED = {
    "two_simplicial_attention_reference": _CPU_LOOP,
    "TwoSimplicialAttentionReference": _CPU_LOOP,
    "two_simplicial_attn_fwd_kernel": "simplicial_forward (C entry point sa2_forward)",
    "two_simplicial_attn_bwd_kv1_kernel": "simplicial_backward (C entry point sa2_backward)",
    "two_simplicial_attn_bwd_kv2_kernel": "simplicial_backward (C entry point sa2_backward)",
    "run_all_correctness_tests": "python -m pytest tests -m gpu",
    "run_all_performance_tests": "python bench.py and python bench_sweep.py",
    "quick_performance_test": "python bench.py",
    "run_all_tests": "python -m pytest tests",
    "test_forward_pass_correctness": "python -m pytest tests -m gpu",
    "test_backward_implementation": "python -m pytest tests -m gpu",
}


def __getattr__(name):
    if name in _NOT_PROVIDED:
        raise AttributeError("%s belongs to the reference's Triton implementation and is not provided; use %s"
                             % (name, _NOT_PROVIDED[name]))
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
