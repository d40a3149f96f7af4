"""CPU-side checks of the C-ABI library and the host wrapper: the library
loads, exports every symbol include/sa2.h declares, validates arguments
before touching the GPU, and the Python operator keeps the reference's
interface (simplicial/triton_impl.py:15-186).  No kernel is launched here."""
import ctypes
import inspect
import os
import re

import pytest
import torch

from simplical_attn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from simplical_attn_amd import build
        build.build_library(verbose=False)
    return _lib.load()


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "sa2.h")).read()
    declared = set(re.findall(r"\b(sa2_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None


def test_version_and_strerror(lib):
    assert lib.sa2_version() == 1
    assert lib.sa2_strerror(0) == b"success"
    seen = set()
    for code in range(-10, 0):
        msg = lib.sa2_strerror(code)
        assert msg and msg not in seen
        seen.add(msg)
    assert b"unknown" in lib.sa2_strerror(-100)


def test_workspace_bytes(lib):
    assert lib.sa2_bwd_workspace_bytes(1, 8192, 16, 128, 512, 32, _lib.SA2_BF16, 0) >= 16 * 8192 * 4
    assert lib.sa2_bwd_workspace_bytes(1, 128, 2, 64, 32, 16, _lib.SA2_F32, 0) >= 2 * 128 * 4
    assert lib.sa2_bwd_workspace_bytes(0, 128, 2, 64, 32, 16, _lib.SA2_F32, 0) == 0
    assert lib.sa2_bwd_workspace_bytes(1, 128, 2, 300, 32, 16, _lib.SA2_F32, 0) == 0


def test_argument_validation_needs_no_gpu(lib):
    strides = _lib.stride_array([(1024, 128, 64)] * 12)
    one = ctypes.c_void_p(256)   # never dereferenced: validation fails first
    args = lambda **kw: dict(dict(B=1, N=8, H=2, D=64, w1=4, w2=4, dtype=0, incl=1), **kw)

    def fwd(a, q=one):
        return lib.sa2_forward(q, one, one, one, one, one, one, a["B"], a["N"], a["H"], a["D"], strides,
                               a["w1"], a["w2"], 0.125, 0.0, 0.0, a["dtype"], a["incl"], 0, None)

    assert fwd(args(), q=None) == -1
    assert fwd(args(dtype=7)) == -2
    assert fwd(args(D=257)) == -3
    assert fwd(args(N=0)) == -3
    assert fwd(args(w1=-1)) == -5
    assert fwd(args(w2=0, incl=0)) == -5
    bad = _lib.stride_array([(1024, 0, 64)] * 12)
    assert lib.sa2_forward(one, one, one, one, one, one, one, 1, 8, 2, 64, bad, 4, 4, 0.125, 0.0, 0.0, 0, 1, 0, None) == -4
    # backward: workspace too small
    assert lib.sa2_backward(one, one, one, one, one, one, one, one, one, one, one, one, one, one, 16,
                            1, 8, 2, 64, strides, 4, 4, 0.125, 0.0, 0.0, 0, 1, 0, None) == -6
    assert lib.sa2_uses_mfma(1, 8192, 16, 128, 512, 32, _lib.SA2_BF16) == 1
    assert lib.sa2_uses_mfma(1, 8192, 16, 128, 512, 32, _lib.SA2_F32) == 0


def test_operator_interface_matches_reference():
    """Names, argument order and defaults of simplicial/triton_impl.py:19, 61, 164, 173."""
    import simplical_attn_amd as sa
    sig = inspect.signature(sa.TwoSimplicialAttention.__init__)
    assert list(sig.parameters) == ["self", "head_dim", "w1", "w2", "scale", "k2_bias", "v2_bias"]
    assert [sig.parameters[k].default for k in ("w1", "w2", "scale", "k2_bias", "v2_bias")] == [64, 64, None, 0.0, 0.0]
    fsig = inspect.signature(sa.TwoSimplicialAttentionFunction.forward)
    assert list(fsig.parameters) == ["ctx", "q", "k1", "k2", "v1", "v2", "w1", "w2", "scale", "k2_bias", "v2_bias"]
    m = sa.TwoSimplicialAttention(64)
    assert m.scale == 1.0 / 8.0 and m.w1 == 64 and m.w2 == 64 and len(list(m.parameters())) == 0
    assert list(inspect.signature(m.forward).parameters) == ["q", "k1", "k2", "v1", "v2"]


def test_reference_package_names():
    """Every name the reference package exports (simplicial/__init__.py:12-27) either exists with the
    reference's signature or raises an AttributeError that says what to use instead."""
    import simplical_attn_amd as sa
    rsig = inspect.signature(sa.two_simplicial_attention_exact)
    assert list(rsig.parameters) == ["q", "k1", "k2", "v1", "v2", "w1", "w2", "scale", "k2_bias", "v2_bias"]
    assert [rsig.parameters[k].default for k in ("scale", "k2_bias", "v2_bias")] == [None, 0.0, 0.0]
    m = sa.TwoSimplicialAttentionExact(16, 4, 4)
    assert m.scale == 0.25 and list(inspect.signature(m.forward).parameters) == ["q", "k1", "k2", "v1", "v2"]
    assert callable(sa.compute_D_kernel)
    # the device yardstick does not pose as the reference's CPU loop
    for name in ("two_simplicial_attention_reference", "TwoSimplicialAttentionReference"):
        with pytest.raises(AttributeError, match="kernel-against-kernel"):
            getattr(sa, name)
    for name in ("two_simplicial_attn_fwd_kernel", "two_simplicial_attn_bwd_kv1_kernel",
                 "two_simplicial_attn_bwd_kv2_kernel", "run_all_correctness_tests", "run_all_performance_tests",
                 "quick_performance_test", "run_all_tests", "test_forward_pass_correctness",
                 "test_backward_implementation"):
        with pytest.raises(AttributeError, match="not provided; use"):
            getattr(sa, name)
    x = torch.zeros(1, 8, 1, 16)
    with pytest.raises(RuntimeError, match="GPU only"):
        sa.two_simplicial_attention_exact(x, x, x, x, x, 4, 4)


def test_cpu_tensors_fail_loudly():
    """There is no CPU fallback: the operator refuses tensors that are not on the GPU."""
    import simplical_attn_amd as sa
    x = torch.zeros(1, 8, 1, 16)
    with pytest.raises(RuntimeError, match="GPU only"):
        sa.TwoSimplicialAttention(16, 4, 4)(x, x, x, x, x)
    with pytest.raises(ValueError):
        sa.simplicial_forward(x[0], x, x, x, x, 4, 4)
    with pytest.raises(TypeError):
        sa.simplicial_forward(x.double(), x, x, x, x, 4, 4)


def test_product_package_does_not_import_the_oracle():
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); import simplical_attn_amd; "
            "assert not any(m.startswith('oracle') for m in sys.modules), 'oracle imported'" % ROOT)
    subprocess.run([sys.executable, "-c", code], check=True)
    for dirpath, _, files in os.walk(os.path.join(ROOT, "simplical_attn_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f
