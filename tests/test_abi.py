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
    assert lib.sa2_uses_mfma(1, 8192, 16, 128, 512, 32, _lib.SA2_F32) == 1      # the fp32 MFMA kernels
    assert lib.sa2_uses_mfma(1, 8192, 16, 256, 512, 32, _lib.SA2_F32) == 0
    assert lib.sa2_uses_mfma(1, 8192, 16, 256, 512, 32, _lib.SA2_BF16) == 1     # the head_dim 256 MFMA kernels
    assert lib.sa2_uses_mfma(1, 8192, 16, 192, 512, 32, _lib.SA2_BF16) == 0


def test_forced_mfma_refuses_layouts_its_loads_cannot_take(lib):
    """The MFMA kernels move 16-byte chunks with 32-bit row offsets.  A 16-bit tensor whose rows are
    off the 16-byte grid, whose rows span 2^31 elements or more, an unsupported head_dim or fp32 must
    never reach them: with SA2_FLAG_FORCE_MFMA the call returns SA2_ERR_UNSUPPORTED and launches
    nothing (pointers here are never dereferenced; with SA2_FLAG_AUTO the same problems take the
    fp32 kernels, which the GPU tests cover)."""
    B, N, H, D = 1, 64, 2, 128
    good = (N * H * D, H * D, D)
    base = 1 << 20                                     # 16-byte aligned, never dereferenced
    FORCE, UNSUPPORTED = _lib.FLAG_FORCE_MFMA, -8

    def fwd(ptrs=None, strides=None, N=N, D=D, dtype=_lib.SA2_BF16):
        ptrs = ptrs or [base] * 6
        st = _lib.stride_array(strides or [good] * 6)
        return lib.sa2_forward(*[ctypes.c_void_p(x) for x in ptrs], ctypes.c_void_p(base), B, N, H, D, st,
                               16, 8, 0.1, 0.0, 0.0, dtype, 1, FORCE, None)

    def bwd(ptrs=None, strides=None, dtype=_lib.SA2_BF16):
        ptrs = ptrs or [base] * 12                     # q k1 k2 v1 v2 out dout dq dk1 dk2 dv1 dv2
        st = _lib.stride_array(strides or [good] * 12)
        ws = lib.sa2_bwd_workspace_bytes(B, N, H, D, 16, 8, dtype, FORCE)
        args = [ctypes.c_void_p(x) for x in ptrs[:7]] + [ctypes.c_void_p(base)] + [ctypes.c_void_p(x) for x in ptrs[7:]]
        return lib.sa2_backward(*args, ctypes.c_void_p(base), ws, B, N, H, D, st, 16, 8, 0.1, 0.0, 0.0, dtype, 1,
                                FORCE, None)

    for t in range(6):                                 # a base pointer 8 bytes off the grid, tensor by tensor
        ptrs = [base] * 6
        ptrs[t] = base + 8
        assert fwd(ptrs=ptrs) == UNSUPPORTED, t
    for axis in (1, 2):                                # a sequence or head stride that is not a multiple of 8 elements
        st = [good] * 6                                # (the batch axis has size 1 here and may carry any stride)
        odd = list(good)
        odd[axis] += 4
        st[1] = tuple(odd)
        assert fwd(strides=st) == UNSUPPORTED, axis
    st = [good] * 6
    st[3] = (good[0], (1 << 31) // (N - 1) // 8 * 8 + 8, D)      # (N-1) * stride_n reaches 2^31 elements
    assert fwd(strides=st) == UNSUPPORTED
    st[3] = (good[0], 1 << 40, D)
    assert fwd(strides=st) == UNSUPPORTED
    assert fwd(D=48, strides=[(N * H * 48, H * 48, 48)] * 6) == UNSUPPORTED
    # fp32 has MFMA kernels of its own (head_dim 32, 64, 128; float4 loads: 16-byte aligned rows)
    assert fwd(D=48, strides=[(N * H * 48, H * 48, 48)] * 6, dtype=_lib.SA2_F32) == UNSUPPORTED
    assert fwd(D=256, strides=[(N * H * 256, H * 256, 256)] * 6, dtype=_lib.SA2_F32) == UNSUPPORTED
    assert fwd(ptrs=[base, base, base + 8, base, base, base], dtype=_lib.SA2_F32) == UNSUPPORTED
    st = [good] * 6
    st[4] = (good[0], H * D + 2, D)
    assert fwd(strides=st, dtype=_lib.SA2_F32) == UNSUPPORTED
    # backward: the same guards, and they cover dout and the gradient tensors too
    for t in range(12):
        ptrs = [base] * 12
        ptrs[t] = base + 8
        assert bwd(ptrs=ptrs) == UNSUPPORTED, t
    st = [good] * 12
    st[6] = (good[0], H * D + 4, D)
    assert bwd(strides=st) == UNSUPPORTED
    ptrs = [base] * 12
    ptrs[9] = base + 4
    assert bwd(ptrs=ptrs, dtype=_lib.SA2_F32) == UNSUPPORTED


def test_operator_interface_matches_reference():
    """Names, argument order and defaults of simplicial/triton_impl.py:19, 61, 164, 173."""
    import simplical_attn_amd as sa
    sig = inspect.signature(sa.TwoSimplicialAttention.__init__)
    positional = [k for k, v in sig.parameters.items() if v.kind == v.POSITIONAL_OR_KEYWORD]
    assert positional == ["self", "head_dim", "w1", "w2", "scale", "k2_bias", "v2_bias"]
    assert [sig.parameters[k].default for k in ("w1", "w2", "scale", "k2_bias", "v2_bias")] == [64, 64, None, 0.0, 0.0]
    # what this build adds is keyword-only and defaults to the reference's behaviour
    extra = {k: v for k, v in sig.parameters.items() if v.kind == v.KEYWORD_ONLY}
    assert list(extra) == ["window_inclusive"] and extra["window_inclusive"].default is True
    fsig = inspect.signature(sa.TwoSimplicialAttentionFunction.forward)
    names = list(fsig.parameters)
    assert names[:11] == ["ctx", "q", "k1", "k2", "v1", "v2", "w1", "w2", "scale", "k2_bias", "v2_bias"]
    # the reference's ten-argument positional call still works: everything after it is defaulted
    assert names[11:] == ["window_inclusive", "kernel_flags"]
    assert fsig.parameters["window_inclusive"].default is True and fsig.parameters["kernel_flags"].default == 0
    assert not hasattr(sa.TwoSimplicialAttentionFunction, "kernel_flags")      # no process-wide switches
    m = sa.TwoSimplicialAttention(64)
    assert m.scale == 1.0 / 8.0 and m.w1 == 64 and m.w2 == 64 and len(list(m.parameters())) == 0
    assert list(inspect.signature(m.forward).parameters) == ["q", "k1", "k2", "v1", "v2"]


def test_reference_package_names():
    """Every name the reference package exports (simplicial/__init__.py:12-27) either exists with the
    reference's signature or raises an AttributeError that says what to use instead."""
    import simplical_attn_amd as sa
    rsig = inspect.signature(sa.two_simplicial_attention_exact)
    assert list(rsig.parameters)[:10] == ["q", "k1", "k2", "v1", "v2", "w1", "w2", "scale", "k2_bias", "v2_bias"]
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


def test_backward_validates_saved_tensors_before_any_pointer_is_taken():
    """simplicial_backward is reachable by any caller (and through the torch.library op): out, dout
    and lse are checked against q before their addresses go to the kernels.  The input checks run
    first, so these tensors can live on the CPU here: a CPU q fails with the 'GPU only' error, and
    everything checked before that fails with a ValueError."""
    import simplical_attn_amd as sa
    from simplical_attn_amd import simplicial_attn as host
    B, N, H, D = 1, 8, 2, 16
    x = torch.zeros(B, N, H, D)
    lse = torch.zeros(B, H, N)
    # the checks themselves, on tensors of one device
    host._check_saved(x, x, lse, x)
    for bad_out in (x[:, :4], x.double(), x[0]):
        with pytest.raises(ValueError, match="out must match q"):
            host._check_saved(x, bad_out, lse, x)
    for bad_dout in (torch.zeros(B, N, H, D + 1), x.half()):
        with pytest.raises(ValueError, match="dout must match q"):
            host._check_saved(x, x, lse, bad_dout)
    with pytest.raises(ValueError, match="float32"):
        host._check_saved(x, x, lse.double(), x)
    with pytest.raises(ValueError, match="contiguous"):
        host._check_saved(x, x, torch.zeros(B, N, H), x)                    # the reference helper's [B,N,H] order
    with pytest.raises(ValueError, match="contiguous"):
        host._check_saved(x, x, torch.zeros(B, N, H).transpose(1, 2), x)    # right shape, wrong strides
    with pytest.raises(ValueError, match="lse must be"):
        host._check_saved(x, x, None, x)
    # and the entry point runs them (after the input checks, which refuse CPU tensors)
    with pytest.raises(RuntimeError, match="GPU only"):
        sa.simplicial_backward(x, x, x, x, x, x, lse, x, 4, 4)
    with pytest.raises(ValueError, match="k1 must match q"):
        sa.simplicial_backward(x, x[:, :4], x, x, x, x, lse, x, 4, 4)


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
