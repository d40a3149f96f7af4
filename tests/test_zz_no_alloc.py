"""sa2_backward_static_workspace (the entry point for callers that cannot allocate: its workspace
is an array inside the library) against sa2_backward (caller-provided workspace), both through
the C ABI, bit for bit, on two calls in a row, the second on a smaller problem: the array keeps
the first call's contents, which the second call must not see."""
import pytest
import torch

from simplical_attn_amd import _lib
from tests.util import make_inputs

pytestmark = pytest.mark.gpu

DT = {torch.bfloat16: _lib.SA2_BF16, torch.float32: _lib.SA2_F32}


def _both_backwards(shape, w, dtype, seed, flags, inclusive=1, needs=(True,) * 5):
    import simplical_attn_amd as sa
    lib = _lib.load()
    dev = torch.device("cuda:0")
    B, N, H, D = shape
    q, k1, k2, v1, v2, dout = [t.to(dev) for t in make_inputs(B, N, H, D, seed, dtype)]
    out, lse = sa.simplicial_forward(q, k1, k2, v1, v2, w[0], w[1], flags=flags, window_inclusive=bool(inclusive))
    stream = torch.cuda.current_stream(dev).cuda_stream
    scale = D ** -0.5
    nbytes = lib.sa2_bwd_workspace_bytes(B, N, H, D, w[0], w[1], DT[dtype], flags)
    assert 0 < nbytes <= _lib.STATIC_WORKSPACE_BYTES
    results = []
    free_before = None
    for static in (False, True):
        # gradients start from different garbage in the two runs: every element must be written
        grads = [torch.full_like(q, 7.0 if static else -3.0) for _ in range(5)]
        strides = _lib.stride_array([(t.stride(0), t.stride(1), t.stride(2))
                                     for t in (q, k1, k2, v1, v2, out, dout, *grads)])
        head = [t.data_ptr() for t in (q, k1, k2, v1, v2, out, dout, lse)]
        head += [g.data_ptr() if need else None for g, need in zip(grads, needs)]      # NULL = not needed
        tail = [B, N, H, D, strides, w[0], w[1], scale, 0.0, 0.0, DT[dtype], inclusive, flags, stream]
        if static:
            # The first call on a device looks up the library's array (the runtime places it in device
            # memory then) and sets kernel attributes; every later call only launches kernels.
            _lib.check(lib.sa2_backward_static_workspace(*head, *tail))
            for g in grads:
                g.fill_(7.0)
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info(dev)[0]
            _lib.check(lib.sa2_backward_static_workspace(*head, *tail))
            torch.cuda.synchronize()
            # the call allocates nothing: the device's free memory is what it was (nothing else runs
            # between the two readings; torch's own allocator is not called either)
            assert torch.cuda.mem_get_info(dev)[0] == free_before
        else:
            ws = torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=dev)
            _lib.check(lib.sa2_backward(*head, ws.data_ptr(), ws.numel(), *tail))
        torch.cuda.synchronize()
        results.append(grads)
    return results


@pytest.mark.parametrize("dtype,flags,first,second", [
    (torch.bfloat16, _lib.FLAG_FORCE_MFMA, ((1, 640, 4, 128), (96, 16)), ((1, 200, 2, 128), (40, 8))),
    (torch.bfloat16, _lib.FLAG_FORCE_MFMA, ((2, 512, 2, 64), (64, 32)), ((1, 96, 2, 64), (32, 5))),
    (torch.float32, _lib.FLAG_AUTO, ((1, 192, 2, 64), (32, 16)), ((1, 70, 1, 64), (16, 4))),
    # a K' window that both backward kernels walk in segments (partial dK', dV' in the workspace too), then a plain one
    (torch.bfloat16, _lib.FLAG_FORCE_MFMA, ((1, 260, 2, 128), (24, 180)), ((1, 130, 1, 128), (16, 12))),
])
@pytest.mark.parametrize("inclusive", [1, 0])
def test_static_workspace_backward_matches_caller_workspace(dtype, flags, first, second, inclusive):
    for call, (shape, w) in enumerate((first, second)):
        plain, static = _both_backwards(shape, w, dtype, seed=11 + call, flags=flags, inclusive=inclusive)
        for name, a, b in zip(("dq", "dk1", "dk2", "dv1", "dv2"), plain, static):
            assert torch.isfinite(b.float()).all(), (call, name)
            assert torch.equal(a, b), "call %d, %s: static-workspace result differs" % (call, name)


@pytest.mark.parametrize("needs", [(False, True, False, True, True), (True, False, True, False, False)])
def test_static_workspace_backward_with_null_gradients(needs):
    """NULL gradient pointers (needs_input_grad false): the requested gradients equal the caller-workspace
    entry point's, the tensors behind the NULL pointers are never written (they are not even passed)."""
    for dtype, flags, shape, w in ((torch.bfloat16, _lib.FLAG_FORCE_MFMA, (1, 320, 2, 128), (64, 16)),
                                   (torch.float32, _lib.FLAG_AUTO, (1, 100, 2, 64), (24, 6))):
        plain, static = _both_backwards(shape, w, dtype, seed=5, flags=flags, needs=needs)
        full, _ = _both_backwards(shape, w, dtype, seed=5, flags=flags)
        for name, need, a, b, f in zip(("dq", "dk1", "dk2", "dv1", "dv2"), needs, plain, static, full):
            if need:
                assert torch.equal(a, b) and torch.equal(b, f), name
            else:
                assert (b == 7.0).all() and (a == -3.0).all(), name          # the fill values: untouched


def test_static_workspace_rejects_what_does_not_fit():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    # c4 needs ~134 MB of dQ partials: beyond the array
    assert lib.sa2_bwd_workspace_bytes(1, 8192, 16, 128, 512, 32, _lib.SA2_BF16, 0) > _lib.STATIC_WORKSPACE_BYTES
    x = torch.zeros(8, device=dev)
    strides = _lib.stride_array([(16 * 8192 * 128, 16 * 128, 128)] * 12)
    p = x.data_ptr()
    rc = lib.sa2_backward_static_workspace(p, p, p, p, p, p, p, p, p, p, p, p, p, 1, 8192, 16, 128, strides,
                                           512, 32, 0.1, 0.0, 0.0, _lib.SA2_BF16, 1, 0, None)
    assert rc == -10
    assert b"SA2_STATIC_WORKSPACE_BYTES" in lib.sa2_strerror(rc)
