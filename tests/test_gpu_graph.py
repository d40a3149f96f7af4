"""The forward and the backward under HIP graph capture (torch.cuda.CUDAGraph): the library makes no
synchronising call, records no memset and launches on the stream it is given, so a step can be
captured once and replayed.  Every replay is compared bit for bit with the eager result on the same
inputs, with eager work and synchronisations between the replays and new input data before each.
Covered: the MFMA kernels (forced), the default dispatch on 16-bit and on fp32 tensors, a head_dim the
default dispatch sends to the fp32 kernels, and the backward entry point that brings its own workspace
(sa2_backward_static_workspace), captured after one warm call."""
import pytest
import torch

from simplical_attn_amd import _lib

pytestmark = pytest.mark.gpu
AUTO, MFMA = 0, 2
NAMES = ("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2")


def _step(sa, x, dout, w1, w2, flags):
    out, lse = sa.simplicial_forward(*x, w1, w2, flags=flags)
    grads = sa.simplicial_backward(*x, out, lse, dout, w1, w2, flags=flags)
    return (out, lse) + tuple(grads)


def _replay_and_compare(capture, eager, fresh, static):
    """capture(): launches on the current stream using the tensors in `static`, returns result tensors;
    eager(inputs): the same work, eagerly, on other tensors."""
    capture()                          # first calls outside the capture: once-per-device set-up of the library
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = capture()
    for replay in range(3):
        new = fresh()
        for s, n in zip(static, new):
            s.copy_(n)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = eager(new)                                   # eager work between the replays
        torch.cuda.synchronize()
        for name, a, b in zip(NAMES[-len(got):], got, want):
            assert torch.isfinite(a.float()).all(), (name, replay)
            assert torch.equal(a, b), (name, replay)


@pytest.mark.parametrize("shape", [
    (2, 256, 2, 64, 40, 8, torch.bfloat16, MFMA), (1, 512, 4, 128, 512, 32, torch.bfloat16, MFMA),
    (1, 300, 2, 128, 33, 80, torch.bfloat16, MFMA), (1, 300, 2, 128, 33, 32, torch.float16, AUTO),
    (2, 200, 2, 64, 40, 8, torch.float32, AUTO), (1, 130, 2, 48, 20, 5, torch.bfloat16, AUTO)])
def test_captured_step_replays_like_eager(shape):
    import simplical_attn_amd as sa
    B, N, H, D, w1, w2, dtype, flags = shape
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(N + w2)
    fresh = lambda: [torch.randn(B, N, H, D, generator=g).to(dtype).to(dev) for _ in range(6)]
    static = fresh()
    _replay_and_compare(lambda: _step(sa, static[:5], static[5], w1, w2, flags),
                        lambda new: _step(sa, new[:5], new[5], w1, w2, flags), fresh, static)


@pytest.mark.parametrize("dtype,flags", [(torch.bfloat16, MFMA), (torch.float32, AUTO)])
def test_captured_static_workspace_backward_replays_like_eager(dtype, flags):
    """The entry point for callers that cannot allocate, under capture.  Its first call on a device
    looks up the address of the library's workspace array (and sets kernel attributes): that call is
    made outside the capture, as the header asks."""
    import simplical_attn_amd as sa
    lib = _lib.load()
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2 = 2, 256, 2, 64, 40, 8
    code = {torch.bfloat16: _lib.SA2_BF16, torch.float32: _lib.SA2_F32}[dtype]
    g = torch.Generator().manual_seed(3)
    fresh = lambda: [torch.randn(B, N, H, D, generator=g).to(dtype).to(dev) for _ in range(6)]
    static = fresh()
    out = torch.empty_like(static[0])
    lse = torch.empty(B, H, N, dtype=torch.float32, device=dev)
    grads = [torch.empty_like(static[0]) for _ in range(5)]
    tens = (*static[:5], out, static[5], *grads)
    strides = _lib.stride_array([(t.stride(0), t.stride(1), t.stride(2)) for t in tens])

    def capture():
        stream = torch.cuda.current_stream(dev).cuda_stream
        _lib.check(lib.sa2_forward(*[t.data_ptr() for t in static[:5]], out.data_ptr(), lse.data_ptr(), B, N, H, D,
                                   strides, w1, w2, D ** -0.5, 0.0, 0.0, code, 1, flags, stream))
        _lib.check(lib.sa2_backward_static_workspace(
            *[t.data_ptr() for t in static[:5]], out.data_ptr(), static[5].data_ptr(), lse.data_ptr(),
            *[t.data_ptr() for t in grads], B, N, H, D, strides, w1, w2, D ** -0.5, 0.0, 0.0, code, 1, flags, stream))
        return grads

    _replay_and_compare(capture, lambda new: _step(sa, new[:5], new[5], w1, w2, flags)[2:], fresh, static)
