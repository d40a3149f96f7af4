"""The forward and the backward under HIP graph capture (torch.cuda.CUDAGraph): the library makes no
synchronising call, records no memset and launches on the stream it is given, so a step can be
captured once and replayed.  Every replay is compared bit for bit with the eager result on the same
inputs, with eager work and synchronisations between the replays and new input data before each."""
import pytest
import torch

pytestmark = pytest.mark.gpu
MFMA = 2


def _step(sa, x, dout, w1, w2):
    out, lse = sa.simplicial_forward(*x, w1, w2, flags=MFMA)
    grads = sa.simplicial_backward(*x, out, lse, dout, w1, w2, flags=MFMA)
    return (out, lse) + tuple(grads)


@pytest.mark.parametrize("shape", [(2, 256, 2, 64, 40, 8), (1, 512, 4, 128, 512, 32), (1, 300, 2, 128, 33, 80)])
def test_captured_step_replays_like_eager(shape):
    import simplical_attn_amd as sa
    B, N, H, D, w1, w2 = shape
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(N + w2)
    fresh = lambda: [torch.randn(B, N, H, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(6)]
    static = fresh()
    # first calls outside the capture: the library sets each kernel's LDS limit once per device
    _step(sa, static[:5], static[5], w1, w2)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = _step(sa, static[:5], static[5], w1, w2)
    for replay in range(3):
        new = fresh()
        for s, n in zip(static, new):
            s.copy_(n)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = _step(sa, new[:5], new[5], w1, w2)          # eager work between the replays
        torch.cuda.synchronize()
        for name, a, b in zip(("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2"), got, want):
            assert torch.isfinite(a.float()).all(), (name, replay)
            assert torch.equal(a, b), (name, replay)
