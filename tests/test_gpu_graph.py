"""The C entry points allocate nothing, synchronise nothing and launch on the stream they are
given, so a forward + backward can be recorded into a HIP graph and replayed."""
import pytest
import torch

from tests.util import make_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_forward_backward_replay_in_a_graph(dtype):
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2 = 1, 320, 2, 128, 96, 32
    static = [x.to(dev) for x in make_inputs(B, N, H, D, seed=100, dtype=dtype)]

    def run():
        out, lse = sa.simplicial_forward(*static[:5], w1, w2)
        grads = sa.simplicial_backward(*static[:5], out, lse, static[5], w1, w2)
        return (out, lse, *grads)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                   # first call outside the capture (library load, attributes)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = run()
    # several replays on fresh data, with eager work and synchronisations in between; the kernels
    # are deterministic, so every replay must reproduce the eager result bit for bit
    for r in range(3):
        fresh = [x.to(dev) for x in make_inputs(B, N, H, D, seed=200 + r, dtype=dtype)]
        for s, f in zip(static, fresh):
            s.copy_(f)
        eager = [t.clone() for t in run()]
        torch.cuda.synchronize()
        for t in recorded:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("out", "lse", "dq", "dk1", "dk2", "dv1", "dv2"), recorded, eager):
            assert torch.equal(a, b), "replay %d: %s differs from the eager result" % (r, name)
