"""GPU parity of the bf16 MFMA backward kernels, through the C ABI.

Tolerance (bf16 path): max|diff| <= 2e-2 * max|ref| per gradient against the
fp64/fp32 oracle's autograd on the same bf16-rounded inputs.  Large shapes are
checked against the oracle on query-row ranges (gradients of K rows j with
[j, j+w1] inside the range, and of K' rows k with [k, k+w2] inside it, are then
complete) and, over whole tensors, against the generic fp32 kernels."""
import pytest
import torch

from tests.util import (assert_close_rel, assert_within, cancellation_bounds, make_inputs, oracle_all, run_device,
                        single_triple)

pytestmark = pytest.mark.gpu
GENERIC, MFMA = 1, 2
BF16_TOL = 2e-2
GRADS = ("dq", "dk1", "dk2", "dv1", "dv2")

SMALL = [  # B, N, H, D, w1, w2, k2_bias, v2_bias
    (1, 64, 1, 64, 16, 8, 0.0, 0.0),
    (2, 100, 2, 128, 40, 5, 0.0, 0.0),
    (1, 256, 2, 64, 512, 32, 0.0, 0.0),
    (1, 200, 1, 128, 0, 0, 0.0, 0.0),
    (1, 130, 2, 64, 33, 1, 0.1, 0.2),
    (1, 96, 1, 128, 7, 64, -0.1, -0.2),
    (2, 160, 3, 128, 64, 32, 1.0, 0.5),
    (1, 33, 1, 64, 31, 32, 0.0, 0.0),
    (1, 300, 2, 128, 130, 3, 0.0, 0.0),
    (1, 1, 1, 64, 4, 4, 0.0, 0.0),
    (2, 130, 2, 32, 33, 8, 0.1, 0.2),         # head_dim 32
    (1, 200, 1, 32, 64, 32, 0.0, 0.0),
    (1, 200, 1, 128, 16, 150, 0.0, 0.1),     # K' window wider than both kernels' LDS buffers: walked in segments of deltas
    (1, 180, 2, 128, 40, 100, 0.2, 0.0),     # K'-side in one piece (q, dO rows from global memory), K-side in segments
    (1, 150, 1, 128, 20, 65, 0.0, 0.0),      # first K' window the K-side kernel walks in two segments (64 is the last in one)
    (1, 190, 1, 128, 12, 113, 0.0, 0.0),     # last K' window the K'-side kernel takes in one segment
    (1, 190, 1, 128, 12, 114, 0.0, 0.0),     # first one in two
    (1, 350, 1, 64, 12, 304, 0.0, 0.0),      # head_dim 64: last K' window of one segment
    (1, 350, 1, 64, 12, 305, 0.1, 0.0),      # first of two (the second holds one delta)
    (1, 390, 1, 64, 9, 362, 0.0, 0.0),
    (2, 300, 2, 128, 16, 230, 0.1, -0.2),    # three segments (112, 112, 7 deltas), several heads
    (1, 100, 1, 128, 16, 300, 0.0, 0.0),     # window wider than the sequence: the later segments are empty
    (1, 700, 1, 64, 20, 650, 0.0, 0.0),      # head_dim 64, three segments
    (1, 900, 1, 32, 8, 850, 0.0, 0.1),       # head_dim 32, both kernels in two segments
]


@pytest.mark.parametrize("case", SMALL)
def test_small_shapes_vs_oracle(case):
    B, N, H, D, w1, w2, kb, vb = case
    inp = make_inputs(B, N, H, D, seed=N + D + w1, dtype=torch.bfloat16)
    got = run_device(inp, w1, w2, None, kb, vb, flags=MFMA)
    want = oracle_all(inp, w1, w2, None, kb, vb)
    # With single-triple windows dq, dk1, dk2 vanish by cancellation and a 16-bit kernel returns
    # rounding noise of a known shape: those are held to its elementwise bound instead.
    noise = cancellation_bounds(inp, want["out"], None, kb, vb) if single_triple(N, w1, w2) else {}
    for name in GRADS:
        if name in noise:
            assert_within(got[name], noise[name], name)
        else:
            assert_close_rel(got[name], want[name], BF16_TOL, name, label="small shapes bf16 (bwd)")


@pytest.mark.parametrize("case", [SMALL[1], SMALL[6], (1, 300, 2, 64, 96, 16, 0.1, 0.0), (2, 160, 2, 128, 64, 33, 0.0, 0.0),
                                  SMALL[12], SMALL[13],                  # K' windows in segments
                                  (1, 400, 1, 64, 24, 330, 0.0, 0.1)])   # the same at head_dim 64
def test_small_shapes_fp16_vs_oracle(case):
    """fp16 elements on the same kernels (fp16 MFMA), K' windows walked in segments included.
    Tolerance: max|diff| <= 1.5e-2 * max|ref| per tensor.  The products q*k2~ and dO*v2~ are rounded to
    fp16 before the MFMAs, as the reference rounds its products to the GEMM type (kernels.py:106,
    301-302); over most of a tensor that costs 1e-3, but on the first query rows, whose windows hold
    a few triples, the weights do not average it out: the worst measured element is dk1 at position 1
    of the biased w2 = 100 case, 1.22e-2 (the same on the on-chip kernels at w2 = 60; the fp32
    kernels, which do not round the products, measure 1.8e-3 there)."""
    B, N, H, D, w1, w2, kb, vb = case
    inp = make_inputs(B, N, H, D, seed=N + D + w1, dtype=torch.float16)
    got = run_device(inp, w1, w2, None, kb, vb, flags=MFMA)
    want = oracle_all(inp, w1, w2, None, kb, vb)
    for name in GRADS:
        assert got[name].dtype == torch.float16
        assert_close_rel(got[name], want[name], 1.5e-2, name, label="small shapes fp16 (bwd)")


def check_rows(got, inp, w1, w2, rows, label=None):
    """Oracle gradients of the loss restricted to query rows [r0, r1): complete for dq on those
    rows, and for K (K') rows whose whole forward reach [j, j+w] lies inside the range or is cut
    off by the end of the sequence."""
    r0, r1 = rows
    N = inp[0].shape[1]
    want = oracle_all(inp, w1, w2, dtype=torch.float32, rows=rows)
    assert_close_rel(got["out"][:, r0:r1], want["out"], BF16_TOL, "out rows %s" % (rows,), label=label)
    assert_close_rel(got["lse"][:, :, r0:r1], want["lse"], BF16_TOL, "lse rows %s" % (rows,), label=label)
    assert_close_rel(got["dq"][:, r0:r1], want["dq"][:, r0:r1], BF16_TOL, "dq rows %s" % (rows,), label=label)
    for name, w in (("dk1", w1), ("dv1", w1), ("dk2", w2), ("dv2", w2)):
        hi = r1 if r1 == N else r1 - w
        assert hi > r0
        assert_close_rel(got[name][:, r0:hi], want[name][:, r0:hi], BF16_TOL, "%s rows %s" % (name, rows),
                         label=label)


def check_large(B, N, H, D, w1, w2, seed, rows, qk_mag=None, more_rows=(), generic=True, label=None):
    inp = make_inputs(B, N, H, D, seed=seed, dtype=torch.bfloat16, qk_mag=qk_mag)
    got = run_device(inp, w1, w2, flags=MFMA)
    for r in (rows,) + tuple(more_rows):
        check_rows(got, inp, w1, w2, r, label)
    if generic:
        ref = run_device(inp, w1, w2, flags=GENERIC)
        for name in GRADS:
            assert_close_rel(got[name], ref[name].float().cpu(), BF16_TOL, name + " vs generic kernels")


def test_config3_forward_backward():
    """Benchmark configuration 3: bf16, B2 H8 N2048 D64, w 512/32, seed 2."""
    check_large(2, 2048, 8, 64, 512, 32, seed=2, rows=(0, 640), more_rows=((2048 - 640, 2048),),
                label="c3 bf16 B2 H8 N2048 D64 w512/32")


def test_config4_headline_shape_gradients():
    """Benchmark configuration 4: bf16, B1 H16 N8192 D128, w 512/32, seed 3: oracle on the first
    rows, the rows straddling i = w1 and the last rows; generic kernels on whole tensors."""
    check_large(1, 8192, 16, 128, 512, 32, seed=3, rows=(448, 1088),
                more_rows=((0, 608), (8192 - 640, 8192)), label="c4 bf16 B1 H16 N8192 D128 w512/32")


def test_segmented_k2_window_on_a_full_grid():
    """bf16 B2 H16 N2048 D128 w 48/130: a grid that fills the chip (the K-side kernel unsplit, walking the K' rows in
    segments of 65 deltas; the K'-side kernel with two workgroups per K' block, 112 + 19 deltas).  Oracle on the first
    rows and the last ones, the fp32 kernels over whole tensors."""
    check_large(2, 2048, 16, 128, 48, 130, seed=11, rows=(0, 320), more_rows=((2048 - 256, 2048),))


def test_config5_long_sequence_gradients():
    """Benchmark configuration 5: bf16, B1 H8 N32768 D128, w 1024/64, q/k/k' ~ N(0, 0.5^2), seed 4.  Checked
    on the first query rows, rows around i = w1 and the end of the sequence, LSE included (the
    generic kernels would take minutes at this size; whole tensors are covered by the doubling
    property below)."""
    check_large(1, 32768, 8, 128, 1024, 64, seed=4, rows=(992, 2048), qk_mag=0.5,
                more_rows=((0, 1120), (32768 - 320, 32768)), generic=False,
                label="c5 bf16 B1 H8 N32768 D128 w1024/64")


def test_config5_whole_tensor_doubling_property():
    """Size-independent check at configuration 5 over whole tensors: doubling v1 is exact in bf16 and
    in every fp32 sum, so out, dq, dk1, dk2 and dv2 double bit for bit while lse and dv1 stay."""
    inp = make_inputs(1, 32768, 8, 128, seed=4, dtype=torch.bfloat16, qk_mag=0.5)
    a = run_device(inp, 1024, 64, flags=MFMA)
    inp2 = list(inp)
    inp2[3] = inp[3] * 2
    b = run_device(inp2, 1024, 64, flags=MFMA)
    assert torch.isfinite(a["lse"]).all()
    assert torch.equal(b["lse"], a["lse"]) and torch.equal(b["dv1"], a["dv1"])
    for name in ("out", "dq", "dk1", "dk2", "dv2"):
        assert torch.isfinite(a[name].float()).all(), name
        assert torch.equal(b[name], a[name] * 2), name


def test_config4_whole_tensor_properties():
    """Size-independent checks at configuration 4 over whole tensors.  Doubling dO is exact in bf16 and in
    every fp32 sum, so all five gradients double bit for bit while out and lse stay; heads are
    independent, so permuting the heads of every input permutes every result bit for bit (each
    (batch, head) lands on other workgroups and another XCD)."""
    inp = make_inputs(1, 8192, 16, 128, seed=3, dtype=torch.bfloat16)
    a = run_device(inp, 512, 32, flags=MFMA)
    inp2 = list(inp)
    inp2[5] = inp[5] * 2
    b = run_device(inp2, 512, 32, flags=MFMA)
    assert torch.equal(b["out"], a["out"]) and torch.equal(b["lse"], a["lse"])
    for name in GRADS:
        assert torch.isfinite(a[name].float()).all(), name
        assert torch.equal(b[name], a[name] * 2), name
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(5))
    c = run_device([t[:, :, perm].contiguous() for t in inp], 512, 32, flags=MFMA)
    assert torch.equal(c["lse"], a["lse"][:, perm])
    for name in ("out",) + tuple(GRADS):
        assert torch.equal(c[name], a[name][:, :, perm]), name


def test_needs_input_grad_subsets_and_determinism():
    from simplical_attn_amd import TwoSimplicialAttentionFunction as Fn
    dev = torch.device("cuda:0")
    inp = make_inputs(1, 200, 2, 128, seed=21, dtype=torch.bfloat16)
    full = run_device(inp, 60, 12, flags=MFMA)
    again = run_device(inp, 60, 12, flags=MFMA)
    for name in GRADS:
        assert torch.equal(full[name], again[name]), name
    for subset in ((0,), (1, 3), (2, 4), (0, 1, 2)):
        leaves = [x.to(dev).requires_grad_(t in subset) for t, x in enumerate(inp[:5])]
        # the same kernel choice as `full` (pre-pass kernels included)
        Fn.apply(*leaves, 60, 12, None, 0.0, 0.0, True, MFMA).backward(inp[5].to(dev))
        for t, name in enumerate(GRADS):
            if t in subset:
                assert torch.equal(leaves[t].grad, full[name]), name
            else:
                assert leaves[t].grad is None


def test_segmented_k2_windows_half_open_subsets_and_determinism():
    """A K' window that both backward kernels walk in segments (head_dim 128, w2 = 180: 112 + 69 deltas on the
    K'-side, 65 + 65 + 51 on the K-side): the half-open window convention against the oracle, bitwise repeatability,
    and the gradient subsets of needs_input_grad bit for bit."""
    import simplical_attn_amd as sa
    dev = torch.device("cuda:0")
    inp = make_inputs(1, 260, 2, 128, seed=5, dtype=torch.bfloat16)
    w1, w2 = 30, 180
    got = run_device(inp, w1, w2, None, 0.1, 0.0, flags=MFMA, inclusive=False)
    want = oracle_all(inp, w1, w2, None, 0.1, 0.0, inclusive=False)
    for name in GRADS:
        assert_close_rel(got[name], want[name], BF16_TOL, name + " half-open, segments")
    x = [t.to(dev) for t in inp]
    out, lse = sa.simplicial_forward(*x[:5], w1, w2, flags=MFMA)
    full = sa.simplicial_backward(*x[:5], out, lse, x[5], w1, w2, flags=MFMA)
    again = sa.simplicial_backward(*x[:5], out, lse, x[5], w1, w2, flags=MFMA)
    for name, a, b in zip(GRADS, full, again):
        assert torch.equal(a, b), name
    for subset in ((0,), (1, 3), (2, 4), (2,)):
        needs = tuple(t in subset for t in range(5))
        part = sa.simplicial_backward(*x[:5], out, lse, x[5], w1, w2, needs=needs, flags=MFMA)
        for t, name in enumerate(GRADS):
            if t in subset:
                assert torch.equal(part[t], full[t]), name
            else:
                assert part[t] is None


def test_headline_shape_scaling_and_swap_properties():
    """Size-independent checks at the headline shape (bf16 B1 H16 N8192 D128 w 512/32), whole
    tensors.  (1) Doubling v1 is exact in bf16 and in every fp32 sum, so out, dq, dk1, dk2 and dv2
    must double bit for bit while lse and dv1 must not change at all.  (2) With w1 = w2 the operator
    is symmetric under (k1, v1) <-> (k2, v2): outputs agree within the bf16 bar and the gradient
    pairs swap (the two sides run through different kernels)."""
    inp = make_inputs(1, 8192, 16, 128, seed=3, dtype=torch.bfloat16)
    a = run_device(inp, 512, 32, flags=MFMA)
    inp2 = list(inp)
    inp2[3] = inp[3] * 2
    b = run_device(inp2, 512, 32, flags=MFMA)
    assert torch.equal(b["lse"], a["lse"]) and torch.equal(b["dv1"], a["dv1"])
    for name in ("out", "dq", "dk1", "dk2", "dv2"):
        assert torch.equal(b[name], a[name] * 2), name
    w = 64
    small = [x[:, :2048, :4].contiguous() for x in inp]
    c = run_device(small, w, w, flags=MFMA)
    q, k1, k2, v1, v2, dout = small
    d = run_device([q, k2, k1, v2, v1, dout], w, w, flags=MFMA)
    assert_close_rel(d["out"], c["out"].float().cpu(), BF16_TOL, "out under swap")
    for x, y in (("dq", "dq"), ("dk1", "dk2"), ("dk2", "dk1"), ("dv1", "dv2"), ("dv2", "dv1")):
        assert_close_rel(d[x], c[y].float().cpu(), BF16_TOL, "%s under swap" % x)


def test_packed_projection_views_take_the_mfma_kernels():
    """q, k1, k2, v1, v2 as slices of one [B, N, 5, H, D] projection output (row stride 5*H*D, no
    copies): the MFMA kernels take per-tensor strides, and every result equals the one from
    contiguous copies bit for bit."""
    import simplical_attn_amd as sa
    from simplical_attn_amd import _lib
    dev = torch.device("cuda:0")
    B, N, H, D, w1, w2 = 2, 200, 3, 128, 70, 12
    g = torch.Generator().manual_seed(77)
    packed = torch.randn(B, N, 5, H, D, generator=g).to(torch.bfloat16).to(dev)
    dout = torch.randn(B, N, H, D, generator=g).to(torch.bfloat16).to(dev)
    views = [packed[:, :, t] for t in range(5)]
    assert all(not v.is_contiguous() for v in views)
    out_v, lse_v = sa.simplicial_forward(*views, w1, w2, flags=_lib.FLAG_FORCE_MFMA)
    grads_v = sa.simplicial_backward(*views, out_v, lse_v, dout, w1, w2, flags=_lib.FLAG_FORCE_MFMA)
    copies = [v.contiguous() for v in views]
    out_c, lse_c = sa.simplicial_forward(*copies, w1, w2, flags=_lib.FLAG_FORCE_MFMA)
    grads_c = sa.simplicial_backward(*copies, out_c, lse_c, dout, w1, w2, flags=_lib.FLAG_FORCE_MFMA)
    assert torch.equal(out_v, out_c) and torch.equal(lse_v, lse_c)
    for a, b in zip(grads_v, grads_c):
        assert torch.equal(a, b)
    want = oracle_all([c.cpu() for c in copies] + [dout.cpu()], w1, w2)
    assert_close_rel(out_v, want["out"], BF16_TOL, "out")
    assert_close_rel(grads_v[0], want["dq"], BF16_TOL, "dq")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_head_dim_16_is_padded_onto_the_mfma_kernels(dtype):
    """head_dim 16 (simplicial/test_correctness.py:32): tensors are zero-padded to 32 columns
    by the host wrapper and run on the MFMA kernels of their element type; results equal those of the MFMA
    kernels on the hand-padded tensors bit for bit (same scale) and meet the oracle at the type's parity bar."""
    import simplical_attn_amd as sa
    B, N, H, D, w1, w2 = 2, 150, 3, 16, 40, 9
    inp = make_inputs(B, N, H, D, seed=16, dtype=dtype)
    got = run_device(inp, w1, w2, None, 0.1, -0.2, flags=0)
    want = oracle_all(inp, w1, w2, None, 0.1, -0.2)
    tol = BF16_TOL if dtype == torch.bfloat16 else 1e-2 if dtype == torch.float16 else 1e-5
    for name in ("out", "lse") + GRADS:
        assert got[name].shape[-1] == (N if name == "lse" else D)
        assert_close_rel(got[name], want[name], tol, name)
    dev = torch.device("cuda:0")
    pad = [torch.nn.functional.pad(x.to(dev), (0, 16)) for x in inp]
    out, lse = sa.simplicial_forward(*pad[:5], w1, w2, D ** -0.5, 0.1, -0.2, flags=MFMA)
    grads = sa.simplicial_backward(*pad[:5], out, lse, pad[5], w1, w2, D ** -0.5, 0.1, -0.2, flags=MFMA)
    assert torch.equal(got["out"], out[..., :D]) and torch.equal(got["lse"], lse)
    assert not out[..., D:].any()
    for name, g in zip(GRADS, grads):
        assert torch.equal(got[name], g[..., :D]), name
        assert not g[..., D:].any(), name
