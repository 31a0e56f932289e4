"""HIP graph capture of launches (torch.cuda.graph): after one eager call with the same shapes, which sizes the
workspaces, a launch records kernels and copies only, so the replayed graph must reproduce the eager result bit for
bit on new input values.  Nothing on the way waits for the device: the two-phase K-nearest-neighbour schedule keeps its
fallback on the device, block-sparse ranges are validated on the host once and then served without a read-back."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _replays_like_eager(fn, inputs, replays=3):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn(*inputs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn(*inputs)
    gen = torch.Generator(device="cuda").manual_seed(1)
    for _ in range(replays):
        for t in inputs:
            if t.numel() > 1:
                t.copy_(torch.randn(t.shape, device="cuda", generator=gen) * t.std())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        ref = fn(*inputs)           # eager work between the replays
        torch.cuda.synchronize()
        if not torch.equal(got, ref):
            return False
    return True


def _scheme_of_last_module():
    from keops_amd import keops_io

    return list(keops_io._loaders.values())[-1].module.meta("scheme")


def test_dense_schemes_under_graph_capture():
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(0)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    x, y, b, g = r(5000, 3), r(7000, 3), r(7000, 2), torch.tensor([0.5], device="cuda")
    conv = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    assert _replays_like_eager(conv, [x, y, b, g])
    assert _replays_like_eager(conv, [r(300, 3), y, b, g])          # few rows: column slabs + merge kernel
    lse = Genred("-g*SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)", "g=Pm(1)"], reduction_op="LogSumExp", axis=1)
    assert _replays_like_eager(lse, [x, y, g])
    lap = Genred("Exp(-Norm2(x-y))*b", ["x=Vi(128)", "y=Vj(128)", "b=Vj(8)"], reduction_op="Sum", axis=1)
    assert _replays_like_eager(lap, [r(3000, 128) / 3, r(4000, 128) / 3, r(4000, 8)])
    assert _scheme_of_last_module() == "chunk"
    fin = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(200)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    assert _replays_like_eager(fin, [x, y, r(7000, 200), g])
    assert _scheme_of_last_module() == "final"


def test_batched_reduction_under_graph_capture():
    from keops_amd.torch import LazyTensor

    gen = torch.Generator(device="cuda").manual_seed(2)
    xb, yb, bb = (torch.randn(*s, device="cuda", generator=gen) for s in ((4, 2000, 3), (4, 3000, 3), (4, 3000, 1)))

    def batched(xb, yb, bb):
        d = ((LazyTensor(xb[:, :, None, :]) - LazyTensor(yb[:, None, :, :])) ** 2).sum(-1)
        return ((-d).exp() * LazyTensor(bb[:, None, :, :])).sum(2)

    assert _replays_like_eager(batched, [xb, yb, bb])


def test_knn_two_phase_schedule_under_capture():
    """20000 x 40000 references run the sampled two-phase schedule (thresholds from a sample, fixed-threshold filter,
    exact replay of the survivors).  Its fallback for overflowing candidate logs is a kernel that is launched behind
    it and returns at once unless the device raised the flag: no read-back, so the same launches record into a graph
    and replay bit for bit on new data."""
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(3)
    x, y = torch.rand(20000, 16, device="cuda", generator=gen), torch.rand(40000, 16, device="cuda", generator=gen)
    knn = Genred("SqDist(x,y)", ["x=Vi(16)", "y=Vj(16)"], reduction_op="ArgKMin", axis=1, opt_arg=8)
    assert _replays_like_eager(knn, [x, y], replays=2)
    assert _scheme_of_last_module() == "knn"


def _block_ranges(edges_i, edges_j, keep):
    """ranges tuple (device int64 tensors) of a block-sparse pattern: keep[a] lists the column blocks of row block a."""
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    ranges_i = [[edges_i[a], edges_i[a + 1]] for a in range(len(edges_i) - 1)]
    ranges_j = [[edges_j[b], edges_j[b + 1]] for b in range(len(edges_j) - 1)]
    red_j, slices_i = [], []
    for a in range(len(ranges_i)):
        red_j += [ranges_j[b] for b in keep[a]]
        slices_i.append(len(red_j))
    red_i, slices_j = [], []
    for b in range(len(ranges_j)):
        red_i += [ranges_i[a] for a in range(len(ranges_i)) if b in keep[a]]
        slices_j.append(len(red_i))
    return (i64(ranges_i), i64(slices_i), i64(red_j), i64(ranges_j), i64(slices_j), i64(red_i))


def _masked_dense(x, y, b, ranges):
    ri, sl, rj = (t.cpu().tolist() for t in ranges[:3])
    out = torch.zeros(x.shape[0], b.shape[1], dtype=torch.float64, device="cuda")
    for a, (s, e) in enumerate(ri):
        for k in range(0 if a == 0 else sl[a - 1], sl[a]):
            js, je = rj[k]
            K = torch.exp(-torch.cdist(x[s:e].double(), y[js:je].double()) ** 2)
            out[s:e] += K @ b[js:je].double()
    return out


def test_block_sparse_ranges_under_graph_capture():
    """The first launch with a set of range tensors reads them back and validates them (it refuses capture, with a
    message that says so); from the second on the workgroup table is built on the device, so the launch records into
    a graph, replays follow new input values and in-place changes of the ranges, and indices that have gone out of
    bounds are clamped and flagged instead of faulting."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(4)
    x, y, b = (torch.randn(n, d, device="cuda", generator=gen) for n, d in ((3000, 3), (3500, 3), (3500, 2)))
    ranges = _block_ranges([0, 700, 1500, 1501, 3000], [0, 900, 2000, 3500], [[0, 1], [1], [0, 2], [2]])
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], reduction_op="Sum", axis=1)

    fresh = tuple(t.clone() for t in ranges)          # tensors the module has not seen: host path only
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="cannot be captured"):
        with torch.cuda.graph(graph):
            conv(x, y, b, ranges=fresh)
    torch.cuda.synchronize()

    ref = conv(x, y, b, ranges=ranges)                 # host path: read back, validated
    err = (ref.double() - _masked_dense(x, y, b, ranges)).norm() / _masked_dense(x, y, b, ranges).norm()
    assert float(err) < 1e-5
    again = conv(x, y, b, ranges=ranges)               # device path
    assert torch.equal(again, ref)
    module = keops_io.last_loader.module
    assert module.ranges_status() == 0

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        conv(x, y, b, ranges=ranges)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = conv(x, y, b, ranges=ranges)
    for k in range(3):
        x.copy_(torch.randn(x.shape, device="cuda", generator=gen))
        b.copy_(torch.randn(b.shape, device="cuda", generator=gen))
        if k == 2:                                      # the pattern changes in place: row block 0 loses column block 1
            ranges[2][1] = torch.tensor([0, 0], device="cuda")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = _masked_dense(x, y, b, ranges)
        assert float((got.double() - want).norm() / want.norm()) < 1e-5
        assert torch.equal(conv(x, y, b, ranges=ranges), got)      # eager work between the replays
    # an index beyond the reduced axis: clamped (the kernels sweep the ranges unchecked) and flagged
    ranges[2][2] = torch.tensor([2000, 10 ** 9], device="cuda")
    clamped = conv(x, y, b, ranges=ranges)
    torch.cuda.synchronize()
    assert module.ranges_status() & 1
    ranges[2][2] = torch.tensor([2000, 3500], device="cuda")
    assert torch.equal(conv(x, y, b, ranges=ranges), clamped)
    assert module.ranges_status() == 0


def test_captured_graph_survives_later_eager_calls_at_other_shapes():
    """A captured graph holds raw pointers into the module's workspace.  A later eager call of the same formula that
    needs a larger workspace must not free it under the graph: the library keeps the graph's buffer alive and gives the
    eager calls a new one, so both keep producing the right results."""
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(5)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    conv = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    x, y, b, g = r(300, 3), r(60000, 3), r(60000, 2), torch.tensor([0.5], device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        conv(x, y, b, g)                      # sizes the slab workspace
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = conv(x, y, b, g)
    graph.replay()
    torch.cuda.synchronize()
    ref = out.clone()
    # a smaller call of the same module (same row bucket) fits the frozen workspace
    small = conv(x[:200].contiguous(), y[:30000].contiguous(), b[:30000].contiguous(), g)
    torch.cuda.synchronize()
    assert torch.isfinite(small).all()
    # a larger one outgrows it (1562 slabs of 400 rows against 234 of 300): new buffer, the old one stays with the graph
    x2 = r(400, 3)
    y2, b2 = r(400000, 3), r(400000, 2)
    big = conv(x2, y2, b2, g)
    torch.cuda.synchronize()
    K = torch.exp(-0.5 * torch.cdist(x2.double(), y2.double()) ** 2)
    assert float((big.double() - K @ b2.double()).norm() / (K @ b2.double()).norm()) < 1e-5
    for _ in range(2):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref)
    # batched launches: the graph reads lookup / offset tables; a call with other batch shapes builds its own
    from keops_amd.torch import LazyTensor

    def batched(xb, yb, bb):
        d = ((LazyTensor(xb[:, :, None, :]) - LazyTensor(yb[:, None, :, :])) ** 2).sum(-1)
        return ((-d).exp() * LazyTensor(bb[:, None, :, :])).sum(2)

    xb, yb, bb = r(4, 700, 3), r(4, 900, 3), r(4, 900, 1)
    with torch.cuda.stream(side):
        batched(xb, yb, bb)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2):
        outb = batched(xb, yb, bb)
    g2.replay()
    torch.cuda.synchronize()
    refb = outb.clone()
    other = batched(r(3, 1100, 3), r(3, 500, 3), r(3, 500, 1))      # other shapes, same module: new tables
    torch.cuda.synchronize()
    assert torch.isfinite(other).all()
    outb.zero_()
    g2.replay()
    torch.cuda.synchronize()
    assert torch.equal(outb, refb)
