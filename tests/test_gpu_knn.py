"""GPU parity of the matrix-core KNN path (keops_knn_mfma.h: bf16 MFMA filter + exact re-rank):
indices AND distances bit-identical to the CPU oracle, ties resolved to the lower index."""
import numpy as np
import pytest
import torch

from common import to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _matrix_core_scheme_at_every_size(monkeypatch):
    """Small problems normally stay on the general-purpose kernel: these tests are about the other one."""
    import keops_amd.get_keops_dll as engine
    from keops_amd import config, keops_io

    monkeypatch.setattr(config, "knn_min_work", 0)
    engine._cache.clear()
    keops_io._loaders.clear()
    yield
    engine._cache.clear()
    keops_io._loaders.clear()


def _knn(D, K, op="KMin_ArgKMin", axis=1):
    from keops_amd.torch import Genred

    return Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op=op, axis=axis, opt_arg=K)


def _uses_mfma_module():
    from keops_amd import keops_io

    return any(ld.module is not None and ld.module.meta("scheme") == "knn" for ld in keops_io._loaders.values())


@pytest.mark.parametrize("M,N,D,K", [(1000, 20000, 64, 10), (777, 5001, 40, 3), (300, 3000, 128, 1), (5000, 9999, 32, 16),
                                     (64, 100, 64, 10), (10, 7, 64, 10)])
def test_knn_bit_exact_small(M, N, D, K):
    rng = np.random.default_rng(2)
    x = rng.random((M, D)).astype(np.float32)
    y = rng.random((N, D)).astype(np.float32)
    if N > 60:
        y[40] = y[5]
        y[N - 1] = y[5]  # exact ties: lower index first
        x[1] = y[5]
    vals, idx = _knn(D, K)(*to_dev(x, y))
    assert _uses_mfma_module()
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    assert np.array_equal(idx.cpu().numpy().reshape(M, K), ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy().reshape(M, K), ref[:, 0::2])
    if N > 60 and K >= 3:
        assert idx[1, :3].tolist() == [5, 40, N - 1]
    only = _knn(D, K, "ArgKMin")(*to_dev(x, y)).cpu().numpy().reshape(M, K)
    assert np.array_equal(only, ref[:, 1::2].astype(np.int64))
    onlyv = _knn(D, K, "KMin")(*to_dev(x, y)).cpu().numpy().reshape(M, K)
    assert np.array_equal(onlyv, ref[:, 0::2])


def test_knn_gaussian_uncentred_data_and_axis0():
    """Data far from the origin (the centring pre-pass keeps the filter tight) and reduction over i."""
    M, N, D, K = 900, 30000, 64, 5
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((M, D)) + 50.0).astype(np.float32)
    y = (rng.standard_normal((N, D)) + 50.0).astype(np.float32)
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    vals, idx = _knn(D, K)(*to_dev(x, y))
    assert np.array_equal(idx.cpu().numpy(), ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy(), ref[:, 0::2])
    # axis=0: for every y_j the K nearest x_i
    ref0 = cpu_reduc("sqdist", [y[:4000], x], 4000, M, 1, reduction="ArgKMin", K=K, scheme="direct_sum")
    idx0 = _knn(D, K, "ArgKMin", axis=0)(*to_dev(x, y[:4000]))
    assert np.array_equal(idx0.cpu().numpy(), ref0.astype(np.int64))


@pytest.mark.parametrize("case", ["huge_reference", "infinite_reference", "nan_reference", "references_1e4_times_larger", "huge_query"])
def test_a_far_or_non_finite_point_does_not_cost_the_others_their_neighbours(case):
    """The filters work on points centred on the references' mean: one reference at 1e30 moved that mean by 1e30 / N and
    every centred point became that number (no neighbour found for any query); an infinite one made it NaN.  The centre
    is now the per-component median of a sample when the mean is far from it (keops_knn_centre): indices and distances
    equal the reference's loops for every query (a query that is itself at 1e30 has all its distances infinite)."""
    M, N, D, K = 3000, 40000, 64, 5
    rng = np.random.default_rng(8)
    x, y = rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)
    if case == "huge_reference":
        y[99, 5] = 1e30
    elif case == "infinite_reference":
        y[99, 5] = np.inf
    elif case == "nan_reference":
        y[99, 5] = np.nan
    elif case == "references_1e4_times_larger":
        y[100:103] *= 1e4
    else:
        x[77, 5] = 1e30
    vals, idx = _knn(D, K)(*to_dev(x, y))
    assert _uses_mfma_module()
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    keep = np.ones(M, bool)
    if case == "huge_query":
        keep[77] = False
        assert np.all(np.isinf(vals[77].cpu().numpy()))
    assert np.array_equal(idx.cpu().numpy()[keep], ref[keep, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy()[keep], ref[keep, 0::2])


def test_knn_config3_query_subset():
    # headline configuration 3: M=100,000 queries, N=1,000,000 references, D=64, K=10, U[0,1), seed 2
    M, N, D, K = 100_000, 1_000_000, 64, 10
    rng = np.random.default_rng(2)
    x = rng.random((M, D), dtype=np.float32)
    y = rng.random((N, D), dtype=np.float32)
    vals, idx = _knn(D, K)(*to_dev(x, y))
    from keops_amd import keops_io

    # bounded data: the device lets the fixed-threshold filter run on signed bytes (keops_knn_filter_i8)
    assert keops_io.last_loader.module.meta("knn_i8") == "1" and keops_io.last_loader.module.path_status() == 1
    rows = np.sort(np.random.default_rng(7).choice(M, 1024, replace=False)).astype(np.int64)
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum", rows=rows)
    sel = torch.from_numpy(rows).cuda()
    assert np.array_equal(idx[sel].cpu().numpy(), ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals[sel].cpu().numpy(), ref[:, 0::2])
    # size-independent properties on the full output: sorted distances, valid and distinct indices,
    # and the returned distance is the exact distance of the returned index
    assert bool((vals[:, 1:] >= vals[:, :-1]).all())
    assert int(idx.min()) >= 0 and int(idx.max()) < N
    s = torch.sort(idx, dim=1).values
    assert bool((s[:, 1:] != s[:, :-1]).all())
    q = torch.arange(0, M, 97, device="cuda")
    xq, yq = torch.from_numpy(x).cuda()[q], torch.from_numpy(y).cuda()[idx[q, 0]]
    d0 = ((xq.double() - yq.double()) ** 2).sum(1)
    assert torch.allclose(vals[q, 0].double(), d0, rtol=1e-5)


@pytest.mark.parametrize("kind,D,K,taken", [("uniform", 64, 10, 1), ("gauss", 100, 3, 1), ("ties", 40, 5, 1), ("offset", 33, 16, 1),
                                            ("outlier", 64, 10, 0), ("heavy", 48, 3, 0), ("tight_clusters", 128, 10, 0)])
def test_byte_filter_or_bf16_filter_chosen_on_the_device(kind, D, K, taken):
    """Two-phase launches in 32 dimensions and more quantise both sets to signed bytes (step = largest centred component
    / 127) and filter with v_mfma_i32_32x32x32_i8: integer products are exact, so |x - y| differs from the distance of
    the quantised points by at most the two quantisation residuals.  Where that slack is large against the search
    radii (outliers, heavy tails, clusters much tighter than their spread) the device keeps the bfloat16 filter.
    Either way the exact re-rank returns the oracle's bits."""
    from keops_amd import keops_io

    M, N = 2500, 60000
    rng = np.random.default_rng(1000 + D + K)
    if kind in ("uniform", "outlier", "offset"):
        x, y = rng.random((M, D)), rng.random((N, D))
        if kind == "outlier":
            y[7, 3], x[11, 0] = 5000.0, -800.0
        if kind == "offset":
            x, y = x + 1000.0, y + 1000.0
    elif kind == "gauss":
        x, y = rng.standard_normal((M, D)), rng.standard_normal((N, D))
    elif kind == "heavy":
        x, y = rng.standard_t(2, (M, D)), rng.standard_t(2, (N, D))
    elif kind == "ties":
        y = rng.integers(0, 4, (N, D)).astype(np.float64)           # many equal distances: the index decides
        x = y[rng.integers(0, N, M)] + (rng.random((M, D)) < 0.02)
    else:
        c = 3 * rng.standard_normal((20, D))
        x = c[rng.integers(0, 20, M)] + 0.1 * rng.standard_normal((M, D))
        y = c[rng.integers(0, 20, N)] + 0.1 * rng.standard_normal((N, D))
    x, y = x.astype(np.float32), y.astype(np.float32)
    vals, idx = _knn(D, K)(*to_dev(x, y))
    module = keops_io.last_loader.module
    assert module.meta("knn_i8") == "1" and module.path_status() == taken
    rows = np.sort(rng.choice(M, 400, replace=False)).astype(np.int64)
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum", rows=rows)
    assert np.array_equal(idx.cpu().numpy().reshape(M, K)[rows], ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy().reshape(M, K)[rows], ref[:, 0::2])


@pytest.mark.parametrize("shape,M,N,D,K,axis", [((40,), 2048, 4096, 3, 8, 1), ((3, 8), 3000, 2500, 40, 10, 1), ((24,), 2500, 3000, 64, 5, 0)])
def test_many_batches_served_as_row_ranges(shape, M, N, D, K, axis):
    """Batches too small to be served one by one: every batch becomes a row range of the block-sparse variant of the
    scheme (queries and references carry every batch dimension), indices relative to the batch as in
    GpuReduc1D_ranges.py:151-158; bit-identical to the oracle run batch by batch."""
    from keops_amd import keops_io

    rng = np.random.default_rng(77 + D)
    x = rng.random(shape + (M, D)).astype(np.float32)
    y = rng.random(shape + (N, D)).astype(np.float32)
    y[..., 5, :] = y[..., 40, :]                                   # ties: the lower index wins
    vals, idx = _knn(D, K, axis=axis)(*to_dev(x, y))
    module = keops_io.last_loader.module
    assert module.meta("scheme") == "knn" and module.meta("ranges") == "1"
    nout, nred = (M, N) if axis == 1 else (N, M)
    assert idx.shape == shape + (nout, K)
    for b in [tuple(0 for _ in shape), tuple(s - 1 for s in shape)]:
        q, r = (x[b], y[b]) if axis == 1 else (y[b], x[b])
        ref = cpu_reduc("sqdist", [q, r], nout, nred, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
        assert np.array_equal(idx[b].cpu().numpy(), ref[:, 1::2].astype(np.int64))
        assert np.array_equal(vals[b].cpu().numpy(), ref[:, 0::2])
    if axis == 1:
        # a broadcast batch dimension cannot be served that way: the general-purpose kernel takes the call
        y1 = y[(0,) * len(shape)]                                   # one reference set for every batch
        _, idx_b = _knn(D, K)(*to_dev(x, y1[(None,) * len(shape)]))
        module = keops_io.last_loader.module
        assert not (module.meta("scheme") == "knn" and module.meta("ranges") == "1")
        b = tuple(s - 1 for s in shape)
        ref = cpu_reduc("sqdist", [x[b], y1], M, N, 1, reduction="ArgKMin", K=K, scheme="direct_sum")
        assert np.array_equal(idx_b[b].cpu().numpy(), ref.astype(np.int64))


@pytest.mark.parametrize("M,N,D,K", [(3000, 70000, 3, 10), (1500, 40000, 2, 4), (2000, 50000, 16, 50), (500, 900, 3, 10),
                                     (1200, 33000, 7, 1)])
def test_knn_low_dimension_split_operands(M, N, D, K):
    """Dense point clouds (D < 32): the filter uses hi + lo bf16 operands; results stay bit-identical
    to the CPU oracle, in the two-phase schedule (N >= 16384, M >= 1024) and in the adaptive one."""
    rng = np.random.default_rng(11)
    x = rng.random((M, D)).astype(np.float32)
    y = rng.random((N, D)).astype(np.float32)
    y[40] = y[5]
    y[N - 1] = y[5]
    x[1] = y[5]
    x[2] = x[2] + 100.0  # an outlier query far from every reference
    vals, idx = _knn(D, K)(*to_dev(x, y))
    from keops_amd import keops_io

    assert any(m.meta("scheme") == "knn" and m.meta("knn_split") == "1" for m in keops_io._modules.values())
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    assert np.array_equal(idx.cpu().numpy().reshape(M, K), ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy().reshape(M, K), ref[:, 0::2])
    if K >= 3:
        assert idx[1, :3].tolist() == [5, 40, N - 1]


def test_knn_low_dimension_clustered_far_from_origin():
    """Tight clusters far from the origin: centring on the global mean leaves large norms compared
    with the neighbour distances; the filter must stay complete (no missed neighbour)."""
    rng = np.random.default_rng(12)
    C, per, D, K = 40, 1000, 3, 8
    centres = 100.0 * rng.random((C, D))
    y = (np.repeat(centres, per, 0) + 0.01 * rng.standard_normal((C * per, D))).astype(np.float32)
    x = (np.repeat(centres, 50, 0) + 0.01 * rng.standard_normal((C * 50, D))).astype(np.float32)
    vals, idx = _knn(D, K)(*to_dev(x, y))
    ref = cpu_reduc("sqdist", [x, y], x.shape[0], y.shape[0], 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    assert np.array_equal(idx.cpu().numpy(), ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy(), ref[:, 0::2])


@pytest.mark.parametrize("D", [64, 3])
def test_knn_two_phase_with_massive_ties(D):
    """Sizes that take the sampled-threshold schedule, on data full of exact ties: integer grid coordinates with
    every reference stored four times (the strict-'<' rule keeps the lower index), and queries that coincide with
    references."""
    M, N, K = 2048, 40000, 10
    rng = np.random.default_rng(61)
    base = rng.integers(0, 4, size=(N // 4, D)).astype(np.float32)
    y = np.concatenate([base, base, base, base], 0)
    x = rng.integers(0, 4, size=(M, D)).astype(np.float32)
    x[:100] = y[:100]
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    vals, idx = _knn(D, K)(*to_dev(x, y))
    assert np.array_equal(idx.cpu().numpy().reshape(M, K), ref[:, 1::2].astype(np.int64))
    assert np.array_equal(vals.cpu().numpy().reshape(M, K), ref[:, 0::2])


def test_knn_two_phase_log_overflow_falls_back():
    """All references identical: every pair passes any threshold, the candidate logs overflow and the adaptive kernel
    that is launched behind the two-phase schedule (idle otherwise; the flag stays on the device) redoes the search;
    the K lowest indices win the ties."""
    M, N, D, K = 1100, 33000, 32, 6
    rng = np.random.default_rng(62)
    x = rng.random((M, D)).astype(np.float32)
    y = np.tile(rng.random((1, D)).astype(np.float32), (N, 1))
    vals, idx = _knn(D, K)(*to_dev(x, y))
    assert np.array_equal(idx.cpu().numpy().reshape(M, K), np.tile(np.arange(K), (M, 1)))
    ref = cpu_reduc("sqdist", [x, y[:K]], M, K, 1, reduction="KMin", K=K, scheme="direct_sum")
    assert np.array_equal(vals.cpu().numpy().reshape(M, K), ref)


def test_batched_knn_one_dense_pass_per_batch(monkeypatch):
    """A few large batches (here: the size limits lowered) run the matrix-core pipeline once per batch, with
    a broadcast batch dimension on the queries; indices are relative to the batch (GpuReduc1D_ranges.py:151-158)
    and must equal a stable argsort of the float32 distances computed in the reference's operation order."""
    from keops_amd import config, keops_io
    from keops_amd.torch import LazyTensor

    import keops_amd.get_keops_dll as engine

    monkeypatch.setattr(config, "knn_batch_min_work", 1)
    engine._cache.clear()
    keops_io._loaders.clear()
    B, M, N, D, K = 3, 700, 1500, 8, 5
    gen = torch.Generator().manual_seed(12)
    x = torch.rand(1, M, D, generator=gen)
    y = torch.rand(B, N, D, generator=gen)
    xd, yd = x.cuda(), y.cuda()
    D_ij = ((LazyTensor(xd[:, :, None, :]) - LazyTensor(yd[:, None, :, :])) ** 2).sum(-1)
    idx = D_ij.argKmin(K, dim=2).cpu()
    used = [ld for key, ld in keops_io._loaders.items() if key[3]]
    assert used and all(ld.module.meta("scheme") == "knn" for ld in used)
    assert idx.shape == (B, M, K)
    for b in range(B):
        d = np.zeros((M, N), np.float32)
        for k in range(D):
            d += (x[0, :, k, None].numpy() - y[b, None, :, k].numpy()) ** 2
        ref = np.argsort(d, axis=1, kind="stable")[:, :K]
        assert np.array_equal(idx[b].numpy(), ref), b
    # values and indices together, reduction over the other axis
    vals, idj = D_ij.Kmin_argKmin(K, dim=1)
    assert vals.shape == (B, N, K) and idj.shape == (B, N, K)
    for b in range(B):
        d = np.zeros((N, M), np.float32)
        for k in range(D):
            d += (x[0, None, :, k].numpy() - y[b, :, None, k].numpy()) ** 2
        ref = np.argsort(d, axis=1, kind="stable")[:, :K]
        assert np.array_equal(idj[b].cpu().numpy(), ref), b
        assert np.array_equal(vals[b].cpu().numpy(), np.take_along_axis(d, ref, 1)), b


@pytest.mark.parametrize("D,K,op", [(16, 5, "KMin_ArgKMin"), (64, 10, "ArgKMin"), (40, 3, "KMin")])
def test_knn_with_block_sparse_ranges_bit_exact(D, K, op):
    """K nearest neighbours restricted by a block-sparse pattern (cluster-to-cluster search): the adaptive matrix-core
    kernel with a range cursor, bit-identical to the oracle's ranges loop; rows that no range covers and rows whose
    ranges hold fewer than K references keep the neutral entries."""
    from keops_amd import keops_io

    rng = np.random.default_rng(D)
    M, N = 5200, 6100
    x = rng.random((M, D)).astype(np.float32)
    y = rng.random((N, D)).astype(np.float32)
    y[4000] = y[4500]          # ties across two ranges of the same row range: lower index first
    # four row ranges (rows 1000..1199 uncovered; the last one sees only 2 references, fewer than K)
    ranges_i = np.array([[0, 1000], [1200, 3000], [3000, 5190], [5190, 5200]], np.int64)
    slices_i = np.array([2, 3, 6, 7], np.int64)
    red_j = np.array([[0, 1500], [4000, 6100], [1500, 4000], [0, 700], [700, 1500], [4200, 5000], [6000, 6002]], np.int64)
    # the other three arrays describe the transposed pattern (not used by a reduction over j)
    ranges_j = np.array([[0, N]], np.int64)
    slices_j = np.array([1], np.int64)
    red_i = np.array([[0, M]], np.int64)
    ranges = tuple(torch.from_numpy(r).cuda() for r in (ranges_i, slices_i, red_j, ranges_j, slices_j, red_i))
    got = _knn(D, K, op)(*to_dev(x, y), ranges=ranges)
    assert keops_io.last_loader.module.meta("scheme") == "knn" and keops_io.last_loader.module.meta("ranges") == "1"
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum",
                    ranges=(ranges_i, slices_i, red_j))
    rv, ri = ref[:, 0::2], ref[:, 1::2].astype(np.int64)
    if op == "KMin_ArgKMin":
        vals, idx = (t.cpu().numpy().reshape(M, K) for t in got)
        assert np.array_equal(idx, ri) and np.array_equal(vals, rv)
    elif op == "ArgKMin":
        assert np.array_equal(got.cpu().numpy().reshape(M, K), ri)
    else:
        assert np.array_equal(got.cpu().numpy().reshape(M, K), rv)
    assert np.isinf(rv[1100]).all() and np.isinf(rv[5195, 2:]).all()      # the cases above are really there
    # second call with the same range tensors: table built on the device, same result
    again = _knn(D, K, op)(*to_dev(x, y), ranges=ranges)
    a0, g0 = (again[0], got[0]) if isinstance(got, tuple) else (again, got)
    assert torch.equal(a0, g0)


def test_small_problem_stays_on_the_general_purpose_kernel(monkeypatch):
    """Below config.knn_min_work the fixed cost of the matrix-core pipeline does not pay: same results from the
    general-purpose kernel."""
    from keops_amd import config, keops_io

    monkeypatch.setattr(config, "knn_min_work", 1 << 32)
    x, y = np.random.default_rng(3).random((2, 900, 64), dtype=np.float32)
    idx = _knn(64, 10, "ArgKMin")(*to_dev(x, y)).cpu().numpy()
    assert not _uses_mfma_module() and len(keops_io._loaders) == 1
    d = np.zeros((900, 900), np.float32)
    for k in range(64):
        d += (x[:, None, k] - y[None, :, k]) ** 2
    assert np.array_equal(idx, np.argsort(d, axis=1, kind="stable")[:, :10])


def _sequential_sqdist(x, y):
    """Float32 squared distances in the reference's operation order (sum of squared differences, component by
    component, no fused multiply-add)."""
    d = np.zeros((x.shape[0], y.shape[0]), np.float32)
    for k in range(x.shape[1]):
        d += (x[:, None, k] - y[None, :, k]) ** 2
    return d


@pytest.mark.parametrize("M,N,D,K,op", [(700, 5000, 300, 10, "ArgKMin"), (300, 3000, 784, 5, "KMin_ArgKMin"),
                                        (100, 2500, 1000, 3, "KMin"), (50, 7, 400, 10, "KMin_ArgKMin")])
def test_knn_beyond_256_components_chunked_sweep_and_exact_rerank(M, N, D, K, op):
    """More than 256 components: the chunked matrix-core sweep keeps K + 6 approximate candidates, the re-rank
    kernel orders them by exact float32 distance and certifies that nothing was left out: bit-exact indices and
    values against a stable argsort of the reference-order distances (N < K: the tail stays (inf, 0))."""
    from keops_amd import keops_io

    rng = np.random.default_rng(D + K)
    x, y = rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)
    out = _knn(D, K, op)(*to_dev(x, y))
    (ld,) = keops_io._loaders.values()
    assert ld.module.meta("scheme") == "chunk" and ld.module.meta("chk_knn") == str(K) and ld._exact is None
    d = _sequential_sqdist(x, y)
    order = np.argsort(d, axis=1, kind="stable")[:, :K]
    vals = np.take_along_axis(d, order, 1)
    if N < K:
        order = np.concatenate([order, np.zeros((M, K - N), order.dtype)], 1)
        vals = np.concatenate([vals, np.full((M, K - N), np.inf, np.float32)], 1)
    if op == "ArgKMin":
        assert np.array_equal(out.cpu().numpy().astype(np.int64), order)
    elif op == "KMin":
        assert np.array_equal(out.cpu().numpy(), vals)
    else:
        assert np.array_equal(out[0].cpu().numpy(), vals) and np.array_equal(out[1].cpu().numpy().astype(np.int64), order)


def test_knn_beyond_256_components_ties_fall_back_to_the_exact_kernel():
    """Every reference row appears 20 times: the K-th distance is tied with rows outside any list of K + 6
    candidates, the launch reports that it cannot certify its result and the call is redone on the exact kernel
    (lowest index first among equal distances)."""
    from keops_amd import keops_io

    M, D, K = 200, 320, 10
    rng = np.random.default_rng(1)
    x = rng.random((M, D), dtype=np.float32)
    y = np.tile(rng.random((60, D), dtype=np.float32), (20, 1))
    idx = _knn(D, K, "ArgKMin")(*to_dev(x, y)).cpu().numpy()
    (ld,) = keops_io._loaders.values()
    assert ld.module.meta("chk_knn") == str(K) and ld._exact is not None
    assert ld._exact.module.meta("scheme") == "conv" and ld._exact.module.meta("vchunk") == str(D)
    assert np.array_equal(idx.astype(np.int64), np.argsort(_sequential_sqdist(x, y), axis=1, kind="stable")[:, :K])


@pytest.mark.parametrize("D,scheme", [(64, "knn"), (400, "chunk")])
def test_min_family_of_sqdist_runs_as_k_equal_one(D, scheme):
    """Min, ArgMin and Min_ArgMin of SqDist share the K-min schemes with K = 1 (same layout, first index wins):
    bit-exact against the reference-order distances, duplicated references included."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N = 600, 4000
    rng = np.random.default_rng(D)
    x, y = rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)
    if scheme == "knn":
        y[N // 2:] = y[:N // 2]          # exact ties: the lower index must win
    d = _sequential_sqdist(x, y)
    ref_i, ref_v = d.argmin(1), d.min(1)
    for op in ("ArgMin", "Min", "Min_ArgMin"):
        keops_io._loaders.clear()
        out = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op=op, axis=1)(*to_dev(x, y))
        (ld,) = keops_io._loaders.values()
        assert ld.module.meta("scheme") == scheme, op
        if op == "ArgMin":
            assert np.array_equal(out.cpu().numpy()[:, 0].astype(np.int64), ref_i)
        elif op == "Min":
            assert np.array_equal(out.cpu().numpy()[:, 0], ref_v)
        else:
            assert np.array_equal(out[0].cpu().numpy()[:, 0], ref_v)
            assert np.array_equal(out[1].cpu().numpy()[:, 0].astype(np.int64), ref_i)


def test_nearest_row_over_the_first_index_beyond_256_components():
    """ArgMin over i (axis=0) at D = 300: the K = 1 member of the family on the chunked sweep with exact re-rank."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, D = 1500, 400, 300
    rng = np.random.default_rng(5)
    x, y = rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)
    out = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="ArgMin", axis=0)(*to_dev(x, y))
    (ld,) = keops_io._loaders.values()
    assert ld.module.meta("chk_knn") == "1"
    assert np.array_equal(out.cpu().numpy()[:, 0].astype(np.int64), _sequential_sqdist(y, x).argmin(1))
