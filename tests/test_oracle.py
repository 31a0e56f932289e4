"""Pins the CPU oracle (oracle/cpu_reduc.c) without the reference: float64 closed forms, scipy
log-sum-exp, numpy stable argsort, brute force on tiny inputs and invariants, chosen so that a
dropped term, a wrong sign or index, or a transposed operand fails at least one check."""
import numpy as np
import pytest
from scipy.special import logsumexp

from oracle.cpu_oracle import cpu_reduc


def _data(M, N, D, Dv, seed=0, dtype=np.float32):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, D)).astype(dtype)
    y = rng.standard_normal((N, D)).astype(dtype)
    b = rng.standard_normal((N, Dv)).astype(dtype)
    return x, y, b


def _d2(x, y):
    x, y = x.astype(np.float64), y.astype(np.float64)
    return ((x[:, None, :] - y[None, :, :]) ** 2).sum(-1)


@pytest.mark.parametrize("Dv", [1, 8])
@pytest.mark.parametrize("scheme", ["direct_sum", "block_sum", "kahan_scheme"])
def test_gauss_closed_form(Dv, scheme):
    M, N = 300, 517
    x, y, b = _data(M, N, 3, Dv)
    g = np.array([0.7], np.float32)
    got = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, scheme=scheme)
    ref = np.exp(-0.7 * _d2(x, y)) @ b.astype(np.float64)
    assert got.shape == (M, Dv)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-6


def test_gauss_special_cases():
    # single coincident point with unit weight -> 1; far-apart points -> 0
    one = np.ones((1, 1), np.float32)
    p = np.array([[0.3, -1.0, 2.0]], np.float32)
    g = np.array([2.0], np.float32)
    assert cpu_reduc("gauss", [p, p, one, g], 1, 1, 1)[0, 0] == 1.0
    far = p + 100.0
    assert cpu_reduc("gauss", [p, far, one, g], 1, 1, 1)[0, 0] == 0.0
    # non-symmetric arguments: a transposed (x,y) would change the answer of an i-indexed output
    x, y, b = _data(5, 7, 3, 1, seed=3)
    got = cpu_reduc("gauss", [x, y, b, g], 5, 7, 1)
    brute = np.zeros((5, 1))
    for i in range(5):
        for j in range(7):
            brute[i, 0] += np.exp(-2.0 * np.sum((x[i].astype(np.float64) - y[j]) ** 2)) * b[j, 0]
    assert np.allclose(got, brute, rtol=1e-5, atol=1e-7)


def test_gauss_linearity_and_permutation():
    M, N = 64, 200
    x, y, b = _data(M, N, 3, 2, seed=1)
    g = np.array([1.0], np.float32)
    a1 = cpu_reduc("gauss", [x, y, b, g], M, N, 2)
    a2 = cpu_reduc("gauss", [x, y, 3 * b, g], M, N, 2)
    assert np.allclose(a2, 3 * a1, rtol=1e-5, atol=1e-6)
    perm = np.random.default_rng(5).permutation(N)
    a3 = cpu_reduc("gauss", [x, y[perm], b[perm], g], M, N, 2)
    assert np.allclose(a3, a1, rtol=1e-4, atol=1e-5)


def test_gauss_float64_and_double_acc():
    M, N = 100, 1000
    x, y, b = _data(M, N, 3, 1, dtype=np.float64)
    g = np.array([0.5])
    got = cpu_reduc("gauss", [x, y, b, g], M, N, 1, dtype=np.float64)
    ref = np.exp(-0.5 * _d2(x, y)) @ b
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 1e-13
    x32, y32, b32 = x.astype(np.float32), y.astype(np.float32), b.astype(np.float32)
    a32 = cpu_reduc("gauss", [x32, y32, b32, g.astype(np.float32)], M, N, 1, scheme="direct_sum")
    a64 = cpu_reduc("gauss", [x32, y32, b32, g.astype(np.float32)], M, N, 1, scheme="direct_sum", acc_double=True)
    ref32 = np.exp(-0.5 * _d2(x32, y32)) @ b32.astype(np.float64)
    assert np.abs(a64 - ref32).max() <= np.abs(a32 - ref32).max() + 1e-7


def test_gauss_gradx_vs_finite_differences_and_closed_form():
    M, N, Dv = 20, 50, 2
    x, y, b = _data(M, N, 3, Dv, seed=2, dtype=np.float64)
    g = np.array([0.8])
    G = np.random.default_rng(9).standard_normal((M, Dv))
    got = cpu_reduc("gauss_gradx", [x, y, b, g, G], M, N, 3, dtype=np.float64)
    K = np.exp(-0.8 * _d2(x, y))
    w = (G @ b.T) * K  # (M,N)
    ref = -2 * 0.8 * (w[:, :, None] * (x[:, None, :] - y[None, :, :])).sum(1)
    assert np.allclose(got, ref, rtol=1e-10, atol=1e-12)

    def loss(xx):
        return np.sum(G * (np.exp(-0.8 * _d2(xx, y)) @ b))

    eps = 1e-6
    for (i, k) in [(0, 0), (3, 2), (19, 1)]:
        xp, xm = x.copy(), x.copy()
        xp[i, k] += eps
        xm[i, k] -= eps
        fd = (loss(xp) - loss(xm)) / (2 * eps)
        assert abs(fd - got[i, k]) < 1e-6 * max(1, abs(fd))


def test_block_sum_period_matches_plain_sum():
    # block_sum only re-associates: result equals the direct sum within O(sqrt(N) eps)
    M, N = 16, 10007
    x, y, b = _data(M, N, 3, 1, seed=4)
    g = np.array([0.1], np.float32)
    a_dir = cpu_reduc("gauss", [x, y, b, g], M, N, 1, scheme="direct_sum")
    a_blk = cpu_reduc("gauss", [x, y, b, g], M, N, 1, scheme="block_sum")
    ref = np.exp(-0.1 * _d2(x, y)) @ b.astype(np.float64)
    assert np.abs(a_blk - ref).max() < 5e-4 and np.abs(a_dir - ref).max() < 5e-3
    # dense-table entry: block_sum over an all-ones table of N columns gives exactly N
    F = np.ones((3, 1000, 1), np.float32)
    assert np.all(cpu_reduc("dense", [F], 3, 1000, 1, scheme="block_sum") == 1000.0)


def test_lse_vs_scipy_and_shift_invariance():
    M, N = 50, 400
    rng = np.random.default_rng(7)
    x, y, _ = _data(M, N, 3, 1, seed=7)
    l = rng.standard_normal((N, 1)).astype(np.float32)
    e = np.array([1 / 0.05], np.float32)
    ms = cpu_reduc("lse_gauss", [x, y, l, e], M, N, 2, reduction="Max_SumShiftExp")
    got = ms[:, 0] + np.log(ms[:, 1])
    f = l.astype(np.float64).T - _d2(x, y) * float(e[0])
    ref = logsumexp(f, axis=1)
    assert np.allclose(got, ref, rtol=2e-6, atol=2e-5)
    assert np.allclose(ms[:, 0], f.max(1), rtol=1e-5, atol=1e-4)  # m really is the running max
    ms2 = cpu_reduc("lse_gauss", [x, y, l + 3.0, e], M, N, 2, reduction="Max_SumShiftExp")
    assert np.allclose(ms2[:, 0] + np.log(ms2[:, 1]), got + 3.0, rtol=1e-5, atol=1e-4)
    # single column: LSE(f) = f
    ms1 = cpu_reduc("lse_gauss", [x, y[:1], l[:1], e], M, 1, 2, reduction="Max_SumShiftExp")
    assert np.allclose(ms1[:, 0] + np.log(ms1[:, 1]), f[:, 0], rtol=1e-5, atol=1e-4)


def test_lse_weighted_dense_table():
    # Max_SumShiftExpWeight on a dense table [f, g1, g2]: sum_j exp(f - m) g
    rng = np.random.default_rng(11)
    M, N = 6, 33
    f = rng.standard_normal((M, N)) * 5
    gw = rng.standard_normal((M, N, 2))
    F = np.concatenate([f[..., None], gw], -1).astype(np.float64)
    for scheme in ("direct_sum", "block_sum", "kahan_scheme"):
        out = cpu_reduc("dense", [F], M, N, 3, reduction="Max_SumShiftExpWeight", scheme=scheme, dtype=np.float64)
        m = f.max(1)
        s = (np.exp(f - m[:, None])[..., None] * gw).sum(1)
        assert np.allclose(out[:, 0], m)
        assert np.allclose(out[:, 1:], s, rtol=1e-12, atol=1e-12)


def test_kmin_vs_stable_argsort_and_ties():
    M, N, D, K = 40, 300, 8, 5
    rng = np.random.default_rng(2)
    x = rng.random((M, D)).astype(np.float32)
    y = rng.random((N, D)).astype(np.float32)
    y[17] = y[3]  # duplicated reference rows: ties must keep the lower index first
    y[250] = y[3]
    x[0] = y[3]
    # distances in the reference's fp32 order: sequential sum of squared differences
    d = np.zeros((M, N), np.float32)
    for k in range(D):
        t = x[:, None, k] - y[None, :, k]
        d = d + t * t
    order = np.argsort(d, axis=1, kind="stable")[:, :K]
    out = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    vals, idx = out[:, 0::2], out[:, 1::2].astype(np.int64)
    assert np.array_equal(idx, order)
    assert np.array_equal(vals, np.take_along_axis(d, order, 1))
    assert list(idx[0, :3]) == [3, 17, 250]
    assert np.array_equal(cpu_reduc("sqdist", [x, y], M, N, 1, reduction="ArgKMin", K=K, scheme="direct_sum").astype(np.int64), order)
    assert np.array_equal(cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin", K=K, scheme="direct_sum"), vals)


def test_kmin_vector_valued_dense():
    rng = np.random.default_rng(3)
    M, N, fd, K = 4, 20, 3, 2
    F = rng.standard_normal((M, N, fd)).astype(np.float32)
    out = cpu_reduc("dense", [F], M, N, fd, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    out = out.reshape(M, K, 2, fd)
    order = np.argsort(F, axis=1, kind="stable")[:, :K, :]
    assert np.array_equal(out[:, :, 1, :].astype(np.int64), order)
    assert np.array_equal(out[:, :, 0, :], np.take_along_axis(F, order, 1))


def test_min_max_argmin_argmax():
    rng = np.random.default_rng(4)
    M, N, fd = 5, 40, 2
    F = rng.integers(0, 6, size=(M, N, fd)).astype(np.float32)  # many ties
    mn = cpu_reduc("dense", [F], M, N, fd, reduction="Min_ArgMin", scheme="direct_sum")
    assert np.array_equal(mn[:, :fd], F.min(1)) and np.array_equal(mn[:, fd:].astype(int), F.argmin(1))
    mx = cpu_reduc("dense", [F], M, N, fd, reduction="Max_ArgMax", scheme="direct_sum")
    assert np.array_equal(mx[:, :fd], F.max(1)) and np.array_equal(mx[:, fd:].astype(int), F.argmax(1))
    assert np.array_equal(cpu_reduc("dense", [F], M, N, fd, reduction="ArgMin", scheme="direct_sum").astype(int), F.argmin(1))
    assert np.array_equal(cpu_reduc("dense", [F], M, N, fd, reduction="Max", scheme="direct_sum"), F.max(1))


def test_laplace_closed_form():
    M, N, D, Dv = 30, 60, 16, 4
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((M, D)) / np.sqrt(D)).astype(np.float32)
    y = (rng.standard_normal((N, D)) / np.sqrt(D)).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    got = cpu_reduc("laplace", [x, y, b], M, N, Dv)
    ref = np.exp(-np.sqrt(_d2(x, y))) @ b.astype(np.float64)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-6


def test_ranges_vs_masked_dense_and_uncovered_rows():
    # block-sparse: equals the dense result with a mask keep[label_i, label_j]
    M, N = 60, 80
    x, y, b = _data(M, N, 3, 1, seed=6)
    g = np.array([0.5], np.float32)
    ranges_x = np.array([[0, 10], [10, 35], [40, 60]], np.int64)  # rows 35..39 uncovered
    ranges_ycl = np.array([[0, 20], [20, 50], [50, 80]], np.int64)
    keep = np.array([[1, 0, 1], [0, 1, 1], [1, 1, 0]], bool)
    red, slices = [], []
    for k in range(3):
        for l in range(3):
            if keep[k, l]:
                red.append(ranges_ycl[l])
        slices.append(len(red))
    got = cpu_reduc("gauss", [x, y, b, g], M, N, 1, ranges=(ranges_x, np.array(slices), np.array(red)))
    Kmat = np.exp(-0.5 * _d2(x, y))
    mask = np.zeros((M, N), bool)
    for k in range(3):
        for l in range(3):
            if keep[k, l]:
                mask[ranges_x[k, 0]:ranges_x[k, 1], ranges_ycl[l, 0]:ranges_ycl[l, 1]] = True
    ref = (Kmat * mask) @ b.astype(np.float64)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-6)
    assert np.all(got[35:40] == 0.0)
    # Arg reductions report global column indices in ranges mode; uncovered rows get (inf, 0)
    out = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="Min_ArgMin", scheme="direct_sum",
                    ranges=(ranges_x, np.array(slices), np.array(red)))
    d = np.where(mask, _d2(x, y), np.inf)
    assert np.array_equal(out[:35, 1].astype(int), d[:35].argmin(1))
    assert np.all(np.isinf(out[35:40, 0])) and np.all(out[35:40, 1] == 0)


def test_row_subset_is_exact():
    M, N = 200, 300
    x, y, b = _data(M, N, 3, 1, seed=8)
    g = np.array([1.0], np.float32)
    full = cpu_reduc("gauss", [x, y, b, g], M, N, 1)
    rows = np.array([5, 17, 199, 0], np.int64)
    assert np.array_equal(cpu_reduc("gauss", [x, y, b, g], M, N, 1, rows=rows), full[rows])


def test_kahan_and_double_accumulation_on_an_ill_conditioned_sum():
    # 10^6 terms of 0.1f: the plain float32 running sum drifts by about 1 %, the compensated sum
    # and the float64 accumulator must not (a Kahan update with a wrong sign or a dropped compensation fails)
    N = 1_000_000
    F = np.full((1, N, 1), 0.1, np.float32)
    exact = float(np.float32(0.1)) * N  # every term is the same float32 value
    direct = float(cpu_reduc("dense", [F], 1, N, 1, scheme="direct_sum")[0, 0])
    kahan = float(cpu_reduc("dense", [F], 1, N, 1, scheme="kahan_scheme")[0, 0])
    dacc = cpu_reduc("dense", [F], 1, N, 1, scheme="direct_sum", acc_double=True)[0, 0]
    assert abs(direct - exact) / exact > 1e-4
    assert abs(kahan - exact) / exact < 1e-7
    # float64 accumulation of float32 terms, rounded once at the end
    assert dacc == np.float32(np.sum(F.astype(np.float64)))
    # block_sum with a float64 accumulator: float32 partial sums of sqrt(N) = 1000 terms, folded in float64
    blocks = np.float32(0.0)
    part = np.float32(0.0)
    for _ in range(1000):
        part = np.float32(part + np.float32(0.1))
    want = np.float32(np.float64(part) * 1000)
    assert cpu_reduc("dense", [F], 1, N, 1, scheme="block_sum", acc_double=True)[0, 0] == want
    del blocks
    # compensated log-sum-exp weights (Max_SumShiftExpWeight, kahan_scheme): f = 0 everywhere, weights 0.1f
    FW = np.concatenate([np.zeros((1, N, 1), np.float32), F], -1)
    ms_d = cpu_reduc("dense", [FW], 1, N, 2, reduction="Max_SumShiftExpWeight", scheme="direct_sum")[0]
    ms_k = cpu_reduc("dense", [FW], 1, N, 2, reduction="Max_SumShiftExpWeight", scheme="kahan_scheme")[0]
    assert ms_k[0] == 0 and abs(float(ms_k[1]) - exact) / exact < 1e-7 and abs(float(ms_d[1]) - exact) / exact > 1e-4


def test_l1_bodies_closed_form_and_order():
    M, N, D, Dv = 23, 41, 37, 2
    rng = np.random.default_rng(12)
    x = rng.standard_normal((M, D)).astype(np.float32)
    y = rng.standard_normal((N, D)).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    d1 = np.abs(x.astype(np.float64)[:, None, :] - y.astype(np.float64)[None, :, :]).sum(-1)
    got = cpu_reduc("l1dist", [x, y], M, N, 1, reduction="Min", scheme="direct_sum")
    assert np.allclose(got[:, 0], d1.min(1), rtol=1e-5)
    # sequential float32 sum in component order, bit for bit
    seq = np.zeros((M, N), np.float32)
    for k in range(D):
        seq = seq + np.abs(x[:, None, k] - y[None, :, k])
    assert np.array_equal(got[:, 0], seq.min(1))
    ker = cpu_reduc("exp_l1", [x / 8, y / 8, b], M, N, Dv)
    ref = np.exp(-d1 / 8) @ b.astype(np.float64)
    assert np.linalg.norm(ker - ref) / np.linalg.norm(ref) < 2e-6
    # transposed operands or a squared difference would change the answer
    assert not np.allclose(ker, np.exp(-(d1 / 8) ** 2) @ b.astype(np.float64), rtol=1e-3)


def test_scalprod_body_uses_a_fused_multiply_add_chain():
    M, N, D, Dv = 9, 31, 50, 3
    rng = np.random.default_rng(13)
    x = rng.standard_normal((M, D)).astype(np.float32)
    y = rng.standard_normal((N, D)).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    got = cpu_reduc("scalprod", [x, y, b], M, N, Dv)
    ref = (x.astype(np.float64) @ y.astype(np.float64).T) @ b.astype(np.float64)
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 2e-6
    # one pair, two components [1, a].[-rn(a*a), a]: the chain fma(a, a, fma(1, -r, 0)) returns the exact
    # residual a*a - rn(a*a); separate multiply and add would return 0, the reverse order too
    a = np.float32(1.0 + 2.0 ** -12 + 2.0 ** -20)
    r = np.float32(a * a)
    resid = float(np.float64(a) * np.float64(a) - np.float64(r))
    assert resid != 0.0
    xx = np.array([[1.0, a]], np.float32)
    yy = np.array([[-r, a]], np.float32)
    one = np.ones((1, 1), np.float32)
    assert float(cpu_reduc("scalprod", [xx, yy, one], 1, 1, 1)[0, 0]) == np.float32(resid)
    # float64 twin
    x64, y64, b64 = x.astype(np.float64), y.astype(np.float64), b.astype(np.float64)
    got64 = cpu_reduc("scalprod", [x64, y64, b64], M, N, Dv, dtype=np.float64)
    assert np.allclose(got64, ref, rtol=1e-13, atol=1e-13)
