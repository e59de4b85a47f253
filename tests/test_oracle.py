"""Pins the CPU oracle against things that do not depend on it: brute force in
numpy, closed forms, dense linear algebra, numpy's FFT, scikit-learn's
bisection, and the committed golden fixtures.  Each check is chosen so that a
plausible slip in the restatement (a dropped term, a wrong sign or index, a
transposed grid axis) fails it.  CPU only.
"""
import json
import os

import numpy as np
import pytest

import oracle
from tsnecuda import synthetic

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


@pytest.fixture(scope="module")
def small():
    n, d, k = 600, 12, 20
    X = synthetic.gaussian_clusters(n, d=d, clusters=3, center_scale=3.0, seed=11)
    idx, d2 = oracle.knn(X, k)
    dn, dmax = oracle.max_normalize(d2)
    p, beta, iters = oracle.perplexity(dn, 6.0, 1e-4, return_search=True)
    P = oracle.symmetrize(p, idx)
    rng = np.random.default_rng(5)
    y = (rng.standard_normal(2 * n) * 3.0).astype(np.float32)
    return dict(X=X, k=k, idx=idx, d2=d2, dn=dn, dmax=dmax, p=p, beta=beta, iters=iters, P=P, y=y, n=n)


# ----------------------------------------------------------------- kNN ------
def fp32_fma_distances(X, i):
    """Canonical distance of row i to all rows: fp32 accumulate, one fused
    multiply-add per dimension, emulated in extended precision (the product of
    two fp32 numbers and the sum with an fp32 accumulator are formed there and
    rounded to fp32 once)."""
    acc = np.zeros(X.shape[0], np.float32)
    for d in range(X.shape[1]):
        diff = (X[i, d] - X[:, d]).astype(np.float32)
        acc = (diff.astype(np.longdouble) * diff.astype(np.longdouble) + acc.astype(np.longdouble)).astype(np.float32)
    return acc


def test_knn_matches_brute_force(small):
    X, k, idx, d2 = small["X"], small["k"], small["idx"], small["d2"]
    for i in (0, 1, 299, 599):
        dist = fp32_fma_distances(X, i)
        cand = np.array([j for j in range(X.shape[0]) if j != i])
        order = cand[np.lexsort((cand, dist[cand]))][: k - 1]
        assert idx[i, 0] == i and d2[i, 0] == 0.0
        assert np.array_equal(idx[i, 1:], order)
        assert np.array_equal(d2[i, 1:], dist[order])
    assert np.all(np.diff(d2[:, 1:], axis=1) >= 0)


def test_knn_matches_sklearn(small):
    from sklearn.neighbors import NearestNeighbors
    X, k, idx = small["X"], small["k"], small["idx"]
    nn = NearestNeighbors(n_neighbors=k, algorithm="brute").fit(X.astype(np.float64))
    ref = nn.kneighbors(X.astype(np.float64), return_distance=False)
    same = [set(a) == set(b) for a, b in zip(ref, idx)]
    assert np.mean(same) >= 0.99  # ties / last-place swaps at fp32 resolution only


def test_knn_ties_and_duplicates():
    # Duplicated points: ties broken by lower index, self still first.
    X = np.zeros((6, 3), np.float32)
    X[3:] = 1.0
    idx, d2 = oracle.knn(X, 4)
    assert np.array_equal(idx[1], [1, 0, 2, 3])
    assert np.array_equal(idx[4], [4, 3, 5, 0])
    assert np.array_equal(d2[4], [0, 0, 0, 3])
    # K larger than N is clamped; rows subset agrees with the full call.
    sub_idx, sub_d2 = oracle.knn(X, 4, rows=(2, 5))
    assert np.array_equal(sub_idx, idx[2:5]) and np.array_equal(sub_d2, d2[2:5])


def test_knn_ivf_rule_and_limits():
    """The approximate search's restatement: with every list probed it is the exact search; with few lists
    probed its candidate rule is what a numpy restatement of the rule gives; recall grows with nprobe."""
    rng = np.random.default_rng(5)
    n, d, k, nlist = 1500, 6, 12, 24
    X = synthetic.gaussian_clusters(n, d=d, clusters=5, center_scale=3.0, seed=11)
    cen = X[rng.choice(n, nlist, replace=False)].copy()
    exact_idx, exact_d = oracle.knn(X, k)
    idx_all, d_all = oracle.knn_ivf(X, k, cen, nlist)
    # ties aside (none in this data), probing everything is the exact search
    assert np.array_equal(idx_all, exact_idx) and np.array_equal(d_all, exact_d)
    recalls = []
    for nprobe in (1, 3, 8):
        idx, d2, list_of, probes = oracle.knn_ivf(X, k, cen, nprobe, return_probes=True)
        # a point's list: its nearest centroid; a list's probes: the centroids nearest to its own (itself
        # first) - numpy, float64, away from ties
        dc = ((X[:, None, :].astype(np.float64) - cen[None].astype(np.float64)) ** 2).sum(-1)
        assert np.array_equal(list_of, dc.argmin(1))
        cc = ((cen[:, None, :].astype(np.float64) - cen[None].astype(np.float64)) ** 2).sum(-1)
        assert np.array_equal(probes[:, 0], np.arange(nlist))
        assert np.array_equal(np.sort(probes, 1), np.sort(np.argsort(cc, 1)[:, :nprobe], 1))
        # the candidate rule, restated: renumber by (list, old number), 128-point tiles, a query's candidates
        order = np.lexsort((np.arange(n), list_of))
        lists_sorted = list_of[order]
        T = (n + 127) // 128
        for r in rng.choice(n, 40, replace=False):  # r: a new number
            qt = r // 128
            mates = order[qt * 128:min(n, qt * 128 + 128)]
            probed = np.unique(probes[list_of[mates]])
            tiles = set(range(max(0, qt - 8), min(T - 1, qt + 8) + 1))
            for l in probed:
                members = np.flatnonzero(lists_sorted == l)
                if members.size:
                    tiles.update(range(members[0] // 128, members[-1] // 128 + 1))
            cand = np.array([c for c in range(n) if c // 128 in tiles and c != r])
            dd = ((X[order[r]].astype(np.float64) - X[order[cand]].astype(np.float64)) ** 2).sum(1)
            best = cand[np.lexsort((cand, dd))[:k - 1]]
            assert np.array_equal(idx[order[r], 1:], order[best])
            assert idx[order[r], 0] == order[r] and d2[order[r], 0] == 0.0
        hits = sum(len(np.intersect1d(idx[i, 1:], exact_idx[i, 1:])) for i in range(n))
        recalls.append(hits / (n * (k - 1)))
    assert recalls[0] <= recalls[1] <= recalls[2] and recalls[2] > 0.9


def test_max_normalize(small):
    dn, dmax, d2 = small["dn"], small["dmax"], small["d2"]
    assert dmax == d2.max()
    assert np.array_equal(dn, (d2 / np.float32(dmax)).astype(np.float32))
    assert dn.max() == 1.0


# ---------------------------------------------------------- perplexity ------
def test_perplexity_invariants(small):
    p, dn = small["p"], small["dn"]
    assert np.all(p[:, 0] == 0.0)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, atol=2e-6)
    q = p[:, 1:].astype(np.float64)
    H = -(q * np.log(q)).sum(axis=1)
    assert np.abs(H - np.log(6.0)).max() < 1e-4 + 5e-6
    # ascending distances -> non-increasing probabilities
    assert np.all(np.diff(p[:, 1:], axis=1) <= 0)
    # p_s proportional to exp(-beta d_s) with the reported beta
    beta = small["beta"].astype(np.float64)[:, None]
    e = np.exp(-beta * dn[:, 1:].astype(np.float64))
    np.testing.assert_allclose(q, e / e.sum(axis=1, keepdims=True), rtol=2e-5)


def test_perplexity_uniform_closed_form():
    # Equal distances: every beta gives the uniform distribution, whose entropy
    # is ln(K-1); asking for exactly that perplexity converges at once.
    K = 9
    d = np.full((4, K), 0.5, np.float32)
    d[:, 0] = 0.0
    p, beta, iters = oracle.perplexity(d, float(K - 1), 1e-4, return_search=True)
    np.testing.assert_allclose(p[:, 1:], 1.0 / (K - 1), rtol=1e-6)
    assert np.all(iters == 1) and np.all(beta == 1.0)


def test_perplexity_bisection_path():
    # Two neighbours at distances 0 and d: entropy is a known function of beta,
    # H(beta) = ln(1+e^{-beta d}) + beta d e^{-beta d}/(1+e^{-beta d}); follow the
    # doubling / halving / bisection rule by hand.
    d = np.array([[0.0, 0.0, 1.0]], np.float32)  # self, a neighbour at 0, one at 1
    target, eps = 1.5, 1e-4
    p, beta, iters = oracle.perplexity(d, target, eps, return_search=True)

    def H(b):
        e = np.exp(-b)
        return np.log(1 + e) + b * e / (1 + e)
    b, lo, hi, n = 1.0, None, None, 0
    while True:
        n += 1
        diff = H(b) - np.log(target)
        if abs(diff) < eps or n >= 200:
            break
        if diff > 0:
            lo = b
            b = b * 2 if hi is None else (b + hi) / 2
        else:
            hi = b
            b = b / 2 if lo is None else (b + lo) / 2
    assert iters[0] == n
    assert abs(beta[0] - b) <= 1e-6 * b
    assert p[0, 0] == 0.0
    np.testing.assert_allclose(p[0, 1:], np.array([1, np.exp(-b)]) / (1 + np.exp(-b)), rtol=1e-5)


def test_perplexity_against_sklearn(small):
    from sklearn.manifold import _utils
    d2 = small["d2"][:, 1:].astype(np.float32)  # sklearn: neighbours without self, unnormalised distances
    ref = _utils._binary_search_perplexity(np.ascontiguousarray(d2), 6.0, 0)
    ours = oracle.perplexity(small["d2"], 6.0, 1e-5)[:, 1:]
    np.testing.assert_allclose(ours, ref, rtol=2e-3, atol=1e-7)


def _ulp_error(got, exact):
    """|got - exact| in units of the last place of the fp32 result nearest to `exact`."""
    exact = np.asarray(exact, np.float64)
    ref = exact.astype(np.float32)
    spacing = np.spacing(np.abs(ref)).astype(np.float64)
    spacing = np.maximum(spacing, 2.0 ** -149)
    return np.abs(got.astype(np.float64) - exact) / spacing


def test_search_exp_against_double_precision():
    # The search's exp is a hand-written operation sequence; what pins it is the double-precision
    # exponential (numpy / libm), over its whole range including results that are subnormal.
    rng = np.random.default_rng(0)
    x = np.concatenate([np.linspace(-103.9, 0.0, 200001), -np.abs(rng.standard_cauchy(100000)),
                        np.linspace(0.0, 88.7, 20001), -rng.random(50000) * 1e-3]).astype(np.float32)
    x = x[x > -104.0]
    got = oracle.expf(x)
    err = _ulp_error(got, np.exp(x.astype(np.float64)))
    assert err.max() <= 2.0, err.max()
    assert np.mean(err <= 1.0) > 0.99
    assert np.all(np.diff(oracle.expf(np.sort(x))) >= 0)  # monotone
    edge = oracle.expf(np.array([0.0, -np.inf, -200.0, np.inf, 100.0], np.float32))
    assert edge[0] == 1.0 and edge[1] == 0.0 and edge[2] == 0.0 and np.isinf(edge[3]) and np.isinf(edge[4])
    assert np.isnan(oracle.expf(np.array([np.nan], np.float32))[0])


def test_search_log_against_double_precision():
    rng = np.random.default_rng(1)
    v = np.concatenate([np.exp(rng.uniform(-103.0, 88.0, 300000)), np.linspace(0.5, 2.0, 100001),
                        1.0 + rng.standard_normal(50000) * 1e-4, rng.uniform(0.0, 100.0, 50000)]).astype(np.float32)
    v = v[v > 0]
    got = oracle.logf(v)
    exact = np.log(v.astype(np.float64))
    err = _ulp_error(got, exact)
    # Next to 1 the result is tiny and its last place with it: bound the absolute error there.
    near_one = np.abs(v - 1.0) < 0.05
    assert err[~near_one].max() <= 2.0, err[~near_one].max()
    assert np.abs(got[near_one] - exact[near_one]).max() <= 2.0 ** -25
    edge = oracle.logf(np.array([1.0, 0.0, np.inf, -1.0, 1e-45], np.float32))
    assert edge[0] == 0.0 and edge[1] == -np.inf and edge[2] == np.inf and np.isnan(edge[3])
    assert abs(edge[4] - np.log(float(np.float32(1e-45)))) < 1e-4


def test_search_row_sum_order():
    import math
    rng = np.random.default_rng(2)
    for k in (1, 3, 63, 64, 65, 90, 128, 129, 1100):
        v = rng.random(k).astype(np.float32)
        exact = math.fsum(float(t) for t in v)
        assert abs(oracle.row_sum(v) - exact) <= 8 * np.spacing(np.float32(exact))
    # Integer-valued floats: every order gives the exact sum.
    v = rng.integers(0, 1000, 500).astype(np.float32)
    assert oracle.row_sum(v) == float(v.astype(np.float64).sum())
    # The order itself, followed by hand on a case where it shows: slots 0 and 64 share partial 0 and cancel
    # there before anything else is added; a sequential sum would have absorbed the 1 at slot 1 into 2^30.
    v = np.zeros(70, np.float32)
    v[0], v[64], v[1] = 2.0 ** 30, -2.0 ** 30, 1.0
    assert oracle.row_sum(v) == 1.0
    assert float(np.add.accumulate(np.array([2.0 ** 30, 1.0, -2.0 ** 30], np.float32))[-1]) == 0.0
    # ... and slots 0 and 32 only meet at the top of the tree (m = 32), after slot 1 met slot 33:
    v = np.zeros(70, np.float32)
    v[0], v[32], v[1], v[33] = 2.0 ** 30, -2.0 ** 30, 1.0, 1.0
    assert oracle.row_sum(v) == 2.0
    # ... whereas slots 0 and 1 meet last (m = 1), so a unit at slot 2 is absorbed by slot 0 first (m = 2):
    v = np.zeros(70, np.float32)
    v[0], v[1], v[2] = 2.0 ** 30, -2.0 ** 30, 1.0
    assert oracle.row_sum(v) == 0.0


# ---------------------------------------------------------- symmetrize ------
def test_symmetrize_dense(small):
    n, k, idx, p, P = small["n"], small["k"], small["idx"], small["p"], small["P"]
    A = np.zeros((n, n), np.float64)
    A[np.repeat(np.arange(n), k), idx.ravel()] = p.ravel()
    S = (A + A.T) / (2.0 * n)
    np.testing.assert_allclose(P, S[np.repeat(np.arange(n), k), idx.ravel()].reshape(n, k), rtol=2e-6, atol=1e-12)
    assert np.all(P[:, 0] == 0.0)
    assert P.sum() <= 1.0 + 1e-6  # one-directional pairs lose half their mass


def test_symmetrize_full_against_dense_and_scipy(small):
    import scipy.sparse as sp
    n, k, idx, p = small["n"], small["k"], small["idx"], small["p"]
    row_ptr, col, val = oracle.symmetrize_full(p, idx)
    A = np.zeros((n, n), np.float64)
    A[np.repeat(np.arange(n), k), idx.ravel()] = p.ravel()
    want = (A + A.T) / (2.0 * n)
    got = sp.csr_matrix((val, col, row_ptr), shape=(n, n))
    assert got.has_sorted_indices and np.all(np.diff(row_ptr) >= k)
    dense = got.toarray().astype(np.float64)
    assert np.abs(dense - want).max() <= 1e-7 * want.max()
    # the pattern is the union of A's and A^T's (the explicit zero of the self entry included)
    pattern = np.zeros((n, n), bool)
    pattern[np.repeat(np.arange(n), k), idx.ravel()] = True
    stored = np.zeros((n, n), bool)
    stored[np.repeat(np.arange(n), np.diff(row_ptr)), col] = True
    assert np.array_equal(stored, pattern | pattern.T)
    # nothing is dropped: the mass is 1, where the pattern-restricted form loses the unmirrored entries
    assert abs(val.astype(np.float64).sum() - 1.0) <= 1e-5
    assert small["P"].astype(np.float64).sum() < val.astype(np.float64).sum()
    # ... and scipy's own (A + A^T) / 2N
    As = sp.csr_matrix((p.ravel().astype(np.float64), idx.ravel(), np.arange(0, n * k + 1, k)), shape=(n, n))
    ref = ((As + As.T) / (2.0 * n)).tocsr()
    assert abs(ref - got).max() <= 1e-7 * want.max()
    # forces over the CSR pattern against the dense sum
    rng = np.random.default_rng(3)
    y = (rng.standard_normal(2 * n) * 2.0).astype(np.float32)
    attr = oracle.attractive_csr(row_ptr, col, val, y)
    yx, yy = y[:n].astype(np.float64), y[n:].astype(np.float64)
    dx, dy = yx[:, None] - yx[None, :], yy[:, None] - yy[None, :]
    wgt = want / (1.0 + dx * dx + dy * dy)
    dense_force = np.concatenate([(wgt * dx).sum(1), (wgt * dy).sum(1)])
    assert rel_l2(attr, dense_force) < 1e-5


# ---------------------------------------------------------- attractive ------
def test_attractive_dense(small):
    n, k, idx, P, y = small["n"], small["k"], small["idx"], small["P"], small["y"]
    xs, ys = y[:n].astype(np.float64), y[n:].astype(np.float64)
    A = np.zeros((n, n), np.float64)
    A[np.repeat(np.arange(n), k), idx.ravel()] = P.ravel()
    dx = xs[:, None] - xs[None, :]
    dy = ys[:, None] - ys[None, :]
    W = A / (1.0 + dx * dx + dy * dy)
    want = np.concatenate([(W * dx).sum(1), (W * dy).sum(1)])
    assert rel_l2(oracle.attractive(P, idx, y), want) < 2e-6
    # relabelling the points permutes the forces
    perm = np.random.default_rng(1).permutation(n)
    inv = np.empty(n, np.int64)
    inv[perm] = np.arange(n)
    y2 = np.concatenate([y[:n][perm], y[n:][perm]])
    got2 = oracle.attractive(P[perm], inv[idx[perm]].astype(np.int32), y2)
    got = oracle.attractive(P, idx, y)
    assert np.array_equal(got2, np.concatenate([got[:n][perm], got[n:][perm]]))


# ----------------------------------------------------------- repulsive ------
def exact_repulsive(y):
    n = y.size // 2
    xs, ys = y[:n].astype(np.float64), y[n:].astype(np.float64)
    dx = xs[:, None] - xs[None, :]
    dy = ys[:, None] - ys[None, :]
    q = 1.0 / (1.0 + dx * dx + dy * dy)
    return np.concatenate([(q * q * dx).sum(1), (q * q * dy).sum(1)]), q.sum() - n


def test_repulsive_fft_equals_direct_convolution(small):
    # Reduced grids: the FFT path and the plain O(G^4) node-to-node sums agree.
    for nb in (4, 7):
        rep_f, z_f, w_f, yt_f, phi_f = oracle.repulsive(small["y"], nb=nb, details=True)
        rep_d, z_d, w_d, yt_d, phi_d = oracle.repulsive(small["y"], nb=nb, direct=True, details=True)
        assert np.array_equal(w_f, w_d)
        assert rel_l2(yt_f, yt_d) < 1e-6
        assert rel_l2(rep_f, rep_d) < 1e-5
        assert abs(z_f - z_d) <= 1e-6 * abs(z_d)


def test_repulsive_grid_against_numpy_fft(small):
    # Full 130 x 3 grid: spread charges re-derived in numpy (row = x node), node
    # potentials by numpy's FFT of the zero-padded problem.
    y, n = small["y"], small["n"]
    rep, z, w, yt, phi = oracle.repulsive(y, details=True)
    nb, p, G = 130, 3, 390
    lo, hi = y.min(), y.max()
    bw = np.float32((hi - lo) / np.float32(nb))
    h = np.float32(bw / np.float32(3))
    xs, ys = y[:n], y[n:]
    bx = np.clip(((xs - lo) / bw).astype(np.int32), 0, nb - 1)
    by = np.clip(((ys - lo) / bw).astype(np.int32), 0, nb - 1)
    tx = ((xs - (bx * bw + lo)) / bw).astype(np.float64)
    ty = ((ys - (by * bw + lo)) / bw).astype(np.float64)
    nodes = np.array([1 / 6, 1 / 2, 5 / 6])

    def lagrange(t):
        out = np.ones((t.size, 3))
        for m in range(3):
            for q in range(3):
                if q != m:
                    out[:, m] *= (t - nodes[q]) / (nodes[m] - nodes[q])
        return out
    Lx, Ly = lagrange(tx), lagrange(ty)
    np.testing.assert_allclose(Lx.sum(1), 1.0, atol=1e-12)  # partition of unity
    charges = np.stack([np.ones(n), xs, ys, xs.astype(np.float64) ** 2 + ys.astype(np.float64) ** 2], 1)
    w_ref = np.zeros((G, G, 4))
    for a in range(3):
        for b in range(3):
            np.add.at(w_ref, (bx * 3 + a, by * 3 + b), (Lx[:, a] * Ly[:, b])[:, None] * charges)
    # the in-box coordinate is a difference of fp32 numbers ~130 box widths from the
    # origin, so fp32 weights carry ~1e-5 of relative noise against this fp64 model
    assert rel_l2(w, w_ref) < 1e-4
    # total charge is conserved plane by plane
    np.testing.assert_allclose(w.reshape(-1, 4).sum(0), charges.sum(0), rtol=1e-4, atol=1e-2)
    a = np.arange(-(G - 1), G)
    kern = (1.0 + (a[:, None] * float(h)) ** 2 + (a[None, :] * float(h)) ** 2) ** -2
    F = 1024
    kpad = np.zeros((F, F))
    kpad[np.ix_(a % F, a % F)] = kern
    yt_ref = np.empty((G, G, 4))
    for t in range(4):
        wpad = np.zeros((F, F))
        wpad[:G, :G] = w[..., t]
        yt_ref[..., t] = np.fft.irfft2(np.fft.rfft2(wpad) * np.fft.rfft2(kpad), s=(F, F))[:G, :G]
    for t in range(4):
        assert rel_l2(yt[..., t], yt_ref[..., t]) < 2e-5  # kernel offsets carry fp32 rounding of the node coordinates


def test_repulsive_against_exact_sums(small):
    # End to end against the O(N^2) definition: agreement to interpolation accuracy.
    y = small["y"]
    rep, z = oracle.repulsive(y)
    rep_x, z_x = exact_repulsive(y)
    assert rel_l2(rep, rep_x) < 5e-3
    assert abs(z - z_x) < 1e-3 * z_x


def test_repulsive_points_on_nodes_is_exact():
    # Points sitting exactly on interpolation nodes: Lagrange weights are 0/1,
    # so the grid sums are the exact sums.  nb = 2 boxes over [0, 6]: nodes at 0.5 + k.
    pts = np.array([[0.5, 0.5], [2.5, 1.5], [5.5, 4.5], [3.5, 3.5], [0.0, 6.0]], np.float64)
    y = np.concatenate([pts[:, 0], pts[:, 1]]).astype(np.float32)
    rep, z, w, yt, phi = oracle.repulsive(y, nb=2, details=True)
    # The two corner points (0,6) fix the bounds but are off-node; compare the
    # node potentials of plane 0 with direct sums over the spread charges instead.
    G = 6
    h = 1.0
    acc = np.zeros((G, G))
    for m in range(G):
        for n_ in range(G):
            dm = (m - np.arange(G))[:, None] * h
            dn = (n_ - np.arange(G))[None, :] * h
            acc[m, n_] = (w[..., 0] / (1 + dm ** 2 + dn ** 2) ** 2).sum()
    np.testing.assert_allclose(yt[..., 0], acc, rtol=1e-5)
    # the on-node points put all their unit charge on one node
    assert abs(w[0, 0, 0] - 1.0) < 1e-5 and abs(w[2, 1, 0] - 1.0) < 1e-5


# -------------------------------------------------------------- update ------
@pytest.mark.parametrize("attr,rep,gain,u,momentum,exag,eta,z,expect", [
    # sign(d) != sign(u): gain + 0.2
    (0.5, 1.0, 1.0, -0.1, 0.5, 12.0, 200.0, 2.0, None),
    # same sign: gain * 0.8
    (0.5, 1.0, 1.0, 0.1, 0.8, 1.0, 200.0, 4.0, None),
    # gain floor 0.01
    (0.5, 0.0, 0.0101, 0.3, 0.8, 1.0, 10.0, 1.0, None),
    # u = -0.0 counts as negative (signbit), d positive -> sign differs
    (1.0, 0.0, 1.0, -0.0, 0.5, 1.0, 1.0, 1.0, None),
    # u = +0.0 with positive d -> same sign
    (1.0, 0.0, 1.0, 0.0, 0.5, 1.0, 1.0, 1.0, None),
])
def test_update_cases(attr, rep, gain, u, momentum, exag, eta, z, expect):
    f = np.float32
    d = f(f(exag) * f(attr)) - f(f(rep) / f(z))
    if np.signbit(d) != np.signbit(f(u)):
        g = f(np.float64(f(gain)) + 0.2)
    else:
        g = f(np.float64(f(gain)) * 0.8)
    if np.float64(g) < 0.01:
        g = f(0.01)
    unew = f(f(f(momentum) * f(u)) - f(f(f(eta) * g) * d))
    y0 = f(3.25)
    Y, G, U = oracle.update(np.array([y0, y0], f), np.array([attr, attr], f), np.array([rep, rep], f),
                            np.array([gain, gain], f), np.array([u, u], f), eta, z, momentum, exag)
    assert G[0] == g and G[1] == g
    assert U[0] == unew
    assert Y[0] == f(y0 + unew)


def test_schedule_switch(small):
    # exaggeration and momentum switch exactly at force_magnify_iters
    P, idx, y, n = small["P"], small["idx"], small["y"] * 1e-3, small["n"]
    g1, u1 = np.ones(2 * n, np.float32), np.zeros(2 * n, np.float32)
    ya, _ = oracle.iterate(P, idx, y, 2, step_begin=0, force_magnify_iters=1, gains=g1, old_forces=u1)
    g2, u2 = np.ones(2 * n, np.float32), np.zeros(2 * n, np.float32)
    yb, _ = oracle.iterate(P, idx, y, 1, step_begin=0, force_magnify_iters=1, gains=g2, old_forces=u2)
    yb, _ = oracle.iterate(P, idx, yb, 1, step_begin=5, force_magnify_iters=1, gains=g2, old_forces=u2)
    assert np.array_equal(ya, yb)
    # hand-rolled first step: exaggerated attraction minus normalised repulsion
    attr = oracle.attractive(P, idx, y)
    rep, z = oracle.repulsive(y)
    y1, _, _ = oracle.update(y, attr, rep, np.ones(2 * n, np.float32), np.zeros(2 * n, np.float32), 200.0, z, 0.5,
                             12.0)
    y1b, _ = oracle.iterate(P, idx, y, 1)
    assert np.array_equal(y1, y1b)


# ------------------------------------------------------------------ KL ------
def test_kl_definition(small):
    n, k, idx, P, y = small["n"], small["k"], small["idx"], small["P"], small["y"]
    xs, ys = y[:n].astype(np.float64), y[n:].astype(np.float64)
    d2 = (xs[:, None] - xs[None, :]) ** 2 + (ys[:, None] - ys[None, :]) ** 2
    Z = (1.0 / (1.0 + d2)).sum() - n
    rows = np.repeat(np.arange(n), k)
    pv = P.ravel().astype(np.float64)
    m = pv > 0
    q = 1.0 / (1.0 + d2[rows, idx.ravel()]) / Z
    want = (pv[m] * np.log(pv[m] / q[m])).sum()
    assert abs(oracle.kl(P, idx, y) - want) < 1e-9 * abs(want)


# --------------------------------------------------------------- init -------
@pytest.mark.parametrize("kind", [0, 1])
def test_init_restatement_against_the_std_classes(kind):
    # oracle.init spells the engine and the distributions out; the std:: classes themselves pin it.
    for seed in (0, 1, 42, 2147483647, -5, 1700000000):
        for n in (1, 7, 5000):
            assert np.array_equal(oracle.init(n, kind, seed), oracle.init(n, kind, seed, std=True))


def test_init_draw_order_and_moments():
    n = 200000
    g = oracle.init(n, 1, 12345).astype(np.float64)
    assert abs(g.mean()) < 3e-4 * 1e-4 * 30 and abs(g.std() / 1e-4 - 1.0) < 0.01
    u = oracle.init(n, 0, 12345).astype(np.float64)
    assert u.min() >= -5.0 and u.max() < 5.0 and abs(u.mean()) < 0.03 and abs(u.std() - 10 / np.sqrt(12)) < 0.02
    # seeds 0 and 1 coincide (the engine replaces a zero state by 1)
    assert np.array_equal(oracle.init(500, 1, 0), oracle.init(500, 1, 1))
    # minstd_rand0's 10000th value from seed 1 is 1043618065 (C++ standard, [rand.predef]): check the engine
    # through the uniform path, whose values are (x - 1) / 2^31 * 10 - 5 of consecutive engine states.
    x = 1
    for _ in range(10000):
        x = x * 16807 % 2147483647
    assert x == 1043618065
    uni = oracle.init(5000, 0, 1)  # 2 * 5000 normal draws first: a data-dependent number of engine calls,
    # so locate the uniform block by recomputing the engine stream and matching its first value
    xs, x = [], 1
    for _ in range(40000):
        x = x * 16807 % 2147483647
        xs.append(x)
    vals = (np.array(xs, np.float64) - 1).astype(np.float32) / np.float32(2147483646.0) * np.float32(10.0) + np.float32(-5.0)
    start = np.flatnonzero(vals == uni[0])
    assert any(np.array_equal(vals[s:s + 10000].astype(np.float32), uni) for s in start if s + 10000 <= len(vals))


# ------------------------------------------------------------- golden -------
def test_golden_small256():
    g = np.load(os.path.join(GOLDEN, "small256.npz"))
    idx, d2 = oracle.knn(g["X"], g["idx"].shape[1])
    assert np.array_equal(idx, g["idx"]) and np.array_equal(d2, g["d2"])
    dn, _ = oracle.max_normalize(d2)
    p = oracle.perplexity(dn, float(g["perplexity"]), 1e-4)
    assert np.array_equal(p, g["p"])
    P = oracle.symmetrize(p, idx)
    assert np.array_equal(P, g["P"])
    assert np.array_equal(oracle.attractive(P, idx, g["y"]), g["attr"])
    rep, z = oracle.repulsive(g["y"])
    assert rel_l2(rep, g["rep"]) < 1e-6 and abs(z - float(g["z"])) <= 1e-6 * abs(z)


def test_golden_c0_inputs_are_stable():
    # The c0 fixture is only meaningful for the exact bytes of the seeded inputs.
    X, fit = synthetic.make_config("c0")
    assert X.shape == (5000, 50) and X.dtype == np.float32
    assert abs(float(X.astype(np.float64).sum()) - 196656.655) < 0.01
    with open(os.path.join(GOLDEN, "c0_fit.json")) as f:
        gold = json.load(f)
    assert 2.0 < gold["kl_exact_z"] < gold["kl_initial"]
