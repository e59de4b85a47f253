"""Parity at the benchmark's own size: config c3, 1,000,000 x 50, K = 90.

The oracle is fast enough for everything but the full neighbour search, so the
stages after kNN are compared directly (same tolerances as at 5000 points) and
kNN through a sample of query rows, each against all million candidates.  The
points are renumbered in locality order first, as RunTsne does.
"""
import numpy as np
import pytest

import oracle

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

N, K, PERPLEXITY, EPS = 1000000, 90, 30.0, 1e-4


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


@pytest.fixture(scope="module")
def c3():
    from tsnecuda import stages, synthetic
    X, fit = synthetic.make_config("c3")
    assert X.shape == (N, 50) and fit["num_neighbors"] == K
    dX = torch.from_numpy(X).cuda()
    order = stages.locality_order(dX)
    dXs = stages.gather_rows(dX, order)
    del dX
    idx, d2, stats = stages.knn_select(dXs, K, 0)
    Xs = dXs.cpu().numpy()
    del dXs
    dn = stages.max_normalize_(d2.clone())
    cond = stages.perplexity(dn, PERPLEXITY, EPS)
    P = stages.symmetrize(cond, idx)
    Y0 = synthetic.initial_embedding(N)
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    return dict(stages=stages, order=order.cpu().numpy(), Xs=Xs, idx=idx, d2=d2, dn=dn, cond=cond, P=P, y0=y0,
                knn_stats=stats)


def test_order_is_a_permutation_and_the_sweep_skips_tiles(c3):
    assert np.array_equal(np.sort(c3["order"]), np.arange(N))
    ran_matrix_sweep, redone, per_mille = c3["knn_stats"]
    assert ran_matrix_sweep == 1 and redone == 0
    assert per_mille <= 300  # four equal clusters: a quarter of the tile pairs, plus the cluster borders


def test_knn_rows_bit_exact(c3):
    """192 query rows spread over the numbering, each against all 1M points."""
    idx, d2 = c3["idx"], c3["d2"]
    for first in (0, 333312, N - 64):
        io, do = oracle.knn(c3["Xs"], K, rows=(first, first + 64))
        assert np.array_equal(io, idx[first:first + 64].cpu().numpy())
        assert np.array_equal(do, d2[first:first + 64].cpu().numpy())
    # structure of every row: self first at distance 0, ascending distances, indices in range and distinct per row
    assert torch.equal(idx[:, 0].long(), torch.arange(N, device="cuda"))
    assert bool((d2[:, 0] == 0).all()) and bool((d2[:, 1:] >= d2[:, :-1]).all())
    assert int(idx.min()) >= 0 and int(idx.max()) < N
    srt = torch.sort(idx, dim=1).values
    assert bool((srt[:, 1:] != srt[:, :-1]).all())


def test_normalise_perplexity_symmetrise(c3):
    d2_h, idx_h = c3["d2"].cpu().numpy(), c3["idx"].cpu().numpy()
    dn_o, _ = oracle.max_normalize(d2_h)
    assert np.array_equal(c3["dn"].cpu().numpy(), dn_o)
    p_o = oracle.perplexity(dn_o, PERPLEXITY, EPS)
    p_g = c3["cond"].cpu().numpy()
    assert np.allclose(p_g.sum(1), 1.0, atol=2e-5)
    # every operation of the search is pinned down on both sides: all million rows follow the oracle's
    # bisection path and the probabilities agree bit for bit
    off_path = float((np.abs(p_g - p_o).max(1) > 1e-5 * np.maximum(p_o.max(1), 1e-30)).mean())
    print("perplexity c3: rows off the oracle's bisection path: %.3g" % off_path)
    assert off_path == 0.0
    assert np.array_equal(p_g.view(np.uint32), p_o.view(np.uint32))
    ent = -(p_g * np.log(np.maximum(p_g, 1e-30))).sum(1)
    assert np.abs(ent - np.log(PERPLEXITY)).max() < 3e-4
    P_o = oracle.symmetrize(p_g, idx_h)  # same conditional probabilities in: isolates the symmetrisation
    assert np.allclose(c3["P"].cpu().numpy(), P_o, rtol=1e-6, atol=1e-12)
    c3["P_h"], c3["idx_h"] = P_o, idx_h


def test_full_symmetrisation(c3):
    """(A + A^T) / 2N as CSR at a million points (180 M triples through the device radix sort): structure,
    mass, symmetry of every entry, and 48 rows rebuilt on the host from the conditional probabilities."""
    import time
    st = c3["stages"]
    cond, idx = c3["cond"], c3["idx"]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    row_ptr, col, val = st.symmetrize_full(cond, idx)
    torch.cuda.synchronize()
    nnz_sym = col.numel()
    print("symmetrize_full c3: %.1f ms, %d non-zeros (%.2f x N K)" % ((time.perf_counter() - t0) * 1e3, nnz_sym,
                                                                     nnz_sym / (N * K)))
    assert N * K <= nnz_sym <= 2 * N * K
    rp = row_ptr.long()
    assert int(rp[0]) == 0 and int(rp[-1]) == nnz_sym and bool((rp[1:] - rp[:-1] >= K).all())
    assert abs(float(val.sum(dtype=torch.float64)) - 1.0) <= 1e-5
    rows = torch.repeat_interleave(torch.arange(N, device="cuda"), rp[1:] - rp[:-1])
    keys = rows * N + col.long()
    assert bool((keys[1:] > keys[:-1]).all())  # rows in order, columns ascending and distinct inside a row
    # symmetry: the transposed keys, sorted, carry the same values
    order = torch.argsort(col.long() * N + rows)
    assert torch.equal(col.long()[order] * N + rows[order], keys)
    assert torch.equal(val[order], val)
    del keys, order
    # sampled rows against the definition
    cond_h = None
    for r in list(range(0, 16)) + list(range(500000, 500016)) + list(range(N - 16, N)):
        own_c = idx[r].long()
        own_v = cond[r]
        src = (idx == r).nonzero()  # (row, slot) of every entry that names r
        inc_c, inc_v = src[:, 0], cond[src[:, 0], src[:, 1]]
        dense = {}
        for c_, v_ in zip(own_c.tolist(), own_v.tolist()):
            dense[c_] = np.float32(v_)
        for c_, v_ in zip(inc_c.tolist(), inc_v.tolist()):
            dense[c_] = np.float32(dense.get(c_, np.float32(0.0)) + np.float32(v_))
        lo, hi = int(rp[r]), int(rp[r + 1])
        assert col[lo:hi].tolist() == sorted(dense)
        want = np.array([np.float32(float(dense[c_]) / (2.0 * N)) for c_ in sorted(dense)], np.float32)
        assert np.array_equal(val[lo:hi].cpu().numpy(), want)
    c3["csr"] = (row_ptr, col, val)


def test_forces_and_fused_steps(c3):
    st = c3["stages"]
    P_h, idx_h = c3["P"].cpu().numpy(), c3["idx"].cpu().numpy()
    plan = st.Plan(N, K)
    plan.prepare_attractive(c3["P"], c3["idx"])
    # an embedding with structure: 60 steps of the GPU loop from the seeded start
    y = torch.from_numpy(c3["y0"]).cuda()
    gains, old = torch.ones_like(y), torch.zeros_like(y)
    plan.iterate_(None, None, y, gains, old, 0, 60, eta=200.0)
    y_h, gains_h, old_h = y.cpu().numpy(), gains.cpu().numpy(), old.cpu().numpy()
    attr = plan.attractive(None, None, y).cpu().numpy()
    assert rel_l2(attr, oracle.attractive(P_h, idx_h, y_h)) <= 1e-4
    rep, z = plan.repulsive(y)
    rep_o, z_o = oracle.repulsive(y_h)
    assert rel_l2(rep.cpu().numpy(), rep_o) <= 1e-4
    assert abs(float(z) - z_o) <= 1e-5 * abs(z_o)
    # three fused steps against three oracle steps from the same state
    plan.iterate_(None, None, y, gains, old, 60, 63, eta=200.0)
    y_o, _ = oracle.iterate(P_h, idx_h, y_h, 3, step_begin=60, eta=200.0, gains=gains_h, old_forces=old_h)
    assert rel_l2(y.cpu().numpy(), y_o) <= 1e-4
    plan.close()


def test_blocked_attractive_with_more_than_1024_column_partitions():
    """4.5 M points are 2198 column partitions of 2048: the re-blocking's scans
    give every thread several partition slots.  A pattern without any locality
    (every strip references every partition, most runs far shorter than a work
    item) against the row-ordered kernel and, on its first and last rows, the
    oracle."""
    from tsnecuda import stages
    n, k = 4500000, 6
    g = torch.Generator(device="cuda").manual_seed(1)
    idx = torch.randint(0, n, (n, k), generator=g, device="cuda", dtype=torch.int32)
    idx[:, 0] = torch.arange(n, device="cuda", dtype=torch.int32)
    P = torch.rand((n, k), generator=g, device="cuda", dtype=torch.float32) * 1e-6
    P[:, 0] = 0.0
    y = torch.randn(2 * n, generator=g, device="cuda", dtype=torch.float32) * 20.0
    plan = stages.Plan(n, k)
    plan.prepare_attractive(P, idx)
    blocked = plan.attractive(None, None, y)
    by_rows = plan.attractive(P, idx, y)
    assert rel_l2(blocked.cpu().numpy(), by_rows.cpu().numpy()) <= 1e-6
    want = oracle.attractive(P.cpu().numpy(), idx.cpu().numpy(), y.cpu().numpy())
    assert rel_l2(blocked.cpu().numpy(), want) <= 1e-4
    plan.close()


def test_c3_fit_objective_within_one_percent():
    """The benchmark's own fit: 1,000,000 x 50, 1000 steps from the seeded start
    through TSNE.fit_transform.  The objective of the returned embedding (the
    library's evaluation: on configs c1 and c2 it agrees with the oracle's
    exact-Z evaluation to 1e-5, and the exact one is an hour of CPU time here)
    within 1 % of the oracle's own 1000-step run, and the trustworthiness of a
    fixed 4000-point subsample within 0.02 of it (tests/golden/c3_fit.json)."""
    import json
    import os
    from sklearn.manifold import trustworthiness
    from tsnecuda import TSNE, synthetic
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c3_fit.json")) as f:
        gold = json.load(f)
    X, fit = synthetic.make_config("c3")
    Y0 = synthetic.initial_embedding(N)
    model = TSNE(perplexity=fit["perplexity"], num_neighbors=fit["num_neighbors"], learning_rate=fit["learning_rate"],
                 n_iter=1000, perplexity_epsilon=1e-4)
    emb = model.fit_transform(X, y=Y0)
    assert emb.shape == (N, 2) and np.isfinite(emb).all()
    sub = np.sort(np.random.default_rng(0).choice(N, size=4000, replace=False))  # as tests/golden/make_golden.py
    t = trustworthiness(X[sub], emb[sub], n_neighbors=12)
    print("c3: KL gpu %.5f oracle %.5f, trustworthiness gpu %.4f oracle %.4f"
          % (model.kl_divergence_, gold["kl_exact_z"], t, gold["trustworthiness_k12_subsample4000"]))
    assert abs(model.kl_divergence_ - gold["kl_exact_z"]) <= 0.01 * gold["kl_exact_z"]
    assert abs(t - gold["trustworthiness_k12_subsample4000"]) <= 0.02
    assert 0.8 < (emb.max() - emb.min()) / (gold["extent"][1] - gold["extent"][0]) < 1.25
