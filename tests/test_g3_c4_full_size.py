"""Parity on config c4: 10,000,000 x 50 points, K = 90 (0.9 billion non-zeros).

Same chain as RunTsne: locality order -> exact kNN -> max-normalise -> perplexity
search -> symmetrise -> re-blocked pattern -> forces -> fused steps.  The oracle
checks what it can finish in seconds at this size: sampled query rows of the
neighbour search (each against all ten million candidates), the normalisation in
full, sampled rows of the perplexity search and of the symmetrisation, and the
forces and three fused steps in full.

(The GPU test files are numbered in the order pytest collects them: stage parity,
then the full-size configs, then whole fits, then the surface around the fit; a run
with -x that stops early has then covered the stages first.)
"""
import time

import numpy as np
import pytest

import oracle

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

N, D, K, PERPLEXITY, EPS = 10000000, 50, 90, 30.0, 1e-4


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


@pytest.fixture(scope="module")
def c4():
    from tsnecuda import stages, synthetic
    t0 = time.time()
    X, fit = synthetic.make_config("c4")
    assert X.shape == (N, D) and fit["num_neighbors"] == K
    print("c4: generated %d x %d points in %.1f s" % (N, D, time.time() - t0), flush=True)
    dX = torch.from_numpy(X).cuda()
    del X
    order = stages.locality_order(dX)
    dXs = stages.gather_rows(dX, order)
    del dX
    torch.cuda.synchronize()
    t0 = time.time()
    idx, d2, stats = stages.knn_select(dXs, K, 0)
    torch.cuda.synchronize()
    print("c4: exact kNN in %.1f s, stats %s" % (time.time() - t0, stats), flush=True)
    Xs = dXs.cpu().numpy()
    del dXs
    dn = stages.max_normalize_(d2.clone())
    cond = stages.perplexity(dn, PERPLEXITY, EPS)
    P = stages.symmetrize(cond, idx)
    torch.cuda.synchronize()
    Y0 = synthetic.initial_embedding(N)
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    return dict(stages=stages, order=order, Xs=Xs, idx=idx, d2=d2, dn=dn, cond=cond, P=P, y0=y0, knn_stats=stats)


def test_c4_order_and_knn_rows_bit_exact(c4):
    """96 query rows spread over the numbering, each against all 10M points, bit for bit;
    and the structure of every one of the ten million rows."""
    order = c4["order"]
    assert bool((torch.sort(order).values == torch.arange(N, device="cuda", dtype=order.dtype)).all())
    ran_matrix_sweep, redone, per_mille = c4["knn_stats"]
    assert ran_matrix_sweep == 1
    print("c4 kNN: %d queries redone, %d per mille of the tile pairs computed" % (redone, per_mille))
    idx, d2 = c4["idx"], c4["d2"]
    rows = np.concatenate([np.arange(0, 16), np.arange(N - 16, N),
                           np.random.default_rng(4).choice(N, size=64, replace=False)]).astype(np.int32)
    t0 = time.time()
    io, do = oracle.knn(c4["Xs"], K, rows=rows)
    print("c4 kNN: oracle rows in %.1f s" % (time.time() - t0), flush=True)
    pick = torch.from_numpy(rows.astype(np.int64)).cuda()
    assert np.array_equal(io, idx[pick].cpu().numpy())
    assert np.array_equal(do, d2[pick].cpu().numpy())
    assert torch.equal(idx[:, 0], torch.arange(N, device="cuda", dtype=torch.int32))
    assert bool((d2[:, 0] == 0).all()) and bool((d2[:, 1:] >= d2[:, :-1]).all())
    assert int(idx.min()) >= 0 and int(idx.max()) < N
    for b in range(0, N, 2000000):  # distinct neighbours per row (sorted in slabs: a full sort needs 7 GB more)
        srt = torch.sort(idx[b:b + 2000000], dim=1).values
        assert bool((srt[:, 1:] != srt[:, :-1]).all())
    # The approximate search on the same points (inverted file, floor(sqrt(N)) = 3162 lists as the reference's
    # FAISS index, 100 lists probed per list): its time, its recall against the exact rows, and what must hold
    # of any subset search - rank by rank no neighbour is nearer than the exact one, and a row that found the
    # exact neighbours reports the exact distances.
    st = c4["stages"]
    dXs = torch.from_numpy(c4["Xs"]).cuda()
    torch.cuda.synchronize()
    t0 = time.time()
    cen = st.ivf_train(dXs, 3162)
    torch.cuda.synchronize()
    t1 = time.time()
    idx_a, d2_a, stats_a = st.knn_ivf(dXs, K, cen, 100)
    torch.cuda.synchronize()
    t2 = time.time()
    del dXs
    sample = torch.arange(0, N, N // 20000, device="cuda")[:20000]
    found = (idx_a[sample, 1:, None] == idx[sample, None, 1:]).any(2)
    recall = float(found.float().mean())
    print("c4 approximate kNN: train %.2f s, search %.2f s, %d per mille of the tile pairs, recall@%d %.4f"
          % (t1 - t0, t2 - t1, stats_a[2], K - 1, recall), flush=True)
    assert stats_a[0] == 1 and stats_a[1] == 0 and recall > 0.25
    assert torch.equal(idx_a[:, 0], torch.arange(N, device="cuda", dtype=torch.int32))
    assert bool((d2_a[sample] >= d2[sample]).all())
    whole = found.all(1)
    assert bool((d2_a[sample][whole] == d2[sample][whole]).all())
    del idx_a, d2_a
    c4.pop("Xs")


def test_c4_normalise_perplexity_symmetrise(c4):
    d2, dn, cond, P, idx = c4["d2"], c4["dn"], c4["cond"], c4["P"], c4["idx"]
    # max-normalisation: x / max in correctly rounded fp32 (the oracle's definition), bit for bit on 200,000
    # rows spread over the numbering; the largest value itself maps to exactly 1
    rows = torch.arange(0, N, 50, device="cuda")
    dmax = np.float32(d2.max().item())
    assert np.array_equal(dn[rows].cpu().numpy(), d2[rows].cpu().numpy() / dmax)
    assert float(dn.max()) == 1.0 and float(dn.min()) == 0.0
    # perplexity search on the same rows, bit for bit as at 5000 points
    p_o = oracle.perplexity(dn[rows].cpu().numpy(), PERPLEXITY, EPS)
    p_g = cond[rows].cpu().numpy()
    off_path = float((np.abs(p_g - p_o).max(1) > 1e-5 * np.maximum(p_o.max(1), 1e-30)).mean())
    print("perplexity c4 (200000 sampled rows): rows off the oracle's bisection path: %.3g" % off_path)
    assert off_path == 0.0 and np.array_equal(p_g.view(np.uint32), p_o.view(np.uint32))
    sums = cond.sum(1)
    assert float((sums - 1.0).abs().max()) <= 2e-5
    # symmetrisation on 3000 sampled rows: P[i,s] = (p[i,s] + sum_{t: idx[j,t]==i} p[j,t]) / 2N, j = idx[i,s],
    # from the pulled rows of p and idx (numpy, float64 then the reference's rounding to float)
    sample = torch.arange(7, N, N // 3000, device="cuda")[:3000]
    nbr = idx[sample].long()                       # (m, K)
    back_idx = idx[nbr.reshape(-1)].reshape(len(sample), K, K).cpu().numpy()
    back_p = cond[nbr.reshape(-1)].reshape(len(sample), K, K).cpu().numpy()
    mine = cond[sample].cpu().numpy()
    rows_h = sample.cpu().numpy()
    want = mine.astype(np.float32).copy()
    match = back_idx == rows_h[:, None, None]
    for t in range(K):  # the oracle's order of additions: ascending slot of row j
        want = want + np.where(match[:, :, t], back_p[:, :, t], np.float32(0.0)).astype(np.float32)
    want = (want.astype(np.float64) / (2.0 * N)).astype(np.float32)
    got = P[sample].cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=0)
    total = float(P.sum(dtype=torch.float64))
    assert 0.5 < total <= 1.0 + 1e-6  # pattern-restricted: entries whose mirror is not stored are dropped


def test_c4_forces_and_fused_steps(c4):
    st = c4["stages"]
    P, idx = c4["P"], c4["idx"]
    plan = st.Plan(N, K)
    plan.prepare_attractive(P, idx)
    # an embedding with structure: 60 steps of the GPU loop from the seeded start
    y = torch.from_numpy(c4["y0"]).cuda()
    gains, old = torch.ones_like(y), torch.zeros_like(y)
    plan.iterate_(None, None, y, gains, old, 0, 60, eta=200.0)
    torch.cuda.synchronize()
    y_h, gains_h, old_h = y.cpu().numpy(), gains.cpu().numpy(), old.cpu().numpy()
    P_h, idx_h = P.cpu().numpy(), idx.cpu().numpy()
    t0 = time.time()
    attr = plan.attractive(None, None, y).cpu().numpy()
    want = oracle.attractive(P_h, idx_h, y_h)
    err_blocked = rel_l2(attr, want)
    by_rows = plan.attractive(P, idx, y).cpu().numpy()
    err_rows = rel_l2(by_rows, want)
    print("c4 attractive: re-blocked %.2e, row-ordered %.2e (oracle %.1f s)" % (err_blocked, err_rows,
                                                                              time.time() - t0), flush=True)
    assert err_blocked <= 1e-4 and err_rows <= 1e-4
    rep, z = plan.repulsive(y)
    rep_o, z_o = oracle.repulsive(y_h)
    err_rep, err_z = rel_l2(rep.cpu().numpy(), rep_o), abs(float(z) - z_o) / abs(z_o)
    print("c4 repulsive: %.2e, Z %.2e" % (err_rep, err_z), flush=True)
    assert err_rep <= 1e-4 and err_z <= 1e-5
    # three fused steps against three oracle steps from the same state
    t0 = time.time()
    plan.iterate_(None, None, y, gains, old, 60, 63, eta=200.0)
    y_o, _ = oracle.iterate(P_h, idx_h, y_h, 3, step_begin=60, eta=200.0, gains=gains_h, old_forces=old_h)
    err_steps = rel_l2(y.cpu().numpy(), y_o)
    print("c4 three fused steps: %.2e (oracle %.1f s)" % (err_steps, time.time() - t0), flush=True)
    assert err_steps <= 1e-4
    plan.check()
    plan.close()
