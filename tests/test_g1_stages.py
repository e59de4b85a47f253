"""Parity of every HIP stage against the CPU oracle, through the C ABI.

Inputs are config c0 (5000 x 50 Gaussian clusters, K = 90, perplexity 30) and
embedding snapshots produced by the oracle's own gradient loop.  Tolerances are
the ones the project states: kNN indices bit-exact, P to 1e-5 relative,
attractive / repulsive forces to 1e-4 relative L2.
"""
import numpy as np
import pytest

import oracle

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


def same_bits(a, b):
    """Two runs of the gradient loop from one start: every sum between the points and the forces is an integer
    sum (fixed point), so neither the order in which workgroups arrive nor how the points were grouped can change
    a bit of the result."""
    a = np.ascontiguousarray(a, np.float32).ravel()
    b = np.ascontiguousarray(b, np.float32).ravel()
    return bool(np.array_equal(a.view(np.uint32), b.view(np.uint32)))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def stages():
    from tsnecuda import stages as st
    st.lib()
    return st


@pytest.fixture(scope="module")
def snapshots(c0_problem):
    """Embeddings after 0, 30 and 300 oracle steps (the last is past the
    exaggeration switch at 250)."""
    c = c0_problem
    snaps = {0: c["y0"].copy()}
    gains = np.ones_like(c["y0"])
    old = np.zeros_like(c["y0"])
    y = c["y0"].copy()
    done = 0
    for upto in (30, 300):
        y, _ = oracle.iterate(c["P"], c["idx"], y, upto - done, step_begin=done, gains=gains, old_forces=old)
        done = upto
        snaps[upto] = y.copy()
    snaps["gains"] = gains
    snaps["old"] = old
    return snaps


def test_knn_bit_exact(stages, c0_problem):
    c = c0_problem
    idx, d2 = stages.knn(dev(c["X"]), c["K"])
    idx, d2 = idx.cpu().numpy(), d2.cpu().numpy()
    assert np.array_equal(idx, c["idx"])
    assert np.array_equal(d2.view(np.uint32), c["d2"].view(np.uint32))


def test_max_normalize_bit_exact(stages, c0_problem):
    c = c0_problem
    out = stages.max_normalize_(dev(c["d2"])).cpu().numpy()
    assert np.array_equal(out.view(np.uint32), c["dn"].view(np.uint32))


def test_perplexity(stages, c0_problem):
    """Every operation of the search is pinned down on both sides (exp and log as
    fixed fp32 operation sequences, the row sums in one stated order), so every row
    follows the oracle's bisection path and the probabilities agree bit for bit -
    which the 1e-5 relative bound of the project then holds with room to spare."""
    c = c0_problem
    eps = 1e-4
    p, beta = stages.perplexity(dev(c["dn"]), c["fit"]["perplexity"], eps, return_betas=True)
    p, beta = p.cpu().numpy(), beta.cpu().numpy()
    assert np.all(p[:, 0] == 0.0)
    np.testing.assert_allclose(p.sum(axis=1), 1.0, atol=1e-5)
    off_path = float((beta != c["beta"]).mean())
    print("perplexity c0: rows off the oracle's bisection path: %.3g" % off_path)
    assert off_path == 0.0
    nz = c["p"] > 0
    assert (np.abs(p[nz] - c["p"][nz]) / c["p"][nz]).max() <= 1e-5
    assert np.array_equal(p.view(np.uint32), c["p"].view(np.uint32))


@pytest.mark.parametrize("data,k,perp", [
    ("c0", 90, 1.5), ("c0", 90, 2.0), ("c0", 90, 5.0), ("c0", 6, 1.2), ("c0", 3, 1.3),
    ("d300", 1023, 30.0), ("d300", 300, 5.0), ("d300", 90, 2.0), ("d300", 1100, 50.0),
])
def test_perplexity_far_below_the_neighbour_count(stages, c0_problem, data, k, perp):
    """Perplexities of 1.2 to 5 on 90 neighbours, and 300-dimensional data whose normalised distances are
    nearly equal within a row: the search then needs precisions at which exp(-beta d) underflows (subnormal
    probabilities, rows whose sum is zero for some of the betas tried, rows that use all 200 evaluations).
    Every row still follows the oracle's path: the same final beta and the same probabilities, bit for bit."""
    from tsnecuda import synthetic
    if data == "c0":
        X = c0_problem["X"]
    else:
        X = synthetic.gaussian_clusters(6000, d=300, clusters=4, center_scale=5.0, seed=7)
    idx, d2 = stages.knn(dev(X), k)
    dn = stages.max_normalize_(d2)
    p, beta = stages.perplexity(dn, perp, 1e-4, return_betas=True)
    p, beta = p.cpu().numpy(), beta.cpu().numpy()
    p_o, beta_o, iters = oracle.perplexity(dn.cpu().numpy(), perp, 1e-4, return_search=True)
    print("perplexity %s k=%d perp=%g: most evaluations %d, rows at the cap %d, subnormal probabilities %d"
          % (data, k, perp, iters.max(), int((iters == 200).sum()), int(((p_o > 0) & (p_o < 1.1754944e-38)).sum())))
    assert np.isfinite(p).all()
    assert float((beta != beta_o).mean()) == 0.0
    assert np.array_equal(p.view(np.uint32), p_o.view(np.uint32))


def test_symmetrize(stages, c0_problem):
    c = c0_problem
    P = stages.symmetrize(dev(c["p"]), dev(c["idx"])).cpu().numpy()
    np.testing.assert_allclose(P, c["P"], rtol=1e-6, atol=0)


@pytest.mark.parametrize("n,k,duplicates", [(5000, 90, False), (4096, 7, False), (30000, 24, True), (5000, 600, False)])
def test_symmetrize_hashed_and_scanning_forms(stages, c0_problem, monkeypatch, n, k, duplicates):
    """The symmetrisation looks a row's number up in a per-row hash table of the row it points to (the default
    from 4096 points up) or scans that row (small problems, thousands of neighbours): the same values,
    bit for bit; where a row names a column twice the hashed form notices and hands over to the scan, which adds
    such values up.  Against the oracle either way."""
    if (n, k) == (5000, 90):
        p, idx = c0_problem["p"], c0_problem["idx"]
    else:
        rng = np.random.default_rng(n + k)
        if duplicates:
            idx = rng.integers(0, n, (n, k)).astype(np.int32)
            idx[:, 0] = np.arange(n)
            idx[::3, 5] = idx[::3, 2]   # columns named twice and three times in a row
            idx[::7, 9] = idx[::7, 2]
        else:
            # row i names the columns i + o for k distinct offsets o (one of five offset sets): many mutual pairs
            sets = np.stack([np.concatenate([[0], 1 + rng.choice(n - 1, size=k - 1, replace=False)]) for _ in range(5)])
            sets[1, 1:] = (n - sets[0, 1:]) % n   # set 1 mirrors set 0: rows of those two sets name each other
            idx = ((np.arange(n)[:, None] + sets[np.arange(n) % 5]) % n).astype(np.int32)
        p = rng.random(idx.shape).astype(np.float32)
        p[:, 0] = 0.0
        p /= p.sum(1, keepdims=True)
    want = oracle.symmetrize(p, idx)
    got = {}
    for form in ("hashed", "scan"):
        if form == "scan":
            monkeypatch.setenv("TSNE_SYMMETRIZE_SCAN", "1")
        else:
            monkeypatch.delenv("TSNE_SYMMETRIZE_SCAN", raising=False)
        got[form] = stages.symmetrize(dev(p), dev(idx)).cpu().numpy()
        np.testing.assert_allclose(got[form], want, rtol=2e-6, atol=0)
    if not duplicates and k != 7:
        assert (want > p / (2.0 * n) * (1.0 + 1e-3)).mean() > 0.005   # the case has pairs in both directions
    assert np.array_equal(got["hashed"].view(np.uint32), got["scan"].view(np.uint32))
    # a column that names no point is refused by the form that would address a table with it
    monkeypatch.delenv("TSNE_SYMMETRIZE_SCAN", raising=False)
    bad = idx.copy()
    bad[n // 2, k // 2] = n
    with pytest.raises(RuntimeError, match="outside"):
        stages.symmetrize(dev(p), dev(bad))


@pytest.mark.parametrize("n,k", [(2, 2), (7, 3), (300, 300), (5000, 90), (70000, 20), (20000, 1)])
def test_symmetrize_full_csr(stages, c0_problem, n, k):
    """(A + A^T) / 2N with the union pattern: the device radix sort + segmented reduce against the oracle's
    CSR, bit for bit (row pointers, columns, values) - one tile and several tiles of the sort, dense rows,
    K = 1 (every row: the explicit zero of the self entry only)."""
    if (n, k) == (5000, 90):
        p, idx = c0_problem["p"], c0_problem["idx"]
    else:
        # row i names the columns i + o for the k offsets o of one of seven offset sets (0 = itself first, the
        # others distinct): distinct columns in every row, in-degrees that vary from row to row
        rng = np.random.default_rng(n * 31 + k)
        sets = np.stack([np.concatenate([[0], 1 + rng.choice(n - 1, size=k - 1, replace=False)]) for _ in range(7)])
        idx = ((np.arange(n)[:, None] + sets[np.arange(n) % 7]) % n).astype(np.int32)
        p = rng.random(idx.shape).astype(np.float32)
        p[:, 0] = 0.0
        p /= np.maximum(p.sum(1, keepdims=True), 1e-30)
    want_ptr, want_col, want_val = oracle.symmetrize_full(p, idx)
    row_ptr, col, val = stages.symmetrize_full(dev(p), dev(idx))
    assert np.array_equal(row_ptr.cpu().numpy(), want_ptr)
    assert np.array_equal(col.cpu().numpy(), want_col)
    assert np.array_equal(val.cpu().numpy().view(np.uint32), want_val.view(np.uint32))
    if k > 1:
        assert abs(float(val.sum(dtype=torch.float64)) - 1.0) <= 1e-5
    # forces over the CSR pattern, stage call and fused loop
    nn = idx.shape[0]
    rng = np.random.default_rng(1)
    y = (rng.standard_normal(2 * nn) * 3.0).astype(np.float32)
    plan = stages.Plan(nn, k)
    got = plan.attractive_csr(row_ptr, col, val, dev(y)).cpu().numpy()
    want = oracle.attractive_csr(want_ptr, want_col, want_val, y)
    if np.linalg.norm(want) > 0:
        assert rel_l2(got, want) <= 1e-4
    plan.close()


def test_iterate_over_the_full_csr_pattern(stages, c0_problem):
    """Steps whose attractive forces come from the fully symmetrised CSR pattern, against the same steps
    with the forces of the oracle's CSR evaluation: the embedding after three steps."""
    c = c0_problem
    n = c["X"].shape[0]
    row_ptr, col, val = stages.symmetrize_full(dev(c["p"]), dev(c["idx"]))
    plan = stages.Plan(n, c["K"])
    plan.set_csr_pattern(row_ptr, col, val)
    dy = dev(c["y0"])
    gains, old = torch.ones_like(dy), torch.zeros_like(dy)
    plan.iterate_(None, None, dy, gains, old, 0, 3)
    # the oracle's loop, its attractive stage replaced by the CSR evaluation
    y = c["y0"].copy()
    g, u = np.ones_like(y), np.zeros_like(y)
    rp, cc, vv = oracle.symmetrize_full(c["p"], c["idx"])
    for _ in range(3):
        rep, z = oracle.repulsive(y)
        y, g, u = oracle.update(y, oracle.attractive_csr(rp, cc, vv, y), rep, g, u, 200.0, z, 0.5, 12.0)
    assert rel_l2(dy.cpu().numpy(), y) <= 1e-4
    plan.set_csr_pattern(None, None, None)
    with pytest.raises(RuntimeError, match="none prepared"):
        plan.iterate_(None, None, dy, gains, old, 0, 1)
    plan.close()


@pytest.mark.parametrize("step", [0, 30, 300])
def test_attractive(stages, c0_problem, snapshots, step):
    c = c0_problem
    plan = stages.Plan(c["X"].shape[0], c["K"])
    got = plan.attractive(dev(c["P"]), dev(c["idx"]), dev(snapshots[step])).cpu().numpy()
    want = oracle.attractive(c["P"], c["idx"], snapshots[step])
    assert rel_l2(got, want) <= 1e-4
    plan.close()


@pytest.mark.parametrize("step", [0, 30, 300])
def test_repulsive(stages, c0_problem, snapshots, step):
    c = c0_problem
    n = c["X"].shape[0]
    plan = stages.Plan(n, c["K"])
    rep, z, w, yt, phi = plan.repulsive(dev(snapshots[step]), details=True)
    rep_o, z_o, w_o, yt_o, phi_o = oracle.repulsive(snapshots[step], details=True)
    w, yt, phi = w.cpu().numpy(), yt.cpu().numpy(), phi.cpu().numpy()
    errs = dict(w=[rel_l2(w[..., t], w_o[..., t]) for t in range(4)],
                yt=[rel_l2(yt[..., t], yt_o[..., t]) for t in range(4)],
                phi=[rel_l2(phi[:, t], phi_o[:, t]) for t in range(4)],
                z=abs(float(z.item()) - z_o) / abs(z_o), rep=rel_l2(rep.cpu().numpy(), rep_o))
    print("repulsive step", step, errs)
    # Every charge plane on its own scale, not only the largest one.
    assert max(errs["w"]) <= 1e-5
    assert max(errs["yt"]) <= 2e-5
    assert max(errs["phi"]) <= 2e-5
    assert errs["z"] <= 1e-5
    assert errs["rep"] <= 1e-4
    # A second call must not see stale charges.
    rep2, z2 = plan.repulsive(dev(snapshots[step]))
    assert rel_l2(rep2.cpu().numpy(), rep_o) <= 1e-4
    plan.close()


def test_update(stages, c0_problem, snapshots):
    c = c0_problem
    n = c["X"].shape[0]
    y = snapshots[300]
    attr = oracle.attractive(c["P"], c["idx"], y)
    rep, z = oracle.repulsive(y)
    rng = np.random.default_rng(0)
    gains = rng.uniform(0.005, 2.0, 2 * n).astype(np.float32)
    old = (rng.standard_normal(2 * n) * 1e-2).astype(np.float32)
    old[::7] = -0.0
    y_o, g_o, u_o = oracle.update(y, attr, rep, gains, old, 200.0, z, 0.8, 1.0)
    plan = stages.Plan(n, c["K"])
    dy, da, dr, dg, du = dev(y), dev(attr), dev(rep), dev(gains), dev(old)
    plan.update_(dy, da, dr, dg, du, 200.0, dev(np.array([z], np.float32)), 0.8, 1.0)
    assert np.array_equal(dg.cpu().numpy(), g_o)
    np.testing.assert_allclose(du.cpu().numpy(), u_o, rtol=1e-6, atol=1e-12)
    np.testing.assert_allclose(dy.cpu().numpy(), y_o, rtol=1e-6, atol=1e-9)
    assert float(da.abs().max()) == 0.0 and float(dr.abs().max()) == 0.0
    plan.close()


@pytest.mark.parametrize("start,steps", [(0, 5), (248, 4)])
def test_iterate_short(stages, c0_problem, start, steps):
    """A few fused steps (across the schedule switch at 250 in the second case)
    against the oracle's loop from the same state."""
    c = c0_problem
    n = c["X"].shape[0]
    gains = np.ones(2 * n, np.float32)
    old = np.zeros(2 * n, np.float32)
    y = c["y0"].copy()
    if start:
        y, _ = oracle.iterate(c["P"], c["idx"], y, start, gains=gains, old_forces=old)
    g_o, u_o = gains.copy(), old.copy()
    y_o, z_o = oracle.iterate(c["P"], c["idx"], y, steps, step_begin=start, gains=g_o, old_forces=u_o)
    plan = stages.Plan(n, c["K"])
    dy, dg, du = dev(y), dev(gains), dev(old)
    z = plan.iterate_(dev(c["P"]), dev(c["idx"]), dy, dg, du, start, start + steps)
    assert rel_l2(dy.cpu().numpy(), y_o) <= 1e-4
    assert abs(float(z.item()) - z_o) <= 1e-4 * abs(z_o)
    plan.close()


@pytest.mark.parametrize("eta,steps", [(200.0, 40), (3000.0, 12)])
def test_iterate_keeps_the_grouping_by_tile(stages, c0_problem, monkeypatch, eta, steps):
    """Inside a loop the repulsive chain keeps its grouping of the points by grid tile while few points
    have left the neighbourhood of their tile.  40 steps at the usual learning rate, of which a good part
    reuse the grouping, and 12 at a learning rate that throws points across several boxes per step (strays,
    spread on the slow path, and early re-grouping), against the oracle's loop and against a plan that
    groups afresh every step (TSNE_KEEP_GROUPING=0); a stage-level call in between (which always groups
    afresh) must not disturb the loop's state."""
    c = c0_problem
    n = c["X"].shape[0]
    y_o, z_o = oracle.iterate(c["P"], c["idx"], c["y0"], steps, eta=eta)

    def run(keep):
        monkeypatch.setenv("TSNE_KEEP_GROUPING", "1" if keep else "0")
        plan = stages.Plan(n, c["K"])
        plan.prepare_attractive(dev(c["P"]), dev(c["idx"]))
        dy = dev(c["y0"])
        gains, old = torch.ones_like(dy), torch.zeros_like(dy)
        half = steps // 2
        plan.iterate_(None, None, dy, gains, old, 0, half, eta=eta)
        plan.repulsive(torch.flip(dy, [0]))  # an unrelated embedding through the stage call
        z = plan.iterate_(None, None, dy, gains, old, half, steps, eta=eta)
        stats = plan.grouping_stats()
        plan.close()
        return dy.cpu().numpy(), float(z.item()), stats

    y_keep, z_keep, (runs, sorts, strays) = run(True)
    y_fresh, z_fresh, (runs_f, sorts_f, strays_f) = run(False)
    err_keep, err_fresh = rel_l2(y_keep, y_o), rel_l2(y_fresh, y_o)
    print("eta %g: %d evaluations, %d groupings, %d strays; against the oracle %.2e (grouping kept) %.2e (afresh)"
          % (eta, runs, sorts, strays, err_keep, err_fresh))
    assert runs == steps + 1 and runs_f == steps + 1 and sorts_f == runs_f and strays_f == 0
    assert 3 <= sorts <= (steps * 3 // 4 if eta < 1000 else steps)
    if eta > 1000:
        assert strays > 0
    # How the points are grouped changes nothing in the sums (integers): the two plans end on the same bits.
    assert same_bits(y_keep, y_fresh) and z_keep == z_fresh
    # Against the oracle the trajectory amplifies the last-bit differences of the forces (the update rule is
    # discontinuous where gradient times momentum is zero to rounding: a coordinate's gain then grows on one
    # side and shrinks on the other, and that coordinate pulls its neighbours along), so the bound is per horizon.
    assert err_keep <= (5e-3 if steps >= 40 else 1e-3)
    assert abs(z_keep - z_o) <= 1e-2 * abs(z_o)


def test_repulsive_with_a_kept_grouping(stages):
    """tsne_hip_repulsive_kept: the evaluation a loop step makes.  The first call groups the points by tile,
    the following ones keep that grouping for embeddings that have moved on - scaled up and jittered by a
    fraction of a box, by a box or two, by many boxes - and must still produce the oracle's charges and forces:
    through regions that follow their points, through the slow path for points that strayed, and through a
    fresh grouping once too many have."""
    n = 6000
    rng = np.random.default_rng(3)
    y = (rng.standard_normal(2 * n) * 3.0).astype(np.float32)
    plan = stages.Plan(n, 30)
    box = float(y.max() - y.min()) / 130.0
    seen_strays = seen_kept = False
    for step, jitter in enumerate([0.0, 0.2, 0.2, 1.0, 0.3, 4.0, 0.1]):
        y = (y * np.float32(1.02) + rng.standard_normal(2 * n).astype(np.float32) * np.float32(jitter * box)).astype(np.float32)
        before = plan.grouping_stats()
        rep, z, w, yt, phi = plan.repulsive(dev(y), details=True, keep_grouping=True)
        runs, sorts, strays = [a - b for a, b in zip(plan.grouping_stats(), before)]
        rep_o, z_o, w_o, yt_o, phi_o = oracle.repulsive(y, details=True)
        print("step %d (jitter %.1f boxes): grouped afresh %d, strays %d" % (step, jitter, sorts, strays))
        assert runs == 1 and (step > 0 or sorts == 1)
        seen_kept = seen_kept or sorts == 0
        seen_strays = seen_strays or strays > 0
        for plane in range(4):
            assert rel_l2(w.cpu().numpy()[..., plane], w_o[..., plane]) <= 2e-5, (step, plane)
        assert rel_l2(rep.cpu().numpy(), rep_o) <= 1e-4 and abs(float(z) - z_o) <= 1e-5 * abs(z_o)
    assert seen_kept and seen_strays
    plan.close()


@pytest.mark.parametrize("prepared", [False, True])
def test_iterate_with_recentring(stages, c0_problem, prepared):
    """The optional re-centring (not in the reference): every update subtracts the centre the
    embedding had before the step.  Against the oracle's loop with the same rule, from a start
    that sits far off the origin; the centre then stays at the size of one step's mean movement,
    and without the option the offset start just stays where it is."""
    c = c0_problem
    n = c["X"].shape[0]
    y0 = c["y0"].copy()
    y0[:n] += np.float32(3e-3)
    y0[n:] -= np.float32(2e-3)
    y_o, z_o = oracle.iterate(c["P"], c["idx"], y0, 6, recenter=True)
    plan = stages.Plan(n, c["K"])
    plan.set_recenter(True)
    dP, di = dev(c["P"]), dev(c["idx"])
    if prepared:
        plan.prepare_attractive(dP, di)
    dy = dev(y0)
    gains, old = torch.ones_like(dy), torch.zeros_like(dy)
    z = plan.iterate_(None if prepared else dP, None if prepared else di, dy, gains, old, 0, 6)
    y = dy.cpu().numpy()
    assert rel_l2(y, y_o) <= 1e-4
    assert abs(float(z.item()) - z_o) <= 1e-4 * abs(z_o)
    extent = float(y.max() - y.min())
    assert abs(y[:n].mean()) <= 1e-2 * extent and abs(y[n:].mean()) <= 1e-2 * extent
    # the centre is a sum over workgroups taken in a fixed order: a second run ends on the same bits
    dy2 = dev(y0)
    gains2, old2 = torch.ones_like(dy2), torch.zeros_like(dy2)
    plan.iterate_(None if prepared else dP, None if prepared else di, dy2, gains2, old2, 0, 6)
    assert same_bits(dy2.cpu().numpy(), y)
    # the same start without the option keeps its offset (and follows the oracle's plain loop)
    plan.set_recenter(False)
    dy = dev(y0)
    gains, old = torch.ones_like(dy), torch.zeros_like(dy)
    plan.iterate_(None if prepared else dP, None if prepared else di, dy, gains, old, 0, 6)
    y_plain, _ = oracle.iterate(c["P"], c["idx"], y0, 6)
    assert rel_l2(dy.cpu().numpy(), y_plain) <= 1e-4
    assert abs(float(dy[:n].mean()) - 3e-3) <= 3e-4
    plan.close()


def test_grid_size_changes_between_steps(stages, c0_problem):
    """The plan's interpolation grid can change between steps (the adaptive rule the reference carries
    as a comment, src/fit_tsne.cu:435): after every change the repulsive forces and fused steps follow the
    oracle run with that grid size - growing, shrinking (nothing of the larger grid may leak into the
    smaller one) and back to the reference's 130."""
    c = c0_problem
    n = c["X"].shape[0]
    rng = np.random.default_rng(21)
    y = (rng.standard_normal(2 * n) * 20).astype(np.float32)
    plan = stages.Plan(n, c["K"])
    dy = dev(y)
    for nb in (130, 150, 36, 170, 130):
        plan.set_boxes(nb)
        rep, z, w, yt, phi = plan.repulsive(dy, details=True)
        rep_o, z_o, w_o, yt_o, phi_o = oracle.repulsive(y, nb=nb, details=True)
        assert w.shape == w_o.shape
        assert rel_l2(rep.cpu().numpy(), rep_o) <= 1e-4, nb
        # At this spread z_i = (1 + r^2) phi_1 - 2 (x phi_2 + y phi_3) + phi_4 cancels some forty-fold, and the fp32
        # transforms leave 1e-7 (phi_1..3) to 1e-6 (phi_4) of a plane's norm against the oracle's double-precision
        # convolution: Z lands 1e-6 to 2e-5 from the oracle's, whichever transform length the grid gets (it enters
        # the repulsive gradient, whose bar is 1e-4, as a factor).
        assert abs(float(z) - z_o) <= 3e-5 * abs(z_o), nb
        assert max(np.abs(yt.cpu().numpy().reshape(-1, 4)[:, t] - np.asarray(yt_o).reshape(-1, 4)[:, t]).max() /
                   np.abs(np.asarray(yt_o).reshape(-1, 4)[:, t]).max() for t in range(4)) <= 5e-6, nb
    dP, di = dev(c["P"]), dev(c["idx"])
    plan.prepare_attractive(dP, di)
    y0 = c["y0"]
    dy = dev(y0)
    gains, old = torch.ones_like(dy), torch.zeros_like(dy)
    plan.iterate_(None, None, dy, gains, old, 0, 4)          # captured or not: 130 boxes
    plan.set_boxes(140)
    plan.iterate_(None, None, dy, gains, old, 4, 8)          # the same steps must not replay the old grid
    g_h, o_h = np.ones(2 * n, np.float32), np.zeros(2 * n, np.float32)
    y_o, _ = oracle.iterate(c["P"], c["idx"], y0, 4, gains=g_h, old_forces=o_h)
    y_o, _ = oracle.iterate(c["P"], c["idx"], y_o, 4, step_begin=4, gains=g_h, old_forces=o_h, nb=140)
    assert rel_l2(dy.cpu().numpy(), y_o) <= 1e-4
    with pytest.raises(RuntimeError, match="n_boxes_per_dim must be"):
        plan.set_boxes(171)
    plan.close()
    # the rule: 125 boxes at least -> 130 in the reference's list; one box per unit of spread above that
    assert [stages.boxes_for_spread(s) for s in (0.0, 10.0, 125.0, 130.0, 130.5, 140.0, 149.9, 150.1, 1e6,
                                                 float("nan"))] == [130, 130, 130, 130, 140, 140, 150, 170, 170, 130]


def test_convolution_forms(stages, c0_problem, monkeypatch):
    """The repulsive convolution runs on 800-point transforms where the padded grid fits (up to 133 boxes) and on
    1024-point ones otherwise, and its column pass keeps the kernel's columns in LDS beside the data or in
    registers: the two column passes give the same bits at either length, the two lengths the same node
    potentials to fp32 round-off, and every form follows the oracle."""
    c = c0_problem
    n = c["X"].shape[0]
    rng = np.random.default_rng(77)
    y = (rng.standard_normal(2 * n) * 6).astype(np.float32)
    rep_o, z_o, _, yt_o, _ = oracle.repulsive(y, nb=130, details=True)
    yt_o = np.asarray(yt_o).reshape(-1, 4)
    plan = stages.Plan(n, c["K"])
    got = {}
    for fft in ("800", "1024"):
        for slim in ("0", "1"):
            monkeypatch.setenv("TSNE_FFT", fft)
            monkeypatch.setenv("TSNE_SLIM_COLUMNS", slim)
            rep, z, _, yt, _ = plan.repulsive(dev(y), details=True)
            got[fft, slim] = (rep.cpu().numpy(), float(z), yt.cpu().numpy().reshape(-1, 4))
            assert rel_l2(got[fft, slim][0], rep_o) <= 1e-4, (fft, slim)
            assert abs(got[fft, slim][1] - z_o) <= 1e-5 * abs(z_o), (fft, slim)
    for fft in ("800", "1024"):
        assert same_bits(got[fft, "0"][0], got[fft, "1"][0]) and got[fft, "0"][1] == got[fft, "1"][1], fft
        assert same_bits(got[fft, "0"][2], got[fft, "1"][2]), fft
    assert not same_bits(got["800", "0"][2], got["1024", "0"][2])   # (the switch did switch)
    for t in range(4):
        scale = np.abs(yt_o[:, t]).max()
        assert np.abs(got["800", "0"][2][:, t] - got["1024", "0"][2][:, t]).max() <= 4e-6 * scale, t
        assert np.abs(got["800", "0"][2][:, t] - yt_o[:, t]).max() <= 4e-6 * scale, t
    plan.close()


@pytest.mark.parametrize("n,d,k,perp", [
    (2, 2, 2, 1.5),         # smallest problem: self plus one neighbour
    (50, 3, 50, 10.0),      # K == N, fewer points than one candidate tile
    (333, 130, 17, 5.0),    # ragged sizes, more dimensions than one staging chunk
    (1000, 7, 300, 60.0),   # wide rows: 64 lanes x 8 values in the perplexity search
    (700, 5, 1, 1.0),       # K == 1: only self
    (1300, 20, 1100, 300.0),  # K > 1024: generic row kernels
])
def test_one_shot_stages_edge_shapes(stages, n, d, k, perp):
    from tsnecuda import synthetic
    X = synthetic.gaussian_clusters(n, d=d, clusters=2, center_scale=2.0, seed=n)
    idx_o, d2_o = oracle.knn(X, k)
    idx, d2 = stages.knn(dev(X), k)
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(d2.cpu().numpy(), d2_o)
    if k == 1:
        return
    dn_o, _ = oracle.max_normalize(d2_o)
    dn = stages.max_normalize_(d2)
    assert np.array_equal(dn.cpu().numpy(), dn_o)
    p_o, beta_o, _ = oracle.perplexity(dn_o, perp, 1e-4, return_search=True)
    p, beta = stages.perplexity(dn, perp, 1e-4, return_betas=True)
    # every kernel variant (16 / 32 / 64 lanes per row, one wave per row) follows the stated order
    assert np.array_equal(beta.cpu().numpy(), beta_o)
    assert np.array_equal(p.cpu().numpy().view(np.uint32), p_o.view(np.uint32))
    P_o = oracle.symmetrize(p_o, idx_o)
    P = stages.symmetrize(dev(p_o), dev(idx_o)).cpu().numpy()
    np.testing.assert_allclose(P, P_o, rtol=1e-6, atol=0)
    # gradient stages on the same pattern
    rng = np.random.default_rng(n)
    y = (rng.standard_normal(2 * n) * 5.0).astype(np.float32)
    plan = stages.Plan(n, k)
    got = plan.attractive(dev(P_o), dev(idx_o), dev(y)).cpu().numpy()
    assert rel_l2(got, oracle.attractive(P_o, idx_o, y)) <= 1e-4
    rep, z = plan.repulsive(dev(y))
    rep_o, z_o, _, _, phi_o = oracle.repulsive(y, details=True)
    # rep = x*phi1 - phi2 cancels; with a handful of far-apart points the two
    # terms are orders of magnitude larger than their difference, so the fp32
    # noise of the transforms (~1e-6 of the terms) is what bounds the error.
    terms = np.concatenate([y[:n] * phi_o[:, 0], phi_o[:, 1], y[n:] * phi_o[:, 0], phi_o[:, 2]])
    cond = np.linalg.norm(terms) / np.linalg.norm(rep_o)
    assert rel_l2(rep.cpu().numpy(), rep_o) <= max(1e-4, 2e-6 * cond)
    # Z = sum_i z_i - N: the subtraction cancels when there are only a few far-apart points.
    assert abs(float(z.item()) - z_o) <= 1e-4 * (abs(z_o) + n)
    plan.close()


def test_knn_duplicates_and_ties(stages):
    # Exact duplicates: ties broken by lower index, self still first.
    X = np.zeros((300, 4), np.float32)
    X[100:] = 1.0
    X[200:] = np.float32(2.5)
    idx_o, d2_o = oracle.knn(X, 120)
    idx, d2 = stages.knn(dev(X), 120)
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(d2.cpu().numpy(), d2_o)


def test_repulsive_error_monitor(stages):
    """tsne_hip_repulsive_error: the interpolated forces against exact O(N m) sums on sampled
    points.  With every point sampled, its two figures must be what numpy finds for the forces
    and potentials the stage itself returns; a sample gives a similar figure."""
    rng = np.random.default_rng(21)
    n = 2500
    y = np.concatenate([rng.standard_normal(n) * 6.0, rng.standard_normal(n) * 4.0 + 1.0]).astype(np.float32)
    plan = stages.Plan(n, 8)
    rep, z, w, yt, phi = plan.repulsive(dev(y), details=True)
    rep, phi = rep.cpu().numpy().astype(np.float64), phi.cpu().numpy().astype(np.float64)
    x64, y64 = y[:n].astype(np.float64), y[n:].astype(np.float64)
    dx, dy = x64[:, None] - x64[None, :], y64[:, None] - y64[None, :]
    q = 1.0 / (1.0 + dx * dx + dy * dy)
    exact = np.concatenate([(dx * q * q).sum(1), (dy * q * q).sum(1)])
    z_exact = (q.sum(1) - 1.0).sum()
    z_interp = ((1 + x64 ** 2 + y64 ** 2) * phi[:, 0] - 2 * (x64 * phi[:, 1] + y64 * phi[:, 2]) + phi[:, 3] - 1.0).sum()
    f_err, z_err, m = plan.repulsive_error(dev(y), n)
    assert m == n
    assert abs(f_err - np.linalg.norm(rep - exact) / np.linalg.norm(exact)) <= 1e-6
    assert abs(z_err - abs(z_interp - z_exact) / z_exact) <= 1e-6
    assert 1e-6 < f_err < 5e-2 and z_err < 1e-2  # the scheme's own error: three nodes per box
    f_s, z_s, m_s = plan.repulsive_error(dev(y), 400)
    assert m_s == 400 and 0.2 * f_err < f_s < 5 * f_err
    plan.close()


@pytest.mark.parametrize("nb", [4, 7, 33])
def test_repulsive_reduced_grids(stages, nb):
    """Other grid sizes than the reference's 130 boxes, against the oracle's
    direct (no FFT) node-to-node sums where those are affordable."""
    rng = np.random.default_rng(nb)
    n = 900
    y = (rng.standard_normal(2 * n) * 2.0).astype(np.float32)
    plan = stages.Plan(n, 8, n_boxes_per_dim=nb)
    rep, z, w, yt, phi = plan.repulsive(dev(y), details=True)
    rep_o, z_o, w_o, yt_o, phi_o = oracle.repulsive(y, nb=nb, direct=(nb <= 7), details=True)
    assert rel_l2(w.cpu().numpy(), w_o) <= 1e-5
    assert rel_l2(yt.cpu().numpy(), yt_o) <= 2e-5
    assert rel_l2(rep.cpu().numpy(), rep_o) <= 1e-4
    assert abs(float(z.item()) - z_o) <= 1e-5 * abs(z_o)
    plan.close()


def test_golden_small256(stages):
    """The committed 256-point fixture, stage by stage through the C ABI."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small256.npz"))
    k = g["idx"].shape[1]
    idx, d2 = stages.knn(dev(g["X"]), k)
    assert np.array_equal(idx.cpu().numpy(), g["idx"]) and np.array_equal(d2.cpu().numpy(), g["d2"])
    p, beta = stages.perplexity(stages.max_normalize_(d2), float(g["perplexity"]), 1e-4, return_betas=True)
    assert np.array_equal(beta.cpu().numpy(), g["beta"])
    assert np.array_equal(p.cpu().numpy(), g["p"])
    np.testing.assert_allclose(stages.symmetrize(dev(g["p"]), dev(g["idx"])).cpu().numpy(), g["P"], rtol=1e-6)
    plan = stages.Plan(256, k)
    dy = dev(g["y"])
    attr = plan.attractive(dev(g["P"]), dev(g["idx"]), dy)
    rep, z = plan.repulsive(dy)
    assert rel_l2(attr.cpu().numpy(), g["attr"]) <= 1e-4
    assert rel_l2(rep.cpu().numpy(), g["rep"]) <= 1e-4
    assert abs(float(z.item()) - float(g["z"])) <= 1e-5 * float(g["z"])
    gains, old = torch.ones_like(dy), torch.zeros_like(dy)
    plan.update_(dy, dev(g["attr"]), dev(g["rep"]), gains, old, 200.0, dev(np.array([g["z"]], np.float32)), 0.5, 12.0)
    np.testing.assert_allclose(dy.cpu().numpy(), g["y1"], rtol=1e-6, atol=1e-9)
    assert np.array_equal(gains.cpu().numpy(), g["g1"])
    plan.close()


def test_errors_are_reported(stages):
    with pytest.raises(RuntimeError, match="exceeds num_points"):
        stages.knn(dev(np.zeros((5, 2), np.float32)), 9)
    with pytest.raises(RuntimeError, match="n_boxes_per_dim"):
        stages.Plan(100, 5, n_boxes_per_dim=1000)
    # neighbour numbers that name no point are refused by the stages that build addresses from them
    idx = np.tile(np.arange(4, dtype=np.int32), (300, 1))
    p = np.full((300, 4), 0.25, np.float32)
    for bad in (300, -1):
        idx_bad = idx.copy()
        idx_bad[17, 2] = bad
        with pytest.raises(RuntimeError, match="outside"):
            stages.symmetrize_full(dev(p), dev(idx_bad))
        plan = stages.Plan(300, 4)
        with pytest.raises(RuntimeError, match="outside"):
            plan.prepare_attractive(dev(p), dev(idx_bad))
        plan.close()


@pytest.mark.parametrize("n,k", [(5000, 90), (20000, 30), (9000, 7), (300, 300), (150000, 12), (1100000, 5)])
def test_attractive_blocked_pattern(stages, monkeypatch, n, k):
    """The re-blocked (row strip x column partition) copy of the pattern gives
    the same forces as the oracle; 20000 and 9000 points span several column
    partitions, 300 x 300 is a dense pattern in a single bucket, 150000 x 12
    gives every strip several work items with dozens of partition runs in
    each (74 partitions, ~95 entries per run), 1100000 x 5 spans three column
    windows of the direct form and has more strips than the device compute units.
    Both forms of the step kernel (partitions staged in LDS; neighbours gathered
    from memory) and the one the library picks by itself: the sums are integer
    sums of the same terms, so all three give the same bits."""
    rng = np.random.default_rng(n + k)
    if n <= 20000:
        idx = np.stack([rng.permutation(n)[:k] for _ in range(n)]).astype(np.int32)
    else:  # (a row may name a column twice: the forces just add)
        idx = rng.integers(0, n, (n, k)).astype(np.int32)
    idx[:, 0] = np.arange(n)
    P = (rng.random((n, k)) * 1e-5).astype(np.float32)
    P[:, 0] = 0.0
    y = (rng.standard_normal(2 * n) * 8.0).astype(np.float32)
    want = oracle.attractive(P, idx, y)
    results = {}
    for form in ("staged", "direct", None):
        if form:
            monkeypatch.setenv("TSNE_ATTRACTIVE_FORM", form)
        else:
            monkeypatch.delenv("TSNE_ATTRACTIVE_FORM")
        plan = stages.Plan(n, k)
        plan.prepare_attractive(dev(P), dev(idx))
        got = plan.attractive(None, None, dev(y)).cpu().numpy()
        assert rel_l2(got, want) <= 1e-4, form
        # integer accumulation: the result does not depend on the order of the additions
        again = plan.attractive(None, None, dev(y)).cpu().numpy()
        assert np.array_equal(got, again)
        plan.close()
        results[form] = got
    assert np.array_equal(results["staged"], results["direct"]) and np.array_equal(results["staged"], results[None])


def test_attractive_wait_that_runs_out_is_reported(stages, monkeypatch):
    """The two roles of the re-blocked attractive kernel wait for each other with
    bounded polls.  With the limit forced to zero from the host every wait runs
    out at once: the kernel still ends normally, the forces are NaN and the plan
    reports it once; a plan prepared without the override is unaffected."""
    n, k = 20000, 30
    rng = np.random.default_rng(77)
    idx = rng.integers(0, n, (n, k)).astype(np.int32)
    P = (rng.random((n, k)) * 1e-5).astype(np.float32)
    y = (rng.standard_normal(2 * n) * 8.0).astype(np.float32)
    monkeypatch.setenv("TSNE_ATTRACTIVE_SPIN_LIMIT", "0")
    monkeypatch.setenv("TSNE_ATTRACTIVE_FORM", "staged")  # (the form with the two roles)
    plan = stages.Plan(n, k)
    plan.prepare_attractive(dev(P), dev(idx))
    got = plan.attractive(None, None, dev(y)).cpu().numpy()
    assert np.isnan(got).all()
    with pytest.raises(RuntimeError, match="timed out"):
        plan.check()
    plan.check()  # the report was cleared
    plan.close()
    monkeypatch.delenv("TSNE_ATTRACTIVE_SPIN_LIMIT")
    plan = stages.Plan(n, k)
    plan.prepare_attractive(dev(P), dev(idx))
    got = plan.attractive(None, None, dev(y)).cpu().numpy()
    assert rel_l2(got, oracle.attractive(P, idx, y)) <= 1e-4
    plan.check()
    plan.close()


def test_iterate_after_preparing_a_second_pattern(stages, c0_problem, monkeypatch):
    """Steps replay captured graphs, which hold the addresses of the re-blocked
    pattern: preparing another pattern in the same plan must drop them.  The
    second run has to follow the second pattern, like a fresh plan does.
    (Problems of this size run without graphs and on one stream unless told otherwise.)"""
    monkeypatch.setenv("TSNE_GRAPH", "1")
    monkeypatch.setenv("TSNE_OVERLAP", "1")
    c = c0_problem
    n, k = c["P"].shape
    dP, di = dev(c["P"]), dev(c["idx"])
    rng = np.random.default_rng(9)
    P2 = (c["P"] * rng.uniform(0.5, 1.5, c["P"].shape)).astype(np.float32)

    def run(plan, first):
        if first:
            plan.prepare_attractive(dP, di)
            y = dev(c["y0"]).clone()
            plan.iterate_(None, None, y, torch.ones_like(y), torch.zeros_like(y), 0, 6, eta=200.0)
        plan.prepare_attractive(dev(P2), di)
        y = dev(c["y0"]).clone()
        gains, old = torch.ones_like(y), torch.zeros_like(y)
        plan.iterate_(None, None, y, gains, old, 0, 6, eta=200.0)
        torch.cuda.synchronize()
        return y.cpu().numpy()

    plan_a, plan_b = stages.Plan(n, k), stages.Plan(n, k)
    twice, once = run(plan_a, True), run(plan_b, False)
    plan_a.close()
    plan_b.close()
    assert rel_l2(twice, once) <= 1e-5


@pytest.mark.parametrize("graph, overlap", [("1", "1"), ("0", "1"), ("0", "0")])
def test_plan_closed_or_reprepared_while_steps_are_in_flight(stages, c0_problem, monkeypatch, graph, overlap):
    """iterate_ returns while its steps (a replaying graph, eager steps on two streams, or on one) still run.
    Closing the plan, or preparing another pattern in it, right away - no synchronisation in
    between - must wait for them: the embedding ends where a synchronised run ends."""
    monkeypatch.setenv("TSNE_GRAPH", graph)
    monkeypatch.setenv("TSNE_OVERLAP", overlap)
    c = c0_problem
    n, k = c["P"].shape
    dP, di = dev(c["P"]), dev(c["idx"])

    def run(after):
        plan = stages.Plan(n, k)
        plan.prepare_attractive(dP, di)
        y = dev(c["y0"]).clone()
        gains, old = torch.ones_like(y), torch.zeros_like(y)
        plan.iterate_(None, None, y, gains, old, 0, 40)
        after(plan)
        torch.cuda.synchronize()
        return y.cpu().numpy()

    def sync_then_close(plan):
        torch.cuda.synchronize()
        plan.close()

    def reprepare(plan):
        plan.prepare_attractive(dP, di)
        plan.close()

    want = run(sync_then_close)
    assert np.isfinite(want).all()
    assert same_bits(run(lambda plan: plan.close()), want)
    assert same_bits(run(reprepare), want)


def test_prepare_reports_unsupported_shapes_apart_from_failures(stages):
    """A pattern the blocked format cannot hold (num_neighbors >= 4096) is status 2, which
    callers may answer by keeping the row-ordered kernel; the plan goes on working with an
    explicit pattern."""
    n, k = 4200, 4100
    rng = np.random.default_rng(3)
    idx = rng.integers(0, n, (n, k)).astype(np.int32)
    P = (rng.random((n, k)) * 1e-6).astype(np.float32)
    y = (rng.standard_normal(2 * n) * 3.0).astype(np.float32)
    plan = stages.Plan(n, k)
    dP, di = dev(P), dev(idx)
    rc = stages.lib().tsne_hip_attractive_prepare(plan._h, dP.data_ptr(), di.data_ptr(), None)
    assert rc == 2
    assert b"too large for the blocked format" in stages.lib().tsne_hip_last_error()
    got = plan.attractive(dP, di, dev(y)).cpu().numpy()
    assert rel_l2(got, oracle.attractive(P, idx, y)) <= 1e-4
    plan.close()


def test_attractive_blocked_clustered_pattern(stages):
    """A pattern whose rows reference only a few column partitions (what the
    locality ordering produces): runs longer than one work item share a staged
    partition, other partitions are skipped."""
    n, k = 40000, 60
    rng = np.random.default_rng(5)
    block = np.arange(n) // 10000  # four blocks of 10000 points
    idx = (block[:, None] * 10000 + rng.integers(0, 10000, (n, k))).astype(np.int32)
    idx[:, 0] = np.arange(n)
    P = (rng.random((n, k)) * 1e-5).astype(np.float32)
    P[:, 0] = 0.0
    y = (rng.standard_normal(2 * n) * 8.0).astype(np.float32)
    want = oracle.attractive(P, idx, y)
    plan = stages.Plan(n, k)
    plan.prepare_attractive(dev(P), dev(idx))
    got = plan.attractive(None, None, dev(y)).cpu().numpy()
    assert rel_l2(got, want) <= 1e-4
    plan.close()


def test_locality_order(stages):
    """The renumbering is a permutation, deterministic, and groups clustered
    points: along the new order the cluster label changes only a few times."""
    from tsnecuda import synthetic
    n = 40000
    X = synthetic.gaussian_clusters(n, d=20, clusters=4, seed=3)
    a = stages.locality_order(dev(X)).cpu().numpy()
    b = stages.locality_order(dev(X)).cpu().numpy()
    assert np.array_equal(a, b)
    assert np.array_equal(np.sort(a), np.arange(n))
    labels = (a % 4)  # gaussian_clusters: label = index mod clusters
    changes = int((labels[1:] != labels[:-1]).sum())
    assert changes <= 63, changes  # (pivot count) - 1 at the very most: every cell is one cluster
    Xs = stages.gather_rows(dev(X), dev(a.astype(np.int32))).cpu().numpy()
    assert np.array_equal(Xs, X[a])
    # small inputs keep their numbering
    small = stages.locality_order(dev(X[:1000])).cpu().numpy()
    assert np.array_equal(small, np.arange(1000))


def test_iterate_with_prepared_pattern(stages, c0_problem):
    c = c0_problem
    n = c["X"].shape[0]
    y_o, z_o = oracle.iterate(c["P"], c["idx"], c["y0"], 5)
    plan = stages.Plan(n, c["K"])
    plan.prepare_attractive(dev(c["P"]), dev(c["idx"]))
    dy = dev(c["y0"])
    gains, old = torch.ones_like(dy), torch.zeros_like(dy)
    z = plan.iterate_(None, None, dy, gains, old, 0, 5)
    assert rel_l2(dy.cpu().numpy(), y_o) <= 1e-4
    assert abs(float(z.item()) - z_o) <= 1e-4 * abs(z_o)
    plan.close()
    with pytest.raises(RuntimeError, match="none prepared"):
        stages.Plan(n, c["K"]).iterate_(None, None, dy, gains, old, 0, 1)


@pytest.mark.parametrize("n,d,k", [
    (3000, 50, 90),    # the benchmark's shape at small N
    (700, 7, 20),      # odd dimension count, fewer candidates than the K' margin wants
    (1500, 126, 33),   # the largest dimension count one wave's registers hold (products on floats)
    (1500, 125, 33),   # the largest on bf16 terms (8 steps of 16 dimensions, the last three carry beta)
    (1300, 13, 25),    # bf16: one step, beta in its last three dimensions
    (1300, 14, 25),    # bf16: beta straddles two steps
    (1400, 61, 30),    # bf16: four full steps
    (1400, 62, 30),    # bf16: five steps (one workgroup per compute unit)
    (1400, 40, 30),    # bf16: three steps
    (1400, 90, 30),    # bf16: six steps
    (1400, 100, 30),   # bf16: seven steps
    (1400, 1, 10),     # one dimension
    (1500, 127, 33),   # the first that is cut into chunks (3 chunks, the norm row opens the last one)
    (2200, 190, 40),   # 3 chunks, the last one full but for the norm row's partner
    (1200, 784, 50),   # config c1's dimension count (13 chunks)
    (900, 1024, 30),   # config c2's (17 chunks: the norm row has a chunk of its own)
    (745, 864, 126),   # six candidate tiles: fewer than the workgroups a query tile could be split over
    (40, 3, 40),       # K == N, a single partial tile
    (2500, 33, 300),   # wide neighbour lists
    (3000, 20, 1023),  # the reference's default neighbour count: the roomier list size no longer fits the LDS
])
def test_knn_matrix_sweep_is_exact(stages, n, d, k):
    """The MFMA candidate sweep + exact re-rank gives the oracle's neighbours bit
    for bit, and agrees with the vector sweep."""
    from tsnecuda import synthetic
    X = synthetic.gaussian_clusters(n, d=d, clusters=3, center_scale=6.0, seed=n + d)
    idx_o, d2_o = oracle.knn(X, k)
    idx, d2, stats = stages.knn_select(dev(X), k, 2)
    assert stats[0] == 1
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(d2.cpu().numpy(), d2_o)
    idx_v, d2_v, stats_v = stages.knn_select(dev(X), k, 1)
    assert stats_v[0] == 0
    assert torch.equal(idx_v, idx) and torch.equal(d2_v, d2)
    # sweep 2 multiplies bf16 terms (except at 126 dimensions); sweep 3 keeps the products on floats
    idx_f, d2_f, stats_f = stages.knn_select(dev(X), k, 3)
    assert stats_f[0] == 1
    assert torch.equal(idx_f, idx) and torch.equal(d2_f, d2)


@pytest.mark.parametrize("scale,d", [(30.0, 12), (2.5, 6), (0.7, 4), (6.0, 160), (0.3, 140), (10.0, 50), (4.0, 100)])
def test_knn_tile_skipping_is_exact(stages, scale, d):
    """On locality-ordered points both sweeps skip candidate tiles by their
    bounding balls.  Well separated clusters (most tiles skipped), touching
    clusters (the bound decides tile by tile) and one blob (nothing to skip) all
    give the oracle's rows bit for bit, and the two sweeps agree (beyond 126
    dimensions the matrix sweep is the chunked one)."""
    from tsnecuda import synthetic
    n, k = 60000, 40
    X = synthetic.gaussian_clusters(n, d=d, clusters=7, center_scale=scale, seed=int(scale * 10) + d)
    dX = dev(X)
    Xs = stages.gather_rows(dX, stages.locality_order(dX))
    idx_v, d2_v, _ = stages.knn_select(Xs, k, 1)
    for sweep in (2, 3):
        idx, d2, stats = stages.knn_select(Xs, k, sweep)
        assert stats[0] == 1
        assert torch.equal(idx_v, idx) and torch.equal(d2_v, d2)
    Xs_h = Xs.cpu().numpy()
    for first in (0, n // 3, n - 96):
        idx_o, d2_o = oracle.knn(Xs_h, k, rows=(first, first + 96))
        assert np.array_equal(idx_v[first:first + 96].cpu().numpy(), idx_o)
        assert np.array_equal(d2_v[first:first + 96].cpu().numpy(), d2_o)


@pytest.mark.parametrize("n,d,k,nlist,nprobe", [(20000, 16, 30, 141, 20), (9000, 50, 90, 94, 5), (30000, 3, 10, 173, 1), (40000, 50, 90, 200, 60)])
def test_knn_ivf_matches_the_oracle_given_the_centroids(stages, n, d, k, nlist, nprobe):
    """The approximate (inverted-file) search: centroids trained on the GPU, then - the centroids given - the
    search is a deterministic function of the points, which the oracle restates: identical neighbours and
    distances, bit for bit.  Recall against the exact search is reported and bounded."""
    from tsnecuda import synthetic
    X = synthetic.gaussian_clusters(n, d=d, clusters=6, center_scale=4.0, seed=n + d)
    dX = dev(X)
    cen = stages.ivf_train(dX, nlist)
    cen_h = cen.cpu().numpy()
    assert cen_h.shape == (nlist, d) and np.isfinite(cen_h).all()
    # trained centroids describe the data better than the points they started from would: every list is used
    idx, d2, stats = stages.knn_ivf(dX, k, cen, nprobe)
    assert stats[0] == 1 and stats[1] == 0  # matrix sweep, no query answered by the exact fallback
    idx_o, d2_o, list_of, probes = oracle.knn_ivf(X, k, cen_h, nprobe, return_probes=True)
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(d2.cpu().numpy().view(np.uint32), d2_o.view(np.uint32))
    assert np.unique(list_of).size > 0.8 * nlist
    exact, _ = stages.knn(dX, k)
    exact = exact.cpu().numpy()
    got = idx.cpu().numpy()
    recall = np.mean([len(np.intersect1d(got[i, 1:], exact[i, 1:])) for i in range(0, n, 7)]) / (k - 1)
    print("knn_ivf n=%d d=%d nlist=%d nprobe=%d: recall %.4f, %d per mille of the tile pairs" % (n, d, nlist, nprobe,
                                                                                                recall, stats[2]))
    assert recall > (0.6 if nprobe >= 5 else 0.4)


def test_knn_ivf_argument_errors(stages):
    X = dev(np.random.default_rng(0).standard_normal((9000, 8)).astype(np.float32))
    cen = stages.ivf_train(X, 30)
    with pytest.raises(RuntimeError, match="nprobe must be"):
        stages.knn_ivf(X, 10, cen, 31)
    wide = dev(np.zeros((9000, 200), np.float32))
    with pytest.raises(RuntimeError, match="at most 12"):
        stages.ivf_train(wide, 30)


def test_knn_chunked_sweep_calibrates_its_margin(stages):
    """Pixel-like vectors in 784 dimensions: a query's neighbour distances lie so
    close together that the default margin between neighbour K and candidate K'
    cannot be verified; the chunked sweep finds that out on a sample of query
    tiles, widens K' and then verifies (nearly) every query.  Results are the
    vector sweep's and the oracle's, bit for bit."""
    from tsnecuda import synthetic
    n, k = 20000, 45
    X = synthetic.pixel_like(n=n, d=784)
    dX = dev(X)
    Xs = stages.gather_rows(dX, stages.locality_order(dX))
    idx, d2, stats = stages.knn_select(Xs, k, 0)
    assert stats[0] == 1 and stats[1] <= n // 100
    idx_v, d2_v, _ = stages.knn_select(Xs, k, 1)
    assert torch.equal(idx_v, idx) and torch.equal(d2_v, d2)
    Xs_h = Xs.cpu().numpy()
    for first in (0, n // 2, n - 32):
        idx_o, d2_o = oracle.knn(Xs_h, k, rows=(first, first + 32))
        assert np.array_equal(idx[first:first + 32].cpu().numpy(), idx_o)
        assert np.array_equal(d2[first:first + 32].cpu().numpy(), d2_o)


def test_knn_chunked_sweep_gives_up_on_unverifiable_data(stages):
    """200 dimensions, far from the origin, tiny mutual distances: no margin
    verifies.  Left to choose, kNN notices on the sample and runs the vector
    sweep; forced onto the matrix sweep, every query is repaired by the vector
    sweep afterwards.  Both are exact."""
    rng = np.random.default_rng(5)
    n, d, k = 9000, 200, 20
    base = rng.standard_normal((1, d)).astype(np.float32) * 300.0
    X = (base + rng.standard_normal((n, d)).astype(np.float32) * 1e-2).astype(np.float32)
    idx_a, d2_a, stats_a = stages.knn_select(dev(X), k, 0)
    assert stats_a[0] == 0
    idx_m, d2_m, stats_m = stages.knn_select(dev(X), k, 2)
    assert stats_m[0] == 1 and stats_m[1] > n // 2
    assert torch.equal(idx_a, idx_m) and torch.equal(d2_a, d2_m)
    for first in (0, n - 48):
        idx_o, d2_o = oracle.knn(X, k, rows=(first, first + 48))
        assert np.array_equal(idx_a[first:first + 48].cpu().numpy(), idx_o)
        assert np.array_equal(d2_a[first:first + 48].cpu().numpy(), d2_o)


@pytest.mark.parametrize("sweep", [2, 3])
def test_knn_matrix_sweep_verification_falls_back(stages, sweep):
    """Points far from the origin with tiny mutual distances: neither the
    |c|^2 - 2 q.c distances on floats (sweep 3) nor the bf16 terms relative to the
    tile centres (sweep 2) can separate them, the verification must notice and the
    vector sweep must repair every such query; duplicates tie on index."""
    rng = np.random.default_rng(3)
    base = rng.standard_normal((1, 16)).astype(np.float32) * 300.0
    X = (base + rng.standard_normal((2000, 16)).astype(np.float32) * 1e-2).astype(np.float32)
    X[1000:1100] = X[0:100]  # exact duplicates
    idx_o, d2_o = oracle.knn(X, 25)
    idx, d2, stats = stages.knn_select(dev(X), 25, sweep)
    assert stats[0] == 1 and stats[1] > 0
    assert np.array_equal(idx.cpu().numpy(), idx_o)
    assert np.array_equal(d2.cpu().numpy(), d2_o)


@pytest.mark.parametrize("sweep", [2, 3])
def test_knn_few_failed_queries_are_redone_by_candidate_range(stages, sweep):
    """A clump of 400 nearly identical points: for some of its members the 300th
    neighbour and the sweep's threshold lie closer together than the matrix sweep
    can tell apart, so they fail its verification (95 of them on this seed with the
    products on floats) while
    the other points pass.  The vector sweep takes just those queries, cut over the chip by candidate range and merged
    (K - 1 = 299 keys per range)."""
    rng = np.random.default_rng(11)
    n, d, k = 20000, 16, 300
    X = rng.standard_normal((n, d)).astype(np.float32)
    clump = rng.choice(n, 400, replace=False)
    X[clump] = (rng.standard_normal((1, d)) + rng.standard_normal((400, d)) * 1e-5).astype(np.float32)
    idx, d2, stats = stages.knn_select(dev(X), k, sweep)
    assert stats[0] == 1 and 0 < stats[1] <= 400
    rows = np.concatenate([clump[:80], rng.choice(n, 24, replace=False)])
    for q in rows:
        idx_o, d2_o = oracle.knn(X, k, rows=(int(q), int(q) + 1))
        assert np.array_equal(idx[q].cpu().numpy(), idx_o[0])
        assert np.array_equal(d2[q].cpu().numpy(), d2_o[0])


def test_iterate_graph_replay_matches_eager(stages, c0_problem, monkeypatch):
    """Steps on one stream or two, launched one by one or as replays of a captured graph of two
    steps, with eager work and synchronisations between the calls, give what the plain loop gives
    (bit for bit: the loop's sums are integer sums)."""
    c = c0_problem
    n = c["P"].shape[0]
    dP, di = dev(c["P"]), dev(c["idx"])

    def run(chunks):
        plan = stages.Plan(n, c["K"])
        plan.prepare_attractive(dP, di)
        y = dev(c["y0"]).clone()
        gains, old = torch.ones_like(y), torch.zeros_like(y)
        step = 0
        for k in chunks:
            plan.iterate_(None, None, y, gains, old, step, step + k, eta=200.0)
            step += k
            torch.cuda.synchronize()
            _ = (y * 2.0).sum().item()  # eager work between the replays
        out = y.cpu().numpy()
        plan.close()
        return out

    # (problems of this size run on one stream and without graphs unless told otherwise)
    monkeypatch.setenv("TSNE_GRAPH", "0")
    monkeypatch.setenv("TSNE_OVERLAP", "0")
    eager = run([12])
    oracle_y, _ = oracle.iterate(c["P"], c["idx"], c["y0"], 12)
    for overlap in ("1", "0"):
        monkeypatch.setenv("TSNE_OVERLAP", overlap)
        monkeypatch.setenv("TSNE_GRAPH", "0")
        stepped = run([5, 4, 3])
        monkeypatch.setenv("TSNE_GRAPH", "1")
        replayed = run([5, 4, 3])  # 2 + 2 + 1 replays of the same graph, odd remainders eager
        for got in (stepped, replayed):
            assert np.isfinite(got).all()
            assert same_bits(got, eager)
    assert rel_l2(eager, oracle_y) <= 1e-3


@pytest.mark.parametrize("n_points", [5000, 70000])
def test_loop_is_bit_repeatable(stages, c0_problem, monkeypatch, n_points):
    """Forty steps from one start, run twice in every arrangement of the loop (one stream or two, captured
    graphs or not, the grouping by tile kept across steps or redone every step): one result, bit for bit.  The
    attractive forces, the box moments of the charge spreading and the partial sums of z are all accumulated in
    64-bit fixed point, and nothing else in a step depends on the order of arrival."""
    from tsnecuda import synthetic
    if n_points == 5000:
        c = c0_problem
        P, idx, y0 = c["P"], c["idx"], c["y0"]
    else:
        # 70000 points run on two streams and replay graphs by default; neighbours from a random pattern
        rng = np.random.default_rng(5)
        k = 24
        idx = rng.integers(0, n_points, size=(n_points, k), dtype=np.int32)
        idx[:, 0] = np.arange(n_points)
        P = (rng.random((n_points, k)) / (n_points * k)).astype(np.float32)
        Y0 = synthetic.initial_embedding(n_points, seed=3)
        y0 = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    dP, di = dev(P), dev(idx)

    def run(graph, overlap, keep):
        monkeypatch.setenv("TSNE_GRAPH", graph)
        monkeypatch.setenv("TSNE_OVERLAP", overlap)
        monkeypatch.setenv("TSNE_KEEP_GROUPING", keep)
        plan = stages.Plan(P.shape[0], P.shape[1])
        plan.prepare_attractive(dP, di)
        y = dev(y0).clone()
        gains, old = torch.ones_like(y), torch.zeros_like(y)
        z = plan.iterate_(None, None, y, gains, old, 0, 40)
        torch.cuda.synchronize()
        plan.close()
        return y.cpu().numpy(), gains.cpu().numpy(), old.cpu().numpy(), float(z.item())

    want = run("0", "0", "1")
    assert np.isfinite(want[0]).all()
    for graph, overlap, keep in [("0", "0", "1"), ("0", "1", "1"), ("1", "1", "1"), ("0", "0", "0"), ("1", "1", "0")]:
        got = run(graph, overlap, keep)
        for a, b in zip(got[:3], want[:3]):
            assert same_bits(a, b), (graph, overlap, keep)
        assert got[3] == want[3]
