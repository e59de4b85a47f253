"""End-to-end fits through the drop-in entry points on the GPU, against the oracle's fits."""
import json
import os

import numpy as np
import pytest

import oracle

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def flat(emb):
    return np.concatenate([emb[:, 0], emb[:, 1]]).astype(np.float32)


def test_c0_fit_objective_within_one_percent(c0_problem):
    """Config c0, 1000 steps from the seeded initial embedding through
    TSNE.fit_transform (ctypes -> pymodule_tsne -> RunTsne).  Gradient descent
    amplifies fp32 round-off, so trajectories are compared through the objective:
    the KL-style value of the final embedding, evaluated by the same evaluator
    with the oracle's P and exact Z, must be within 1 % of the oracle's own run
    (tests/golden/c0_fit.json)."""
    from tsnecuda import TSNE, synthetic
    c = c0_problem
    with open(os.path.join(GOLDEN, "c0_fit.json")) as f:
        gold = json.load(f)
    Y0 = synthetic.initial_embedding(c["X"].shape[0])
    model = TSNE(perplexity=c["fit"]["perplexity"], num_neighbors=c["K"], learning_rate=c["fit"]["learning_rate"],
                 n_iter=1000, perplexity_epsilon=1e-4)
    emb = model.fit_transform(c["X"], y=Y0)
    assert emb.shape == (5000, 2) and emb.dtype == np.float32 and emb.flags["F_CONTIGUOUS"]
    assert np.isfinite(emb).all()
    kl = oracle.kl(c["P"], c["idx"], flat(emb))
    print("KL gpu %.5f oracle %.5f initial %.5f" % (kl, gold["kl_exact_z"], gold["kl_initial"]))
    assert abs(kl - gold["kl_exact_z"]) <= 0.01 * gold["kl_exact_z"]
    # the library's own evaluation of the same embedding (interpolated Z, its own P) agrees with the
    # oracle's evaluator (exact Z, oracle P)
    assert abs(model.kl_divergence_ - kl) <= 2e-3 * kl
    # same overall scale of the layout
    assert 0.8 < (emb.max() - emb.min()) / (gold["extent"][1] - gold["extent"][0]) < 1.25
    # and the same neighbourhood preservation, by an implementation that shares nothing with this build
    from sklearn.manifold import trustworthiness
    t = trustworthiness(c["X"], emb, n_neighbors=12)
    print("trustworthiness gpu %.4f oracle %.4f" % (t, gold["trustworthiness_k12"]))
    assert abs(t - gold["trustworthiness_k12"]) <= 0.01


@pytest.mark.parametrize("name", ["c1", "c2"])
def test_larger_configs_objective_within_one_percent(name):
    """Configs c1 (60000 x 784 pixel-like) and c2 (50000 x 1024 feature-like), 1000
    steps from the seeded start: the objective of the final embedding (exact Z,
    evaluated by the oracle on the neighbours and P of the GPU stages, which are
    compared with the oracle's elsewhere) within 1 % of the oracle's own run, and
    the trustworthiness of a fixed 4000-point subsample within 0.02 of it
    (tests/golden/c1_fit.json, c2_fit.json)."""
    from sklearn.manifold import trustworthiness
    from tsnecuda import TSNE, stages, synthetic
    with open(os.path.join(GOLDEN, "%s_fit.json" % name)) as f:
        gold = json.load(f)
    X, fit = synthetic.make_config(name)
    n, k = X.shape[0], fit["num_neighbors"]
    Y0 = synthetic.initial_embedding(n)
    model = TSNE(perplexity=fit["perplexity"], num_neighbors=k, learning_rate=fit["learning_rate"], n_iter=1000,
                 perplexity_epsilon=1e-4)
    emb = model.fit_transform(X, y=Y0)
    assert emb.shape == (n, 2) and np.isfinite(emb).all()
    idx, d2 = stages.knn(torch.from_numpy(X).cuda(), k)
    P = stages.symmetrize(stages.perplexity(stages.max_normalize_(d2), fit["perplexity"], 1e-4), idx)
    kl = oracle.kl(P.cpu().numpy(), idx.cpu().numpy(), flat(emb))
    sub = np.sort(np.random.default_rng(0).choice(n, size=4000, replace=False))  # as tests/golden/make_golden.py
    t = trustworthiness(X[sub], emb[sub], n_neighbors=12)
    print("%s: KL gpu %.5f oracle %.5f (library's own %.5f), trustworthiness gpu %.4f oracle %.4f"
          % (name, kl, gold["kl_exact_z"], model.kl_divergence_, t, gold["trustworthiness_k12_subsample4000"]))
    assert abs(kl - gold["kl_exact_z"]) <= 0.01 * gold["kl_exact_z"]
    assert abs(model.kl_divergence_ - kl) <= 5e-3 * kl
    assert abs(t - gold["trustworthiness_k12_subsample4000"]) <= 0.02
    assert 0.8 < (emb.max() - emb.min()) / (gold["extent"][1] - gold["extent"][0]) < 1.25


def test_fit_is_repeatable_for_a_given_start(c0_problem):
    """Two fits from the same start give the same embedding, bit for bit: the one-shot stages are exact or
    evaluated in a fixed order, and every accumulation of the gradient loop whose order of arrival varies
    (attractive forces, box moments of the charge spreading, partial sums of z) is an integer sum."""
    from tsnecuda import TSNE, synthetic
    for n, steps in ((2000, 300), (20000, 60)):
        X = c0_problem["X"][:n] if n <= 5000 else synthetic.gaussian_clusters(n, d=20, clusters=6, seed=2)
        Y0 = synthetic.initial_embedding(n, seed=9)
        kw = dict(perplexity=20.0, num_neighbors=60, n_iter=steps, perplexity_epsilon=1e-4)
        a = TSNE(**kw).fit_transform(X, y=Y0)
        b = TSNE(**kw).fit_transform(X, y=Y0)
        assert np.isfinite(a).all()
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_renumbering_is_invisible_to_the_caller(monkeypatch):
    """RunTsne renumbers 16384 or more points in locality order on entry and
    restores the caller's numbering on exit: a short fit gives the same
    embedding, row for row, with the renumbering switched off."""
    from tsnecuda import TSNE, synthetic
    n = 20000
    X = synthetic.gaussian_clusters(n, d=16, clusters=5, seed=11)
    Y0 = synthetic.initial_embedding(n, seed=4)
    kw = dict(perplexity=20.0, num_neighbors=60, n_iter=15, perplexity_epsilon=1e-4)
    monkeypatch.setenv("TSNE_LOCALITY_ORDER", "1")
    a = TSNE(**kw).fit_transform(X, y=Y0)
    snaps = TSNE(return_style="snapshots", num_snapshots=3, **kw).fit_transform(X, y=Y0)
    monkeypatch.setenv("TSNE_LOCALITY_ORDER", "0")
    b = TSNE(**kw).fit_transform(X, y=Y0)
    assert np.linalg.norm(a - b) <= 1e-3 * np.linalg.norm(b)
    assert np.linalg.norm(snaps[-1] - b) <= 1e-3 * np.linalg.norm(b)
    # the first snapshot is the embedding after one step: still close to the start, row for row
    assert np.abs(snaps[0] - Y0).max() < 1e-2


@pytest.mark.parametrize("n,d,k,clusters,perp", [
    (16385, 7, 30, 3, 18.0),    # just above the renumbering threshold, odd count (scalar update kernel)
    (20001, 3, 90, 1, 30.0),    # one blob: nothing for the kNN sweep to skip
    (8192, 126, 16, 4, 9.0),    # smallest matrix-sweep problem, largest matrix-sweep dimension
    (8195, 127, 16, 4, 9.0),    # one dimension more: chunked matrix sweep
    (17000, 300, 30, 5, 18.0),  # chunked matrix sweep on renumbered points, margin tried on a sample of query tiles
    (40000, 50, 40, 6, 24.0),   # several column partitions and strips, clustered
    (12000, 10, 1023, 3, 30.0),  # the neighbour count of the reference's C++ default options
    (9000, 50, 90, 4, 2.0),     # a perplexity far below the neighbour count: subnormal probabilities, rows at the
                                # search's cap of 200 evaluations
])
def test_whole_pipeline_against_the_oracle(n, d, k, clusters, perp):
    """RunTsne end to end (renumbering, kNN, P, eight gradient steps, numbering
    restored) against the oracle's pipeline from the same explicit start, row
    for row."""
    from tsnecuda import TSNE, synthetic
    X = synthetic.gaussian_clusters(n, d=d, clusters=clusters, center_scale=5.0, seed=n + d)
    Y0 = synthetic.initial_embedding(n, seed=k)
    emb = TSNE(perplexity=perp, num_neighbors=k, n_iter=8, perplexity_epsilon=1e-4).fit_transform(X, y=Y0)
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    y_o, _, _, _ = oracle.fit(X, y0, k, perp, eps=1e-4, iterations=8)
    got = flat(emb)
    assert np.isfinite(got).all()
    err = np.linalg.norm(got - y_o) / np.linalg.norm(y_o)
    print("n=%d d=%d k=%d perplexity %g: embedding after 8 steps against the oracle's %.2e" % (n, d, k, perp, err))
    assert err <= 2e-3
