#!/usr/bin/env python3
"""Regenerates the fixtures in this directory from the CPU oracle.

The reference's own tests hold no golden vectors for this path (its test
sources do not compile), so the fixtures are the oracle's outputs on small
seeded inputs; the oracle itself is pinned by the closed-form / brute-force
checks in tests/test_oracle.py.

  small256.npz   256 x 16 points, K = 16: neighbours, P, forces and one update
                 step from a fixed embedding (a few hundred KB at most)
  c0_fit.json    config c0 (5000 x 50, K = 90, perplexity 30): objective value
                 and trustworthiness of the oracle's 1000-step fit from the seeded
                 initial embedding

  c1_fit.json, c2_fit.json   the same for configs c1 and c2 (trustworthiness on a fixed subsample)

Run from the repository root:  python tests/golden/make_golden.py [small] [c0] [c1] [c2]
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tsne-cuda_amd"))

import oracle  # noqa: E402
from sklearn.manifold import trustworthiness  # noqa: E402
from tsnecuda import synthetic  # noqa: E402


def small_case():
    n, d, k, perp = 256, 16, 16, 5.0
    X = synthetic.gaussian_clusters(n, d=d, clusters=3, center_scale=4.0, seed=7)
    idx, d2 = oracle.knn(X, k)
    dn, dmax = oracle.max_normalize(d2)
    p, beta, iters = oracle.perplexity(dn, perp, 1e-4, return_search=True)
    P = oracle.symmetrize(p, idx)
    Y0 = synthetic.initial_embedding(n, seed=8, scale=1.0)  # unit-scale embedding: non-trivial forces
    y = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    attr = oracle.attractive(P, idx, y)
    rep, z = oracle.repulsive(y)
    gains = np.ones_like(y)
    old = np.zeros_like(y)
    y1, g1, u1 = oracle.update(y, attr, rep, gains, old, 200.0, z, 0.5, 12.0)
    np.savez_compressed(os.path.join(HERE, "small256.npz"), X=X, idx=idx, d2=d2, dn=dn, p=p, beta=beta,
                        iters=iters, P=P, y=y, attr=attr, rep=rep, z=np.float32(z), y1=y1, g1=g1, u1=u1,
                        perplexity=np.float32(perp))


def c0_fit():
    X, fit = synthetic.make_config("c0")
    Y0 = synthetic.initial_embedding(X.shape[0])
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]])
    y, z, idx, P = oracle.fit(X, y0, fit["num_neighbors"], fit["perplexity"], eps=1e-4, iterations=1000,
                              eta=fit["learning_rate"])
    out = {
        "config": "c0: 5000 x 50, K=90, perplexity 30, lr 200, 1000 steps, exaggeration 12 for 250, VECTOR init seed 1",
        "kl_exact_z": oracle.kl(P, idx, y),
        "kl_initial": oracle.kl(P, idx, y0),
        "z_final_interpolated": z,
        "extent": [float(y.min()), float(y.max())],
        "p_sum": float(P.astype(np.float64).sum()),
        # fraction of each point's 12 nearest embedding neighbours that are also near in the input space
        # (sklearn's definition, an independent implementation)
        "trustworthiness_k12": float(trustworthiness(X, np.stack([y[:X.shape[0]], y[X.shape[0]:]], axis=1),
                                                     n_neighbors=12)),
    }
    with open(os.path.join(HERE, "c0_fit.json"), "w") as f:
        json.dump(out, f, indent=1)
    print(out)


def subsample(n, m=4000):
    """The m points on which the larger configs' trustworthiness is evaluated (the full pairwise matrix of
    60000 points does not fit a test)."""
    return np.sort(np.random.default_rng(0).choice(n, size=m, replace=False))


def larger_fit(name):
    """Configs c1 (60000 x 784) and c2 (50000 x 1024): objective and subsample trustworthiness of the
    oracle's 1000-step fit; a few minutes of CPU time each."""
    X, fit = synthetic.make_config(name)
    n = X.shape[0]
    Y0 = synthetic.initial_embedding(n)
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]])
    y, z, idx, P = oracle.fit(X, y0, fit["num_neighbors"], fit["perplexity"], eps=1e-4, iterations=1000,
                              eta=fit["learning_rate"])
    sub = subsample(n)
    emb = np.stack([y[:n], y[n:]], axis=1)
    out = {
        "config": "%s: %d x %d, K=%d, perplexity %g, lr %g, 1000 steps, exaggeration 12 for 250, VECTOR init seed 1"
                  % (name, n, X.shape[1], fit["num_neighbors"], fit["perplexity"], fit["learning_rate"]),
        "kl_exact_z": oracle.kl(P, idx, y),
        "kl_initial": oracle.kl(P, idx, y0),
        "extent": [float(y.min()), float(y.max())],
        "trustworthiness_k12_subsample4000": float(trustworthiness(X[sub], emb[sub], n_neighbors=12)),
    }
    with open(os.path.join(HERE, "%s_fit.json" % name), "w") as f:
        json.dump(out, f, indent=1)
    print(out)


if __name__ == "__main__":
    which = sys.argv[1:] or ["small", "c0", "c1", "c2"]  # c3 (1,000,000 points) only when named: about an hour
    if "small" in which:
        small_case()
    if "c0" in which:
        c0_fit()
    for name in ("c1", "c2", "c3"):
        if name in which:
            larger_fit(name)
