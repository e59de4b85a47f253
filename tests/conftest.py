import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tsne-cuda_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def c0_problem():
    """Config c0 (5000 x 50, K=90, perplexity 30) taken through the oracle's
    one-shot stages; shared by the CPU and GPU tests."""
    import numpy as np
    import oracle
    from tsnecuda import synthetic
    X, fit = synthetic.make_config("c0")
    K = fit["num_neighbors"]
    idx, d2 = oracle.knn(X, K)
    dn, dmax = oracle.max_normalize(d2)
    p, beta, iters = oracle.perplexity(dn, fit["perplexity"], 1e-4, return_search=True)
    P = oracle.symmetrize(p, idx)
    Y0 = synthetic.initial_embedding(X.shape[0])
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    return dict(X=X, K=K, idx=idx, d2=d2, dn=dn, dmax=dmax, p=p, beta=beta, iters=iters, P=P, y0=y0, fit=fit)
