"""tsnecuda for MI355X: FIt-SNE on hand-written HIP kernels behind the
``tsnecuda.TSNE(...).fit_transform`` interface."""
from .TSNE import TSNE

__all__ = ["TSNE", "test"]


def test():
    """Smoke run on 5000 x 50 uniform random points (the reference's
    ``tsnecuda.test()``, src/python/tsnecuda/__init__.py:4-7)."""
    import numpy as np
    X = np.random.random((5000, 50))
    TSNE(verbose=1).fit_transform(X)
