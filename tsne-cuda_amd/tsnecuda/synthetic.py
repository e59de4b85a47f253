"""Deterministic synthetic inputs for the benchmark and parity configurations.

A counter-based generator (splitmix64 -> uniform -> Box-Muller) written with
numpy integer arithmetic only, so the same seed gives the same float32 bytes on
every machine and numpy version.  Nothing here touches the GPU.
"""
import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(counter):
    """splitmix64 output function applied to an array of uint64 counters."""
    with np.errstate(over="ignore"):
        z = (counter + np.uint64(0x9E3779B97F4A7C15)) & _MASK
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
        return z ^ (z >> np.uint64(31))


def uniform01(seed, stream, n, offset=0):
    """n doubles in (0, 1): 53 random bits plus a half-ulp shift (never 0 or 1)."""
    with np.errstate(over="ignore"):
        base = _splitmix64(np.array([seed], np.uint64) * np.uint64(0x632BE59BD9B4E019) + np.uint64(stream))
        ctr = base + np.arange(offset, offset + n, dtype=np.uint64) * np.uint64(0xD1342543DE82EF95)
    bits = _splitmix64(ctr) >> np.uint64(11)
    return (bits.astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, stream, n, offset=0):
    """n standard normals (Box-Muller, cosine branch only: one normal per pair)."""
    u1 = uniform01(seed, 2 * stream, n, offset)
    u2 = uniform01(seed, 2 * stream + 1, n, offset)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def gaussian_clusters(n, d=50, clusters=4, center_scale=10.0, seed=0, chunk=1 << 18):
    """Isotropic Gaussian clusters: centers ~ N(0, center_scale^2 I), sigma 1,
    label = i mod clusters (equal sizes).  float32 (n, d), C-contiguous."""
    centers = (normal(seed, 1, clusters * d) * center_scale).reshape(clusters, d)
    out = np.empty((n, d), np.float32)
    for b in range(0, n, chunk):
        e = min(n, b + chunk)
        noise = normal(seed, 2, (e - b) * d, offset=b * d).reshape(e - b, d)
        labels = np.arange(b, e) % clusters
        out[b:e] = (centers[labels] + noise).astype(np.float32)
    return out


def pixel_like(n=60000, d=784, clusters=10, seed=0, chunk=1 << 14):
    """Pixel-like vectors: per-cluster template with ~80% zeros and the rest
    U[0,255]; per-point noise U(-30,30); clipped to [0,255]; divided by 255."""
    nz = uniform01(seed, 11, clusters * d).reshape(clusters, d) < 0.2
    vals = uniform01(seed, 12, clusters * d).reshape(clusters, d) * 255.0
    templates = np.where(nz, vals, 0.0)
    out = np.empty((n, d), np.float32)
    for b in range(0, n, chunk):
        e = min(n, b + chunk)
        noise = (uniform01(seed, 13, (e - b) * d, offset=b * d).reshape(e - b, d) * 60.0) - 30.0
        labels = np.arange(b, e) % clusters
        out[b:e] = (np.clip(templates[labels] + noise, 0.0, 255.0) / 255.0).astype(np.float32)
    return out


def relu_features(n=50000, d=1024, clusters=10, seed=0, chunk=1 << 14):
    """Classifier-feature-like vectors: ReLU(N(mu_c, 1)), mu_c ~ N(0, I)."""
    mu = normal(seed, 21, clusters * d).reshape(clusters, d)
    out = np.empty((n, d), np.float32)
    for b in range(0, n, chunk):
        e = min(n, b + chunk)
        noise = normal(seed, 22, (e - b) * d, offset=b * d).reshape(e - b, d)
        labels = np.arange(b, e) % clusters
        out[b:e] = np.maximum(0.0, mu[labels] + noise).astype(np.float32)
    return out


def initial_embedding(n, seed=1, scale=1e-4):
    """Explicit initial embedding, Fortran-ordered float32 (n, 2): 1e-4 * N(0,1),
    the scale of the reference's Gaussian init (src/fit_tsne.cu:200-201)."""
    flat = (normal(seed, 31, 2 * n) * scale).astype(np.float32)
    return np.asfortranarray(flat.reshape(2, n).T)


CONFIGS = {
    # name: (generator, kwargs, fit parameters)
    "c0": (gaussian_clusters, dict(n=5000, d=50), dict(perplexity=30.0, num_neighbors=90, learning_rate=200.0)),
    "c1": (pixel_like, dict(n=60000, d=784), dict(perplexity=15.0, num_neighbors=45, learning_rate=10.0)),
    "c2": (relu_features, dict(n=50000, d=1024), dict(perplexity=30.0, num_neighbors=90, learning_rate=200.0)),
    "c3": (gaussian_clusters, dict(n=1000000, d=50), dict(perplexity=30.0, num_neighbors=90, learning_rate=200.0)),
    "c4": (gaussian_clusters, dict(n=10000000, d=50), dict(perplexity=30.0, num_neighbors=90, learning_rate=200.0)),
}


def make_config(name, n=None):
    """Returns (X, fit_kwargs) for one of the named configurations; n overrides
    the point count (same distribution, fewer points)."""
    gen, kw, fit = CONFIGS[name]
    kw = dict(kw)
    if n is not None:
        kw["n"] = n
    return gen(**kw), dict(fit)
