"""ctypes front end of the CPU oracle (``liboracle.so``).

Test infrastructure: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package.  The shipped
library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "liboracle.so")
_lib = None

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_c_float_p = ctypes.POINTER(ctypes.c_float)
_c_int_p = ctypes.POINTER(ctypes.c_int)


def build(force=False):
    """Compile liboracle.so with the committed Makefile."""
    cmd = ["make", "-C", _DIR] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_num_threads.restype = ctypes.c_int
        L.oracle_max_normalize.restype = ctypes.c_float
        L.oracle_iterate.restype = ctypes.c_float
        L.oracle_fit.restype = ctypes.c_float
        L.oracle_kl.restype = ctypes.c_double
        L.oracle_row_sum.restype = ctypes.c_float
        L.oracle_symmetrize_full.restype = ctypes.c_int64
        _lib = L
    return _lib


def _opt(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def num_threads():
    return int(lib().oracle_num_threads())


def knn(X, K, rows=None):
    """Exact kNN (self first).  rows=(begin, end) restricts the query rows to a range;
    rows=<int array> to the listed rows (outputs in that order)."""
    X = np.ascontiguousarray(X, np.float32)
    N, D = X.shape
    K = min(K, N)
    if rows is not None and not isinstance(rows, tuple):
        rows = np.ascontiguousarray(rows, np.int32)
        idx = np.empty((rows.size, K), np.int32)
        d2 = np.empty((rows.size, K), np.float32)
        lib().oracle_knn_row_list(_opt(X), N, D, K, _opt(rows), int(rows.size), _opt(idx), _opt(d2))
        return idx, d2
    b, e = (0, N) if rows is None else rows
    idx = np.empty((e - b, K), np.int32)
    d2 = np.empty((e - b, K), np.float32)
    lib().oracle_knn_rows(_opt(X), N, D, K, b, e, _opt(idx), _opt(d2))
    return idx, d2


def knn_ivf(X, K, centroids, nprobe, return_probes=False):
    """The library's approximate (inverted-file) search: (idx, d2[, list of every point, probes of every
    list]) in the caller's numbering."""
    X = np.ascontiguousarray(X, np.float32)
    centroids = np.ascontiguousarray(centroids, np.float32)
    N, D = X.shape
    nlist = centroids.shape[0]
    idx = np.empty((N, K), np.int32)
    d2 = np.empty((N, K), np.float32)
    list_of = np.empty(N, np.int32)
    probes = np.empty((nlist, nprobe), np.int32)
    lib().oracle_knn_ivf(_opt(X), N, D, K, _opt(centroids), nlist, nprobe, _opt(idx), _opt(d2), _opt(list_of),
                         _opt(probes))
    return (idx, d2, list_of, probes) if return_probes else (idx, d2)


def max_normalize(d2):
    out = np.array(d2, np.float32, copy=True, order="C")
    m = lib().oracle_max_normalize(_opt(out), ctypes.c_int64(out.size))
    return out, float(m)


def perplexity(d2, perplexity, eps, return_search=False):
    d2 = np.ascontiguousarray(d2, np.float32)
    N, K = d2.shape
    p = np.empty((N, K), np.float32)
    beta = np.empty(N, np.float32)
    iters = np.empty(N, np.int32)
    lib().oracle_perplexity(_opt(d2), N, K, ctypes.c_float(perplexity), ctypes.c_float(eps), _opt(p), _opt(beta),
                            _opt(iters))
    return (p, beta, iters) if return_search else p


def expf(x):
    """The search's exp (a fixed sequence of fp32 operations), element-wise."""
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x)
    lib().oracle_expf_array(_opt(x), ctypes.c_int64(x.size), _opt(out))
    return out


def logf(v):
    """The search's log, element-wise."""
    v = np.ascontiguousarray(v, np.float32)
    out = np.empty_like(v)
    lib().oracle_logf_array(_opt(v), ctypes.c_int64(v.size), _opt(out))
    return out


def row_sum(v):
    """Sum of a row in the search's stated order (64 interleaved partial sums, then a balanced tree)."""
    v = np.ascontiguousarray(v, np.float32).ravel()
    return float(lib().oracle_row_sum(_opt(v), int(v.size)))


def init(n, kind, seed, std=False):
    """Initial embedding (flat 2N) of the reference's random initialisations: kind 0 = UNIFORM(-5, 5),
    1 = GAUSSIAN (1e-4 N(0,1) after 2N discarded draws).  std=True: through the std:: classes themselves."""
    Y = np.empty(2 * n, np.float32)
    (lib().oracle_init_std if std else lib().oracle_init)(int(n), int(kind), int(seed), _opt(Y))
    return Y


def symmetrize(p, idx):
    p = np.ascontiguousarray(p, np.float32)
    idx = np.ascontiguousarray(idx, np.int32)
    N, K = p.shape
    P = np.empty((N, K), np.float32)
    lib().oracle_symmetrize(_opt(p), _opt(idx), N, K, _opt(P))
    return P


def symmetrize_full(p, idx):
    """(A + A^T) / 2N with the union pattern as CSR (row_ptr, col_idx, values), columns ascending."""
    p = np.ascontiguousarray(p, np.float32)
    idx = np.ascontiguousarray(idx, np.int32)
    N, K = p.shape
    row_ptr = np.empty(N + 1, np.int32)
    col = np.empty(2 * N * K, np.int32)
    val = np.empty(2 * N * K, np.float32)
    nnz = int(lib().oracle_symmetrize_full(_opt(p), _opt(idx), N, K, _opt(row_ptr), _opt(col), _opt(val)))
    return row_ptr, col[:nnz].copy(), val[:nnz].copy()


def attractive_csr(row_ptr, col_idx, values, Y):
    """Attractive forces over a CSR pattern; Y flat 2N -> flat 2N."""
    row_ptr = np.ascontiguousarray(row_ptr, np.int32)
    col_idx = np.ascontiguousarray(col_idx, np.int32)
    values = np.ascontiguousarray(values, np.float32)
    Y = np.ascontiguousarray(Y, np.float32).ravel()
    N = row_ptr.size - 1
    out = np.empty(2 * N, np.float32)
    lib().oracle_attractive_csr(_opt(row_ptr), _opt(col_idx), _opt(values), _opt(Y), N, _opt(out))
    return out


def attractive(P, idx, Y):
    """Y: flat 2N (xs then ys) -> flat 2N forces."""
    P = np.ascontiguousarray(P, np.float32)
    idx = np.ascontiguousarray(idx, np.int32)
    Y = np.ascontiguousarray(Y, np.float32).ravel()
    N, K = P.shape
    out = np.empty(2 * N, np.float32)
    lib().oracle_attractive(_opt(P), _opt(idx), _opt(Y), N, K, _opt(out))
    return out


def repulsive(Y, nb=130, p=3, direct=False, details=False):
    """Returns (rep[2N], Z) and, with details, also (w, y_tilde, phi)."""
    Y = np.ascontiguousarray(Y, np.float32).ravel()
    N = Y.size // 2
    G = nb * p
    rep = np.empty(2 * N, np.float32)
    Z = ctypes.c_float(0)
    w = np.empty((G, G, 4), np.float32) if details else None
    yt = np.empty((G, G, 4), np.float32) if details else None
    phi = np.empty((N, 4), np.float32) if details else None
    lib().oracle_repulsive(_opt(Y), N, nb, p, _opt(rep), ctypes.byref(Z), _opt(w), _opt(yt), _opt(phi),
                           1 if direct else 0)
    if details:
        return rep, float(Z.value), w, yt, phi
    return rep, float(Z.value)


def update(Y, attr, rep, gains, old_forces, eta, normalization, momentum, exaggeration):
    """In place on copies; returns (Y, gains, old_forces)."""
    Y = np.array(Y, np.float32, copy=True).ravel()
    attr = np.array(attr, np.float32, copy=True).ravel()
    rep = np.array(rep, np.float32, copy=True).ravel()
    gains = np.array(gains, np.float32, copy=True).ravel()
    old = np.array(old_forces, np.float32, copy=True).ravel()
    N = Y.size // 2
    lib().oracle_update(_opt(Y), _opt(attr), _opt(rep), _opt(gains), _opt(old), N, ctypes.c_float(eta),
                        ctypes.c_float(normalization), ctypes.c_float(momentum), ctypes.c_float(exaggeration))
    return Y, gains, old


def iterate(P, idx, Y, steps, step_begin=0, force_magnify_iters=250, eta=200.0, pre_momentum=0.5,
            post_momentum=0.8, early_exaggeration=12.0, gains=None, old_forces=None, nb=130, p=3, recenter=False):
    """Runs gradient steps [step_begin, step_begin+steps).  Returns (Y, Z) and
    updates gains / old_forces in place when given.  recenter: the library's optional
    re-centring (every step subtracts the centre the embedding had before the step)."""
    P = np.ascontiguousarray(P, np.float32)
    idx = np.ascontiguousarray(idx, np.int32)
    Y = np.array(Y, np.float32, copy=True).ravel()
    N, K = P.shape
    Z = lib().oracle_iterate(_opt(P), _opt(idx), _opt(Y), _opt(gains), _opt(old_forces), N, K, step_begin,
                             step_begin + steps, force_magnify_iters, ctypes.c_float(eta),
                             ctypes.c_float(pre_momentum), ctypes.c_float(post_momentum),
                             ctypes.c_float(early_exaggeration), nb, p, 1 if recenter else 0)
    return Y, float(Z)


def fit(X, Y0, num_neighbors, perplexity, eps=1e-4, iterations=1000, force_magnify_iters=250, eta=200.0,
        pre_momentum=0.5, post_momentum=0.8, early_exaggeration=12.0):
    """Whole pipeline from an explicit initial embedding.  Returns (Y, Z, idx, P)."""
    X = np.ascontiguousarray(X, np.float32)
    N, D = X.shape
    K = min(num_neighbors, N)
    Y = np.array(Y0, np.float32, copy=True).ravel()
    idx = np.empty((N, K), np.int32)
    P = np.empty((N, K), np.float32)
    Z = lib().oracle_fit(_opt(X), N, D, num_neighbors, ctypes.c_float(perplexity), ctypes.c_float(eps), _opt(Y),
                         iterations, force_magnify_iters, ctypes.c_float(eta), ctypes.c_float(pre_momentum),
                         ctypes.c_float(post_momentum), ctypes.c_float(early_exaggeration), _opt(idx), _opt(P))
    return Y, float(Z), idx, P


def kl(P, idx, Y, Z=0.0):
    P = np.ascontiguousarray(P, np.float32)
    idx = np.ascontiguousarray(idx, np.int32)
    Y = np.ascontiguousarray(Y, np.float32).ravel()
    N, K = P.shape
    return float(lib().oracle_kl(_opt(P), _opt(idx), _opt(Y), N, K, ctypes.c_double(Z)))
