"""ctypes bindings of the stage-level C ABI (``include/tsnecuda/tsne_stages.h``).

Arguments are torch CUDA tensors; only their device pointers and sizes cross
the boundary.  Every call runs on torch's current stream, so torch events and
synchronisation see the work.  Raises ``RuntimeError`` with the library's
message when a call fails.
"""
import ctypes
import os

import torch

_lib = None
_vp = ctypes.c_void_p


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtsnecuda.so")
        if not os.path.exists(path):
            raise OSError("%s not found: build it with `make -C tsne-cuda_amd` first" % path)
        L = ctypes.CDLL(path)
        L.tsne_hip_last_error.restype = ctypes.c_char_p
        c_int, c_float, c_i64 = ctypes.c_int, ctypes.c_float, ctypes.c_int64
        L.tsne_hip_knn.argtypes = [_vp, c_int, c_int, c_int, _vp, _vp, _vp]
        L.tsne_hip_knn_select.argtypes = [_vp, c_int, c_int, c_int, _vp, _vp, _vp, c_int, ctypes.POINTER(c_int)]
        L.tsne_hip_knn_select.restype = c_int
        L.tsne_hip_ivf_train.argtypes = [_vp, c_int, c_int, c_int, c_int, _vp, _vp]
        L.tsne_hip_ivf_train.restype = c_int
        L.tsne_hip_knn_ivf.argtypes = [_vp, c_int, c_int, c_int, _vp, c_int, c_int, _vp, _vp, _vp, ctypes.POINTER(c_int)]
        L.tsne_hip_knn_ivf.restype = c_int
        L.tsne_hip_locality_order.argtypes = [_vp, c_int, c_int, _vp, _vp]
        L.tsne_hip_gather_rows.argtypes = [_vp, _vp, c_int, c_int, _vp, _vp]
        L.tsne_hip_max_normalize.argtypes = [_vp, c_i64, _vp]
        L.tsne_hip_max_normalize_noalloc.argtypes = [_vp, c_i64, _vp]
        L.tsne_hip_max_normalize_noalloc.restype = c_int
        L.tsne_hip_perplexity.argtypes = [_vp, c_int, c_int, c_float, c_float, _vp, _vp, _vp]
        L.tsne_hip_symmetrize.argtypes = [_vp, _vp, c_int, c_int, _vp, _vp]
        L.tsne_hip_symmetrize_full.argtypes = [_vp, _vp, c_int, c_int, _vp, _vp, _vp, ctypes.POINTER(c_i64), _vp]
        L.tsne_hip_symmetrize_full.restype = c_int
        L.tsne_hip_attractive_csr.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp]
        L.tsne_hip_attractive_csr.restype = c_int
        L.tsne_hip_plan_set_csr_pattern.argtypes = [_vp, _vp, _vp, _vp]
        L.tsne_hip_plan_set_csr_pattern.restype = c_int
        L.tsne_hip_plan_create.argtypes = [ctypes.POINTER(_vp), c_int, c_int, c_int, c_int]
        L.tsne_hip_plan_check.argtypes = [_vp]
        L.tsne_hip_plan_set_recenter.argtypes = [_vp, c_int]
        L.tsne_hip_plan_set_recenter.restype = c_int
        L.tsne_hip_plan_grouping_stats.argtypes = [_vp, _vp]
        L.tsne_hip_plan_grouping_stats.restype = c_int
        L.tsne_hip_plan_set_boxes.argtypes = [_vp, c_int]
        L.tsne_hip_plan_set_boxes.restype = c_int
        L.tsne_hip_boxes_for_spread.argtypes = [c_float]
        L.tsne_hip_boxes_for_spread.restype = c_int
        L.tsne_hip_plan_destroy.argtypes = [_vp]
        L.tsne_hip_plan_destroy.restype = None
        L.tsne_hip_attractive.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp]
        L.tsne_hip_attractive_prepare.argtypes = [_vp, _vp, _vp, _vp]
        L.tsne_hip_attractive_prepare.restype = c_int
        L.tsne_hip_repulsive.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]
        L.tsne_hip_repulsive_kept.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]
        L.tsne_hip_update.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, c_float, _vp, c_float, c_float, _vp]
        L.tsne_hip_iterate.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, c_int, c_int, c_int, c_float, c_float,
                                       c_float, c_float, _vp, _vp]
        L.tsne_hip_sum_squares.argtypes = [_vp, _vp, c_i64, _vp, _vp]
        L.tsne_hip_repulsive_error.argtypes = [_vp, _vp, c_int, ctypes.POINTER(ctypes.c_double), _vp]
        L.tsne_hip_repulsive_error.restype = c_int
        L.tsne_hip_profile_kernel_name.argtypes = [c_int]
        L.tsne_hip_profile_kernel_name.restype = ctypes.c_char_p
        L.tsne_hip_profile_begin.argtypes = [_vp]
        L.tsne_hip_profile_end.argtypes = [_vp, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_int)]
        L.tsne_hip_profile_attractive_begin.argtypes = [_vp]
        L.tsne_hip_profile_attractive_end.argtypes = [_vp, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(c_int)]
        for name in ("profile_begin", "profile_end", "profile_kernel_count", "profile_attractive_begin",
                     "profile_attractive_end"):
            getattr(L, "tsne_hip_" + name).restype = c_int
        for name in ("locality_order", "gather_rows", "knn", "max_normalize", "perplexity", "symmetrize", "plan_create", "attractive",
                     "repulsive", "update", "iterate", "sum_squares"):
            getattr(L, "tsne_hip_" + name).restype = c_int
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise RuntimeError(lib().tsne_hip_last_error().decode())


def _ptr(t):
    return None if t is None else _vp(t.data_ptr())


def _stream():
    return _vp(torch.cuda.current_stream().cuda_stream)


def _f32(t):
    assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
    return t


def knn(points, num_neighbors):
    points = _f32(points)
    n, d = points.shape
    idx = torch.empty((n, num_neighbors), dtype=torch.int32, device=points.device)
    dist = torch.empty((n, num_neighbors), dtype=torch.float32, device=points.device)
    _check(lib().tsne_hip_knn(_ptr(points), n, d, num_neighbors, _ptr(idx), _ptr(dist), _stream()))
    return idx, dist


def knn_select(points, num_neighbors, sweep):
    """knn() with an explicit sweep (1 = vector ALU, 2 = matrix instructions,
    3 = matrix instructions with the products on floats instead of bf16 terms).
    Returns (indices, sq_dist, stats) with stats = (matrix sweep ran, queries redone,
    per mille of tile pairs computed)."""
    points = _f32(points)
    n, d = points.shape
    idx = torch.empty((n, num_neighbors), dtype=torch.int32, device=points.device)
    dist = torch.empty((n, num_neighbors), dtype=torch.float32, device=points.device)
    stats = (ctypes.c_int * 3)()
    _check(lib().tsne_hip_knn_select(_ptr(points), n, d, num_neighbors, _ptr(idx), _ptr(dist), _stream(), sweep,
                                     stats))
    return idx, dist, (int(stats[0]), int(stats[1]), int(stats[2]))


def ivf_train(points, nlist, iterations=10):
    """nlist k-means centroids (nlist x D) for the inverted-file search."""
    points = _f32(points)
    n, d = points.shape
    centroids = torch.empty((nlist, d), dtype=torch.float32, device=points.device)
    _check(lib().tsne_hip_ivf_train(_ptr(points), n, d, nlist, iterations, _ptr(centroids), _stream()))
    return centroids


def knn_ivf(points, num_neighbors, centroids, nprobe=20):
    """Approximate neighbours through the inverted file given by `centroids`.
    Returns (indices, sq_dist, stats) in the caller's numbering."""
    points, centroids = _f32(points), _f32(centroids)
    n, d = points.shape
    idx = torch.empty((n, num_neighbors), dtype=torch.int32, device=points.device)
    dist = torch.empty((n, num_neighbors), dtype=torch.float32, device=points.device)
    stats = (ctypes.c_int * 3)()
    _check(lib().tsne_hip_knn_ivf(_ptr(points), n, d, num_neighbors, _ptr(centroids), centroids.shape[0], nprobe,
                                  _ptr(idx), _ptr(dist), _stream(), stats))
    return idx, dist, (int(stats[0]), int(stats[1]), int(stats[2]))


def locality_order(points):
    """order[new] = old (int32): the renumbering RunTsne applies on entry."""
    points = _f32(points)
    n, d = points.shape
    order = torch.empty(n, dtype=torch.int32, device=points.device)
    _check(lib().tsne_hip_locality_order(_ptr(points), n, d, _ptr(order), _stream()))
    return order


def gather_rows(rows, order):
    rows = _f32(rows)
    n, d = rows.shape
    assert order.is_cuda and order.dtype == torch.int32 and order.numel() == n
    out = torch.empty_like(rows)
    _check(lib().tsne_hip_gather_rows(_ptr(rows), _ptr(order), n, d, _ptr(out), _stream()))
    return out


def max_normalize_(values):
    _check(lib().tsne_hip_max_normalize(_ptr(_f32(values)), values.numel(), _stream()))
    return values


def max_normalize_noalloc_(values, n=None):
    """max_normalize_ through the entry point that allocates nothing (asynchronous;
    calls on one GPU must not overlap).  n: number of leading values (default all)."""
    _check(lib().tsne_hip_max_normalize_noalloc(_ptr(_f32(values)), values.numel() if n is None else n, _stream()))
    return values


def perplexity(sq_dist, perplexity, epsilon, return_betas=False):
    sq_dist = _f32(sq_dist)
    n, k = sq_dist.shape
    pij = torch.empty_like(sq_dist)
    betas = torch.empty(n, dtype=torch.float32, device=sq_dist.device) if return_betas else None
    _check(lib().tsne_hip_perplexity(_ptr(sq_dist), n, k, perplexity, epsilon, _ptr(pij), _ptr(betas), _stream()))
    return (pij, betas) if return_betas else pij


def symmetrize(pij, idx):
    pij = _f32(pij)
    n, k = pij.shape
    out = torch.empty_like(pij)
    _check(lib().tsne_hip_symmetrize(_ptr(pij), _ptr(idx), n, k, _ptr(out), _stream()))
    return out


def symmetrize_full(pij, idx):
    """(A + A^T) / 2N with the union pattern as CSR tensors (row_ptr, col_idx, values)."""
    pij = _f32(pij)
    n, k = pij.shape
    row_ptr = torch.empty(n + 1, dtype=torch.int32, device=pij.device)
    col = torch.empty(2 * n * k, dtype=torch.int32, device=pij.device)
    val = torch.empty(2 * n * k, dtype=torch.float32, device=pij.device)
    nnz = ctypes.c_int64(0)
    _check(lib().tsne_hip_symmetrize_full(_ptr(pij), _ptr(idx), n, k, _ptr(row_ptr), _ptr(col), _ptr(val),
                                          ctypes.byref(nnz), _stream()))
    return row_ptr, col[:nnz.value], val[:nnz.value]


def boxes_for_spread(spread):
    """FIt-SNE's grid-size rule with the reference's constants (125 boxes at least, one per unit
    of spread, rounded up in its list of sizes; 170 at most)."""
    return int(lib().tsne_hip_boxes_for_spread(ctypes.c_float(spread)))


class Plan(object):
    """Scratch memory of the gradient loop for one problem size."""

    def __init__(self, num_points, num_neighbors, n_boxes_per_dim=130, device=0):
        self._h = _vp()
        self.num_points, self.num_neighbors, self.n_boxes = num_points, num_neighbors, n_boxes_per_dim
        self.n_nodes = 3 * n_boxes_per_dim
        self.device = torch.device("cuda", device)
        _check(lib().tsne_hip_plan_create(ctypes.byref(self._h), num_points, num_neighbors, n_boxes_per_dim,
                                          device))

    def close(self):
        if self._h:
            lib().tsne_hip_plan_destroy(self._h)
            self._h = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self):
        """Raises if a kernel of this plan reported trouble since the last call
        (synchronises the device first)."""
        torch.cuda.synchronize(self.device)
        _check(lib().tsne_hip_plan_check(self._h))

    def set_recenter(self, enable):
        """Optional re-centring inside iterate_ (off by default, as in the reference)."""
        _check(lib().tsne_hip_plan_set_recenter(self._h, 1 if enable else 0))

    def grouping_stats(self):
        """(repulsive evaluations so far, those that grouped the points by tile afresh, points spread
        on the slow path because they had strayed from their tile)."""
        out = (ctypes.c_uint * 3)()
        _check(lib().tsne_hip_plan_grouping_stats(self._h, out))
        return int(out[0]), int(out[1]), int(out[2])

    def set_boxes(self, n_boxes_per_dim):
        """Size of the interpolation grid from the next step on (the reference runs 130)."""
        _check(lib().tsne_hip_plan_set_boxes(self._h, n_boxes_per_dim))
        self.n_nodes = 3 * n_boxes_per_dim

    def prepare_attractive(self, pij, idx):
        """Re-blocks (pij, idx) into the plan; afterwards attractive() and
        iterate_() may be called with pij = idx = None."""
        _check(lib().tsne_hip_attractive_prepare(self._h, _ptr(_f32(pij)), _ptr(idx), _stream()))

    def attractive(self, pij, idx, embedding):
        out = torch.empty(2 * self.num_points, dtype=torch.float32, device=self.device)
        _check(lib().tsne_hip_attractive(self._h, _ptr(None if pij is None else _f32(pij)), _ptr(idx),
                                         _ptr(_f32(embedding)), _ptr(out), _stream()))
        return out

    def attractive_csr(self, row_ptr, col_idx, values, embedding):
        out = torch.empty(2 * self.num_points, dtype=torch.float32, device=self.device)
        _check(lib().tsne_hip_attractive_csr(self._h, _ptr(row_ptr), _ptr(col_idx), _ptr(_f32(values)),
                                             _ptr(_f32(embedding)), _ptr(out), _stream()))
        return out

    def set_csr_pattern(self, row_ptr, col_idx, values):
        """iterate_(None, None, ...) then takes its attractive forces from this CSR pattern (the tensors
        must stay alive); three Nones clear it."""
        self._csr = (row_ptr, col_idx, values)
        _check(lib().tsne_hip_plan_set_csr_pattern(self._h, _ptr(row_ptr), _ptr(col_idx), _ptr(values)))

    def repulsive(self, embedding, details=False, keep_grouping=False):
        n, g = self.num_points, self.n_nodes
        rep = torch.empty(2 * n, dtype=torch.float32, device=self.device)
        z = torch.empty(1, dtype=torch.float32, device=self.device)
        w = yt = phi = None
        if details:
            w = torch.empty((g, g, 4), dtype=torch.float32, device=self.device)
            yt = torch.empty((g, g, 4), dtype=torch.float32, device=self.device)
            phi = torch.empty((n, 4), dtype=torch.float32, device=self.device)
        fn = lib().tsne_hip_repulsive_kept if keep_grouping else lib().tsne_hip_repulsive
        _check(fn(self._h, _ptr(_f32(embedding)), _ptr(rep), _ptr(z), _ptr(w), _ptr(yt), _ptr(phi), _stream()))
        return (rep, z, w, yt, phi) if details else (rep, z)

    def update_(self, embedding, attr, rep, gains, old_forces, eta, normalization, momentum, exaggeration):
        _check(lib().tsne_hip_update(self._h, _ptr(_f32(embedding)), _ptr(_f32(attr)), _ptr(_f32(rep)),
                                     _ptr(_f32(gains)), _ptr(_f32(old_forces)), eta, _ptr(_f32(normalization)),
                                     momentum, exaggeration, _stream()))

    def iterate_(self, pij, idx, embedding, gains, old_forces, step_begin, step_end, force_magnify_iters=250,
                 eta=200.0, pre_momentum=0.5, post_momentum=0.8, early_exaggeration=12.0):
        z = torch.empty(1, dtype=torch.float32, device=self.device)  # written by the call
        _check(lib().tsne_hip_iterate(self._h, _ptr(None if pij is None else _f32(pij)), _ptr(idx),
                                      _ptr(_f32(embedding)),
                                      _ptr(_f32(gains)), _ptr(_f32(old_forces)), step_begin, step_end,
                                      force_magnify_iters, eta, pre_momentum, post_momentum, early_exaggeration,
                                      _ptr(z), _stream()))
        return z

    def profile_begin(self):
        _check(lib().tsne_hip_profile_begin(self._h))

    def profile_end(self):
        """{kernel name: (total ms, launches)} of the iterate_ calls since profile_begin."""
        n = lib().tsne_hip_profile_kernel_count()
        ms = (ctypes.c_double * n)()
        cnt = (ctypes.c_int * n)()
        _check(lib().tsne_hip_profile_end(self._h, ms, cnt))
        return {lib().tsne_hip_profile_kernel_name(i).decode(): (ms[i], cnt[i]) for i in range(n)}

    def profile_attractive_begin(self):
        _check(lib().tsne_hip_profile_attractive_begin(self._h))

    def profile_attractive_end(self):
        """(total ms, launches) of the attractive kernel in the iterate_ calls since profile_attractive_begin,
        with the loop's kernels on two streams as in an unprofiled run."""
        ms, cnt = ctypes.c_double(), ctypes.c_int()
        _check(lib().tsne_hip_profile_attractive_end(self._h, ctypes.byref(ms), ctypes.byref(cnt)))
        return ms.value, cnt.value

    def repulsive_error(self, embedding, sample_count):
        """(relative L2 error of the interpolated repulsive forces, relative error of the
        normalisation terms, points sampled) against exact sums on sampled points."""
        out = (ctypes.c_double * 3)()
        _check(lib().tsne_hip_repulsive_error(self._h, _ptr(_f32(embedding)), sample_count, out, _stream()))
        return float(out[0]), float(out[1]), int(out[2])

    def sum_squares(self, values):
        out = torch.empty(1, dtype=torch.float32, device=self.device)
        _check(lib().tsne_hip_sum_squares(self._h, _ptr(_f32(values)), values.numel(), _ptr(out), _stream()))
        return out
