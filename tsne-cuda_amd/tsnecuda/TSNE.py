"""ctypes front end of ``libtsnecuda.so``.

Mirrors the constructor keywords, defaults, validation errors and
``fit_transform(X, y=None)`` behaviour of the reference's
``src/python/tsnecuda/TSNE.py:36-258``; every argument is handed to the
``pymodule_tsne`` entry point of the shared library that sits next to this
file.  No arithmetic happens in Python.
"""
import ctypes
import os

import numpy as np

_LIB_NAME = "libtsnecuda.so"


def _c_string(text):
    """NUL-terminated uint8 array, the form the C side receives strings in."""
    return np.frombuffer(text.encode("latin-1") + b"\0", dtype=np.uint8).copy()


def _load_library():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)
    if not os.path.exists(path):
        raise OSError(
            "%s not found: build it with `make -C tsne-cuda_amd` (hipcc, gfx950) before using tsnecuda" % path)
    lib = ctypes.CDLL(path)
    f32_2d_out = np.ctypeslib.ndpointer(np.float32, ndim=2, flags="ALIGNED, F_CONTIGUOUS, WRITEABLE")
    f32_2d_c = np.ctypeslib.ndpointer(np.float32, ndim=2, flags="ALIGNED, CONTIGUOUS")
    f32_2d_f = np.ctypeslib.ndpointer(np.float32, ndim=2, flags="ALIGNED, F_CONTIGUOUS")
    u8 = np.ctypeslib.ndpointer(np.uint8, flags="ALIGNED, CONTIGUOUS")
    c_int, c_float, c_bool = ctypes.c_int, ctypes.c_float, ctypes.c_bool
    lib.pymodule_tsne.restype = None
    lib.tsne_hip_last_kl_divergence.restype = ctypes.c_double
    lib.tsne_hip_last_kl_divergence.argtypes = []
    lib.pymodule_tsne.argtypes = [
        f32_2d_out,                          # result
        f32_2d_c,                            # points
        ctypes.POINTER(np.ctypeslib.c_intp),  # dims
        c_float, c_float, c_float, c_float,  # perplexity, learning_rate, early_exaggeration, magnitude_factor
        c_int, c_int, c_int, c_int,          # num_neighbors, iterations, iterations_no_progress, force_magnify_iters
        c_float, c_float, c_float,           # perplexity_search_epsilon, pre/post exaggeration momentum
        c_float, c_float, c_float,           # theta, epssq, min_gradient_norm
        c_int, f32_2d_f,                     # initialization_type, preinit_data
        c_bool, u8, c_int,                   # dump_points, dump_file, dump_interval
        c_bool, u8, c_int,                   # use_interactive, viz_server, viz_timeout
        c_int, c_int, c_int,                 # verbosity, print_interval, gpu_device
        c_int, c_int, c_int,                 # return_style, num_snapshots, distance_metric
    ]
    return lib


class TSNE(object):
    """t-SNE embedding into two dimensions on one MI355X."""

    _METRICS = {"euclidean": 1, "L2": 1, "innerproduct": 0}
    _RETURN_STYLES = {"once": 0, "snapshots": 1}

    def __init__(self,
                 n_components=2,
                 perplexity=50.0,
                 early_exaggeration=12.0,
                 learning_rate=200.0,
                 num_neighbors=32,
                 force_magnify_iters=250,
                 pre_momentum=0.5,
                 post_momentum=0.8,
                 theta=0.5,
                 epssq=0.0025,
                 n_iter=1000,
                 n_iter_without_progress=1000,
                 min_grad_norm=0.0,
                 perplexity_epsilon=1e-3,
                 metric='euclidean',
                 init='random',
                 return_style='once',
                 num_snapshots=5,
                 verbose=0,
                 random_seed=None,
                 use_interactive=False,
                 viz_timeout=10000,
                 viz_server="tcp://localhost:5556",
                 dump_points=False,
                 dump_file="dump.txt",
                 dump_interval=1,
                 print_interval=10,
                 device=0,
                 magnitude_factor=5):
        self.n_components = int(n_components)
        if self.n_components != 2:
            raise NotImplementedError('The current fit-tsne implementation does not support '
                                      'projection into dimensions other than 2 for now.')
        if metric not in self._METRICS:
            raise NotImplementedError("Only 'euclidean' and 'innerproduct' metrics are currently supported.")
        # Recorded and passed on; neighbours are always by squared L2 distance,
        # as in the reference (src/util/distance_utils.cu:91).
        self.metric = self._METRICS[metric]
        if init != 'random':
            raise NotImplementedError("Non-Random initialization is not currently supported. "
                                      "Please use init='random' for now.")
        if return_style not in self._RETURN_STYLES:
            raise ValueError('Invalid return style...')
        self.return_style = self._RETURN_STYLES[return_style]
        self.num_snapshots = int(num_snapshots)

        self.perplexity = float(perplexity)
        self.learning_rate = float(learning_rate)
        self.early_exaggeration = float(early_exaggeration)
        self.iterations = int(n_iter)
        self.iterations_no_progress = int(n_iter_without_progress)
        self.min_gradient_norm = float(min_grad_norm)
        self.init = init
        self.verbosity = int(verbose)
        # Accepted for signature compatibility; the C entry point has no seed
        # argument (it seeds from the clock), exactly as in the reference.
        self.random_seed = random_seed

        self.num_neighbors = int(num_neighbors)
        self.force_magnify_iters = int(force_magnify_iters)
        self.perplexity_search_epsilon = float(perplexity_epsilon)
        self.pre_exaggeration_momentum = float(pre_momentum)
        self.post_exaggeration_momentum = float(post_momentum)
        self.theta = float(theta)
        self.epssq = float(epssq)
        self.gpu_device = int(device)
        self.print_interval = int(print_interval)
        self.magnitude_factor = float(magnitude_factor)

        self.dump_file = str(dump_file)
        self.dump_points = bool(dump_points)
        self.dump_interval = int(dump_interval)

        self.use_interactive = bool(use_interactive)
        self.viz_server = str(viz_server)
        self.viz_timeout = int(viz_timeout)

        self._path = os.path.dirname(os.path.abspath(__file__))
        self._lib = _load_library()

    def fit_transform(self, X, y=None):
        """Embeds X (n_points, n_dimensions) and returns the (n_points, 2)
        float32 Fortran-ordered embedding.  ``y`` (n_points, 2), if given, is
        the initial embedding; otherwise the start is Gaussian noise of scale
        1e-4.  With ``return_style='snapshots'`` the result has shape
        (num_snapshots, n_points, 2), one Fortran-ordered embedding per
        snapshot, the last being the final embedding."""
        X = np.asarray(X)
        if X.ndim != 2:
            raise ValueError("X must be a 2-D array of shape (n_points, n_dimensions)")
        self.points = np.require(X, np.float32, ['CONTIGUOUS', 'ALIGNED'])
        n = self.points.shape[0]
        if self.return_style == 1:
            # One (n, 2) Fortran-ordered block per snapshot, contiguous in memory.
            store = np.zeros((max(self.num_snapshots, 1), 2, n), np.float32)
            result = store[0].T
        else:
            store = None
            result = np.zeros((n, self.n_components), np.float32, order='F')
        result = np.require(result, np.float32, ['F_CONTIGUOUS', 'ALIGNED', 'WRITEABLE'])

        if y is None:
            self.initialization_type = 1
            self.preinit_data = np.zeros((1, 1), np.float32)
        else:
            self.initialization_type = 3
            self.preinit_data = np.require(y, np.float32, ['F_CONTIGUOUS', 'ALIGNED'])
            if self.preinit_data.shape != (n, 2):
                raise ValueError("y must have shape (n_points, 2)")

        self.dump_file_ = _c_string(self.dump_file)
        self.viz_server_ = _c_string(self.viz_server)
        self._lib.pymodule_tsne(
            result, self.points, self.points.ctypes.shape,
            self.perplexity, self.learning_rate, self.early_exaggeration, self.magnitude_factor,
            self.num_neighbors, self.iterations, self.iterations_no_progress, self.force_magnify_iters,
            self.perplexity_search_epsilon, self.pre_exaggeration_momentum, self.post_exaggeration_momentum,
            self.theta, self.epssq, self.min_gradient_norm,
            self.initialization_type, self.preinit_data,
            self.dump_points, self.dump_file_, self.dump_interval,
            self.use_interactive, self.viz_server_, self.viz_timeout,
            self.verbosity, self.print_interval, self.gpu_device,
            self.return_style, self.num_snapshots, self.metric)
        # Objective of the returned embedding on the stored neighbour pattern (sklearn's attribute name;
        # the reference sets no such attribute).
        self.kl_divergence_ = float(self._lib.tsne_hip_last_kl_divergence())
        if store is not None:
            self.embedding = store.transpose(0, 2, 1)
        else:
            self.embedding = result
        return self.embedding

    def trustworthiness(self, n_neighbors=12, max_sample=4096):
        """Trustworthiness of the last fit's embedding (1 is best): how far the
        ``n_neighbors`` nearest points of every point in the embedding are from
        being its nearest points in the input space (the measure scikit-learn's
        ``sklearn.manifold.trustworthiness`` computes).  Evaluated on all points
        up to ``max_sample`` (at most 8192) of them, beyond that on a fixed
        pseudo-random sample, whose indices are left in ``trust_sample_``.  Also
        stored as ``trustworthiness_``.  The reference has no such output."""
        if not hasattr(self, "embedding") or not hasattr(self, "points"):
            raise RuntimeError("trustworthiness() needs a fit: call fit_transform first")
        emb = self.embedding[-1] if self.embedding.ndim == 3 else self.embedding
        emb = np.require(emb, np.float32, ['F_CONTIGUOUS', 'ALIGNED'])
        n, d = self.points.shape
        out = ctypes.c_double(0.0)
        sample = np.zeros(int(max_sample), np.int32)
        fn = self._lib.tsnecuda_trustworthiness
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                       ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
        rc = fn(self.points.ctypes.data, emb.ctypes.data, n, d, int(n_neighbors), int(max_sample), self.gpu_device,
                ctypes.byref(out), sample.ctypes.data)
        if rc != 0:
            self._lib.tsne_hip_last_error.restype = ctypes.c_char_p
            raise RuntimeError(self._lib.tsne_hip_last_error().decode())
        self.trust_sample_ = sample[:min(n, int(max_sample))].copy()
        self.trustworthiness_ = float(out.value)
        return self.trustworthiness_
