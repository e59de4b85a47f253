"""Host-side checks that need no GPU: the shared library loads and exports every
symbol the public headers declare, the Python front end mirrors the reference's
keyword surface (src/python/tsnecuda/TSNE.py:38-95,129-130), and the synthetic
generators are deterministic."""
import ctypes
import glob
import inspect
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "tsne-cuda_amd", "tsnecuda", "libtsnecuda.so")


def declared_c_functions():
    names = set()
    for header in glob.glob(os.path.join(ROOT, "include", "tsnecuda", "*.h")):
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for block in re.findall(r'extern "C" \{(.*?)\n\}', text, flags=re.S):
            names.update(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{]*\)\s*;", block))
    return names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build the library first: make -C tsne-cuda_amd"
    lib = ctypes.CDLL(LIB)
    names = declared_c_functions()
    assert {"pymodule_tsne", "tsne_hip_knn", "tsne_hip_perplexity", "tsne_hip_symmetrize", "tsne_hip_attractive",
            "tsne_hip_repulsive", "tsne_hip_update", "tsne_hip_iterate", "tsne_hip_plan_create"} <= names
    for name in sorted(names):
        assert hasattr(lib, name), name


def test_cpp_entry_points_are_exported():
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", "-C", LIB], capture_output=True, text=True).stdout
    assert "tsnecuda::RunTsne(tsnecuda::Options&, tsnecuda::GpuOptions&)" in out
    assert "tsnecuda::GpuOptions::GpuOptions(int)" in out


def test_error_reporting_without_gpu():
    lib = ctypes.CDLL(LIB)
    lib.tsne_hip_last_error.restype = ctypes.c_char_p
    # argument checks run before anything touches a device
    assert lib.tsne_hip_knn(None, 10, 2, 3, None, None, None) != 0
    assert b"null pointer" in lib.tsne_hip_last_error()
    plan = ctypes.c_void_p()
    assert lib.tsne_hip_plan_create(ctypes.byref(plan), 0, 5, 130, 0) != 0
    assert b"num_points" in lib.tsne_hip_last_error()
    assert lib.tsne_hip_plan_create(ctypes.byref(plan), 10, 5, 500, 0) != 0
    assert b"n_boxes_per_dim" in lib.tsne_hip_last_error()


def test_tsne_keyword_surface():
    from tsnecuda import TSNE
    sig = inspect.signature(TSNE.__init__)
    expected = dict(n_components=2, perplexity=50.0, early_exaggeration=12.0, learning_rate=200.0, num_neighbors=32,
                    force_magnify_iters=250, pre_momentum=0.5, post_momentum=0.8, theta=0.5, epssq=0.0025,
                    n_iter=1000, n_iter_without_progress=1000, min_grad_norm=0.0, perplexity_epsilon=1e-3,
                    metric='euclidean', init='random', return_style='once', num_snapshots=5, verbose=0,
                    random_seed=None, use_interactive=False, viz_timeout=10000, viz_server="tcp://localhost:5556",
                    dump_points=False, dump_file="dump.txt", dump_interval=1, print_interval=10, device=0,
                    magnitude_factor=5)
    got = {k: v.default for k, v in sig.parameters.items() if k != "self"}
    assert got == expected
    assert list(got) == list(expected)  # positional order too


def test_tsne_validation_errors():
    from tsnecuda import TSNE
    with pytest.raises(NotImplementedError):
        TSNE(n_components=3)
    with pytest.raises(NotImplementedError):
        TSNE(metric="cosine")
    with pytest.raises(NotImplementedError):
        TSNE(init="pca")
    with pytest.raises(ValueError):
        TSNE(return_style="all")
    t = TSNE(metric="innerproduct", return_style="snapshots", num_snapshots=7)
    assert t.metric == 0 and t.return_style == 1 and t.num_snapshots == 7
    assert TSNE(metric="L2").metric == 1


def test_pymodule_argtypes_match_header():
    from tsnecuda import TSNE
    header = open(os.path.join(ROOT, "include", "tsnecuda", "pymodule_ext.h")).read()
    params = re.search(r"void pymodule_tsne\((.*?)\);", header, flags=re.S).group(1)
    n_params = len([p for p in params.split(",") if p.strip()])
    assert n_params == 31
    assert len(TSNE()._lib.pymodule_tsne.argtypes) == n_params


def test_synthetic_generators_are_deterministic():
    from tsnecuda import synthetic
    a = synthetic.gaussian_clusters(1000, d=50)
    b = synthetic.gaussian_clusters(1000, d=50)
    assert np.array_equal(a, b) and a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    # chunking does not change the stream
    assert np.array_equal(synthetic.gaussian_clusters(1000, d=50, chunk=64), a)
    px = synthetic.pixel_like(500)
    assert px.shape == (500, 784) and px.min() >= 0.0 and px.max() <= 1.0
    assert 0.6 < (px < 0.12).mean() < 0.9  # ~80 % of the template entries are zero (plus clipped noise)
    rf = synthetic.relu_features(400)
    assert rf.shape == (400, 1024) and rf.min() == 0.0 and 0.35 < (rf == 0).mean() < 0.65
    y0 = synthetic.initial_embedding(100)
    assert y0.flags["F_CONTIGUOUS"] and y0.shape == (100, 2) and abs(float(y0.std()) - 1e-4) < 3e-5
    u = synthetic.uniform01(0, 0, 100000)
    assert 0.0 < u.min() and u.max() < 1.0 and abs(u.mean() - 0.5) < 5e-3
    z = synthetic.normal(0, 0, 200000)
    assert abs(z.mean()) < 1e-2 and abs(z.std() - 1.0) < 1e-2
