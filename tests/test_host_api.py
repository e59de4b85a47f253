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


def _load(fn, path):
    lib = ctypes.CDLL(LIB)
    f = getattr(lib, fn)
    f.restype = ctypes.POINTER(ctypes.c_float)
    f.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int)]
    dims = (ctypes.c_int * 2)()
    ptr = f(str(path).encode(), dims)
    if not ptr:
        return None
    out = np.ctypeslib.as_array(ptr, shape=(dims[0], dims[1])).copy()
    lib.tsnecuda_free_points.argtypes = [ctypes.POINTER(ctypes.c_float)]
    lib.tsnecuda_free_points(ptr)
    return out


def test_mnist_reader(tmp_path, capfd):
    """idx3-ubyte: big-endian magic 2051, count, rows, columns, one byte per
    pixel; values / 255, one image per row (src/util/data_utils.cu:12-79)."""
    rng = np.random.default_rng(0)
    pixels = rng.integers(0, 256, size=(1234, 7, 5), dtype=np.uint8)  # more images than one read batch
    path = tmp_path / "images.idx3-ubyte"
    with open(path, "wb") as f:
        f.write(np.array([2051, 1234, 7, 5], dtype=">i4").tobytes())
        f.write(pixels.tobytes())
    got = _load("tsnecuda_load_mnist", path)
    assert got.shape == (1234, 35) and got.dtype == np.float32
    assert np.array_equal(got, pixels.reshape(1234, 35).astype(np.float32) / np.float32(255.0))
    assert "Num Images: 1234" in capfd.readouterr().out
    # wrong magic number, truncated file, missing file: no data
    bad = tmp_path / "labels.idx1-ubyte"
    bad.write_bytes(np.array([2049, 10, 1, 1], dtype=">i4").tobytes() + bytes(10))
    assert _load("tsnecuda_load_mnist", bad) is None
    short = tmp_path / "short.idx3-ubyte"
    short.write_bytes(np.array([2051, 100, 7, 5], dtype=">i4").tobytes() + bytes(99 * 35))
    assert _load("tsnecuda_load_mnist", short) is None
    assert _load("tsnecuda_load_mnist", tmp_path / "missing") is None
    err = capfd.readouterr().err
    assert "Magic number: 2049" in err and "ends after 99 of 100" in err and "cannot read" in err


def test_cifar_readers(tmp_path):
    """CIFAR-10: five files of 10000 records (1 label byte + 3072 pixels);
    CIFAR-100: one file of 50000 records with 2 label bytes
    (src/util/data_utils.cu:81-159)."""
    rng = np.random.default_rng(1)
    pixels = rng.integers(0, 256, size=(50000, 3072), dtype=np.uint8)
    want = pixels.astype(np.float32) / np.float32(255.0)
    for b in range(5):
        rec = np.concatenate([rng.integers(0, 10, size=(10000, 1), dtype=np.uint8), pixels[b * 10000:(b + 1) * 10000]],
                             axis=1)
        (tmp_path / ("data_batch_%d.bin" % (b + 1))).write_bytes(rec.tobytes())
    got = _load("tsnecuda_load_cifar10", tmp_path)
    assert got.shape == (50000, 3072) and np.array_equal(got, want)
    rec = np.concatenate([rng.integers(0, 100, size=(50000, 2), dtype=np.uint8), pixels], axis=1)
    (tmp_path / "train.bin").write_bytes(rec.tobytes())
    got = _load("tsnecuda_load_cifar100", tmp_path / "train.bin")
    assert got.shape == (50000, 3072) and np.array_equal(got, want)
    (tmp_path / "data_batch_5.bin").unlink()
    assert _load("tsnecuda_load_cifar10", tmp_path) is None


def test_command_line_options(capfd):
    """The `tsne` program takes the reference's option letters and names
    (src/exe/main.cu:25-40); parsing needs no GPU."""
    import subprocess
    exe = os.path.join(ROOT, "tsne-cuda_amd", "tsnecuda", "tsne")
    assert os.path.exists(exe), "build first: make -C tsne-cuda_amd"
    out = subprocess.run([exe, "--help"], capture_output=True, text=True)
    assert out.returncode == 0
    for line in ("-l, --learning-rate arg", "-p, --perplexity arg", "-e, --early-ex arg", "-s, --data arg",
                 "-k, --num-points arg", "-u, --nearest-neighbors arg", "-n, --num-steps arg", "-i, --viz",
                 "-d, --dump", "-m, --magnitude-factor arg", "-t, --init arg", "-f, --fname arg",
                 "-c, --connection arg", "-q, --dim arg", "-j, --device arg", "-h, --help"):
        assert line in out.stdout, line
    assert "(default: 50.0)" in out.stdout and "(default: 32)" in out.stdout
    bad = subprocess.run([exe, "--no-such-option"], capture_output=True, text=True)
    assert bad.returncode != 0 and "does not exist" in bad.stderr
    bad = subprocess.run([exe, "-n", "many"], capture_output=True, text=True)
    assert bad.returncode != 0 and "failed to parse" in bad.stderr
    unknown = subprocess.run([exe, "-s", "imagenet"], capture_output=True, text=True)
    assert unknown.returncode == 0 and "Dataset not recognized..." in unknown.stdout
    missing = subprocess.run([exe, "--data=mnist", "-f", "/nonexistent/file"], capture_output=True, text=True)
    assert missing.returncode != 0 and "cannot read" in missing.stderr
