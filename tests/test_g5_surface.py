"""The surface around the fit, on the GPU: random starts, exit messages, snapshots, dump file, progress lines,
quality outputs, the optional modes, the command-line program."""
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


@pytest.fixture(autouse=True)
def fixed_random_start(monkeypatch):
    """Fits without an explicit start draw it from Options::random_seed, which the reference's constructors
    take from the clock; TSNE_RANDOM_SEED (this library's extension) replaces it, so that every run of these
    tests starts from the same embedding.  Assertions here are still chosen not to depend on the start."""
    monkeypatch.setenv("TSNE_RANDOM_SEED", "20240229")


def test_gaussian_init_and_snapshots(c0_problem):
    from tsnecuda import TSNE
    X = c0_problem["X"][:1500]
    snaps = TSNE(perplexity=15.0, num_neighbors=45, n_iter=40, return_style="snapshots", num_snapshots=5,
                 perplexity_epsilon=1e-4).fit_transform(X)
    assert snaps.shape == (5, 1500, 2) and np.isfinite(snaps).all()
    # snapshot 0 is taken after the first step from the 1e-4 Gaussian start; the layout grows afterwards
    assert np.abs(snaps[0]).max() < 1.0
    assert np.abs(snaps[-1]).max() > np.abs(snaps[0]).max()
    assert not np.array_equal(snaps[1], snaps[2])


REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("n,seed", [(300, 7), (20000, 1700000000)])
def test_random_initialisations_follow_the_reference_draw_order(tmp_path, kind, n, seed):
    """RunTsne with zero iterations returns its initial embedding.  With Options::random_seed
    fixed (only the C++ surface can: tests/harness/options_harness.cpp) it must be, bit for bit,
    what src/fit_tsne.cu:184-204 draws: 2N normals discarded, then 2N x 1e-4 (GAUSSIAN) or 2N
    uniform values in [-5, 5) (UNIFORM) - also through the locality renumbering (20000 points)."""
    import subprocess
    exe = os.path.join(REPO, "tests", "harness", "options_harness")
    assert os.path.exists(exe), "build the harness with `make -C tsne-cuda_amd`"
    out = tmp_path / "init.bin"
    env = {k: v for k, v in os.environ.items() if k != "TSNE_RANDOM_SEED"}  # the seed under test is Options::random_seed
    run = subprocess.run([exe, str(n), "4", str(kind), str(seed), "0", str(out)], capture_output=True, text=True,
                         timeout=120, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    got = np.fromfile(out, np.float32)
    want = oracle.init(n, kind, seed)
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


_EXIT_SNIPPET = """
import ctypes, sys
import numpy as np
lib = ctypes.CDLL(sys.argv[1])
c_float, c_int, c_bool, vp = ctypes.c_float, ctypes.c_int, ctypes.c_bool, ctypes.c_void_p
lib.pymodule_tsne.restype = None
lib.pymodule_tsne.argtypes = [vp, vp, vp] + [c_float] * 4 + [c_int] * 4 + [c_float] * 6 + [c_int, vp, c_bool, vp,
    c_int, c_bool, vp, c_int, c_int, c_int, c_int, c_int, c_int, c_int]
init, preinit_null, style = int(sys.argv[2]), int(sys.argv[3]), int(sys.argv[4])
X = np.random.default_rng(0).random((200, 5)).astype(np.float32)
res = np.zeros((200, 2), np.float32, order="F")
pre = np.zeros((200, 2), np.float32, order="F")
dims = (ctypes.c_ssize_t * 2)(200, 5)
empty = ctypes.create_string_buffer(b"")
lib.pymodule_tsne(res.ctypes.data, X.ctypes.data, ctypes.cast(dims, vp), 10.0, 200.0, 12.0, 5.0, 30, 5, 1000, 250,
                  1e-3, 0.5, 0.8, 0.5, 0.0025, 0.0, init, None if preinit_null else pre.ctypes.data, False,
                  ctypes.cast(empty, vp), 1, False, ctypes.cast(empty, vp), 1000, 0, 10, 0, style, 2, 1)
print("returned")
"""


@pytest.mark.parametrize("init,preinit_null,style,message", [
    (2, 0, 0, "E: RESUME initialization not yet supported fully..."),  # src/ext/pymodule_ext.cu:78-81
    (7, 0, 0, "E: Invalid initialization supplied"),                   # :86-88
    (3, 1, 0, "E: Invalid initialization. Initialization points are null."),  # src/fit_tsne.cu:218-222
    (1, 0, 5, "E: Invalid return style supplied"),                     # src/ext/pymodule_ext.cu:114-115
])
def test_pymodule_exits_with_the_reference_messages(tmp_path, init, preinit_null, style, message):
    """The shim has no status to return: invalid encodings print the reference's message and
    exit(1), which only a child process can observe."""
    import subprocess
    import sys
    script = tmp_path / "call.py"
    script.write_text(_EXIT_SNIPPET)
    lib = os.path.join(REPO, "tsne-cuda_amd", "tsnecuda", "libtsnecuda.so")
    run = subprocess.run([sys.executable, str(script), lib, str(init), str(preinit_null), str(style)],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 1, (run.returncode, run.stdout, run.stderr)
    assert message in run.stderr
    assert "returned" not in run.stdout


def test_pymodule_child_process_runs_a_valid_call(tmp_path):
    """The same child-process call with valid encodings returns (so the exits above are the shim's)."""
    import subprocess
    import sys
    script = tmp_path / "call.py"
    script.write_text(_EXIT_SNIPPET)
    lib = os.path.join(REPO, "tsne-cuda_amd", "tsnecuda", "libtsnecuda.so")
    run = subprocess.run([sys.executable, str(script), lib, "1", "0", "0"], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and "returned" in run.stdout, run.stderr


def test_trustworthiness_output_against_sklearn(c0_problem):
    """TSNE.trustworthiness() after a fit: the library's own evaluation against scikit-learn's
    (an independent implementation) - on all points where they fit the sample, and on the
    sample the library reports otherwise."""
    from sklearn.manifold import trustworthiness
    from tsnecuda import TSNE
    X = c0_problem["X"][:3000]
    model = TSNE(perplexity=20.0, num_neighbors=60, n_iter=300, perplexity_epsilon=1e-4)
    emb = model.fit_transform(X)
    for k in (5, 12, 30):
        got = model.trustworthiness(n_neighbors=k)
        assert got == model.trustworthiness_
        assert abs(got - trustworthiness(X, emb, n_neighbors=k)) <= 1e-6
    assert np.array_equal(model.trust_sample_, np.arange(3000))
    # a sample of 1000 of the 3000 points: the definition applied to those points and their embedding
    got = model.trustworthiness(n_neighbors=12, max_sample=1000)
    sub = model.trust_sample_
    assert sub.shape == (1000,) and np.all(np.diff(sub) > 0) and sub.max() < 3000
    assert abs(got - trustworthiness(X[sub], emb[sub], n_neighbors=12)) <= 1e-6
    # a shuffled embedding is not trustworthy
    model.embedding = np.asfortranarray(emb[np.random.default_rng(0).permutation(3000)])
    assert model.trustworthiness(n_neighbors=12) < got - 0.2
    with pytest.raises(RuntimeError, match="n_neighbors must be"):
        model.trustworthiness(n_neighbors=600, max_sample=1000)
    with pytest.raises(RuntimeError, match="needs a fit"):
        TSNE().trustworthiness()


def test_repulsion_monitor_lines(c0_problem, capfd, monkeypatch):
    from tsnecuda import TSNE
    monkeypatch.setenv("TSNE_REPULSION_MONITOR", "300")
    TSNE(perplexity=10.0, num_neighbors=30, n_iter=40, verbose=1, print_interval=20,
         perplexity_epsilon=1e-4).fit_transform(c0_problem["X"][:1500])
    out = capfd.readouterr().out
    lines = [l for l in out.split("\n") if "Repulsion interpolation error" in l]
    assert len(lines) == 2 and lines[0].startswith("[Step 0]") and "(300 points)" in lines[0]
    err = float(lines[1].split("forces ")[1].split(",")[0])
    assert 0.0 < err < 0.1


def test_fit_with_full_symmetrisation(c0_problem, monkeypatch, capfd):
    """TSNE_SYMMETRIZE=full: the gradient loop over (A + A^T) / 2N with the union pattern (CSR).  The fit's
    objective is then taken over that pattern, whose mass is 1 (the default pattern drops ~a fifth of it
    at K = 90), so it comes out higher; the embedding is as trustworthy as the default one's."""
    from tsnecuda import TSNE
    c = c0_problem
    X = c["X"]
    Y0 = synthetic_start(X.shape[0])
    kw = dict(perplexity=30.0, num_neighbors=90, n_iter=500, perplexity_epsilon=1e-4)
    base = TSNE(**kw)
    base.fit_transform(X, y=Y0)
    t_base = base.trustworthiness(12)
    monkeypatch.setenv("TSNE_SYMMETRIZE", "full")
    full = TSNE(verbose=1, print_interval=250, **kw)
    emb = full.fit_transform(X, y=Y0)
    out = capfd.readouterr().out
    assert "non-zeros after full symmetrisation" in out
    stored = int(out.split(" non-zeros after full symmetrisation")[0].split("(")[-1])
    rp, cc, vv = oracle.symmetrize_full(c["p"], c["idx"])
    assert stored == cc.size
    assert np.isfinite(emb).all() and full.kl_divergence_ > 0
    assert abs(full.trustworthiness(12) - t_base) <= 0.02
    # the objective of the returned embedding over the CSR pattern, re-evaluated on the host (exact Z)
    n = X.shape[0]
    ex, ey = emb[:, 0].astype(np.float64), emb[:, 1].astype(np.float64)
    rows = np.repeat(np.arange(n), np.diff(rp))
    d2 = (ex[rows] - ex[cc]) ** 2 + (ey[rows] - ey[cc]) ** 2
    dx, dy = ex[:, None] - ex[None, :], ey[:, None] - ey[None, :]
    Z = (1.0 / (1.0 + dx * dx + dy * dy)).sum() - n
    pos = vv > 0
    kl = float((vv[pos].astype(np.float64) * (np.log(vv[pos].astype(np.float64)) + np.log1p(d2[pos]) + np.log(Z))).sum())
    assert abs(full.kl_divergence_ - kl) <= 0.01 * kl


def test_fit_with_approximate_neighbours(monkeypatch, capfd):
    """TSNE_KNN=ivf: the neighbour search through the inverted file (floor(sqrt(N)) lists, as the
    reference's FAISS index).  The embedding of clustered data is as trustworthy as with exact neighbours."""
    from tsnecuda import TSNE, synthetic
    X, fit = synthetic.make_config("c3", n=40000)
    Y0 = synthetic_start(X.shape[0])
    kw = dict(perplexity=30.0, num_neighbors=90, n_iter=400, perplexity_epsilon=1e-4)
    exact = TSNE(**kw)
    exact.fit_transform(X, y=Y0)
    t_exact = exact.trustworthiness(12)
    monkeypatch.setenv("TSNE_KNN", "ivf")
    monkeypatch.setenv("TSNE_KNN_NPROBE", "40")
    approx = TSNE(verbose=1, print_interval=200, **kw)
    emb = approx.fit_transform(X, y=Y0)
    out = capfd.readouterr().out
    assert "(inverted file: 200 lists, 40 probed per list, " in out
    per_mille = int(out.split("probed per list, ")[1].split(" per mille")[0])
    assert 0 < per_mille < 600
    assert np.isfinite(emb).all()
    t_approx = approx.trustworthiness(12)
    print("trustworthiness: exact neighbours %.4f, inverted file %.4f" % (t_exact, t_approx))
    assert t_approx >= t_exact - 0.03


def test_approximate_neighbours_fall_back_for_very_many_neighbours(monkeypatch, capfd):
    """The inverted-file search restricts the register-resident matrix sweep; 1400 neighbours in 100 dimensions
    are more than its candidate lists hold, and the fit then searches exactly (and says so) instead of ending."""
    from tsnecuda import TSNE, synthetic
    X = synthetic.gaussian_clusters(6000, d=100, clusters=3, seed=8)
    Y0 = synthetic_start(X.shape[0])
    kw = dict(perplexity=50.0, num_neighbors=1400, n_iter=4, perplexity_epsilon=1e-4)
    exact = TSNE(**kw).fit_transform(X, y=Y0)
    monkeypatch.setenv("TSNE_KNN", "ivf")
    emb = TSNE(verbose=1, **kw).fit_transform(X, y=Y0)
    out = capfd.readouterr().out
    assert "(inverted file: not for 1400 neighbours, exact search instead)" in out
    assert np.array_equal(emb, exact)


def test_fit_with_adaptive_grid(monkeypatch, capfd):
    """TSNE_ADAPTIVE_BOXES=1: every 50 steps the grid follows the spread of the embedding.  From a start that
    is 160 units wide the first check moves from 130 to 170 boxes; the interpolation error of the repulsive
    forces reported then is lower than with the reference's fixed grid."""
    from tsnecuda import TSNE, synthetic
    X, fit = synthetic.make_config("c0")
    n = X.shape[0]
    Y0 = (np.random.default_rng(2).random((n, 2)) * 160.0 - 80.0).astype(np.float32)
    monkeypatch.setenv("TSNE_REPULSION_MONITOR", "400")
    kw = dict(perplexity=30.0, num_neighbors=90, n_iter=101, verbose=1, print_interval=100, early_exaggeration=1.0,
              learning_rate=1.0, perplexity_epsilon=1e-4)

    def monitored_error():
        TSNE(**kw).fit_transform(X, y=Y0)
        out = capfd.readouterr().out
        line = [l for l in out.split("\n") if l.startswith("[Step 100] Repulsion interpolation error")][0]
        return out, float(line.split("forces ")[1].split(",")[0])

    out_fixed, err_fixed = monitored_error()
    assert "Interpolation grid" not in out_fixed
    monkeypatch.setenv("TSNE_ADAPTIVE_BOXES", "1")
    out_adaptive, err_adaptive = monitored_error()
    assert "[Step 50] Interpolation grid: 170 boxes per dimension (spread " in out_adaptive
    print("repulsion error at step 100: fixed grid %.3g, adaptive %.3g" % (err_fixed, err_adaptive))
    assert err_adaptive < err_fixed


def synthetic_start(n):
    from tsnecuda import synthetic
    return synthetic.initial_embedding(n)


def test_dump_file_format(tmp_path, c0_problem):
    """Text dump: header "N 2" then N lines "x y" per dumped step
    (src/fit_tsne.cu:347-352,563-570)."""
    from tsnecuda import TSNE
    X = c0_problem["X"][:300]
    path = str(tmp_path / "dump.txt")
    emb = TSNE(perplexity=10.0, num_neighbors=30, n_iter=6, dump_points=True, dump_file=path, dump_interval=2,
               perplexity_epsilon=1e-4).fit_transform(X)
    lines = open(path).read().split("\n")
    assert lines[0] == "300 2"
    body = [l for l in lines[1:] if l]
    assert len(body) == 3 * 300  # steps 0, 2, 4
    last = np.array([[float(v) for v in l.split()] for l in body[-300:]])
    assert last.shape == (300, 2) and np.isfinite(last).all()
    assert emb.shape == (300, 2)


def test_min_grad_norm_stops_early(c0_problem, capfd):
    from tsnecuda import TSNE
    X = c0_problem["X"][:500]
    TSNE(perplexity=10.0, num_neighbors=30, n_iter=200, min_grad_norm=1e9, verbose=1,
         perplexity_epsilon=1e-4).fit_transform(X)
    out = capfd.readouterr().out
    assert "Reached minimum gradient norm" in out
    assert "_time_knn:" in out and "total_time:" in out


def test_command_line_program(tmp_path):
    """`tsne` on its built-in two-cluster data set (src/exe/main.cu:172-213): runs RunTsne with the given
    options, prints the reference's progress and timing lines, and dumps every step when asked to.  The
    program seeds its Gaussian start from the clock like the reference's; what is asserted of its own run
    holds for any start (format, counts, finiteness, that the layout grows away from the 1e-4 start), and
    the seeded extension is checked by running the program twice."""
    import subprocess
    exe = os.path.join(REPO, "tsne-cuda_amd", "tsnecuda", "tsne")
    cmd = [exe, "-k", "600", "--dim=8", "-n", "30", "-u", "20", "--perplexity", "8", "-d"]

    def run(where, seed):
        where.mkdir()
        env = {k: v for k, v in os.environ.items() if k != "TSNE_RANDOM_SEED"}
        if seed is not None:
            env["TSNE_RANDOM_SEED"] = seed
        out = subprocess.run(cmd, capture_output=True, text=True, cwd=where, timeout=120, env=env)
        assert out.returncode == 0, out.stderr
        assert "Starting TSNE calculation with 600 points." in out.stdout
        assert "[Step 0] Avg. Gradient Norm:" in out.stdout and "[Step 20] Avg. Gradient Norm:" in out.stdout
        assert "_time_knn:" in out.stdout and "total_time:" in out.stdout
        lines = (where / "dump_ys.txt").read_text().split("\n")
        assert lines[0] == "600 2"
        body = np.array([[float(v) for v in l.split()] for l in lines[1:] if l])
        assert body.shape == (30 * 600, 2) and np.isfinite(body).all()
        return body.reshape(30, 600, 2)

    steps = run(tmp_path / "clock", None)
    # the first dumped step is still the 1e-4 start moved once; thirty exaggerated steps later the layout is larger
    assert np.abs(steps[0]).max() < 1.0
    assert np.abs(steps[-1]).max() > 2.0 * np.abs(steps[0]).max()
    a = run(tmp_path / "seeded_a", "77")
    b = run(tmp_path / "seeded_b", "77")
    # one seed, one start: the first dumped step agrees to the loop's own repeatability
    assert np.abs(a[0] - b[0]).max() <= 1e-3 * np.abs(a[0]).max()
    assert np.abs(a[0] - steps[0]).max() > 1e-3 * np.abs(a[0]).max()


def test_package_smoke_run_with_all_defaults(capfd):
    """tsnecuda.test(): 5000 x 50 uniform random points (float64 input) with
    every keyword at its default (perplexity 50, 32 neighbours, Gaussian start,
    1000 steps), as src/python/tsnecuda/__init__.py:4-7 does."""
    import tsnecuda
    tsnecuda.test()
    out = capfd.readouterr().out
    assert "[Step 0] Avg. Gradient Norm:" in out and "total_time:" in out
    # and the same call returns a finite float32 embedding
    emb = tsnecuda.TSNE().fit_transform(np.random.default_rng(0).random((3000, 20)))
    assert emb.shape == (3000, 2) and emb.dtype == np.float32 and np.isfinite(emb).all()
