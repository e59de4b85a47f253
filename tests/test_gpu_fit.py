"""End-to-end fits through the drop-in entry points on the GPU."""
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


def test_c0_fit_objective_within_one_percent(c0_problem):
    """Config c0, 1000 steps from the seeded initial embedding through
    TSNE.fit_transform (ctypes -> pymodule_tsne -> RunTsne).  Gradient descent
    amplifies fp32 round-off, so trajectories are compared through the objective:
    the KL-style value of the final embedding, evaluated by the same evaluator
    with the oracle's P and exact Z, must be within 1 % of the oracle's own run
    (tests/golden/c0_fit.json)."""
    from tsnecuda import TSNE, synthetic
    c = c0_problem
    with open(os.path.join(GOLDEN, "c0_fit.json")) as f:
        gold = json.load(f)
    Y0 = synthetic.initial_embedding(c["X"].shape[0])
    model = TSNE(perplexity=c["fit"]["perplexity"], num_neighbors=c["K"], learning_rate=c["fit"]["learning_rate"],
                 n_iter=1000, perplexity_epsilon=1e-4)
    emb = model.fit_transform(c["X"], y=Y0)
    assert emb.shape == (5000, 2) and emb.dtype == np.float32 and emb.flags["F_CONTIGUOUS"]
    assert np.isfinite(emb).all()
    kl = oracle.kl(c["P"], c["idx"], flat(emb))
    print("KL gpu %.5f oracle %.5f initial %.5f" % (kl, gold["kl_exact_z"], gold["kl_initial"]))
    assert abs(kl - gold["kl_exact_z"]) <= 0.01 * gold["kl_exact_z"]
    # the library's own evaluation of the same embedding (interpolated Z, its own P) agrees with the
    # oracle's evaluator (exact Z, oracle P)
    assert abs(model.kl_divergence_ - kl) <= 2e-3 * kl
    # same overall scale of the layout
    assert 0.8 < (emb.max() - emb.min()) / (gold["extent"][1] - gold["extent"][0]) < 1.25
    # and the same neighbourhood preservation, by an implementation that shares nothing with this build
    from sklearn.manifold import trustworthiness
    t = trustworthiness(c["X"], emb, n_neighbors=12)
    print("trustworthiness gpu %.4f oracle %.4f" % (t, gold["trustworthiness_k12"]))
    assert abs(t - gold["trustworthiness_k12"]) <= 0.01


@pytest.mark.parametrize("name", ["c1", "c2"])
def test_larger_configs_objective_within_one_percent(name):
    """Configs c1 (60000 x 784 pixel-like) and c2 (50000 x 1024 feature-like), 1000
    steps from the seeded start: the objective of the final embedding (exact Z,
    evaluated by the oracle on the neighbours and P of the GPU stages, which are
    compared with the oracle's elsewhere) within 1 % of the oracle's own run, and
    the trustworthiness of a fixed 4000-point subsample within 0.02 of it
    (tests/golden/c1_fit.json, c2_fit.json)."""
    from sklearn.manifold import trustworthiness
    from tsnecuda import TSNE, stages, synthetic
    with open(os.path.join(GOLDEN, "%s_fit.json" % name)) as f:
        gold = json.load(f)
    X, fit = synthetic.make_config(name)
    n, k = X.shape[0], fit["num_neighbors"]
    Y0 = synthetic.initial_embedding(n)
    model = TSNE(perplexity=fit["perplexity"], num_neighbors=k, learning_rate=fit["learning_rate"], n_iter=1000,
                 perplexity_epsilon=1e-4)
    emb = model.fit_transform(X, y=Y0)
    assert emb.shape == (n, 2) and np.isfinite(emb).all()
    idx, d2 = stages.knn(torch.from_numpy(X).cuda(), k)
    P = stages.symmetrize(stages.perplexity(stages.max_normalize_(d2), fit["perplexity"], 1e-4), idx)
    kl = oracle.kl(P.cpu().numpy(), idx.cpu().numpy(), flat(emb))
    sub = np.sort(np.random.default_rng(0).choice(n, size=4000, replace=False))  # as tests/golden/make_golden.py
    t = trustworthiness(X[sub], emb[sub], n_neighbors=12)
    print("%s: KL gpu %.5f oracle %.5f (library's own %.5f), trustworthiness gpu %.4f oracle %.4f"
          % (name, kl, gold["kl_exact_z"], model.kl_divergence_, t, gold["trustworthiness_k12_subsample4000"]))
    assert abs(kl - gold["kl_exact_z"]) <= 0.01 * gold["kl_exact_z"]
    assert abs(model.kl_divergence_ - kl) <= 5e-3 * kl
    assert abs(t - gold["trustworthiness_k12_subsample4000"]) <= 0.02
    assert 0.8 < (emb.max() - emb.min()) / (gold["extent"][1] - gold["extent"][0]) < 1.25


def test_fit_is_repeatable_for_a_given_start(c0_problem):
    """Two short fits from the same start agree closely.  Not bitwise: the
    charge spreading and the Z reduction use floating-point atomics, and the
    early exaggerated steps amplify that round-off quickly, hence 10 steps.
    The update rule itself is discontinuous (a coordinate's gain grows or shrinks
    with the sign of gradient times momentum): where that product is zero to
    rounding, two runs may take different branches for that coordinate, which then
    moves differently and pulls its neighbours along - seen for one coordinate in
    4000 here, five steps before the end - so nearly all coordinates must agree to a
    per cent of the embedding's extent and the whole to two per cent."""
    from tsnecuda import TSNE, synthetic
    X = c0_problem["X"][:2000]
    Y0 = synthetic.initial_embedding(2000, seed=9)
    kw = dict(perplexity=20.0, num_neighbors=60, n_iter=10, perplexity_epsilon=1e-4)
    a = TSNE(**kw).fit_transform(X, y=Y0)
    b = TSNE(**kw).fit_transform(X, y=Y0)
    close = np.abs(a - b) <= 1e-2 * np.abs(a).max()
    assert close.mean() >= 0.99
    assert np.linalg.norm(a - b) <= 2e-2 * np.linalg.norm(a)


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
    run = subprocess.run([exe, str(n), "4", str(kind), str(seed), "0", str(out)], capture_output=True, text=True,
                         timeout=120)
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


def test_renumbering_is_invisible_to_the_caller(monkeypatch):
    """RunTsne renumbers 16384 or more points in locality order on entry and
    restores the caller's numbering on exit: a short fit gives the same
    embedding, row for row, with the renumbering switched off."""
    from tsnecuda import TSNE, synthetic
    n = 20000
    X = synthetic.gaussian_clusters(n, d=16, clusters=5, seed=11)
    Y0 = synthetic.initial_embedding(n, seed=4)
    kw = dict(perplexity=20.0, num_neighbors=60, n_iter=15, perplexity_epsilon=1e-4)
    monkeypatch.setenv("TSNE_LOCALITY_ORDER", "1")
    a = TSNE(**kw).fit_transform(X, y=Y0)
    snaps = TSNE(return_style="snapshots", num_snapshots=3, **kw).fit_transform(X, y=Y0)
    monkeypatch.setenv("TSNE_LOCALITY_ORDER", "0")
    b = TSNE(**kw).fit_transform(X, y=Y0)
    assert np.linalg.norm(a - b) <= 1e-3 * np.linalg.norm(b)
    assert np.linalg.norm(snaps[-1] - b) <= 1e-3 * np.linalg.norm(b)
    # the first snapshot is the embedding after one step: still close to the start, row for row
    assert np.abs(snaps[0] - Y0).max() < 1e-2


@pytest.mark.parametrize("n,d,k,clusters", [
    (16385, 7, 30, 3),    # just above the renumbering threshold, odd count (scalar update kernel)
    (20001, 3, 90, 1),    # one blob: nothing for the kNN sweep to skip
    (8192, 126, 16, 4),   # smallest matrix-sweep problem, largest matrix-sweep dimension
    (8195, 127, 16, 4),   # one dimension more: chunked matrix sweep
    (17000, 300, 30, 5),  # chunked matrix sweep on renumbered points, margin tried on a sample of query tiles
    (40000, 50, 40, 6),   # several column partitions and strips, clustered
    (12000, 10, 1023, 3),  # the neighbour count of the reference's C++ default options
])
def test_whole_pipeline_against_the_oracle(n, d, k, clusters):
    """RunTsne end to end (renumbering, kNN, P, eight gradient steps, numbering
    restored) against the oracle's pipeline from the same explicit start: row
    for row, to the loop's own repeatability."""
    from tsnecuda import TSNE, synthetic
    X = synthetic.gaussian_clusters(n, d=d, clusters=clusters, center_scale=5.0, seed=n + d)
    Y0 = synthetic.initial_embedding(n, seed=k)
    # a perplexity close to the neighbour count: in high dimension the normalised distances of a row are
    # nearly equal, and concentrating them on few neighbours needs precisions at which exp(-beta d)
    # underflows fp32 -- rows on which the reference's own search is ill-conditioned
    perp = min(30.0, (k - 1) / 1.6)
    emb = TSNE(perplexity=perp, num_neighbors=k, n_iter=8, perplexity_epsilon=1e-4).fit_transform(X, y=Y0)
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]]).astype(np.float32)
    y_o, _, _, _ = oracle.fit(X, y0, k, perp, eps=1e-4, iterations=8)
    got = flat(emb)
    assert np.isfinite(got).all()
    assert np.linalg.norm(got - y_o) <= 2e-3 * np.linalg.norm(y_o)


def test_command_line_program(tmp_path):
    """`tsne` on its built-in two-cluster data set (src/exe/main.cu:172-213):
    runs RunTsne with the given options, prints the reference's progress and
    timing lines, and dumps every step when asked to."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tsne-cuda_amd", "tsnecuda", "tsne")
    out = subprocess.run([exe, "-k", "600", "--dim=8", "-n", "30", "-u", "20", "--perplexity", "8", "-d"],
                         capture_output=True, text=True, cwd=tmp_path, timeout=120)
    assert out.returncode == 0, out.stderr
    assert "Starting TSNE calculation with 600 points." in out.stdout
    assert "[Step 0] Avg. Gradient Norm:" in out.stdout and "_time_knn:" in out.stdout
    lines = (tmp_path / "dump_ys.txt").read_text().split("\n")
    assert lines[0] == "600 2"
    body = np.array([[float(v) for v in l.split()] for l in lines[1:] if l])
    assert body.shape == (30 * 600, 2) and np.isfinite(body).all()
    # two well separated clusters of 300 points: after 30 exaggerated steps each half is closer to its own
    # centroid than to the other's
    last = body[-600:]
    a, b = last[:300].mean(0), last[300:].mean(0)
    own = np.linalg.norm(last[:300] - a, axis=1) < np.linalg.norm(last[:300] - b, axis=1)
    assert own.mean() > 0.95


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
