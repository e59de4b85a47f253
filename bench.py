#!/usr/bin/env python3
"""Benchmark of the FIt-SNE gradient pipeline on one MI355X.

A "step" is one gradient iteration (repulsive + attractive forces + update) of
the 1,000,000 x 50 configuration (config c3) with the inputs resident in HBM.
Prints ONE JSON line: gradient iterations per second, plus per-phase times of
the one-shot stages, the end-to-end fit time through the drop-in entry point,
the roofline of the dominant kernel (attractive forces, HBM-bound) and the CPU
baseline (the oracle's gradient loop on the host cores, bounded sample).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3] [--points N]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "tsne-cuda_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def traffic_from_profile(path):
    """HBM bytes per launch of the attractive kernel from the committed rocprofv3 summary: the per-kernel
    averages of its FETCH_SIZE and WRITE_SIZE passes, each scaled by what the same counter read for the plain
    256 MiB device copies of the same run (262144 KiB read and written per launch; the summary lists them as
    `calibration_copy_256MiB`)."""
    if not os.path.exists(path):
        return None, None
    avg, copy_max = {}, {}
    for line in open(path):
        f = line.split()
        if len(f) < 5 or f[-4] not in ("FETCH_SIZE", "WRITE_SIZE"):
            continue
        try:
            a, m = float(f[-2]), float(f[-1])
        except ValueError:
            continue
        if f[0].startswith("attractive_blocked_kernel"):
            avg[f[-4]] = a
        elif f[0] == "calibration_copy_256MiB":
            copy_max[f[-4]] = a
    if set(avg) != {"FETCH_SIZE", "WRITE_SIZE"} or set(copy_max) != {"FETCH_SIZE", "WRITE_SIZE"}:
        return None, None
    kib = 262144.0  # one calibration copy
    total = sum(avg[c] * (kib / copy_max[c]) * 1024.0 for c in avg)
    return total, "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes over this command, profiles/" + os.path.basename(path)


def profile_commit(path):
    """The commit the counter summary says it was taken at (a line `commit: <hash>` in the file), so that a
    summary older than the kernel it describes is visible in the bench line."""
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.lower().startswith("commit:"):
            return line.split(":", 1)[1].strip()
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--points", type=int, default=None, help="override the point count of the workload")
    ap.add_argument("--no-fit", action="store_true", help="skip the end-to-end fit through pymodule_tsne")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-approx", action="store_true", help="skip the timing of the optional approximate neighbour search")
    ap.add_argument("--no-overlap", action="store_true",
                    help="run the repulsive chain and the attractive kernel one after the other (TSNE_OVERLAP=0): "
                         "per-kernel durations in a trace then are those of kernels running alone")
    ap.add_argument("--repeats", type=int, default=5,
                    help="times the stretch of --steps steps is timed (each bracketed by a device synchronisation "
                         "on both sides); the median is reported")
    ap.add_argument("--fit-repeats", type=int, default=3, help="end-to-end fits timed (the median is reported)")
    ap.add_argument("--no-small", action="store_true",
                    help="skip the end-to-end fits of the smaller configurations (c0, c1, c2) and the CPU fit of c0")
    ap.add_argument("--cpu-steps", type=int, default=150, help="gradient steps of the CPU baseline sample")
    ap.add_argument("--cpu-knn-rows", type=int, default=4096, help="query rows of the CPU baseline's kNN sample")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run 10 plain 256 MiB device copies (known traffic, to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is single-GPU (one MI355X per process, no collectives); run with --gpus 1")
    if args.no_overlap:
        os.environ["TSNE_OVERLAP"] = "0"  # read once by the library, at its first gradient step

    import numpy as np
    import torch
    from tsnecuda import TSNE, stages, synthetic

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    stages.lib()  # fails loudly if libtsnecuda.so is missing

    t0 = time.time()
    X, fit = synthetic.make_config(args.workload, n=args.points)
    n, d = X.shape
    k = min(fit["num_neighbors"], n)
    Y0 = synthetic.initial_embedding(n)
    y0 = np.concatenate([Y0[:, 0], Y0[:, 1]])
    gen_s = time.time() - t0

    def timed(fn):
        torch.cuda.synchronize()
        a = time.perf_counter()
        out = fn()
        torch.cuda.synchronize()
        return out, time.perf_counter() - a

    # ---- one-shot stages, inputs resident in HBM -------------------------
    # As RunTsne does on entry, the points are renumbered in locality order first
    # (the numbering is arbitrary; kNN and the attractive kernel run faster on it).
    dX = torch.from_numpy(X).cuda()
    order, order_s = timed(lambda: stages.locality_order(dX))
    dXs, gather_s = timed(lambda: stages.gather_rows(dX, order))
    del dX
    (idx, d2, knn_stats), knn_s = timed(lambda: stages.knn_select(dXs, k, 0))  # 0: what tsne_hip_knn does
    # The optional approximate search (inverted file, floor(sqrt(N)) lists as the reference's FAISS index, 100
    # lists probed per list: what TSNE_KNN=ivf runs): training and search timed, recall against the exact rows.
    approx = None
    if d <= 126 and n >= 4096 and not args.no_approx:
        import math
        nlist = int(math.isqrt(n))
        cen, train_s = timed(lambda: stages.ivf_train(dXs, nlist))
        (idx_a, _, stats_a), search_s = timed(lambda: stages.knn_ivf(dXs, k, cen, min(100, nlist)))
        rows = torch.arange(0, n, max(1, n // 4096), device="cuda")[:4096]
        hits = (idx_a[rows, 1:, None] == idx[rows, None, 1:]).any(2).float().mean().item()
        approx = {"nlist": nlist, "nprobe_per_list": min(100, nlist), "train_s": train_s, "search_s": search_s,
                  "recall_at_%d" % (k - 1): hits, "recall_rows": int(rows.numel()),
                  "tile_pairs_per_mille": stats_a[2]}
        del idx_a, cen
    del dXs
    order_h = order.cpu().numpy().astype(np.int64)
    y0 = np.concatenate([y0[:n][order_h], y0[n:][order_h]])
    _, norm_s = timed(lambda: stages.max_normalize_(d2))
    cond, perp_s = timed(lambda: stages.perplexity(d2, fit["perplexity"], 1e-4))
    P, sym_s = timed(lambda: stages.symmetrize(cond, idx))
    # (the optional full form, (A + A^T) / 2N with the union pattern as CSR: timed for its roofline row only)
    (_, csr_col, _), sym_full_s = timed(lambda: stages.symmetrize_full(cond, idx))
    nnz_sym = int(csr_col.numel())
    del cond, d2, csr_col

    # ---- gradient loop ----------------------------------------------------
    plan = stages.Plan(n, k)
    _, reblock_s = timed(lambda: plan.prepare_attractive(P, idx))
    y = torch.from_numpy(y0).cuda()
    gains, old = torch.ones_like(y), torch.zeros_like(y)
    eta = fit["learning_rate"]
    _, warm_s = timed(lambda: plan.iterate_(None, None, y, gains, old, 0, args.warmup, eta=eta))
    # EXACTLY --steps steps per timed stretch, consecutive stretches of the same fit; the median stretch is reported.
    loop_runs, done = [], args.warmup
    for _ in range(max(1, args.repeats)):
        z, run_s = timed(lambda: plan.iterate_(None, None, y, gains, old, done, done + args.steps, eta=eta))
        loop_runs.append(run_s)
        done += args.steps
    loop_s = sorted(loop_runs)[len(loop_runs) // 2]
    ms_per_step = loop_s * 1e3 / args.steps
    iters_per_s = args.steps / loop_s

    # ---- per-kernel durations: a pair of HIP events per launch (the kernel's own start and end), handed to
    # every kernel of a further stretch of the same loop by the library ----
    prof_steps = min(args.steps, 200)
    plan.profile_begin()
    plan.iterate_(None, None, y, gains, old, done, done + prof_steps, eta=eta)
    prof = plan.profile_end()
    kernels_us = {name: 1e3 * ms / max(cnt, 1) for name, (ms, cnt) in prof.items()}
    done += prof_steps
    # ... and the dominant kernel's duration as the product runs it: beside the repulsive chain on the other
    # stream (a pair of HIP events around that kernel alone, on the stream it is launched on).
    overlapped_ms = None
    if not args.no_overlap:
        plan.profile_attractive_begin()
        plan.iterate_(None, None, y, gains, old, done, done + prof_steps, eta=eta)
        total_ms, launches = plan.profile_attractive_end()
        done += prof_steps
        overlapped_ms = total_ms / launches if launches else None
    # ---- a stretch late in the fit: past the end of the early exaggeration (step 250), where the embedding has
    # spread out and the grouping of the points by grid tile lasts longer than in the first hundred steps ----
    late_from = max(done, 300)
    plan.iterate_(None, None, y, gains, old, done, late_from, eta=eta)
    late_runs, done = [], late_from
    for _ in range(max(1, args.repeats)):
        z, run_s = timed(lambda: plan.iterate_(None, None, y, gains, old, done, done + args.steps, eta=eta))
        late_runs.append(run_s)
        done += args.steps
    late_s = sorted(late_runs)[len(late_runs) // 2]
    attr_ms = kernels_us["attractive_kernel"] * 1e-3  # start-to-end events of whichever attractive kernel ran
    attr_bytes = 8.0 * n * k + 16.0 * n  # P and index streams; read positions, write forces
    achieved = attr_bytes / (attr_ms * 1e-3) / 1e9

    # ---- every phase against its roofline -----------------------------------
    # Algorithmic bytes per launch of the loop's kernels (G = 390 interpolation nodes per side, four charge
    # planes; the transposed spectra are 2 plane pairs x 800 x 512 complex; 21 fixed-point moments per box).
    G2, spectra, moments = 390.0 * 390.0, 2 * 800 * 512 * 8.0, 21 * 130 * 130 * 8.0
    loop_bytes = {
        "tile_count_kernel": 12.0 * n,                      # positions in, (tile, rank) codes out
        "tile_scatter_kernel": 20.0 * n,                    # positions and codes in, positions grouped by tile out
        "spread_kernel": 8.0 * n + moments,                 # grouped positions in, box moments out
        "conv_rows_forward_kernel": moments + spectra,      # box moments in (-> node charges), row spectra out
        "conv_columns_kernel": 2.0 * spectra + moments,     # row spectra in, convolved columns out, box moments cleared
        "conv_rows_inverse_kernel": spectra + 16.0 * G2,    # in, node potentials out
        "gather_forces_kernel": 16.0 * n + 16.0 * G2,       # positions and node potentials in, forces out
        "attractive_kernel": attr_bytes,
        "update_kernel": 72.0 * n,                          # 5 arrays of 2N in, 4 out (incl. the packed copy)
    }
    phase_rooflines = {
        name: {"bound": "hbm", "bytes": b, "achieved": b / (kernels_us[name] * 1e-6) / 1e9, "unit": "GB/s",
               "frac": b / (kernels_us[name] * 1e-6) / 1e9 / HBM_PEAK_GBS}
        for name, b in loop_bytes.items() if kernels_us.get(name)}
    if knn_stats[0] == 1:
        # Flop the matrix sweep executed per tile pair it did not skip: three products of bf16 terms
        # (v_mfma_f32_32x32x16_bf16) over the dimensions + 3, padded to 16 (up to 125 dimensions) or to 32 (chunked
        # sweep, beyond 126); at exactly 126 dimensions float products over 128 (v_mfma_f32_32x32x2_f32).
        tiles = -(-n // 128)
        if d == 126:
            per_pair, peak, pipe = 2.0 * 128 * 128 * 128, 157.3, "fp32"
        else:
            pad = 16 if d + 3 <= 128 else 32
            per_pair, peak, pipe = 2.0 * 128 * 128 * 3 * (-(-(d + 3) // pad) * pad), 2500.0, "bf16"
        flop = per_pair * tiles * tiles * knn_stats[2] / 1000.0
        phase_rooflines["knn"] = {"bound": "mfma", "flop": flop, "achieved": flop / knn_s / 1e12, "unit": "TFLOP/s",
                                  "frac": flop / knn_s / 1e12 / peak, "tile_pairs_per_mille": knn_stats[2],
                                  "note": pipe + " matrix peak; time of the whole kNN call (sweep, re-rank, packing)"}

    # One-shot stages that are HBM problems (algorithmic bytes: what the stage must read and write once).
    nnz = float(n) * k
    for name, secs, b in (("perplexity", perp_s, 8.0 * nnz), ("symmetrize", sym_s, 12.0 * nnz),
                          ("symmetrize_full", sym_full_s, 8.0 * nnz + 8.0 * nnz_sym + 4.0 * (n + 1))):
        phase_rooflines[name] = {"bound": "hbm", "bytes": b, "achieved": b / secs / 1e9, "unit": "GB/s",
                                 "frac": b / secs / 1e9 / HBM_PEAK_GBS}
    phase_rooflines["symmetrize_full"]["nnz"] = nnz_sym

    if args.calibrate:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- end-to-end fit through the drop-in entry point (host buffers) ----
    fit_s, fit_runs, kl_final = None, [], None
    if not args.no_fit:
        model = TSNE(perplexity=fit["perplexity"], num_neighbors=k, learning_rate=eta, n_iter=1000,
                     perplexity_epsilon=1e-4)
        fit_runs = []
        for _ in range(args.fit_repeats):
            a = time.perf_counter()
            emb = model.fit_transform(X, y=Y0)
            fit_runs.append(time.perf_counter() - a)
        fit_s = sorted(fit_runs)[len(fit_runs) // 2]  # median; the stages above have warmed the library up
        kl_final = model.kl_divergence_
        assert np.isfinite(emb).all()

    # ---- CPU baseline: the oracle's gradient loop on the host cores -------
    cpu = None
    if not args.no_cpu:
        import oracle
        P_h, idx_h = P.cpu().numpy(), idx.cpu().numpy()
        a = time.perf_counter()
        oracle.iterate(P_h, idx_h, y0, args.cpu_steps, eta=eta)
        cpu_s = time.perf_counter() - a
        # ... and its exact kNN on a slice of the query rows against all points.
        knn_rows = min(n, args.cpu_knn_rows)
        a = time.perf_counter()
        oracle.knn(X, k, rows=(0, knn_rows))
        knn_cpu_s = time.perf_counter() - a
        cpu = {"value": args.cpu_steps / cpu_s, "unit": "iter/s", "cores": oracle.num_threads(), "kind": "port",
               "sample": "%d gradient steps of the same %d x %d workload (P and neighbours from the GPU stages) and "
                         "the exact kNN of %d query rows against all %d points, C++/OpenMP restatement"
                         % (args.cpu_steps, n, k, knn_rows, n),
               "knn_query_rows_per_s": knn_rows / knn_cpu_s,
               "fit_seconds_extrapolated": n / (knn_rows / knn_cpu_s) + 1000.0 / (args.cpu_steps / cpu_s)}

    # The CPU oracle's own 1000-step fit of the same configuration from the same start (a fixture: the fit
    # takes an hour of CPU time at 1M points), for the objective of the GPU fit to stand beside.
    oracle_kl = None
    gold_path = os.path.join(ROOT, "tests", "golden", "%s_fit.json" % args.workload)
    if args.points is None and os.path.exists(gold_path):
        with open(gold_path) as f:
            oracle_kl = json.load(f).get("kl_exact_z")

    # HBM bytes per launch of the dominant kernel: not measurable from inside this process (it takes two
    # rocprofv3 counter passes), so it is read from the committed summary of those passes over this same
    # command; the counters belong to that exact workload, so other sizes - or a missing summary - report null.
    traffic, traffic_source, traffic_commit = None, None, None
    if args.workload == "c3" and n == 1000000 and k == 90:
        prof_path = os.path.join(ROOT, "profiles", "bench_c3_1M_hbm_counters.txt")
        traffic, traffic_source = traffic_from_profile(prof_path)
        traffic_commit = profile_commit(prof_path)

    # ---- the smaller configurations end to end, and c0 in full on the CPU ----
    small = None
    if not args.no_small and args.points is None:
        small = {}
        for name in ("c0", "c1", "c2"):
            Xc, fc = synthetic.make_config(name)
            Yc = synthetic.initial_embedding(Xc.shape[0])
            mc = TSNE(perplexity=fc["perplexity"], num_neighbors=fc["num_neighbors"], learning_rate=fc["learning_rate"],
                      n_iter=1000, perplexity_epsilon=1e-4)
            runs = []
            for _ in range(3):
                a = time.perf_counter()
                mc.fit_transform(Xc, y=Yc)
                runs.append(time.perf_counter() - a)
            small[name] = {"shape": "%d x %d" % Xc.shape, "gpu_fit_seconds": sorted(runs)[1],
                           "kl_divergence": mc.kl_divergence_}
            if name == "c0" and not args.no_cpu:
                # The configuration the reference's CPU path is quoted on, run in full on the host cores.
                import oracle
                yc = np.concatenate([Yc[:, 0], Yc[:, 1]])
                a = time.perf_counter()
                _, _, idx_c, P_c = oracle.fit(Xc, yc, fc["num_neighbors"], fc["perplexity"], eps=1e-4, iterations=1000,
                                              eta=fc["learning_rate"])
                small[name]["cpu_fit_seconds"] = time.perf_counter() - a
                small[name]["cpu_cores"] = oracle.num_threads()
            del Xc
    out = {
        "metric": "gradient_iters_per_sec",
        "value": iters_per_s,
        "unit": "iter/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%s: %d x %d fp32, perplexity %g, K=%d, lr %g; step = one gradient iteration"
                               % (args.workload, n, d, fit["perplexity"], k, eta)},
        "loop_seconds_runs": loop_runs,
        "late_ms_per_step": late_s * 1e3 / args.steps,
        "late_iters_per_sec": args.steps / late_s,
        "late_stretch": "steps %d-%d of the same fit (exaggeration 1, momentum 0.8), median of %d stretches of %d"
                        % (late_from, done, len(late_runs), args.steps),
        "fit_seconds": fit_s,
        "fit_seconds_runs": fit_runs,
        "smaller_configs": small,
        "fit_kl_divergence": kl_final,
        "fit_kl_divergence_oracle": oracle_kl,
        "phases_s": {"locality_order": order_s + gather_s, "knn": knn_s, "max_normalize": norm_s, "perplexity": perp_s, "symmetrize": sym_s,
                     "symmetrize_full_csr": sym_full_s, "reblock_pattern": reblock_s,
                     "gradient_loop_%d_steps" % args.steps: loop_s, "data_generation_host": gen_s},
        "roofline": {"bound": "hbm", "kernel": "attractive_blocked_kernel", "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": traffic_source, "traffic_profile_commit": traffic_commit,
                     "bytes_per_launch": attr_bytes, "ms_per_launch": attr_ms,
                     "overlapped_ms_per_launch": overlapped_ms,
                     "overlapped_frac": (attr_bytes / (overlapped_ms * 1e-3) / 1e9 / HBM_PEAK_GBS) if overlapped_ms else None},
        "kernels_us": kernels_us,
        "phase_rooflines": phase_rooflines,
        "knn_approximate": approx,
        "cpu_baseline": cpu,
        "final_Z": float(z.item()),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
