// Host orchestration of the whole fit: tsnecuda::RunTsne, GpuOptions, and the
// extern "C" pymodule_tsne shim.
//
// Follows the stage order, schedule, outputs and messages of the reference's
// src/fit_tsne.cu:16-627 and src/ext/pymodule_ext.cu:6-123.  What differs is
// where data lives: the points go to the GPU once, neighbour indices,
// distances and probabilities never come back to the host, and the gradient
// loop enqueues whole stretches of steps without a host round trip (the
// reference reads min/max and Z back every step).
#include <chrono>
#include <cmath>
#include <cstring>
#include <fstream>
#include <iostream>
#include <random>
#include <string>
#include <vector>

#include "../../include/tsnecuda/fit_tsne.h"
#include "../../include/tsnecuda/pymodule_ext.h"
#include "../../include/tsnecuda/tsne_stages.h"
#include "plan.h"
#include "stages.h"

namespace {

// GPU or library failure: message and exit, the reference's convention
// (src/util/cuda_utils.cu:235-246).
[[noreturn]] void die(const char *what) {
    std::cerr << "E: " << what << ": " << tsnehip::last_error() << std::endl;
    std::exit(1);
}
#define TSNE_OR_DIE(call, what) \
    do {                        \
        if ((call) != 0) die(what); \
    } while (0)

void hip_or_die(hipError_t e, const char *what) {
    if (e != hipSuccess) {
        tsnehip::set_error("%s", hipGetErrorString(e));
        die(what);
    }
}

struct DeviceBuffer {
    void *ptr = nullptr;
    DeviceBuffer() {}
    explicit DeviceBuffer(size_t bytes) { hip_or_die(hipMalloc(&ptr, bytes ? bytes : 1), "device allocation"); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    ~DeviceBuffer() { release(); }
    void release() {
        if (ptr) (void)hipFree(ptr);
        ptr = nullptr;
    }
    void swap(DeviceBuffer &other) { std::swap(ptr, other.ptr); }
    template <typename T>
    T *as() const {
        return static_cast<T *>(ptr);
    }
};

struct PhaseClock {
    std::chrono::high_resolution_clock::time_point t0;
    void start() { t0 = std::chrono::high_resolution_clock::now(); }
    double stop() {
        return std::chrono::duration<double>(std::chrono::high_resolution_clock::now() - t0).count();
    }
};

thread_local double g_last_kl = -1.0;

int env_int(const char *name, int fallback) {
    const char *v = std::getenv(name);
    return v ? std::atoi(v) : fallback;
}

}  // namespace

namespace tsnecuda {

GpuOptions::GpuOptions(int device) {
    this->device = device;
    hipDeviceProp_t prop;
    hip_or_die(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    hip_or_die(hipSetDevice(device), "hipSetDevice");
    warp_size = prop.warpSize;
    sm_count = prop.multiProcessorCount;
    // Runtime overrides and clamping as in src/include/options.h:352-374.
    integration_kernel_threads = env_int("TSNE_INTEG_THREADS", integration_kernel_threads);
    integration_kernel_factor = env_int("TSNE_INTEG_FACTOR", integration_kernel_factor);
    fft_kernel_threads = env_int("TSNE_FFT_THREADS", fft_kernel_threads);
    attr_kernel_threads = env_int("TSNE_ATTR_THREADS", attr_kernel_threads);
    rep_kernel_threads = env_int("TSNE_REP_THREADS", rep_kernel_threads);
    const int cap = prop.maxThreadsPerBlock;
    auto clamp = [cap](int t) { return t < 1 ? 1 : (t > cap ? cap : t); };
    integration_kernel_threads = clamp(integration_kernel_threads);
    fft_kernel_threads = clamp(fft_kernel_threads);
    attr_kernel_threads = clamp(attr_kernel_threads);
    rep_kernel_threads = clamp(rep_kernel_threads);
    if (integration_kernel_factor < 1) integration_kernel_factor = 1;
}

void RunTsne(Options &opt, GpuOptions &gpu_opt) {
    if (!opt.validate()) {
        std::cout << "E: Invalid options file. Terminating." << std::endl;
        return;
    }
    const bool verbose = opt.verbosity > 0;
    PhaseClock clock, wall;
    wall.start();
    double t_init = 0, t_knn = 0, t_sym = 0, t_low = 0, t_fft = 0, t_rep = 0, t_attr = 0, t_apply = 0,
           t_other = 0;

    clock.start();
    if (verbose) std::cout << "Initializing HIP device... " << std::flush;
    hip_or_die(hipSetDevice(gpu_opt.device), "hipSetDevice");
    hipStream_t stream = nullptr;  // default stream, as the reference

    const int N = opt.num_points;
    const int D = opt.num_dims;
    const int K = opt.num_neighbors < N ? opt.num_neighbors : N;  // src/fit_tsne.cu:84
    const size_t nnz = (size_t)N * K;

    int snap_num = 0, snap_interval = 1;
    if (opt.return_style == RETURN_STYLE::SNAPSHOT) snap_interval = opt.iterations / (opt.num_snapshots - 1);
    if (snap_interval < 1) snap_interval = 1;

    DeviceBuffer d_points(sizeof(float) * (size_t)N * D);
    hip_or_die(hipMemcpy(d_points.ptr, opt.points, sizeof(float) * (size_t)N * D, hipMemcpyHostToDevice),
               "copy of the input points");
    // Renumber the points so that neighbours in the input space get close
    // numbers (the kNN sweep and the attractive kernel are faster that way);
    // the caller's numbering is restored wherever an embedding leaves this
    // function.  order[new] = old.  TSNE_LOCALITY_ORDER=0 keeps the numbering.
    std::vector<int> order;
    bool renumbered = false;
    if (env_int("TSNE_LOCALITY_ORDER", 1) != 0 && tsnehip::locality_pivot_count(N) > 0) {
        TSNE_OR_DIE(tsnehip::locality_order(d_points.as<float>(), N, D, order, stream), "locality ordering");
        DeviceBuffer d_order(sizeof(int) * (size_t)N), d_sorted(sizeof(float) * (size_t)N * D);
        hip_or_die(hipMemcpy(d_order.ptr, order.data(), sizeof(int) * (size_t)N, hipMemcpyHostToDevice),
                   "copy of the point order");
        TSNE_OR_DIE(tsnehip::launch_gather_rows(d_points.as<float>(), d_order.as<int>(), N, D, d_sorted.as<float>(),
                                                stream),
                    "point renumbering");
        hip_or_die(hipStreamSynchronize(stream), "point renumbering");
        d_points.swap(d_sorted);
        renumbered = true;
    }
    // Embeddings cross this boundary as 2N floats, xs then ys, in the caller's numbering.
    std::vector<float> h_swap;
    auto to_internal = [&](std::vector<float> &emb) {
        if (!renumbered) return;
        h_swap.resize(emb.size());
        for (int i = 0; i < N; ++i) {
            h_swap[i] = emb[order[i]];
            h_swap[(size_t)N + i] = emb[(size_t)N + order[i]];
        }
        emb.swap(h_swap);
    };
    auto to_caller = [&](const float *internal, float *out) {
        if (!renumbered) {
            if (out != internal) std::memcpy(out, internal, sizeof(float) * 2 * (size_t)N);
            return;
        }
        for (int i = 0; i < N; ++i) {
            out[order[i]] = internal[i];
            out[(size_t)N + order[i]] = internal[(size_t)N + i];
        }
    };
    t_init = clock.stop();

    // ---- neighbours ------------------------------------------------------
    clock.start();
    if (verbose) std::cout << "done.\nKNN Computation... " << std::flush;
    DeviceBuffer d_idx(sizeof(int) * nnz), d_dist(sizeof(float) * nnz), d_scratch(sizeof(float));
    // Exact by default.  Options::approximate_neighbors or TSNE_KNN=ivf: inverted file with floor(sqrt(N)) lists,
    // as the reference's FAISS search (src/util/distance_utils.cu:85-120); wider inputs than it takes stay exact.
    const char *knn_env = std::getenv("TSNE_KNN");
    const bool approximate = (opt.approximate_neighbors || (knn_env && std::string(knn_env) == "ivf")) && D <= 126 &&
                             N >= 4096;
    bool searched = false;
    if (approximate) {
        int nprobe = env_int("TSNE_KNN_NPROBE", opt.knn_nprobe);
        if (nprobe <= 0) nprobe = 100;
        int nlist = 0, knn_stats[3] = {0, 0, 0};
        const int rc = tsnehip::run_knn_approximate(d_points.as<float>(), N, D, K, nprobe, d_idx.as<int>(),
                                                    d_dist.as<float>(), &nlist, knn_stats, stream);
        // (neighbour counts whose candidate lists the restricted sweep cannot hold keep the exact search)
        if (rc != 0 && rc != tsnehip::kShapeNotSupported) TSNE_OR_DIE(rc, "approximate kNN");
        searched = rc == 0;
        if (verbose && searched)
            std::cout << "(inverted file: " << nlist << " lists, " << std::min(nprobe, nlist) << " probed per list, "
                      << knn_stats[2] << " per mille of the tile pairs compared) " << std::flush;
        if (verbose && !searched)
            std::cout << "(inverted file: not for " << K << " neighbours, exact search instead) " << std::flush;
    }
    if (!searched) {
        TSNE_OR_DIE(tsnehip::run_knn(d_points.as<float>(), N, D, K, d_idx.as<int>(), d_dist.as<float>(), stream),
                    "kNN");
    }
    d_points.release();
    TSNE_OR_DIE(tsnehip::launch_max_normalize(d_dist.as<float>(), (int64_t)nnz, d_scratch.as<float>(), stream),
                "max-normalisation");
    hip_or_die(hipStreamSynchronize(stream), "kNN");
    t_knn = clock.stop();

    // ---- P matrix --------------------------------------------------------
    clock.start();
    if (verbose) std::cout << "done.\nComputing Pij matrix... " << std::endl;
    // TSNE_SYMMETRIZE=full (or Options::full_symmetrization): P = (A + A^T) / 2N with the union pattern, in CSR
    // form, instead of the reference's pattern-restricted form; the attractive forces then run over the CSR rows.
    const char *sym_env = std::getenv("TSNE_SYMMETRIZE");
    const bool full_sym = opt.full_symmetrization || (sym_env && std::string(sym_env) == "full");
    DeviceBuffer d_pij, d_row_ptr, d_col, d_val;
    {
        DeviceBuffer d_cond(sizeof(float) * nnz);
        TSNE_OR_DIE(tsnehip::launch_perplexity(d_dist.as<float>(), N, K, opt.perplexity,
                                               opt.perplexity_search_epsilon, d_cond.as<float>(), nullptr,
                                               stream),
                    "perplexity search");
        if (full_sym) {
            DeviceBuffer row_ptr(sizeof(int) * ((size_t)N + 1)), col(sizeof(int) * 2 * nnz), val(sizeof(float) * 2 * nnz);
            int64_t stored = 0;
            TSNE_OR_DIE(tsnehip::symmetrize_full(d_cond.as<float>(), d_idx.as<int>(), N, K, row_ptr.as<int>(),
                                                 col.as<int>(), val.as<float>(), &stored, stream),
                        "full symmetrisation");
            if (verbose) std::cout << "(" << stored << " non-zeros after full symmetrisation) " << std::flush;
            d_row_ptr.swap(row_ptr);
            d_col.swap(col);
            d_val.swap(val);
        } else {
            DeviceBuffer pij(sizeof(float) * nnz);
            TSNE_OR_DIE(tsnehip::launch_symmetrize(d_cond.as<float>(), d_idx.as<int>(), N, K, pij.as<float>(), stream),
                        "symmetrisation");
            d_pij.swap(pij);
        }
        hip_or_die(hipStreamSynchronize(stream), "P matrix");
    }
    d_dist.release();
    t_sym = clock.stop();

    // ---- initial embedding (src/fit_tsne.cu:181-235) ----------------------
    clock.start();
    if (verbose) std::cout << "done.\nInitializing low dim points... " << std::flush;
    std::vector<float> h_emb((size_t)2 * N);
    {
        // Options' constructors seed from the clock (src/include/options.h:108-109).  TSNE_RANDOM_SEED, this
        // library's extension, replaces that seed so that a run through the Python surface or the command-line
        // program, neither of which can set Options::random_seed, can be repeated.
        const char *seed_env = std::getenv("TSNE_RANDOM_SEED");
        std::default_random_engine generator(seed_env && *seed_env ? std::atoi(seed_env) : opt.random_seed);
        std::normal_distribution<float> normal(0.0, 1.0);
        // The reference first draws an unused noise vector; consuming the same
        // draws keeps the generator in step for the random initialisations (the
        // others never touch the generator again, so they skip the draws).
        if (opt.initialization == TSNE_INIT::UNIFORM || opt.initialization == TSNE_INIT::GAUSSIAN)
            for (size_t i = 0; i < h_emb.size(); ++i) h_emb[i] = 0.001 * normal(generator);
        if (opt.initialization == TSNE_INIT::UNIFORM) {
            std::uniform_real_distribution<float> uniform(-5, 5);
            for (size_t i = 0; i < h_emb.size(); ++i) h_emb[i] = uniform(generator);
        } else if (opt.initialization == TSNE_INIT::GAUSSIAN) {
            for (size_t i = 0; i < h_emb.size(); ++i) h_emb[i] = 0.0001 * normal(generator);
        } else if (opt.initialization == TSNE_INIT::RESUME || opt.initialization == TSNE_INIT::VECTOR) {
            if (opt.preinit_data == nullptr) {
                std::cerr << "E: Invalid initialization. Initialization points are null." << std::endl;
                std::exit(1);
            }
            std::memcpy(h_emb.data(), opt.preinit_data, sizeof(float) * h_emb.size());
        } else {
            std::cerr << "E: Invalid initialization type specified." << std::endl;
            std::exit(1);
        }
    }
    DeviceBuffer d_emb(sizeof(float) * 2 * (size_t)N), d_gains(sizeof(float) * 2 * (size_t)N),
        d_old(sizeof(float) * 2 * (size_t)N), d_norm(sizeof(float));
    to_internal(h_emb);
    hip_or_die(hipMemcpy(d_emb.ptr, h_emb.data(), sizeof(float) * h_emb.size(), hipMemcpyHostToDevice),
               "copy of the initial embedding");
    // Gains start at 1 (bit pattern of 1.0f), the momentum buffer at 0.
    hip_or_die(hipMemsetD32(reinterpret_cast<hipDeviceptr_t>(d_gains.ptr), 0x3f800000, 2 * (size_t)N),
               "gains initialisation");
    hip_or_die(hipMemset(d_old.ptr, 0, sizeof(float) * 2 * (size_t)N), "momentum initialisation");
    t_low = clock.stop();

    // ---- interpolation grid and scratch (src/fit_tsne.cu:246-342) --------
    clock.start();
    if (verbose) std::cout << "done.\nInitializing HIP memory... " << std::flush;
    const int n_boxes_per_dim = 130;  // 125 rounded up in the reference's allowed list
    tsne_hip_plan *plan = nullptr;
    TSNE_OR_DIE(tsne_hip_plan_create(&plan, N, K, n_boxes_per_dim, gpu_opt.device), "plan creation");
    // Re-centring is this library's option (Options::recenter_embedding or TSNE_RECENTER=1); off, as in the reference.
    plan->recenter = opt.recenter_embedding || env_int("TSNE_RECENTER", 0) != 0;
    // Re-block the sparse pattern for the LDS-staged attractive kernel; shapes it
    // cannot hold (very large K or N) keep the row-ordered kernel.
    // (The row-ordered pattern stays: the objective of the final embedding is evaluated on it.)
    bool blocked = false;
    if (full_sym) {
        plan->csr_row_ptr = d_row_ptr.as<int>();
        plan->csr_col_idx = d_col.as<int>();
        plan->csr_values = d_val.as<float>();
    } else {
        const int prepared = tsnehip::prepare_blocked(plan, d_pij.as<float>(), d_idx.as<int>(), stream);
        if (prepared != 0 && prepared != tsnehip::kShapeNotSupported) die("re-blocking of the sparse pattern");
        blocked = prepared == 0;
        if (!blocked && verbose)
            std::cout << "(" << tsnehip::last_error() << "; using the row-ordered attractive kernel) " << std::flush;
    }
    // No explicit N x K pattern goes to the steps when the plan holds the pattern itself (re-blocked or CSR).
    const bool plan_pattern = blocked || full_sym;

    std::ofstream dump_file;
    if (opt.get_dump_points()) {
        dump_file.open(opt.get_dump_file());
        dump_file << N << " " << 2 << std::endl;
    }
    if (opt.get_use_interactive())
        std::cout << "This version is not built with ZMQ for interative viz. Rebuild with WITH_ZMQ=TRUE for viz."
                  << std::endl;
    if (verbose) std::cout << "done." << std::endl;
    t_fft = clock.stop();

    // ---- gradient loop (src/fit_tsne.cu:402-580) -------------------------
    // Steps are enqueued back to back; the host only joins the stream at the
    // steps whose results it must look at (progress print, early stop, dump,
    // snapshot).
    const bool want_dump = opt.get_dump_points();
    const int dump_interval = opt.get_dump_interval() > 0 ? opt.get_dump_interval() : 1;
    const int print_interval = opt.print_interval > 0 ? opt.print_interval : 1;
    const bool want_snap = opt.return_style == RETURN_STYLE::SNAPSHOT && opt.return_data != nullptr;
    const bool want_stop = opt.min_gradient_norm > 0.0f;
    const int monitor_points = verbose ? env_int("TSNE_REPULSION_MONITOR", 0) : 0;
    // Options::adaptive_boxes or TSNE_ADAPTIVE_BOXES=1: every kGridCheckSteps steps the grid follows the spread
    // of the embedding (src/fit_tsne.cu:435, commented out in the reference, which keeps 130 boxes).
    const bool adaptive_boxes = opt.adaptive_boxes || env_int("TSNE_ADAPTIVE_BOXES", 0) != 0;
    constexpr size_t kGridCheckSteps = 50;
    hipEvent_t ev[4];
    if (verbose)
        for (auto &e : ev) hip_or_die(hipEventCreate(&e), "event creation");

    std::vector<float> h_out;
    float normalization = -1.0f;
    int slot = 0;
    clock.start();
    TSNE_OR_DIE(tsnehip::launch_bounds(plan, d_emb.as<float>(), slot, stream), "bounds");
    if (plan->recenter) TSNE_OR_DIE(tsnehip::launch_centre_sums(plan, d_emb.as<float>(), slot, stream), "centre");
    TSNE_OR_DIE(tsnehip::launch_pack_xy(plan, d_emb.as<float>(), stream), "pack");
    t_other += clock.stop();
    const size_t iterations = (size_t)opt.iterations;
    for (size_t step = 0; step != iterations; ++step) {
        const bool late = step >= (size_t)opt.force_magnify_iters && opt.force_magnify_iters >= 0;
        const float momentum = late ? opt.post_exaggeration_momentum : opt.pre_exaggeration_momentum;
        const float exaggeration = late ? 1.0f : opt.early_exaggeration;
        const bool printing = verbose && step % print_interval == 0;
        const bool timing = printing;  // phase timers sample the steps that already synchronise

        if (adaptive_boxes && step > 0 && step % kGridCheckSteps == 0) {
            unsigned int enc[4];  // min_enc[2], max_enc[2]: the bounds the next step will use are in `slot`
            hip_or_die(hipStreamSynchronize(stream), "grid size");
            hip_or_die(hipMemcpy(enc, plan->scalars, sizeof(enc), hipMemcpyDeviceToHost), "grid size");
            const float spread = tsnehip::ordered_to_float_host(enc[2 + slot]) - tsnehip::ordered_to_float_host(enc[slot]);
            const int boxes = tsne_hip_boxes_for_spread(spread);
            if (boxes != plan->n_boxes) {
                if (verbose)
                    std::cout << "[Step " << step << "] Interpolation grid: " << boxes << " boxes per dimension (spread "
                              << spread << ")" << std::endl;
                TSNE_OR_DIE(tsne_hip_plan_set_boxes(plan, boxes), "grid size");
            }
        }
        const bool want_norm = step + 1 == iterations || want_stop;
        if (!verbose && !want_stop && !want_dump && !want_snap) {
            // Nothing looks at the steps in between: everything up to the schedule switch, or up to the last
            // step (launched singly below: it delivers the normalisation), goes out as one batch on the plan's
            // own stream (tied to `stream` by an event at either end), where problems of up to about a million points
            // replay a captured graph of two steps: ~4 ms to set up per schedule, 10-15 us saved per step.
            size_t run_end = iterations - 1;
            if (!late && opt.force_magnify_iters >= 0)
                run_end = std::min(run_end, (size_t)opt.force_magnify_iters);
            if (adaptive_boxes) run_end = std::min(run_end, (step / kGridCheckSteps + 1) * kGridCheckSteps);
            if (run_end > step + 1) {
                const size_t count = std::min<size_t>(run_end - step, 1u << 30);
                hipStream_t batch_stream = plan->loop_stream;
                hip_or_die(hipEventRecord(plan->enter_event, stream), "event");
                hip_or_die(hipStreamWaitEvent(batch_stream, plan->enter_event, 0), "event");
                TSNE_OR_DIE(tsnehip::launch_steps(plan, plan_pattern ? nullptr : d_pij.as<float>(),
                                                  plan_pattern ? nullptr : d_idx.as<int>(), d_emb.as<float>(),
                                                  d_gains.as<float>(), d_old.as<float>(), opt.learning_rate,
                                                  momentum, exaggeration, (int)count, slot, batch_stream),
                            "gradient steps");
                hip_or_die(hipEventRecord(plan->leave_event, batch_stream), "event");
                hip_or_die(hipStreamWaitEvent(stream, plan->leave_event, 0), "event");
                step += count - 1;
                continue;
            }
        }
        if (!timing) {
            // Repulsive chain and attractive kernel side by side (plan's side stream), joined before the update.
            TSNE_OR_DIE(tsnehip::launch_step(plan, plan_pattern ? nullptr : d_pij.as<float>(),
                                             plan_pattern ? nullptr : d_idx.as<int>(), d_emb.as<float>(),
                                             d_gains.as<float>(), d_old.as<float>(), opt.learning_rate, momentum,
                                             exaggeration, slot, want_norm ? d_norm.as<float>() : nullptr, stream),
                        "gradient step");
        } else {
            // Sampled steps run the phases one after the other so that the phase timers mean something.
            hip_or_die(hipEventRecord(ev[0], stream), "event");
            TSNE_OR_DIE(tsnehip::launch_repulsive(plan, d_emb.as<float>(), slot, plan->rep, nullptr, nullptr, stream,
                                                  true),
                        "repulsive forces");
            hip_or_die(hipEventRecord(ev[1], stream), "event");
            TSNE_OR_DIE(full_sym ? tsnehip::launch_attractive_csr(plan, plan->csr_row_ptr, plan->csr_col_idx,
                                                                  plan->csr_values, plan->attr, stream)
                        : blocked ? tsnehip::launch_attractive_blocked(plan, plan->attr, stream)
                                  : tsnehip::launch_attractive(plan, d_pij.as<float>(), d_idx.as<int>(), plan->attr,
                                                               stream),
                        "attractive forces");
            hip_or_die(hipEventRecord(ev[2], stream), "event");
            if (want_norm) TSNE_OR_DIE(tsnehip::launch_finish_z(plan, d_norm.as<float>(), stream), "normalisation");
            TSNE_OR_DIE(tsnehip::launch_update(plan, d_emb.as<float>(), plan->attr, plan->rep, d_gains.as<float>(),
                                               d_old.as<float>(), opt.learning_rate, nullptr, momentum, exaggeration,
                                               slot ^ 1, stream),
                        "update");
        }
        slot ^= 1;
        if (timing) hip_or_die(hipEventRecord(ev[3], stream), "event");
        // Norm of the step just taken (the reference prints it as "Avg. Gradient Norm").
        float grad_norm = 0.0f;
        if (want_stop || printing) {
            TSNE_OR_DIE(tsnehip::launch_sum_squares(d_old.as<float>(), 2 * (int64_t)N, d_scratch.as<float>(), stream),
                        "gradient norm");
            float sumsq = 0.0f;
            hip_or_die(hipMemcpy(&sumsq, d_scratch.ptr, sizeof(float), hipMemcpyDeviceToHost), "gradient norm");
            grad_norm = std::sqrt(sumsq);
        }
        if (timing) {
            float ms = 0;
            hip_or_die(hipEventSynchronize(ev[3]), "event");
            // Sampled steps stand for the print_interval steps around them.
            const double weight = (double)std::min<size_t>(print_interval, iterations - step) * 1e-3;
            hip_or_die(hipEventElapsedTime(&ms, ev[0], ev[1]), "event");
            t_rep += ms * weight;
            hip_or_die(hipEventElapsedTime(&ms, ev[1], ev[2]), "event");
            t_attr += ms * weight;
            hip_or_die(hipEventElapsedTime(&ms, ev[2], ev[3]), "event");
            t_apply += ms * weight;
        }
        if (want_stop && grad_norm < opt.min_gradient_norm) {
            if (verbose) std::cout << "Reached minimum gradient norm: " << grad_norm << std::endl;
            break;
        }
        if (printing) std::cout << "[Step " << step << "] Avg. Gradient Norm: " << grad_norm << std::endl;
        // TSNE_REPULSION_MONITOR=<points>: on the printed steps, the error of the interpolated repulsive forces
        // of the embedding just produced against exact sums over all points, on that many sampled points.
        if (printing && monitor_points > 0) {
            double err[3] = {0.0, 0.0, 0.0};
            TSNE_OR_DIE(tsnehip::repulsive_error(plan, d_emb.as<float>(), slot, monitor_points, 12345u + (unsigned)step,
                                                 err, stream),
                        "repulsion monitor");
            std::cout << "[Step " << step << "] Repulsion interpolation error: forces " << err[0]
                      << ", normalization " << err[1] << " (" << (int)err[2] << " points)" << std::endl;
        }

        if (want_dump && step % dump_interval == 0) {
            hip_or_die(hipMemcpy(h_emb.data(), d_emb.ptr, sizeof(float) * h_emb.size(), hipMemcpyDeviceToHost),
                       "dump");
            h_out.resize(h_emb.size());
            to_caller(h_emb.data(), h_out.data());
            for (int i = 0; i < N; ++i) dump_file << h_out[i] << " " << h_out[i + N] << std::endl;
        }
        // At most num_snapshots - 1 in-loop snapshots, so that the final
        // embedding always fits as the last of num_snapshots blocks.
        if (want_snap && step % snap_interval == 0 && snap_num < opt.num_snapshots - 1) {
            hip_or_die(hipMemcpy(h_emb.data(), d_emb.ptr, sizeof(float) * 2 * N, hipMemcpyDeviceToHost), "snapshot");
            to_caller(h_emb.data(), opt.return_data + (size_t)snap_num * 2 * N);
            snap_num += 1;
        }
    }
    hip_or_die(hipStreamSynchronize(stream), "gradient loop");
    if (blocked) TSNE_OR_DIE(tsnehip::check_attractive_waits(plan), "gradient loop");
    if (opt.iterations > 0)
        hip_or_die(hipMemcpy(&normalization, d_norm.ptr, sizeof(float), hipMemcpyDeviceToHost), "normalisation");

    if (verbose) {
        for (auto &e : ev) (void)hipEventDestroy(e);
        // Same names and format as the reference's PRINT_IL_TIMER lines
        // (src/fit_tsne.cu:586-601).  Charges and kernel precomputation run
        // inside the n-body kernels here, so their own lines read 0.  The three
        // force phases are what they cost one after the other (sampled on the
        // printed steps); in the other steps the n-body chain runs beside the
        // attractive kernel, so total_time is the wall clock, not their sum.
        const double total = wall.stop();
        std::cout << "_time_initialization: " << (float)t_init << "s" << std::endl;
        std::cout << "_time_knn: " << (float)t_knn << "s" << std::endl;
        std::cout << "_time_symmetry: " << (float)t_sym << "s" << std::endl;
        std::cout << "_time_init_low_dim: " << (float)t_low << "s" << std::endl;
        std::cout << "_time_init_fft: " << (float)t_fft << "s" << std::endl;
        std::cout << "_time_compute_charges: " << 0.0f << "s" << std::endl;
        std::cout << "_time_precompute_2d: " << 0.0f << "s" << std::endl;
        std::cout << "_time_nbodyfft: " << (float)t_rep << "s" << std::endl;
        std::cout << "_time_norm: " << 0.0f << "s" << std::endl;
        std::cout << "_time_attr: " << (float)t_attr << "s" << std::endl;
        std::cout << "_time_apply_forces: " << (float)t_apply << "s" << std::endl;
        std::cout << "_time_other: " << (float)t_other << "s" << std::endl;
        std::cout << "total_time: " << (float)total << "s" << std::endl;
    }
    if (want_dump) dump_file.close();

    // Final embedding after the snapshots taken so far, or alone (src/fit_tsne.cu:611-620).
    if (opt.return_data != nullptr) {
        float *dst = opt.return_data;
        if (opt.return_style == RETURN_STYLE::SNAPSHOT) dst += (size_t)snap_num * 2 * N;
        hip_or_die(hipMemcpy(h_emb.data(), d_emb.ptr, sizeof(float) * 2 * N, hipMemcpyDeviceToHost), "result copy");
        to_caller(h_emb.data(), dst);
    }
    // Objective of the final embedding: Z of the final positions from one more
    // repulsive evaluation (the loop's last Z belongs to the positions before
    // the last update), the pattern sum from the row-ordered P.
    {
        DeviceBuffer d_kl(2 * sizeof(double));
        float z_final = 0.0f;
        double terms[2] = {0.0, 0.0};
        TSNE_OR_DIE(tsnehip::launch_repulsive(plan, d_emb.as<float>(), slot, plan->rep, nullptr, nullptr, stream),
                    "final normalisation");
        TSNE_OR_DIE(tsnehip::launch_finish_z(plan, d_norm.as<float>(), stream), "final normalisation");
        TSNE_OR_DIE(full_sym ? tsnehip::launch_kl_terms_csr(d_row_ptr.as<int>(), d_col.as<int>(), d_val.as<float>(),
                                                            d_emb.as<float>(), N, d_kl.as<double>(), stream)
                             : tsnehip::launch_kl_terms(d_pij.as<float>(), d_idx.as<int>(), d_emb.as<float>(), N, K,
                                                        d_kl.as<double>(), stream),
                    "objective");
        hip_or_die(hipMemcpy(&z_final, d_norm.ptr, sizeof(float), hipMemcpyDeviceToHost), "objective");
        hip_or_die(hipMemcpy(terms, d_kl.ptr, sizeof(terms), hipMemcpyDeviceToHost), "objective");
        opt.trained_kl_divergence = z_final > 0.0f ? terms[0] + terms[1] * std::log((double)z_final) : -1.0;
        g_last_kl = opt.trained_kl_divergence;
    }
    tsne_hip_plan_destroy(plan);
    opt.trained = true;
    opt.trained_norm = normalization;
}

}  // namespace tsnecuda

extern "C" double tsne_hip_last_kl_divergence(void) { return g_last_kl; }

extern "C" void pymodule_tsne(float *result, float *points, ssize_t *dims, float perplexity, float learning_rate,
                              float early_exaggeration, float magnitude_factor, int num_neighbors, int iterations,
                              int iterations_no_progress, int force_magnify_iters,
                              float perplexity_search_epsilon, float pre_exaggeration_momentum,
                              float post_exaggeration_momentum, float theta, float epssq, float min_gradient_norm,
                              int initialization_type, float *preinit_data, bool dump_points, char *dump_file,
                              int dump_interval, bool use_interactive, char *viz_server, int viz_timeout,
                              int verbosity, int print_interval, int gpu_device, int return_style,
                              int num_snapshots, int distance_metric) {
    tsnecuda::GpuOptions gpu_opt(gpu_device);
    tsnecuda::Options opt(result, points, (int)dims[0], (int)dims[1]);
    opt.perplexity = perplexity;
    opt.learning_rate = learning_rate;
    opt.early_exaggeration = early_exaggeration;
    opt.magnitude_factor = magnitude_factor;
    opt.num_neighbors = num_neighbors;
    opt.iterations = iterations;
    opt.iterations_no_progress = iterations_no_progress;
    opt.force_magnify_iters = force_magnify_iters;
    opt.perplexity_search_epsilon = perplexity_search_epsilon;
    opt.pre_exaggeration_momentum = pre_exaggeration_momentum;
    opt.post_exaggeration_momentum = post_exaggeration_momentum;
    opt.theta = theta;
    opt.epssq = epssq;
    opt.min_gradient_norm = min_gradient_norm;
    opt.verbosity = verbosity;
    opt.print_interval = print_interval;
    opt.distance_metric = tsnecuda::MetricType(distance_metric);

    // Encodings of src/ext/pymodule_ext.cu:70-116.
    if (initialization_type == 0) {
        opt.initialization = tsnecuda::TSNE_INIT::UNIFORM;
    } else if (initialization_type == 1) {
        opt.initialization = tsnecuda::TSNE_INIT::GAUSSIAN;
    } else if (initialization_type == 2) {
        std::cerr << "E: RESUME initialization not yet supported fully..." << std::endl;
        std::exit(1);
    } else if (initialization_type == 3) {
        opt.initialization = tsnecuda::TSNE_INIT::VECTOR;
        opt.preinit_data = preinit_data;
    } else {
        std::cerr << "E: Invalid initialization supplied" << std::endl;
        std::exit(1);
    }
    if (dump_points) opt.enable_dump(std::string(dump_file), dump_interval);
    if (use_interactive) opt.enable_viz(std::string(viz_server), viz_timeout);
    if (return_style == 0) {
        opt.return_style = tsnecuda::RETURN_STYLE::ONCE;
    } else if (return_style == 1) {
        opt.return_style = tsnecuda::RETURN_STYLE::SNAPSHOT;
        opt.num_snapshots = num_snapshots;
    } else {
        std::cerr << "E: Invalid return style supplied" << std::endl;
        std::exit(1);
    }
    tsnecuda::RunTsne(opt, gpu_opt);
    (void)hipDeviceSynchronize();
}
