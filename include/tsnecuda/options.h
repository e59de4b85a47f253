/*
 * tsnecuda::Options and tsnecuda::GpuOptions for the MI355X (gfx950) build.
 *
 * Source-compatible with the reference's src/include/options.h:20-376: same
 * type names, public field names, defaults, constructors, setters and getters,
 * so code written against the reference compiles against this header.  Two
 * deliberate differences:
 *   * Options::distance_metric is a tsnecuda::MetricType (values 0 = inner
 *     product, 1 = L2, as faiss::MetricType) instead of the FAISS type, because
 *     FAISS is not part of this build.  As in the reference the field is
 *     recorded and never read: neighbours are always by squared L2 distance.
 *   * GpuOptions is filled from the HIP device properties (wavefront 64,
 *     compute-unit count); its constructor lives in the library, so this header
 *     needs no GPU toolkit.
 */
#ifndef TSNECUDA_OPTIONS_H_
#define TSNECUDA_OPTIONS_H_

#include <ctime>
#include <iostream>
#include <string>

namespace tsnecuda {

enum TSNE_INIT { UNIFORM, GAUSSIAN, RESUME, VECTOR };

enum RETURN_STYLE { ONCE, SNAPSHOT };

enum DISTANCE_METRIC { INNER_PRODUCT, L2, L1, LINF, CANBERRA, BRAYCURTIS, JENSENSHANNON };

enum MetricType { METRIC_INNER_PRODUCT = 0, METRIC_L2 = 1 };

class Options {
   private:
    // Text dump of the embedding every dump_interval steps.
    bool dump_points = false;
    int dump_interval = 100;
    std::string dump_file = "";

    // Live visualisation endpoint (recorded; this build has no ZMQ, like the
    // reference's default NO_ZMQ build).
    bool use_interactive = false;
    std::string viz_server = "tcp://localhost:5556";
    int viz_timeout = 10000;

   public:
    // Input points: num_points x num_dims, row-major, host memory, borrowed.
    float *points = nullptr;
    int num_points = 0;
    int num_dims = 0;

    // Algorithm parameters.
    float perplexity = 50.0f;
    float learning_rate = 200.0f;
    float early_exaggeration = 12.0f;
    float magnitude_factor = 5.0f;
    int num_neighbors = 1023;
    int iterations = 1000;
    int iterations_no_progress = 1000;
    int force_magnify_iters = 250;
    float perplexity_search_epsilon = 1e-4;

    float pre_exaggeration_momentum = 0.5;
    float post_exaggeration_momentum = 0.8;
    float theta = 0.5f;
    float epssq = 0.05 * 0.05;

    float min_gradient_norm = 0.0;

    MetricType distance_metric = METRIC_INNER_PRODUCT;

    // Initial embedding.
    TSNE_INIT initialization = TSNE_INIT::GAUSSIAN;
    float *preinit_data = nullptr;

    int verbosity = 20;
    int print_interval = 10;

    // Output: 2 * num_points floats (xs then ys) per returned embedding.
    RETURN_STYLE return_style = RETURN_STYLE::ONCE;
    float *return_data = nullptr;
    int num_snapshots = 0;

    // Written by RunTsne.
    float trained_norm = -1.0;
    // Objective of the returned embedding on the stored pattern, sum P (ln P + ln(1 + d^2) + ln Z), set by
    // RunTsne (the reference documents no such output and never evaluates its FunctionalKlDivergence,
    // src/include/util/thrust_transform_functions.h:26-31).
    double trained_kl_divergence = -1.0;
    bool trained = false;

    int random_seed = 0;

    // Not in the reference: subtract the embedding's centre in every update (its loop never re-centres,
    // src/kernels/apply_forces.cu:11-57).  Off by default; TSNE_RECENTER=1 in the environment also enables it.
    bool recenter_embedding = false;

    // Not in the reference's live code: symmetrise P as (A + A^T) / 2N with the union pattern (its commented-out
    // cuSPARSE routine, src/util/math_utils.cu:76-225) instead of the pattern-restricted form it runs
    // (src/util/math_utils.cu:269-308).  Off by default; TSNE_SYMMETRIZE=full in the environment also enables it.
    bool full_symmetrization = false;

    // Approximate neighbours through an inverted file, the structure of the reference's FAISS search
    // (src/util/distance_utils.cu:85-120: floor(sqrt(N)) lists, 20 probed); the default here is the exact search.
    // knn_nprobe: lists probed by each list (0: 100, which on 50-dimensional Gaussian clusters finds about as many
    // of the true neighbours as FAISS's 20 lists per query).  TSNE_KNN=ivf and TSNE_KNN_NPROBE=<n> in the
    // environment do the same.  Inputs of more than 126 dimensions keep the exact search.
    bool approximate_neighbors = false;
    int knn_nprobe = 0;

    // FIt-SNE's rule for the size of the interpolation grid, which the reference carries as a comment
    // (src/fit_tsne.cu:435) while it runs a fixed 130 boxes per dimension: every 50 steps the grid is set to
    // max(125, spread of the embedding) boxes, rounded up in the reference's list of sizes (at most 170 here).
    // Off by default; TSNE_ADAPTIVE_BOXES=1 in the environment also enables it.
    bool adaptive_boxes = false;

    Options() {}

    Options(float *return_data, float *points, int num_points, int num_dims)
        : points(points), num_points(num_points), num_dims(num_dims), return_data(return_data) {
        this->random_seed = time(NULL);
    }

    Options(float *points, int num_points, int num_dims, float perplexity, float learning_rate,
            float magnitude_factor, int num_neighbors, int iterations, int iterations_no_progress,
            int force_magnify_iters, float perplexity_search_epsilon, float pre_exaggeration_momentum,
            float post_exaggeration_momentum, float theta, float epssq, float min_gradient_norm,
            TSNE_INIT initialization, float *preinit_data, bool dump_points, int dump_interval,
            RETURN_STYLE return_style, float *return_data, int num_snapshots, bool use_interactive,
            std::string viz_server, int verbosity, int print_interval, MetricType distance_metric)
        : dump_points(dump_points),
          dump_interval(dump_interval),
          use_interactive(use_interactive),
          viz_server(viz_server),
          points(points),
          num_points(num_points),
          num_dims(num_dims),
          perplexity(perplexity),
          learning_rate(learning_rate),
          magnitude_factor(magnitude_factor),
          num_neighbors(num_neighbors),
          iterations(iterations),
          iterations_no_progress(iterations_no_progress),
          force_magnify_iters(force_magnify_iters),
          perplexity_search_epsilon(perplexity_search_epsilon),
          pre_exaggeration_momentum(pre_exaggeration_momentum),
          post_exaggeration_momentum(post_exaggeration_momentum),
          theta(theta),
          epssq(epssq),
          min_gradient_norm(min_gradient_norm),
          distance_metric(distance_metric),
          initialization(initialization),
          preinit_data(preinit_data),
          verbosity(verbosity),
          print_interval(print_interval),
          return_style(return_style),
          return_data(return_data),
          num_snapshots(num_snapshots) {
        this->random_seed = time(NULL);
    }

    bool enable_dump(std::string filename, int interval = 1) {
        dump_points = true;
        dump_file = filename;
        dump_interval = interval;
        return true;
    }

    bool enable_viz(std::string server_address = "tcp://localhost:5556", int timeout = 10000) {
        use_interactive = true;
        viz_server = server_address;
        viz_timeout = timeout;
        return true;
    }

    // Same acceptance rule and message as the reference (src/include/options.h:163-180).
    bool validate() {
        const bool has_input = points != nullptr && num_points != 0 && num_dims != 0;
        if (!has_input) return false;
        if (return_style == RETURN_STYLE::SNAPSHOT && num_snapshots < 2) {
            std::cout << "E: Need to record more than 1 snapshot when using snapshot capture. Use 'once' capture "
                         "if you only want one return."
                      << std::endl;
            return false;
        }
        return true;
    }

    bool get_dump_points() { return dump_points; }
    std::string get_dump_file() { return dump_file; }
    int get_dump_interval() { return dump_interval; }
    bool get_use_interactive() { return use_interactive; }
    int get_viz_timeout() { return viz_timeout; }
    std::string get_viz_server() { return viz_server; }
};

class GpuOptions {
   public:
    int device = 0;

    // Launch parameters.  integration_*, fft_*, attr_* and rep_* can be
    // overridden through TSNE_INTEG_THREADS, TSNE_INTEG_FACTOR,
    // TSNE_FFT_THREADS, TSNE_ATTR_THREADS and TSNE_REP_THREADS and are clamped
    // to the device limit, as in the reference.  The gfx950 kernels are
    // written for fixed workgroup shapes, so these are recorded for callers
    // that read them back; the remaining fields are the reference's vestigial
    // Barnes-Hut parameters, kept so that code touching them still compiles.
    int integration_kernel_threads = 256;
    int integration_kernel_factor = 1;
    int fft_kernel_threads = 256;
    int attr_kernel_threads = 256;
    int rep_kernel_threads = 256;
    int repulsive_kernel_threads = 256;
    int repulsive_kernel_factor = 5;
    int bounding_kernel_threads = 512;
    int bounding_kernel_factor = 3;
    int tree_kernel_threads = 1024;
    int tree_kernel_factor = 2;
    int sort_kernel_threads = 64;
    int sort_kernel_factor = 6;
    int summary_kernel_threads = 128;
    int summary_kernel_factor = 6;
    int warp_size = 64;
    int sm_count = 256;

    // Queries the device, makes it current (hipSetDevice) and applies the
    // environment overrides.
    explicit GpuOptions(int device);
};

}  // namespace tsnecuda

#endif  // TSNECUDA_OPTIONS_H_
