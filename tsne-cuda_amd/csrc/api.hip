// Stage-level C ABI: argument checks, plan lifetime, and the fused gradient loop.
#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/tsnecuda/tsne_stages.h"
#include "plan.h"
#include "stages.h"

namespace tsnehip {

namespace {
thread_local char g_error[512] = "";
}

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
const char *last_error() { return g_error; }

bool sync_kernels_enabled() {
    static const bool enabled = []() {
        const char *v = std::getenv("TSNE_SYNC_KERNELS");
        return v != nullptr && std::atoi(v) != 0;
    }();
    return enabled;
}

int profile_mark(tsne_hip_plan *p, int id, hipStream_t) {
    if (p->profiling || (p->profiling_attractive && id == kKernelAttractive)) p->pending_kernel = id;
    return 0;
}

int profile_events(tsne_hip_plan *p, hipEvent_t *start, hipEvent_t *stop) {
    *start = *stop = nullptr;
    if (!(p->profiling || p->profiling_attractive) || p->pending_kernel < 0) return 0;
    while (p->events.size() < p->events_used + 2) {
        hipEvent_t e;
        TSNE_TRY(hipEventCreate(&e));
        p->events.push_back(e);
    }
    *start = p->events[p->events_used];
    *stop = p->events[p->events_used + 1];
    p->event_kernel.resize(p->events_used / 2 + 1);
    p->event_kernel[p->events_used / 2] = p->pending_kernel;
    p->events_used += 2;
    p->pending_kernel = -1;
    return 0;
}

namespace {

const char *const kLoopKernelNames[kKernelCount] = {
    "tile_count_kernel",        "tile_scatter_kernel",  "spread_kernel",     "conv_rows_forward_kernel", "conv_columns_kernel",
    "conv_rows_inverse_kernel", "gather_forces_kernel", "attractive_kernel", "update_kernel"};

LagrangeConsts make_lagrange() {
    // fp32 arithmetic in the order of src/fit_tsne.cu:303-321.
    LagrangeConsts lc;
    const float h = 1 / (float)kInterp;
    lc.spacing[0] = h / 2;
    for (int i = 1; i < kInterp; ++i) lc.spacing[i] = lc.spacing[i - 1] + h;
    for (int i = 0; i < kInterp; ++i) {
        lc.denom[i] = 1;
        for (int j = 0; j < kInterp; ++j)
            if (i != j) lc.denom[i] *= lc.spacing[i] - lc.spacing[j];
    }
    return lc;
}

int check_plan(const tsne_hip_plan *p, const char *who) {
    if (!p) {
        set_error("%s: plan is null", who);
        return 1;
    }
    int dev = -1;
    TSNE_TRY(hipGetDevice(&dev));
    if (dev != p->device) {
        set_error("%s: plan belongs to device %d but device %d is current", who, p->device, dev);
        return 1;
    }
    return 0;
}

#define TSNE_REQUIRE(cond, ...)      \
    do {                             \
        if (!(cond)) {               \
            set_error(__VA_ARGS__);  \
            return 1;                \
        }                            \
    } while (0)

}  // namespace
}  // namespace tsnehip

namespace tsnehip {

// Up to this many points a step is a chain of short dependent kernels that the attractive kernel hardly
// lengthens: one stream without events and without a captured graph is then the fastest form (fits of 5000, 60000
// and 50000 points 5 %, 3.5 % and 2.7 % shorter than with two streams and graphs, whose events cost 7-10 us per
// step and whose instantiation 4 ms per stretch of constant parameters; at 100000 points two streams are 4 % ahead).
constexpr int kSingleStreamPoints = 65536;

// TSNE_OVERLAP: 0 never, 1 always, unset: by the size of the problem.
static bool overlap_enabled(const tsne_hip_plan *p) {
    const char *v = std::getenv("TSNE_OVERLAP");  // read on every call, like TSNE_GRAPH
    // (the direct form of the attractive kernel gathers its positions from memory, as the chain's spreading and
    // gathering kernels do theirs, and from about seven million points on each of them slows the others down by
    // more than the overlap hides: ms per step on two streams / on one - 4 M points 1.01 / 1.03, 6 M 1.58 / 1.61,
    // 8 M 2.54 / 2.44, 10 M 3.70 / 3.37)
    constexpr int kDirectOverlapPoints = 7000000;
    return v ? v[0] != '0'
             : (p->num_points > kSingleStreamPoints && !(p->blocked_direct && p->num_points > kDirectOverlapPoints));
}

// Overlapped form: a step's repulsive chain and its attractive kernel run on two streams, the update behind the
// chain on the chain's stream.  A dependency between two kernels of one stream costs 2-3 us, one across streams
// about 9 us when the waiting stream gets there before the event has fired (measured between the chain's last
// kernel and an update on the other stream) and next to nothing when it fired long before.  So the transitions
// a step waits for are kept inside a stream:
//  * problems whose step is its chain (up to a quarter of a million points): chain(k), update(k), chain(k+1) ...
//    on the caller's stream, the attractive kernel on the side stream (it starts 9 us late and has the time);
//  * larger ones, whose step is the attractive kernel and what of the chain cannot run beside it: the attractive
//    kernel of step k+1 follows update(k) on the same stream, so chain and attractive kernel change streams every
//    step (pairs of steps, see launch_steps); a single step keeps the chain on the side stream and the attractive
//    kernel and the update on the caller's.
// Every form leaves the caller's stream joined with the side stream.  (Measured without captured graphs, where the
// streams are what the hardware queues see: fits of 5000-60000 points 15 % shorter than with the update on the
// attractive kernel's stream, a million points 2.8 % more iterations per second.  A captured graph holds the same
// dependencies whichever stream they were recorded on and runs as before.)
// Attractive forces of a step: the explicit N x K pattern if given, else the plan's CSR pattern if one is set,
// else the re-blocked pattern.
static int launch_step_attractive(tsne_hip_plan *p, const float *pij, const int *indices, hipStream_t s) {
    if (pij) return launch_attractive(p, pij, indices, p->attr, s);
    if (p->csr_row_ptr) return launch_attractive_csr(p, p->csr_row_ptr, p->csr_col_idx, p->csr_values, p->attr, s);
    return launch_attractive_blocked(p, p->attr, s);
}

static bool overlap_active(const tsne_hip_plan *p) {
    return overlap_enabled(p) && !p->profiling && p->side_stream != nullptr;
}

// Where the attractive kernel's workgroups (one per compute unit) hold strips of a thousand rows and more (a
// quarter of a million points and up: as much as 125 KB of LDS each), a step is that kernel plus what of the
// chain cannot run beside it, and the kernel is enqueued before the chain (in a captured graph: its node comes
// first), so that its workgroups are placed while the units are empty.  Enqueued after the chain's nine kernels
// it started 10 us later, and on every unit above the LDS block of a workgroup of the chain's first kernels:
// the 34 KB left on a unit were then in two pieces, neither large enough for a workgroup of the row passes
// (32 KB), which waited for the attractive kernel to end.  Smaller problems wait for the chain, not for the
// attractive kernel, and lose by the chain's later start (measured: 3-10 % slower from 5000 to 60000 points,
// even at 200000, 1 % faster at 400000, 4 % at 800000).
static bool attractive_is_critical(const tsne_hip_plan *p, const float *pij) {
    if (const char *v = std::getenv("TSNE_ATTRACTIVE_CRITICAL")) return v[0] != '0';
    return !pij && !p->csr_row_ptr && p->blocked_ready && p->strip_rows >= 1024;
}

// One overlapped step: chain and update on `cs`, attractive kernel on `as`; `prev` (one of the two) is the stream
// whose work so far includes the update before.
static int launch_step_on(tsne_hip_plan *p, const float *pij, const int *indices, float *embedding, float *gains,
                          float *old_forces, float eta, float momentum, float exaggeration, int slot,
                          float *normalization, hipStream_t cs, hipStream_t as, hipStream_t prev,
                          bool attractive_first) {
    TSNE_TRY(hipEventRecord(p->fork_event, prev));
    TSNE_TRY(hipStreamWaitEvent(prev == cs ? as : cs, p->fork_event, 0));
    if (attractive_first && launch_step_attractive(p, pij, indices, as)) return 1;
    if (launch_repulsive(p, embedding, slot, p->rep, nullptr, nullptr, cs, true)) return 1;
    if (normalization && launch_finish_z(p, normalization, cs)) return 1;
    if (!attractive_first && launch_step_attractive(p, pij, indices, as)) return 1;
    TSNE_TRY(hipEventRecord(p->join_event, as));
    TSNE_TRY(hipStreamWaitEvent(cs, p->join_event, 0));
    return launch_update(p, embedding, p->attr, p->rep, gains, old_forces, eta, nullptr, momentum, exaggeration,
                         slot ^ 1, cs);
}

int launch_step(tsne_hip_plan *p, const float *pij, const int *indices, float *embedding, float *gains,
                float *old_forces, float eta, float momentum, float exaggeration, int slot, float *normalization,
                hipStream_t s) {
    if (!overlap_active(p)) {
        if (launch_repulsive(p, embedding, slot, p->rep, nullptr, nullptr, s, true)) return 1;
        if (launch_step_attractive(p, pij, indices, s)) return 1;
        if (normalization && launch_finish_z(p, normalization, s)) return 1;
        return launch_update(p, embedding, p->attr, p->rep, gains, old_forces, eta, nullptr, momentum, exaggeration,
                             slot ^ 1, s);
    }
    hipStream_t side = p->side_stream;
    if (!attractive_is_critical(p, pij))
        return launch_step_on(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot,
                              normalization, s, side, s, false);
    TSNE_TRY(hipEventRecord(p->fork_event, s));  // everything up to the previous step's update
    TSNE_TRY(hipStreamWaitEvent(side, p->fork_event, 0));
    if (launch_step_attractive(p, pij, indices, s)) return 1;
    if (launch_repulsive(p, embedding, slot, p->rep, nullptr, nullptr, side, true)) return 1;
    if (normalization && launch_finish_z(p, normalization, side)) return 1;
    TSNE_TRY(hipEventRecord(p->join_event, side));
    TSNE_TRY(hipStreamWaitEvent(s, p->join_event, 0));
    return launch_update(p, embedding, p->attr, p->rep, gains, old_forces, eta, nullptr, momentum, exaggeration,
                         slot ^ 1, s);
}

// Two steps; where the attractive kernel is what a step waits for, with the streams' parts exchanged between them
// (the first step's update runs on the side stream and the second step's attractive kernel follows it there; the
// second step's update runs on the caller's stream again).
static int launch_two_steps(tsne_hip_plan *p, const float *pij, const int *indices, float *embedding, float *gains,
                            float *old_forces, float eta, float momentum, float exaggeration, int slot,
                            hipStream_t s) {
    // (with more strips than compute units the attractive kernel runs in rounds and the exchange measured 2 % slower)
    if (overlap_active(p) && attractive_is_critical(p, pij) && p->n_strips <= p->num_cus) {
        hipStream_t side = p->side_stream;
        return launch_step_on(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot, nullptr,
                              side, s, s, true) ||
               launch_step_on(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot ^ 1,
                              nullptr, s, side, side, true);
    }
    return launch_step(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot, nullptr, s) ||
           launch_step(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot ^ 1, nullptr, s);
}

// Replaying a captured graph saves launch gaps wherever the chain of nine short kernels is what a step waits for.
static bool graphs_enabled(const tsne_hip_plan *p) {
    const char *v = std::getenv("TSNE_GRAPH");  // read on every call: cheap, and lets one process try both
    const int mode = v ? (v[0] == '0' ? 0 : 1) : -1;
    if (p->profiling || p->profiling_attractive || sync_kernels_enabled() || mode == 0) return false;
    // Measured gain per step beside two streams without a graph: 2 % at 100000 points, 0-0.5 % from 200000 to a
    // million (and none against one stream up to kSingleStreamPoints); setting a graph up costs about 4 ms
    // whatever the size.
    return mode == 1 || (p->num_points > kSingleStreamPoints && p->num_points <= 1048576);
}

int launch_steps(tsne_hip_plan *p, const float *pij, const int *indices, float *embedding, float *gains,
                 float *old_forces, float eta, float momentum, float exaggeration, int count, int &slot,
                 hipStream_t s) {
    if (count >= 2 && s != nullptr && graphs_enabled(p)) {
        hipGraphExec_t exec = nullptr;
        for (const auto &g : p->step_graphs)
            if (g.pij == pij && g.indices == indices && g.embedding == embedding && g.gains == gains &&
                g.old_forces == old_forces && g.eta == eta && g.momentum == momentum &&
                g.exaggeration == exaggeration && g.slot == slot)
                exec = g.exec;
        if (!exec) {
            // Capture two steps (the bounds slot is back where it started) including the side stream's part.
            hipGraph_t graph = nullptr;
            TSNE_TRY(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
            const int rc =
                launch_two_steps(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot, s);
            const hipError_t end = hipStreamEndCapture(s, &graph);
            if (rc) {
                if (graph) (void)hipGraphDestroy(graph);
                return 1;
            }
            TSNE_TRY(end);
            const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            TSNE_TRY(inst);
            p->step_graphs.push_back({pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot,
                                      exec});
        }
        for (; count >= 2; count -= 2) TSNE_TRY(hipGraphLaunch(exec, s));
    }
    for (; count >= 2; count -= 2)  // (the bounds slot is back where it started after two steps)
        if (launch_two_steps(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot, s))
            return 1;
    if (count > 0) {
        if (launch_step(p, pij, indices, embedding, gains, old_forces, eta, momentum, exaggeration, slot, nullptr, s))
            return 1;
        slot ^= 1;
    }
    return 0;
}

}  // namespace tsnehip

using namespace tsnehip;

extern "C" {

const char *tsne_hip_last_error(void) { return last_error(); }

int tsne_hip_knn(const float *points, int num_points, int num_dims, int num_neighbors, int *indices,
                 float *sq_dist, void *stream) {
    TSNE_REQUIRE(points && indices && sq_dist, "knn: null pointer argument");
    return run_knn(points, num_points, num_dims, num_neighbors, indices, sq_dist, (hipStream_t)stream);
}

int tsne_hip_knn_select(const float *points, int num_points, int num_dims, int num_neighbors, int *indices,
                        float *sq_dist, void *stream, int sweep, int *stats) {
    TSNE_REQUIRE(points && indices && sq_dist, "knn: null pointer argument");
    TSNE_REQUIRE(sweep >= 0 && sweep <= 3, "knn: sweep must be 0 (choose), 1 (vector), 2 (matrix) or 3 (matrix on floats), got %d",
                 sweep);
    return run_knn_mode(points, num_points, num_dims, num_neighbors, indices, sq_dist, (hipStream_t)stream, sweep,
                        stats);
}

int tsne_hip_locality_order(const float *points, int num_points, int num_dims, int *order, void *stream) {
    TSNE_REQUIRE(points && order, "locality_order: null pointer argument");
    TSNE_REQUIRE(num_points > 0 && num_dims > 0, "locality_order: num_points and num_dims must be positive");
    hipStream_t s = (hipStream_t)stream;
    std::vector<int> host;
    if (locality_order(points, num_points, num_dims, host, s)) return 1;
    TSNE_TRY(hipMemcpyAsync(order, host.data(), sizeof(int) * (size_t)num_points, hipMemcpyHostToDevice, s));
    TSNE_TRY(hipStreamSynchronize(s));  // `host` goes out of scope
    return 0;
}

int tsne_hip_gather_rows(const float *rows_in, const int *order, int num_rows, int num_cols, float *rows_out,
                         void *stream) {
    TSNE_REQUIRE(rows_in && order && rows_out, "gather_rows: null pointer argument");
    TSNE_REQUIRE(num_rows > 0 && num_cols > 0, "gather_rows: num_rows and num_cols must be positive");
    return launch_gather_rows(rows_in, order, num_rows, num_cols, rows_out, (hipStream_t)stream);
}

int tsne_hip_max_normalize(float *values, int64_t n, void *stream) {
    TSNE_REQUIRE(values && n > 0, "max_normalize: need a non-empty array");
    hipStream_t s = (hipStream_t)stream;
    float *scratch = nullptr;
    TSNE_TRY(hipMalloc(&scratch, sizeof(float)));
    int rc = launch_max_normalize(values, n, scratch, s);
    if (!rc && hipStreamSynchronize(s) != hipSuccess) {
        set_error("max_normalize: stream synchronisation failed");
        rc = 1;
    }
    (void)hipFree(scratch);
    return rc;
}

int tsne_hip_perplexity(const float *sq_dist, int num_points, int num_neighbors, float perplexity,
                        float epsilon, float *pij, float *betas, void *stream) {
    TSNE_REQUIRE(sq_dist && pij, "perplexity: null pointer argument");
    TSNE_REQUIRE(num_points > 0 && num_neighbors > 0, "perplexity: empty problem (%d x %d)", num_points,
                 num_neighbors);
    TSNE_REQUIRE(perplexity > 0.0f, "perplexity: target must be positive (got %g)", (double)perplexity);
    return launch_perplexity(sq_dist, num_points, num_neighbors, perplexity, epsilon, pij, betas,
                             (hipStream_t)stream);
}

int tsne_hip_symmetrize(const float *pij_non_symmetric, const int *indices, int num_points,
                        int num_neighbors, float *pij, void *stream) {
    TSNE_REQUIRE(pij_non_symmetric && indices && pij, "symmetrize: null pointer argument");
    TSNE_REQUIRE(pij_non_symmetric != pij, "symmetrize: input and output must not alias");
    TSNE_REQUIRE(num_points > 0 && num_neighbors > 0, "symmetrize: empty problem (%d x %d)", num_points,
                 num_neighbors);
    return launch_symmetrize(pij_non_symmetric, indices, num_points, num_neighbors, pij, (hipStream_t)stream);
}

void tsne_hip_plan_destroy(tsne_hip_plan *p) {
    if (!p) return;
    // tsne_hip_iterate returns while its steps (or a replaying graph) are still running: nothing of the plan
    // may go before its streams and its device are idle.
    int current = -1;
    const bool switched = hipGetDevice(&current) == hipSuccess && current != p->device &&
                          hipSetDevice(p->device) == hipSuccess;
    if (p->loop_stream) (void)hipStreamSynchronize(p->loop_stream);
    if (p->side_stream) (void)hipStreamSynchronize(p->side_stream);
    (void)hipDeviceSynchronize();
    for (hipEvent_t e : p->events) (void)hipEventDestroy(e);
    if (p->fork_event) (void)hipEventDestroy(p->fork_event);
    if (p->join_event) (void)hipEventDestroy(p->join_event);
    for (auto &g : p->step_graphs) (void)hipGraphExecDestroy(g.exec);
    p->step_graphs.clear();
    if (p->enter_event) (void)hipEventDestroy(p->enter_event);
    if (p->leave_event) (void)hipEventDestroy(p->leave_event);
    if (p->loop_stream) (void)hipStreamDestroy(p->loop_stream);
    if (p->side_stream) (void)hipStreamDestroy(p->side_stream);
    release_blocked(p);
    (void)hipFree(p->yxy);
    (void)hipFree(p->tile_xy);
    (void)hipFree(p->tile_perm);
    (void)hipFree(p->tile_count);
    (void)hipFree(p->tile_cursor);
    (void)hipFree(p->point_code);
    (void)hipFree(p->wg_tile_base);
    (void)hipFree(p->chunks);
    (void)hipFree(p->num_chunks);
    (void)hipFree(p->box_moments);
    (void)hipFree(p->centre_parts);
    (void)hipFree(p->node_potentials);
    (void)hipFree(p->row_spectra);
    (void)hipFree(p->col_results);
    (void)hipFree(p->kernel_rows);
    (void)hipFree(p->twiddles);
    (void)hipFree(p->twiddles_short);
    (void)hipFree(p->scalars);
    (void)hipFree(p->attr);
    (void)hipFree(p->rep);
    delete p;
    if (switched) (void)hipSetDevice(current);
}

int tsne_hip_plan_create(tsne_hip_plan **plan, int num_points, int num_neighbors, int n_boxes_per_dim,
                         int device) {
    TSNE_REQUIRE(plan, "plan_create: null output pointer");
    *plan = nullptr;
    TSNE_REQUIRE(num_points > 0, "plan_create: num_points must be positive (got %d)", num_points);
    TSNE_REQUIRE(num_neighbors > 0, "plan_create: num_neighbors must be positive (got %d)", num_neighbors);
    TSNE_REQUIRE(n_boxes_per_dim >= 2 && n_boxes_per_dim <= kMaxBoxes,
                 "plan_create: n_boxes_per_dim must be in [2, %d] (got %d)", kMaxBoxes, n_boxes_per_dim);
    TSNE_TRY(hipSetDevice(device));
    tsne_hip_plan *p = new (std::nothrow) tsne_hip_plan();
    TSNE_REQUIRE(p, "plan_create: out of host memory");
    p->num_points = num_points;
    p->num_neighbors = num_neighbors;
    p->n_boxes = n_boxes_per_dim;
    p->n_nodes = n_boxes_per_dim * kInterp;
    p->device = device;
    p->lagrange = make_lagrange();
    if (const char *v = std::getenv("TSNE_KEEP_GROUPING")) p->keep_grouping = v[0] != '0';
    // The grid buffers hold the largest grid: tsne_hip_plan_set_boxes may change the size between steps.
    const size_t G2 = (size_t)(kMaxBoxes * kInterp) * (kMaxBoxes * kInterp);
    const size_t spec = (size_t)2 * kFft * kNodePad;
    const size_t N = (size_t)num_points;
    const size_t moment_bytes = sizeof(unsigned long long) * kMoments * kMaxBoxes * kMaxBoxes;
    {
        // Fixed-point scales.  Moments are sums of values in [0, 1], at most N of them in a box, and at most 4096
        // between two flushes of a workgroup's LDS region, where 2^50 is the most the conversion allows.
        int log2n = 0;
        while (((size_t)1 << log2n) < N) ++log2n;
        p->moment_scale = std::ldexp(1.0, std::min(50, 62 - log2n));
        // z_i is an interpolated sum of N kernel values in (0, 1]; the interpolation weights sum to one with
        // magnitudes up to 3.6, so |sum_i z_i| < 4 N^2.
        p->z_scale = std::ldexp(1.0, std::min(40, 61 - 2 * log2n));
        // L_m(t) = (t - s_k)(t - s_l) / denom_m in monomials.
        for (int m = 0; m < kInterp; ++m) {
            const double sk = p->lagrange.spacing[(m + 1) % kInterp], sl = p->lagrange.spacing[(m + 2) % kInterp];
            const double d = p->lagrange.denom[m];
            p->monomials.c[m][0] = sk * sl / d;
            p->monomials.c[m][1] = -(sk + sl) / d;
            p->monomials.c[m][2] = 1.0 / d;
        }
    }
    p->max_chunks = (int)(N / kChunkPoints) + kMaxTiles + 1;
    {
        int cus = 256;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, p->device) != hipSuccess) cus = 256;
        // One workgroup per compute unit: beside the attractive kernel's workgroup a unit has registers for one (128
        // per lane), and two per unit, alone, measured 3 us slower per launch and 1.2 % fewer iterations per second.
        p->spread_grid = cus;
        p->num_cus = cus;
        p->stream_grid = cus + cus / 2;
    }
    // yxy carries one spare pair so that two-point (float4) loads may straddle the end.
    bool ok = hipMalloc(&p->yxy, sizeof(float2) * (N + 2)) == hipSuccess &&
              hipMalloc(&p->tile_xy, sizeof(float2) * N) == hipSuccess &&
              hipMalloc(&p->tile_perm, sizeof(int) * N) == hipSuccess &&
              hipMalloc(&p->tile_count, sizeof(int) * kMaxTiles) == hipSuccess &&
              hipMalloc(&p->tile_cursor, sizeof(int) * kMaxTiles) == hipSuccess &&
              hipMalloc(&p->point_code, sizeof(unsigned int) * N) == hipSuccess &&
              hipMalloc(&p->wg_tile_base, sizeof(int) * (size_t)kSortBlocks * kMaxTiles) == hipSuccess &&
              hipMalloc(&p->chunks, sizeof(int4) * p->max_chunks) == hipSuccess &&
              hipMalloc(&p->num_chunks, 2 * sizeof(int)) == hipSuccess &&
              hipMalloc(&p->box_moments, moment_bytes) == hipSuccess &&
              hipMalloc(&p->centre_parts, sizeof(double2) * 2 * kMaxCentreParts) == hipSuccess &&
              hipMalloc(&p->node_potentials, sizeof(float4) * G2) == hipSuccess &&
              hipMalloc(&p->row_spectra, sizeof(float2) * spec) == hipSuccess &&
              hipMalloc(&p->col_results, sizeof(float2) * spec) == hipSuccess &&
              hipMalloc(&p->kernel_rows, sizeof(float) * (size_t)(kFft / 2 + 1) * kNodePad) == hipSuccess &&
              hipMalloc(&p->twiddles, sizeof(float2) * kFft) == hipSuccess &&
              hipMalloc(&p->twiddles_short, sizeof(float2) * kFftShort) == hipSuccess &&
              hipMalloc(&p->scalars, sizeof(LoopScalars)) == hipSuccess &&
              hipMalloc(&p->attr, sizeof(float) * 2 * N) == hipSuccess &&
              hipMalloc(&p->rep, sizeof(float) * 2 * N) == hipSuccess;
    if (ok) {
        std::vector<float2> tw(kFft), tws(kFftShort);
        for (int k = 0; k < kFft; ++k) {
            const double ang = -2.0 * M_PI * (double)k / (double)kFft;
            tw[k] = make_float2((float)std::cos(ang), (float)std::sin(ang));
        }
        for (int k = 0; k < kFftShort; ++k) {
            const double ang = -2.0 * M_PI * (double)k / (double)kFftShort;
            tws[k] = make_float2((float)std::cos(ang), (float)std::sin(ang));
        }
        ok = hipMemcpy(p->twiddles, tw.data(), sizeof(float2) * kFft, hipMemcpyHostToDevice) == hipSuccess &&
             hipMemcpy(p->twiddles_short, tws.data(), sizeof(float2) * kFftShort, hipMemcpyHostToDevice) ==
                 hipSuccess &&
             hipMemset(p->yxy, 0, sizeof(float2) * (N + 2)) == hipSuccess &&
             hipMemset(p->box_moments, 0, moment_bytes) == hipSuccess &&
             hipMemset(p->centre_parts, 0, sizeof(double2) * 2 * kMaxCentreParts) == hipSuccess &&
             hipMemset(p->tile_count, 0, sizeof(int) * kMaxTiles) == hipSuccess &&
             hipMemset(p->num_chunks, 0, 2 * sizeof(int)) == hipSuccess &&
             hipMemset(p->row_spectra, 0, sizeof(float2) * spec) == hipSuccess &&
             hipMemset(p->col_results, 0, sizeof(float2) * spec) == hipSuccess &&
             hipMemset(p->kernel_rows, 0, sizeof(float) * (size_t)(kFft / 2 + 1) * kNodePad) == hipSuccess &&
             hipMemset(p->scalars, 0, sizeof(LoopScalars)) == hipSuccess &&
             hipMemset(p->attr, 0, sizeof(float) * 2 * N) == hipSuccess &&
             hipMemset(p->rep, 0, sizeof(float) * 2 * N) == hipSuccess;
    }
    ok = ok && hipStreamCreateWithFlags(&p->side_stream, hipStreamNonBlocking) == hipSuccess &&
         hipEventCreateWithFlags(&p->fork_event, hipEventDisableTiming) == hipSuccess &&
         hipEventCreateWithFlags(&p->join_event, hipEventDisableTiming) == hipSuccess &&
         hipStreamCreateWithFlags(&p->loop_stream, hipStreamNonBlocking) == hipSuccess &&
         hipEventCreateWithFlags(&p->enter_event, hipEventDisableTiming) == hipSuccess &&
         hipEventCreateWithFlags(&p->leave_event, hipEventDisableTiming) == hipSuccess;
    if (!ok) {
        set_error("plan_create: device allocation or initialisation failed: %s",
                  hipGetErrorString(hipGetLastError()));
        tsne_hip_plan_destroy(p);
        return 1;
    }
    *plan = p;
    return 0;
}

int tsne_hip_attractive(tsne_hip_plan *plan, const float *pij, const int *indices, const float *embedding,
                        float *attractive_forces, void *stream) {
    if (check_plan(plan, "attractive")) return 1;
    TSNE_REQUIRE(embedding && attractive_forces, "attractive: null pointer argument");
    TSNE_REQUIRE((pij == nullptr) == (indices == nullptr), "attractive: pij and indices must both be given or both be null");
    hipStream_t s = (hipStream_t)stream;
    if (launch_pack_xy(plan, embedding, s)) return 1;
    if (!pij) return launch_attractive_blocked(plan, attractive_forces, s);
    return launch_attractive(plan, pij, indices, attractive_forces, s);
}

int tsne_hip_attractive_prepare(tsne_hip_plan *plan, const float *pij, const int *indices, void *stream) {
    if (check_plan(plan, "attractive_prepare")) return 1;
    TSNE_REQUIRE(pij && indices, "attractive_prepare: null pointer argument");
    return prepare_blocked(plan, pij, indices, (hipStream_t)stream);
}

int tsne_hip_repulsive(tsne_hip_plan *plan, const float *embedding, float *repulsive_forces,
                       float *normalization, float *node_charges, float *node_potentials,
                       float *point_potentials, void *stream) {
    if (check_plan(plan, "repulsive")) return 1;
    TSNE_REQUIRE(embedding && repulsive_forces && normalization, "repulsive: null pointer argument");
    hipStream_t s = (hipStream_t)stream;
    if (launch_bounds(plan, embedding, 0, s)) return 1;
    if (launch_repulsive(plan, embedding, 0, repulsive_forces, point_potentials, node_charges, s)) return 1;
    if (node_potentials)
        TSNE_TRY(hipMemcpyAsync(node_potentials, plan->node_potentials,
                                sizeof(float4) * (size_t)plan->n_nodes * plan->n_nodes, hipMemcpyDeviceToDevice,
                                s));
    return launch_finish_z(plan, normalization, s);
}

int tsne_hip_repulsive_kept(tsne_hip_plan *plan, const float *embedding, float *repulsive_forces,
                            float *normalization, float *node_charges, float *node_potentials,
                            float *point_potentials, void *stream) {
    if (check_plan(plan, "repulsive_kept")) return 1;
    TSNE_REQUIRE(embedding && repulsive_forces && normalization, "repulsive_kept: null pointer argument");
    hipStream_t s = (hipStream_t)stream;
    if (launch_bounds(plan, embedding, 0, s, false)) return 1;
    if (launch_pack_xy(plan, embedding, s)) return 1;
    if (launch_repulsive(plan, embedding, 0, repulsive_forces, point_potentials, node_charges, s, true)) return 1;
    if (node_potentials)
        TSNE_TRY(hipMemcpyAsync(node_potentials, plan->node_potentials,
                                sizeof(float4) * (size_t)plan->n_nodes * plan->n_nodes, hipMemcpyDeviceToDevice,
                                s));
    return launch_finish_z(plan, normalization, s);
}

int tsne_hip_update(tsne_hip_plan *plan, float *embedding, float *attractive_forces, float *repulsive_forces,
                    float *gains, float *old_forces, float eta, const float *normalization, float momentum,
                    float exaggeration, void *stream) {
    if (check_plan(plan, "update")) return 1;
    TSNE_REQUIRE(embedding && attractive_forces && repulsive_forces && gains && old_forces && normalization,
                 "update: null pointer argument");
    return launch_update(plan, embedding, attractive_forces, repulsive_forces, gains, old_forces, eta,
                         normalization, momentum, exaggeration, -1, (hipStream_t)stream);
}

int tsne_hip_iterate(tsne_hip_plan *plan, const float *pij, const int *indices, float *embedding, float *gains,
                     float *old_forces, int step_begin, int step_end, int force_magnify_iters, float eta,
                     float pre_exaggeration_momentum, float post_exaggeration_momentum,
                     float early_exaggeration, float *normalization, void *stream) {
    if (check_plan(plan, "iterate")) return 1;
    TSNE_REQUIRE(embedding && gains && old_forces, "iterate: null pointer argument");
    TSNE_REQUIRE((pij == nullptr) == (indices == nullptr), "iterate: pij and indices must both be given or both be null");
    TSNE_REQUIRE(pij || plan->blocked_ready || plan->csr_row_ptr, "iterate: no pattern given and none prepared");
    TSNE_REQUIRE(step_begin <= step_end, "iterate: step range [%d, %d) is reversed", step_begin, step_end);
    if (step_begin == step_end) return 0;
    // The loop runs on the plan's own stream, tied to the caller's stream by an event at either end.
    hipStream_t caller = (hipStream_t)stream, s = plan->loop_stream;
    TSNE_TRY(hipEventRecord(plan->enter_event, caller));
    TSNE_TRY(hipStreamWaitEvent(s, plan->enter_event, 0));
    // Bounds and the interleaved copy of the starting embedding; from then on
    // the update kernel keeps both current.
    // A call that takes up where the last one left off (same buffer, next step) keeps the chain's grouping of the
    // points by tile; should the caller have changed the positions in between, the grouping is merely a poor one
    // (the spread kernel finds the strays and the next step groups afresh).
    const bool continues = embedding == plan->loop_embedding && step_begin == plan->loop_next_step;
    plan->loop_embedding = embedding;
    plan->loop_next_step = step_end;
    int slot = 0;
    if (launch_bounds(plan, embedding, slot, s, !continues)) return 1;
    if (plan->recenter && launch_centre_sums(plan, embedding, slot, s)) return 1;
    if (launch_pack_xy(plan, embedding, s)) return 1;
    // Schedule of src/fit_tsne.cu:416-420: two stretches of constant parameters.  The normalisation of the last
    // step is read afterwards: its partial sums stay in the loop scalars until the next step's chain clears them.
    const int switch_at = std::min(std::max(force_magnify_iters, step_begin), step_end);
    if (launch_steps(plan, pij, indices, embedding, gains, old_forces, eta, pre_exaggeration_momentum,
                     early_exaggeration, switch_at - step_begin, slot, s))
        return 1;
    if (launch_steps(plan, pij, indices, embedding, gains, old_forces, eta, post_exaggeration_momentum, 1.0f,
                     step_end - switch_at, slot, s))
        return 1;
    if (normalization && launch_finish_z(plan, normalization, s)) return 1;
    if (profile_mark(plan, -1, s)) return 1;
    TSNE_TRY(hipEventRecord(plan->leave_event, s));
    TSNE_TRY(hipStreamWaitEvent(caller, plan->leave_event, 0));
    return 0;
}

int tsne_hip_profile_kernel_count(void) { return kKernelCount; }

const char *tsne_hip_profile_kernel_name(int id) {
    return (id >= 0 && id < kKernelCount) ? kLoopKernelNames[id] : "";
}

int tsne_hip_profile_begin(tsne_hip_plan *plan) {
    if (check_plan(plan, "profile_begin")) return 1;
    plan->profiling = true;
    plan->events_used = 0;
    plan->pending_kernel = -1;
    return 0;
}

int tsne_hip_profile_end(tsne_hip_plan *plan, double *total_ms, int *launches) {
    if (check_plan(plan, "profile_end")) return 1;
    TSNE_REQUIRE(total_ms && launches, "profile_end: null output");
    plan->profiling = false;
    for (int k = 0; k < kKernelCount; ++k) {
        total_ms[k] = 0.0;
        launches[k] = 0;
    }
    if (plan->events_used == 0) return 0;
    // (the loop's stream is in order and the last timed kernel is its last: when that one has ended, all have)
    TSNE_TRY(hipEventSynchronize(plan->events[plan->events_used - 1]));
    for (size_t e = 0; e + 1 < plan->events_used; e += 2) {
        const int id = plan->event_kernel[e / 2];
        float ms = 0.0f;
        TSNE_TRY(hipEventElapsedTime(&ms, plan->events[e], plan->events[e + 1]));
        total_ms[id] += ms;
        launches[id] += 1;
    }
    plan->events_used = 0;
    return 0;
}

int tsne_hip_profile_attractive_begin(tsne_hip_plan *plan) {
    if (check_plan(plan, "profile_attractive_begin")) return 1;
    plan->profiling_attractive = true;
    plan->events_used = 0;
    plan->pending_kernel = -1;
    return 0;
}

int tsne_hip_profile_attractive_end(tsne_hip_plan *plan, double *total_ms, int *launches) {
    if (check_plan(plan, "profile_attractive_end")) return 1;
    TSNE_REQUIRE(total_ms && launches, "profile_attractive_end: null output");
    plan->profiling_attractive = false;
    *total_ms = 0.0;
    *launches = 0;
    const size_t used = plan->events_used;
    plan->events_used = 0;
    if (used < 2) return 0;
    // (every attractive kernel ends before the update of its step starts, and the updates are in sequence)
    TSNE_TRY(hipEventSynchronize(plan->events[used - 1]));
    for (size_t e = 0; e + 1 < used; e += 2) {
        float ms = 0.0f;
        TSNE_TRY(hipEventElapsedTime(&ms, plan->events[e], plan->events[e + 1]));
        *total_ms += ms;
        *launches += 1;
    }
    return 0;
}

int tsne_hip_symmetrize_full(const float *pij_non_symmetric, const int *indices, int num_points, int num_neighbors,
                             int *row_ptr, int *col_idx, float *values, int64_t *nnz, void *stream) {
    TSNE_REQUIRE(pij_non_symmetric && indices && row_ptr && col_idx && values, "symmetrize_full: null pointer argument");
    TSNE_REQUIRE(num_points > 0 && num_neighbors > 0, "symmetrize_full: empty problem (%d x %d)", num_points,
                 num_neighbors);
    return symmetrize_full(pij_non_symmetric, indices, num_points, num_neighbors, row_ptr, col_idx, values, nnz,
                           (hipStream_t)stream);
}

int tsne_hip_attractive_csr(tsne_hip_plan *plan, const int *row_ptr, const int *col_idx, const float *values,
                            const float *embedding, float *attractive_forces, void *stream) {
    if (check_plan(plan, "attractive_csr")) return 1;
    TSNE_REQUIRE(row_ptr && col_idx && values && embedding && attractive_forces, "attractive_csr: null pointer argument");
    hipStream_t s = (hipStream_t)stream;
    if (launch_pack_xy(plan, embedding, s)) return 1;
    return launch_attractive_csr(plan, row_ptr, col_idx, values, attractive_forces, s);
}

int tsne_hip_plan_set_csr_pattern(tsne_hip_plan *plan, const int *row_ptr, const int *col_idx, const float *values) {
    if (check_plan(plan, "plan_set_csr_pattern")) return 1;
    TSNE_REQUIRE((row_ptr != nullptr) == (col_idx != nullptr) && (row_ptr != nullptr) == (values != nullptr),
                 "plan_set_csr_pattern: give all three arrays or none");
    // Captured steps hold the pattern they were captured with.
    TSNE_TRY(hipDeviceSynchronize());
    for (auto &g : plan->step_graphs) (void)hipGraphExecDestroy(g.exec);
    plan->step_graphs.clear();
    plan->csr_row_ptr = row_ptr;
    plan->csr_col_idx = col_idx;
    plan->csr_values = values;
    return 0;
}

int tsne_hip_plan_set_recenter(tsne_hip_plan *plan, int enable) {
    if (check_plan(plan, "plan_set_recenter")) return 1;
    // Captured steps carry the option as a kernel argument.
    if ((enable != 0) != plan->recenter) {
        TSNE_TRY(hipDeviceSynchronize());
        for (auto &g : plan->step_graphs) (void)hipGraphExecDestroy(g.exec);
        plan->step_graphs.clear();
    }
    plan->recenter = enable != 0;
    return 0;
}

int tsne_hip_plan_set_boxes(tsne_hip_plan *plan, int n_boxes_per_dim) {
    if (check_plan(plan, "plan_set_boxes")) return 1;
    TSNE_REQUIRE(n_boxes_per_dim >= 2 && n_boxes_per_dim <= kMaxBoxes,
                 "plan_set_boxes: n_boxes_per_dim must be in [2, %d] (got %d)", kMaxBoxes, n_boxes_per_dim);
    if (n_boxes_per_dim == plan->n_boxes) return 0;
    // Nothing of the old grid survives a step: the box moments are cleared inside the chain that consumed them,
    // every other grid buffer is written before it is read, and all of them are sized for the largest grid.
    // Captured steps carry the grid size as kernel arguments and launch shapes.
    TSNE_TRY(hipSetDevice(plan->device));
    TSNE_TRY(hipDeviceSynchronize());
    for (auto &g : plan->step_graphs) (void)hipGraphExecDestroy(g.exec);
    plan->step_graphs.clear();
    plan->n_boxes = n_boxes_per_dim;
    plan->n_nodes = n_boxes_per_dim * kInterp;
    // (a grouping of the points by tile belongs to the grid it was made on)
    TSNE_TRY(hipMemset(&plan->scalars->reuse_sort, 0, sizeof(int)));
    return 0;
}

int tsne_hip_plan_grouping_stats(tsne_hip_plan *plan, unsigned int *out) {
    if (check_plan(plan, "plan_grouping_stats")) return 1;
    TSNE_REQUIRE(out, "plan_grouping_stats: null output");
    TSNE_TRY(hipSetDevice(plan->device));
    TSNE_TRY(hipMemcpy(out, &plan->scalars->chain_runs, 3 * sizeof(unsigned int), hipMemcpyDeviceToHost));
    return 0;
}

int tsne_hip_boxes_for_spread(float spread) {
    // src/fit_tsne.cu:248-266 (the list of grid sizes) and :435 (the rule, commented out there; FIt-SNE's
    // max(min_num_intervals, spread / intervals_per_integer) with 125 and 1).
    static const int allowed[] = {25, 36, 50, 55, 60, 65, 70, 75, 80, 85, 90, 96, 100, 110, 120, 130, 140, 150};
    float want = 125.0f;
    if (spread == spread && spread > want) want = spread;  // (a NaN spread keeps the minimum)
    for (int a : allowed)
        if ((float)a >= want) return a;
    return kMaxBoxes;  // the transform length ends the list here (its next entries: 175, 200, 1125)
}

int tsne_hip_plan_check(tsne_hip_plan *plan) {
    if (check_plan(plan, "plan_check")) return 1;
    TSNE_TRY(hipSetDevice(plan->device));
    return check_attractive_waits(plan);
}

int tsne_hip_sum_squares(tsne_hip_plan *plan, const float *values, int64_t n, float *out, void *stream) {
    if (check_plan(plan, "sum_squares")) return 1;
    TSNE_REQUIRE(values && out && n > 0, "sum_squares: need a non-empty array and an output");
    return launch_sum_squares(values, n, out, (hipStream_t)stream);
}

}  // extern "C"
