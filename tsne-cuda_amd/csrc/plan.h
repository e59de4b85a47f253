// Scratch memory and constants of the gradient loop (internal).
#ifndef TSNE_HIP_PLAN_H_
#define TSNE_HIP_PLAN_H_

#include <vector>

#include <hip/hip_ext.h>

#include "common.h"

namespace tsnehip {

constexpr int kInterp = 3;        // interpolation nodes per box and dimension (src/fit_tsne.cu:248)
constexpr int kTerms = 4;         // charges per point (src/fit_tsne.cu:254)
constexpr int kFft = 1024;        // padded transform length, >= 2 * 3 * n_boxes - 1
constexpr int kFftShort = 800;    // ... and the one used where it is enough: up to 133 boxes (400 nodes) per side
constexpr int kNodePad = 512;     // leading dimension of the transposed spectra (>= nodes per dim)
constexpr int kMaxBoxes = 170;    // 3 * 170 = 510 nodes <= kNodePad
constexpr int kTileBoxes = 5;     // boxes per side of a spreading tile (25 boxes x 21 moments x 8 B = 4.2 KB of LDS;
                                  // measured alone at 1M points: 4 -> 29 us, 5 -> 28 us, 7 -> 33 us, 10 -> 49 us)
constexpr int kMaxTiles = 34 * 34;  // ceil(kMaxBoxes / kTileBoxes)^2
constexpr int kChunkPoints = 1024;  // points one workgroup spreads into its private LDS tile
constexpr int kSortBlocks = 256;    // most workgroups of the tile count / scatter kernels

// Lagrange node positions inside a box and the basis denominators, formed in
// fp32 exactly as the reference does on the host (src/fit_tsne.cu:303-321).
struct LagrangeConsts {
    float spacing[kInterp];
    float denom[kInterp];
};

// Box moments per box: sum over the box's points of u^i v^j, (u, v) the in-box coordinates, for (i <= 4, j <= 2)
// or (i <= 2, j <= 4).
constexpr int kMoments = 21;
// Monomial coefficients of the three Lagrange basis polynomials of a box, L_m(t) = c[m][0] + c[m][1] t + c[m][2] t^2,
// in double from the fp32 node positions and denominators.
struct LagrangeMonomials {
    double c[kInterp][3];
};

// Kernels of one gradient step, in launch order (profiling slots).
enum LoopKernel {
    kKernelTileCount = 0,
    kKernelTileScatter,
    kKernelSpread,
    kKernelConvRowsForward,
    kKernelConvColumns,
    kKernelConvRowsInverse,
    kKernelGather,
    kKernelAttractive,
    kKernelUpdate,
    kKernelCount
};

}  // namespace tsnehip

struct tsne_hip_plan {
    int num_points = 0;
    int num_neighbors = 0;
    int n_boxes = 0;
    int n_nodes = 0;  // n_boxes * kInterp
    int device = 0;
    tsnehip::LagrangeConsts lagrange;

    float2 *yxy = nullptr;         // N interleaved (x, y) pairs for the neighbour gathers
    float2 *tile_xy = nullptr;     // N positions grouped by spreading tile (rebuilt every step)
    int *tile_count = nullptr;     // points per tile
    int *tile_cursor = nullptr;    // first position of every tile's run in tile_xy
    unsigned int *point_code = nullptr;  // N: (tile << 22 | rank among its workgroup's points of that tile), by the count kernel
    int *wg_tile_base = nullptr;   // kSortBlocks x kMaxTiles: where a workgroup's points start inside a tile's run
    int *tile_perm = nullptr;      // N: the point at every position of tile_xy (kept while the grouping is reused)
    int4 *chunks = nullptr;        // (tile, first point, count, box offset of the first point in the tile's LDS region)
    int *num_chunks = nullptr;  // [0] chunks of the current step, [1] ticket counter of the tile count kernel
    int max_chunks = 0;
    int spread_grid = 256;         // workgroups of the spreading kernel (one per CU)
    int num_cus = 256;            // compute units of the device
    int stream_grid = 384;        // workgroups of the kernels that only stream arrays (update): 1.5 per compute unit
    const float *loop_embedding = nullptr;  // where tsne_hip_iterate last left off: the buffer and the step after its last
    int loop_next_step = -1;
    bool keep_grouping = true;     // loops may carry the grouping by tile from step to step (TSNE_KEEP_GROUPING=0: never)
    // Box moments of the charge spreading, 64-bit fixed point (scale moment_scale): [x box][moment][y box].  All
    // zero between steps: the spread kernel adds to them, the forward row pass reads them, the column pass
    // clears them.  Sized for the largest grid.
    unsigned long long *box_moments = nullptr;
    double moment_scale = 0.0;          // 2^s with N 2^s < 2^62: a box can hold every point
    double z_scale = 0.0;               // fixed-point scale of the partial sums of z (4 N^2 z_scale < 2^63)
    tsnehip::LagrangeMonomials monomials;
    float4 *node_potentials = nullptr;  // n_nodes^2
    float2 *row_spectra = nullptr;      // 2 plane pairs x kFft x kNodePad (transposed)
    float2 *col_results = nullptr;      // same shape
    float *kernel_rows = nullptr;       // (kFft/2+1) x kNodePad: row spectra of the Cauchy kernel
    float2 *twiddles = nullptr;         // kFft roots of unity
    float2 *twiddles_short = nullptr;   // kFftShort roots of unity
    tsnehip::LoopScalars *scalars = nullptr;
    float *attr = nullptr;  // 2N, used by tsne_hip_iterate
    float *rep = nullptr;   // 2N

    // Re-blocked copy of the sparse pattern for the LDS-staged attractive kernel.
    float *ent_p = nullptr;         // entries {probability, packed (column in partition | row in strip << 11)},
                                    // 8 bytes each, grouped by (row strip, column partition), in items of
                                    // consecutive entries that are interleaved over the strips
    unsigned int *seg = nullptr;    // per strip seg_stride words: counts, run starts, partitions in opening order
    int strip_rows = 0, n_strips = 0, n_parts = 0, list_words = 0, seg_stride = 0;  // strip_rows: of the longest strip
    int *strip_row0 = nullptr;      // n_strips + 1: first row of every strip
    // Second form of the re-blocked pattern, for strips whose runs are short (see attractive_blocked.hip): the
    // column of an entry is packed relative to a window of 2^19 points, wseg lists per strip where each
    // window's entries start, and the step kernel gathers the neighbours' positions from memory.
    bool blocked_direct = false;
    unsigned int *wseg = nullptr;
    int wseg_stride = 0, n_windows = 0;
    int spin_limit = 0;             // polls before a wave of the attractive kernel gives up a wait
    bool blocked_ready = false;
    // Optional CSR pattern (borrowed pointers; tsne_hip_plan_set_csr_pattern): when set, steps without an explicit
    // N x K pattern take their attractive forces from it.
    const int *csr_row_ptr = nullptr, *csr_col_idx = nullptr;
    const float *csr_values = nullptr;
    bool recenter = false;          // the loop's updates re-centre the embedding (tsne_hip_plan_set_recenter)
    double2 *centre_parts = nullptr;  // 2 bounds slots x kMaxCentreParts: coordinate sums per workgroup

    // The repulsive chain and the attractive kernel of a step are independent: the fused loop runs
    // the chain on this side stream (default priority) and joins before the update.
    hipStream_t side_stream = nullptr;
    hipEvent_t fork_event = nullptr, join_event = nullptr;
    // The fused loop runs on this stream of the plan's own (default priority), tied to the caller's stream
    // by an event at either end: stream capture needs a stream that is not the legacy default one.
    hipStream_t loop_stream = nullptr;
    hipEvent_t enter_event = nullptr, leave_event = nullptr;
    // Replayable graphs of two consecutive steps (launch-bound problem sizes), one per distinct set of
    // arguments seen.
    struct StepGraph {
        const float *pij;
        const int *indices;
        float *embedding, *gains, *old_forces;
        float eta, momentum, exaggeration;
        int slot;
        hipGraphExec_t exec;
    };
    std::vector<StepGraph> step_graphs;

    // Optional per-kernel timing: every kernel of the loop is launched with a pair of events of its own that
    // receive its start and its end (hipExtLaunchKernelGGL), so a kernel's time is its own duration, without the
    // gaps between launches.  profile_mark names the kernel that the next launch belongs to.
    bool profiling = false;
    std::vector<hipEvent_t> events;  // pairs: start, stop
    std::vector<int> event_kernel;   // kernel id per pair
    size_t events_used = 0;          // events handed out (two per timed launch)
    int pending_kernel = -1;         // set by profile_mark, consumed by the next launch
    // The other mode: the loop runs as it does unprofiled (two streams), and only the attractive kernel is
    // launched with a pair of events (its duration beside the repulsive chain).
    bool profiling_attractive = false;
};

namespace tsnehip {

// Names the kernel (`id`, or -1 for none) that the next TSNE_LOOP_KERNEL launch is timed as (no-op unless
// profiling is on).
int profile_mark(tsne_hip_plan *p, int id, hipStream_t s);
// The pair of events for the launch that follows a profile_mark (both null when that launch is not timed).
int profile_events(tsne_hip_plan *p, hipEvent_t *start, hipEvent_t *stop);

// Launch of one of the loop's kernels from a function that returns an int status and has the plan at hand.
#define TSNE_LOOP_KERNEL(plan_, kernel_, grid_, block_, lds_, stream_, ...)                                       \
    do {                                                                                                         \
        hipEvent_t start_ = nullptr, stop_ = nullptr;                                                            \
        if (((plan_)->profiling || (plan_)->profiling_attractive) &&                                             \
            ::tsnehip::profile_events(plan_, &start_, &stop_))                                                   \
            return 1;                                                                                            \
        if (start_)                                                                                              \
            hipExtLaunchKernelGGL(kernel_, dim3(grid_), dim3(block_), (std::uint32_t)(lds_), stream_, start_,     \
                                  stop_, 0, __VA_ARGS__);                                                        \
        else                                                                                                     \
            hipLaunchKernelGGL(kernel_, dim3(grid_), dim3(block_), (std::uint32_t)(lds_), stream_, __VA_ARGS__);  \
    } while (0)

// Stage launchers shared between the stage-level ABI and the fused loop.
// `slot` selects which pair of bounds in LoopScalars the launch reads.
// new_embedding: the plan's grouping of the points by grid tile (if any) was made for other positions and is dropped.
int launch_bounds_reset(tsne_hip_plan *p, int slot, hipStream_t s, bool new_embedding = true);
int launch_bounds(tsne_hip_plan *p, const float *embedding, int slot, hipStream_t s, bool new_embedding = true);
// keep_grouping: the call is a step of a gradient loop over this embedding buffer, so the grouping of the points by
// spreading tile may be carried over from the step before (the kernels decide on the device); otherwise it is redone.
int launch_repulsive(tsne_hip_plan *p, const float *embedding, int slot, float *rep, float *point_potentials,
                     float *charges_out, hipStream_t s, bool keep_grouping = false);
// Writes Z = z_sum - N to the device scalar *normalization.
int launch_finish_z(tsne_hip_plan *p, float *normalization, hipStream_t s);
int launch_pack_xy(tsne_hip_plan *p, const float *embedding, hipStream_t s);
// out[0] = sum P ln(P (1 + d^2)), out[1] = sum P over the row-ordered pattern (device doubles).
int launch_kl_terms(const float *pij, const int *indices, const float *embedding, int N, int K, double *out,
                    hipStream_t s);
// One gradient step: repulsive chain, attractive forces (prepared pattern when pij is null), optional
// normalisation output, update.  Unless profiling is on or TSNE_OVERLAP=0 is set, the chain goes to the plan's
// side stream and overlaps the attractive kernel on s; the update on s waits for it, so s alone orders the results.
int launch_step(tsne_hip_plan *p, const float *pij, const int *indices, float *embedding, float *gains,
                float *old_forces, float eta, float momentum, float exaggeration, int slot, float *normalization,
                hipStream_t s);
// `count` consecutive steps with one set of schedule parameters on stream s, starting with bounds slot
// `slot` (updated).  Problem sizes whose steps are launch-bound replay a captured graph of two steps
// (TSNE_GRAPH=0 / 1 forces it off / on); s must not be the legacy default stream then.
int launch_steps(tsne_hip_plan *p, const float *pij, const int *indices, float *embedding, float *gains,
                 float *old_forces, float eta, float momentum, float exaggeration, int count, int &slot,
                 hipStream_t s);
// Makes stream s wait for the steps launch_step left on the side stream (no-op when there are none);
// needed before anything else reads the loop's arrays.
int launch_attractive(tsne_hip_plan *p, const float *pij, const int *indices, float *attr, hipStream_t s);
// Returns 0, kShapeNotSupported when the blocked format cannot hold the problem (more than 8192 column
// partitions, num_neighbors >= 4096, or a strip of more than 2^31 entries; the row-ordered kernel then
// serves), or 1 for any other failure (allocation, launch).
int prepare_blocked(tsne_hip_plan *p, const float *pij, const int *indices, hipStream_t s);
void release_blocked(tsne_hip_plan *p);
int launch_attractive_blocked(tsne_hip_plan *p, float *attr, hipStream_t s);
int launch_attractive_csr(tsne_hip_plan *p, const int *row_ptr, const int *col_idx, const float *values, float *attr,
                          hipStream_t s);
int check_attractive_waits(tsne_hip_plan *p);
int launch_sum_squares(const float *values, int64_t n, float *out, hipStream_t s);
int launch_centre_sums(tsne_hip_plan *p, const float *embedding, int slot, hipStream_t s);
// Error of the interpolated repulsive forces against exact sums on a sample of the points (quality.hip).
int repulsive_error(tsne_hip_plan *p, const float *embedding, int slot, int sample_count, unsigned int seed,
                    double *result, hipStream_t s);
int launch_update(tsne_hip_plan *p, float *embedding, float *attr, float *rep, float *gains, float *old_forces,
                  float eta, const float *normalization, float momentum, float exaggeration, int next_slot,
                  hipStream_t s);

}  // namespace tsnehip

#endif  // TSNE_HIP_PLAN_H_
