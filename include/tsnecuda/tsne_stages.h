/*
 * Stage-level C ABI of libtsnecuda (MI355X / gfx950 build).
 *
 * One entry point per stage of the FIt-SNE pipeline, each taking plain DEVICE
 * pointers and sizes, so that a stage can be driven and checked in isolation on
 * identical inputs.  Every function returns 0 on success and non-zero on error;
 * tsne_hip_last_error() then returns a description.  `stream` is a hipStream_t
 * passed as void* (NULL = the default stream); calls are asynchronous on that
 * stream unless stated otherwise.
 *
 * Layouts (all fp32 / int32):
 *   points      num_points x num_dims, row-major
 *   indices     num_points x num_neighbors, row-major, neighbour 0 is the point itself
 *   sq_dist     same shape, squared L2 distances, ascending per row
 *   pij         same shape
 *   embedding   2 * num_points: all x coordinates, then all y coordinates
 *   forces      same layout as embedding
 *
 * Each declaration cites the reference interface it stands in for (paths are
 * relative to the CannyLab/tsne-cuda checkout).
 */
#ifndef TSNECUDA_TSNE_STAGES_H_
#define TSNECUDA_TSNE_STAGES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tsne_hip_plan tsne_hip_plan;

/* Description of the last error raised on the calling thread ("" if none). */
const char *tsne_hip_last_error(void);

/* Exact k nearest neighbours by squared L2 distance, self first with distance
 * exactly 0, the rest ascending by (distance, index).  Distances are
 * accumulated in fp32 over ascending dimension with one fused multiply-add per
 * dimension.  Replaces tsnecuda::util::KNearestNeighbors
 * (src/util/distance_utils.cu:79-121, include/util/distance_utils.h) together
 * with PostprocessNeighborIndices (src/util/distance_utils.cu:139-154): indices
 * are int32 from the start.  num_neighbors must be <= num_points.
 * Synchronises the stream before returning. */
int tsne_hip_knn(const float *points, int num_points, int num_dims, int num_neighbors, int *indices,
                 float *sq_dist, void *stream);

/* tsne_hip_knn with an explicit choice of the distance sweep: 0 = choose by
 * shape (what tsne_hip_knn does), 1 = vector-ALU sweep, 2 = matrix-instruction
 * (MFMA) candidate sweep followed by an exact re-rank and verification (up to
 * 126 dimensions the queries stay in registers; beyond, both operands stream in
 * chunks of 64 dimensions; except at 126 dimensions the candidate distances are
 * products of bf16 terms, two per coordinate, on the bf16 matrix pipe), 3 = as 2
 * with the candidate distances as products of floats throughout.  Results are
 * identical whichever sweep runs.  stats
 * (host pointer to three ints, may be NULL): [0] = 1 if the matrix sweep ran,
 * [1] = queries that failed the verification of the sweep over all query tiles
 * (they are swept again with a wider margin or by the vector sweep), [2] = per
 * mille of the (query tile, candidate tile) pairs the matrix sweep computed (it
 * skips candidate tiles whose bounding ball lies beyond every threshold of the
 * query tile, which pays on locality-ordered points).  Same reference
 * counterpart as tsne_hip_knn. */
int tsne_hip_knn_select(const float *points, int num_points, int num_dims, int num_neighbors, int *indices,
                        float *sq_dist, void *stream, int sweep, int *stats);

/* Approximate neighbours through an inverted file, the structure of the reference's own
 * search (FAISS IndexIVFFlat, nlist = floor(sqrt(N)), nprobe = 20, L2:
 * src/util/distance_utils.cu:85-120), for sizes at which the exact search dominates a fit.
 *
 * tsne_hip_ivf_train: nlist centroids (device, nlist x num_dims floats) from `iterations`
 * Lloyd iterations on a pseudo-random sample of up to 64 points per list.  At most 128
 * dimensions.  Synchronises the stream.
 *
 * tsne_hip_knn_ivf: every point is filed under its nearest centroid; a list probes the
 * nprobe lists whose centroids are nearest to its own (itself included), and a query is
 * compared with the points of the lists probed by the lists of its 128-point tile (consecutive
 * points of the list-by-list numbering; mostly one list) and with the 8 tiles either side of
 * its own; among those candidates the result is exact (same distances, order and self-first
 * rule as tsne_hip_knn).  (FAISS probes the lists nearest to the query itself; here the
 * probes hang on the query's list so that the queries of a tile, whose distances the
 * matrix sweep computes together, share them.)  Given the centroids the result is a deterministic function of the points.
 * At most 126 dimensions, num_points >= 8192, nprobe <= 32.  stats as in tsne_hip_knn_select
 * ([1]: queries whose candidates failed the sweep's verification - near-duplicate points -
 * and were answered by the exact sweep over all points instead).  Synchronises the stream. */
int tsne_hip_ivf_train(const float *points, int num_points, int num_dims, int nlist, int iterations, float *centroids,
                       void *stream);
int tsne_hip_knn_ivf(const float *points, int num_points, int num_dims, int num_neighbors, const float *centroids,
                     int nlist, int nprobe, int *indices, float *sq_dist, void *stream, int *stats);

/* Locality ordering of the points: order[new] = old (int32, device, num_points
 * entries) such that points that are close in the input space get close numbers
 * (nearest of 64 to 256 pivots taken from the data, pivots chained greedily;
 * deterministic; the identity for fewer than 16384 points).  Nothing in t-SNE
 * depends on the numbering of the points; RunTsne renumbers them this way on
 * entry and restores the caller's numbering on exit because the attractive-force
 * kernel and the neighbour search are faster on locally ordered points.  No
 * counterpart in the reference, whose neighbour search gets its locality from the
 * FAISS IVF lists (src/util/distance_utils.cu:101-127).  Synchronises the stream. */
int tsne_hip_locality_order(const float *points, int num_points, int num_dims, int *order, void *stream);

/* rows_out[r] = rows_in[order[r]] for num_rows rows of num_cols floats. */
int tsne_hip_gather_rows(const float *rows_in, const int *order, int num_rows, int num_cols, float *rows_out,
                         void *stream);

/* Objective of the embedding the last RunTsne / pymodule_tsne call of this thread returned:
 * sum over the stored pattern of P (ln P + ln(1 + |y_i - y_j|^2) + ln Z), Z from the same
 * interpolation scheme as the gradient; negative if no fit has run.  No counterpart in the
 * reference, which never evaluates a divergence (its FunctionalKlDivergence,
 * src/include/util/thrust_transform_functions.h:26-31, has no call site). */
double tsne_hip_last_kl_divergence(void);

/* In-place division of n values by their largest absolute value.
 * Replaces tsnecuda::util::MaxNormalizeDeviceVector (src/util/math_utils.cu:66-74). */
int tsne_hip_max_normalize(float *values, int64_t n, void *stream);

/* tsne_hip_max_normalize for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The reduction scalar lives in a 256-byte
 * array that is part of the library's device image (one copy per GPU, held until
 * the process ends) instead of a per-call allocation: the call allocates and
 * frees nothing, is asynchronous on `stream` (it does not synchronise), and
 * records kernels only.  n may be at most 2^32 values; larger inputs are
 * rejected with an error.  All calls on one GPU share that GPU's array: calls
 * that overlap on one GPU (different streams or host threads) race and must be
 * serialised by the caller.  The result is bit-identical to tsne_hip_max_normalize. */
int tsne_hip_max_normalize_noalloc(float *values, int64_t n, void *stream);

/* Per-row search for the Gaussian precision that gives the requested
 * perplexity; writes row-normalised conditional probabilities.
 * Replaces tsnecuda::SearchPerplexity (src/kernels/perplexity_search.cu:81-141,
 * include/kernels/perplexity_search.h).  betas (optional, may be NULL)
 * receives the precision each row ended with. */
int tsne_hip_perplexity(const float *sq_dist, int num_points, int num_neighbors, float perplexity,
                        float epsilon, float *pij, float *betas, void *stream);

/* Pattern-restricted symmetrisation P[i,s] = (p[i,s] + sum_{t: idx[j,t]==i} p[j,t]) / 2N,
 * j = idx[i,s].  Replaces tsnecuda::util::SymmetrizeMatrixV2
 * (src/util/math_utils.cu:269-308). */
int tsne_hip_symmetrize(const float *pij_non_symmetric, const int *indices, int num_points,
                        int num_neighbors, float *pij, void *stream);

/* Full symmetrisation P = (A + A^T) / 2N, A[i, idx[i,s]] = p[i,s], as a CSR matrix with
 * the union pattern of A and A^T (nothing is dropped, so the entries sum to 1; rows have
 * ascending columns).  This is what the reference holds as a commented-out cuSPARSE
 * routine (src/util/math_utils.cu:76-225: sort, transpose, csrgeam with both factors
 * 1/(2N)); the gradient loops of both the reference and RunTsne use the pattern-restricted
 * tsne_hip_symmetrize by default (TSNE_SYMMETRIZE=full in the environment switches RunTsne
 * to this one).  Built with a device radix sort of the (row, column, value) triples and
 * a segmented reduce.  row_ptr: num_points + 1 ints; col_idx / values: room for
 * 2 * num_points * num_neighbors entries; *nnz (host, may be NULL) receives the number of
 * entries written.  Allocates its work buffers and synchronises the stream. */
int tsne_hip_symmetrize_full(const float *pij_non_symmetric, const int *indices, int num_points, int num_neighbors,
                             int *row_ptr, int *col_idx, float *values, int64_t *nnz, void *stream);

/* Scratch memory and constants for the gradient loop of one problem size.
 * n_boxes_per_dim is 130 in the reference (src/fit_tsne.cu:246-272); other
 * values (2..170) exist for testing on reduced grids.  Stands in for the
 * buffer/plan setup of src/fit_tsne.cu:274-342.  The plan is bound to `device`. */
int tsne_hip_plan_create(tsne_hip_plan **plan, int num_points, int num_neighbors, int n_boxes_per_dim,
                         int device);
void tsne_hip_plan_destroy(tsne_hip_plan *plan);

/* Re-blocks the fixed sparse pattern (pij, indices) once into the plan: entries
 * grouped by (row strip, column partition) so that the attractive kernel can
 * stage neighbour positions in LDS.  Costs 8 bytes per non-zero of device
 * memory; pij and indices are not referenced after the call has completed on
 * the stream.  Afterwards tsne_hip_attractive and tsne_hip_iterate accept
 * pij = indices = NULL and use the re-blocked copy.  Has no counterpart in the
 * reference (its P matrix stays in N x K order, src/fit_tsne.cu:153).
 * Returns 2 (with tsne_hip_last_error) when the blocked format cannot hold the
 * problem - more than 16,777,216 points or num_neighbors >= 4096 - in which case
 * the plan keeps working with an explicit (pij, indices); 1 for any other failure. */
int tsne_hip_attractive_prepare(tsne_hip_plan *plan, const float *pij, const int *indices, void *stream);

/* attr_i = sum_s P[i,s] (y_i - y_j) / (1 + |y_i - y_j|^2), j = idx[i,s].
 * Replaces tsnecuda::ComputeAttractiveForcesV3 (src/kernels/attr_forces.cu:186-240).
 * pij = indices = NULL: use the pattern given to tsne_hip_attractive_prepare. */
int tsne_hip_attractive(tsne_hip_plan *plan, const float *pij, const int *indices, const float *embedding,
                        float *attractive_forces, void *stream);

/* Attractive forces over a CSR pattern (any sparse P, e.g. the one tsne_hip_symmetrize_full
 * builds): attr_i = sum_{e in row i} values[e] (y_i - y_j) / (1 + |y_i - y_j|^2), j = col_idx[e].
 * Same reference counterpart as tsne_hip_attractive. */
int tsne_hip_attractive_csr(tsne_hip_plan *plan, const int *row_ptr, const int *col_idx, const float *values,
                            const float *embedding, float *attractive_forces, void *stream);

/* Makes tsne_hip_iterate (called with pij = indices = NULL) take its attractive forces from
 * a CSR pattern; the three arrays are borrowed and must stay valid; three NULLs clear it.
 * Synchronises the device. */
int tsne_hip_plan_set_csr_pattern(tsne_hip_plan *plan, const int *row_ptr, const int *col_idx, const float *values);

/* FFT-interpolated repulsive forces and the normalisation Z = sum_i z_i - N
 * (written to the device scalar *normalization).  Replaces, for one iteration,
 * ComputeChargesQij + minmax + PrecomputeFFT2D + NbodyFFT2D +
 * ComputeRepulsiveForces (src/fit_tsne.cu:425-469, src/kernels/rep_forces.cu,
 * src/kernels/nbodyfft.cu).  Optional outputs (may be NULL): node_charges and
 * node_potentials, (3*n_boxes)^2 x 4 floats each; point_potentials, N x 4. */
int tsne_hip_repulsive(tsne_hip_plan *plan, const float *embedding, float *repulsive_forces,
                       float *normalization, float *node_charges, float *node_potentials,
                       float *point_potentials, void *stream);

/* tsne_hip_repulsive as a step of a gradient loop evaluates it: the grouping of the points by
 * grid tile that the previous evaluation through this function left in the plan is kept while
 * few points have left the neighbourhood of their tile (those are spread on a slower path and
 * counted, see tsne_hip_plan_grouping_stats), otherwise the points are grouped afresh.  Same
 * results as tsne_hip_repulsive up to the order of floating-point additions.  No counterpart
 * in the reference. */
int tsne_hip_repulsive_kept(tsne_hip_plan *plan, const float *embedding, float *repulsive_forces,
                       float *normalization, float *node_charges, float *node_potentials,
                       float *point_potentials, void *stream);

/* Gains / momentum update of all 2N coordinates; zeroes both force arrays.
 * normalization is a device scalar.  Replaces tsnecuda::ApplyForces
 * (src/kernels/apply_forces.cu:59-82). */
int tsne_hip_update(tsne_hip_plan *plan, float *embedding, float *attractive_forces, float *repulsive_forces,
                    float *gains, float *old_forces, float eta, const float *normalization, float momentum,
                    float exaggeration, void *stream);

/* Gradient steps [step_begin, step_end) of the loop at src/fit_tsne.cu:402-580
 * with no host synchronisation inside: bounds, Z and the schedule switch at
 * force_magnify_iters stay on the device.  embedding, gains and old_forces are
 * updated in place.  normalization (device scalar, may be NULL) receives the Z
 * of the last step.  pij = indices = NULL: use the pattern given to
 * tsne_hip_attractive_prepare. */
int tsne_hip_iterate(tsne_hip_plan *plan, const float *pij, const int *indices, float *embedding, float *gains,
                     float *old_forces, int step_begin, int step_end, int force_magnify_iters, float eta,
                     float pre_exaggeration_momentum, float post_exaggeration_momentum,
                     float early_exaggeration, float *normalization, void *stream);

/* Optional re-centring of the embedding inside tsne_hip_iterate (off by default; the
 * reference's loop never re-centres, src/kernels/apply_forces.cu:11-57, its CPU
 * ancestor FIt-SNE does after every step).  When enabled, every update subtracts
 * the centre (mean x, mean y) the embedding had before the step, fused into the
 * update kernel: the forces are translation invariant, so this is re-centring after
 * every step, applied one step late and without a pass of its own. */
int tsne_hip_plan_set_recenter(tsne_hip_plan *plan, int enable);

/* Grid size of the interpolation scheme, changeable between steps.  The reference fixes
 * 125 boxes per dimension, rounded up to 130 in its list of sizes (src/fit_tsne.cu:246-266),
 * and carries FIt-SNE's adaptive rule as a comment (src/fit_tsne.cu:435):
 * max(min_num_intervals, (max_coord - min_coord) / intervals_per_integer), rounded up in
 * that list.  tsne_hip_boxes_for_spread applies that rule (125 and 1) to a coordinate
 * spread and returns 130, 140, 150 or - past the list entries the 1024-point transforms
 * can hold - 170; tsne_hip_plan_set_boxes makes a plan use a size in [2, 170] from its
 * next step on (it waits for the device and drops captured steps when the size changes). */
int tsne_hip_plan_set_boxes(tsne_hip_plan *plan, int n_boxes_per_dim);
int tsne_hip_boxes_for_spread(float spread);

/* Inside a gradient loop the repulsive evaluation keeps its grouping of the points by grid tile
 * from step to step while few points have left the neighbourhood of their tile, instead of
 * counting and scattering all points every step (the reference has no such stage: its spread is
 * 36 global atomics per point, src/kernels/nbodyfft.cu:107-139).  out[0..2]: repulsive evaluations
 * of this plan so far, those that grouped the points afresh, and points that were spread on the
 * slow path because they had strayed from their tile.  Waits for the device's pending work. */
int tsne_hip_plan_grouping_stats(tsne_hip_plan *plan, unsigned int *out);

/* Whether a kernel of this plan has reported trouble since the last call (no
 * counterpart in the reference).  Call it after synchronising the streams the
 * plan was used on.  The one condition reported today: waves of the re-blocked
 * attractive kernel coordinate through bounded waits, and a workgroup whose
 * wait ran out writes NaN forces and counts itself here.  Returns 0 when
 * nothing was reported, 1 (with tsne_hip_last_error) otherwise; clears the
 * report. */
int tsne_hip_plan_check(tsne_hip_plan *plan);

/* How far the interpolated repulsive forces of `embedding` (device, 2N floats) are from
 * exact sums over all points, on sample_count pseudo-randomly chosen points (all of them if
 * sample_count >= num_points).  result (host, three doubles): [0] relative L2 error of
 * the sampled forces F_i = sum_j (y_i - y_j) / (1 + |y_i - y_j|^2)^2, [1] relative error
 * of the sampled part of the normalisation sum_i sum_{j != i} 1 / (1 + |y_i - y_j|^2),
 * [2] the number of points sampled.  The scheme's own error (three nodes per box, 130
 * boxes: src/fit_tsne.cu:246-272) is what shows, typically 1e-3 to 1e-2.  No counterpart
 * in the reference.  Allocates its work buffers and synchronises the stream.  RunTsne
 * prints the same measure on its progress steps when TSNE_REPULSION_MONITOR=<points> is
 * set in the environment. */
int tsne_hip_repulsive_error(tsne_hip_plan *plan, const float *embedding, int sample_count, double *result,
                             void *stream);

/* Trustworthiness (Venna & Kaski) of an embedding: how far the n_neighbors nearest
 * points of every point in the embedding are from being its nearest points in the input
 * space; 1 is best.  HOST pointers: points num_points x num_dims row-major, embedding
 * 2 * num_points floats (xs then ys, i.e. a Fortran-ordered (num_points, 2) array).
 * Evaluated on the points themselves up to max_sample (<= 8192) of them, beyond that on a
 * fixed pseudo-random sample of max_sample points (neighbourhoods and ranks taken inside
 * the sample - the definition applied to the sampled points and their embedding);
 * sample_out (may be NULL, room for max_sample ints) receives the sampled indices,
 * ascending.  Squared L2 distances in both spaces, ties broken by lower index.  No
 * counterpart in the reference, which reports no quality measure.  Synchronous. */
int tsnecuda_trustworthiness(const float *points, const float *embedding, int num_points, int num_dims,
                             int n_neighbors, int max_sample, int device, double *trustworthiness, int *sample_out);

/* Squared L2 norm of n device floats into the device scalar *out
 * (tsnecuda::util::L2NormDeviceVector without the root, src/util/math_utils.cu:51-57). */
int tsne_hip_sum_squares(tsne_hip_plan *plan, const float *values, int64_t n, float *out, void *stream);

/* Per-kernel timing of tsne_hip_iterate with HIP events on the loop's own
 * stream (the measured counterpart of the reference's _time_* phase timers,
 * src/fit_tsne.cu:8-14,586-601).  Between profile_begin and profile_end every
 * kernel launch of tsne_hip_iterate carries a pair of events that receive the
 * kernel's own start and end (the gaps between launches are not counted);
 * profile_end waits for them and fills total_ms[k] / launches[k] for
 * k < tsne_hip_profile_kernel_count(). */
int tsne_hip_profile_kernel_count(void);
const char *tsne_hip_profile_kernel_name(int id);
int tsne_hip_profile_begin(tsne_hip_plan *plan);
int tsne_hip_profile_end(tsne_hip_plan *plan, double *total_ms, int *launches);
/* The same for the attractive kernel alone while the loop runs as it does unprofiled (its kernels on two
 * streams, the repulsive chain beside the attractive kernel): that one kernel's launches carry the pair of
 * events; *total_ms / *launches give its duration beside the chain (no reference counterpart:
 * the reference runs its phases one after the other). */
int tsne_hip_profile_attractive_begin(tsne_hip_plan *plan);
int tsne_hip_profile_attractive_end(tsne_hip_plan *plan, double *total_ms, int *launches);

#ifdef __cplusplus
}
#endif

#endif /* TSNECUDA_TSNE_STAGES_H_ */
