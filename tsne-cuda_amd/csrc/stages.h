// Internal launchers of the one-shot stages (defined next to their kernels).
#ifndef TSNE_HIP_STAGES_INTERNAL_H_
#define TSNE_HIP_STAGES_INTERNAL_H_

#include <vector>

#include "common.h"

namespace tsnehip {

int run_knn(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s);
// Restriction of the sweep's candidate tiles for the approximate (inverted-file) search: the points are numbered
// list by list; tile_lists holds, per query tile of 128 points, a bitmap over the lists its queries probe
// (list_words 32-bit words each), list_tiles the first and last 128-point tile of every list (first > last for
// an empty list).  All device pointers.
struct KnnProbes {
    const unsigned int *tile_lists;
    int list_words;
    int nlist;
    const int *list_tiles;
};
// probes != nullptr: only the matrix sweep's register-resident form can take it (error otherwise); queries whose
// candidates fail the sweep's verification are then answered by the exact vector sweep over all points.
int run_knn_mode(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s, int mode,
                 int *stats, const KnnProbes *probes = nullptr);
// Inverted-file search (ivf.hip).  Trains nlist centroids (Lloyd iterations on a sample) into centroids (device,
// nlist x D).
int ivf_train(const float *points, int N, int D, int nlist, int iterations, float *centroids, hipStream_t s);
// Approximate neighbours through the inverted file given by `centroids`: every point goes to the list of its
// nearest centroid, the points are renumbered list by list (order_out[new] = old, device, N ints) and each is
// searched among the lists its tile's queries probe (nprobe nearest centroids each).  indices / sq_dist come out
// in the NEW numbering (row r = point order_out[r], entries are new numbers).  stats as in run_knn_mode.
int run_knn_approximate(const float *points, int N, int D, int K, int nprobe, int *indices, float *sq_dist,
                        int *nlist_out, int *stats, hipStream_t s);
int run_knn_ivf(const float *points, int N, int D, int K, const float *centroids, int nlist, int nprobe,
                int *order_out, int *indices, float *sq_dist, int *stats, hipStream_t s);
// `count` distinct pseudo-random indices below n, ascending (all of them when count >= n).
std::vector<int> sample_indices(int n, int count, unsigned int seed);
// Locality ordering (locality.hip): order_host[new] = old; synchronises the stream.
int locality_pivot_count(int N);
int locality_order(const float *points, int N, int D, std::vector<int> &order_host, hipStream_t s);
int launch_gather_rows(const float *src, const int *order, int N, int D, float *dst, hipStream_t s);
int launch_max_normalize(float *values, int64_t n, float *scratch, hipStream_t s);
int launch_perplexity(const float *sq_dist, int N, int K, float perplexity, float eps, float *pij, float *betas,
                      hipStream_t s);
int launch_symmetrize(const float *p, const int *idx, int N, int K, float *P, hipStream_t s);
// 0 if all n neighbour indices lie in [0, N), else 1 with the error set (named after `who`); synchronises the stream.
int validate_indices(const int *idx, int64_t n, int N, const char *who, hipStream_t s);
// (A + A^T) / 2N in CSR form with the union pattern (symmetrize_full.hip): device radix sort of the (row,
// column, value) triples of A and A^T, then a segmented reduce.  row_ptr: N + 1 ints; col_idx / values: room
// for 2 * N * K entries.  Allocates its work buffers and synchronises the stream; *nnz_out (host) = entries.
int symmetrize_full(const float *p, const int *idx, int N, int K, int *row_ptr, int *col_idx, float *values,
                    int64_t *nnz_out, hipStream_t s);
// Stable radix sort of n (64-bit key, float) pairs by the low key_bits bits (8 per pass); scratch arrays of
// the same sizes, hist: 256 counts per tile of radix_sort_tile() keys, plus 256.
int radix_sort_tile();
int radix_sort_pairs(unsigned long long *keys, float *vals, unsigned long long *keys_alt, float *vals_alt, int64_t n,
                     int key_bits, unsigned int *hist, hipStream_t s);
int launch_kl_terms_csr(const int *row_ptr, const int *col_idx, const float *values, const float *embedding, int N,
                        double *out, hipStream_t s);

}  // namespace tsnehip

#endif  // TSNE_HIP_STAGES_INTERNAL_H_
