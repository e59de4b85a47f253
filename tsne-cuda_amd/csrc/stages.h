// Internal launchers of the one-shot stages (defined next to their kernels).
#ifndef TSNE_HIP_STAGES_INTERNAL_H_
#define TSNE_HIP_STAGES_INTERNAL_H_

#include <vector>

#include "common.h"

namespace tsnehip {

int run_knn(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s);
int run_knn_mode(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s, int mode,
                 int *stats);
// Locality ordering (locality.hip): order_host[new] = old; synchronises the stream.
int locality_pivot_count(int N);
int locality_order(const float *points, int N, int D, std::vector<int> &order_host, hipStream_t s);
int launch_gather_rows(const float *src, const int *order, int N, int D, float *dst, hipStream_t s);
int launch_max_normalize(float *values, int64_t n, float *scratch, hipStream_t s);
int launch_perplexity(const float *sq_dist, int N, int K, float perplexity, float eps, float *pij, float *betas,
                      hipStream_t s);
int launch_symmetrize(const float *p, const int *idx, int N, int K, float *P, hipStream_t s);
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
