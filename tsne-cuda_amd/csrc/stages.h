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

}  // namespace tsnehip

#endif  // TSNE_HIP_STAGES_INTERNAL_H_
