// Approximate nearest neighbours through an inverted file (gfx950).
//
// The reference's neighbour search is FAISS IndexIVFFlat with nlist = floor(sqrt(N)) lists and nprobe = 20
// (src/util/distance_utils.cu:85-120): k-means centroids, every point filed under its nearest centroid, a
// query compared with the points of the nprobe lists whose centroids are nearest to it.  FAISS is not part of
// the reference's sources and its result is not a stable target, so the default search here is exact (knn.hip);
// this file is the approximate mode for sizes at which the exact search dominates a fit (ten million points:
// 26 s).  It keeps FAISS's structure and parameters and runs the search itself on the exact search's matrix
// sweep, which works on tiles of 128 consecutive points:
//
//   1. train:   Lloyd iterations on a pseudo-random sample of 64 points per list (ivf_train);
//   2. file:    every point goes to the list of its nearest centroid, by (distance, list number); distances
//               are fp32, one fused multiply-add per dimension in ascending order (ivf_probe_kernel); the
//               points are renumbered list by list (list, then old number: a radix sort of
//               list * 2^b + number), so a list is a range of the numbering;
//   3. probe:   a LIST probes the nprobe lists whose centroids are nearest to its own centroid (itself
//               first), and a query probes what its list probes.  FAISS lets every query probe the lists
//               nearest to the query itself; the sweep, however, computes whole tiles of 128 x 128 distances,
//               so what a tile visits is the union over its 128 queries - and in data without structure below
//               the cluster level (the benchmark's 50-dimensional Gaussians) the per-query lists of 128
//               neighbours in the numbering barely overlap: their union was a fifth of all points at ten
//               million, as slow as the exact search.  Per list, tile mates share their probes;
//   4. search:  a query tile visits its neighbourhood in the numbering (8 tiles either side, as the exact
//               sweep does) and every tile that overlaps a list probed by the list of one of its queries.
//               Within those candidates the result is exact: same distances, same order, self first
//               (knn.hip does the rest).
//
// Given the centroids, every step is a deterministic function of the points, which is what the parity tests
// hold against a CPU restatement (identical candidate sets, hence identical neighbours); recall against the
// exact search is what the approximation costs.
#include <algorithm>
#include <cmath>
#include <vector>

#include "plan.h"
#include "stages.h"

namespace tsnehip {

namespace {

typedef unsigned long long u64;

struct Buffer {
    void *ptr = nullptr;
    ~Buffer() {
        if (ptr) (void)hipFree(ptr);
    }
    bool alloc(size_t bytes) { return hipMalloc(&ptr, bytes ? bytes : 1) == hipSuccess; }
    template <typename T>
    T *as() const {
        return static_cast<T *>(ptr);
    }
};

// One thread per point: the point in registers (DMAX floats), the centroids read at wave-uniform addresses.
// list_of[i]: the nearest centroid of point i by (distance, centroid number).
template <int DMAX>
__global__ __launch_bounds__(256) void ivf_assign_kernel(const float *__restrict__ points, int n, int D,
                                                         const float *__restrict__ centroids, int nlist,
                                                         int *__restrict__ list_of) {
#pragma clang fp contract(off)
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = i < n;
    float x[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) x[d] = (live && d < D) ? points[(size_t)i * D + d] : 0.0f;
    float best_d = INFINITY;
    int best_l = 0;
    for (int c = 0; c < nlist; ++c) {
        const float *cen = centroids + (size_t)c * D;
        float acc = 0.0f;
#pragma unroll
        for (int d = 0; d < DMAX; ++d) {
            if (d < D) {
                const float df = x[d] - cen[d];
                acc = fmaf(df, df, acc);
            }
        }
        if (acc < best_d) {  // ascending centroid number: on equal distances the earlier one stays
            best_d = acc;
            best_l = c;
        }
    }
    if (live) list_of[i] = best_l;
}

int launch_assign(const float *points, int n, int D, const float *centroids, int nlist, int *list_of, hipStream_t s) {
    const int blocks = div_up(n, 256);
    if (D <= 32) {
        ivf_assign_kernel<32><<<blocks, 256, 0, s>>>(points, n, D, centroids, nlist, list_of);
    } else if (D <= 64) {
        ivf_assign_kernel<64><<<blocks, 256, 0, s>>>(points, n, D, centroids, nlist, list_of);
    } else {
        ivf_assign_kernel<128><<<blocks, 256, 0, s>>>(points, n, D, centroids, nlist, list_of);
    }
    TSNE_LAUNCHED(s);
    return 0;
}

// One workgroup per list: the nprobe lists whose centroids are nearest to its own, in ascending (distance,
// list number) - round r selects the smallest pair above the one round r - 1 selected, recomputing the
// distances (the same fma chain every round, so the same bits); nlist * nprobe distance evaluations per list
// are small change next to the search itself.  out[l * nprobe + r].
__global__ __launch_bounds__(256) void list_probe_kernel(const float *__restrict__ centroids, int nlist, int D,
                                                         int nprobe, int *__restrict__ out) {
#pragma clang fp contract(off)
    extern __shared__ float own[];  // D floats
    __shared__ float part_d[4];
    __shared__ int part_l[4];
    const int l = blockIdx.x, tid = threadIdx.x;
    for (int d = tid; d < D; d += 256) own[d] = centroids[(size_t)l * D + d];
    __syncthreads();
    float last_d = -INFINITY;
    int last_l = -1;
    for (int r = 0; r < nprobe; ++r) {
        float best_d = INFINITY;
        int best_l = 0x7fffffff;
        for (int c = tid; c < nlist; c += 256) {
            const float *cen = centroids + (size_t)c * D;
            float acc = 0.0f;
            for (int d = 0; d < D; ++d) {
                const float df = own[d] - cen[d];
                acc = fmaf(df, df, acc);
            }
            const bool above = acc > last_d || (acc == last_d && c > last_l);
            if (above && (acc < best_d || (acc == best_d && c < best_l))) {
                best_d = acc;
                best_l = c;
            }
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) {
            const float od = __shfl_xor(best_d, m);
            const int ol = __shfl_xor(best_l, m);
            if (od < best_d || (od == best_d && ol < best_l)) {
                best_d = od;
                best_l = ol;
            }
        }
        if ((tid & 63) == 0) {
            part_d[tid >> 6] = best_d;
            part_l[tid >> 6] = best_l;
        }
        __syncthreads();
        best_d = part_d[0];
        best_l = part_l[0];
#pragma unroll
        for (int w = 1; w < 4; ++w)
            if (part_d[w] < best_d || (part_d[w] == best_d && part_l[w] < best_l)) {
                best_d = part_d[w];
                best_l = part_l[w];
            }
        __syncthreads();
        last_d = best_d;
        last_l = best_l;
        if (tid == 0) out[(size_t)l * nprobe + r] = best_l;
    }
}

// ---- k-means ----
__global__ __launch_bounds__(256) void gather_sample_kernel(const float *__restrict__ points,
                                                            const int *__restrict__ sample, int S, int D,
                                                            float *__restrict__ out) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < (int64_t)S * D;
         e += (int64_t)gridDim.x * blockDim.x)
        out[e] = points[(size_t)sample[e / D] * D + e % D];
}

__global__ __launch_bounds__(256) void kmeans_accumulate_kernel(const float *__restrict__ x,
                                                                const int *__restrict__ assign, int S, int D,
                                                                float *__restrict__ sums, int *__restrict__ counts) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < (int64_t)S * D;
         e += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(e / D), d = (int)(e % D);
        const int c = assign[i];
        atomicAdd(&sums[(size_t)c * D + d], x[e]);
        if (d == 0) atomicAdd(&counts[c], 1);
    }
}

// A list nobody was assigned to keeps its centroid.
__global__ __launch_bounds__(256) void kmeans_update_kernel(float *__restrict__ centroids,
                                                            const float *__restrict__ sums,
                                                            const int *__restrict__ counts, int nlist, int D) {
    for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < nlist * D; e += gridDim.x * blockDim.x) {
        const int c = counts[e / D];
        if (c > 0) centroids[e] = sums[e] / (float)c;
    }
}

// ---- filing ----
__global__ __launch_bounds__(256) void list_keys_kernel(const int *__restrict__ probes, int n, int nprobe,
                                                        int index_bits, u64 *__restrict__ keys) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) keys[i] = ((u64)(unsigned int)probes[(size_t)i * nprobe] << index_bits) | (u64)(unsigned int)i;
    // (probes: the points' lists, nprobe entries per point of which the first counts)
}

// order[new] = old; list_start[l] = first new number of list l (list_start[nlist] = n).
__global__ __launch_bounds__(256) void unpack_order_kernel(const u64 *__restrict__ keys, int n, int index_bits,
                                                           int nlist, int *__restrict__ order,
                                                           int *__restrict__ list_start) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const u64 key = keys[t];
    order[t] = (int)(key & ((1ull << index_bits) - 1ull));
    const int list = (int)(key >> index_bits);
    const int prev = t == 0 ? -1 : (int)(keys[t - 1] >> index_bits);
    for (int l = prev + 1; l <= list; ++l) list_start[l] = t;
    if (t == n - 1)
        for (int l = list + 1; l <= nlist; ++l) list_start[l] = n;
}

__global__ __launch_bounds__(256) void list_tiles_kernel(const int *__restrict__ list_start, int nlist,
                                                         int *__restrict__ list_tiles) {
    const int l = blockIdx.x * blockDim.x + threadIdx.x;
    if (l >= nlist) return;
    const int a = list_start[l], b = list_start[l + 1];
    list_tiles[2 * l] = b > a ? a / 128 : 1;
    list_tiles[2 * l + 1] = b > a ? (b - 1) / 128 : 0;
}

// One workgroup per tile of 128 points (new numbering): the union of the lists its points' lists probe.
__global__ __launch_bounds__(128) void tile_lists_kernel(const int *__restrict__ list_of,
                                                         const int *__restrict__ list_probes,
                                                         const int *__restrict__ order, int n, int nprobe,
                                                         int list_words, unsigned int *__restrict__ tile_lists) {
    extern __shared__ unsigned int bits[];
    for (int w = threadIdx.x; w < list_words; w += 128) bits[w] = 0u;
    __syncthreads();
    const int q = blockIdx.x * 128 + threadIdx.x;
    if (q < n) {
        const int *mine = list_probes + (size_t)list_of[order[q]] * nprobe;
        for (int r = 0; r < nprobe; ++r) {
            const int l = mine[r];
            atomicOr(&bits[l >> 5], 1u << (l & 31));
        }
    }
    __syncthreads();
    for (int w = threadIdx.x; w < list_words; w += 128) tile_lists[(size_t)blockIdx.x * list_words + w] = bits[w];
}

// Results of the search in the new numbering back to the caller's: row order[r] <- row r, entries mapped.
__global__ __launch_bounds__(256) void unpermute_kernel(const int *__restrict__ idx_new, const float *__restrict__ d_new,
                                                        const int *__restrict__ order, int n, int K,
                                                        int *__restrict__ idx_out, float *__restrict__ d_out) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < (int64_t)n * K;
         e += (int64_t)gridDim.x * blockDim.x) {
        const int r = (int)(e / K), sidx = (int)(e % K);
        const size_t dst = (size_t)order[r] * K + sidx;
        idx_out[dst] = order[idx_new[e]];
        d_out[dst] = d_new[e];
    }
}

int bits_for(int n) {
    int b = 1;
    while ((1ll << b) < (long long)n) ++b;
    return b;
}

}  // namespace

int ivf_train(const float *points, int N, int D, int nlist, int iterations, float *centroids, hipStream_t s) {
    if (nlist < 1 || nlist > N) {
        set_error("ivf_train: nlist must be in [1, num_points] (got %d for %d points)", nlist, N);
        return 1;
    }
    if (D > 128) {
        set_error("ivf_train: at most 128 dimensions (got %d)", D);
        return 1;
    }
    const std::vector<int> sample = sample_indices(N, (int)std::min<int64_t>(N, (int64_t)64 * nlist), 777u);
    const int S = (int)sample.size();
    // The first nlist sampled points, in pseudo-random order, start as centroids: draw them from the sample
    // with the same generator so that they are spread over the numbering, not its first points.
    const std::vector<int> seeds = sample_indices(S, nlist, 4242u);
    Buffer d_sample, d_x, d_assign, d_sums, d_counts, d_seed_rows;
    if (!d_sample.alloc(sizeof(int) * (size_t)S) || !d_x.alloc(sizeof(float) * (size_t)S * D) ||
        !d_assign.alloc(sizeof(int) * (size_t)S) || !d_sums.alloc(sizeof(float) * (size_t)nlist * D) ||
        !d_counts.alloc(sizeof(int) * (size_t)nlist) || !d_seed_rows.alloc(sizeof(int) * (size_t)nlist)) {
        set_error("ivf_train: out of device memory");
        return 1;
    }
    TSNE_TRY(hipMemcpyAsync(d_sample.ptr, sample.data(), sizeof(int) * (size_t)S, hipMemcpyHostToDevice, s));
    gather_sample_kernel<<<std::min(div_up((int64_t)S * D, 256), 65536), 256, 0, s>>>(points, d_sample.as<int>(), S, D,
                                                                                    d_x.as<float>());
    TSNE_LAUNCHED(s);
    TSNE_TRY(hipMemcpyAsync(d_seed_rows.ptr, seeds.data(), sizeof(int) * (size_t)nlist, hipMemcpyHostToDevice, s));
    gather_sample_kernel<<<std::min(div_up((int64_t)nlist * D, 256), 65536), 256, 0, s>>>(
        d_x.as<float>(), d_seed_rows.as<int>(), nlist, D, centroids);
    TSNE_LAUNCHED(s);
    for (int it = 0; it < iterations; ++it) {
        if (launch_assign(d_x.as<float>(), S, D, centroids, nlist, d_assign.as<int>(), s)) return 1;
        TSNE_TRY(hipMemsetAsync(d_sums.ptr, 0, sizeof(float) * (size_t)nlist * D, s));
        TSNE_TRY(hipMemsetAsync(d_counts.ptr, 0, sizeof(int) * (size_t)nlist, s));
        kmeans_accumulate_kernel<<<std::min(div_up((int64_t)S * D, 256), 65536), 256, 0, s>>>(
            d_x.as<float>(), d_assign.as<int>(), S, D, d_sums.as<float>(), d_counts.as<int>());
        TSNE_LAUNCHED(s);
        kmeans_update_kernel<<<div_up(nlist * D, 256), 256, 0, s>>>(centroids, d_sums.as<float>(), d_counts.as<int>(),
                                                                   nlist, D);
        TSNE_LAUNCHED(s);
    }
    TSNE_TRY(hipStreamSynchronize(s));  // the host vectors and work buffers go out of scope
    return 0;
}

int run_knn_ivf(const float *points, int N, int D, int K, const float *centroids, int nlist, int nprobe,
                int *order_out, int *indices, float *sq_dist, int *stats, hipStream_t s) {
    if (nprobe < 1 || nprobe > nlist) {
        set_error("knn_ivf: nprobe must be in [1, nlist] (got %d, nlist %d)", nprobe, nlist);
        return 1;
    }
    if (D > 126) {
        set_error("knn_ivf: the approximate search takes at most 126 dimensions (got %d)", D);
        return 1;
    }
    const int T = div_up(N, 128), list_words = div_up(nlist, 32);
    const int index_bits = bits_for(N), key_bits = index_bits + bits_for(nlist);
    const int sort_tiles = div_up(N, radix_sort_tile());
    Buffer probes, list_probes, keys, keys_alt, vals, vals_alt, hist, list_start, list_tiles, tile_lists, sorted;
    if (!probes.alloc(sizeof(int) * (size_t)N) || !list_probes.alloc(sizeof(int) * (size_t)nlist * nprobe) ||
        !keys.alloc(sizeof(u64) * (size_t)N) ||
        !keys_alt.alloc(sizeof(u64) * (size_t)N) || !vals.alloc(sizeof(float) * (size_t)N) ||
        !vals_alt.alloc(sizeof(float) * (size_t)N) || !hist.alloc(sizeof(unsigned int) * 256 * ((size_t)sort_tiles + 1)) ||
        !list_start.alloc(sizeof(int) * ((size_t)nlist + 1)) || !list_tiles.alloc(sizeof(int) * 2 * (size_t)nlist) ||
        !tile_lists.alloc(sizeof(unsigned int) * (size_t)T * list_words) ||
        !sorted.alloc(sizeof(float) * (size_t)N * D)) {
        set_error("knn_ivf: out of device memory");
        return 1;
    }
    if (launch_assign(points, N, D, centroids, nlist, probes.as<int>(), s)) return 1;
    list_probe_kernel<<<nlist, 256, sizeof(float) * D, s>>>(centroids, nlist, D, nprobe, list_probes.as<int>());
    TSNE_LAUNCHED(s);
    list_keys_kernel<<<div_up(N, 256), 256, 0, s>>>(probes.as<int>(), N, 1, index_bits, keys.as<u64>());
    TSNE_LAUNCHED(s);
    TSNE_TRY(hipMemsetAsync(vals.ptr, 0, sizeof(float) * (size_t)N, s));  // the sort moves pairs; the values are unused
    if (radix_sort_pairs(keys.as<u64>(), vals.as<float>(), keys_alt.as<u64>(), vals_alt.as<float>(), N, key_bits,
                         hist.as<unsigned int>(), s))
        return 1;
    unpack_order_kernel<<<div_up(N, 256), 256, 0, s>>>(keys.as<u64>(), N, index_bits, nlist, order_out,
                                                       list_start.as<int>());
    TSNE_LAUNCHED(s);
    list_tiles_kernel<<<div_up(nlist, 256), 256, 0, s>>>(list_start.as<int>(), nlist, list_tiles.as<int>());
    TSNE_LAUNCHED(s);
    tile_lists_kernel<<<T, 128, sizeof(unsigned int) * list_words, s>>>(probes.as<int>(), list_probes.as<int>(),
                                                                        order_out, N, nprobe, list_words,
                                                                        tile_lists.as<unsigned int>());
    TSNE_LAUNCHED(s);
    if (launch_gather_rows(points, order_out, N, D, sorted.as<float>(), s)) return 1;
    KnnProbes info;
    info.tile_lists = tile_lists.as<unsigned int>();
    info.list_words = list_words;
    info.nlist = nlist;
    info.list_tiles = list_tiles.as<int>();
    // (synchronises the stream before it returns: the work buffers above may then go)
    return run_knn_mode(sorted.as<float>(), N, D, K, indices, sq_dist, s, 2, stats, &info);
}

// The search in the caller's numbering: run_knn_ivf, then rows and neighbour numbers mapped back.
int run_knn_ivf_caller_order(const float *points, int N, int D, int K, const float *centroids, int nlist, int nprobe,
                             int *indices, float *sq_dist, int *stats, hipStream_t s) {
    const size_t nnz = (size_t)N * K;
    Buffer order, idx_new, d_new;
    if (!order.alloc(sizeof(int) * (size_t)N) || !idx_new.alloc(sizeof(int) * nnz) ||
        !d_new.alloc(sizeof(float) * nnz)) {
        set_error("knn_ivf: out of device memory");
        return 1;
    }
    if (const int rc = run_knn_ivf(points, N, D, K, centroids, nlist, nprobe, order.as<int>(), idx_new.as<int>(),
                                   d_new.as<float>(), stats, s))
        return rc;  // (kShapeNotSupported: the restricted sweep cannot hold this many neighbours)
    unpermute_kernel<<<(int)std::min<int64_t>(div_up((int64_t)nnz, 256), 65536), 256, 0, s>>>(
        idx_new.as<int>(), d_new.as<float>(), order.as<int>(), N, K, indices, sq_dist);
    TSNE_TRY(hipGetLastError());
    TSNE_TRY(hipStreamSynchronize(s));
    return 0;
}

// Train and search in one call, with the reference's choice of nlist = floor(sqrt(N)) (src/fit_tsne.cu:118 via
// src/util/distance_utils.cu:92) and its ten k-means rounds.
int run_knn_approximate(const float *points, int N, int D, int K, int nprobe, int *indices, float *sq_dist,
                        int *nlist_out, int *stats, hipStream_t s) {
    int nlist = (int)std::floor(std::sqrt((double)N));
    if (nlist < 1) nlist = 1;
    if (nprobe > nlist) nprobe = nlist;
    Buffer centroids;
    if (!centroids.alloc(sizeof(float) * (size_t)nlist * D)) {
        set_error("knn_ivf: out of device memory");
        return 1;
    }
    if (ivf_train(points, N, D, nlist, 10, centroids.as<float>(), s)) return 1;
    if (nlist_out) *nlist_out = nlist;
    return run_knn_ivf_caller_order(points, N, D, K, centroids.as<float>(), nlist, nprobe, indices, sq_dist, stats, s);
}

}  // namespace tsnehip

using namespace tsnehip;

extern "C" int tsne_hip_ivf_train(const float *points, int num_points, int num_dims, int nlist, int iterations,
                                  float *centroids, void *stream) {
    if (!points || !centroids || num_points < 1 || num_dims < 1 || iterations < 0) {
        set_error("ivf_train: bad argument");
        return 1;
    }
    return ivf_train(points, num_points, num_dims, nlist, iterations, centroids, (hipStream_t)stream);
}

extern "C" int tsne_hip_knn_ivf(const float *points, int num_points, int num_dims, int num_neighbors,
                                const float *centroids, int nlist, int nprobe, int *indices, float *sq_dist,
                                void *stream, int *stats) {
    if (!points || !centroids || !indices || !sq_dist) {
        set_error("knn_ivf: null pointer argument");
        return 1;
    }
    if (num_points < 1 || num_dims < 1 || num_neighbors < 1 || num_neighbors > num_points) {
        set_error("knn_ivf: need 1 <= num_neighbors <= num_points and num_dims >= 1");
        return 1;
    }
    return run_knn_ivf_caller_order(points, num_points, num_dims, num_neighbors, centroids, nlist, nprobe, indices,
                                    sq_dist, stats, (hipStream_t)stream);
}
