// Locality ordering of the input points (gfx950).
//
// Nothing in t-SNE depends on how the points are numbered, but two stages run
// faster when points that are close in the input space have close numbers:
//
//   * the re-blocked attractive kernel only stages the column partitions a row
//     strip actually references, and
//   * the kNN sweep can skip candidate tiles whose bounding ball is farther from
//     a query tile than the current k-th distances.
//
// The ordering is a coarse one: M pivots are drawn from the data (a fixed
// pseudo-random draw), every point is labelled with its nearest pivot, the pivots are chained
// greedily (each next to its nearest unvisited one) and the points are sorted by
// the chain position of their pivot, original number second.  It is
// deterministic.  The reference has no counterpart: its neighbour search gets its
// locality from the FAISS IVF lists (src/util/distance_utils.cu:101-127).
#include <algorithm>
#include <cmath>
#include <limits>
#include <vector>

#include "stages.h"

namespace tsnehip {

namespace {

constexpr int kMaxPivots = 256;
constexpr int kAssignThreads = 256;

// pivots_t: D x M (pivot j, dimension d at [d * M + j]); rows: M x D copy for the host.
struct PivotIds {
    int id[kMaxPivots];
};

__global__ void gather_pivots_kernel(const float *__restrict__ points, int D, int M, PivotIds pivots,
                                     float *__restrict__ pivots_t, float *__restrict__ rows) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (int64_t)M * D) return;
    const int j = (int)(t / D), d = (int)(t % D);
    const float v = points[(int64_t)pivots.id[j] * D + d];
    pivots_t[(size_t)d * M + j] = v;
    rows[t] = v;
}

// One wave labels one point at a time; lane l holds pivots l, l + 64, ...
template <int PER_LANE>
__global__ __launch_bounds__(kAssignThreads) void pivot_assign_kernel(const float *__restrict__ points, int N,
                                                                      int D, int M,
                                                                      const float *__restrict__ pivots_t,
                                                                      int *__restrict__ labels) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = (blockIdx.x * kAssignThreads + threadIdx.x) / kWave;
    const int n_waves = gridDim.x * (kAssignThreads / kWave);
    for (int i = wave; i < N; i += n_waves) {
        const float *x = points + (size_t)i * D;
        float acc[PER_LANE];
#pragma unroll
        for (int u = 0; u < PER_LANE; ++u) acc[u] = 0.0f;
        for (int d = 0; d < D; ++d) {
            const float xv = x[d];
#pragma unroll
            for (int u = 0; u < PER_LANE; ++u) {
                const int j = lane + u * kWave;
                const float diff = xv - pivots_t[(size_t)d * M + (j < M ? j : 0)];
                acc[u] = fmaf(diff, diff, acc[u]);
            }
        }
        float best = INFINITY;
        int best_j = 0;
#pragma unroll
        for (int u = 0; u < PER_LANE; ++u) {
            const int j = lane + u * kWave;
            if (j < M && acc[u] < best) {
                best = acc[u];
                best_j = j;
            }
        }
#pragma unroll
        for (int m = kWave / 2; m > 0; m >>= 1) {
            const float ob = __shfl_xor(best, m, kWave);
            const int oj = __shfl_xor(best_j, m, kWave);
            if (ob < best || (ob == best && oj < best_j)) {
                best = ob;
                best_j = oj;
            }
        }
        if (lane == 0) labels[i] = best_j;
    }
}

__global__ void gather_rows_kernel(const float *__restrict__ src, const int *__restrict__ order, int64_t N, int D,
                                   float *__restrict__ dst) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= N * D) return;
    const int64_t r = t / D;
    dst[t] = src[(int64_t)order[r] * D + (t - r * D)];
}

struct Scratch {
    void *p = nullptr;
    ~Scratch() { (void)hipFree(p); }
    bool alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1) == hipSuccess; }
    template <typename T>
    T *as() { return static_cast<T *>(p); }
};

}  // namespace

int locality_pivot_count(int N) {
    if (N < 16384) return 0;  // too few points for the ordering to matter
    // At least 64: every cluster of the data should own a pivot (with 10 equal clusters the chance
    // that one of them is missed by 64 random draws is 0.1 %).
    int m = 64;
    while (m * 2 <= N / 2048 && m * 2 <= kMaxPivots) m *= 2;
    return m;
}

// order_host[new] = old.  Synchronises the stream.
int locality_order(const float *points, int N, int D, std::vector<int> &order_host, hipStream_t s) {
    order_host.resize(N);
    const int M = locality_pivot_count(N);
    if (M == 0) {
        for (int i = 0; i < N; ++i) order_host[i] = i;
        return 0;
    }
    Scratch pivots_t, rows, labels;
    if (!pivots_t.alloc(sizeof(float) * (size_t)M * D) || !rows.alloc(sizeof(float) * (size_t)M * D) ||
        !labels.alloc(sizeof(int) * (size_t)N)) {
        set_error("locality_order: out of device memory");
        return 1;
    }
    // Pivots: a fixed pseudo-random draw (splitmix64 of the pivot number), so that no regular
    // pattern in the caller's numbering can line up with it; the draw is the same on every call.
    PivotIds pivots;
    for (int j = 0; j < M; ++j) {
        uint64_t z = (uint64_t)(j + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        pivots.id[j] = (int)(z % (uint64_t)N);
    }
    gather_pivots_kernel<<<div_up((int64_t)M * D, 256), 256, 0, s>>>(points, D, M, pivots, pivots_t.as<float>(),
                                                                    rows.as<float>());
    TSNE_LAUNCHED(s);
    const int grid = std::min(div_up(N, kAssignThreads / kWave), 4096);
    if (M <= 64)
        pivot_assign_kernel<1><<<grid, kAssignThreads, 0, s>>>(points, N, D, M, pivots_t.as<float>(), labels.as<int>());
    else if (M <= 128)
        pivot_assign_kernel<2><<<grid, kAssignThreads, 0, s>>>(points, N, D, M, pivots_t.as<float>(), labels.as<int>());
    else
        pivot_assign_kernel<4><<<grid, kAssignThreads, 0, s>>>(points, N, D, M, pivots_t.as<float>(), labels.as<int>());
    TSNE_LAUNCHED(s);

    std::vector<float> h_rows((size_t)M * D);
    std::vector<int> h_labels(N);
    TSNE_TRY(hipMemcpyAsync(h_rows.data(), rows.p, sizeof(float) * h_rows.size(), hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipMemcpyAsync(h_labels.data(), labels.p, sizeof(int) * (size_t)N, hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipStreamSynchronize(s));

    // Greedy chain over the pivots: start at pivot 0, always continue with the
    // nearest pivot not yet placed.
    std::vector<int> chain_pos(M, -1);
    {
        std::vector<char> placed(M, 0);
        int cur = 0;
        for (int pos = 0; pos < M; ++pos) {
            placed[cur] = 1;
            chain_pos[cur] = pos;
            double best = std::numeric_limits<double>::infinity();
            int next = -1;
            for (int j = 0; j < M; ++j) {
                if (placed[j]) continue;
                double d2 = 0.0;
                for (int d = 0; d < D; ++d) {
                    const double diff = (double)h_rows[(size_t)cur * D + d] - (double)h_rows[(size_t)j * D + d];
                    d2 += diff * diff;
                }
                if (d2 < best) {
                    best = d2;
                    next = j;
                }
            }
            if (next < 0) break;
            cur = next;
        }
    }
    // Stable counting sort of the points by chain position.
    std::vector<int64_t> start(M + 1, 0);
    for (int i = 0; i < N; ++i) start[chain_pos[h_labels[i]] + 1] += 1;
    for (int c = 0; c < M; ++c) start[c + 1] += start[c];
    for (int i = 0; i < N; ++i) order_host[start[chain_pos[h_labels[i]]]++] = i;
    return 0;
}

// dst[r] = src[order[r]] for N rows of D floats (order on the device).
int launch_gather_rows(const float *src, const int *order, int N, int D, float *dst, hipStream_t s) {
    gather_rows_kernel<<<div_up((int64_t)N * D, 256), 256, 0, s>>>(src, order, N, D, dst);
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
