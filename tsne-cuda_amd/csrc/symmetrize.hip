// Pattern-restricted symmetrisation of the conditional probabilities for gfx950.
//
//   P[i,s] = (p[i,s] + sum_{t : idx[j,t] == i} p[j,t]) / (2 N),   j = idx[i,s]
//
// Semantics: src/util/math_utils.cu:269-291 of the reference (the N x K pattern
// is kept; pairs present in only one direction keep half their mass).  The
// reference gives every non-zero its own thread that walks row j alone; here a
// group of lanes owns row i and the whole group scans each row j together, so
// every index row is fetched with coalesced loads and the match is found with a
// ballot.
#include "plan.h"
#include "stages.h"

#include <algorithm>

namespace tsnehip {

namespace {

template <int LANES>
__global__ __launch_bounds__(256) void symmetrize_kernel(const float *__restrict__ p, const int *__restrict__ idx,
                                                         int N, int K, float *__restrict__ P) {
    constexpr int kRowsPerBlock = 256 / LANES;
    const int row = blockIdx.x * kRowsPerBlock + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    if (row >= N) return;  // whole groups leave together
    const size_t base = (size_t)row * K;
    const double denom = 2.0 * (double)N;
    for (int s0 = 0; s0 < K; s0 += LANES) {
        const int my_s = s0 + lane;
        const int my_j = my_s < K ? idx[base + my_s] : 0;
        float my_acc = my_s < K ? p[base + my_s] : 0.0f;
        const int count = min(LANES, K - s0);
        for (int t = 0; t < count; ++t) {
            const int j = __shfl(my_j, t, LANES);
            const size_t jb = (size_t)j * K;
            float found = 0.0f;
            for (int u = lane; u < K; u += LANES)
                if (idx[jb + u] == row) found += p[jb + u];
            found = group_sum<LANES>(found);
            if (lane == t) my_acc += found;
        }
        if (my_s < K) P[base + my_s] = (float)((double)my_acc / denom);
    }
}

__global__ __launch_bounds__(256) void index_range_kernel(const int *__restrict__ idx, int64_t n, int N,
                                                          int *__restrict__ flag) {
    bool bad = false;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x)
        bad = bad || (unsigned int)idx[e] >= (unsigned int)N;
    if (__any(bad) && (threadIdx.x & (kWave - 1)) == 0) atomicOr(flag, 1);
}

}  // namespace

// The stages that turn neighbour numbers into addresses of their own (sort keys, LDS bitmaps, row pointers)
// first make sure that every one of them names a point: 0 if all n indices lie in [0, N), else 1 with the error
// set.  Synchronises the stream.
int validate_indices(const int *idx, int64_t n, int N, const char *who, hipStream_t s) {
    int *flag = nullptr;
    TSNE_TRY(hipMalloc(&flag, sizeof(int)));
    int host = 0;
    hipError_t e = hipMemsetAsync(flag, 0, sizeof(int), s);
    if (e == hipSuccess) {
        index_range_kernel<<<(int)std::min<int64_t>(div_up(n, 256 * 8), 2048), 256, 0, s>>>(idx, n, N, flag);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(&host, flag, sizeof(int), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(flag);
    TSNE_TRY(e);
    if (host) {
        set_error("%s: a neighbour index lies outside [0, %d)", who, N);
        return 1;
    }
    return 0;
}

int launch_symmetrize(const float *p, const int *idx, int N, int K, float *P, hipStream_t s) {
    if (K <= 16) {
        symmetrize_kernel<16><<<div_up(N, 256 / 16), 256, 0, s>>>(p, idx, N, K, P);
    } else if (K <= 96) {
        symmetrize_kernel<32><<<div_up(N, 256 / 32), 256, 0, s>>>(p, idx, N, K, P);
    } else {
        symmetrize_kernel<64><<<div_up(N, 256 / 64), 256, 0, s>>>(p, idx, N, K, P);
    }
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
