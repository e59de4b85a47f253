// Quality measures of a fit (gfx950): trustworthiness of an embedding and the error of the
// interpolated repulsive forces against exact sums.  Neither has a counterpart in the reference, which
// reports no quality measure at all (its FunctionalKlDivergence, thrust_transform_functions.h:26-31, has no
// call site); both are evaluated on a sample of the points, so that they stay cheap at any size.
#include <algorithm>
#include <cmath>
#include <vector>

#include "../../include/tsnecuda/tsne_stages.h"
#include "plan.h"
#include "stages.h"

namespace tsnehip {

// `count` distinct pseudo-random indices below n, ascending: a full-period linear congruential sequence modulo
// the next power of two, values >= n skipped (a permutation of [0, 2^b), so no index repeats).
std::vector<int> sample_indices(int n, int count, unsigned int seed) {
    std::vector<int> out;
    if (count >= n) {
        out.resize(n);
        for (int i = 0; i < n; ++i) out[i] = i;
        return out;
    }
    unsigned int bits = 1;
    while ((1ull << bits) < (unsigned long long)n) ++bits;
    const unsigned long long mask = (1ull << bits) - 1ull;
    unsigned long long x = (unsigned long long)seed & mask;
    out.reserve(count);
    while ((int)out.size() < count) {
        x = (x * 1664525ull + 1013904223ull) & mask;
        if (x < (unsigned long long)n) out.push_back((int)x);
    }
    std::sort(out.begin(), out.end());
    return out;
}

namespace {

struct DeviceArray {
    void *ptr = nullptr;
    ~DeviceArray() {
        if (ptr) (void)hipFree(ptr);
    }
    bool alloc(size_t bytes) { return hipMalloc(&ptr, bytes ? bytes : 1) == hipSuccess; }
    template <typename T>
    T *as() const {
        return static_cast<T *>(ptr);
    }
};

constexpr int kTrustThreads = 256;
constexpr int kTrustMaxSample = 8192;  // two 8-byte arrays of that many entries in LDS

// Block-wide reductions over kTrustThreads threads (red: kTrustThreads / kWave slots of LDS).
__device__ __forceinline__ unsigned long long block_min_key(unsigned long long v, unsigned long long *red) {
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        const unsigned long long o = __shfl_xor(v, m, kWave);
        v = o < v ? o : v;
    }
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    unsigned long long r = red[0];
#pragma unroll
    for (int k = 1; k < kTrustThreads / kWave; ++k) r = red[k] < r ? red[k] : r;
    return r;
}
__device__ __forceinline__ int block_sum_int(int v, int *red) {
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    int r = 0;
#pragma unroll
    for (int k = 0; k < kTrustThreads / kWave; ++k) r += red[k];
    return r;
}

// Non-negative doubles order like their bit patterns; ties go to the lower index.
__device__ __forceinline__ bool key_less(unsigned long long da, int ja, unsigned long long db, int jb) {
    return da < db || (da == db && ja < jb);
}

// One workgroup per sampled point i.  xt: the sample's points, dimension-major (D x M); emb: the sample's
// embedding, M xs then M ys.  For each of the n_neighbors nearest points of i in the embedding (by
// (distance, index), i excluded) the rank of that point among i's input-space neighbours (1 = nearest) minus
// n_neighbors, where positive, goes into *penalty: the sum in the definition of trustworthiness
// (Venna & Kaski; scikit-learn's sklearn.manifold.trustworthiness computes the same sum).  Squared distances
// are taken in double on the float coordinates (differences and their squares are then exact, the sums rounded
// at 1e-16), so that which point is the n-th neighbour does not hang on fp32 rounding: one point more or less
// among the nearest moves the sum by its whole rank.
__global__ __launch_bounds__(kTrustThreads) void trustworthiness_kernel(const float *__restrict__ xt,
                                                                        const float *__restrict__ emb, int M, int D,
                                                                        int n_neighbors,
                                                                        unsigned long long *__restrict__ penalty) {
#pragma clang fp contract(off)
    extern __shared__ unsigned long long lds[];
    unsigned long long *d_in = lds, *d_emb = lds + M;  // bit patterns of the squared distances
    __shared__ unsigned long long red_key[kTrustThreads / kWave];
    __shared__ int red_int[kTrustThreads / kWave];
    const int i = blockIdx.x;
    const double ex = emb[i], ey = emb[M + i];
    for (int j = threadIdx.x; j < M; j += kTrustThreads) {
        double acc = 0.0;
        for (int d = 0; d < D; ++d) {
            const double df = (double)xt[(size_t)d * M + i] - (double)xt[(size_t)d * M + j];
            acc += df * df;
        }
        d_in[j] = (unsigned long long)__double_as_longlong(acc);
        const double dx = ex - (double)emb[j], dy = ey - (double)emb[M + j];
        d_emb[j] = (unsigned long long)__double_as_longlong(dx * dx + dy * dy);
    }
    __syncthreads();
    unsigned long long last_d = 0ull;
    int last_j = -1;  // nothing taken yet: every (distance, index) lies above (0, -1)
    unsigned long long total = 0ull;
    for (int round = 0; round < n_neighbors; ++round) {
        // the smallest embedding (distance, index) above the one taken last: the distance, then the index
        unsigned long long best = ~0ull;
        for (int j = threadIdx.x; j < M; j += kTrustThreads)
            if (j != i && key_less(last_d, last_j, d_emb[j], j) && d_emb[j] < best) best = d_emb[j];
        best = block_min_key(best, red_key);
        if (best == ~0ull) break;
        unsigned long long best_j = ~0ull;
        for (int j = threadIdx.x; j < M; j += kTrustThreads)
            if (j != i && d_emb[j] == best && key_less(last_d, last_j, best, j) && (unsigned long long)j < best_j)
                best_j = (unsigned long long)j;
        const int j = (int)block_min_key(best_j, red_key);
        last_d = best;
        last_j = j;
        const unsigned long long in_d = d_in[j];
        int closer = 0;
        for (int l = threadIdx.x; l < M; l += kTrustThreads)
            if (l != i && key_less(d_in[l], l, in_d, j)) closer += 1;
        const int rank = block_sum_int(closer, red_int) + 1;
        if (rank > n_neighbors) total += (unsigned long long)(rank - n_neighbors);
    }
    if (threadIdx.x == 0 && total) atomicAdd(penalty, total);
}

// Exact repulsive force and normalisation term of sampled points: for point i = sample[b],
//   F_i = sum_j (y_i - y_j) / (1 + |y_i - y_j|^2)^2,   z_i = sum_{j != i} 1 / (1 + |y_i - y_j|^2)
// (what the interpolation scheme approximates: src/kernels/rep_forces.cu:18-31 on the potentials of
// src/kernels/nbodyfft.cu), accumulated in double.  out: 3 doubles per sampled point (Fx, Fy, z).
__global__ __launch_bounds__(256) void exact_repulsive_kernel(const float *__restrict__ emb, int N,
                                                              const int *__restrict__ sample,
                                                              double *__restrict__ out) {
    __shared__ double red[3][256 / kWave];
    const int i = sample[blockIdx.x];
    const double xi = emb[i], yi = emb[N + i];
    double fx = 0.0, fy = 0.0, z = 0.0;
    for (int j = threadIdx.x; j < N; j += 256) {
        const double dx = xi - (double)emb[j], dy = yi - (double)emb[N + j];
        const double q = 1.0 / (1.0 + dx * dx + dy * dy);
        if (j != i) z += q;
        fx += dx * q * q;
        fy += dy * q * q;
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        fx += __shfl_xor(fx, m, kWave);
        fy += __shfl_xor(fy, m, kWave);
        z += __shfl_xor(z, m, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        red[0][threadIdx.x / kWave] = fx;
        red[1][threadIdx.x / kWave] = fy;
        red[2][threadIdx.x / kWave] = z;
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        double t = 0.0;
        for (int k = 0; k < 256 / kWave; ++k) t += red[threadIdx.x][k];
        out[3 * (size_t)blockIdx.x + threadIdx.x] = t;
    }
}

}  // namespace

// Relative L2 error of the interpolated repulsive forces, and relative error of the interpolated
// normalisation terms, on `sample_count` sampled points of `embedding` (device, 2N floats).  result (host):
// {force error, normalisation error, points sampled}.  slot < 0: the bounds of the embedding are computed first
// (into slot 0); otherwise `slot` holds them already (inside a loop: the slot the next step will read - the
// evaluation then only overwrites scratch that step overwrites anyway).  Synchronises the stream.
int repulsive_error(tsne_hip_plan *p, const float *embedding, int slot, int sample_count, unsigned int seed,
                    double *result, hipStream_t s) {
    const int N = p->num_points;
    const std::vector<int> sample = sample_indices(N, std::max(1, sample_count), seed);
    const int m = (int)sample.size();
    DeviceArray d_rep, d_phi, d_z, d_sample, d_exact;
    if (!d_rep.alloc(sizeof(float) * 2 * (size_t)N) || !d_phi.alloc(sizeof(float) * 4 * (size_t)N) ||
        !d_z.alloc(sizeof(float)) || !d_sample.alloc(sizeof(int) * (size_t)m) ||
        !d_exact.alloc(sizeof(double) * 3 * (size_t)m)) {
        set_error("repulsive_error: out of device memory");
        return 1;
    }
    TSNE_TRY(hipMemcpyAsync(d_sample.ptr, sample.data(), sizeof(int) * (size_t)m, hipMemcpyHostToDevice, s));
    if (slot < 0) {
        slot = 0;
        if (launch_bounds(p, embedding, slot, s)) return 1;
    }
    if (launch_repulsive(p, embedding, slot, d_rep.as<float>(), d_phi.as<float>(), nullptr, s)) return 1;
    exact_repulsive_kernel<<<m, 256, 0, s>>>(embedding, N, d_sample.as<int>(), d_exact.as<double>());
    TSNE_LAUNCHED(s);
    std::vector<float> rep(2 * (size_t)N), phi(4 * (size_t)N), emb(2 * (size_t)N);
    std::vector<double> exact(3 * (size_t)m);
    TSNE_TRY(hipMemcpyAsync(rep.data(), d_rep.ptr, sizeof(float) * rep.size(), hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipMemcpyAsync(phi.data(), d_phi.ptr, sizeof(float) * phi.size(), hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipMemcpyAsync(emb.data(), embedding, sizeof(float) * emb.size(), hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipMemcpyAsync(exact.data(), d_exact.ptr, sizeof(double) * exact.size(), hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipStreamSynchronize(s));
    double num = 0.0, den = 0.0, z_interp = 0.0, z_exact = 0.0;
    for (int t = 0; t < m; ++t) {
        const int i = sample[t];
        const double ex = exact[3 * (size_t)t], ey = exact[3 * (size_t)t + 1];
        const double dx = (double)rep[i] - ex, dy = (double)rep[(size_t)N + i] - ey;
        num += dx * dx + dy * dy;
        den += ex * ex + ey * ey;
        const double x = emb[i], y = emb[(size_t)N + i];
        const float *f = &phi[4 * (size_t)i];
        // src/kernels/rep_forces.cu:18-22, minus the point's own term (1 at distance 0)
        z_interp += (1.0 + x * x + y * y) * f[0] - 2.0 * (x * f[1] + y * f[2]) + f[3] - 1.0;
        z_exact += exact[3 * (size_t)t + 2];
    }
    result[0] = den > 0.0 ? std::sqrt(num / den) : 0.0;
    result[1] = z_exact != 0.0 ? std::fabs(z_interp - z_exact) / std::fabs(z_exact) : 0.0;
    result[2] = (double)m;
    return 0;
}

}  // namespace tsnehip

using namespace tsnehip;

extern "C" int tsne_hip_repulsive_error(tsne_hip_plan *plan, const float *embedding, int sample_count,
                                        double *result, void *stream) {
    if (!plan || !embedding || !result) {
        set_error("repulsive_error: null argument");
        return 1;
    }
    int dev = -1;
    TSNE_TRY(hipGetDevice(&dev));
    if (dev != plan->device) {
        set_error("repulsive_error: plan belongs to device %d but device %d is current", plan->device, dev);
        return 1;
    }
    return repulsive_error(plan, embedding, -1, sample_count, 12345u, result, (hipStream_t)stream);
}

extern "C" int tsnecuda_trustworthiness(const float *points, const float *embedding, int num_points, int num_dims,
                                        int n_neighbors, int max_sample, int device, double *trustworthiness,
                                        int *sample_out) {
    if (!points || !embedding || !trustworthiness) {
        set_error("trustworthiness: null argument");
        return 1;
    }
    if (num_points < 2 || num_dims < 1) {
        set_error("trustworthiness: need at least two points of at least one dimension");
        return 1;
    }
    if (max_sample < 2 || max_sample > kTrustMaxSample) {
        set_error("trustworthiness: max_sample must be in [2, %d] (got %d)", kTrustMaxSample, max_sample);
        return 1;
    }
    const std::vector<int> sample = sample_indices(num_points, max_sample, 2024u);
    const int M = (int)sample.size();
    if (n_neighbors < 1 || 2 * n_neighbors >= M) {
        set_error("trustworthiness: n_neighbors must be in [1, %d) for %d sampled points (got %d)", M / 2, M,
                  n_neighbors);
        return 1;
    }
    TSNE_TRY(hipSetDevice(device));
    // The sample's points dimension-major, its embedding as xs then ys.
    std::vector<float> xt((size_t)num_dims * M), emb(2 * (size_t)M);
    for (int t = 0; t < M; ++t) {
        const float *row = points + (size_t)sample[t] * num_dims;
        for (int d = 0; d < num_dims; ++d) xt[(size_t)d * M + t] = row[d];
        emb[t] = embedding[sample[t]];
        emb[(size_t)M + t] = embedding[(size_t)num_points + sample[t]];
    }
    DeviceArray d_xt, d_emb, d_pen;
    if (!d_xt.alloc(sizeof(float) * xt.size()) || !d_emb.alloc(sizeof(float) * emb.size()) ||
        !d_pen.alloc(sizeof(unsigned long long))) {
        set_error("trustworthiness: out of device memory");
        return 1;
    }
    TSNE_TRY(hipMemcpy(d_xt.ptr, xt.data(), sizeof(float) * xt.size(), hipMemcpyHostToDevice));
    TSNE_TRY(hipMemcpy(d_emb.ptr, emb.data(), sizeof(float) * emb.size(), hipMemcpyHostToDevice));
    TSNE_TRY(hipMemset(d_pen.ptr, 0, sizeof(unsigned long long)));
    const size_t lds = sizeof(unsigned long long) * 2 * (size_t)M;
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(trustworthiness_kernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    trustworthiness_kernel<<<M, kTrustThreads, lds, nullptr>>>(d_xt.as<float>(), d_emb.as<float>(), M, num_dims,
                                                               n_neighbors, d_pen.as<unsigned long long>());
    TSNE_TRY(hipGetLastError());
    unsigned long long penalty = 0ull;
    TSNE_TRY(hipMemcpy(&penalty, d_pen.ptr, sizeof(penalty), hipMemcpyDeviceToHost));
    const double n = (double)M, k = (double)n_neighbors;
    *trustworthiness = 1.0 - (double)penalty * (2.0 / (n * k * (2.0 * n - 3.0 * k - 1.0)));
    if (sample_out)
        for (int t = 0; t < M; ++t) sample_out[t] = sample[t];
    return 0;
}
