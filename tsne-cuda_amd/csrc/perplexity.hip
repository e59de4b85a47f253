// Max-normalisation and per-row perplexity search for gfx950.
//
// Semantics: src/util/math_utils.cu:66-74 and
// src/kernels/perplexity_search.cu:10-141 of the reference.  The reference
// iterates all rows in lock-step (<= 200 rounds of: exponentiate nnz values,
// two cuBLAS row reductions, an entropy transform, a per-row update kernel and
// a host-side "all found" reduction).  Rows never interact, so here a group of
// lanes owns a row, keeps its distances in registers and runs the whole
// bisection privately: the distances are read once and the probabilities
// written once.
//
// Reproducible arithmetic.  Whether a row stops at one bisection step or the
// next hangs on the last bits of its entropy, so every operation of the search
// is pinned down: exp and log are the fixed operation sequences of det_math.h,
// nothing is contracted, and the two row sums (of p and of p ln p) are formed in
// one stated order whatever the kernel variant:
//   * 64 interleaved partial sums, partial c taking the values of the slots
//     s = c, c + 64, c + 128, ... in ascending order, starting from +0;
//   * then a balanced tree: partial[c] + partial[c ^ m] for m = 32, 16, 8, 4, 2, 1.
// A CPU restatement that follows the same order gets the same probabilities bit
// for bit.  (The reference's sums are cuBLAS sgemv calls whose order is not
// documented, and its exp/log are the fast intrinsics.)
#include "det_math.h"
#include "plan.h"

#include <algorithm>
#include <cfloat>
#include <mutex>

#include "../../include/tsnecuda/tsne_stages.h"

// Scratch of tsne_hip_max_normalize_noalloc: the device scalar that receives the largest absolute value.
// Every GPU holds its own copy of this array at its own address until the process ends; in host code the
// name is only a handle for hipGetSymbolAddress, never a device address.
static __device__ __align__(256) float scratch[64];

namespace tsnehip {

namespace {

__global__ __launch_bounds__(256) void abs_max_kernel(const float *__restrict__ v, int64_t n, float *out) {
    float m = 0.0f;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x)
        m = fmaxf(m, fabsf(v[t]));
    m = group_max<kWave>(m);
    // Non-negative floats order like their bit patterns.
    if ((threadIdx.x & (kWave - 1)) == 0) atomicMax(reinterpret_cast<unsigned int *>(out), __float_as_uint(m));
}

__global__ __launch_bounds__(256) void divide_kernel(float *__restrict__ v, int64_t n, const float *denom) {
    const float d = *denom;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x)
        v[t] = v[t] / d;
}

__global__ void zero_scalar_kernel(float *p) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *p = 0.0f;
}

// thrust_transform_functions.h:32-37: x*log(x) with NaN/Inf mapped to 0.
__device__ __forceinline__ float entropy_term(float v) {
#pragma clang fp contract(off)
    const float e = v * det_logf(v);
    return (e != e || isinf(e)) ? 0.0f : e;
}

// The stated summation order for a group of LANES lanes whose lane l holds the slots l + v * LANES: a lane
// owns 64 / LANES of the 64 partial sums (classes l + LANES * (v mod (64 / LANES))); it forms them one after
// the other, combines them by the upper levels of the tree, and the lower levels run across the lanes.
template <int LANES, int VPL>
__device__ __forceinline__ float ordered_row_sum(const float (&val)[VPL]) {
#pragma clang fp contract(off)
    constexpr int kClasses = kWave / LANES;
    float q[kClasses];
#pragma unroll
    for (int c = 0; c < kClasses; ++c) q[c] = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) q[v % kClasses] += val[v];
    // Class index c * LANES + lane: the tree's level m = 32 pairs classes c and c ^ (32 / LANES), and so on down.
#pragma unroll
    for (int m = kClasses / 2; m > 0; m >>= 1)
#pragma unroll
        for (int c = 0; c < m; ++c) q[c] += q[c + m];
    return group_sum<LANES>(q[0]);
}

// One row per LANES-lane group, VPL values per lane held in registers.
template <int LANES, int VPL>
__global__ __launch_bounds__(256) void perplexity_kernel(const float *__restrict__ sq_dist, int N, int K,
                                                         float log_target, float eps, float *__restrict__ pij,
                                                         float *__restrict__ betas) {
#pragma clang fp contract(off)
    constexpr int kRowsPerBlock = 256 / LANES;
    const int row = blockIdx.x * kRowsPerBlock + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    const bool live = row < N;
    const size_t base = (size_t)(live ? row : 0) * K;

    float d[VPL];
    bool self[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const int s = lane + v * LANES;
        d[v] = (live && s < K) ? sq_dist[base + s] : 0.0f;
        // perplexity_search.cu:32: neighbour 0 at distance 0 is the point itself.
        self[v] = (s == 0 && d[v] == 0.0f);
    }

    float beta = 1.0f, lo = -FLT_MAX, hi = FLT_MAX;
    float p[VPL];
    float sum = 1.0f;
    bool done = !live;
    for (int it = 0; it < 200; ++it) {
        if (!done) {
            float et[VPL];
#pragma unroll
            for (int v = 0; v < VPL; ++v) {
                const int s = lane + v * LANES;
                float pv = 0.0f;
                if (s < K && !self[v]) pv = det_expf(-beta * d[v]);
                p[v] = pv;
                et[v] = s < K ? entropy_term(pv) : 0.0f;
            }
            sum = ordered_row_sum<LANES, VPL>(p);
            const float ent = ordered_row_sum<LANES, VPL>(et);
            const float H = (-ent / sum) + det_logf(sum);
            const float diff = H - log_target;
            const bool found = (diff < eps && -diff < eps);
            if (found || it == 199) {
                done = true;
            } else if (diff > 0) {
                lo = beta;
                beta = (hi == FLT_MAX || hi == -FLT_MAX) ? beta * 2.0f : (beta + hi) / 2.0f;
            } else {
                hi = beta;
                beta = (lo == -FLT_MAX || lo == FLT_MAX) ? beta / 2.0f : (beta + lo) / 2.0f;
            }
        }
        if (__all(done)) break;
    }
    if (live) {
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            const int s = lane + v * LANES;
            if (s < K) pij[base + s] = p[v] / sum;
        }
        if (betas && lane == 0) betas[row] = beta;
    }
}

// Any K: one wave per row, distances re-read from memory every round.
__global__ __launch_bounds__(256) void perplexity_generic_kernel(const float *__restrict__ sq_dist, int N, int K,
                                                                 float log_target, float eps,
                                                                 float *__restrict__ pij,
                                                                 float *__restrict__ betas) {
#pragma clang fp contract(off)
    const int row = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    if (row >= N) return;
    const size_t base = (size_t)row * K;
    float beta = 1.0f, lo = -FLT_MAX, hi = FLT_MAX, sum = 1.0f;
    for (int it = 0; it < 200; ++it) {
        float ls = 0.0f, le = 0.0f;
        for (int s = lane; s < K; s += kWave) {
            const float dv = sq_dist[base + s];
            const float pv = (s == 0 && dv == 0.0f) ? 0.0f : det_expf(-beta * dv);
            ls += pv;
            le += entropy_term(pv);
        }
        sum = group_sum<kWave>(ls);
        const float ent = group_sum<kWave>(le);
        const float H = (-ent / sum) + det_logf(sum);
        const float diff = H - log_target;
        const bool found = (diff < eps && -diff < eps);
        if (found || it == 199) break;
        if (diff > 0) {
            lo = beta;
            beta = (hi == FLT_MAX || hi == -FLT_MAX) ? beta * 2.0f : (beta + hi) / 2.0f;
        } else {
            hi = beta;
            beta = (lo == -FLT_MAX || lo == FLT_MAX) ? beta / 2.0f : (beta + lo) / 2.0f;
        }
    }
    for (int s = lane; s < K; s += kWave) {
        const float dv = sq_dist[base + s];
        const float pv = (s == 0 && dv == 0.0f) ? 0.0f : det_expf(-beta * dv);
        pij[base + s] = pv / sum;
    }
    if (betas && lane == 0) betas[row] = beta;
}

}  // namespace

// scratch: one device float.
int launch_max_normalize(float *values, int64_t n, float *scratch, hipStream_t s) {
    zero_scalar_kernel<<<1, 64, 0, s>>>(scratch);
    TSNE_LAUNCHED(s);
    const int blocks = std::max(1, (int)std::min<int64_t>(div_up(n, 256 * 4), 4096));
    abs_max_kernel<<<blocks, 256, 0, s>>>(values, n, scratch);
    TSNE_LAUNCHED(s);
    divide_kernel<<<blocks, 256, 0, s>>>(values, n, scratch);
    TSNE_LAUNCHED(s);
    return 0;
}

namespace {
constexpr int kMaxDevices = 64;
constexpr int64_t kNoAllocMaxValues = (int64_t)1 << 32;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// The address of `scratch` on the current device, looked up once per device.
int noalloc_scratch(float **out) {
    int dev = -1;
    TSNE_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) {
        set_error("max_normalize_noalloc: device %d is outside the supported range [0, %d)", dev, kMaxDevices);
        return 1;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float *ptr = nullptr;
        TSNE_TRY(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) {
            set_error("max_normalize_noalloc: hipGetSymbolAddress returned a null address");
            return 1;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

int launch_perplexity(const float *sq_dist, int N, int K, float perplexity, float eps, float *pij, float *betas,
                      hipStream_t s) {
    const float log_target = det_logf(perplexity);
#define TSNE_PERP(LANES, VPL)                                                                                  \
    perplexity_kernel<LANES, VPL><<<div_up(N, 256 / LANES), 256, 0, s>>>(sq_dist, N, K, log_target, eps, pij, \
                                                                         betas)
    if (K <= 32) {
        TSNE_PERP(16, 2);
    } else if (K <= 64) {
        TSNE_PERP(32, 2);
    } else if (K <= 96) {
        TSNE_PERP(32, 3);
    } else if (K <= 128) {
        TSNE_PERP(64, 2);
    } else if (K <= 256) {
        TSNE_PERP(64, 4);
    } else if (K <= 512) {
        TSNE_PERP(64, 8);
    } else if (K <= 1024) {
        TSNE_PERP(64, 16);
    } else {
        perplexity_generic_kernel<<<div_up(N, 256 / kWave), 256, 0, s>>>(sq_dist, N, K, log_target, eps, pij, betas);
    }
#undef TSNE_PERP
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip

extern "C" int tsne_hip_max_normalize_noalloc(float *values, int64_t n, void *stream) {
    using namespace tsnehip;
    if (!values || n <= 0) {
        set_error("max_normalize_noalloc: need a non-empty array");
        return 1;
    }
    if (n > kNoAllocMaxValues) {
        set_error("max_normalize_noalloc: %lld values exceed the supported maximum of %lld", (long long)n,
                  (long long)kNoAllocMaxValues);
        return 1;
    }
    float *ptr = nullptr;
    if (noalloc_scratch(&ptr)) return 1;
    // launch_max_normalize clears the scalar with a kernel (no memset node, so the call may be captured).
    return launch_max_normalize(values, n, ptr, (hipStream_t)stream);
}
