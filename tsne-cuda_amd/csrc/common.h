// Shared host/device helpers for the gfx950 kernels of libtsnecuda.
#ifndef TSNE_HIP_COMMON_H_
#define TSNE_HIP_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <cstdio>
#include <cstdlib>

namespace tsnehip {

// Error reporting: stage functions return non-zero and leave a message here.
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
const char *last_error();

// TSNE_SYNC_KERNELS=1 makes every launch synchronise, as the reference's
// TSNE_MAYBE_SYNC does (src/include/util/cuda_utils.h:46-70).
bool sync_kernels_enabled();

#define TSNE_TRY(expr)                                                                              \
    do {                                                                                            \
        hipError_t tsne_err_ = (expr);                                                              \
        if (tsne_err_ != hipSuccess) {                                                              \
            ::tsnehip::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(tsne_err_),      \
                                 __FILE__, __LINE__);                                               \
            return 1;                                                                               \
        }                                                                                           \
    } while (0)

// After a kernel launch: surface launch errors; optionally synchronise.
#define TSNE_LAUNCHED(stream)                                                                       \
    do {                                                                                            \
        TSNE_TRY(hipGetLastError());                                                                \
        if (::tsnehip::sync_kernels_enabled()) TSNE_TRY(hipStreamSynchronize(stream));              \
    } while (0)

// Return code of the launchers that have a fallback: the shape is beyond what this form of the kernel holds
// (as opposed to 1, a failure).
constexpr int kShapeNotSupported = 2;

inline int div_up(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

constexpr int kWave = 64;

// Host-side inverse of the order-preserving float -> uint32 map below.
inline float ordered_to_float_host(unsigned int u) {
    const unsigned int bits = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
    float f;
    std::memcpy(&f, &bits, sizeof(f));
    return f;
}

#ifdef __HIPCC__
// Order-preserving map between float and uint32 so min/max can use integer atomics.
__device__ __forceinline__ unsigned int float_to_ordered(float f) {
    const unsigned int u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ordered_to_float(unsigned int u) {
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int m = WIDTH / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_min(float v) {
#pragma unroll
    for (int m = WIDTH / 2; m > 0; m >>= 1) v = fminf(v, __shfl_xor(v, m, kWave));
    return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int m = WIDTH / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
    return v;
}
#endif  // __HIPCC__

// Per-iteration device scalars shared by the gradient-loop kernels.
// Two bound slots alternate between iterations: the update kernel of step s
// accumulates the bounds that step s+1 reads.
struct LoopScalars {
    unsigned int min_enc[2];  // ordered-uint encoding of the smallest coordinate
    unsigned int max_enc[2];  // ... and of the largest
    float sumsq;              // scratch for the gradient-norm reduction
    float vmax;               // largest probability of the re-blocked pattern (fixed-point scale)
    // sum_i z_i of the current step in kZParts partial sums (Z = their sum - N): a thousand workgroups each
    // end with one atomic add, and atomics on a single address are performed one after the other.  The sums are
    // 64-bit fixed point (the plan's z_scale), so that they do not depend on the order in which the workgroups
    // arrive.
    long long z_part[16];
    // Workgroups of the re-blocked attractive kernel in which a wave gave up waiting for an LDS counter (their
    // rows come out as NaN).  Never non-zero unless the kernel's roles lose step; the host checks it after a loop.
    unsigned int wait_timeouts;
    // The grouping of the points by spreading tile is kept over the steps for as long as few points have left
    // the neighbourhood of their tile: `strays` counts the points of the current step's spread that had (they are
    // spread with global atomics instead), `sort_age` the steps since the grouping was made, and `reuse_sort`,
    // set at the end of a step's chain, tells the next step's kernels to keep it.
    unsigned int strays;
    int sort_age;
    int reuse_sort;
    // Running totals since the plan was made: chain evaluations, those that grouped the points afresh, strays.
    unsigned int chain_runs, chain_sorts, strays_total;
    // Optional re-centring (off unless the plan asks for it): per bounds slot, how many workgroups left their
    // sums of the x and of the y coordinates of the embedding that slot's bounds describe (in the plan's
    // centre_parts; the reader adds them in a fixed order).
    int center_count[2];
};
constexpr int kZParts = 16;
constexpr int kMaxCentreParts = 2048;  // most workgroups of a kernel that leaves coordinate sums

}  // namespace tsnehip

#endif  // TSNE_HIP_COMMON_H_
