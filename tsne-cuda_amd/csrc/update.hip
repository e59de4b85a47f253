// Gains / momentum update of the embedding for gfx950.
//
// Semantics: src/kernels/apply_forces.cu:11-57 of the reference (no factor 4,
// no re-centring, sign test through signbit, gain constants in double).  In the
// fused loop the same pass also refreshes the interleaved (x, y) copy used by
// the neighbour gathers and accumulates the bounds of the new embedding, which
// replaces the reference's per-step host-synchronising minmax_element
// (src/fit_tsne.cu:430-432).
#include "plan.h"

#include <algorithm>
#include <cstdint>

namespace tsnehip {

namespace {

// A workgroup's smallest and largest coordinate into the bounds of `slot`.  Hundreds of workgroups end
// here and atomics on one address are performed one after the other, so a workgroup first looks
// (a device-scope load, performed where the atomics are) whether its value would change anything:
// min and max only move one way, a stale look can only cause a superfluous atomic.
__device__ __forceinline__ void publish_bounds(LoopScalars *sc, int slot, float lo, float hi) {
    const unsigned int lo_enc = float_to_ordered(lo), hi_enc = float_to_ordered(hi);
    if (lo_enc < __hip_atomic_load(&sc->min_enc[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        atomicMin(&sc->min_enc[slot], lo_enc);
    if (hi_enc > __hip_atomic_load(&sc->max_enc[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        atomicMax(&sc->max_enc[slot], hi_enc);
}

__device__ __forceinline__ float step_coordinate(float &gain, float &u, float attr, float rep, float exaggeration,
                                                 float normalization, float momentum, float eta) {
#pragma clang fp contract(off)
    const float d = exaggeration * attr - (rep / normalization);
    float g = gain;
    g = (signbit(d) != signbit(u)) ? (float)((double)g + 0.2) : (float)((double)g * 0.8);
    g = ((double)g < 0.01) ? (float)0.01 : g;
    u = momentum * u - eta * g * d;
    gain = g;
    return u;
}

// Re-centring (optional, no counterpart in the reference, whose loop never re-centres:
// src/kernels/apply_forces.cu:11-57): the update subtracts from every new position the centre of the embedding
// as it stood before the step (its coordinate sums were left by the update before, or by centre_sums_kernel at
// the start of a loop) and leaves the sums of what it writes.  All forces are translation invariant, so the
// trajectory is that of exact re-centring after every step, one step late.  Without the option the centre reads
// as (+0, +0) and x - 0 is x, bit for bit.
// Every workgroup leaves its own pair of sums; the reader adds the pairs in the order of the workgroups, so the
// centre does not depend on the order in which they finished.
struct Centre {
    float x, y;
};
template <bool FUSED>
__device__ __forceinline__ Centre load_centre(const LoopScalars *sc, const double2 *parts, int next_slot, int N,
                                              int recenter) {
    Centre c{0.0f, 0.0f};
    if (FUSED && recenter) {
        __shared__ double2 tree[256];
        const int slot = next_slot ^ 1;
        const int count = sc->center_count[slot];
        double2 acc = make_double2(0.0, 0.0);
        for (int k = threadIdx.x; k < count; k += 256) {
            const double2 v = parts[(size_t)slot * kMaxCentreParts + k];
            acc.x += v.x;
            acc.y += v.y;
        }
        tree[threadIdx.x] = acc;
        __syncthreads();
        for (int half = 128; half >= 1; half >>= 1) {
            if ((int)threadIdx.x < half) {
                tree[threadIdx.x].x += tree[threadIdx.x + half].x;
                tree[threadIdx.x].y += tree[threadIdx.x + half].y;
            }
            __syncthreads();
        }
        c.x = (float)(tree[0].x / (double)N);
        c.y = (float)(tree[0].y / (double)N);
    }
    return c;
}
// A workgroup's sums of the x and y coordinates it wrote, into its place among the next slot's parts
// (256 threads; every thread of the workgroup calls this).
__device__ __forceinline__ void publish_centre(LoopScalars *sc, double2 *parts, int next_slot, float sx, float sy) {
    __shared__ double2 wave_sum[256 / kWave];
    double dx = (double)sx, dy = (double)sy;
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        dx += __shfl_xor(dx, m, kWave);
        dy += __shfl_xor(dy, m, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) wave_sum[threadIdx.x / kWave] = make_double2(dx, dy);
    __syncthreads();
    if (threadIdx.x == 0) {
        double2 t = wave_sum[0];
        for (int k = 1; k < 256 / kWave; ++k) {
            t.x += wave_sum[k].x;
            t.y += wave_sum[k].y;
        }
        parts[(size_t)next_slot * kMaxCentreParts + blockIdx.x] = t;
        if (blockIdx.x == 0) sc->center_count[next_slot] = (int)gridDim.x;
    }
}

__global__ __launch_bounds__(256) void centre_sums_kernel(const float *__restrict__ emb, int N, LoopScalars *sc,
                                                          double2 *parts, int slot) {
    float sx = 0.0f, sy = 0.0f;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < N; i += gridDim.x * blockDim.x) {
        sx += emb[i];
        sy += emb[N + i];
    }
    publish_centre(sc, parts, slot, sx, sy);
}

// Z of the step: the caller's scalar, or (z_ptr null) the loop's own - the fixed-point partial sums of z_i,
// an integer sum, less N (src/kernels/rep_forces.cu:54).
__device__ __forceinline__ float load_normalization(const float *z_ptr, const LoopScalars *sc, double z_inv_scale,
                                                    int N) {
    if (z_ptr) return *z_ptr;
    long long z = 0ll;
    for (int k = 0; k < kZParts; ++k) z += sc->z_part[k];
    return (float)((double)z * z_inv_scale) - (float)N;
}

template <bool FUSED>
__global__ __launch_bounds__(256) void update_kernel(float *__restrict__ emb, float *__restrict__ attr,
                                                     float *__restrict__ rep, float *__restrict__ gains,
                                                     float *__restrict__ old, int N, float eta,
                                                     const float *__restrict__ z_ptr, double z_inv_scale,
                                                     float momentum,
                                                     float exaggeration, float2 *__restrict__ yxy, LoopScalars *sc,
                                                     double2 *centre_parts, int next_slot, int recenter) {
    const float normalization = load_normalization(z_ptr, sc, z_inv_scale, N);
    float lo = INFINITY, hi = -INFINITY;
    const Centre c = load_centre<FUSED>(sc, centre_parts, next_slot, N, recenter);
    float sx = 0.0f, sy = 0.0f;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < N; i += gridDim.x * blockDim.x) {
        float gx = gains[i], gy = gains[N + i];
        float ux = old[i], uy = old[N + i];
        step_coordinate(gx, ux, attr[i], rep[i], exaggeration, normalization, momentum, eta);
        step_coordinate(gy, uy, attr[N + i], rep[N + i], exaggeration, normalization, momentum, eta);
        const float x = (emb[i] + ux) - c.x;
        const float y = (emb[N + i] + uy) - c.y;
        sx += x;
        sy += y;
        emb[i] = x;
        emb[N + i] = y;
        attr[i] = 0.0f;
        attr[N + i] = 0.0f;
        rep[i] = 0.0f;
        rep[N + i] = 0.0f;
        old[i] = ux;
        old[N + i] = uy;
        gains[i] = gx;
        gains[N + i] = gy;
        if (FUSED) {
            yxy[i] = make_float2(x, y);
            lo = fminf(lo, fminf(x, y));
            hi = fmaxf(hi, fmaxf(x, y));
        }
    }
    if (FUSED) {
        // One pair of atomics per workgroup: same-address atomics serialise.
        __shared__ float wlo[256 / kWave], whi[256 / kWave];
        lo = group_min<kWave>(lo);
        hi = group_max<kWave>(hi);
        if ((threadIdx.x & (kWave - 1)) == 0) {
            wlo[threadIdx.x / kWave] = lo;
            whi[threadIdx.x / kWave] = hi;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int k = 1; k < 256 / kWave; ++k) {
                lo = fminf(lo, wlo[k]);
                hi = fmaxf(hi, whi[k]);
            }
            publish_bounds(sc, next_slot, lo, hi);
        }
        if (recenter) publish_centre(sc, centre_parts, next_slot, sx, sy);
    }
}

// Four consecutive points per thread, 16-byte accesses.  Requires N % 4 == 0 and 16-byte aligned
// arrays (then the y halves at offset N are aligned too).
template <bool FUSED>
__global__ __launch_bounds__(256) void update_vec4_kernel(float *__restrict__ emb, float *__restrict__ attr,
                                                          float *__restrict__ rep, float *__restrict__ gains,
                                                          float *__restrict__ old, int N, float eta,
                                                          const float *__restrict__ z_ptr, double z_inv_scale,
                                                          float momentum, float exaggeration,
                                                          float2 *__restrict__ yxy, LoopScalars *sc,
                                                          double2 *centre_parts, int next_slot, int recenter) {
    const float normalization = load_normalization(z_ptr, sc, z_inv_scale, N);
    float lo = INFINITY, hi = -INFINITY;
    const Centre c = load_centre<FUSED>(sc, centre_parts, next_slot, N, recenter);
    float sx = 0.0f, sy = 0.0f;
    const int n4 = N / 4;
    float4 *emb4 = reinterpret_cast<float4 *>(emb), *attr4 = reinterpret_cast<float4 *>(attr);
    float4 *rep4 = reinterpret_cast<float4 *>(rep), *gains4 = reinterpret_cast<float4 *>(gains);
    float4 *old4 = reinterpret_cast<float4 *>(old);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += gridDim.x * blockDim.x) {
        const float4 ex = emb4[i], ey = emb4[n4 + i];
        const float4 ax = attr4[i], ay = attr4[n4 + i];
        const float4 rx = rep4[i], ry = rep4[n4 + i];
        float4 gx = gains4[i], gy = gains4[n4 + i];
        float4 ux = old4[i], uy = old4[n4 + i];
        step_coordinate(gx.x, ux.x, ax.x, rx.x, exaggeration, normalization, momentum, eta);
        step_coordinate(gx.y, ux.y, ax.y, rx.y, exaggeration, normalization, momentum, eta);
        step_coordinate(gx.z, ux.z, ax.z, rx.z, exaggeration, normalization, momentum, eta);
        step_coordinate(gx.w, ux.w, ax.w, rx.w, exaggeration, normalization, momentum, eta);
        step_coordinate(gy.x, uy.x, ay.x, ry.x, exaggeration, normalization, momentum, eta);
        step_coordinate(gy.y, uy.y, ay.y, ry.y, exaggeration, normalization, momentum, eta);
        step_coordinate(gy.z, uy.z, ay.z, ry.z, exaggeration, normalization, momentum, eta);
        step_coordinate(gy.w, uy.w, ay.w, ry.w, exaggeration, normalization, momentum, eta);
        const float4 nx = make_float4((ex.x + ux.x) - c.x, (ex.y + ux.y) - c.x, (ex.z + ux.z) - c.x, (ex.w + ux.w) - c.x);
        const float4 ny = make_float4((ey.x + uy.x) - c.y, (ey.y + uy.y) - c.y, (ey.z + uy.z) - c.y, (ey.w + uy.w) - c.y);
        sx += (nx.x + nx.y) + (nx.z + nx.w);
        sy += (ny.x + ny.y) + (ny.z + ny.w);
        emb4[i] = nx;
        emb4[n4 + i] = ny;
        // The reference clears the force arrays here (src/kernels/apply_forces.cu:48-51); the stage-level
        // call keeps that, the fused loop does not need it: both force kernels overwrite every element.
        if (!FUSED) {
            attr4[i] = zero;
            attr4[n4 + i] = zero;
            rep4[i] = zero;
            rep4[n4 + i] = zero;
        }
        old4[i] = ux;
        old4[n4 + i] = uy;
        gains4[i] = gx;
        gains4[n4 + i] = gy;
        if (FUSED) {
            float4 *y4 = reinterpret_cast<float4 *>(yxy) + 2 * (size_t)i;
            y4[0] = make_float4(nx.x, ny.x, nx.y, ny.y);
            y4[1] = make_float4(nx.z, ny.z, nx.w, ny.w);
            lo = fminf(lo, fminf(fminf(fminf(nx.x, nx.y), fminf(nx.z, nx.w)), fminf(fminf(ny.x, ny.y), fminf(ny.z, ny.w))));
            hi = fmaxf(hi, fmaxf(fmaxf(fmaxf(nx.x, nx.y), fmaxf(nx.z, nx.w)), fmaxf(fmaxf(ny.x, ny.y), fmaxf(ny.z, ny.w))));
        }
    }
    if (FUSED) {
        __shared__ float wlo[256 / kWave], whi[256 / kWave];
        lo = group_min<kWave>(lo);
        hi = group_max<kWave>(hi);
        if ((threadIdx.x & (kWave - 1)) == 0) {
            wlo[threadIdx.x / kWave] = lo;
            whi[threadIdx.x / kWave] = hi;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int k = 1; k < 256 / kWave; ++k) {
                lo = fminf(lo, wlo[k]);
                hi = fmaxf(hi, whi[k]);
            }
            publish_bounds(sc, next_slot, lo, hi);
        }
        if (recenter) publish_centre(sc, centre_parts, next_slot, sx, sy);
    }
}

__global__ void clear_scalar_kernel(float *p) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *p = 0.0f;
}

__global__ __launch_bounds__(256) void sum_squares_kernel(const float *__restrict__ v, int64_t n, float *out) {
    __shared__ float partial[256 / kWave];
    float acc = 0.0f;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x) {
        const float x = v[t];
        acc += x * x;
    }
    acc = group_sum<kWave>(acc);
    if ((threadIdx.x & (kWave - 1)) == 0) partial[threadIdx.x / kWave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.0f;
        for (int k = 0; k < 256 / kWave; ++k) t += partial[k];
        atomicAdd(out, t);
    }
}

}  // namespace

// normalization == nullptr: Z is taken from the loop scalars (sum of z_part - N).
// next_slot >= 0: also refresh the (x, y) copy and accumulate the new bounds.
int launch_update(tsne_hip_plan *p, float *embedding, float *attr, float *rep, float *gains, float *old_forces,
                  float eta, const float *normalization, float momentum, float exaggeration, int next_slot,
                  hipStream_t s) {
    const int N = p->num_points;
    const float *z_ptr = normalization;
    const double z_inv = 1.0 / p->z_scale;
    if (profile_mark(p, kKernelUpdate, s)) return 1;
    auto aligned16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (N % 4 == 0 && aligned16(embedding) && aligned16(attr) && aligned16(rep) && aligned16(gains) &&
        aligned16(old_forces)) {
        // Eighteen arrays are streamed at once; the fewer workgroups walk them with a grid stride, the narrower
        // the window of each array that is open at any time.  Measured at 1 M points: 256-384 workgroups 19 us,
        // 512 25 us, one item per thread (977 workgroups) 39 us.
        const int blocks = std::min(std::min(div_up(N / 4, 256), p->stream_grid), kMaxCentreParts);
        if (next_slot >= 0) {
            TSNE_LOOP_KERNEL(p, (update_vec4_kernel<true>), blocks, 256, 0, s, embedding, attr, rep, gains, old_forces, N, eta, z_ptr, z_inv,
                                                            momentum, exaggeration, p->yxy, p->scalars,
                                                            p->centre_parts, next_slot, p->recenter ? 1 : 0);
        } else {
            TSNE_LOOP_KERNEL(p, (update_vec4_kernel<false>), blocks, 256, 0, s, embedding, attr, rep, gains, old_forces, N, eta, z_ptr, z_inv,
                                                             momentum, exaggeration, nullptr, p->scalars, nullptr, 0, 0);
        }
        TSNE_LAUNCHED(s);
        return 0;
    }
    const int blocks = std::min(std::min(div_up(N, 256), 4 * p->stream_grid), kMaxCentreParts);  // 4-byte accesses: the same window
    if (next_slot >= 0) {
        TSNE_LOOP_KERNEL(p, (update_kernel<true>), blocks, 256, 0, s, embedding, attr, rep, gains, old_forces, N, eta, z_ptr, z_inv,
                                                   momentum, exaggeration, p->yxy, p->scalars, p->centre_parts, next_slot,
                                                   p->recenter ? 1 : 0);
    } else {
        TSNE_LOOP_KERNEL(p, (update_kernel<false>), blocks, 256, 0, s, embedding, attr, rep, gains, old_forces, N, eta, z_ptr, z_inv,
                                                    momentum, exaggeration, nullptr, p->scalars, nullptr, 0, 0);
    }
    TSNE_LAUNCHED(s);
    return 0;
}

// Coordinate sums of `embedding` into the centre sums of `slot` (start of a re-centred loop).
int launch_centre_sums(tsne_hip_plan *p, const float *embedding, int slot, hipStream_t s) {
    const int blocks = std::min(div_up(p->num_points, 256 * 4), 1024);
    centre_sums_kernel<<<std::max(blocks, 1), 256, 0, s>>>(embedding, p->num_points, p->scalars, p->centre_parts, slot);
    TSNE_LAUNCHED(s);
    return 0;
}

int launch_sum_squares(const float *values, int64_t n, float *out, hipStream_t s) {
    clear_scalar_kernel<<<1, 64, 0, s>>>(out);  // a kernel, not a memset node, so the call can be graph-captured
    TSNE_LAUNCHED(s);
    const int blocks = (int)std::min<int64_t>(div_up(n, 256 * 4), 2048);
    sum_squares_kernel<<<std::max(blocks, 1), 256, 0, s>>>(values, n, out);
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
