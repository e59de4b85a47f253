// Attractive forces over the fixed N x K neighbour pattern for gfx950.
//
//   attr_i = sum_s P[i,s] * (y_i - y_j) / (1 + |y_i - y_j|^2),   j = idx[i,s]
//
// Semantics: src/kernels/attr_forces.cu:129-184 of the reference, which writes
// 2*nnz products to a workspace and reduces them in a second kernel.  Here a
// group of lanes owns a row: P and idx stream in coalesced, neighbour positions
// are gathered as interleaved (x, y) pairs with one 8-byte load, and the row
// sum is a lane reduction, so the only HBM traffic is the 8 bytes per non-zero
// plus the positions.
#include <algorithm>

#include "plan.h"

namespace tsnehip {

namespace {

// A group of LANES lanes owns ROWS consecutive rows and covers each with SLOTS
// strided slots (LANES * SLOTS >= K).  All index and probability loads of the
// ROWS rows are issued before the first gather, and all gathers before the
// arithmetic, so a wave keeps ROWS * SLOTS independent loads per lane in flight
// instead of living for two short dependent round trips.
template <int LANES, int SLOTS, int ROWS>
__global__ __launch_bounds__(256) void attractive_kernel(const float *__restrict__ pij, const int *__restrict__ idx,
                                                         const float2 *__restrict__ yxy, float *__restrict__ attr,
                                                         int N, int K) {
    constexpr int kGroups = 256 / LANES;
    const int lane = threadIdx.x % LANES;
    const int row0 = (blockIdx.x * kGroups + threadIdx.x / LANES) * ROWS;
    int j[ROWS][SLOTS];
    float pv[ROWS][SLOTS];
    float2 yi[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int row = row0 + r;
        const bool live = row < N;
        const size_t base = (size_t)(live ? row : 0) * K;
        yi[r] = yxy[live ? row : 0];
#pragma unroll
        for (int t = 0; t < SLOTS; ++t) {
            const int s = lane + t * LANES;
            const bool ok = live && s < K;
            j[r][t] = ok ? idx[base + s] : 0;
            pv[r][t] = ok ? pij[base + s] : 0.0f;  // zero weight for padding slots
        }
    }
    float2 yj[ROWS][SLOTS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int t = 0; t < SLOTS; ++t) yj[r][t] = yxy[j[r][t]];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        float ax = 0.0f, ay = 0.0f;
#pragma unroll
        for (int t = 0; t < SLOTS; ++t) {
            const float dx = yi[r].x - yj[r][t].x;
            const float dy = yi[r].y - yj[r][t].y;
            const float w = pv[r][t] * __builtin_amdgcn_rcpf(1.0f + dx * dx + dy * dy);
            ax += w * dx;
            ay += w * dy;
        }
        ax = group_sum<LANES>(ax);
        ay = group_sum<LANES>(ay);
        const int row = row0 + r;
        if (lane == 0 && row < N) {
            attr[row] = ax;
            attr[N + row] = ay;
        }
    }
}

// Any K: LANES lanes per row, strided loop.
template <int LANES>
__global__ __launch_bounds__(256) void attractive_generic_kernel(const float *__restrict__ pij,
                                                                 const int *__restrict__ idx,
                                                                 const float2 *__restrict__ yxy,
                                                                 float *__restrict__ attr, int N, int K) {
    constexpr int kRowsPerBlock = 256 / LANES;
    const int row = blockIdx.x * kRowsPerBlock + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    float ax = 0.0f, ay = 0.0f;
    if (row < N) {
        const float2 yi = yxy[row];
        const size_t base = (size_t)row * K;
#pragma unroll 4
        for (int s = lane; s < K; s += LANES) {
            const int jj = idx[base + s];
            const float pv = pij[base + s];
            const float2 yj = yxy[jj];
            const float dx = yi.x - yj.x;
            const float dy = yi.y - yj.y;
            const float w = pv * __builtin_amdgcn_rcpf(1.0f + dx * dx + dy * dy);
            ax += w * dx;
            ay += w * dy;
        }
    }
    ax = group_sum<LANES>(ax);
    ay = group_sum<LANES>(ay);
    if (lane == 0 && row < N) {
        attr[row] = ax;
        attr[N + row] = ay;
    }
}

__global__ __launch_bounds__(256) void pack_xy_kernel(const float *__restrict__ emb, int N,
                                                      float2 *__restrict__ yxy) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < N) yxy[i] = make_float2(emb[i], emb[N + i]);
}

}  // namespace

int launch_pack_xy(tsne_hip_plan *p, const float *embedding, hipStream_t s) {
    pack_xy_kernel<<<div_up(p->num_points, 256), 256, 0, s>>>(embedding, p->num_points, p->yxy);
    TSNE_LAUNCHED(s);
    return 0;
}

// Expects plan->yxy to hold the current embedding as (x, y) pairs.
int launch_attractive(tsne_hip_plan *p, const float *pij, const int *indices, float *attr, hipStream_t s) {
    const int N = p->num_points, K = p->num_neighbors;
    if (profile_mark(p, kKernelAttractive, s)) return 1;
#define TSNE_ATTR(LANES, SLOTS, ROWS)                                                              \
    TSNE_LOOP_KERNEL(p, (attractive_kernel<LANES, SLOTS, ROWS>), div_up(N, (256 / LANES) * ROWS), 256, 0, s, pij,  \
                     indices, p->yxy, attr, N, K)
    if (K <= 16) {
        TSNE_ATTR(16, 1, 8);
    } else if (K <= 32) {
        TSNE_ATTR(16, 2, 4);
    } else if (K <= 64) {
        TSNE_ATTR(32, 2, 4);
    } else if (K <= 96) {
        TSNE_ATTR(32, 3, 4);
    } else if (K <= 128) {
        TSNE_ATTR(64, 2, 4);
    } else if (K <= 256) {
        TSNE_ATTR(64, 4, 2);
    } else {
        TSNE_LOOP_KERNEL(p, (attractive_generic_kernel<64>), div_up(N, 256 / 64), 256, 0, s, pij, indices, p->yxy, attr, N, K);
    }
#undef TSNE_ATTR
    TSNE_LAUNCHED(s);
    return 0;
}


namespace {

// sum over the pattern of P ln(P (1 + d^2)); the ln Z term is added by the caller (sum P is the
// second output).  Double accumulation, one pair of atomics per workgroup.
__global__ __launch_bounds__(256) void kl_terms_kernel(const float *__restrict__ pij, const int *__restrict__ idx,
                                                       const float *__restrict__ emb, int N, int K,
                                                       double *__restrict__ out) {
    double kl = 0.0, mass = 0.0;
    const int64_t nnz = (int64_t)N * K;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x) {
        const float p = pij[e];
        if (p > 0.0f) {
            const int i = (int)(e / K), j = idx[e];
            const float dx = emb[i] - emb[j], dy = emb[N + i] - emb[N + j];
            kl += (double)p * (log((double)p) + log1p((double)dx * dx + (double)dy * dy));
            mass += (double)p;
        }
    }
    __shared__ double red[2][256 / kWave];
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        kl += __shfl_xor(kl, m, kWave);
        mass += __shfl_xor(mass, m, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        red[0][threadIdx.x / kWave] = kl;
        red[1][threadIdx.x / kWave] = mass;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < 256 / kWave; ++k) {
            kl += red[0][k];
            mass += red[1][k];
        }
        atomicAdd(&out[0], kl);
        atomicAdd(&out[1], mass);
    }
}

__global__ void clear_pair_kernel(double *out) {
    if (threadIdx.x < 2 && blockIdx.x == 0) out[threadIdx.x] = 0.0;
}

}  // namespace

// out[0] = sum P ln(P (1 + d^2)), out[1] = sum P over the pattern (device doubles).
int launch_kl_terms(const float *pij, const int *indices, const float *embedding, int N, int K, double *out,
                    hipStream_t s) {
    clear_pair_kernel<<<1, 64, 0, s>>>(out);
    TSNE_LAUNCHED(s);
    const int blocks = (int)std::min<int64_t>(div_up((int64_t)N * K, 256 * 8), 2048);
    kl_terms_kernel<<<std::max(blocks, 1), 256, 0, s>>>(pij, indices, embedding, N, K, out);
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
