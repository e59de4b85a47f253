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
#include "plan.h"

namespace tsnehip {

namespace {

template <int LANES>
__global__ __launch_bounds__(256) void attractive_kernel(const float *__restrict__ pij, const int *__restrict__ idx,
                                                         const float2 *__restrict__ yxy, float *__restrict__ attr,
                                                         int N, int K) {
    constexpr int kRowsPerBlock = 256 / LANES;
    const int row = blockIdx.x * kRowsPerBlock + threadIdx.x / LANES;
    const int lane = threadIdx.x % LANES;
    float ax = 0.0f, ay = 0.0f;
    if (row < N) {
        const float2 yi = yxy[row];
        const size_t base = (size_t)row * K;
#pragma unroll 4
        for (int s = lane; s < K; s += LANES) {
            const int j = idx[base + s];
            const float pv = pij[base + s];
            const float2 yj = yxy[j];
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
    if (K <= 16) {
        attractive_kernel<16><<<div_up(N, 256 / 16), 256, 0, s>>>(pij, indices, p->yxy, attr, N, K);
    } else if (K <= 96) {
        attractive_kernel<32><<<div_up(N, 256 / 32), 256, 0, s>>>(pij, indices, p->yxy, attr, N, K);
    } else {
        attractive_kernel<64><<<div_up(N, 256 / 64), 256, 0, s>>>(pij, indices, p->yxy, attr, N, K);
    }
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
