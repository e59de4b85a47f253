// Exact brute-force k nearest neighbours for gfx950.
//
// Stands in for the FAISS IVF-Flat search of the reference
// (src/util/distance_utils.cu:79-121), which is approximate; this one is exact
// and reproducible: the squared distance of a pair is accumulated in fp32 over
// ascending dimension with one fused multiply-add per dimension, neighbours are
// ordered by (distance, index), and the point itself is forced into slot 0 with
// distance exactly 0 (the perplexity search depends on that,
// src/kernels/perplexity_search.cu:30-32).
//
// Layout: the points are transposed once to [dim][point] so that a tile of
// candidates is a run of contiguous floats per dimension.  A workgroup owns 64
// queries and sweeps all candidates in tiles of 128; each thread keeps a 4 x 8
// block of running distances in registers.  Selection is a filter against the
// query's current k-th best (almost every candidate dies on one 64-bit
// compare); survivors are appended to a per-query list that is compacted with
// an LDS bitonic sort whenever a further tile might overflow it.
#include "common.h"

#include <algorithm>
#include <climits>

namespace tsnehip {

namespace {

constexpr int kQT = 64;   // queries per workgroup
constexpr int kCT = 128;  // candidates per tile
constexpr int kDC = 32;   // dimensions staged per chunk

typedef unsigned long long u64;

__device__ __forceinline__ u64 pack_key(float d, int j) {
    return ((u64)float_to_ordered(d) << 32) | (unsigned int)j;
}

__global__ __launch_bounds__(256) void transpose_points_kernel(const float *__restrict__ X, int N, int D, int Npad,
                                                               float *__restrict__ Xt) {
    __shared__ float tile[32][33];
    const int i0 = blockIdx.x * 32, d0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8) {
        const int i = i0 + r, d = d0 + tx;
        tile[r][tx] = (i < N && d < D) ? X[(size_t)i * D + d] : 0.0f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        const int d = d0 + r, i = i0 + tx;
        if (d < D && i < Npad) Xt[(size_t)d * Npad + i] = tile[tx][r];
    }
}

// Sorts sortbuf[0..cap) ascending (cap a power of two), all 256 threads.
__device__ __forceinline__ void bitonic_sort(u64 *sortbuf, int cap, int tid) {
    for (int k = 2; k <= cap; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int t = tid; t < cap / 2; t += 256) {
                const int lo = ((t & ~(j - 1)) << 1) | (t & (j - 1));
                const int hi = lo | j;
                const bool up = (lo & k) == 0;
                const u64 a = sortbuf[lo], b = sortbuf[hi];
                if ((a > b) == up) {
                    sortbuf[lo] = b;
                    sortbuf[hi] = a;
                }
            }
            __syncthreads();
        }
    }
}

// Keeps the `want` best entries of query slot qq and tightens its threshold.
__device__ __forceinline__ void compact_query(u64 *list, int cap, int want, int *cnt, u64 *thr, int qq,
                                              u64 *sortbuf, int tid) {
    const int n = cnt[qq];
    for (int e = tid; e < cap; e += 256) sortbuf[e] = e < n ? list[(size_t)qq * cap + e] : ~0ull;
    __syncthreads();
    bitonic_sort(sortbuf, cap, tid);
    const int keep = min(n, want);
    for (int e = tid; e < keep; e += 256) list[(size_t)qq * cap + e] = sortbuf[e];
    if (tid == 0) {
        cnt[qq] = keep;
        if (n >= want) thr[qq] = sortbuf[want - 1];
    }
    __syncthreads();
}

__global__ __launch_bounds__(256) void knn_sweep_kernel(const float *__restrict__ Xt, int N, int Npad, int D, int K,
                                                        int cap, u64 *__restrict__ lists, int num_qtiles,
                                                        int *__restrict__ out_idx, float *__restrict__ out_d) {
    __shared__ __attribute__((aligned(16))) float xq[kDC][kQT];
    __shared__ __attribute__((aligned(16))) float xc[kDC][kCT];
    __shared__ u64 thr[kQT];
    __shared__ int cnt[kQT];
    extern __shared__ u64 sortbuf[];

    const int tid = threadIdx.x;
    const int tq = tid >> 4, tc = tid & 15;
    const int want = K - 1;
    u64 *list = lists + (size_t)blockIdx.x * kQT * cap;

    for (int qt = blockIdx.x; qt < num_qtiles; qt += gridDim.x) {
        const int q0 = qt * kQT;
        if (tid < kQT) {
            thr[tid] = ~0ull;
            cnt[tid] = 0;
        }
        __syncthreads();
        for (int c0 = 0; c0 < N; c0 += kCT) {
            float acc[4][8];
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 8; ++b) acc[a][b] = 0.0f;
            for (int d0 = 0; d0 < D; d0 += kDC) {
                const int dn = min(kDC, D - d0);
                __syncthreads();
                for (int e = tid; e < dn * (kQT / 4); e += 256) {
                    const int dd = e / (kQT / 4), v = e % (kQT / 4);
                    *reinterpret_cast<float4 *>(&xq[dd][v * 4]) =
                        *reinterpret_cast<const float4 *>(Xt + (size_t)(d0 + dd) * Npad + q0 + v * 4);
                }
                for (int e = tid; e < dn * (kCT / 4); e += 256) {
                    const int dd = e / (kCT / 4), v = e % (kCT / 4);
                    *reinterpret_cast<float4 *>(&xc[dd][v * 4]) =
                        *reinterpret_cast<const float4 *>(Xt + (size_t)(d0 + dd) * Npad + c0 + v * 4);
                }
                __syncthreads();
                for (int dd = 0; dd < dn; ++dd) {
                    const float4 qv = *reinterpret_cast<const float4 *>(&xq[dd][tq * 4]);
                    const float4 ca = *reinterpret_cast<const float4 *>(&xc[dd][tc * 8]);
                    const float4 cb = *reinterpret_cast<const float4 *>(&xc[dd][tc * 8 + 4]);
                    const float qs[4] = {qv.x, qv.y, qv.z, qv.w};
                    const float cs[8] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
#pragma unroll
                    for (int a = 0; a < 4; ++a)
#pragma unroll
                        for (int b = 0; b < 8; ++b) {
                            const float df = qs[a] - cs[b];
                            acc[a][b] = fmaf(df, df, acc[a][b]);
                        }
                }
            }
            // Filter against the current k-th best of each query.
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int ql = tq * 4 + a;
                const int q = q0 + ql;
                const u64 limit = thr[ql];
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    const int j = c0 + tc * 8 + b;
                    const u64 key = pack_key(acc[a][b], j);
                    if (j < N && q < N && j != q && key < limit) {
                        const int slot = atomicAdd(&cnt[ql], 1);
                        list[(size_t)ql * cap + slot] = key;
                    }
                }
            }
            __syncthreads();
            const int crowded = (tid < kQT) && (cnt[tid] > cap - kCT);
            if (__syncthreads_or(crowded)) {
                for (int ql = 0; ql < kQT; ++ql)
                    if (cnt[ql] > cap - kCT) compact_query(list, cap, want, cnt, thr, ql, sortbuf, tid);
            }
        }
        // Final ordering and output: self first, then the K-1 best others.
        for (int ql = 0; ql < kQT; ++ql) {
            const int q = q0 + ql;
            if (q >= N) break;
            compact_query(list, cap, want, cnt, thr, ql, sortbuf, tid);
            for (int e = tid; e < K; e += 256) {
                int j = q;
                float d = 0.0f;
                if (e > 0) {
                    const u64 key = sortbuf[e - 1];
                    j = (int)(unsigned int)(key & 0xffffffffu);
                    d = ordered_to_float((unsigned int)(key >> 32));
                }
                out_idx[(size_t)q * K + e] = j;
                out_d[(size_t)q * K + e] = d;
            }
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(256) void knn_self_only_kernel(int N, int *__restrict__ out_idx,
                                                            float *__restrict__ out_d) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < N) {
        out_idx[i] = i;
        out_d[i] = 0.0f;
    }
}

}  // namespace

int run_knn(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s) {
    if (N <= 0 || D <= 0 || K <= 0) {
        set_error("knn: num_points, num_dims and num_neighbors must be positive (got %d, %d, %d)", N, D, K);
        return 1;
    }
    if (K > N) {
        set_error("knn: num_neighbors (%d) exceeds num_points (%d)", K, N);
        return 1;
    }
    if (K == 1) {
        knn_self_only_kernel<<<div_up(N, 256), 256, 0, s>>>(N, indices, sq_dist);
        TSNE_LAUNCHED(s);
        TSNE_TRY(hipStreamSynchronize(s));
        return 0;
    }
    int cap = 256;
    while (cap < K - 1 + kCT) cap <<= 1;
    if (cap > 4096) {
        set_error("knn: num_neighbors = %d is not supported (limit %d)", K, 4096 - kCT + 1);
        return 1;
    }
    const int Npad = div_up(N, kCT) * kCT;
    const int num_qtiles = div_up(N, kQT);
    int device = 0, cus = 256;
    TSNE_TRY(hipGetDevice(&device));
    TSNE_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    const int grid = std::min(num_qtiles, cus * 3);

    float *Xt = nullptr;
    u64 *lists = nullptr;
    TSNE_TRY(hipMalloc(&Xt, sizeof(float) * (size_t)D * Npad));
    if (hipMalloc(&lists, sizeof(u64) * (size_t)grid * kQT * cap) != hipSuccess) {
        (void)hipFree(Xt);
        set_error("knn: out of device memory for the candidate lists");
        return 1;
    }
    int rc = 0;
    do {
        dim3 tgrid(div_up(Npad, 32), div_up(D, 32));
        transpose_points_kernel<<<tgrid, 256, 0, s>>>(points, N, D, Npad, Xt);
        if (hipGetLastError() != hipSuccess) { rc = 1; break; }
        knn_sweep_kernel<<<grid, 256, sizeof(u64) * cap, s>>>(Xt, N, Npad, D, K, cap, lists, num_qtiles, indices,
                                                              sq_dist);
        if (hipGetLastError() != hipSuccess) { rc = 1; break; }
        if (hipStreamSynchronize(s) != hipSuccess) { rc = 1; break; }
    } while (0);
    if (rc) set_error("knn: kernel launch or execution failed: %s", hipGetErrorString(hipGetLastError()));
    (void)hipFree(Xt);
    (void)hipFree(lists);
    return rc;
}

}  // namespace tsnehip
