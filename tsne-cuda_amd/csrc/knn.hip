// Exact brute-force k nearest neighbours for gfx950.
//
// Stands in for the FAISS IVF-Flat search of the reference
// (src/util/distance_utils.cu:79-121), which is approximate; this one is exact
// and reproducible: the squared distance of a pair is accumulated in fp32 over
// ascending dimension with one fused multiply-add per dimension ("canonical"
// distance), neighbours are ordered by (distance, index), and the point itself
// is forced into slot 0 with distance exactly 0 (the perplexity search depends
// on that, src/kernels/perplexity_search.cu:30-32).
//
// Two sweeps share the selection machinery (a per-query candidate list filtered
// against the query's current k-th best and compacted by an LDS bitonic sort):
//
//  * VALU sweep: canonical distances directly, 64 queries x 128-candidate tiles,
//    4 x 8 register block per thread.  Exact by construction; any dimension.
//
//  * MFMA sweep (up to 126 dimensions): v_mfma_f32_32x32x2f32 evaluates
//    |c|^2 - 2 q.c for 32 candidates x 32 queries at a time.  The queries are
//    the B operand and stay in registers for the whole sweep (scaled by -2,
//    with one extra dimension that multiplies the candidate's |c|^2 by 1); the
//    candidates stream through LDS in the A operand's lane layout.  A lane owns
//    one query column of the 32 x 32 result, so filtering is a min over its 16
//    accumulators against one threshold register.  These distances are only
//    approximate (cancellation), so the sweep keeps K' > K candidates; a second
//    kernel recomputes their canonical distances, sorts, and proves that nothing
//    outside the list can belong to the top K: every discarded candidate has an
//    approximate distance >= tau (the K'-th best), hence a canonical distance
//    >= tau - g for a rigorous rounding bound g, and the query passes when its
//    K-th canonical distance is below that.  Queries that do not pass are redone
//    by the VALU sweep, so the result is exact either way.
//    Except at 126 dimensions the products run on the bf16 matrix pipe instead
//    (v_mfma_f32_32x32x16_bf16, two bf16 terms per coordinate, three products):
//    the candidates are stored relative to the centre m of their own 128-point
//    tile, which keeps what the split leaves out small, |q - m|^2 is added on
//    the vector ALU per (query, tile), and the keys are the distances less the
//    tile's error bound - lower bounds, so the proof above needs no g.
//
//  * Chunked MFMA sweep (more than 126 dimensions): the same products (bf16
//    terms by default), but the queries no longer fit a wave's registers, so
//    both operands stream in chunks of 64 dimensions (32 on bf16 terms; candidates through LDS,
//    queries straight into registers from a pre-scaled packed copy) while the
//    32 x 128 results of a wave accumulate in registers; |q - m|^2 is formed
//    chunk by chunk from the query-side operand and the centre's chunk.  With hundreds of dimensions a query's neighbour
//    distances lie close together and the rounding bound g grows, so the margin
//    K' - K is first tried on a sample of query tiles and doubled until the
//    sample verifies (or the vector sweep is taken instead); the query tiles of
//    the few queries that still fail are swept once more with twice the margin
//    before the vector sweep gets what is left.  Sweeps of few query tiles split
//    every tile's candidates over several workgroups; a merge kernel reduces
//    their lists to what a single list would have kept.
#include "common.h"
#include "stages.h"

#include <algorithm>
#include <climits>
#include <cmath>
#include <cstring>
#include <vector>

namespace tsnehip {

namespace {

typedef unsigned long long u64;
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kQT = 64;   // VALU sweep: queries per workgroup
constexpr int kCT = 128;  // candidates per tile (both sweeps)
constexpr int kDC = 32;   // VALU sweep: dimensions staged per chunk
constexpr int kMQ = 128;  // MFMA sweep: queries per workgroup (4 waves x 32)
constexpr int kMfmaMaxSteps = 64;  // k-steps of 2 dimensions: up to 126 dimensions + 2 augmented
static_assert(kMQ == kCT, "query tiles and candidate tiles share the packed layout");

// v_min3_f32 / v_min_f32 without the quieting moves the library fminf adds for signalling NaNs.
// The compiler's wait states between a matrix instruction and a vector instruction that reads its result do
// not cover instructions inside inline assembly: a chain of these over an accumulator has to start from
// matrix_result(), an ordinary instruction on one of the accumulator's registers, and depend on its value.
__device__ __forceinline__ float min3(float a, float b, float c) {
    float r;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float min2(float a, float b) {
    float r;
    asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float matrix_result(float x) { return __builtin_canonicalizef(x); }

__device__ __forceinline__ u64 pack_key(float d, int j) {
    return ((u64)float_to_ordered(d) << 32) | (unsigned int)j;
}
__device__ __forceinline__ float key_distance(u64 key) { return ordered_to_float((unsigned int)(key >> 32)); }
__device__ __forceinline__ int key_index(u64 key) { return (int)(unsigned int)(key & 0xffffffffu); }

// Transposed copy of the points, [dim][point], padded to Npad points (vector sweep).
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

// |x|^2 of every point (fp32, one fma per dimension) and the largest of them.
__global__ __launch_bounds__(256) void norms_kernel(const float *__restrict__ X, int N, int D, int Npad,
                                                    float *__restrict__ norms, float *__restrict__ max_norm) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    float nrm = 0.0f;
    if (i < N) {
        const float *x = X + (size_t)i * D;
        for (int d = 0; d < D; ++d) nrm = fmaf(x[d], x[d], nrm);
    }
    if (i < Npad) norms[i] = nrm;
    nrm = group_max<kWave>(nrm);
    if ((threadIdx.x & (kWave - 1)) == 0) atomicMax(reinterpret_cast<unsigned int *>(max_norm), __float_as_uint(nrm));
}

// Points in the A-operand layout of v_mfma_f32_32x32x2f32, tile by tile, so that
// a 128-candidate tile is one contiguous run of float4:
//   Xp[tile][block of 32 points (4)][group of 4 k-steps (S4)][lane (64)] float4
// where lane = (dimension % 2) * 32 + point % 32 and component = k-step % 4,
// k-step = dimension / 2.  Dimension Dnorm carries |x|^2, padding is zero.
__global__ __launch_bounds__(256) void pack_points_kernel(const float *__restrict__ X,
                                                          const float *__restrict__ norms, int N, int D, int Dnorm,
                                                          int S4, int Npad, float4 *__restrict__ Xp,
                                                          bool query_side) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one float4 of Xp per thread
    const int64_t total = (int64_t)Npad * S4 * 2;
    if (t >= total) return;
    const int lane = (int)(t & 63);
    const int64_t rest = t >> 6;
    const int s4 = (int)(rest % S4);
    const int64_t blk = rest / S4;  // tile * 4 + block
    const int i = (int)(blk * 32 + (lane & 31));
    const int h = lane >> 5;
    float v[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int d = 2 * (4 * s4 + c) + h;
        v[c] = 0.0f;
        if (i < N) {
            if (d < D) v[c] = query_side ? -2.0f * X[(size_t)i * D + d] : X[(size_t)i * D + d];
            else if (d == Dnorm) v[c] = query_side ? 1.0f : norms[i];
        }
    }
    Xp[t] = make_float4(v[0], v[1], v[2], v[3]);
}

// Nearest bf16 of a finite float (ties to even), as its 16 bits, and the float such bits stand for.
__device__ __forceinline__ unsigned int bf16_bits(float v) {
    const unsigned int u = __float_as_uint(v);
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float bf16_value(unsigned int bits) { return __uint_as_float(bits << 16); }

// Points for the bf16 sweep: relative to the centre m of their own tile's bounding ball (small numbers, so
// that what the bf16 terms leave out is small), every coordinate split into two bf16 terms (high = nearest
// bf16, low = nearest bf16 of the rest), in the A-operand layout of v_mfma_f32_32x32x16_bf16.  Per tile
//   [block of 32 points (4)][term (2: high, low)][step of 16 dimensions (S16)][lane (64)] 8 x bf16
// (lane = 32 * (dimension % 16 / 8) + point % 32, element = dimension % 8), then 64 float4 written by
// pack_tile_centres_kernel.  Dimensions D, D + 1 and D + 2 of the high term carry
// beta = |x - m|^2 + 2 m.(x - m) as three bf16 terms (24 bits: the float exactly), so that against the
// query-side operand (-2 q_d, and 1 in those three dimensions) the product is |q - x|^2 - |q - m|^2.
__global__ __launch_bounds__(256) void pack_points_bf16_kernel(const float *__restrict__ X,
                                                               const float *__restrict__ centers_t, int N, int D,
                                                               int S16, int T, int Npad, uint4 *__restrict__ Xb) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one lane's 8 values per thread
    const int64_t total = (int64_t)Npad * S16 * 4;
    if (t >= total) return;
    const int lane = (int)(t & 63);
    int64_t rest = t >> 6;
    const int s16 = (int)(rest % S16);
    rest /= S16;
    const int term = (int)(rest & 1);
    const int64_t blk = rest >> 1;  // tile * 4 + block
    const int tile = (int)(blk >> 2);
    const int i = (int)(blk * 32 + (lane & 31));
    const int d0 = 16 * s16 + 8 * (lane >> 5);
    unsigned int h[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    if (i < N) {
        float beta = 0.0f;
        if (term == 0 && d0 + 8 > D && d0 < D + 3) {
            float sq = 0.0f, dot = 0.0f;
            for (int d = 0; d < D; ++d) {
                const float m = centers_t[(size_t)d * T + tile];
                const float delta = X[(size_t)i * D + d] - m;
                sq = fmaf(delta, delta, sq);
                dot = fmaf(m, delta, dot);
            }
            beta = fmaf(2.0f, dot, sq);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int d = d0 + j;
            if (d < D) {
                const float v = X[(size_t)i * D + d] - centers_t[(size_t)d * T + tile];
                const unsigned int hi = bf16_bits(v);
                h[j] = term == 0 ? hi : bf16_bits(v - bf16_value(hi));
            } else if (d < D + 3 && term == 0) {
                float r = beta;
                unsigned int part = bf16_bits(r);
                for (int k = D; k < d; ++k) {
                    r -= bf16_value(part);
                    part = bf16_bits(r);
                }
                h[j] = part;
            }
        }
    }
    const int64_t in_tile = t - (int64_t)tile * (S16 * 512);
    Xb[(int64_t)tile * (S16 * 512 + 64) + in_tile] =
        make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
}

// The 64 float4 that close a tile of the bf16 sweep's points: floats 0 .. 16 S16 - 1 the centre m (zero beyond
// D), floats 128 and 129 the tile's error coefficients ga, gb.  A candidate distance the sweep computes for
// a query q against this tile is off by at most |q| ga + gb:
//  - the two bf16 terms leave out, per dimension, low x low and what they do not represent: with u = 2^-8
//    less than 3.1 * 2^-16 |q_d delta_d|, twice that after the factor -2, and sum |q_d delta_d| <= |q| r
//    (r: the ball's radius);
//  - the 3 D + 3 products are accumulated in fp32 in the matrix unit's order: 4 (3 D + 6) 2^-24 (the factor
//    four covers that order) times the sum of the terms' magnitudes, at most 2 |q| r + r^2 + 2 |m| r;
//  - the rounding of x - m, of beta and of the final additions is below a hundredth of the above.
__global__ __launch_bounds__(64) void pack_tile_centres_kernel(const float *__restrict__ centers_t,
                                                               const float *__restrict__ radius, int D, int S16,
                                                               int T, float4 *__restrict__ Xb) {
    const int tile = blockIdx.x, l = threadIdx.x;
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (l < 32) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (4 * l + c < D) v[c] = centers_t[(size_t)(4 * l + c) * T + tile];
    } else if (l == 32) {
        float m2 = 0.0f;
        for (int d = 0; d < D; ++d) {
            const float m = centers_t[(size_t)d * T + tile];
            m2 = fmaf(m, m, m2);
        }
        const float r = radius[tile], mlen = sqrtf(m2) * (1.0f + 1e-6f);
        const float split = 6.2f / 65536.0f, acc = 4.0f * (float)(3 * D + 6) * 5.9604644775390625e-08f;
        v[0] = 1.01f * (split + 2.0f * acc) * r;
        v[1] = 1.01f * acc * (r * r + 2.0f * mlen * r) + 1e-30f;
    }
    Xb[(size_t)tile * (S16 * 512 + 64) + S16 * 512 + l] = make_float4(v[0], v[1], v[2], v[3]);
}

// The bf16 operands of the chunked sweep, in its layout [tile][block of 32 points (4)][chunk of 32 dimensions]
// [slot (4)][lane (64)] 8 x bf16 with slot = 2 * term + step (step: 16 dimensions of the chunk; lane and
// element as in pack_points_bf16_kernel).  Candidate side: the points relative to their tile's centre in two
// terms, beta in dimensions D .. D + 2 of the high term.  Query side: -2 x in two terms, 1 in those three.
__global__ __launch_bounds__(256) void pack_points_bf16_chunked_kernel(const float *__restrict__ X,
                                                                       const float *__restrict__ centers_t, int N,
                                                                       int D, int n_chunks, int T, int Npad,
                                                                       uint4 *__restrict__ Xb, bool query_side) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // one lane's 8 values per thread
    const int64_t total = (int64_t)Npad * n_chunks * 8;
    if (t >= total) return;
    const int lane = (int)(t & 63);
    int64_t rest = t >> 6;
    const int slot = (int)(rest & 3);
    rest >>= 2;
    const int chunk = (int)(rest % n_chunks);
    const int64_t blk = rest / n_chunks;  // tile * 4 + block
    const int tile = (int)(blk >> 2);
    const int term = slot >> 1, step = slot & 1;
    const int i = (int)(blk * 32 + (lane & 31));
    const int d0 = 32 * chunk + 16 * step + 8 * (lane >> 5);
    unsigned int h[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
    if (i < N) {
        float beta = 0.0f;
        if (!query_side && term == 0 && d0 + 8 > D && d0 < D + 3) {
            float sq = 0.0f, dot = 0.0f;
            for (int d = 0; d < D; ++d) {
                const float m = centers_t[(size_t)d * T + tile];
                const float delta = X[(size_t)i * D + d] - m;
                sq = fmaf(delta, delta, sq);
                dot = fmaf(m, delta, dot);
            }
            beta = fmaf(2.0f, dot, sq);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int d = d0 + j;
            if (d < D) {
                const float x = X[(size_t)i * D + d];
                const float v = query_side ? -2.0f * x : x - centers_t[(size_t)d * T + tile];
                const unsigned int hi = bf16_bits(v);
                h[j] = term == 0 ? hi : bf16_bits(v - bf16_value(hi));
            } else if (d < D + 3 && term == 0) {
                if (query_side) {
                    h[j] = 0x3f80u;
                } else {
                    float r = beta;
                    unsigned int part = bf16_bits(r);
                    for (int k = D; k < d; ++k) {
                        r -= bf16_value(part);
                        part = bf16_bits(r);
                    }
                    h[j] = part;
                }
            }
        }
    }
    Xb[t] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
}

// Tile centres for the chunked bf16 sweep: centres_p[tile][32 n_chunks] and the two error coefficients of
// pack_tile_centres_kernel in tile_coef[2 tile], [2 tile + 1].  Beyond D the centre is zero, except -1/2 in
// dimensions D .. D + 2: the sweep forms |q - m|^2 from the query-side operand, which holds 1 there and
// stands for -2 q, so those three dimensions add nothing.
__global__ __launch_bounds__(64) void pack_chunked_centres_kernel(const float *__restrict__ centers_t,
                                                                  const float *__restrict__ radius, int D,
                                                                  int n_chunks, int T, float *__restrict__ centres_p,
                                                                  float *__restrict__ tile_coef) {
    const int tile = blockIdx.x, l = threadIdx.x;
    float m2 = 0.0f;
    for (int d = l; d < 32 * n_chunks; d += 64) {
        const float m = d < D ? centers_t[(size_t)d * T + tile] : 0.0f;
        centres_p[(size_t)tile * 32 * n_chunks + d] = d >= D && d < D + 3 ? -0.5f : m;
        m2 = fmaf(m, m, m2);
    }
    m2 = group_sum<kWave>(m2);
    if (l == 0) {
        const float r = radius[tile], mlen = sqrtf(m2) * (1.0f + 1e-5f);
        const float split = 6.2f / 65536.0f, acc = 4.0f * (float)(3 * D + 6) * 5.9604644775390625e-08f;
        tile_coef[2 * tile] = 1.01f * (split + 2.0f * acc) * r;
        tile_coef[2 * tile + 1] = 1.01f * acc * (r * r + 2.0f * mlen * r) + 1e-30f;
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

// Wave-private selection for the matrix sweep, where a query's list, counter and threshold are
// only ever touched by the wave that owns the query.  The sweep never needs its candidates in
// order, only the `want` smallest of them and the distance of the last one kept, so a compaction
// is a radix select on the distance bits, six bits per pass: lane l owns histogram bin l, a wave
// scan finds the bin that holds the want-th smallest.  The bits are taken relative to the smallest
// distance present, which skips the leading bits all keys share.  No workgroup barrier is involved
// (LDS operations of a wave execute in order; the wavefront fences only stop the compiler from
// reordering them), so the other waves keep issuing matrix instructions meanwhile.
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
    // Within the rows of 16 lanes by DPP row shifts (a lane without a source adds 0), then the row totals
    // across the rows by the two row broadcasts (lane 15 of a row to the next row: rows 1 and 3; lane 31 to
    // rows 2 and 3).  Twelve vector instructions; six ds_bpermute round trips through LDS before.
    (void)lane;
    int x = v;
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, true);   // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, true);   // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, true);   // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, true);   // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31
    return x;
}

// list: this query's entries in global memory (n = *cnt of them); buf: cap keys of LDS; hist: 64 words
// of LDS.  Afterwards list[0, min(n, want)) holds the entries kept (in no particular order), *cnt their
// number, and *thr is lowered to (distance of the want-th smallest, all index bits set) when n >= want.
// Returns the number of entries kept.
// With slack > 0 the selection may stop early: once the histogram bin that holds the want-th smallest
// has few enough entries that keeping all of them stays within want + slack, everything up to the
// bin's upper edge is kept and that edge becomes the threshold.  A compaction in the middle of a sweep
// only needs some threshold below which everything was kept; the last one of a query passes slack = 0.
//
// HALVES: the list is two regions of `half` entries, each appended to by one of the query's two lanes
// (entries 0 .. c0-1 of the first, the rest of the *cnt entries in the second); the entries kept go back
// alternately into the two regions (entry p to region p & 1, position p >> 1), so both keep room.
template <bool HALVES = false>
__device__ __forceinline__ int wave_select(u64 *list, int want, int *cnt, u64 *thr, u64 *buf, unsigned int *hist,
                                           int lane, int slack = 0, int half = 0, int c0 = 0) {
    __threadfence_block();  // this wave's appends to the list are complete
    const int n = *cnt;
    if (n < want) return n;
    auto wr = [&](int p, u64 key) {
        if (HALVES) list[(p & 1) * half + (p >> 1)] = key;
        else list[p] = key;
    };
    unsigned int lo = ~0u, hi = 0u;
    // Four loads in flight: the list comes from global memory and a load at a time would cost its latency each.
    auto load_run = [&](const u64 *src, int count, u64 *dst) {
        for (int e0 = lane; e0 < count; e0 += 4 * kWave) {
            u64 key[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) key[u] = src[min(e0 + u * kWave, count - 1)];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = e0 + u * kWave;
                if (e < count) {
                    dst[e] = key[u];
                    const unsigned int bits = (unsigned int)(key[u] >> 32);
                    lo = min(lo, bits);
                    hi = max(hi, bits);
                }
            }
        }
    };
    if (HALVES) {
        load_run(list, c0, buf);
        load_run(list + half, n - c0, buf + c0);
    } else {
        load_run(list, n, buf);
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        lo = min(lo, (unsigned int)__shfl_xor((int)lo, m, kWave));
        hi = max(hi, (unsigned int)__shfl_xor((int)hi, m, kWave));
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    // Radix select of the want-th smallest value of (bits - lo).
    unsigned int prefix = 0u;
    int rank = want;  // 1-based rank among the keys that match the prefix
    int shift = 32 - __clz((int)(hi - lo));  // significant bits of the range (0 when all distances are equal)
    if (hi == lo) shift = 0;
    while (shift > 0) {
        const int w = shift < 6 ? shift : 6;
        shift -= w;
        hist[lane] = 0u;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        for (int e = lane; e < n; e += kWave) {
            const unsigned int v = (unsigned int)(buf[e] >> 32) - lo;
            if ((unsigned int)((u64)v >> (shift + w)) == prefix) atomicAdd(&hist[(v >> shift) & ((1u << w) - 1u)], 1u);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        const int c = (int)hist[lane];
        const int incl = wave_inclusive_scan(c, lane);
        const int b = __ffsll((long long)__ballot(incl >= rank)) - 1;  // some lane qualifies: the last one holds all matches
        rank -= __builtin_amdgcn_readlane(incl - c, b);  // (b is the same in every lane)
        prefix = (prefix << w) | (unsigned int)b;
        if (slack > 0 && shift > 0) {
            const int kept = (want - rank) + __builtin_amdgcn_readlane(c, b);  // below the bin + the whole bin
            if (kept <= want + slack) {
                // Keep everything up to the upper edge of the bin.
                const u64 edge = (u64)lo + ((((u64)prefix + 1ull) << shift) - 1ull);
                const unsigned int dedge = edge > 0xffffffffull ? 0xffffffffu : (unsigned int)edge;
                int base = 0;
                const u64 below_lanes = (1ull << lane) - 1ull;
                for (int e0 = 0; e0 < n; e0 += kWave) {
                    const int e = e0 + lane;
                    const u64 key = e < n ? buf[e] : 0ull;
                    const bool keep = e < n && (unsigned int)(key >> 32) <= dedge;
                    const u64 m = __ballot(keep);
                    if (keep) wr(base + __popcll(m & below_lanes), key);
                    base += __popcll(m);
                }
                if (lane == 0) {
                    *cnt = base;
                    *thr = ((u64)dedge << 32) | 0xffffffffull;
                }
                __threadfence_block();
                return base;
            }
        }
    }
    const unsigned int dstar = lo + prefix;
    // Keep everything below dstar and the first `rank` entries equal to it.
    const int need_eq = rank, c_lt = want - rank;
    int base_lt = 0, base_eq = 0;
    const u64 below = (1ull << lane) - 1ull;
    for (int e0 = 0; e0 < n; e0 += kWave) {
        const int e = e0 + lane;
        const u64 key = e < n ? buf[e] : 0ull;
        const unsigned int bits = (unsigned int)(key >> 32);
        const bool lt = e < n && bits < dstar, eq = e < n && bits == dstar;
        const u64 m_lt = __ballot(lt), m_eq = __ballot(eq);
        if (lt) wr(base_lt + __popcll(m_lt & below), key);
        if (eq) {
            const int k = base_eq + __popcll(m_eq & below);
            if (k < need_eq) wr(c_lt + k, key);
        }
        base_lt += __popcll(m_lt);
        base_eq += __popcll(m_eq);
    }
    if (lane == 0) {
        *cnt = want;
        *thr = ((u64)dstar << 32) | 0xffffffffull;
    }
    __threadfence_block();
    return want;
}

// Bounding ball of every tile of kCT consecutive points: the centre is the tile's mean, the
// radius the largest distance of a member to it, inflated by 1e-3 (far more than the fp32
// rounding of the sums) so that it is an upper bound.  centers_t is D x T (dimension-major).
// One workgroup of 128 threads per tile; dynamic LDS: D floats.
__global__ __launch_bounds__(128) void tile_balls_kernel(const float *__restrict__ X, int N, int D, int T,
                                                         float *__restrict__ centers_t, float *__restrict__ radius) {
    extern __shared__ float c[];
    __shared__ float wmax[2];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int first = t * kCT;
    const int count = min(kCT, N - first);
    for (int d = tid; d < D; d += 128) {
        float sum = 0.0f;
        for (int i = 0; i < count; ++i) sum += X[(size_t)(first + i) * D + d];
        sum /= (float)count;
        c[d] = sum;
        centers_t[(size_t)d * T + t] = sum;
    }
    __syncthreads();
    float d2 = 0.0f;
    if (tid < count) {
        const float *x = X + (size_t)(first + tid) * D;
        for (int d = 0; d < D; ++d) {
            const float diff = x[d] - c[d];
            d2 = fmaf(diff, diff, d2);
        }
    }
    d2 = group_max<kWave>(d2);
    if ((tid & (kWave - 1)) == 0) wmax[tid / kWave] = d2;
    __syncthreads();
    if (tid == 0) radius[t] = sqrtf(fmaxf(wmax[0], wmax[1])) * (1.0f + 1e-3f) + 1e-30f;
}

constexpr int kHomeTiles = 8;  // candidate tiles on either side of the query tile that are always swept

// Whether tile t may hold a point closer than sqrt(tmax) to some point of the tile whose ball is
// (qcenter, ra): with c, r the balls, every pair of members is at least |c_a - c_t| - r_a - r_t apart
// (triangle inequality); 1e-3 relative slack on the centre distance, the radii are upper bounds.
// Anything that is not a number keeps the tile.
// Eight loads in flight and two partial sums: one load at a time would cost its latency per dimension
// (any summation order will do, the slack covers the rounding).
__device__ __forceinline__ bool tile_may_matter(const float *qcenter, float ra, const float *__restrict__ centers_t,
                                                const float *__restrict__ radius, int D, int T, int t, float tmax) {
    float s0 = 0.0f, s1 = 0.0f;
    int d = 0;
    for (; d + 8 <= D; d += 8) {
        float c[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) c[u] = centers_t[(size_t)(d + u) * T + t];
#pragma unroll
        for (int u = 0; u < 8; u += 2) {
            const float e0 = qcenter[d + u] - c[u], e1 = qcenter[d + u + 1] - c[u + 1];
            s0 = fmaf(e0, e0, s0);
            s1 = fmaf(e1, e1, s1);
        }
    }
    for (; d < D; ++d) {
        const float diff = qcenter[d] - centers_t[(size_t)d * T + t];
        s0 = fmaf(diff, diff, s0);
    }
    const float lb = sqrtf(s0 + s1) * (1.0f - 1e-3f) - (ra + radius[t]);
    return !(lb > 0.0f && lb * lb > tmax);
}

// ---------------------------------------------------------------------------
// VALU sweep.  qlist == nullptr: queries are 0..N-1; otherwise the nq listed ones.
// Sweeping all queries with tile balls given (bitmap_words > 0), the candidate tiles are visited in
// two phases as in the matrix sweep: the query tile's neighbourhood in the numbering first, then
// only the tiles whose ball may hold a point below the largest k-th distance found so far.  The
// distances here are the canonical ones, so a skipped tile is strictly farther than every threshold.
// Dynamic LDS: cap keys, then D floats (the query tile's ball centre), then the visit bitmap.
//
// slices > 1 (listed queries only): a handful of queries would occupy a handful of workgroups for a sweep over
// all points, so the candidate tiles are cut into `slices` ranges and a (query tile, range) pair is one unit of
// work; each unit leaves its K-1 best keys in slice_keys[(slot * slices + range) * (K-1) ...] (padded with ~0)
// and knn_merge_slices_kernel forms the rows.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void knn_sweep_kernel(const float *__restrict__ Xt, int N, int Npad, int D, int K,
                                                        int cap, u64 *__restrict__ lists, int num_qtiles,
                                                        const int *__restrict__ qlist, int nq,
                                                        int *__restrict__ out_idx, float *__restrict__ out_d,
                                                        const float *__restrict__ centers_t,
                                                        const float *__restrict__ radius, int bitmap_words,
                                                        int slices, u64 *__restrict__ slice_keys) {
    __shared__ __attribute__((aligned(16))) float xq[kDC][kQT];
    __shared__ __attribute__((aligned(16))) float xc[kDC][kCT];
    __shared__ u64 thr[kQT];
    __shared__ int cnt[kQT];
    __shared__ int qid[kQT];
    extern __shared__ u64 sortbuf[];
    float *qcenter = reinterpret_cast<float *>(sortbuf + cap);
    unsigned int *bitmap = reinterpret_cast<unsigned int *>(qcenter + D);
    __shared__ float tmax_part[kQT / kWave];

    const int tid = threadIdx.x;
    const int tq = tid >> 4, tc = tid & 15;
    const int want = K - 1;
    const int T = (N + kCT - 1) / kCT;
    u64 *list = lists + (size_t)blockIdx.x * kQT * cap;

    for (int unit = blockIdx.x; unit < num_qtiles * slices; unit += gridDim.x) {
        const int qt = unit / slices, slice = unit - qt * slices;
        if (tid < kQT) {
            const int slot = qt * kQT + tid;
            thr[tid] = ~0ull;
            cnt[tid] = 0;
            qid[tid] = slot < nq ? (qlist ? qlist[slot] : slot) : -1;
        }
        __syncthreads();
        auto process = [&](int c0) {
            float acc[4][8];
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 8; ++b) acc[a][b] = 0.0f;
            for (int d0 = 0; d0 < D; d0 += kDC) {
                const int dn = min(kDC, D - d0);
                __syncthreads();
                for (int e = tid; e < dn * kQT; e += 256) {
                    const int dd = e / kQT, ql = e % kQT;
                    const int q = qid[ql];
                    xq[dd][ql] = q >= 0 ? Xt[(size_t)(d0 + dd) * Npad + q] : 0.0f;
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
                const int q = qid[ql];
                const u64 limit = thr[ql];
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    const int j = c0 + tc * 8 + b;
                    const u64 key = pack_key(acc[a][b], j);
                    if (j < N && q >= 0 && j != q && key < limit) {
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
        };
        const bool prune = bitmap_words > 0 && qlist == nullptr;
        const int bt = (qt * kQT) / kCT;  // the ball tile this query tile lies in
        int h0 = prune ? max(bt - kHomeTiles, 0) : 0, h1 = prune ? min(bt + kHomeTiles, T - 1) : T - 1;
        if (slices > 1) {  // this unit's range of the candidate tiles
            h0 = (int)(((long long)T * slice) / slices);
            h1 = (int)(((long long)T * (slice + 1)) / slices) - 1;
        }
        for (int ct = h0; ct <= h1; ++ct) process(ct * kCT);
        if (prune && (h0 > 0 || h1 < T - 1)) {
            // Thresholds from what the neighbourhood held, then the tiles that may still matter.
            for (int ql = 0; ql < kQT; ++ql)
                if (qid[ql] >= 0) compact_query(list, cap, want, cnt, thr, ql, sortbuf, tid);
            for (int w = tid; w < bitmap_words; w += 256) bitmap[w] = 0u;
            for (int d = tid; d < D; d += 256) qcenter[d] = centers_t[(size_t)d * T + bt];
            if (tid < kQT) {
                float v = -INFINITY;
                if (qid[tid] >= 0) {
                    const u64 t = thr[tid];
                    v = t == ~0ull ? INFINITY : key_distance(t);
                    v += 1e-5f * fabsf(v) + 1e-30f;
                }
                v = group_max<kWave>(v);
                if ((tid & (kWave - 1)) == 0) tmax_part[tid / kWave] = v;
            }
            __syncthreads();
            float tmax = tmax_part[0];
#pragma unroll
            for (int w = 1; w < kQT / kWave; ++w) tmax = fmaxf(tmax, tmax_part[w]);
            const float ra = radius[bt];
            for (int t = tid; t < T; t += 256)
                if ((t < h0 || t > h1) && tile_may_matter(qcenter, ra, centers_t, radius, D, T, t, tmax))
                    atomicOr(&bitmap[t >> 5], 1u << (t & 31));
            __syncthreads();
            for (int w = 0; w < bitmap_words; ++w) {
                unsigned int word = bitmap[w];
                while (word) {
                    const int t = w * 32 + __ffs((int)word) - 1;
                    word &= word - 1u;
                    process(t * kCT);
                }
            }
        }
        // Final ordering and output: self first, then the K-1 best others.
        for (int ql = 0; ql < kQT; ++ql) {
            const int q = qid[ql];
            if (q < 0) break;
            compact_query(list, cap, want, cnt, thr, ql, sortbuf, tid);
            if (slices > 1) {
                // (compact_query leaves the sorted keys in sortbuf, ~0 beyond the entries there were)
                u64 *dst = slice_keys + ((size_t)(qt * kQT + ql) * slices + slice) * want;
                for (int e = tid; e < want; e += 256) dst[e] = sortbuf[e];
                __syncthreads();
                continue;
            }
            for (int e = tid; e < K; e += 256) {
                int j = q;
                float d = 0.0f;
                if (e > 0) {
                    const u64 key = sortbuf[e - 1];
                    j = key_index(key);
                    d = key_distance(key);
                }
                out_idx[(size_t)q * K + e] = j;
                out_d[(size_t)q * K + e] = d;
            }
            __syncthreads();
        }
    }
}

// Rows of the listed queries from the keys their `slices` units left: one workgroup per query sorts the
// slices * (K-1) keys (sort_n: that count rounded up to a power of two; dynamic LDS: sort_n keys).
__global__ __launch_bounds__(256) void knn_merge_slices_kernel(const u64 *__restrict__ slice_keys, int slices, int K,
                                                               int sort_n, const int *__restrict__ qlist,
                                                               int *__restrict__ out_idx, float *__restrict__ out_d) {
    extern __shared__ u64 merge_sortbuf[];
    const int tid = threadIdx.x, slot = blockIdx.x, want = K - 1;
    const int q = qlist[slot];
    const int total = slices * want;
    for (int e = tid; e < sort_n; e += 256) merge_sortbuf[e] = e < total ? slice_keys[(size_t)slot * total + e] : ~0ull;
    __syncthreads();
    bitonic_sort(merge_sortbuf, sort_n, tid);
    for (int e = tid; e < K; e += 256) {
        int j = q;
        float d = 0.0f;
        if (e > 0) {
            const u64 key = merge_sortbuf[e - 1];
            j = key_index(key);
            d = key_distance(key);
        }
        out_idx[(size_t)q * K + e] = j;
        out_d[(size_t)q * K + e] = d;
    }
}

struct SweepArgs {
    const float4 *Xp;
    const float *X;  // the points as given (bf16 sweep: the query side is formed from them)
    const float *centres_p, *tile_coef;  // chunked bf16 sweep: tile centres by chunk, error coefficients
    int N, D, Dnorm, want, cap;
    u64 *lists;
    int num_qtiles;
    int *cand;
    float *tau;
    const float *norms;      // |x|^2 per point
    const float *centers_t;  // D x T tile centres
    const float *radius;     // T tile radii (upper bounds)
    int bitmap_words;        // ceil(T / 32)
    int trigger;             // a list longer than this is compacted after the tile (<= cap - kCT)
    unsigned long long *tiles_swept;  // statistics: (query tile, candidate tile) pairs computed
    const float4 *Bp;  // chunked sweep only: query-side packed copy (-2 x_d, 1 in the |c|^2 row)
    int n_chunks;      // chunked sweep only: chunks of kChunkSteps k-steps per point
    // Chunked sweep only.  The num_qtiles query tiles are qtile_list[i], or first + i step without a list.
    // Every query tile is swept by `parts` workgroups, part p taking the candidate tiles t with t % parts == p.
    // One part writes cand / tau directly (row i * kMQ + query in tile); several parts write the keys they
    // keep (all bits set where a part has fewer) to row (i * kMQ + query in tile) * parts + p of part_keys,
    // and knn_merge_parts_kernel picks the `want` best of a query's parts afterwards.
    const int *qtile_list;
    int qtile_first, qtile_step;
    int parts;
    u64 *part_keys;
    int select_slack;  // entries beyond `want` a compaction in mid-sweep may keep (see wave_select)
    // Approximate search (register-resident sweep only; null = exact): the points are numbered list by list of
    // an inverted file, and after its neighbourhood in the numbering a query tile only visits the tiles that
    // overlap the lists some query of the tile probes.  probe_tile_lists: per query tile a bitmap over the
    // lists (probe_list_words words); probe_list_tiles: first and last tile of every list (first > last: empty).
    const unsigned int *probe_tile_lists;
    int probe_list_words, probe_nlist;
    const int *probe_list_tiles;
};

// ---------------------------------------------------------------------------
// MFMA sweep, in two arithmetic variants.
// BF16 = false: KSTEPS = Daug / 2 k-steps of v_mfma_f32_32x32x2f32 on the points as floats.
// BF16 = true: KSTEPS steps of 16 dimensions of v_mfma_f32_32x32x16_bf16 on the points relative to their
// tile's centre, split into two bf16 terms per coordinate; high x high, high x low and low x high are
// accumulated (three instructions per step), which leaves out terms below 3.1 * 2^-16 of |q_d delta_d| per
// dimension.  The keys stored are the products plus |q - centre|^2 less the tile's error bound (see
// pack_tile_centres_kernel): lower bounds of the distances.  A step of 16 dimensions takes half the
// matrix-pipe time of one fp32 step of 2.
// Dynamic LDS: one candidate tile, copied verbatim from the packed points
//   a[cand block (4)][step group (S4)][lane (64)] float4   (4 steps per float4)            fp32
//   a[cand block (4)][term (2)][step (KSTEPS)][lane (64)] 8 x bf16                          bf16
// followed by one sort buffer (cap keys) per wave and the visit bitmap (one bit per tile).
//
// Tiles are visited in two phases.  First the query tile's own neighbourhood in the point
// numbering (kHomeTiles tiles on either side), which gives every query a finite threshold.
// Then only the tiles whose bounding ball can still hold a point below the largest of those
// thresholds: with c, r the centre and radius of a tile's ball, every point x of tile t has
// |q - x| >= |c_a - c_t| - r_a - r_t for every query q of tile a (triangle inequality), so the
// tile is skipped when that bound, squared, exceeds max_q (threshold_q + |q|^2).  A threshold
// only ever decreases and the final verification of a query compares with its final threshold,
// so a skipped tile cannot hold one of its neighbours.  On numberings without locality the
// balls are large and nothing is skipped.
// Output per query: the `want` best candidates by approximate distance
// (cand, -1 padded) and tau = the approximate distance of the last one kept
// (+inf when fewer than `want` candidates exist), both without the |q|^2 term.
// ---------------------------------------------------------------------------
// Workgroups per compute unit the register budget is set for (bf16: the query's coordinates stay in
// registers beside the two operand terms).  Measured: three workgroups with 330 bytes of spills per lane
// ran at half the speed of two at 4 steps; two workgroups beat one at 5 to 7 steps in spite of 100 to 380
// bytes of spills (300,000 points, 64 / 90 / 100 dimensions: 0.040 -> 0.027 s, 0.044 -> 0.033 s,
// 0.045 -> 0.040 s); at 8 steps two tiles of 66 KB do not fit a compute unit's LDS.
constexpr int bf16_sweep_occupancy(int steps) { return steps <= 2 ? 3 : (steps <= 7 ? 2 : 1); }
template <int KSTEPS, bool BF16>
constexpr int sweep_occupancy() {
    return BF16 ? bf16_sweep_occupancy(KSTEPS) : (KSTEPS <= 28 ? 3 : 1);
}

template <int KSTEPS, bool BF16>
__global__ __launch_bounds__(256, (sweep_occupancy<KSTEPS, BF16>())) void knn_mfma_sweep_kernel(const SweepArgs args) {
    const float4 *__restrict__ Xp = args.Xp;
    const int N = args.N, D = args.D, Dnorm = args.Dnorm, want = args.want, cap = args.cap;
    const int num_qtiles = args.num_qtiles;
    u64 *__restrict__ lists = args.lists;
    int *__restrict__ cand = args.cand;
    float *__restrict__ tau = args.tau;
    constexpr int S4 = BF16 ? 2 * KSTEPS : (KSTEPS + 3) / 4;  // 16-byte slots per lane and candidate block
    constexpr int kMainFloat4 = 4 * S4 * 64;              // float4 of matrix operands per candidate tile
    constexpr int kTileFloat4 = kMainFloat4 + (BF16 ? 64 : 0);  // ... and the centre block of the bf16 layout
    constexpr int kLoadsPerThread = kMainFloat4 / 256;    // == S4
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    float4 *a_lds = reinterpret_cast<float4 *>(lds_raw);
    u64 *sortbuf = reinterpret_cast<u64 *>(a_lds + kTileFloat4) + (size_t)(threadIdx.x >> 6) * cap;  // per wave
    unsigned int *bitmap = reinterpret_cast<unsigned int *>(reinterpret_cast<u64 *>(a_lds + kTileFloat4) + 4 * (size_t)cap);
    __shared__ u64 thr[kMQ];
    __shared__ int cnt[kMQ];
    __shared__ int fill[256];  // entries in each lane's region of its query's list
    __shared__ float qcenter[128];
    __shared__ unsigned int hist_all[4][kWave];
    __shared__ float tmax_part[2];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int qn = lane & 31, kh = lane >> 5;
    u64 *list = lists + (size_t)blockIdx.x * kMQ * cap;

    // One candidate tile: global -> registers (in flight during the matrix instructions) -> LDS.
    // The staging array is a native vector type with compile-time indices: as an array of
    // HIP float4 structs it was placed in scratch memory, where every load waited for the last.
    v4f stage[kLoadsPerThread], stage_centre;
    auto fetch = [&](int tile) {
        const v4f *src = reinterpret_cast<const v4f *>(Xp) + (size_t)tile * kTileFloat4 + tid;
#pragma unroll
        for (int r = 0; r < kLoadsPerThread; ++r) stage[r] = src[r * 256];
        if (BF16 && tid < 64) stage_centre = src[kMainFloat4];
    };
    auto stash = [&](int buf) {
        v4f *dst = reinterpret_cast<v4f *>(a_lds) + buf * kTileFloat4 + tid;
#pragma unroll
        for (int r = 0; r < kLoadsPerThread; ++r) dst[r * 256] = stage[r];
        if (BF16 && tid < 64) dst[kMainFloat4] = stage_centre;
    };
    const int num_ctiles = (N + kCT - 1) / kCT;

    for (int qt = blockIdx.x; qt < num_qtiles; qt += gridDim.x) {
        const int q0 = qt * kMQ;
        const int q = q0 + wave * 32 + qn;  // this lane's query (>= N in the last tile: padded zeros)
        if (tid < kMQ) {
            thr[tid] = ~0ull;
            cnt[tid] = 0;
        }
        // A query's list is two regions of cap / 2 entries, one per lane of the pair that shares the query:
        // a lane appends to its own region with a counter of its own, so an append needs neither a count of
        // the passing elements nor an atomic to reserve room.
        const int half = cap >> 1;
        // The counter is a register; around a selection it passes through LDS (fill[tid]), where the whole
        // wave can read and set it.
        int my_n = 0;
        // Selection over the list of query b of this wave (all lanes take part); returns the caller's updated
        // counter: the entries kept go back alternately into the two regions.
        // With fewer than `want` entries nothing is dropped; `spread` then still deals them out alternately,
        // for a query whose one region fills up while the other stays empty (and for the output pass, which
        // reads that order).
        auto select_query = [&](int b, int slack, bool spread) {
            const int ql = wave * 32 + b;
            const int c0n = fill[wave * 64 + b], c1n = fill[wave * 64 + b + 32];
            int kept = c0n + c1n;
            if (kept < want) {
                if (!spread) return;
                u64 *lq = list + (size_t)ql * cap;
                __threadfence_block();  // this wave's appends to the list are complete
                for (int e = lane; e < kept; e += kWave) sortbuf[e] = e < c0n ? lq[e] : lq[half + e - c0n];
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                for (int e = lane; e < kept; e += kWave) lq[(e & 1) * half + (e >> 1)] = sortbuf[e];
                __threadfence_block();
            } else {
                if (lane == 0) cnt[ql] = kept;
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                kept = wave_select<true>(list + (size_t)ql * cap, want, &cnt[ql], &thr[ql], sortbuf,
                                         hist_all[wave], lane, slack, half, c0n);
            }
            if (lane == 0) {
                fill[wave * 64 + b] = (kept + 1) >> 1;
                fill[wave * 64 + b + 32] = kept >> 1;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        };
        // B operand from the same packed layout (query tiles and candidate tiles coincide: kMQ == kCT):
        // -2 q_d for the real dimensions, 1 for the |c|^2 row, 0 elsewhere.
        float bq[BF16 ? 1 : 4 * S4];
        v8bf bq_hi[BF16 ? KSTEPS : 1], bq_lo[BF16 ? KSTEPS : 1];
        float qf[BF16 ? 8 * KSTEPS : 1];  // this lane's half of the query's coordinates
        float q_len = 0.0f;               // |q|, rounded up
        if constexpr (BF16) {
            // -2 q_d in two bf16 terms; 1 in the three dimensions of the high term that carry beta.
            const float *xq = args.X + (size_t)(q < N ? q : 0) * D;
            if (q < N) q_len = sqrtf(args.norms[q]) * (1.0f + 1e-6f);
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) {
                unsigned int oh[4], ol[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    unsigned int h2[2], l2[2];
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const int d = 16 * s + 8 * kh + 2 * k + e;
                        const float v = q < N && d < D ? xq[d] : 0.0f;
                        qf[8 * s + 2 * k + e] = v;
                        const float w = -2.0f * v;
                        const unsigned int hi = bf16_bits(w);
                        h2[e] = d < D ? hi : (d < D + 3 ? 0x3f80u : 0u);
                        l2[e] = d < D ? bf16_bits(w - bf16_value(hi)) : 0u;
                    }
                    oh[k] = h2[0] | (h2[1] << 16);
                    ol[k] = l2[0] | (l2[1] << 16);
                }
                bq_hi[s] = __builtin_bit_cast(v8bf, make_uint4(oh[0], oh[1], oh[2], oh[3]));
                bq_lo[s] = __builtin_bit_cast(v8bf, make_uint4(ol[0], ol[1], ol[2], ol[3]));
            }
        } else {
            const float4 *src = Xp + (size_t)qt * kTileFloat4 + (size_t)wave * S4 * 64 + lane;
#pragma unroll
            for (int s4 = 0; s4 < S4; ++s4) {
                const float4 v = src[s4 * 64];
                const float c[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int d = 2 * (4 * s4 + k) + kh;
                    bq[4 * s4 + k] = d < D ? -2.0f * c[k] : (d == Dnorm ? 1.0f : 0.0f);
                }
            }
        }
        const int buf = 0;  // one LDS tile: the next tile waits in registers until this one has been read
        // One tile: compute it from LDS buffer `buf` while the next one travels through registers.
        auto process = [&](int ct, int next_ct) {
            const int c0 = ct * kCT;
            if (next_ct >= 0) fetch(next_ct);
            const u64 limit = thr[wave * 32 + qn];
            // ~0 is "no threshold yet": its distance field does not decode to a number.
            const float limit_d = limit == ~0ull ? INFINITY : key_distance(limit);
            // bf16: the matrix product lacks |q - m|^2 (m: the tile's centre), and the keys carry a lower bound
            // of the distance: the product plus `off` = |q - m|^2 (rounded down) - the tile's error bound.
            // The products are tested against the threshold less `off`, rounded up.
            float off = 0.0f, limit_acc = limit_d;
            if constexpr (BF16) {
                const float4 *cen = a_lds + buf * kTileFloat4 + kMainFloat4;
                float f = 0.0f;
#pragma unroll
                for (int s = 0; s < KSTEPS; ++s) {
                    const float4 m0 = cen[4 * s + 2 * kh], m1 = cen[4 * s + 2 * kh + 1];
                    const float m[8] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float diff = qf[8 * s + j] - m[j];
                        f = fmaf(diff, diff, f);
                    }
                }
                f += __shfl_xor(f, 32);
                const float4 g = cen[32];
                off = f * (1.0f - (float)(D + 4) * 5.9604644775390625e-08f) - fmaf(q_len, g.x, g.y);
                limit_acc = limit_d - off;
                limit_acc += 2.4e-7f * (fabsf(limit_d) + fabsf(off));  // (inf stays inf)
            }
            // Two candidate blocks at a time: two independent accumulator chains keep the matrix pipe busy.
            auto multiply = [&](int cb, v16f &acc0, v16f &acc1) {
                acc0 = v16f{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                acc1 = acc0;
                const float4 *a0 = a_lds + (size_t)(buf * 4 + cb) * S4 * 64 + lane;
                const float4 *a1 = a0 + S4 * 64;
                if constexpr (BF16) {
                    const v4f *b0 = reinterpret_cast<const v4f *>(a0), *b1 = reinterpret_cast<const v4f *>(a1);
                    // The operands of step s + 1 are read from LDS while the products of step s run.
                    v4f next[4] = {b0[0], b1[0], b0[KSTEPS * 64], b1[KSTEPS * 64]};
#pragma unroll
                    for (int s = 0; s < KSTEPS; ++s) {
                        const v8bf xh = __builtin_bit_cast(v8bf, next[0]);
                        const v8bf yh = __builtin_bit_cast(v8bf, next[1]);
                        const v8bf xl = __builtin_bit_cast(v8bf, next[2]);
                        const v8bf yl = __builtin_bit_cast(v8bf, next[3]);
                        if (s + 1 < KSTEPS) {
                            next[0] = b0[(s + 1) * 64];
                            next[1] = b1[(s + 1) * 64];
                            next[2] = b0[(KSTEPS + s + 1) * 64];
                            next[3] = b1[(KSTEPS + s + 1) * 64];
                        }
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xh, bq_hi[s], acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(yh, bq_hi[s], acc1, 0, 0, 0);
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xh, bq_lo[s], acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(yh, bq_lo[s], acc1, 0, 0, 0);
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xl, bq_hi[s], acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(yl, bq_hi[s], acc1, 0, 0, 0);
                    }
                } else {
#pragma unroll
                    for (int s4 = 0; s4 < S4; ++s4) {
                        const float4 x = a0[s4 * 64], y = a1[s4 * 64];
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, bq[4 * s4], acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.x, bq[4 * s4], acc1, 0, 0, 0);
                        if (4 * s4 + 1 < KSTEPS) {
                            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, bq[4 * s4 + 1], acc0, 0, 0, 0);
                            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.y, bq[4 * s4 + 1], acc1, 0, 0, 0);
                        }
                        if (4 * s4 + 2 < KSTEPS) {
                            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, bq[4 * s4 + 2], acc0, 0, 0, 0);
                            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.z, bq[4 * s4 + 2], acc1, 0, 0, 0);
                        }
                        if (4 * s4 + 3 < KSTEPS) {
                            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, bq[4 * s4 + 3], acc0, 0, 0, 0);
                            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.w, bq[4 * s4 + 3], acc1, 0, 0, 0);
                        }
                    }
                }
            };
            auto filter = [&](int cb, v16f &acc0, v16f &acc1) {
                // Register v of lane l holds candidate row 8*(v/4) + 4*(l/32) + v%4 of the block, query column l%32.
                // Smallest of the lane's 32 values, three operands per instruction (the accumulators are
                // never signalling NaNs, so the library fminf's quieting moves are left out).
                // The minima of the four runs of eight registers are kept: the filter skips a run in which no
                // lane of the wave has a passing element.
                float run_min[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const v16f &a = g < 2 ? acc0 : acc1;
                    const int o = 8 * (g & 1);
                    float m = matrix_result(a[o + 7]);
                    m = min3(m, a[o], a[o + 1]);
                    m = min3(m, a[o + 2], a[o + 3]);
                    m = min3(m, a[o + 4], a[o + 5]);
                    run_min[g] = min2(m, a[o + 6]);
                }
                const float best = fminf(min3(run_min[0], run_min[1], run_min[2]), run_min[3]);
                // A query meets about K' ln(N / K') passing candidates during the sweep and the 64 lanes
                // serve different queries, so most block pairs have some lane that passes.  A passing lane
                // stores its keys one after the other at the end of its own region of the query's list.
                // The test is on the distance alone; an element that ties with the threshold's distance
                // but not its index is appended too and sorted out by the next compaction.
                if (best <= limit_acc) {
                    const int jbase = c0 + cb * 32 + 4 * kh;  // element (half, v) is candidate jbase + 32 half + 8 (v / 4) + v % 4
                    // Only the last tile has candidates beyond N and only the query's own tile holds the
                    // query: those two tiles knock the excluded elements out by raising them to +inf.
                    if (c0 + kCT > N || (unsigned int)(q0 - c0) < (unsigned int)kCT) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int j = jbase + 8 * (e >> 2) + (e & 3);
                            if (j >= N || j == q) acc0[e] = INFINITY;
                            if (j + 32 >= N || j + 32 == q) acc1[e] = INFINITY;
                        }
                    }
                    const float lim = q < N ? limit_acc : -INFINITY;
                    u64 *const dst0 = list + ((wave * 32 + qn) * cap + kh * half + my_n);
                    u64 *dst = dst0;
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        // (the minima are from before the exclusions above: lower bounds, which is all this needs)
                        if (__ballot(run_min[g] <= lim) == 0) continue;
#pragma unroll
                        for (int v = 0; v < 8; ++v) {
                            const int e = 8 * g + v;
                            const float dist = e < 16 ? acc0[e & 15] : acc1[e & 15];
                            if (dist <= lim) {
                                int jb = jbase;
                                asm volatile("" : "+v"(jb));  // the index is formed here, not held in 32 registers
                                *dst++ = pack_key(BF16 ? dist + off : dist, jb + 32 * (e >> 4) + 8 * ((e & 15) >> 2) + (e & 3));
                            }
                        }
                    }
                    my_n += (int)(dst - dst0);
                }
            };
            // The filter's stores to the lists count among the outstanding memory operations that the wait for
            // the next tile's registers has to see through, so the second block pair is filtered only after the
            // next tile has gone to LDS: what that wait then meets are the first pair's stores, a whole pair of
            // matrix products old.
            v16f acc0, acc1;
            multiply(0, acc0, acc1);
            filter(0, acc0, acc1);
            multiply(2, acc0, acc1);
            __syncthreads();  // all waves are done with tile `buf`
            if (next_ct >= 0) {
                stash(buf);
                __syncthreads();
            }
            filter(2, acc0, acc1);
            // Lists that a further tile could overflow are compacted by their own wave, right away.
            {
                // (a region takes at most 64 entries per tile)
                u64 crowded = __ballot(my_n > half - kCT / 2);
                crowded = (crowded | (crowded >> 32)) & 0xffffffffull;  // lanes l, l+32 share a query
                if (crowded) {
                    fill[tid] = my_n;
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    while (crowded) {
                        const int b = __ffsll((long long)crowded) - 1;
                        crowded &= crowded - 1;
                        select_query(b, args.select_slack, true);
                    }
                    my_n = fill[tid];
                }
            }
        };

        // Phase 1: the query tile's neighbourhood; phase 2: the tiles the bitmap keeps.
        const int T = num_ctiles;
        const int h0 = max(qt - kHomeTiles, 0), h1 = min(qt + kHomeTiles, T - 1);
        int word_idx = -1;
        unsigned int cur_word = 0u;
        // Next set bit of the bitmap, ascending; every wave walks the same words.
        auto next_tile = [&]() -> int {
            while (cur_word == 0u) {
                ++word_idx;
                if (word_idx >= args.bitmap_words) return -1;
                cur_word = bitmap[word_idx];
            }
            const int b = __ffs((int)cur_word) - 1;
            cur_word &= cur_word - 1u;
            return word_idx * 32 + b;
        };
        fetch(h0);
        __syncthreads();
        stash(0);
        __syncthreads();
        bool home = true;
        int cur = h0;
        unsigned int swept = 0;
        while (cur >= 0) {
            ++swept;
            int nxt = home ? (cur < h1 ? cur + 1 : -1) : next_tile();
            process(cur, nxt);
            if (nxt < 0 && home && (h0 > 0 || h1 < T - 1)) {
                home = false;
                // Thresholds from what the neighbourhood held.
                fill[tid] = my_n;
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                for (int b = 0; b < 32; ++b)
                    if (q0 + wave * 32 + b < N) select_query(b, 0, false);
                my_n = fill[tid];
                for (int w = tid; w < args.bitmap_words; w += 256) bitmap[w] = 0u;
                if (tid < D) qcenter[tid] = args.centers_t[(size_t)tid * T + qt];
                __syncthreads();
                if (tid < kMQ) {
                    // Largest squared distance any query of the tile would still accept (rounded up).
                    float v = -INFINITY;
                    if (q0 + tid < N) {
                        const u64 t = thr[tid];
                        v = t == ~0ull ? INFINITY : key_distance(t) + (BF16 ? 0.0f : args.norms[q0 + tid]);
                        v += 1e-5f * fabsf(v) + 1e-30f;
                    }
                    v = group_max<kWave>(v);
                    if (lane == 0) tmax_part[wave] = v;
                }
                __syncthreads();
                const float tmax = fmaxf(tmax_part[0], tmax_part[1]);
                const float ra = args.radius[qt];
                if (args.probe_tile_lists) {
                    // Approximate search: only tiles of probed lists are eligible (the ball test still drops
                    // those among them that cannot matter, which changes nothing in the result).
                    const unsigned int *mine = args.probe_tile_lists + (size_t)qt * args.probe_list_words;
                    for (int l = tid; l < args.probe_nlist; l += 256) {
                        if (!((mine[l >> 5] >> (l & 31)) & 1u)) continue;
                        const int t0 = args.probe_list_tiles[2 * l], t1 = args.probe_list_tiles[2 * l + 1];
                        for (int t = t0; t <= t1; ++t)
                            if ((t < h0 || t > h1) &&
                                tile_may_matter(qcenter, ra, args.centers_t, args.radius, D, T, t, tmax))
                                atomicOr(&bitmap[t >> 5], 1u << (t & 31));
                    }
                } else {
                    for (int t = tid; t < T; t += 256)
                        if ((t < h0 || t > h1) &&
                            tile_may_matter(qcenter, ra, args.centers_t, args.radius, D, T, t, tmax))
                            atomicOr(&bitmap[t >> 5], 1u << (t & 31));
                }
                __syncthreads();
                nxt = next_tile();
                if (nxt >= 0) {
                    fetch(nxt);
                    stash(buf);  // the barrier that ended the last tile freed both buffers
                    __syncthreads();
                }
                // Nothing this block loaded is left in flight as far as the compiler can tell: a load it
                // takes to be possibly outstanding here makes it wait for all loads, the next tile's
                // included, at the first register reuse after process() has issued them.
                __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
            }
            cur = nxt;
        }
        if (tid == 0) atomicAdd(args.tiles_swept, (unsigned long long)swept);
        // Final ordering and output, every wave for its own 32 queries.
        fill[tid] = my_n;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        for (int b = 0; b < 32; ++b) {
            const int ql = wave * 32 + b;
            const int qq = q0 + ql;
            if (qq >= N) break;
            select_query(b, 0, true);
            const int n = fill[wave * 64 + b] + fill[wave * 64 + b + 32];
            const u64 *lq = list + (size_t)ql * cap;  // entry e of the n kept: region e & 1, position e >> 1
            for (int e = lane; e < want; e += kWave)
                cand[(size_t)qq * want + e] = e < n ? key_index(lq[(e & 1) * half + (e >> 1)]) : -1;
            // Every candidate that was dropped, by a compaction or by the filter, had a distance >= the
            // threshold of the moment, and thresholds only decrease.
            if (lane == 0) tau[qq] = thr[ql] == ~0ull ? INFINITY : key_distance(thr[ql]);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
        __syncthreads();  // before the next query tile re-initialises thr / cnt and the LDS tiles
    }
}

// ---------------------------------------------------------------------------
// MFMA sweep for more dimensions than one wave's registers hold (more than 126).
// The k-steps are cut into chunks of kChunkSteps (64 dimensions).  Per candidate tile and chunk the
// workgroup keeps the chunk of the tile in LDS (32 KB, layout [block (4)][step group (8)][lane (64)]
// float4, copied verbatim from the packed points), every wave loads the same chunk of its 32 queries
// from the packed query-side copy (already scaled: -2 q_d, 1 in the |c|^2 row) and the products of
// all four candidate blocks accumulate over the chunks in 64 registers.  The next chunk of the tile
// (or the first of the next tile) and of the queries travel through registers meanwhile.  Visiting
// order, tile skipping, filter, lists and output are those of the kernel above.
// BF16 = true: a chunk is 32 dimensions, 16 KB (two LDS buffers) as [block (4)][term (2)][step of 16 dimensions (2)][lane (64)]
// 8 x bf16 of the points relative to their tile's centre, the query side two terms of -2 q likewise, and the
// products are those of the kernel above (three v_mfma_f32_32x32x16_bf16 per step); |q - centre|^2 is summed
// over the chunks from the query side's two terms and the centre's chunk (pack_chunked_centres_kernel), and
// the keys are lower bounds of the distances as there.
// Dynamic LDS: one tile chunk, one sort buffer (cap keys) per wave, the visit bitmap, D floats
// (centre of the query tile's ball).
// ---------------------------------------------------------------------------
constexpr int kChunkSteps = 32;
constexpr int kChunkS4 = kChunkSteps / 4;            // float4 per lane, block and chunk
constexpr int kChunkFloat4 = 4 * kChunkS4 * 64;      // float4 per tile chunk

template <bool BF16>
__global__ __launch_bounds__(256, 2) void knn_mfma_chunked_sweep_kernel(const SweepArgs args) {
    const int N = args.N, D = args.D, want = args.want, cap = args.cap;
    const int num_qtiles = args.num_qtiles, n_chunks = args.n_chunks;
    u64 *__restrict__ lists = args.lists;
    int *__restrict__ cand = args.cand;
    float *__restrict__ tau = args.tau;
    // Slots of 16 bytes per lane, block and chunk: 8 groups of four k-steps (64 dimensions) on floats; on bf16
    // terms 2 terms x 2 steps of 16 dimensions (32 dimensions: with 64 the chunk loop's registers did not fit
    // and the compiler spilled the prefetched chunks the moment they were loaded).
    constexpr int kSlots = BF16 ? 4 : kChunkS4;
    constexpr int kSteps16 = 2;                     // bf16: steps of 16 dimensions per chunk
    constexpr int kChunkF4 = 4 * kSlots * 64;       // float4 per tile chunk
    // bf16: two LDS buffers of 16 KB, so that the next chunk goes to LDS while the other waves may still read the
    // current one, and one workgroup barrier per chunk does (floats: one buffer of 32 KB, two barriers).
    constexpr int kBufs = BF16 ? 2 : 1;
    int buf = 0;  // the buffer that holds the chunk being computed
    const size_t tile_stride = (size_t)n_chunks * kChunkF4;  // float4 per packed tile
    const size_t block_stride = (size_t)n_chunks * kSlots * 64;  // float4 per 32-point block of a tile
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    v4f *a_lds = reinterpret_cast<v4f *>(lds_raw);
    u64 *sortbuf = reinterpret_cast<u64 *>(a_lds + kBufs * kChunkF4) + (size_t)(threadIdx.x >> 6) * cap;  // per wave
    unsigned int *bitmap = reinterpret_cast<unsigned int *>(reinterpret_cast<u64 *>(a_lds + kBufs * kChunkF4) + 4 * (size_t)cap);
    float *qcenter = reinterpret_cast<float *>(bitmap + args.bitmap_words);
    __shared__ u64 thr[kMQ];
    __shared__ int cnt[kMQ];
    __shared__ unsigned int hist_all[4][kWave];
    __shared__ float tmax_part[2];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int qn = lane & 31, kh = lane >> 5;
    u64 *list = lists + (size_t)blockIdx.x * kMQ * cap;

    // Chunk c of a candidate tile: global -> registers -> LDS.  Element e = 256 r + tid of the chunk is
    // float4 (e % 512) of block e / 512 = r / 2.
    v4f stage[kSlots];
    auto fetch = [&](int tile, int c) {
        const v4f *src = reinterpret_cast<const v4f *>(args.Xp) + (size_t)tile * tile_stride + (size_t)c * (kSlots * 64) + tid;
        // element 256 r + tid of the chunk: block (256 r + tid) / (64 kSlots), float4 (256 r + tid) % (64 kSlots) of it
#pragma unroll
        for (int r = 0; r < kSlots; ++r)
            stage[r] = src[(size_t)((256 * r) / (64 * kSlots)) * block_stride + (256 * r) % (64 * kSlots)];
    };
    auto stash = [&](int b) {
#pragma unroll
        for (int r = 0; r < kSlots; ++r) a_lds[b * kChunkF4 + r * 256 + tid] = stage[r];
    };
    const int num_ctiles = (N + kCT - 1) / kCT;

    const int P = args.parts;
    for (int w = blockIdx.x; w < num_qtiles * P; w += gridDim.x) {
        const int qi = w / P, part = w - qi * P;
        const int qt = args.qtile_list ? args.qtile_list[qi] : args.qtile_first + qi * args.qtile_step;
        const int q0 = qt * kMQ;
        const int q = q0 + wave * 32 + qn;  // this lane's query (>= N in the last tile: padded zeros)
        if (tid < kMQ) {
            thr[tid] = ~0ull;
            cnt[tid] = 0;
        }
        const float q_len = BF16 && q < N ? sqrtf(args.norms[q]) * (1.0f + 1e-6f) : 0.0f;  // |q|, rounded up
        // This wave's block of the query-side copy.
        const v4f *bsrc = reinterpret_cast<const v4f *>(args.Bp) + (size_t)qt * tile_stride + (size_t)wave * block_stride + lane;
        v4f bcur[kSlots], bnext[kSlots];
#pragma unroll
        for (int s4 = 0; s4 < kSlots; ++s4) bcur[s4] = bsrc[s4 * 64];

        // One tile: its first chunk is in LDS and the queries' first chunk in bcur on entry; the same holds
        // for next_ct on exit.
        auto process = [&](int ct, int next_ct) {
            const int c0 = ct * kCT;
            v16f acc[4];
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[b][e] = 0.0f;
            float f_part = 0.0f;  // bf16: this lane's share of |q - m|^2 (m: the tile's centre)
            for (int c = 0; c < n_chunks; ++c) {
                const bool last = c + 1 == n_chunks;
                v4f mc[2 * kSteps16];  // bf16: the centre's 16 coordinates that go with this lane's 16 of the chunk
                if constexpr (BF16) {
                    const v4f *msrc = reinterpret_cast<const v4f *>(args.centres_p) + (size_t)ct * (8 * n_chunks) + 8 * c + 2 * kh;
#pragma unroll
                    for (int step = 0; step < kSteps16; ++step) {
                        mc[2 * step] = msrc[4 * step];
                        mc[2 * step + 1] = msrc[4 * step + 1];
                    }
                }
                if (!last) fetch(ct, c + 1);
                else if (next_ct >= 0) fetch(next_ct, 0);
                {
                    const v4f *bn = bsrc + (size_t)(last ? 0 : c + 1) * (kSlots * 64);
#pragma unroll
                    for (int s4 = 0; s4 < kSlots; ++s4) bnext[s4] = bn[s4 * 64];
                }
                if constexpr (BF16) {
#pragma unroll
                    for (int step = 0; step < kSteps16; ++step) {
                        v4f xh[4], xl[4];
#pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            xh[b] = a_lds[buf * kChunkF4 + (b * kSlots + step) * 64 + lane];
                            xl[b] = a_lds[buf * kChunkF4 + (b * kSlots + kSteps16 + step) * 64 + lane];
                        }
                        const v8bf qh = __builtin_bit_cast(v8bf, bcur[step]), ql = __builtin_bit_cast(v8bf, bcur[kSteps16 + step]);
#pragma unroll
                        for (int b = 0; b < 4; ++b)
                            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, xh[b]), qh, acc[b], 0, 0, 0);
#pragma unroll
                        for (int b = 0; b < 4; ++b)
                            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, xh[b]), ql, acc[b], 0, 0, 0);
#pragma unroll
                        for (int b = 0; b < 4; ++b)
                            acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, xl[b]), qh, acc[b], 0, 0, 0);
                        // |q - m|^2 from the query's two terms: q_d = -(high + low) / 2 to within 2^-16 |q_d|.
                        const uint4 uh = __builtin_bit_cast(uint4, bcur[step]), ul = __builtin_bit_cast(uint4, bcur[kSteps16 + step]);
                        const unsigned int wh[4] = {uh.x, uh.y, uh.z, uh.w}, wl[4] = {ul.x, ul.y, ul.z, ul.w};
                        const float m[8] = {mc[2 * step][0], mc[2 * step][1], mc[2 * step][2], mc[2 * step][3],
                                            mc[2 * step + 1][0], mc[2 * step + 1][1], mc[2 * step + 1][2], mc[2 * step + 1][3]};
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const float s0 = __uint_as_float(wh[k] << 16) + __uint_as_float(wl[k] << 16);
                            const float s1 = __uint_as_float(wh[k] & 0xffff0000u) + __uint_as_float(wl[k] & 0xffff0000u);
                            const float e0 = fmaf(-0.5f, s0, -m[2 * k]), e1 = fmaf(-0.5f, s1, -m[2 * k + 1]);
                            f_part = fmaf(e0, e0, f_part);
                            f_part = fmaf(e1, e1, f_part);
                        }
                    }
                } else {
#pragma unroll
                    for (int s4 = 0; s4 < kChunkS4; ++s4) {
                        v4f x[4];
#pragma unroll
                        for (int b = 0; b < 4; ++b) x[b] = a_lds[(b * kChunkS4 + s4) * 64 + lane];
#pragma unroll
                        for (int k = 0; k < 4; ++k)
#pragma unroll
                            for (int b = 0; b < 4; ++b)
                                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(x[b][k], bcur[s4][k], acc[b], 0, 0, 0);
                    }
                }
                if (!last) {
                    if constexpr (BF16) {
                        stash(buf ^ 1);  // (last read a chunk ago, before the barrier that ended that chunk)
                        __syncthreads();
                        buf ^= 1;
                    } else {
                        __syncthreads();  // all waves have read this chunk
                        stash(0);
                        __syncthreads();
                    }
#pragma unroll
                    for (int s4 = 0; s4 < kSlots; ++s4) bcur[s4] = bnext[s4];
                }
            }
            const u64 limit = thr[wave * 32 + qn];
            // ~0 is "no threshold yet": its distance field does not decode to a number.
            const float limit_d = limit == ~0ull ? INFINITY : key_distance(limit);
            // Never +inf: excluded elements are raised to +inf and must fail the test also while the query
            // has no threshold yet (a part can hold fewer than `want` real candidates, so nothing would
            // push them out of the list later).
            // bf16: the keys are lower bounds of the distances: product + `off`, off = |q - m|^2 rounded down
            // (the rounding of its sum, and the 2^-16 |q| by which the query's two terms miss q) less the tile's
            // error bound; the products are tested against the threshold less `off`, rounded up.
            float off = 0.0f, limit_acc = limit_d;
            if constexpr (BF16) {
                const float f = f_part + __shfl_xor(f_part, 32);
                off = f * (1.0f - (float)(D + 4) * 5.9604644775390625e-08f) - 2.1f / 65536.0f * q_len * sqrtf(f) -
                      fmaf(q_len, args.tile_coef[2 * ct], args.tile_coef[2 * ct + 1]);
                limit_acc = limit_d - off;
                limit_acc += 2.4e-7f * (fabsf(limit_d) + fabsf(off));
            }
            const float lim = q < N ? fminf(limit_acc, 3.4028234663852886e38f) : -INFINITY;
            const bool edge_tile = c0 + kCT > N || (unsigned int)(q0 - c0) < (unsigned int)kCT;
#pragma unroll
            for (int cb = 0; cb < 4; cb += 2) {
                v16f &acc0 = acc[cb], &acc1 = acc[cb + 1];
                // Register v of lane l holds candidate row 8*(v/4) + 4*(l/32) + v%4 of the block, query column l%32.
                float best = matrix_result(acc0[0]);
#pragma unroll
                for (int v = 1; v + 1 < 16; v += 2) best = min3(best, acc0[v], acc0[v + 1]);
                best = min3(best, acc0[15], matrix_result(acc1[0]));
#pragma unroll
                for (int v = 1; v + 1 < 16; v += 2) best = min3(best, acc1[v], acc1[v + 1]);
                best = min2(best, acc1[15]);
                if (best <= limit_acc) {
                    const int jbase = c0 + cb * 32 + 4 * kh;  // element (half, v) is candidate jbase + 32 half + 8 (v / 4) + v % 4
                    // Candidates beyond N (last tile) and the query itself (its own tile) are raised to +inf.
                    if (edge_tile) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int j = jbase + 8 * (e >> 2) + (e & 3);
                            if (j >= N || j == q) acc0[e] = INFINITY;
                            if (j + 32 >= N || j + 32 == q) acc1[e] = INFINITY;
                        }
                    }
                    // Count, reserve the list slots with one LDS atomic, then store the keys.
                    int n = 0;
#pragma unroll
                    for (int e = 0; e < 32; ++e) n += ((e < 16 ? acc0[e & 15] : acc1[e & 15]) <= lim) ? 1 : 0;
                    if (n != 0) {
                        const int slot = atomicAdd(&cnt[wave * 32 + qn], n);
                        u64 *dst = list + (size_t)(wave * 32 + qn) * cap + slot;
                        float lim2 = lim;
                        asm volatile("" : "+v"(lim2));  // compare again rather than keep 32 lane masks alive
#pragma unroll
                        for (int e = 0; e < 32; ++e) {
                            const float dist = e < 16 ? acc0[e & 15] : acc1[e & 15];
                            if (dist <= lim2)
                                *dst++ = pack_key(BF16 ? dist + off : dist, jbase + 32 * (e >> 4) + 8 * ((e & 15) >> 2) + (e & 3));
                        }
                    }
                }
            }
            // Lists that a further tile could overflow are compacted by their own wave, right away.
            {
                u64 crowded = __ballot(cnt[wave * 32 + qn] > args.trigger) & 0xffffffffull;  // lanes l, l+32 share a query
                while (crowded) {
                    const int ql = wave * 32 + (__ffsll((long long)crowded) - 1);
                    crowded &= crowded - 1;
                    wave_select(list + (size_t)ql * cap, want, &cnt[ql], &thr[ql], sortbuf, hist_all[wave], lane,
                                args.select_slack);
                }
            }
            if constexpr (BF16) {
                if (next_ct >= 0) stash(buf ^ 1);
                __syncthreads();  // the next tile's first chunk is in LDS; all waves are done with this tile's last
                if (next_ct >= 0) buf ^= 1;
            } else {
                __syncthreads();  // all waves are done with the tile's last chunk
                if (next_ct >= 0) {
                    stash(0);
                    __syncthreads();
                }
            }
#pragma unroll
            for (int s4 = 0; s4 < kSlots; ++s4) bcur[s4] = bnext[s4];
        };

        // Phase 1: the query tile's neighbourhood; phase 2: the tiles the bitmap keeps.
        const int T = num_ctiles;
        const int h0 = max(qt - kHomeTiles * P, 0), h1 = min(qt + kHomeTiles * P, T - 1);  // >= kHomeTiles tiles of every part
        int word_idx = -1;
        unsigned int cur_word = 0u;
        auto next_tile = [&]() -> int {
            while (cur_word == 0u) {
                ++word_idx;
                if (word_idx >= args.bitmap_words) return -1;
                cur_word = bitmap[word_idx];
            }
            const int b = __ffs((int)cur_word) - 1;
            cur_word &= cur_word - 1u;
            return word_idx * 32 + b;
        };
        int cur = h0 + (part - h0 % P + P) % P;  // this part's first tile of the neighbourhood
        if (cur > h1) cur = -1;  // fewer tiles than parts: nothing for this part, its lists stay empty
        if (cur >= 0) fetch(cur, 0);
        __syncthreads();  // the previous query tile's last reads of the LDS chunk
        buf = 0;
        if (cur >= 0) stash(0);
        __syncthreads();
        bool home = true;
        unsigned int swept = 0;
        while (cur >= 0) {
            ++swept;
            int nxt = home ? (cur + P <= h1 ? cur + P : -1) : next_tile();
            process(cur, nxt);
            if (nxt < 0 && home && (h0 > 0 || h1 < T - 1)) {
                home = false;
                for (int b = 0; b < 32; ++b) {
                    const int ql = wave * 32 + b;
                    if (q0 + ql < N)
                        wave_select(list + (size_t)ql * cap, want, &cnt[ql], &thr[ql], sortbuf, hist_all[wave], lane);
                }
                for (int w = tid; w < args.bitmap_words; w += 256) bitmap[w] = 0u;
                for (int d = tid; d < D; d += 256) qcenter[d] = args.centers_t[(size_t)d * T + qt];
                __syncthreads();
                if (tid < kMQ) {
                    // Largest squared distance any query of the tile would still accept (rounded up).
                    float v = -INFINITY;
                    if (q0 + tid < N) {
                        const u64 t = thr[tid];
                        v = t == ~0ull ? INFINITY : key_distance(t) + (BF16 ? 0.0f : args.norms[q0 + tid]);
                        v += 1e-5f * fabsf(v) + 1e-30f;
                    }
                    v = group_max<kWave>(v);
                    if (lane == 0) tmax_part[wave] = v;
                }
                __syncthreads();
                const float tmax = fmaxf(tmax_part[0], tmax_part[1]);
                const float ra = args.radius[qt];
                for (int t = tid; t < T; t += 256)
                    if ((t < h0 || t > h1) && t % P == part &&
                        tile_may_matter(qcenter, ra, args.centers_t, args.radius, D, T, t, tmax))
                        atomicOr(&bitmap[t >> 5], 1u << (t & 31));
                __syncthreads();
                nxt = next_tile();
                if (nxt >= 0) {
                    fetch(nxt, 0);
                    stash(buf);  // the barrier that ended the last tile freed the LDS chunks
                    __syncthreads();
                }
                __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), as in the kernel above
            }
            cur = nxt;
        }
        if (tid == 0) atomicAdd(args.tiles_swept, (unsigned long long)swept);
        // Final ordering and output, every wave for its own 32 queries.
        for (int b = 0; b < 32; ++b) {
            const int ql = wave * 32 + b;
            const int qq = q0 + ql;
            if (qq >= N) break;
            const int n = wave_select(list + (size_t)ql * cap, want, &cnt[ql], &thr[ql], sortbuf, hist_all[wave], lane);
            const size_t row = (size_t)qi * kMQ + ql;
            if (P == 1) {
                for (int e = lane; e < want; e += kWave)
                    cand[row * want + e] = e < n ? key_index(list[(size_t)ql * cap + e]) : -1;
                if (lane == 0) tau[row] = thr[ql] == ~0ull ? INFINITY : key_distance(thr[ql]);
            } else {
                u64 *dst = args.part_keys + (row * P + part) * want;
                for (int e = lane; e < want; e += kWave) dst[e] = e < n ? list[(size_t)ql * cap + e] : ~0ull;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
        __syncthreads();  // before the next query tile re-initialises thr / cnt and the LDS chunk
    }
}

// ---------------------------------------------------------------------------
// Merge of the parts of the chunked sweep: the `want` best keys of a query's parts * want, exactly what
// a single list would have kept (every part kept its own `want` best), and their threshold.  One wave
// per query row, four rows per workgroup.  Dynamic LDS: 4 x parts * want keys.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void knn_merge_parts_kernel(u64 *__restrict__ part_keys, int parts, int want,
                                                              int n_rows, int *__restrict__ cand,
                                                              float *__restrict__ tau) {
    extern __shared__ u64 merge_buf[];
    __shared__ unsigned int hist_all[4][kWave];
    __shared__ u64 thr[4];
    __shared__ int cnt[4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + wave;
    if (row >= n_rows) return;  // no workgroup barrier below
    const int total = parts * want;
    u64 *list = part_keys + (size_t)row * total;
    if (lane == 0) {
        thr[wave] = ~0ull;
        cnt[wave] = total;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    // The filler keys sort last; a threshold with all distance bits set means "fewer than `want` candidates".
    wave_select(list, want, &cnt[wave], &thr[wave], merge_buf + (size_t)wave * total, hist_all[wave], lane);
    for (int e = lane; e < want; e += kWave) cand[(size_t)row * want + e] = key_index(list[e]);
    if (lane == 0) tau[row] = (thr[wave] >> 32) == 0xffffffffull ? INFINITY : key_distance(thr[wave]);
}

// ---------------------------------------------------------------------------
// Re-rank: canonical distances of a query's candidates, sort by (distance,
// index), verify, write.  One wave per query, four queries per workgroup.
// Dynamic LDS: 4 x sort_n keys.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void knn_rerank_kernel(const float *__restrict__ X,
                                                         const float *__restrict__ norms, int N, int D, int K,
                                                         int want, int sort_n, const int *__restrict__ cand,
                                                         const float *__restrict__ tau,
                                                         const float *__restrict__ max_norm,
                                                         int *__restrict__ out_idx, float *__restrict__ out_d,
                                                         int *__restrict__ fail_count, int *__restrict__ fail_list,
                                                         const int *__restrict__ qtile_list, int qtile_first,
                                                         int qtile_step, int n_slots, int lower_bounds) {
    extern __shared__ u64 keys_all[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // Query slot w belongs to query tile qtile_list[w / kMQ], or first + (w / kMQ) step without a list
    // (all queries: first 0, step 1).  cand holds `want` candidates per slot, tau one threshold.
    const int w = blockIdx.x * 4 + wave;
    const int wt = w < n_slots ? w / kMQ : 0;
    const int q = (qtile_list ? qtile_list[wt] : qtile_first + wt * qtile_step) * kMQ + (w % kMQ);
    u64 *keys = keys_all + (size_t)wave * sort_n;
    const bool live = w < n_slots && q < N;
    const float *xq = X + (size_t)(live ? q : 0) * D;
    for (int c = lane; c < sort_n; c += kWave) {
        u64 key = ~0ull;
        if (live && c < want) {
            const int j = cand[(size_t)w * want + c];
            if (j >= 0) {
                const float *xj = X + (size_t)j * D;
                float acc = 0.0f;
                if ((D & 3) == 0 && D >= 64 && (reinterpret_cast<uintptr_t>(X) & 15) == 0) {
                    // Long rows, 16-byte aligned: 128 bytes of the candidate's row per lane and step, so that a
                    // cache line is used whole by the load that fetches it (the lanes walk 64 different rows);
                    // the same fma chain.
                    const v4f *q4 = reinterpret_cast<const v4f *>(xq);
                    const v4f *j4 = reinterpret_cast<const v4f *>(xj);
                    const int n4 = D / 4;
                    int d4 = 0;
                    for (; d4 + 8 <= n4; d4 += 8) {
                        v4f b[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u) b[u] = j4[d4 + u];
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const v4f a = q4[d4 + u];
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                const float df = a[k] - b[u][k];
                                acc = fmaf(df, df, acc);
                            }
                        }
                    }
                    for (; d4 < n4; ++d4) {
                        const v4f a = q4[d4], b = j4[d4];
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const float df = a[k] - b[k];
                            acc = fmaf(df, df, acc);
                        }
                    }
                } else if ((D & 1) == 0 && (reinterpret_cast<uintptr_t>(X) & 7) == 0) {
                    // rows are 8-byte aligned: two dimensions per load, the same fma chain
                    const float2 *q2 = reinterpret_cast<const float2 *>(xq);
                    const float2 *j2 = reinterpret_cast<const float2 *>(xj);
                    const int n2 = D / 2;
                    int d = 0;
                    // eight loads (64 bytes of the candidate's row) in flight per lane
                    for (; d + 8 <= n2; d += 8) {
                        float2 b[8];
#pragma unroll
                        for (int u = 0; u < 8; ++u) b[u] = j2[d + u];
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            const float2 a = q2[d + u];
                            const float d0 = a.x - b[u].x, d1 = a.y - b[u].y;
                            acc = fmaf(d0, d0, acc);
                            acc = fmaf(d1, d1, acc);
                        }
                    }
                    for (; d < n2; ++d) {
                        const float2 a = q2[d], b = j2[d];
                        const float d0 = a.x - b.x, d1 = a.y - b.y;
                        acc = fmaf(d0, d0, acc);
                        acc = fmaf(d1, d1, acc);
                    }
                } else {
                    for (int d = 0; d < D; ++d) {
                        const float df = xq[d] - xj[d];
                        acc = fmaf(df, df, acc);
                    }
                }
                key = pack_key(acc, j);
            }
        }
        keys[c] = key;
    }
    // Bitonic sort of each wave's own keys: no workgroup barrier, a wave's LDS operations execute in
    // order and the wavefront fences only keep the compiler from reordering them.
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    for (int k = 2; k <= sort_n; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int t = lane; t < sort_n / 2; t += kWave) {
                const int lo = ((t & ~(j - 1)) << 1) | (t & (j - 1));
                const int hi = lo | j;
                const bool up = (lo & k) == 0;
                const u64 a = keys[lo], b = keys[hi];
                if ((a > b) == up) {
                    keys[lo] = b;
                    keys[hi] = a;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
    }
    if (!live) return;
    // Sweep on floats: every candidate outside the list has an approximate distance >= tau (without
    // |q|^2), so its canonical distance is >= tau + |q|^2 - g.  g bounds |approximate - canonical|: both are
    // sums of at most D + 3 rounded terms of magnitude <= (|q| + |c|)^2, and the canonical distance carries
    // a relative error of (D + 2) 2^-24 of itself; a factor of four covers the matrix unit's
    // accumulation order and the rounding of the stored norms.
    // Sweep on bf16 terms (lower_bounds): the sweep's keys are lower bounds of the distances, so every
    // candidate outside the list has a distance >= tau, and a canonical distance within (D + 2) 2^-24 of that.
    const float kth = key_distance(keys[K - 2]);
    const float t = tau[w];
    bool pass = isinf(t) && t > 0.0f;
    if (!pass) {
        const double eps = 5.9604644775390625e-08;  // 2^-24
        if (lower_bounds) {
            pass = (double)kth + (D + 4) * eps * ((double)kth + fabs((double)t)) < (double)t;
        } else {
            const double nq = norms[q], nmax = *max_norm;
            const double g = 4.0 * (D + 4) * eps * (nq + nmax + 2.0 * sqrt(nq * nmax)) + (D + 4) * eps * (double)kth;
            pass = (double)kth < (double)t + nq - g;
        }
    }
    if (pass) {
        for (int e = lane; e < K; e += kWave) {
            out_idx[(size_t)q * K + e] = e == 0 ? q : key_index(keys[e - 1]);
            out_d[(size_t)q * K + e] = e == 0 ? 0.0f : key_distance(keys[e - 1]);
        }
    } else if (lane == 0) {
        fail_list[atomicAdd(fail_count, 1)] = q;
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

struct DeviceMem {
    void *p = nullptr;
    ~DeviceMem() {
        if (p) (void)hipFree(p);
    }
    bool alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1) == hipSuccess; }
    template <typename T>
    T *as() const {
        return static_cast<T *>(p);
    }
};

int next_pow2(int v) {
    int n = 1;
    while (n < v) n <<= 1;
    return n;
}

template <int KSTEPS, bool BF16>
int launch_mfma_sweep(const SweepArgs &args, int grid, hipStream_t s) {
    constexpr int S4 = BF16 ? 2 * KSTEPS : (KSTEPS + 3) / 4;
    // one tile (bf16: with its centre block) + a sort buffer per wave + the visit bitmap
    const size_t lds = sizeof(float4) * (4 * S4 * 64 + (BF16 ? 64 : 0)) + sizeof(u64) * 4 * args.cap +
                       sizeof(unsigned int) * args.bitmap_words;
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(knn_mfma_sweep_kernel<KSTEPS, BF16>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    knn_mfma_sweep_kernel<KSTEPS, BF16><<<grid, 256, lds, s>>>(args);
    TSNE_TRY(hipGetLastError());
    return 0;
}

// Steps of 16 dimensions of the bf16 sweep: up to 125 dimensions + the three |c|^2 terms.
int dispatch_bf16_sweep(int steps, const SweepArgs &args, int grid, hipStream_t s) {
    switch (steps) {
        case 1: return launch_mfma_sweep<1, true>(args, grid, s);
        case 2: return launch_mfma_sweep<2, true>(args, grid, s);
        case 3: return launch_mfma_sweep<3, true>(args, grid, s);
        case 4: return launch_mfma_sweep<4, true>(args, grid, s);
        case 5: return launch_mfma_sweep<5, true>(args, grid, s);
        case 6: return launch_mfma_sweep<6, true>(args, grid, s);
        case 7: return launch_mfma_sweep<7, true>(args, grid, s);
        case 8: return launch_mfma_sweep<8, true>(args, grid, s);
        default:
            set_error("knn: no bf16 matrix-instruction sweep for %d steps", steps);
            return 1;
    }
}


// Instantiated step counts: every count up to 32 (62 dimensions), then multiples of 4.
int dispatch_mfma_sweep(int ksteps, const SweepArgs &args, int grid, hipStream_t s) {
#define TSNE_MFMA_CASE(KS) \
    case KS:               \
        return launch_mfma_sweep<KS, false>(args, grid, s);
    switch (ksteps) {
        TSNE_MFMA_CASE(2) TSNE_MFMA_CASE(3) TSNE_MFMA_CASE(4) TSNE_MFMA_CASE(5) TSNE_MFMA_CASE(6)
        TSNE_MFMA_CASE(7) TSNE_MFMA_CASE(8) TSNE_MFMA_CASE(9) TSNE_MFMA_CASE(10) TSNE_MFMA_CASE(11)
        TSNE_MFMA_CASE(12) TSNE_MFMA_CASE(13) TSNE_MFMA_CASE(14) TSNE_MFMA_CASE(15) TSNE_MFMA_CASE(16)
        TSNE_MFMA_CASE(17) TSNE_MFMA_CASE(18) TSNE_MFMA_CASE(19) TSNE_MFMA_CASE(20) TSNE_MFMA_CASE(21)
        TSNE_MFMA_CASE(22) TSNE_MFMA_CASE(23) TSNE_MFMA_CASE(24) TSNE_MFMA_CASE(25) TSNE_MFMA_CASE(26)
        TSNE_MFMA_CASE(27) TSNE_MFMA_CASE(28) TSNE_MFMA_CASE(29) TSNE_MFMA_CASE(30) TSNE_MFMA_CASE(31)
        TSNE_MFMA_CASE(32) TSNE_MFMA_CASE(36) TSNE_MFMA_CASE(40) TSNE_MFMA_CASE(44) TSNE_MFMA_CASE(48)
        TSNE_MFMA_CASE(52) TSNE_MFMA_CASE(56) TSNE_MFMA_CASE(60) TSNE_MFMA_CASE(64)
        default:
            set_error("knn: no matrix-instruction sweep for %d steps", ksteps);
            return 1;
    }
#undef TSNE_MFMA_CASE
}

int valu_cap(int K) {
    int cap = 256;
    while (cap < K - 1 + kCT) cap <<= 1;
    return cap;
}

// VALU sweep over all points (qlist == nullptr) or over the nq listed queries.
int run_valu_sweep(const float *points, const float *Xt, int N, int Npad, int D, int K, const int *qlist, int nq,
                   int cus, int *indices, float *sq_dist, hipStream_t s) {
    const int cap = valu_cap(K);
    const int num_qtiles = div_up(nq, kQT);
    // A few listed queries: cut the candidates into ranges so that the whole chip works on them (as many
    // ranges as keep about four workgroups per CU busy, the merge's sort within 8192 keys, and at least one
    // candidate tile per range).
    int slices = 1;
    if (qlist != nullptr && K > 1)
        while (slices < 64 && num_qtiles * slices * 2 <= 4 * cus && slices * 2 * (K - 1) <= 8192 &&
               slices * 2 <= div_up(N, kCT))
            slices *= 2;
    const int grid = std::min(num_qtiles * slices, cus * 3);
    // Tile balls for skipping far-away candidate tiles: only when all queries are swept and the
    // neighbourhood that is always swept does not cover everything anyway.
    const int T = div_up(N, kCT);
    const bool prune = qlist == nullptr && T > 2 * kHomeTiles + 1;
    const int bitmap_words = prune ? div_up(T, 32) : 0;
    DeviceMem lists, centers, radius, slice_keys;
    if (!lists.alloc(sizeof(u64) * (size_t)grid * kQT * cap) ||
        (slices > 1 && !slice_keys.alloc(sizeof(u64) * (size_t)num_qtiles * kQT * slices * (K - 1))) ||
        (prune && (!centers.alloc(sizeof(float) * (size_t)D * T) || !radius.alloc(sizeof(float) * T)))) {
        set_error("knn: out of device memory for the candidate lists");
        return 1;
    }
    if (prune) {
        tile_balls_kernel<<<T, 128, sizeof(float) * D, s>>>(points, N, D, T, centers.as<float>(), radius.as<float>());
        TSNE_TRY(hipGetLastError());
    }
    const size_t lds = sizeof(u64) * cap + (prune ? sizeof(float) * D + sizeof(unsigned int) * bitmap_words : 0);
    knn_sweep_kernel<<<grid, 256, lds, s>>>(Xt, N, Npad, D, K, cap, lists.as<u64>(), num_qtiles, qlist, nq, indices,
                                            sq_dist, centers.as<float>(), radius.as<float>(), bitmap_words, slices,
                                            slice_keys.as<u64>());
    TSNE_TRY(hipGetLastError());
    if (slices > 1) {
        int sort_n = 256;
        while (sort_n < slices * (K - 1)) sort_n <<= 1;
        knn_merge_slices_kernel<<<nq, 256, sizeof(u64) * sort_n, s>>>(slice_keys.as<u64>(), slices, K, sort_n, qlist,
                                                                     indices, sq_dist);
        TSNE_TRY(hipGetLastError());
    }
    TSNE_TRY(hipStreamSynchronize(s));
    return 0;
}

}  // namespace

// mode: 0 = choose, 1 = VALU sweep only, 2 = matrix-instruction sweep (error if the shape does not fit),
// 3 = as 2 with the products on floats where 2 multiplies bf16 terms (every dimension count but 126).
// stats (optional, 3 ints): [0] = 1 if the matrix-instruction sweep ran, [1] = queries redone by the VALU sweep,
// [2] = per mille of the (query tile, candidate tile) pairs the matrix sweep computed.
int run_knn_mode(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s, int mode,
                 int *stats, const KnnProbes *probes) {
    if (stats) stats[0] = stats[1] = stats[2] = 0;
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
    if (valu_cap(K) > 4096) {
        set_error("knn: num_neighbors = %d is not supported (limit %d)", K, 4096 - kCT + 1);
        return 1;
    }
    int device = 0, cus = 256;
    TSNE_TRY(hipGetDevice(&device));
    TSNE_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));

    // Matrix-instruction sweep geometry.
    const int Dnorm = (D + 1) & ~1;        // |x|^2 row: first even row after the real dimensions
    int ksteps = (Dnorm + 2) / 2;          // k-steps incl. the augmented pair
    const bool chunked = ksteps > kMfmaMaxSteps;  // more dimensions than one wave's registers hold
    // Unless mode 3 asks for products of floats, the sweeps multiply bf16 terms (two per coordinate) of the
    // points relative to their tile's centre; three more dimensions carry a per-point term.
    const bool force_f32 = mode == 3;
    if (mode == 3) mode = 2;
    const bool bf16 = !chunked && !force_f32 && D + 3 <= 128;
    const bool bf16_chunked = chunked && !force_f32;
    const int n_chunks = chunked ? (bf16_chunked ? div_up(D + 3, 32) : div_up(ksteps, kChunkSteps)) : 0;
    if (chunked) ksteps = n_chunks * (bf16_chunked ? kChunkSteps / 2 : kChunkSteps);  // (slots of 16 bytes per lane x 4)
    else if (ksteps > 32) ksteps = (ksteps + 3) & ~3;
    const int steps16 = div_up(D + 3, 16);
    const int num_tiles = div_up(N, kCT);
    const int bitmap_words = div_up(num_tiles, 32);
    // Room for the candidates kept, as many again and one more tile where the LDS sort buffers of that
    // size fit: a list that is nearly full right after a selection would be selected again after every tile.
    const size_t tile_lds = chunked ? sizeof(float4) * kChunkFloat4 + sizeof(float) * D  // (bf16: two chunks of half the size)
                                    : sizeof(float4) * (bf16 ? 512 * steps16 + 64 : 4 * ((ksteps + 3) / 4) * 64);
    auto lds_with = [&](int cap) -> size_t {
        return tile_lds + sizeof(u64) * 4 * cap + sizeof(unsigned int) * bitmap_words;
    };
    auto list_cap = [&](int want) {
        int cap = next_pow2(2 * want + kCT);
        if (cap > 4096 || lds_with(cap) > 150 * 1024) cap = next_pow2(want + kCT);
        return cap < 256 ? 256 : cap;
    };
    auto sweep_lds = [&](int want) -> size_t { return lds_with(list_cap(want)); };
    auto sweep_fits = [&](int want) { return list_cap(want) <= 4096 && sweep_lds(want) <= 150 * 1024; };
    int want = std::min(N - 1, (K - 1) + std::max(32, (K - 1) / 2));  // K' candidates kept per query
    const bool mfma_fits = sweep_fits(want);
    bool use_mfma = mode == 2 || (mode == 0 && mfma_fits && N >= 8192);
    if (mode == 2 && !mfma_fits) {
        set_error("knn: the matrix-instruction sweep does not fit %d dimensions / %d neighbours", D, K);
        return kShapeNotSupported;
    }
    if (probes && (!use_mfma || chunked)) {
        set_error("knn: the approximate search runs on the register-resident matrix sweep only (at most 126 "
                  "dimensions; got %d dimensions, %d neighbours)", D, K);
        return kShapeNotSupported;
    }

    const int Npad = div_up(N, kCT) * kCT;
    // Transposed points for the vector sweep (built only when that sweep runs).
    DeviceMem Xt;
    auto build_transposed = [&]() -> int {
        if (!Xt.alloc(sizeof(float) * (size_t)D * Npad)) {
            set_error("knn: out of device memory for the transposed points");
            return 1;
        }
        dim3 tgrid(div_up(Npad, 32), div_up(D, 32));
        transpose_points_kernel<<<tgrid, 256, 0, s>>>(points, N, D, Npad, Xt.as<float>());
        TSNE_TRY(hipGetLastError());
        return 0;
    };
    if (!use_mfma) {
        if (build_transposed()) return 1;
        return run_valu_sweep(points, Xt.as<float>(), N, Npad, D, K, nullptr, N, cus, indices, sq_dist, s);
    }

    const int S4 = bf16 ? 2 * steps16 : (ksteps + 3) / 4;  // 16-byte slots per lane and block of the packed points
    DeviceMem Xp, Bp, norms, scal, fail_list, centers, radius;
    const int num_qtiles = div_up(N, kMQ);
    const size_t tile_float4 = bf16 ? 512 * (size_t)steps16 + 64 : (size_t)kCT * S4 * 2;  // float4 per packed tile
    if (!Xp.alloc(sizeof(float4) * tile_float4 * num_tiles) || !norms.alloc(sizeof(float) * Npad) ||
        (chunked && !Bp.alloc(sizeof(float4) * (size_t)Npad * S4 * 2)) ||
        !scal.alloc(4 * sizeof(int)) || !fail_list.alloc(sizeof(int) * N) ||
        !centers.alloc(sizeof(float) * (size_t)D * num_tiles) || !radius.alloc(sizeof(float) * num_tiles)) {
        set_error("knn: out of device memory for the candidate buffers");
        return 1;
    }
    TSNE_TRY(hipMemsetAsync(scal.p, 0, 4 * sizeof(int), s));  // [0] max |x|^2 (float bits), [1] fail count, [2..3] tiles swept (64-bit)
    norms_kernel<<<div_up(Npad, 256), 256, 0, s>>>(points, N, D, Npad, norms.as<float>(), scal.as<float>());
    TSNE_TRY(hipGetLastError());
    if (!bf16 && !bf16_chunked) {
        pack_points_kernel<<<div_up((int64_t)Npad * S4 * 2, 256), 256, 0, s>>>(points, norms.as<float>(), N, D, Dnorm,
                                                                              S4, Npad, Xp.as<float4>(), false);
        TSNE_TRY(hipGetLastError());
    }
    if (chunked && !bf16_chunked) {
        pack_points_kernel<<<div_up((int64_t)Npad * S4 * 2, 256), 256, 0, s>>>(points, norms.as<float>(), N, D, Dnorm,
                                                                              S4, Npad, Bp.as<float4>(), true);
        TSNE_TRY(hipGetLastError());
    }
    tile_balls_kernel<<<num_tiles, 128, sizeof(float) * D, s>>>(points, N, D, num_tiles, centers.as<float>(),
                                                               radius.as<float>());
    TSNE_TRY(hipGetLastError());
    if (bf16) {
        pack_points_bf16_kernel<<<div_up((int64_t)Npad * steps16 * 4, 256), 256, 0, s>>>(
            points, centers.as<float>(), N, D, steps16, num_tiles, Npad, Xp.as<uint4>());
        TSNE_TRY(hipGetLastError());
        pack_tile_centres_kernel<<<num_tiles, 64, 0, s>>>(centers.as<float>(), radius.as<float>(), D, steps16,
                                                         num_tiles, Xp.as<float4>());
        TSNE_TRY(hipGetLastError());
    }
    DeviceMem centres_p, tile_coef;
    if (bf16_chunked) {
        if (!centres_p.alloc(sizeof(float) * 32 * (size_t)n_chunks * num_tiles) ||
            !tile_coef.alloc(sizeof(float) * 2 * (size_t)num_tiles)) {
            set_error("knn: out of device memory for the tile centres");
            return 1;
        }
        const int64_t pieces = (int64_t)Npad * n_chunks * 8;
        pack_points_bf16_chunked_kernel<<<div_up(pieces, 256), 256, 0, s>>>(points, centers.as<float>(), N, D, n_chunks,
                                                                           num_tiles, Npad, Xp.as<uint4>(), false);
        TSNE_TRY(hipGetLastError());
        pack_points_bf16_chunked_kernel<<<div_up(pieces, 256), 256, 0, s>>>(points, centers.as<float>(), N, D, n_chunks,
                                                                           num_tiles, Npad, Bp.as<uint4>(), true);
        TSNE_TRY(hipGetLastError());
        pack_chunked_centres_kernel<<<num_tiles, 64, 0, s>>>(centers.as<float>(), radius.as<float>(), D, n_chunks,
                                                            num_tiles, centres_p.as<float>(), tile_coef.as<float>());
        TSNE_TRY(hipGetLastError());
    }

    // Sweep + re-rank of `count` query tiles: those of tile_list (device), or first, first + step, ... without a
    // list.  Keeps `keep` candidates per query and part.  failed = queries of those tiles whose verification
    // failed (listed in fail_list), swept = tile pairs computed.
    auto sweep_and_rerank = [&](int keep, const int *tile_list, int first, int step, int count, int &failed,
                                unsigned long long &swept) -> int {
        const int cap = list_cap(keep);
        // One workgroup sweeps a query tile against all its candidate tiles, which takes long with hundreds
        // of dimensions, and the tiles differ in how many candidate tiles they can skip: unless there are
        // several query tiles per workgroup slot to even that out, the chunked kernel splits every tile's
        // candidates over up to 8 workgroups.
        const int slots = cus * (bf16 ? bf16_sweep_occupancy(steps16) : (!chunked && ksteps <= 28 ? 3 : 2));
        int parts = 1;
        if (chunked)
            while (parts < 8 && count * parts < 3 * slots && parts * 2 * keep <= 2048 && parts * 2 <= num_tiles)
                parts *= 2;
        const int grid = std::min(count * parts, slots);
        const size_t n_slots = (size_t)(tile_list || step != 1 ? count * kMQ : N);
        DeviceMem lists, cand, tau, part_keys;
        if (!lists.alloc(sizeof(u64) * (size_t)grid * kMQ * cap) || !cand.alloc(sizeof(int) * n_slots * keep) ||
            !tau.alloc(sizeof(float) * n_slots) ||
            (parts > 1 && !part_keys.alloc(sizeof(u64) * n_slots * parts * keep))) {
            set_error("knn: out of device memory for the candidate lists");
            return 1;
        }
        TSNE_TRY(hipMemsetAsync(scal.as<int>() + 1, 0, 3 * sizeof(int), s));
        SweepArgs args;
        args.Xp = Xp.as<float4>();
        args.X = points;
        args.centres_p = centres_p.as<float>();
        args.tile_coef = tile_coef.as<float>();
        args.N = N;
        args.D = D;
        args.Dnorm = Dnorm;
        args.want = keep;
        args.cap = cap;
        args.lists = lists.as<u64>();
        args.num_qtiles = count;
        args.cand = cand.as<int>();
        args.tau = tau.as<float>();
        args.norms = norms.as<float>();
        args.centers_t = centers.as<float>();
        args.radius = radius.as<float>();
        args.bitmap_words = bitmap_words;
        args.trigger = cap - kCT;  // as late as possible: a later selection costs the same and sees more candidates
        args.select_slack = (cap - kCT - keep) / 4;
        args.tiles_swept = reinterpret_cast<unsigned long long *>(scal.as<int>() + 2);
        args.Bp = Bp.as<float4>();
        args.n_chunks = n_chunks;
        args.qtile_list = tile_list;
        args.qtile_first = first;
        args.qtile_step = step;
        args.parts = parts;
        args.part_keys = part_keys.as<u64>();
        args.probe_tile_lists = probes ? probes->tile_lists : nullptr;
        args.probe_list_words = probes ? probes->list_words : 0;
        args.probe_nlist = probes ? probes->nlist : 0;
        args.probe_list_tiles = probes ? probes->list_tiles : nullptr;
        if (chunked) {
            const size_t lds = sweep_lds(keep);
            if (bf16_chunked) {
                TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(knn_mfma_chunked_sweep_kernel<true>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                knn_mfma_chunked_sweep_kernel<true><<<grid, 256, lds, s>>>(args);
            } else {
                TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(knn_mfma_chunked_sweep_kernel<false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                knn_mfma_chunked_sweep_kernel<false><<<grid, 256, lds, s>>>(args);
            }
            TSNE_TRY(hipGetLastError());
        } else if (bf16 ? dispatch_bf16_sweep(steps16, args, grid, s) : dispatch_mfma_sweep(ksteps, args, grid, s)) {
            return 1;
        }
        if (parts > 1) {
            // rows of a partial last tile are merged too: the sweep left them unwritten, the re-rank skips them
            const size_t lds = sizeof(u64) * 4 * parts * keep;
            TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(knn_merge_parts_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            knn_merge_parts_kernel<<<div_up((int)n_slots, 4), 256, lds, s>>>(part_keys.as<u64>(), parts, keep,
                                                                            (int)n_slots, cand.as<int>(),
                                                                            tau.as<float>());
            TSNE_TRY(hipGetLastError());
        }
        const int sort_n = next_pow2(keep) < 64 ? 64 : next_pow2(keep);
        TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(knn_rerank_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)(sizeof(u64) * 4 * sort_n)));
        knn_rerank_kernel<<<div_up((int)n_slots, 4), 256, sizeof(u64) * 4 * sort_n, s>>>(
            points, norms.as<float>(), N, D, K, keep, sort_n, cand.as<int>(), tau.as<float>(), scal.as<float>(),
            indices, sq_dist, scal.as<int>() + 1, fail_list.as<int>(), tile_list, first, step, (int)n_slots,
            bf16 || bf16_chunked ? 1 : 0);
        TSNE_TRY(hipGetLastError());
        int host_scal[4] = {0, 0, 0, 0};
        TSNE_TRY(hipMemcpyAsync(host_scal, scal.p, sizeof(host_scal), hipMemcpyDeviceToHost, s));
        TSNE_TRY(hipStreamSynchronize(s));
        failed = host_scal[1];
        std::memcpy(&swept, host_scal + 2, sizeof(swept));
        return 0;
    };

    int failed = 0;
    unsigned long long swept = 0;
    // The verification needs the distance gap between neighbour K and candidate K' to exceed the rounding
    // bound of the approximate distances, which grows with the dimension count and with the points'
    // distance from the origin.  With many dimensions the neighbour distances of a query lie close
    // together, so the chunked sweep first tries its margin on a sample of query tiles and doubles K'
    // while more than a tenth of the sample fails; data that no margin verifies goes to the vector sweep.
    if (chunked && num_qtiles >= 64) {
        const int sample_tiles = 16, step = num_qtiles / sample_tiles;
        bool verified = false;
        for (int attempt = 0; attempt < 3 && !verified; ++attempt) {
            if (sweep_and_rerank(want, nullptr, step / 2, step, sample_tiles, failed, swept)) return 1;
            if (failed * 10 <= sample_tiles * kMQ) {
                verified = true;
            } else {
                const int wider = std::min(N - 1, 2 * want);
                if (wider == want || !sweep_fits(wider)) break;
                want = wider;
            }
        }
        if (!verified && mode == 0) {
            if (build_transposed()) return 1;
            return run_valu_sweep(points, Xt.as<float>(), N, Npad, D, K, nullptr, N, cus, indices, sq_dist, s);
        }
    }
    if (sweep_and_rerank(want, nullptr, 0, 1, num_qtiles, failed, swept)) return 1;
    if (stats) {
        stats[0] = 1;
        stats[1] = failed;
        stats[2] = (int)((1000.0 * (double)swept) / ((double)num_tiles * (double)num_tiles) + 0.5);
    }
    // Few failures, or failures scattered thinly over the query tiles, go straight to the vector sweep, which
    // spreads a list of queries over the chip by candidate range.  Where a quarter or more of the queries of the
    // tiles concerned failed, the chunked sweep takes those tiles once more with twice the margin (a vector sweep
    // of that many queries over all points in hundreds of dimensions takes longer than the matrix sweep of their
    // tiles); what fails again, and every failure of the register-resident sweep, goes to the vector sweep.
    if (failed > 4 * kQT && chunked && failed * 10 <= N) {
        const int wider = std::min(N - 1, 2 * want);
        if (wider != want && sweep_fits(wider)) {
            std::vector<int> queries(failed), tiles;
            TSNE_TRY(hipMemcpy(queries.data(), fail_list.p, sizeof(int) * (size_t)failed, hipMemcpyDeviceToHost));
            for (int q : queries) tiles.push_back(q / kMQ);
            std::sort(tiles.begin(), tiles.end());
            tiles.erase(std::unique(tiles.begin(), tiles.end()), tiles.end());
            if ((size_t)failed * 4 >= tiles.size() * kMQ) {
                DeviceMem tile_list;
                if (!tile_list.alloc(sizeof(int) * tiles.size())) {
                    set_error("knn: out of device memory for the retry list");
                    return 1;
                }
                TSNE_TRY(hipMemcpy(tile_list.p, tiles.data(), sizeof(int) * tiles.size(), hipMemcpyHostToDevice));
                unsigned long long swept_again = 0;
                if (sweep_and_rerank(wider, tile_list.as<int>(), 0, 1, (int)tiles.size(), failed, swept_again))
                    return 1;
            }
        }
    }
    if (failed > 0) {
        if (build_transposed()) return 1;
        return run_valu_sweep(points, Xt.as<float>(), N, Npad, D, K, fail_list.as<int>(), failed, cus, indices, sq_dist, s);
    }
    return 0;
}

int run_knn(const float *points, int N, int D, int K, int *indices, float *sq_dist, hipStream_t s) {
    return run_knn_mode(points, N, D, K, indices, sq_dist, s, 0, nullptr, nullptr);
}

}  // namespace tsnehip
