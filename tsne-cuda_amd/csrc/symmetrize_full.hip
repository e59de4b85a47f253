// Full symmetrisation of the conditional probabilities into CSR form (gfx950):
//
//   P = (A + A^T) / (2N),   A[i, idx[i,s]] = p[i,s]
//
// with the union pattern of A and A^T (an entry present in one direction only keeps half its mass, and
// nothing is dropped - the pattern-restricted form in symmetrize.hip, which is what the reference runs,
// drops the entries whose mirror is not stored).  The reference holds this variant only as a commented-out
// cuSPARSE routine (src/util/math_utils.cu:76-225: sort the rows, transpose, csrgeam with both factors
// 1/(2N)); here it is a device radix sort and a segmented reduce, all in this file:
//
//   1. every stored (i, j, p) yields the triples (i, j, p) and (j, i, p), keyed by row * 2^b + column
//      (b = bits of N - 1);
//   2. a stable least-significant-digit radix sort of the 2 nnz (key, value) pairs, 8 bits per pass:
//      per pass a histogram kernel (digit counts per tile of 8192 keys), a scan of the digit-major table of
//      counts (one workgroup per digit, then the digits' bases), and a scatter kernel in which a wave owns 512
//      consecutive keys of the tile and ranks them with ballots (lanes of equal digit found by eight ballots;
//      no atomics), orders the tile in LDS and writes every digit's keys as one coalesced run;
//   3. runs of equal keys are the segments: their heads are flagged, an exclusive scan of the flags gives
//      every head its place in the output, and the head sums its run (two values at most when the rows of A
//      hold distinct columns), divides by 2N and writes column and value; the first head of a row writes the
//      row pointer.
//
// Rows come out with ascending columns.  Values: the run's sum in fp32 (in sorted, i.e. original, order),
// divided by 2.0 * N in double, rounded to float - the arithmetic of the pattern-restricted kernel.
#include <algorithm>

#include "plan.h"
#include "stages.h"

namespace tsnehip {

namespace {

typedef unsigned long long u64;

constexpr int kSortThreads = 1024;
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSortItems = 8;  // keys per lane; a wave owns kSortItems * 64 consecutive keys of its tile
constexpr int kSortTile = kSortThreads * kSortItems;
constexpr int kRadix = 256;

struct Buffer {
    void *ptr = nullptr;
    ~Buffer() {
        if (ptr) (void)hipFree(ptr);
    }
    bool alloc(size_t bytes) { return hipMalloc(&ptr, bytes ? bytes : 1) == hipSuccess; }
    template <typename T>
    T *as() const {
        return static_cast<T *>(ptr);
    }
};

__global__ __launch_bounds__(256) void triples_kernel(const float *__restrict__ p, const int *__restrict__ idx,
                                                      int64_t nnz, int K, int col_bits, u64 *__restrict__ keys,
                                                      float *__restrict__ vals) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x) {
        const u64 i = (u64)(e / K), j = (u64)(unsigned int)idx[e];
        const float v = p[e];
        keys[2 * e] = (i << col_bits) | j;
        vals[2 * e] = v;
        keys[2 * e + 1] = (j << col_bits) | i;
        vals[2 * e + 1] = v;
    }
}

// The lanes of the wave whose (valid) key has the same digit as this lane's.
__device__ __forceinline__ u64 match_digit(unsigned int digit, bool valid) {
    u64 mask = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const bool bit = (digit >> b) & 1u;
        const u64 with = __ballot(bit);
        mask &= bit ? with : ~with;
    }
    return mask;
}

// Digit counts of every tile: hist[digit * n_tiles + tile].
__global__ __launch_bounds__(kSortThreads) void radix_hist_kernel(const u64 *__restrict__ keys, int64_t n, int shift,
                                                                  unsigned int *__restrict__ hist, int n_tiles) {
    __shared__ unsigned int wave_cnt[kSortWaves][kRadix];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    for (int e = tid; e < kSortWaves * kRadix; e += kSortThreads) (&wave_cnt[0][0])[e] = 0u;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kSortTile + (int64_t)wave * (kSortItems * kWave);
    for (int r = 0; r < kSortItems; ++r) {
        const int64_t t = base + r * kWave + lane;
        const bool valid = t < n;
        const unsigned int d = valid ? (unsigned int)(keys[t] >> shift) & (kRadix - 1) : 0u;
        const u64 mask = match_digit(d, valid);
        // (one lane per digit present in the wave adds the digit's count: distinct addresses, the wave's own row)
        if (valid && lane == __ffsll((long long)mask) - 1) wave_cnt[wave][d] += (unsigned int)__popcll(mask);
    }
    __syncthreads();
    if (tid < kRadix) {
        unsigned int c = 0u;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) c += wave_cnt[w][tid];
        hist[(size_t)tid * n_tiles + blockIdx.x] = c;
    }
}

// In-place exclusive scan of `total` counts by one workgroup.
__global__ __launch_bounds__(1024) void single_block_scan_kernel(unsigned int *__restrict__ data, int64_t total) {
    __shared__ unsigned int sums[1024];
    const int tid = threadIdx.x;
    const int64_t chunk = (total + 1023) / 1024;
    const int64_t begin = tid * chunk < total ? tid * chunk : total;
    const int64_t end = begin + chunk < total ? begin + chunk : total;
    unsigned int s = 0u;
    for (int64_t t = begin; t < end; ++t) s += data[t];
    sums[tid] = s;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const unsigned int add = tid >= off ? sums[tid - off] : 0u;
        __syncthreads();
        sums[tid] += add;
        __syncthreads();
    }
    unsigned int run = sums[tid] - s;
    for (int64_t t = begin; t < end; ++t) {
        const unsigned int c = data[t];
        data[t] = run;
        run += c;
    }
}

// The table of counts is digit-major: row d holds digit d's count in every tile.  One workgroup per digit turns
// its row into exclusive prefixes (where the digit's keys of a tile start among all keys with that digit) and
// leaves the digit's total; a second, tiny kernel turns the totals into the digits' bases.
__global__ __launch_bounds__(1024) void radix_scan_rows_kernel(unsigned int *__restrict__ hist, int n_tiles,
                                                               unsigned int *__restrict__ digit_total) {
    __shared__ unsigned int sums[1024];
    const int tid = threadIdx.x;
    unsigned int *row = hist + (size_t)blockIdx.x * n_tiles;
    const int chunk = (n_tiles + 1023) / 1024;
    const int begin = min(n_tiles, tid * chunk), end = min(n_tiles, begin + chunk);
    unsigned int s = 0u;
    for (int t = begin; t < end; ++t) s += row[t];
    sums[tid] = s;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const unsigned int add = tid >= off ? sums[tid - off] : 0u;
        __syncthreads();
        sums[tid] += add;
        __syncthreads();
    }
    unsigned int run = sums[tid] - s;
    for (int t = begin; t < end; ++t) {
        const unsigned int c = row[t];
        row[t] = run;
        run += c;
    }
    if (tid == 1023) digit_total[blockIdx.x] = sums[1023];
}

__global__ __launch_bounds__(kRadix) void radix_digit_bases_kernel(unsigned int *__restrict__ digit_total) {
    __shared__ unsigned int sums[kRadix];
    const int tid = threadIdx.x;
    const unsigned int c = digit_total[tid];
    sums[tid] = c;
    __syncthreads();
    for (int off = 1; off < kRadix; off <<= 1) {
        const unsigned int add = tid >= off ? sums[tid - off] : 0u;
        __syncthreads();
        sums[tid] += add;
        __syncthreads();
    }
    digit_total[tid] = sums[tid] - c;
}

// Stable scatter of one pass.  A key's place among the tile's keys in digit order is (keys of the tile with
// a smaller digit) + (same digit in earlier waves of the tile) + (same digit earlier in the wave's own keys);
// the tile is first put into that order in LDS, so that the keys of one digit leave for their run of
// consecutive global positions - (digit's base) + (same digit in earlier tiles) + (place in the tile's run) -
// in coalesced stores instead of 64 scattered ones per wave instruction.
__global__ __launch_bounds__(kSortThreads) void radix_scatter_kernel(const u64 *__restrict__ keys_in,
                                                                     const float *__restrict__ vals_in, int64_t n,
                                                                     int shift, const unsigned int *__restrict__ hist,
                                                                     const unsigned int *__restrict__ digit_base,
                                                                     int n_tiles, u64 *__restrict__ keys_out,
                                                                     float *__restrict__ vals_out) {
    __shared__ unsigned int wave_base[kSortWaves][kRadix];
    __shared__ unsigned int digit_start[kRadix];  // first place of a digit's keys within the tile
    __shared__ unsigned int scan[kRadix];
    extern __shared__ __attribute__((aligned(16))) unsigned char tile_raw[];
    u64 *tile_keys = reinterpret_cast<u64 *>(tile_raw);
    float *tile_vals = reinterpret_cast<float *>(tile_keys + kSortTile);
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const u64 below = (1ull << lane) - 1ull;
    for (int e = tid; e < kSortWaves * kRadix; e += kSortThreads) (&wave_base[0][0])[e] = 0u;
    __syncthreads();
    const int64_t tile_begin = (int64_t)blockIdx.x * kSortTile;
    const int tile_count = (int)(n - tile_begin < kSortTile ? n - tile_begin : kSortTile);
    const int64_t base = tile_begin + (int64_t)wave * (kSortItems * kWave);
    u64 key[kSortItems];
    float val[kSortItems];
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const int64_t t = base + r * kWave + lane;
        key[r] = t < n ? keys_in[t] : 0ull;
        val[r] = t < n ? vals_in[t] : 0.0f;
    }
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const bool valid = base + r * kWave + lane < n;
        const unsigned int d = (unsigned int)(key[r] >> shift) & (kRadix - 1);
        const u64 mask = match_digit(d, valid);
        if (valid && lane == __ffsll((long long)mask) - 1) wave_base[wave][d] += (unsigned int)__popcll(mask);
    }
    __syncthreads();
    unsigned int tile_digit_count = 0u;
    if (tid < kRadix) {
        unsigned int run = 0u;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const unsigned int c = wave_base[w][tid];
            wave_base[w][tid] = run;  // same digit in earlier waves of the tile
            run += c;
        }
        tile_digit_count = run;
        scan[tid] = run;
    }
    __syncthreads();
    for (int off = 1; off < kRadix; off <<= 1) {
        unsigned int add = 0u;
        if (tid < kRadix && tid >= off) add = scan[tid - off];
        __syncthreads();
        if (tid < kRadix) scan[tid] += add;
        __syncthreads();
    }
    if (tid < kRadix) digit_start[tid] = scan[tid] - tile_digit_count;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const bool valid = base + r * kWave + lane < n;
        const unsigned int d = (unsigned int)(key[r] >> shift) & (kRadix - 1);
        const u64 mask = match_digit(d, valid);
        unsigned int place = 0u;
        if (valid) place = digit_start[d] + wave_base[wave][d] + (unsigned int)__popcll(mask & below);
        // every lane of the group has read the wave's base before its first lane moves it on (one wave: in order)
        __builtin_amdgcn_wave_barrier();
        if (valid && lane == __ffsll((long long)mask) - 1) wave_base[wave][d] += (unsigned int)__popcll(mask);
        __builtin_amdgcn_wave_barrier();
        if (valid) {
            tile_keys[place] = key[r];
            tile_vals[place] = val[r];
        }
    }
    __syncthreads();
    for (int sidx = tid; sidx < tile_count; sidx += kSortThreads) {
        const u64 k = tile_keys[sidx];
        const unsigned int d = (unsigned int)(k >> shift) & (kRadix - 1);
        const unsigned int pos = digit_base[d] + hist[(size_t)d * n_tiles + blockIdx.x] + ((unsigned int)sidx - digit_start[d]);
        keys_out[pos] = k;
        vals_out[pos] = tile_vals[sidx];
    }
}

constexpr size_t kSortTileLds = (sizeof(u64) + sizeof(float)) * kSortTile;

// ---- exclusive scan of 32-bit counts over the whole device: tile sums, one workgroup over the sums, tiles ----
constexpr int kScanThreads = 1024;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;

__device__ __forceinline__ unsigned int block_exclusive_scan(unsigned int v, unsigned int *lds, unsigned int &total) {
    const int tid = threadIdx.x;
    lds[tid] = v;
    __syncthreads();
    for (int off = 1; off < kScanThreads; off <<= 1) {
        const unsigned int add = tid >= off ? lds[tid - off] : 0u;
        __syncthreads();
        lds[tid] += add;
        __syncthreads();
    }
    total = lds[kScanThreads - 1];
    const unsigned int r = lds[tid] - v;
    __syncthreads();
    return r;
}

__global__ __launch_bounds__(kScanThreads) void head_flags_tile_sums_kernel(const u64 *__restrict__ keys, int64_t n,
                                                                            unsigned int *__restrict__ tile_sums) {
    __shared__ unsigned int lds[kScanThreads];
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    unsigned int c = 0u;
    for (int k = 0; k < kScanItems; ++k) {
        const int64_t t = base + k;
        if (t < n && (t == 0 || keys[t] != keys[t - 1])) c += 1u;
    }
    unsigned int total;
    block_exclusive_scan(c, lds, total);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// Heads of runs of equal keys write the output: place = heads before it (tile offset + scan inside the tile).
__global__ __launch_bounds__(kScanThreads) void emit_csr_kernel(const u64 *__restrict__ keys,
                                                                const float *__restrict__ vals, int64_t n,
                                                                const unsigned int *__restrict__ tile_offsets,
                                                                int col_bits, int N, int *__restrict__ row_ptr,
                                                                int *__restrict__ col_idx, float *__restrict__ values) {
    __shared__ unsigned int lds[kScanThreads];
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
    bool head[kScanItems];
    unsigned int c = 0u;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        const int64_t t = base + k;
        head[k] = t < n && (t == 0 || keys[t] != keys[t - 1]);
        c += head[k] ? 1u : 0u;
    }
    unsigned int total;
    unsigned int pos = tile_offsets[blockIdx.x] + block_exclusive_scan(c, lds, total);
    const u64 col_mask = (1ull << col_bits) - 1ull;
    const double denom = 2.0 * (double)N;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        const int64_t t = base + k;
        if (t >= n) break;
        if (head[k]) {
            const u64 key = keys[t];
            float sum = vals[t];
            for (int64_t u = t + 1; u < n && keys[u] == key; ++u) sum += vals[u];
            col_idx[pos] = (int)(key & col_mask);
            values[pos] = (float)((double)sum / denom);
            // the first entry of a row (and of the rows before it that are empty) starts here
            const int row = (int)(key >> col_bits);
            const int prev_row = t == 0 ? -1 : (int)(keys[t - 1] >> col_bits);
            for (int r = prev_row + 1; r <= row; ++r) row_ptr[r] = (int)pos;
            pos += 1u;
        }
        if (t == n - 1) {
            const int row = (int)(keys[t] >> col_bits);
            for (int r = row + 1; r <= N; ++r) row_ptr[r] = (int)pos;  // pos: one past the last head
        }
    }
}

// attr_i = sum over row i of the CSR pattern of P (y_i - y_j) / (1 + |y_i - y_j|^2): a wave per row.
__global__ __launch_bounds__(256) void attractive_csr_kernel(const int *__restrict__ row_ptr,
                                                             const int *__restrict__ col_idx,
                                                             const float *__restrict__ values,
                                                             const float2 *__restrict__ yxy, int N,
                                                             float *__restrict__ attr) {
    const int row = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    if (row >= N) return;
    const float2 yi = yxy[row];
    float ax = 0.0f, ay = 0.0f;
    for (int e = row_ptr[row] + lane; e < row_ptr[row + 1]; e += kWave) {
        const float2 yj = yxy[col_idx[e]];
        const float dx = yi.x - yj.x, dy = yi.y - yj.y;
        const float w = values[e] / (1.0f + dx * dx + dy * dy);
        ax += w * dx;
        ay += w * dy;
    }
    ax = group_sum<kWave>(ax);
    ay = group_sum<kWave>(ay);
    if (lane == 0) {
        attr[row] = ax;
        attr[N + row] = ay;
    }
}

// out[0] += sum P ln(P (1 + d^2)), out[1] += sum P over the CSR pattern.
__global__ __launch_bounds__(256) void kl_terms_csr_kernel(const int *__restrict__ row_ptr,
                                                           const int *__restrict__ col_idx,
                                                           const float *__restrict__ values,
                                                           const float *__restrict__ emb, int N,
                                                           double *__restrict__ out) {
    const int lane = threadIdx.x & (kWave - 1);
    double kl = 0.0, mass = 0.0;
    for (int row = blockIdx.x * (256 / kWave) + threadIdx.x / kWave; row < N; row += gridDim.x * (256 / kWave)) {
        const float xi = emb[row], yi = emb[N + row];
        for (int e = row_ptr[row] + lane; e < row_ptr[row + 1]; e += kWave) {
            const float p = values[e];
            if (p > 0.0f) {
                const int j = col_idx[e];
                const float dx = xi - emb[j], dy = yi - emb[N + j];
                kl += (double)p * (log((double)p) + log1p((double)dx * dx + (double)dy * dy));
                mass += (double)p;
            }
        }
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        kl += __shfl_xor(kl, m, kWave);
        mass += __shfl_xor(mass, m, kWave);
    }
    if (lane == 0) {
        atomicAdd(&out[0], kl);
        atomicAdd(&out[1], mass);
    }
}

__global__ void clear_pair_csr_kernel(double *out) {
    if (threadIdx.x < 2 && blockIdx.x == 0) out[threadIdx.x] = 0.0;
}

int bits_for(int n) {  // bits of n - 1, at least 1
    int b = 1;
    while ((1ll << b) < (long long)n) ++b;
    return b;
}

}  // namespace

// Sorts n (key, value) pairs by the low key_bits bits of the key, stable; the result is in (keys, vals).
// keys_alt / vals_alt: scratch of the same size.  hist: 256 * (tiles + 1) counts (tiles of radix_sort_tile() keys).
int radix_sort_tile() { return kSortTile; }
int radix_sort_pairs(u64 *keys, float *vals, u64 *keys_alt, float *vals_alt, int64_t n, int key_bits,
                     unsigned int *hist, hipStream_t s) {
    const int n_tiles = div_up(n, kSortTile);
    unsigned int *digit_base = hist + (size_t)kRadix * n_tiles;
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(radix_scatter_kernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSortTileLds));
    u64 *kin = keys, *kout = keys_alt;
    float *vin = vals, *vout = vals_alt;
    int passes = 0;
    for (int shift = 0; shift < key_bits; shift += 8, ++passes) {
        radix_hist_kernel<<<n_tiles, kSortThreads, 0, s>>>(kin, n, shift, hist, n_tiles);
        TSNE_LAUNCHED(s);
        radix_scan_rows_kernel<<<kRadix, 1024, 0, s>>>(hist, n_tiles, digit_base);
        TSNE_LAUNCHED(s);
        radix_digit_bases_kernel<<<1, kRadix, 0, s>>>(digit_base);
        TSNE_LAUNCHED(s);
        radix_scatter_kernel<<<n_tiles, kSortThreads, kSortTileLds, s>>>(kin, vin, n, shift, hist, digit_base, n_tiles,
                                                                       kout, vout);
        TSNE_LAUNCHED(s);
        std::swap(kin, kout);
        std::swap(vin, vout);
    }
    if (passes & 1) {  // the sorted pairs sit in the scratch arrays
        TSNE_TRY(hipMemcpyAsync(keys, keys_alt, sizeof(u64) * (size_t)n, hipMemcpyDeviceToDevice, s));
        TSNE_TRY(hipMemcpyAsync(vals, vals_alt, sizeof(float) * (size_t)n, hipMemcpyDeviceToDevice, s));
    }
    return 0;
}

int symmetrize_full(const float *p, const int *idx, int N, int K, int *row_ptr, int *col_idx, float *values,
                    int64_t *nnz_out, hipStream_t s) {
    const int64_t nnz = (int64_t)N * K, n = 2 * nnz;
    // (positions, row pointers and the entry count are 32-bit signed)
    if (n >= ((int64_t)1 << 31)) {
        set_error("symmetrize_full: %lld triples exceed the 31-bit positions of the sort and the row pointers",
                  (long long)n);
        return 1;
    }
    // A column outside [0, N) would spill into the row bits of its sort key.
    if (validate_indices(idx, nnz, N, "symmetrize_full", s)) return 1;
    const int col_bits = bits_for(N);
    const int n_tiles = div_up(n, kSortTile), scan_tiles = div_up(n, kScanTile);
    Buffer keys, vals, keys_alt, vals_alt, hist, tile_sums;
    if (!keys.alloc(sizeof(u64) * (size_t)n) || !vals.alloc(sizeof(float) * (size_t)n) ||
        !keys_alt.alloc(sizeof(u64) * (size_t)n) || !vals_alt.alloc(sizeof(float) * (size_t)n) ||
        !hist.alloc(sizeof(unsigned int) * (size_t)kRadix * (n_tiles + 1)) ||
        !tile_sums.alloc(sizeof(unsigned int) * (size_t)scan_tiles)) {
        set_error("symmetrize_full: out of device memory (%lld triples)", (long long)n);
        return 1;
    }
    triples_kernel<<<(int)std::min<int64_t>(div_up(nnz, 256), 65536), 256, 0, s>>>(p, idx, nnz, K, col_bits,
                                                                                   keys.as<u64>(), vals.as<float>());
    TSNE_LAUNCHED(s);
    if (radix_sort_pairs(keys.as<u64>(), vals.as<float>(), keys_alt.as<u64>(), vals_alt.as<float>(), n, 2 * col_bits,
                         hist.as<unsigned int>(), s))
        return 1;
    head_flags_tile_sums_kernel<<<scan_tiles, kScanThreads, 0, s>>>(keys.as<u64>(), n, tile_sums.as<unsigned int>());
    TSNE_LAUNCHED(s);
    single_block_scan_kernel<<<1, 1024, 0, s>>>(tile_sums.as<unsigned int>(), scan_tiles);
    TSNE_LAUNCHED(s);
    emit_csr_kernel<<<scan_tiles, kScanThreads, 0, s>>>(keys.as<u64>(), vals.as<float>(), n,
                                                        tile_sums.as<unsigned int>(), col_bits, N, row_ptr, col_idx,
                                                        values);
    TSNE_LAUNCHED(s);
    int total = 0;
    TSNE_TRY(hipMemcpyAsync(&total, row_ptr + N, sizeof(int), hipMemcpyDeviceToHost, s));
    TSNE_TRY(hipStreamSynchronize(s));  // also: the work buffers go out of scope
    if (nnz_out) *nnz_out = total;
    return 0;
}

int launch_attractive_csr(tsne_hip_plan *p, const int *row_ptr, const int *col_idx, const float *values, float *attr,
                          hipStream_t s) {
    if (profile_mark(p, kKernelAttractive, s)) return 1;
    TSNE_LOOP_KERNEL(p, (attractive_csr_kernel), div_up(p->num_points, 256 / kWave), 256, 0, s, row_ptr, col_idx, values, p->yxy,
                                                                             p->num_points, attr);
    TSNE_LAUNCHED(s);
    return 0;
}

int launch_kl_terms_csr(const int *row_ptr, const int *col_idx, const float *values, const float *embedding, int N,
                        double *out, hipStream_t s) {
    clear_pair_csr_kernel<<<1, 64, 0, s>>>(out);
    TSNE_LAUNCHED(s);
    kl_terms_csr_kernel<<<std::min(div_up(N, 256 / kWave), 4096), 256, 0, s>>>(row_ptr, col_idx, values, embedding, N,
                                                                               out);
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
