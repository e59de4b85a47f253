// Pattern-restricted symmetrisation of the conditional probabilities for gfx950.
//
//   P[i,s] = (p[i,s] + sum_{t : idx[j,t] == i} p[j,t]) / (2 N),   j = idx[i,s]
//
// Semantics: src/util/math_utils.cu:269-291 of the reference (the N x K pattern
// is kept; pairs present in only one direction keep half their mass).  The
// reference gives every non-zero its own thread that walks row j alone: N K^2
// index reads, 32 GB at a million points and 90 neighbours.  Two forms here:
//   * hashed (the default from 4096 points up): every row's (column, value)
//     pairs go once into a small open-addressing table of the row's own (a power
//     of two >= 1.25 K slots of 8 bytes, linear probing, built in LDS by a group
//     of lanes per row); a non-zero then looks for its row number in the table of
//     row j: one or two 64-byte sectors instead of the 720 bytes of row j;
//   * scanning (small problems, more than 1638 neighbours, rows that name a column
//     twice, or when the tables do not fit in memory): a group of lanes owns row i
//     and the whole group scans each row j
//     together, so every index row is fetched with coalesced loads and the match
//     is found with a ballot.
#include "plan.h"
#include "stages.h"

#include <algorithm>
#include <cstdlib>

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

// ---- hashed form ----------------------------------------------------------
struct Slot {
    int key;  // column, -1: empty
    float value;
};
__device__ __forceinline__ unsigned int slot_of(int key, int log2_slots) {
    return ((unsigned int)key * 0x9E3779B1u) >> (32 - log2_slots);
}

// A group of LANES lanes per row builds the row's table in LDS (insertions race for empty slots with a
// compare-and-swap; which slot a column ends up in does not matter to a lookup) and writes it out whole.  A row
// that names a column twice raises *repeated: the caller then takes the scanning form, which adds such values up.
template <int LANES>
__global__ __launch_bounds__(256) void build_tables_kernel(const float *__restrict__ p, const int *__restrict__ idx,
                                                           int N, int K, int log2_slots, Slot *__restrict__ table,
                                                           int *__restrict__ repeated) {
    extern __shared__ Slot lds_tables[];
    constexpr int kRows = 256 / LANES;
    const int slots = 1 << log2_slots;
    const unsigned int mask = (unsigned int)slots - 1u;
    const int group = threadIdx.x / LANES, lane = threadIdx.x % LANES;
    const int row = blockIdx.x * kRows + group;
    Slot *mine = lds_tables + (size_t)group * slots;
    for (int e = lane; e < slots; e += LANES) mine[e] = Slot{-1, 0.0f};
    __syncthreads();
    bool twice = false;
    if (row < N) {
        const size_t base = (size_t)row * K;
        for (int t = lane; t < K; t += LANES) {
            const int key = idx[base + t];
            const float v = p[base + t];
            unsigned int at = slot_of(key, log2_slots);
            for (;;) {  // (more slots than pairs: an empty one is always met)
                const int old = atomicCAS(&mine[at].key, -1, key);
                if (old == -1) {
                    mine[at].value = v;
                    break;
                }
                if (old == key) {
                    twice = true;
                    break;
                }
                at = (at + 1u) & mask;
            }
        }
    }
    if (__any(twice) && (threadIdx.x & (kWave - 1)) == 0) atomicOr(repeated, 1);
    __syncthreads();
    if (row < N) {
        Slot *out = table + ((size_t)row << log2_slots);
        for (int e = lane; e < slots; e += LANES) out[e] = mine[e];
    }
}

__global__ __launch_bounds__(256) void symmetrize_hashed_kernel(const float *__restrict__ p, const int *__restrict__ idx,
                                                                int N, int K, int log2_slots,
                                                                const Slot *__restrict__ table, float *__restrict__ P) {
    const size_t nnz = (size_t)N * K;
    const double denom = 2.0 * (double)N;
    const unsigned int mask = (1u << log2_slots) - 1u;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < nnz; e += (size_t)gridDim.x * 256) {
        const int row = (int)(e / K);
        const int j = idx[e];
        const Slot *theirs = table + ((size_t)j << log2_slots);
        float found = 0.0f;
        unsigned int at = slot_of(row, log2_slots);
        for (;;) {
            const Slot here = theirs[at];
            if (here.key == row) {
                found = here.value;
                break;
            }
            if (here.key < 0) break;
            at = (at + 1u) & mask;
        }
        P[e] = (float)((double)(p[e] + found) / denom);
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
    // Hashed form: tables of next_pow2(1.25 K) slots per row.  A column outside [0, N) would address another
    // row's table, so the indices are checked first (the scanning form only compares them).
    int log2_slots = 3;
    while ((1 << log2_slots) < K + (K + 3) / 4) ++log2_slots;
    const size_t table_bytes = ((size_t)N << log2_slots) * sizeof(Slot);
    const bool scan_only = std::getenv("TSNE_SYMMETRIZE_SCAN") != nullptr;  // (for measurements and tests)
    if (N >= 4096 && log2_slots <= 11 && table_bytes <= ((size_t)64 << 30) && !scan_only) {
        Slot *table = nullptr;
        int *repeated = nullptr;
        if (hipMalloc(&table, table_bytes) == hipSuccess && hipMalloc(&repeated, sizeof(int)) == hipSuccess) {
            int rc = validate_indices(idx, (int64_t)N * K, N, "symmetrize", s);
            int twice = 0;
            if (!rc) {
                hipError_t e = hipMemsetAsync(repeated, 0, sizeof(int), s);
                if (e == hipSuccess) {
                    if (log2_slots <= 8) {
                        build_tables_kernel<16><<<div_up(N, 16), 256, sizeof(Slot) * 16 << log2_slots, s>>>(
                            p, idx, N, K, log2_slots, table, repeated);
                    } else {
                        TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(build_tables_kernel<64>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                                     (int)(sizeof(Slot) * 4 << 11)));
                        build_tables_kernel<64><<<div_up(N, 4), 256, sizeof(Slot) * 4 << log2_slots, s>>>(
                            p, idx, N, K, log2_slots, table, repeated);
                    }
                    symmetrize_hashed_kernel<<<(int)std::min<int64_t>(div_up((int64_t)N * K, 256), 1 << 20), 256, 0,
                                               s>>>(p, idx, N, K, log2_slots, table, P);
                    e = hipGetLastError();
                }
                if (e == hipSuccess) e = hipMemcpyAsync(&twice, repeated, sizeof(int), hipMemcpyDeviceToHost, s);
                if (e == hipSuccess) e = hipStreamSynchronize(s);  // the tables go
                if (e != hipSuccess) {
                    set_error("symmetrize: %s", hipGetErrorString(e));
                    rc = 1;
                }
            }
            (void)hipFree(table);
            (void)hipFree(repeated);
            if (rc || !twice) return rc;
            // (some row names a column twice: the scanning form below adds those values up)
        } else {
            (void)hipFree(table);
            (void)hipFree(repeated);
            (void)hipGetLastError();  // no room for the tables: the scanning form needs none
        }
    }
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
