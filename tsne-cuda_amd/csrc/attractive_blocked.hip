// Attractive forces from a re-blocked copy of the sparse pattern (gfx950).
//
// The row-ordered kernel in attractive.hip gathers neighbour positions from
// all over an 8 MB array: at 1M points half of those gathers miss the L2 and
// every miss moves a whole cache line, so the kernel spends its time on ~8x its
// algorithmic traffic.  The pattern never changes during the gradient loop, so
// it is re-blocked once:
//
//   * rows are cut into strips (one workgroup each, <= 4096 rows),
//   * columns into partitions of kPartPoints points,
//   * inside a strip the entries are grouped by partition; an entry is 8 bytes:
//     the probability and a packed (column within partition | row within strip).
//
// A workgroup keeps its strip's positions and force accumulators in LDS and
// walks the partitions in order; for each one it stages that partition's
// positions in LDS, so every neighbour gather is an LDS read and every
// accumulation an LDS atomic.  HBM sees the 8 bytes per entry once, coalesced,
// plus the positions once per workgroup (served by the L2, since all
// workgroups walk the partitions in step).  The next partition and its entries
// are prefetched into registers while the current one is being consumed.
//
// Accumulators are 64-bit fixed point: on gfx950 an LDS float atomic add costs
// ~190 clocks per wave instruction while 64-bit integer LDS atomics run about
// 25x faster, and integer sums do not depend on the order of the additions.
// With p_max the largest probability, |contribution| <= p_max / 2 (because
// |d| / (1 + d^2) <= 1/2), so the scale 2^51 / p_max keeps every contribution
// below 2^50 and a row sum of K < 4096 terms below 2^62.
//
// Semantics are those of src/kernels/attr_forces.cu:129-184 of the reference;
// only the order of the fp32 additions inside a row differs.
#include "plan.h"

namespace tsnehip {

namespace {

constexpr int kColBits = 13;
constexpr int kPartPoints = 8192;   // == 1 << kColBits; 64 KB of (x, y) pairs
constexpr int kStripMax = 4096;     // rows per strip: 32 KB of positions + 64 KB of accumulators
constexpr double kRoundMagic = 6755399441055744.0;  // 1.5 * 2^52: adding it rounds a double to an integer
constexpr int kBlock = 1024;
constexpr int kMaxParts = 1024;
static_assert(kBlock == kMaxParts, "the partition scan uses one thread per slot");
constexpr int kPrefetch = 4;        // entries per thread in one work item
constexpr unsigned int kItemEntries = kPrefetch * kBlock;

// ---------------------------------------------------------------------------
// Re-blocking: one workgroup per strip.  Histogram of the strip's entries over
// the partitions, exclusive scan, then a scatter that ranks entries inside a
// partition with LDS atomics.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void reblock_kernel(const float *__restrict__ pij, const int *__restrict__ idx,
                                                         int N, int K, int strip_rows, int max_items,
                                                         int seg_stride, float *__restrict__ ent_p,
                                                         unsigned int *__restrict__ ent_c,
                                                         unsigned int *__restrict__ seg, float *__restrict__ p_max) {
    __shared__ unsigned int cursor[kMaxParts];
    __shared__ unsigned int scan[kMaxParts];
    const int tid = threadIdx.x;
    const int strip = blockIdx.x;
    const int row0 = strip * strip_rows;
    const int nrows = min(strip_rows, N - row0);
    const size_t base = (size_t)row0 * K;
    const unsigned int count = (unsigned int)nrows * (unsigned int)K;
    for (int b = tid; b < kMaxParts; b += kBlock) cursor[b] = 0;
    __syncthreads();
    for (unsigned int e = tid; e < count; e += kBlock) atomicAdd(&cursor[idx[base + e] / kPartPoints], 1u);
    __syncthreads();
    // Inclusive Hillis-Steele scan over kMaxParts == kBlock slots.
    unsigned int mine = cursor[tid];
    scan[tid] = mine;
    __syncthreads();
    for (int off = 1; off < kMaxParts; off <<= 1) {
        const unsigned int add = tid >= off ? scan[tid - off] : 0u;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    const unsigned int first = scan[tid] - mine;
    cursor[tid] = first;
    __syncthreads();
    // Work list of the strip: every referenced partition contributes ceil(entries / kItemEntries) items
    // (runs of at most kItemEntries entries that share the partition); a second scan, over the item counts.
    const unsigned int items = (mine + kItemEntries - 1u) / kItemEntries;
    scan[tid] = items;
    __syncthreads();
    for (int off = 1; off < kMaxParts; off <<= 1) {
        const unsigned int add = tid >= off ? scan[tid - off] : 0u;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    unsigned int *hdr = seg + (size_t)strip * seg_stride;
    unsigned int *item_begin = hdr + 1;
    unsigned int *item_part = hdr + 2 + max_items;
    for (unsigned int it = 0; it < items; ++it) {
        const unsigned int slot = scan[tid] - items + it;
        item_begin[slot] = first + it * kItemEntries;
        item_part[slot] = (unsigned int)tid;
    }
    if (tid == kMaxParts - 1) {
        hdr[0] = scan[tid];
        item_begin[scan[tid]] = count;
    }
    // Entries are visited neighbour slot by neighbour slot, so that neighbouring positions of a
    // partition's run belong to different rows: a wave of the force kernel then spreads its LDS
    // atomics over many accumulators even when most neighbours of a row share one partition.
    float biggest = 0.0f;
    for (unsigned int v = tid; v < count; v += kBlock) {
        const unsigned int slot = v / (unsigned int)nrows;
        const unsigned int row_local = v - slot * (unsigned int)nrows;
        const unsigned int e = row_local * (unsigned int)K + slot;
        const int col = idx[base + e];
        const int part = col / kPartPoints;
        const unsigned int pos = atomicAdd(&cursor[part], 1u);
        const float pv = pij[base + e];
        biggest = fmaxf(biggest, fabsf(pv));
        ent_p[base + pos] = pv;
        ent_c[base + pos] = (unsigned int)(col - part * kPartPoints) | (row_local << kColBits);
    }
    biggest = group_max<kWave>(biggest);
    // Non-negative floats order like their bit patterns.
    if ((tid & (kWave - 1)) == 0) atomicMax(reinterpret_cast<unsigned int *>(p_max), __float_as_uint(biggest));
}

__global__ void clear_pmax_kernel(float *p_max) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *p_max = 0.0f;
}

// ---------------------------------------------------------------------------
// One workgroup per strip; dynamic LDS: part[kPartPoints] float2, then
// yi[kStripMax] float2, then acc_x[kStripMax] and acc_y[kStripMax], 64-bit fixed point.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void add_force(unsigned long long *acc, unsigned int rl, float vx, float vy,
                                          double scale) {
    const double tx = fma((double)vx, scale, kRoundMagic);
    const double ty = fma((double)vy, scale, kRoundMagic);
    const long long ix = __double_as_longlong(tx) - __double_as_longlong(kRoundMagic);
    const long long iy = __double_as_longlong(ty) - __double_as_longlong(kRoundMagic);
    // x sums and y sums live in separate arrays: consecutive rows then fall
    // into consecutive 8-byte slots and the atomics of a wave spread over all banks.
    atomicAdd(&acc[rl], (unsigned long long)ix);
    atomicAdd(&acc[kStripMax + rl], (unsigned long long)iy);
}

__global__ __launch_bounds__(kBlock) void attractive_blocked_kernel(const float *__restrict__ ent_p,
                                                                    const unsigned int *__restrict__ ent_c,
                                                                    const unsigned int *__restrict__ seg,
                                                                    const float2 *__restrict__ yxy,
                                                                    const float *__restrict__ p_max,
                                                                    float *__restrict__ attr, int N, int K,
                                                                    int strip_rows, int max_items, int seg_stride) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    float2 *part = reinterpret_cast<float2 *>(lds_raw);
    float2 *yi = part + kPartPoints;
    unsigned long long *acc = reinterpret_cast<unsigned long long *>(yi + kStripMax);

    const int tid = threadIdx.x;
    const int strip = blockIdx.x;
    const int row0 = strip * strip_rows;
    const int nrows = min(strip_rows, N - row0);
    const size_t base = (size_t)row0 * K;
    // The work list is read through the constant address space: it is never written while this
    // kernel runs, and constant-space loads at uniform addresses are scalar loads, which do not
    // queue behind the vector loads in flight.
    typedef const __attribute__((address_space(4))) unsigned int *ConstWords;
    ConstWords hdr = (ConstWords)(seg + (size_t)strip * seg_stride);
    const int n_items = (int)hdr[0];
    ConstWords my_seg = hdr + 1;               // n_items + 1 entry offsets
    ConstWords my_part = hdr + 2 + max_items;  // partition of each item
    const float pm = *p_max;
    const double scale = pm > 0.0f ? 2251799813685248.0 / (double)pm : 1.0;  // 2^51 / p_max

    for (int r = tid; r < nrows; r += kBlock) {
        yi[r] = yxy[row0 + r];
        acc[r] = 0ull;
        acc[kStripMax + r] = 0ull;
    }

    constexpr int kPartLoads = kPartPoints / (2 * kBlock);  // float4 (two points) loads per thread
    static_assert(kPartPoints % (2 * kBlock) == 0, "partition staging assumes whole float4 rounds");
    const float4 *yxy4 = reinterpret_cast<const float4 *>(yxy);
    float4 *part4 = reinterpret_cast<float4 *>(part);
    const int last_pair_all = (N - 1) / 2;  // yxy is padded, so a pair may run one point past N

    // Register sets rotate between "being consumed" and "in flight", so the
    // prefetch of later phases overlaps the LDS work of phase p without any
    // register copies (a copy would have to wait for the load it copies).
    struct PhaseRegs {
        float pv[kPrefetch];
        unsigned int pc[kPrefetch];
        float4 stage[kPartLoads];
        unsigned int b, e;
        bool fresh;  // the item starts a new partition (uniform over the workgroup)
    };
    // All loads are unconditional (addresses clamped into range) so that none waits for another.
    const size_t last_entry = (size_t)nrows * K - 1;
    auto issue = [&](PhaseRegs &R, int item) {
        R.b = my_seg[item];
        R.e = my_seg[item + 1];
        const int p = (int)my_part[item];
        R.fresh = item == 0 || p != (int)my_part[item - 1];
#pragma unroll
        for (int k = 0; k < kPrefetch; ++k) {
            const size_t t = min((size_t)R.b + tid + k * kBlock, last_entry);
            R.pv[k] = ent_p[base + t];
            R.pc[k] = ent_c[base + t];
        }
        // Every item issues the same number of loads, so the compiler's outstanding-load counts stay
        // exact and no wait ever covers a younger prefetch.  An item that re-uses the staged partition
        // points all lanes at one address instead: a single cache line per load, nothing to ingest.
#pragma unroll
        for (int k = 0; k < kPartLoads; ++k)
            R.stage[k] = yxy4[R.fresh ? min(p * (kPartPoints / 2) + tid + k * kBlock, last_pair_all) : 0];
    };
    auto consume = [&](PhaseRegs &R) {
#pragma unroll
        for (int k = 0; k < kPrefetch; ++k) {
            const unsigned int t = R.b + tid + k * kBlock;
            if (t < R.e) {
                const unsigned int rl = R.pc[k] >> kColBits;
                const float2 yj = part[R.pc[k] & ((1u << kColBits) - 1u)];
                const float2 y0 = yi[rl];
                const float dx = y0.x - yj.x, dy = y0.y - yj.y;
                const float w = R.pv[k] * __builtin_amdgcn_rcpf(1.0f + dx * dx + dy * dy);
                add_force(acc, rl, w * dx, w * dy, scale);
            }
        }
    };
    auto stage_to_lds = [&](PhaseRegs &R) {
        if (!R.fresh) return;  // same partition as the previous item: it is already staged
        __syncthreads();       // everyone is done reading the previous partition (first time: yi / acc are set)
#pragma unroll
        for (int k = 0; k < kPartLoads; ++k) part4[tid + k * kBlock] = R.stage[k];
        __syncthreads();
    };

    // Prefetch distance two: while item p is consumed, the loads of items
    // p+1 and p+2 are in flight (a memory round trip is several items long).
    PhaseRegs R0, R1, R2;
    if (0 < n_items) issue(R0, 0);
    if (1 < n_items) issue(R1, 1);
    for (int p = 0; p < n_items; p += 3) {
        stage_to_lds(R0);
        if (p + 2 < n_items) issue(R2, p + 2);
        consume(R0);
        if (p + 1 >= n_items) break;
        stage_to_lds(R1);
        if (p + 3 < n_items) issue(R0, p + 3);
        consume(R1);
        if (p + 2 >= n_items) break;
        stage_to_lds(R2);
        if (p + 4 < n_items) issue(R1, p + 4);
        consume(R2);
    }
    __syncthreads();
    const double inv_scale = 1.0 / scale;
    for (int r = tid; r < nrows; r += kBlock) {
        attr[row0 + r] = (float)((double)(long long)acc[r] * inv_scale);
        attr[N + row0 + r] = (float)((double)(long long)acc[kStripMax + r] * inv_scale);
    }
}

constexpr size_t kBlockedLds =
    sizeof(float2) * kPartPoints + sizeof(float2) * kStripMax + sizeof(unsigned long long) * 2 * kStripMax;
static_assert(kBlockedLds <= 160 * 1024, "one workgroup must fit the 160 KB of LDS");

}  // namespace

void release_blocked(tsne_hip_plan *p) {
    (void)hipFree(p->ent_p);
    (void)hipFree(p->ent_c);
    (void)hipFree(p->seg);
    p->ent_p = nullptr;
    p->ent_c = nullptr;
    p->seg = nullptr;
    p->blocked_ready = false;
}

int prepare_blocked(tsne_hip_plan *p, const float *pij, const int *indices, hipStream_t s) {
    release_blocked(p);
    const int N = p->num_points, K = p->num_neighbors;
    const int n_parts = div_up(N, kPartPoints);
    if (n_parts > kMaxParts) {
        set_error("attractive_prepare: %d points need %d column partitions, more than the %d supported", N, n_parts,
                  kMaxParts);
        return 1;
    }
    int cus = 256;
    TSNE_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, p->device));
    int strip_rows = div_up(N, cus);
    strip_rows = strip_rows < 64 ? 64 : strip_rows;
    strip_rows = strip_rows > kStripMax ? kStripMax : strip_rows;
    // (row within strip) << kColBits must fit 32 bits and strip_rows * K must fit the 32-bit segment offsets.
    // Segment offsets are 32-bit and a row sum of K fixed-point terms must stay below 2^62.
    if ((int64_t)strip_rows * K >= (int64_t)1 << 31 || K >= 4096) {
        set_error("attractive_prepare: num_neighbors = %d is too large for the blocked format", K);
        return 1;
    }
    p->strip_rows = strip_rows;
    p->n_strips = div_up(N, strip_rows);
    p->n_parts = n_parts;
    // A strip's work list: one item per referenced partition plus one per further kItemEntries entries.
    p->max_items = n_parts + (int)(((int64_t)strip_rows * K) / kItemEntries) + 1;
    p->seg_stride = 2 * p->max_items + 4;
    const size_t nnz = (size_t)N * K;
    bool ok = hipMalloc(&p->ent_p, sizeof(float) * nnz) == hipSuccess &&
              hipMalloc(&p->ent_c, sizeof(unsigned int) * nnz) == hipSuccess &&
              hipMalloc(&p->seg, sizeof(unsigned int) * (size_t)p->n_strips * p->seg_stride) == hipSuccess;
    if (!ok) {
        release_blocked(p);
        set_error("attractive_prepare: out of device memory for the re-blocked pattern (%zu bytes)", nnz * 8);
        return 1;
    }
    clear_pmax_kernel<<<1, 64, 0, s>>>(&p->scalars->vmax);
    TSNE_LAUNCHED(s);
    reblock_kernel<<<p->n_strips, kBlock, 0, s>>>(pij, indices, N, K, strip_rows, p->max_items, p->seg_stride, p->ent_p,
                                                  p->ent_c, p->seg,
                                                  &p->scalars->vmax);
    TSNE_LAUNCHED(s);
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(attractive_blocked_kernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBlockedLds));
    p->blocked_ready = true;
    return 0;
}

// Expects plan->yxy to hold the current embedding as (x, y) pairs.
int launch_attractive_blocked(tsne_hip_plan *p, float *attr, hipStream_t s) {
    if (!p->blocked_ready) {
        set_error("attractive: the re-blocked pattern has not been prepared");
        return 1;
    }
    if (profile_mark(p, kKernelAttractive, s)) return 1;
    attractive_blocked_kernel<<<p->n_strips, kBlock, kBlockedLds, s>>>(p->ent_p, p->ent_c, p->seg, p->yxy,
                                                                       &p->scalars->vmax, attr, p->num_points,
                                                                       p->num_neighbors, p->strip_rows, p->max_items,
                                                                       p->seg_stride);
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
