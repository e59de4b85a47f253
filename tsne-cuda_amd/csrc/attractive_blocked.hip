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
//     the probability and a packed (column within partition | row within strip),
//   * a strip's list names the partitions it references, in order, and the
//     entry at which each partition's run starts.
//
// A workgroup keeps its strip's positions and force accumulators in LDS and
// walks its entries; the partition the current entries refer to is staged in
// LDS, so every neighbour gather is an LDS read and every accumulation an LDS atomic.
// HBM sees the 8 bytes per entry once, coalesced, plus the positions of the
// referenced partitions once per workgroup (mostly served by the L2).
//
// Accumulators are 64-bit fixed point: on gfx950 an LDS float atomic add costs
// ~190 clocks per wave instruction while 64-bit integer LDS atomics run about
// 25x faster, and integer sums do not depend on the order of the additions.
// With p_max the largest probability, |contribution| <= p_max / 2 (because
// |d| / (1 + d^2) <= 1/2), so the scale 2^51 / p_max keeps every contribution
// below 2^50 and a row sum of K < 4096 terms below 2^62.
//
// Semantics are those of src/kernels/attr_forces.cu:129-184 of the reference;
// only the order of the additions inside a row differs.
#include <algorithm>
#include <cstdlib>
#include <vector>

#include "plan.h"
#include "stages.h"

namespace tsnehip {

namespace {

constexpr int kColBits = 11;
constexpr int kPartPoints = 2048;   // == 1 << kColBits; 16 KB of (x, y) pairs, two of them in LDS
constexpr int kStripMax = 3968;     // rows per strip: 31 KB of positions + 62 KB of accumulators; with the two
                                    // partitions 125 KB, which leaves 35 KB of a CU's LDS to the kernels of the
                                    // repulsive chain that run beside this one
constexpr double kRoundMagic = 6755399441055744.0;  // 1.5 * 2^52: adding it rounds a double to an integer
constexpr int kBlock = 1024;
constexpr int kMaxParts = 8192;     // column partitions: up to 16.7 M points
constexpr int kPrefetch = 4;        // entries per thread in one work item
constexpr int kStreamThreads = 768; // force kernel: waves 0-11 stream entries ...
constexpr int kStreamWaves = kStreamThreads / kWave;
constexpr int kLoadThreads = kBlock - kStreamThreads;  // ... waves 12-15 stage the partitions
constexpr int kLoadWaves = kLoadThreads / kWave;
constexpr unsigned int kItemEntries = kPrefetch * kStreamThreads;
// The second form ("direct"): where a strip's runs are short - ten million points in four clusters: a strip of
// 3968 rows references all 1220 partitions of its cluster, 290 entries each - staging 16 KB of positions per run
// costs several times the entries themselves, and every run is a hand-over between the kernel's two roles.  The
// entries then keep the same order (by partition, so that the workgroups, which walk their strips at about the
// same pace, ask the caches for the same stretch of the position array at about the same time), but their
// column is packed relative to a window of 2^19 points and the step kernel gathers every neighbour's position
// from memory itself: no staging, no roles, no waits.  What bounds it then is the number of distinct cache lines
// a wave's 64 position loads touch, so a strip's entries are sorted by column (a device radix sort by (strip,
// column), once): 64 consecutive entries of a run of 470 over a partition's 128 lines of 16 positions meet
// about 17 lines instead of 50.
constexpr int kWindowBits = 19;
constexpr int kWindowPoints = 1 << kWindowBits;
constexpr int kMaxWindows = 32;     // 2^24 points
constexpr int kDirectThreads = 1024;  // sixteen waves, all of them streaming
constexpr int kDirectWaves = kDirectThreads / kWave;
constexpr unsigned int kDirectItem = kPrefetch * kDirectThreads;  // entries per item of the direct form
constexpr unsigned int kDirectPiece = 128;  // consecutive entries of an item that one wave's lanes hold (two each)
constexpr int kDirectStripMax = 6784;  // rows per strip of the direct form when the strips outnumber the compute
                                       // units anyway: 159 KB of positions and accumulators, the whole LDS
static_assert((kDirectStripMax - 1) >> (32 - kWindowBits) == 0, "row within strip and column within window share 32 bits");
constexpr int kSpinLimit = 1 << 18; // polls of an LDS counter before a wave gives up waiting (about ten milliseconds;
                                    // a wait normally ends within a microsecond): every wave reaches the kernel's end.
                                    // TSNE_ATTRACTIVE_SPIN_LIMIT (read when the pattern is prepared) overrides it, so
                                    // that a test can make the waits fail (0: every wait) without any kernel hanging.

// ---------------------------------------------------------------------------
// Re-blocking: one workgroup per strip.  Histogram of the strip's entries over
// the partitions, exclusive scan, then a scatter that ranks entries inside a
// partition with LDS atomics.  A thread owns kSlotsPerThread consecutive
// partition slots in the scans.
// ---------------------------------------------------------------------------
constexpr int kSlotsPerThread = kMaxParts / kBlock;
static_assert(kMaxParts % kBlock == 0, "the partition scans give every thread the same number of slots");

// Exclusive prefix sums over all kMaxParts slots (thread t holds slots t * kSlotsPerThread ...); returns the
// total.  scan: kBlock words of LDS.  Ends with the LDS array free for reuse.
__device__ __forceinline__ unsigned int scan_slots(const unsigned int (&value)[kSlotsPerThread],
                                                   unsigned int (&before)[kSlotsPerThread], unsigned int *scan,
                                                   int tid) {
    unsigned int mine = 0u;
#pragma unroll
    for (int i = 0; i < kSlotsPerThread; ++i) {
        before[i] = mine;
        mine += value[i];
    }
    scan[tid] = mine;
    __syncthreads();
    for (int off = 1; off < kBlock; off <<= 1) {  // inclusive Hillis-Steele scan of the per-thread sums
        const unsigned int add = tid >= off ? scan[tid - off] : 0u;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    const unsigned int base = scan[tid] - mine;
    const unsigned int total = scan[kBlock - 1];
#pragma unroll
    for (int i = 0; i < kSlotsPerThread; ++i) before[i] += base;
    __syncthreads();
    return total;
}

// Where entry `pos` of a strip lives: the strips' items are interleaved (item 0 of every strip, then item 1 of
// every strip, ...).  The workgroups of the force kernel advance through their strips at about the same pace, so
// at any moment the chip reads one window of a few items' worth of consecutive addresses, like a plain
// sequential read, instead of one stream per strip megabytes apart.  Every item starts on a 16-byte boundary.
// Inside an item, every 128 entries are stored as 64 pairs (j, j + 64): a lane of the force kernel loads a pair
// at a time, and the 64 lanes of a wave then hold 64 consecutive entries in each half of their registers
// (consecutive entries belong to consecutive rows, whose accumulators lie in different LDS banks).
template <unsigned int ITEM = kItemEntries>
__device__ __forceinline__ size_t entry_slot(unsigned int pos, int strip, int n_strips) {
    const unsigned int item = pos / ITEM;
    const unsigned int in_item = pos - item * ITEM;
    const unsigned int j = in_item & 127u;
    return ((size_t)item * n_strips + strip) * ITEM + (in_item - j) + 2u * (j & 63u) + (j >> 6);
}
static_assert(kItemEntries % 128 == 0, "items hold whole groups of 64 entry pairs");

// Order of the entries inside a partition's run.  The force kernel's wave handles 64 consecutive entries at a
// time and touches, per entry, the position and the two accumulators of the entry's row: 8-byte slots, 32 of
// which span the LDS banks.  A run is therefore dealt out by row residue: its entries are bucketed by
// (row mod 32) and emitted round robin, one from every bucket that still has one, so that any 64 consecutive
// entries hit every bank pair twice (until the fuller buckets are all that is left, at the end of the run).
// That needs two counters per (referenced partition, residue) in LDS; a strip that references more than
// kBalancedParts partitions keeps the order of arrival instead (neighbour slot by neighbour slot).
constexpr int kBalancedParts = 320;
constexpr int kResidues = 32;
constexpr int kResidueStride = kResidues + 1;  // odd: the 32 counters of different partitions spread over the banks
constexpr size_t kReblockLds = sizeof(unsigned int) * 2 * kBalancedParts * kResidueStride;

__global__ __launch_bounds__(kBlock) void reblock_kernel(const float *__restrict__ pij, const int *__restrict__ idx,
                                                         int N, int K, const int *__restrict__ strip_row0,
                                                         int list_words,
                                                         int seg_stride, float *__restrict__ ent_p,
                                                         unsigned int *__restrict__ seg, float *__restrict__ p_max) {
    __shared__ unsigned int cursor[kMaxParts];
    __shared__ unsigned short fresh_of[kMaxParts];  // partition -> its place among the partitions the strip references
    __shared__ unsigned int scan[kBlock];
    extern __shared__ unsigned int residue_count[];                             // [place][kResidueStride]
    unsigned int *residue_cursor = residue_count + kBalancedParts * kResidueStride;  // same shape
    const int tid = threadIdx.x;
    const int strip = blockIdx.x;
    const int row0 = strip_row0[strip];
    const int nrows = strip_row0[strip + 1] - row0;
    const size_t base = (size_t)row0 * K;
    const unsigned int count = (unsigned int)nrows * (unsigned int)K;
    for (int b = tid; b < kMaxParts; b += kBlock) cursor[b] = 0;
    __syncthreads();
    for (unsigned int e = tid; e < count; e += kBlock) atomicAdd(&cursor[idx[base + e] / kPartPoints], 1u);
    __syncthreads();
    unsigned int mine[kSlotsPerThread], first[kSlotsPerThread];
#pragma unroll
    for (int i = 0; i < kSlotsPerThread; ++i) mine[i] = cursor[tid * kSlotsPerThread + i];
    scan_slots(mine, first, scan, tid);
#pragma unroll
    for (int i = 0; i < kSlotsPerThread; ++i) cursor[tid * kSlotsPerThread + i] = first[i];
    // Layout of a strip's list: {first row, partitions referenced, rows, -}, then for the k-th referenced partition the
    // first entry of its run (n_parts + 4 words, unused ones hold ~0), then the partitions themselves in the
    // same order (n_parts words).
    unsigned int *hdr = seg + (size_t)strip * seg_stride;
    unsigned int *run_start = hdr + 4;
    unsigned int *fresh_parts = run_start + list_words;
    // Second scan, over the "referenced at all" flags: the order in which partitions are opened.
    unsigned int flag[kSlotsPerThread], order[kSlotsPerThread];
#pragma unroll
    for (int i = 0; i < kSlotsPerThread; ++i) flag[i] = mine[i] > 0u ? 1u : 0u;
    const unsigned int n_fresh = scan_slots(flag, order, scan, tid);
#pragma unroll
    for (int i = 0; i < kSlotsPerThread; ++i)
        if (flag[i]) {
            fresh_parts[order[i]] = (unsigned int)(tid * kSlotsPerThread + i);
            run_start[order[i]] = first[i];
            fresh_of[tid * kSlotsPerThread + i] = (unsigned short)order[i];
        }
    for (unsigned int b = n_fresh + tid; b < (unsigned int)list_words; b += kBlock) run_start[b] = ~0u;
    if (tid == 0) {
        hdr[0] = (unsigned int)row0;
        hdr[1] = n_fresh;
        hdr[2] = (unsigned int)nrows;
    }
    const bool balanced = n_fresh <= (unsigned int)kBalancedParts;
    if (balanced) {
        for (unsigned int b = tid; b < 2u * kBalancedParts * kResidueStride; b += kBlock) residue_count[b] = 0u;
        __syncthreads();
        for (unsigned int e = tid; e < count; e += kBlock) {
            const unsigned int row_local = e / (unsigned int)K;
            const unsigned int place = fresh_of[idx[base + e] / kPartPoints];
            atomicAdd(&residue_count[place * kResidueStride + (row_local & (kResidues - 1))], 1u);
        }
    }
    __syncthreads();
    // Entries are visited neighbour slot by neighbour slot, so that the entries of one row lie far apart
    // in a partition's run (also within a residue's bucket): a wave of the force kernel never meets a row twice.
    float biggest = 0.0f;
    for (unsigned int v = tid; v < count; v += kBlock) {
        const unsigned int slot = v / (unsigned int)nrows;
        const unsigned int row_local = v - slot * (unsigned int)nrows;
        const unsigned int e = row_local * (unsigned int)K + slot;
        const int col = idx[base + e];
        const int part = col / kPartPoints;
        unsigned int pos;
        if (balanced) {
            const unsigned int q = row_local & (kResidues - 1);
            const unsigned int *counts = residue_count + fresh_of[part] * kResidueStride;
            const unsigned int j = atomicAdd(&residue_cursor[fresh_of[part] * kResidueStride + q], 1u);
            // Round j of the dealing: everything of the rounds before it, then the buckets before q that reach round j.
            pos = cursor[part];
#pragma unroll 8
            for (unsigned int other = 0; other < (unsigned int)kResidues; ++other) {
                const unsigned int c = counts[other];
                pos += min(c, j) + ((other < q && c > j) ? 1u : 0u);
            }
        } else {
            pos = atomicAdd(&cursor[part], 1u);
        }
        const float pv = pij[base + e];
        biggest = fmaxf(biggest, fabsf(pv));
        reinterpret_cast<uint2 *>(ent_p)[entry_slot(pos, strip, (int)gridDim.x)] =
            make_uint2(__float_as_uint(pv), (unsigned int)(col - part * kPartPoints) | (row_local << kColBits));
    }
    biggest = group_max<kWave>(biggest);
    // Non-negative floats order like their bit patterns.
    if ((tid & (kWave - 1)) == 0) atomicMax(reinterpret_cast<unsigned int *>(p_max), __float_as_uint(biggest));
}

__global__ void clear_pmax_kernel(float *p_max) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *p_max = 0.0f;
}

// ---------------------------------------------------------------------------
// One workgroup per strip; dynamic LDS: part[2][kPartPoints] float2, then
// yi[kStripMax] float2, then acc_x[kStripMax] and acc_y[kStripMax], 64-bit fixed point.
//
// The waves have two roles.  Waves 0-11 stream the strip's entries in items of
// kItemEntries (three rotating register sets, two items in flight, all loads
// unconditional so that the outstanding-load counts the compiler works with are
// exact) and do the LDS gathers and accumulations.  Waves 12-15 only stage
// partitions: the k-th partition the strip references goes into LDS buffer
// k & 1, the two after the one being written wait in registers.
//
// No barrier separates the roles, only two counters per LDS buffer b:
//   staged[b]   += 1 by every staging wave once its part of a partition is written
//                  to b; a streaming wave enters run k when
//                  staged[k & 1] >= kLoadWaves * (k / 2 + 1),
//   released[b] += 1 by every streaming wave that leaves a run in b; a staging wave
//                  overwrites buffer k & 1 with partition k once
//                  released[k & 1] >= kStreamWaves * (k / 2), i.e. all streaming
//                  waves have left partition k - 2.
// Partition k + 2 is only written after every streaming wave has left partition k,
// which they only entered after every staging wave had written it: a buffer's
// counters never run ahead by a generation, so the thresholds are exact.
// A streaming wave therefore never waits for another streaming wave, and waits for
// the staging waves only when they are less than one partition ahead.  A count
// is made after a release fence and a wait ends with an acquire fence, both at
// workgroup scope and on the LDS address space only (the entry loads from memory
// stay in flight across them; measured cost: none); the counters only grow.
// Every wait is a bounded poll.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void add_force(unsigned long long *acc, unsigned int rl, float vx, float vy,
                                          double scale, int y_offset = kStripMax) {
    // magic + v * scale is a double in [2^52, 2^53), where doubles are the integers: its bit pattern is the
    // magic's plus round(v * scale).  The patterns themselves are summed; every row has exactly K entries, so
    // its accumulators start at -K times the magic's pattern (mod 2^64) and end at the sum of the integers.
    const double tx = fma((double)vx, scale, kRoundMagic);
    const double ty = fma((double)vy, scale, kRoundMagic);
    // x sums and y sums live in separate arrays: consecutive rows then fall
    // into consecutive 8-byte slots and the atomics of a wave spread over all banks.
    atomicAdd(&acc[rl], (unsigned long long)__double_as_longlong(tx));
    atomicAdd(&acc[y_offset + rl], (unsigned long long)__double_as_longlong(ty));
}

// Polls *counter until it reaches `need`; after kSpinLimit polls the wave sets *gave_up and goes on (the
// workgroup then reports it and writes NaN forces).  The compiler barriers keep the buffer accesses of the
// caller on their side of the wait.
__device__ __forceinline__ void wait_for_count(const unsigned int *counter, unsigned int need, int spin_limit,
                                               unsigned int *gave_up) {
    asm volatile("" ::: "memory");
    for (int spin = 0;; ++spin) {
        if (spin >= spin_limit) {  // (a limit of 0 gives up without looking)
            *gave_up = 1u;
            break;
        }
        if (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= need) break;
        __builtin_amdgcn_s_sleep(1);
    }
    // Acquire, for LDS only: the buffer accesses that follow are not issued before the count has been seen.
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// One count from this wave, after everything it has issued to the LDS so far.
__device__ __forceinline__ void count_wave(unsigned int *counter, int lane) {
    // Release, for LDS only (the wave's loads from memory stay in flight): every LDS access issued so far has
    // been performed before the count is.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    if (lane == 0) __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    asm volatile("" ::: "memory");
}

// RUNTIME_LIMIT: the poll limit is the argument (the override for tests); otherwise it is the constant, with
// which the compiler lays the wait loops out better (197 against 203 us per launch at a million points).
// At most 64 registers (the second launch bound): the kernel's sixteen waves then take half of a compute unit's
// register file and leave room for the eight waves of 128 registers of a spreading workgroup beside them.
template <bool RUNTIME_LIMIT>
__global__ __launch_bounds__(kBlock, 8) void attractive_blocked_kernel(const float *__restrict__ ent_p,
                                                                    const unsigned int *__restrict__ seg,
                                                                    const float2 *__restrict__ yxy,
                                                                    LoopScalars *__restrict__ scalars,
                                                                    float *__restrict__ attr, int N, int K,
                                                                    int list_words, int seg_stride,
                                                                    int spin_limit_arg) {
    const int spin_limit = RUNTIME_LIMIT ? spin_limit_arg : kSpinLimit;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    float2 *part = reinterpret_cast<float2 *>(lds_raw);  // two buffers of kPartPoints
    float2 *yi = part + 2 * kPartPoints;
    unsigned long long *acc = reinterpret_cast<unsigned long long *>(yi + kStripMax);
    __shared__ unsigned int staged[2], released[2], gave_up;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int strip = blockIdx.x;
    // The list is read through the constant address space: it is never written while this
    // kernel runs, and constant-space loads at uniform addresses are scalar loads, which do not
    // queue behind the vector loads in flight.
    typedef const __attribute__((address_space(4))) unsigned int *ConstWords;
    ConstWords hdr = (ConstWords)(seg + (size_t)strip * seg_stride);
    const int row0 = (int)hdr[0];
    const int n_fresh = (int)hdr[1];
    const int nrows = (int)hdr[2];
    ConstWords run_start = hdr + 4;  // ~0 after the last run
    ConstWords fresh_parts = run_start + list_words;
    const float pm = scalars->vmax;
    const double scale = pm > 0.0f ? 2251799813685248.0 / (double)pm : 1.0;  // 2^51 / p_max

    const unsigned long long acc_start =
        0ull - (unsigned long long)K * (unsigned long long)__double_as_longlong(kRoundMagic);
    for (int r = tid; r < nrows; r += kBlock) {
        yi[r] = yxy[row0 + r];
        acc[r] = acc_start;
        acc[kStripMax + r] = acc_start;
    }
    if (tid == 0) {
        staged[0] = 0u;
        staged[1] = 0u;
        released[0] = 0u;
        released[1] = 0u;
        gave_up = 0u;
    }
    __syncthreads();

    if (tid >= kStreamThreads) {
        // ---- staging waves ----
        const int lt = tid - kStreamThreads;
        constexpr int kPartLoads = kPartPoints / (2 * kLoadThreads);  // float4 (two points) loads per thread
        static_assert(kPartPoints % (2 * kLoadThreads) == 0, "partition staging assumes whole float4 rounds");
        // A native vector type with compile-time indices: an array of HIP float4 structs ends up
        // in scratch memory, where every load waits for the one before.
        typedef float Quad __attribute__((ext_vector_type(4)));
        const Quad *yxy4 = reinterpret_cast<const Quad *>(yxy);
        Quad *part4 = reinterpret_cast<Quad *>(part);
        const int last_pair_all = (N - 1) / 2;  // yxy is padded, so a pair may run one point past N
        // The fetches are unconditional (past the last partition they repeat it) so that the compiler's
        // outstanding-load counts are exact and a write to LDS waits for its own register set only.
        Quad stage_a[kPartLoads], stage_b[kPartLoads];
        auto fetch = [&](Quad (&stage)[kPartLoads], int k) {
            const int p = (int)fresh_parts[min(k, n_fresh - 1)];
#pragma unroll
            for (int u = 0; u < kPartLoads; ++u)
                stage[u] = yxy4[min(p * (kPartPoints / 2) + lt + u * kLoadThreads, last_pair_all)];
        };
        auto publish = [&](const Quad (&stage)[kPartLoads], int k) {
            wait_for_count(&released[k & 1], (unsigned int)(kStreamWaves * (k >> 1)), spin_limit, &gave_up);
            Quad *dst = part4 + (k & 1) * (kPartPoints / 2);
#pragma unroll
            for (int u = 0; u < kPartLoads; ++u) dst[lt + u * kLoadThreads] = stage[u];
            count_wave(&staged[k & 1], lane);
        };
        if (n_fresh > 0) {
            fetch(stage_a, 0);
            fetch(stage_b, 1);
            int k = 0;
            for (; k + 1 < n_fresh; k += 2) {
                publish(stage_a, k);
                fetch(stage_a, k + 2);
                publish(stage_b, k + 1);
                fetch(stage_b, k + 3);
            }
            if (k < n_fresh) publish(stage_a, k);
        }
    } else {
        // ---- streaming waves ----
        typedef unsigned int Entry __attribute__((ext_vector_type(2)));  // {probability bits, packed row / column}
        const Entry *ent = reinterpret_cast<const Entry *>(ent_p);
        const unsigned int count = (unsigned int)nrows * (unsigned int)K;
        const unsigned int n_items = (count + kItemEntries - 1u) / kItemEntries;
        // A lane loads two neighbouring entries at a time (16 bytes); the entries are read once per launch and
        // marked as such, so that they do not push the partitions' positions out of the caches.
        typedef unsigned int EntryPair __attribute__((ext_vector_type(4)));
        static_assert(kPrefetch % 2 == 0, "entries are loaded in pairs");
        struct PhaseRegs {
            Entry en[kPrefetch];  // en[2 j + h]: entry 128 ((tid + j kStreamThreads) / 64) + 64 h + lane of the item
        };
        const EntryPair *pairs = reinterpret_cast<const EntryPair *>(ent) + (size_t)strip * (kItemEntries / 2) + tid;
        const size_t item_pitch = (size_t)gridDim.x * (kItemEntries / 2);  // pairs from one item of a strip to the next
        auto issue = [&](PhaseRegs &R, unsigned int item) {
            const EntryPair *src = pairs + (size_t)min(item, n_items - 1u) * item_pitch;
#pragma unroll
            for (int j = 0; j < kPrefetch / 2; ++j) {
                const EntryPair v = __builtin_nontemporal_load(src + j * kStreamThreads);
                R.en[2 * j] = Entry{v.x, v.y};
                R.en[2 * j + 1] = Entry{v.z, v.w};
            }
        };
        // The run this wave is in (-1: none yet), the buffer that holds its partition, and where the next
        // two runs start (fetched a run ahead of their use; ~0 when there is none).
        int run = -1;
        const float2 *cur = part;
        unsigned int next_start = run_start[0], after_next_start = run_start[1];
        // Entries [from, to) of the item, all in the current run.
        auto span = [&](PhaseRegs &R, unsigned int first, unsigned int from, unsigned int to) {
#pragma unroll
            for (int k = 0; k < kPrefetch; ++k) {
                const unsigned int t = first + 128 * ((tid + (k >> 1) * kStreamThreads) >> 6) + 64 * (k & 1) + lane;
                if (t >= from && t < to) {
                    const unsigned int rl = R.en[k].y >> kColBits;
                    const float2 yj = cur[R.en[k].y & ((1u << kColBits) - 1u)];
                    const float2 y0 = yi[rl];
                    const float dx = y0.x - yj.x, dy = y0.y - yj.y;
                    const float w = __uint_as_float(R.en[k].x) * __builtin_amdgcn_rcpf(1.0f + dx * dx + dy * dy);
                    add_force(acc, rl, w * dx, w * dy, scale);
                }
            }
        };
        auto consume = [&](PhaseRegs &R, unsigned int item) {
            const unsigned int first = item * kItemEntries;
            const unsigned int end = min(first + kItemEntries, count);  // (an item past the last one: end < first)
            unsigned int from = first;
            while (next_start < end) {  // a run starts inside this item
                span(R, first, from, next_start);
                if (run >= 0) count_wave(&released[run & 1], lane);
                ++run;
                wait_for_count(&staged[run & 1], (unsigned int)(kLoadWaves * ((run >> 1) + 1)), spin_limit, &gave_up);
                cur = part + (run & 1) * kPartPoints;
                from = next_start;
                next_start = after_next_start;
                after_next_start = run_start[run + 2];
            }
            span(R, first, from, end);
        };
        // Prefetch distance two: while item p is consumed, the loads of items p+1 and p+2 are in flight.
        // Items past the last one load the last item again and consume nothing.
        PhaseRegs R0, R1, R2;
        issue(R0, 0u);
        issue(R1, 1u);
        for (unsigned int p = 0; p < n_items; p += 3) {
            issue(R2, p + 2);
            consume(R0, p);
            issue(R0, p + 3);
            consume(R1, p + 1);
            issue(R1, p + 4);
            consume(R2, p + 2);
        }
    }
    __syncthreads();
    const double inv_scale = gave_up ? (double)NAN : 1.0 / scale;
    for (int r = tid; r < nrows; r += kBlock) {
        attr[row0 + r] = (float)((double)(long long)acc[r] * inv_scale);
        attr[N + row0 + r] = (float)((double)(long long)acc[kStripMax + r] * inv_scale);
    }
    if (gave_up && tid == 0) atomicAdd(&scalars->wait_timeouts, 1u);
}

// ---------------------------------------------------------------------------
// Preparation of the direct form.  Sort key of an entry: (row within strip) << 40 | strip << 24 | column; the
// sort orders by the low 24 + strip bits, i.e. by (strip, column), and is stable.  A strip's entries then are the
// rows * K sorted pairs from row0 * K on.  Every window's entries are padded to a multiple of kDirectPiece, so
// that each piece of that many consecutive entries - what one wave of the step kernel takes at a time - lies in
// one window; the padding entries name a row past the strip's last.  A strip's list: {first row, windows, rows,
// entries with padding}, then the entry at which every window's entries start, the padded entry count, ~0, ~0.
// ---------------------------------------------------------------------------
typedef unsigned long long u64;
constexpr int kDirectColBits = 24;
static_assert(kMaxWindows * kWindowPoints == 1 << kDirectColBits, "columns of the direct form fit their key bits");

// uniform_rows > 0: every strip has that many rows (the last one fewer); otherwise the boundaries are searched
// (at most 1024 strips).
__global__ __launch_bounds__(256) void direct_keys_kernel(const float *__restrict__ pij, const int *__restrict__ idx,
                                                          long long nnz, int K, const int *__restrict__ strip_row0,
                                                          int n_strips, int uniform_rows, u64 *__restrict__ keys,
                                                          float *__restrict__ vals) {
    __shared__ int bounds[1025];
    if (!uniform_rows) {
        for (int b = threadIdx.x; b <= n_strips; b += 256) bounds[b] = strip_row0[b];
        __syncthreads();
    }
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < nnz; e += (long long)gridDim.x * 256) {
        const int i = (int)(e / K);
        int strip, first;
        if (uniform_rows) {
            strip = i / uniform_rows;
            first = strip * uniform_rows;
        } else {
            int lo = 0, hi = n_strips;  // the last boundary <= i
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (bounds[mid] <= i) lo = mid; else hi = mid;
            }
            strip = lo;
            first = bounds[lo];
        }
        keys[e] = ((u64)(unsigned int)(i - first) << 40) | ((u64)(unsigned int)strip << kDirectColBits) |
                  (u64)(unsigned int)idx[e];
        vals[e] = pij[e];
    }
}

// One workgroup of 128 threads per strip: where the strip's entries of every window start (a binary search in
// its sorted keys), the padding ahead of every window (wpad: kMaxWindows + 1 words per strip), the strip's list,
// and the padding entries themselves.
__global__ __launch_bounds__(128) void direct_windows_kernel(const u64 *__restrict__ keys, int K,
                                                             const int *__restrict__ strip_row0, int n_windows,
                                                             unsigned int *__restrict__ wseg, int wseg_stride,
                                                             unsigned int *__restrict__ wpad,
                                                             float *__restrict__ ent_p) {
    __shared__ unsigned int ustart[kMaxWindows + 1], pad[kMaxWindows + 1];
    const int strip = blockIdx.x, tid = threadIdx.x;
    const int row0 = strip_row0[strip], nrows = strip_row0[strip + 1] - row0;
    const u64 *mine = keys + (size_t)row0 * K;
    const unsigned int count = (unsigned int)nrows * (unsigned int)K;
    if (tid <= n_windows) {
        const unsigned int want = (unsigned int)tid << kWindowBits;  // first column of the window
        unsigned int lo = 0u, hi = count;                           // first entry whose column is >= want
        while (lo < hi) {
            const unsigned int mid = (lo + hi) >> 1;
            if ((unsigned int)(mine[mid] & ((1u << kDirectColBits) - 1u)) < want) lo = mid + 1u; else hi = mid;
        }
        ustart[tid] = tid == n_windows ? count : lo;
    }
    __syncthreads();
    if (tid == 0) {
        unsigned int total = 0u;
        for (int w = 0; w < n_windows; ++w) {
            pad[w] = total;
            const unsigned int len = ustart[w + 1] - ustart[w];
            total += ((len + kDirectPiece - 1u) & ~(kDirectPiece - 1u)) - len;
        }
        pad[n_windows] = total;
    }
    __syncthreads();
    unsigned int *whdr = wseg + (size_t)strip * wseg_stride;
    if (tid <= n_windows) {
        wpad[(size_t)strip * (kMaxWindows + 1) + tid] = pad[tid];
        whdr[4 + tid] = ustart[tid] + pad[tid];
    }
    if (tid == 0) {
        whdr[0] = (unsigned int)row0;
        whdr[1] = (unsigned int)n_windows;
        whdr[2] = (unsigned int)nrows;
        whdr[3] = count + pad[n_windows];
        whdr[4 + n_windows + 1] = ~0u;
        whdr[4 + n_windows + 2] = ~0u;
    }
    for (int w = 0; w < n_windows; ++w) {
        const unsigned int dummies = pad[w + 1] - pad[w];  // they follow the window's last entry
        if ((unsigned int)tid < dummies)
            reinterpret_cast<uint2 *>(ent_p)[entry_slot<kDirectItem>(ustart[w + 1] + pad[w] + tid, strip, (int)gridDim.x)] =
                make_uint2(0u, ~0u);
    }
}

__global__ __launch_bounds__(256) void direct_emit_kernel(const u64 *__restrict__ keys, const float *__restrict__ vals,
                                                          long long nnz, int K, const int *__restrict__ strip_row0,
                                                          int n_strips, const unsigned int *__restrict__ wpad,
                                                          float *__restrict__ ent_p, float *__restrict__ p_max) {
    float biggest = 0.0f;
    for (long long q = (long long)blockIdx.x * 256 + threadIdx.x; q < nnz; q += (long long)gridDim.x * 256) {
        const u64 key = keys[q];
        const unsigned int col = (unsigned int)(key & ((1u << kDirectColBits) - 1u));
        const int strip = (int)((key >> kDirectColBits) & 0xffffu);
        const unsigned int row_local = (unsigned int)(key >> 40);
        const unsigned int e = (unsigned int)(q - (long long)strip_row0[strip] * K);
        const unsigned int pos = e + wpad[(size_t)strip * (kMaxWindows + 1) + (col >> kWindowBits)];
        const float pv = vals[q];
        biggest = fmaxf(biggest, fabsf(pv));
        reinterpret_cast<uint2 *>(ent_p)[entry_slot<kDirectItem>(pos, strip, n_strips)] =
            make_uint2(__float_as_uint(pv), (col & (kWindowPoints - 1u)) | (row_local << kWindowBits));
    }
    biggest = group_max<kWave>(biggest);
    if ((threadIdx.x & (kWave - 1)) == 0) atomicMax(reinterpret_cast<unsigned int *>(p_max), __float_as_uint(biggest));
}

// ---------------------------------------------------------------------------
// Direct form of the step kernel: one workgroup (sixteen waves) per strip; LDS holds the strip's positions and
// its force accumulators, the entries stream from memory as in the staged kernel (three rotating register sets,
// two items in flight), and every entry's neighbour position is a load of its own, issued for all entries of
// the item before the first is used.  Same arithmetic, same fixed-point sums.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kDirectThreads) void attractive_direct_kernel(const float *__restrict__ ent_p,
                                                                        const unsigned int *__restrict__ wseg,
                                                                        const float2 *__restrict__ yxy,
                                                                        const LoopScalars *__restrict__ scalars,
                                                                        float *__restrict__ attr, int N, int K,
                                                                        int wseg_stride, int rows_cap) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    float2 *yi = reinterpret_cast<float2 *>(lds_raw);
    unsigned long long *acc = reinterpret_cast<unsigned long long *>(yi + rows_cap);
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int strip = blockIdx.x;
    typedef const __attribute__((address_space(4))) unsigned int *ConstWords;
    ConstWords hdr = (ConstWords)(wseg + (size_t)strip * wseg_stride);
    const int row0 = (int)hdr[0];
    const int nrows = (int)hdr[2];
    ConstWords window_start = hdr + 4;  // the count after the last window, then ~0
    const float pm = scalars->vmax;
    const double scale = pm > 0.0f ? 2251799813685248.0 / (double)pm : 1.0;  // 2^51 / p_max
    const unsigned long long acc_start =
        0ull - (unsigned long long)K * (unsigned long long)__double_as_longlong(kRoundMagic);
    for (int r = tid; r < nrows; r += kDirectThreads) {
        yi[r] = yxy[row0 + r];
        acc[r] = acc_start;
        acc[rows_cap + r] = acc_start;
    }
    __syncthreads();

    typedef unsigned int Entry __attribute__((ext_vector_type(2)));  // {probability bits, packed row / column}
    typedef unsigned int EntryPair __attribute__((ext_vector_type(4)));
    const unsigned int count = hdr[3];  // (with the windows' padding)
    const unsigned int n_items = (count + kDirectItem - 1u) / kDirectItem;
    struct PhaseRegs {
        Entry en[kPrefetch];  // en[2 j + h]: entry 128 ((tid + j kDirectThreads) / 64) + 64 h + lane of the item
    };
    const EntryPair *pairs = reinterpret_cast<const EntryPair *>(ent_p) + (size_t)strip * (kDirectItem / 2) + tid;
    const size_t item_pitch = (size_t)gridDim.x * (kDirectItem / 2);
    auto issue = [&](PhaseRegs &R, unsigned int item) {
        const EntryPair *src = pairs + (size_t)min(item, n_items - 1u) * item_pitch;
#pragma unroll
        for (int j = 0; j < kPrefetch / 2; ++j) {
            const EntryPair v = __builtin_nontemporal_load(src + j * kDirectThreads);
            R.en[2 * j] = Entry{v.x, v.y};
            R.en[2 * j + 1] = Entry{v.z, v.w};
        }
    };
    // A lane's four entries of an item are two pairs (t, t + 64), one pair in each of two pieces of kDirectPiece
    // consecutive entries, and a piece lies in one window: the window of each of the wave's two pieces is tracked
    // in scalar registers (windows are listed whether or not the strip has entries in them).
    static_assert(kPrefetch == 4 && kDirectPiece == 2 * kWave, "two pieces of 128 entries per wave and item");
    const unsigned int wave = (unsigned int)__builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_windows = (int)hdr[1];
    int win[2] = {0, 0};
    unsigned int boundary[2] = {window_start[1], window_start[1]};  // where the window after win[j] starts
    // Item R: every position load first, then the loads of the item two ahead (into Rn), then the arithmetic.
    // Loads return in the order of issue as far as a wave's counters can tell: entry loads issued ahead of the
    // position loads would have to land (from HBM) before the first position could be used.  Everything is
    // unconditional - an item past the last one loads the last item again and none of its entries is in range -
    // so that the outstanding-load counts the compiler works with are exact.
    auto consume = [&](PhaseRegs &R, unsigned int item, PhaseRegs &Rn, unsigned int next_item) {
        const unsigned int first = item * kDirectItem;
        float2 yj[kPrefetch];
        bool on[kPrefetch];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const unsigned int t0 = first + kDirectPiece * (wave + (unsigned int)j * kDirectWaves);
            while (t0 >= boundary[j]) {  // (rare: a few dozen times per strip)
                ++win[j];
                boundary[j] = window_start[win[j] + 1];
            }
            const float2 *base = yxy + (size_t)min(win[j], n_windows - 1) * kWindowPoints;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int k = 2 * j + h;
                const unsigned int t = t0 + 64u * (unsigned int)h + (unsigned int)lane;
                on[k] = t < count && (R.en[k].y >> kWindowBits) < (unsigned int)nrows;
                yj[k] = base[on[k] ? (R.en[k].y & (kWindowPoints - 1u)) : 0u];
            }
        }
        issue(Rn, next_item);
#pragma unroll
        for (int k = 0; k < kPrefetch; ++k) {
            if (on[k]) {
                const unsigned int rl = R.en[k].y >> kWindowBits;
                const float2 y0 = yi[rl];
                const float dx = y0.x - yj[k].x, dy = y0.y - yj[k].y;
                const float w = __uint_as_float(R.en[k].x) * __builtin_amdgcn_rcpf(1.0f + dx * dx + dy * dy);
                add_force(acc, rl, w * dx, w * dy, scale, rows_cap);
            }
        }
    };
    PhaseRegs R0, R1, R2;
    issue(R0, 0u);
    issue(R1, 1u);
    for (unsigned int p = 0; p < n_items; p += 3) {
        consume(R0, p, R2, p + 2);
        consume(R1, p + 1, R0, p + 3);
        consume(R2, p + 2, R1, p + 4);
    }
    __syncthreads();
    const double inv_scale = 1.0 / scale;
    for (int r = tid; r < nrows; r += kDirectThreads) {
        attr[row0 + r] = (float)((double)(long long)acc[r] * inv_scale);
        attr[N + row0 + r] = (float)((double)(long long)acc[rows_cap + r] * inv_scale);
    }
}

constexpr size_t kDirectLds = sizeof(float2) * kDirectStripMax + sizeof(unsigned long long) * 2 * kDirectStripMax;
static_assert(kDirectLds <= 160 * 1024, "one workgroup must fit the 160 KB of LDS");

constexpr size_t kBlockedLds =
    sizeof(float2) * 2 * kPartPoints + sizeof(float2) * kStripMax + sizeof(unsigned long long) * 2 * kStripMax;
static_assert(kBlockedLds <= 160 * 1024, "one workgroup must fit the 160 KB of LDS");

}  // namespace

// ---------------------------------------------------------------------------
// Strip boundaries.  What a strip costs the force kernel is its entries plus a fixed price for every column
// partition it references (staging the partition, and a second pass over the item in which its run starts):
// measured at a million points, 0.42 us per partition against 0.21 ns per entry, i.e. a partition costs what
// about 2000 entries do.  With equal strips the few that straddle two clusters of the data reference twice the
// partitions of the others and finish 40 % later, and the launch lasts as long as its slowest workgroup.  When
// all strips run at once (no more strips than CUs) their boundaries are therefore chosen so that the predicted
// costs are equal: the rows are cut into micro-strips of 64, a kernel finds the partitions every micro-strip
// references (a bitmap), and the host merges consecutive micro-strips greedily under the smallest cost limit
// that needs no more strips than there are CUs (bisection on the limit).
// ---------------------------------------------------------------------------
namespace {

constexpr int kMicroRows = 64;
constexpr long long kPartCostEntries = 2000;

__global__ __launch_bounds__(256) void micro_strip_parts_kernel(const int *__restrict__ idx, int N, int K, int words,
                                                                unsigned int *__restrict__ bitmaps) {
    extern __shared__ unsigned int bits[];
    for (int w = threadIdx.x; w < words; w += 256) bits[w] = 0u;
    __syncthreads();
    const int row0 = blockIdx.x * kMicroRows;
    const int nrows = min(kMicroRows, N - row0);
    const size_t base = (size_t)row0 * K;
    for (int e = threadIdx.x; e < nrows * K; e += 256) {
        const int part = idx[base + e] / kPartPoints;
        atomicOr(&bits[part >> 5], 1u << (part & 31));
    }
    __syncthreads();
    for (int w = threadIdx.x; w < words; w += 256) bitmaps[(size_t)blockIdx.x * words + w] = bits[w];
}

}  // namespace

// row0 (n_strips + 1 entries, ascending, row0[0] = 0, row0[n_strips] = N) of strips with at most kStripMax rows
// and equal predicted cost, at most max_strips of them.
static int balanced_strips(const int *indices, int N, int K, int n_parts, int max_strips, std::vector<int> &row0,
                           hipStream_t s) {
    const int micro = div_up(N, kMicroRows), words = div_up(n_parts, 32);
    unsigned int *d_bits = nullptr;
    TSNE_TRY(hipMalloc(&d_bits, sizeof(unsigned int) * (size_t)micro * words));
    micro_strip_parts_kernel<<<micro, 256, sizeof(unsigned int) * words, s>>>(indices, N, K, words, d_bits);
    std::vector<unsigned int> bits((size_t)micro * words);
    hipError_t err = hipGetLastError();
    if (err == hipSuccess) err = hipStreamSynchronize(s);
    if (err == hipSuccess)
        err = hipMemcpy(bits.data(), d_bits, sizeof(unsigned int) * bits.size(), hipMemcpyDeviceToHost);
    (void)hipFree(d_bits);
    TSNE_TRY(err);
    std::vector<unsigned int> acc(words);
    // Greedy merge under a cost limit; returns the number of strips (boundaries in `out` when given).
    auto cut = [&](long long limit, std::vector<int> *out) {
        int strips = 0, m = 0;
        if (out) out->assign(1, 0);
        while (m < micro) {
            std::fill(acc.begin(), acc.end(), 0u);
            int rows = 0, parts = 0;
            while (m < micro) {
                const int add_rows = std::min(kMicroRows, N - m * kMicroRows);
                int new_parts = parts;
                const unsigned int *b = &bits[(size_t)m * words];
                for (int w = 0; w < words; ++w) new_parts += __builtin_popcount(b[w] & ~acc[w]);
                const long long cost = (long long)(rows + add_rows) * K + kPartCostEntries * new_parts;
                if (rows > 0 && (rows + add_rows > kStripMax || cost > limit)) break;
                for (int w = 0; w < words; ++w) acc[w] |= b[w];
                rows += add_rows;
                parts = new_parts;
                ++m;
            }
            ++strips;
            if (out) out->push_back(m * kMicroRows < N ? m * kMicroRows : N);
        }
        return strips;
    };
    long long lo = 0, hi = (long long)kStripMax * K + kPartCostEntries * n_parts;  // hi always suffices when N fits
    while (lo + 1 < hi) {
        const long long mid = lo + (hi - lo) / 2;
        if (cut(mid, nullptr) <= max_strips)
            hi = mid;
        else
            lo = mid;
    }
    cut(hi, &row0);
    return 0;
}

void release_blocked(tsne_hip_plan *p) {
    // Steps may still be running (tsne_hip_iterate is asynchronous) and captured steps hold the addresses
    // about to be freed: wait for the plan's own streams and the device before anything is destroyed.
    if (p->loop_stream) (void)hipStreamSynchronize(p->loop_stream);
    if (p->side_stream) (void)hipStreamSynchronize(p->side_stream);
    (void)hipDeviceSynchronize();
    for (auto &g : p->step_graphs) (void)hipGraphExecDestroy(g.exec);
    p->step_graphs.clear();
    (void)hipFree(p->ent_p);
    (void)hipFree(p->seg);
    (void)hipFree(p->strip_row0);
    (void)hipFree(p->wseg);
    p->wseg = nullptr;
    p->blocked_direct = false;
    p->ent_p = nullptr;
    p->seg = nullptr;
    p->strip_row0 = nullptr;
    p->blocked_ready = false;
}

// Fills ent_p and wseg of the direct form (both allocated, strip_row0 on the device, p_max cleared).
static int prepare_direct(tsne_hip_plan *p, const float *pij, const int *indices, int uniform_rows, hipStream_t s) {
    const int N = p->num_points, K = p->num_neighbors;
    const long long nnz = (long long)N * K;
    int strip_bits = 1;
    while ((1 << strip_bits) < p->n_strips) ++strip_bits;
    struct Scratch {
        void *ptr = nullptr;
        ~Scratch() {
            if (ptr) (void)hipFree(ptr);
        }
    } keys, keys_alt, vals, vals_alt, hist, wpad;
    const int sort_tiles = div_up(nnz, radix_sort_tile());
    if (hipMalloc(&keys.ptr, sizeof(u64) * (size_t)nnz) != hipSuccess ||
        hipMalloc(&keys_alt.ptr, sizeof(u64) * (size_t)nnz) != hipSuccess ||
        hipMalloc(&vals.ptr, sizeof(float) * (size_t)nnz) != hipSuccess ||
        hipMalloc(&vals_alt.ptr, sizeof(float) * (size_t)nnz) != hipSuccess ||
        hipMalloc(&hist.ptr, sizeof(unsigned int) * 256 * ((size_t)sort_tiles + 1)) != hipSuccess ||
        hipMalloc(&wpad.ptr, sizeof(unsigned int) * (size_t)p->n_strips * (kMaxWindows + 1)) != hipSuccess) {
        set_error("attractive_prepare: out of device memory for sorting %lld entries", nnz);
        return 1;
    }
    const int blocks = (int)std::min<long long>(div_up(nnz, 256), 65536);
    direct_keys_kernel<<<blocks, 256, 0, s>>>(pij, indices, nnz, K, p->strip_row0, p->n_strips, uniform_rows,
                                              static_cast<u64 *>(keys.ptr), static_cast<float *>(vals.ptr));
    TSNE_LAUNCHED(s);
    if (radix_sort_pairs(static_cast<u64 *>(keys.ptr), static_cast<float *>(vals.ptr), static_cast<u64 *>(keys_alt.ptr),
                         static_cast<float *>(vals_alt.ptr), nnz, kDirectColBits + strip_bits,
                         static_cast<unsigned int *>(hist.ptr), s))
        return 1;
    direct_windows_kernel<<<p->n_strips, 128, 0, s>>>(static_cast<u64 *>(keys.ptr), K, p->strip_row0, p->n_windows,
                                                      p->wseg, p->wseg_stride, static_cast<unsigned int *>(wpad.ptr),
                                                      p->ent_p);
    TSNE_LAUNCHED(s);
    direct_emit_kernel<<<blocks, 256, 0, s>>>(static_cast<u64 *>(keys.ptr), static_cast<float *>(vals.ptr), nnz, K,
                                              p->strip_row0, p->n_strips, static_cast<unsigned int *>(wpad.ptr),
                                              p->ent_p, &p->scalars->vmax);
    TSNE_LAUNCHED(s);
    TSNE_TRY(hipStreamSynchronize(s));  // the scratch arrays go out of scope
    return 0;
}

int prepare_blocked(tsne_hip_plan *p, const float *pij, const int *indices, hipStream_t s) {
    release_blocked(p);
    const int N = p->num_points, K = p->num_neighbors;
    const int n_parts = div_up(N, kPartPoints);
    if (n_parts > kMaxParts) {
        set_error("attractive_prepare: %d points need %d column partitions, more than the %d supported", N, n_parts,
                  kMaxParts);
        return kShapeNotSupported;
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
        return kShapeNotSupported;
    }
    // Columns address LDS bitmaps and partition tables below: all of them must name a point.
    if (validate_indices(indices, (int64_t)N * K, N, "attractive_prepare", s)) return 1;
    // Equal strips, or - when they all run at once - strips of equal predicted cost.
    std::vector<int> row0;
    if (div_up(N, kStripMax) <= cus && N > cus * kMicroRows && std::getenv("TSNE_EQUAL_STRIPS") == nullptr) {
        if (balanced_strips(indices, N, K, n_parts, cus, row0, s)) return 1;
    } else {
        for (int r = 0; r < N; r += strip_rows) row0.push_back(r);
        row0.push_back(N);
    }
    p->n_strips = (int)row0.size() - 1;
    strip_rows = 0;
    for (int i = 0; i < p->n_strips; ++i) strip_rows = std::max(strip_rows, row0[i + 1] - row0[i]);
    p->strip_rows = strip_rows;  // the longest strip
    p->n_parts = n_parts;
    // A strip's list: the run starts (padded: the force kernel reads two past the last run) and the partitions.
    p->list_words = (n_parts + 4 + 3) & ~3;
    p->seg_stride = 4 + p->list_words + ((n_parts + 3) & ~3);
    if (hipMalloc(&p->strip_row0, sizeof(int) * row0.size()) != hipSuccess ||
        hipMemcpy(p->strip_row0, row0.data(), sizeof(int) * row0.size(), hipMemcpyHostToDevice) != hipSuccess) {
        release_blocked(p);
        set_error("attractive_prepare: out of device memory for the strip boundaries");
        return 1;
    }
    // Which form: the direct one where the strips outnumber the compute units, so that the staged form would run
    // them in rounds.  (TSNE_ATTRACTIVE_FORM=staged / direct overrides.)  Measured, ms per step staged / direct,
    // four clusters of 50 dimensions, K = 90: 1.00 M points (252 strips) 0.214 / 0.235; 1.05 M 0.318 / 0.258;
    // 1.2 M 0.341 / 0.283; 1.5 M 0.458 / 0.336; 2 M 0.554 / 0.475; 3 M 0.945 / 0.705; 10 M 6.4 / 3.4 (there a
    // strip's runs are 290 entries long, and staging 16 KB for each is seven times the entries' own traffic).
    // Fits of 50000 to 60000 points, whose strips all run at once, were 2 % slower in the direct form.
    {
        p->blocked_direct = p->n_strips > cus;
        if (const char *v = std::getenv("TSNE_ATTRACTIVE_FORM")) p->blocked_direct = v[0] == 'd';
        // (the direct form's keys hold 24 bits of column and 16 of strip; its sort counts in 31 bits)
        // (strips that are not all of one length are at most as many as the compute units)
        if (div_up(N, kWindowPoints) > kMaxWindows || (int64_t)N * K >= ((int64_t)1 << 31) || cus > 1024)
            p->blocked_direct = false;
    }
    int direct_uniform_rows = 0;
    if (p->blocked_direct && p->n_strips > cus) {
        // As few rounds of strips over the compute units as the longest strips allow, and the strips of those
        // rounds of equal length (a multiple of the wave).
        const int rounds = div_up(N, (int64_t)cus * kDirectStripMax);
        direct_uniform_rows = std::min(kDirectStripMax, div_up(div_up(N, (int64_t)cus * rounds), kWave) * kWave);
        // More strips than compute units whatever their size: the direct form then takes strips as long as the
        // LDS holds (every strip walks the positions of all the columns it references once).
        row0.clear();
        for (int r = 0; r < N; r += direct_uniform_rows) row0.push_back(r);
        row0.push_back(N);
        p->n_strips = (int)row0.size() - 1;
        p->strip_rows = strip_rows = std::min(N, direct_uniform_rows);
        (void)hipFree(p->strip_row0);
        p->strip_row0 = nullptr;
        if (hipMalloc(&p->strip_row0, sizeof(int) * row0.size()) != hipSuccess ||
            hipMemcpy(p->strip_row0, row0.data(), sizeof(int) * row0.size(), hipMemcpyHostToDevice) != hipSuccess) {
            release_blocked(p);
            set_error("attractive_prepare: out of device memory for the strip boundaries");
            return 1;
        }
    }
    p->n_windows = p->blocked_direct ? div_up(N, kWindowPoints) : 0;
    p->wseg_stride = (4 + p->n_windows + 3 + 3) & ~3;
    // Entries: whole items for every strip (the last item of a strip is padded; the padding is never consumed);
    // the direct form pads every window's entries to whole pieces.
    const size_t strip_entries = (size_t)strip_rows * K + (size_t)kDirectPiece * p->n_windows;
    const size_t item_entries = p->blocked_direct ? kDirectItem : kItemEntries;
    const size_t items_per_strip = (strip_entries + item_entries - 1) / item_entries;
    const size_t nnz = items_per_strip * p->n_strips * item_entries;
    bool ok = hipMalloc(&p->ent_p, 2 * sizeof(float) * nnz) == hipSuccess &&
              hipMalloc(&p->seg, p->blocked_direct ? sizeof(unsigned int)
                                                   : sizeof(unsigned int) * (size_t)p->n_strips * p->seg_stride) == hipSuccess &&
              (!p->blocked_direct ||
               hipMalloc(&p->wseg, sizeof(unsigned int) * (size_t)p->n_strips * p->wseg_stride) == hipSuccess);
    if (!ok) {
        release_blocked(p);
        set_error("attractive_prepare: out of device memory for the re-blocked pattern (%zu bytes)", nnz * 8);
        return 1;
    }
    clear_pmax_kernel<<<1, 64, 0, s>>>(&p->scalars->vmax);
    TSNE_LAUNCHED(s);
    if (p->blocked_direct) {
        if (const int rc = prepare_direct(p, pij, indices, direct_uniform_rows, s)) {
            release_blocked(p);
            return rc;
        }
    } else {
        TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(reblock_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)kReblockLds));
        reblock_kernel<<<p->n_strips, kBlock, kReblockLds, s>>>(pij, indices, N, K, p->strip_row0, p->list_words,
                                                                p->seg_stride, p->ent_p, p->seg, &p->scalars->vmax);
        TSNE_LAUNCHED(s);
    }
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(attractive_direct_kernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDirectLds));
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(attractive_blocked_kernel<false>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBlockedLds));
    TSNE_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(attractive_blocked_kernel<true>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBlockedLds));
    p->spin_limit = kSpinLimit;
    if (const char *v = std::getenv("TSNE_ATTRACTIVE_SPIN_LIMIT")) p->spin_limit = std::max(0, std::atoi(v));
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
    if (p->blocked_direct) {
        // (LDS for the longest strip only: what is left of a compute unit's 160 KB hosts the repulsive chain's kernels)
        const int rows_cap = (p->strip_rows + kWave - 1) / kWave * kWave;
        TSNE_LOOP_KERNEL(p, (attractive_direct_kernel), p->n_strips, kDirectThreads, (size_t)24 * rows_cap, s, p->ent_p, p->wseg, p->yxy, p->scalars, attr, p->num_points, p->num_neighbors, p->wseg_stride, rows_cap);
        TSNE_LAUNCHED(s);
        return 0;
    }
    const auto kernel = p->spin_limit == kSpinLimit ? attractive_blocked_kernel<false> : attractive_blocked_kernel<true>;
    TSNE_LOOP_KERNEL(p, (kernel), p->n_strips, kBlock, kBlockedLds, s, p->ent_p, p->seg, p->yxy, p->scalars, attr, p->num_points,
                                                    p->num_neighbors, p->list_words, p->seg_stride,
                                                    p->spin_limit);
    TSNE_LAUNCHED(s);
    return 0;
}

// After the stream has been synchronised: whether any attractive launch since the last check lost step
// between its waves (see LoopScalars::wait_timeouts).  Clears the count.
int check_attractive_waits(tsne_hip_plan *p) {
    unsigned int n = 0;
    TSNE_TRY(hipMemcpy(&n, &p->scalars->wait_timeouts, sizeof(n), hipMemcpyDeviceToHost));
    if (n == 0) return 0;
    TSNE_TRY(hipMemset(&p->scalars->wait_timeouts, 0, sizeof(n)));
    set_error("attractive: %u workgroup(s) timed out waiting for a staged partition; their forces are NaN", n);
    return 1;
}

}  // namespace tsnehip
