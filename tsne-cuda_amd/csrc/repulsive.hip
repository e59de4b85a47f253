// FFT-interpolated repulsive forces for gfx950.
//
// One gradient step evaluates, for every point i and the four charge terms
// q_j = (1, x_j, y_j, x_j^2 + y_j^2),
//     phi_i[t] = sum_j q_j[t] / (1 + |y_i - y_j|^2)^2
// by (1) spreading the charges onto an n_nodes x n_nodes grid of equispaced
// interpolation nodes with 3x3 Lagrange weights, (2) convolving the grid with
// the squared-Cauchy kernel, (3) interpolating the node potentials back.
// Semantics follow src/kernels/nbodyfft.cu and src/kernels/rep_forces.cu of the
// reference; the structure does not:
//   * bounds, box width and Z never leave the device;
//   * charges, box indices and Lagrange weights are recomputed in registers
//     instead of being stored (src/kernels/nbodyfft.cu:43-105,
//     src/kernels/rep_forces.cu:57-76);
//   * the convolution zero-pads to 800 points (grids of up to 133 boxes per
//     side) or 1024 and runs as in-place mixed-radix FFTs in LDS: a
//     decimation-in-frequency forward transform leaves its output in
//     digit-reversed order, the decimation-in-time inverse consumes that
//     order, so nothing is ever permuted.  Two real charge planes ride in one
//     complex transform; the kernel is real and even, so its spectrum is real
//     and the planes never mix.  fp32 round-off does leak between the two
//     planes of a pair in proportion to the larger one, so planes of like
//     magnitude are paired: (1, r^2 / m^2) and (x, y), with m the largest
//     absolute coordinate.
#include "plan.h"

#include <algorithm>

namespace tsnehip {

namespace {

constexpr int kLog2Fft = 10;
constexpr int kRowThreads = 512;  // threads of a row-pass workgroup (four transforms)

__device__ __forceinline__ int rev4(int x) {
    // Reverse the five base-4 digits of a 10-bit index.
    const unsigned int y = __brev((unsigned int)x) >> (32 - kLog2Fft);
    return (int)(((y & 0x155u) << 1) | ((y >> 1) & 0x155u));
}

__device__ __forceinline__ float2 cmul(float2 a, float2 b) {
    return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x);
}
__device__ __forceinline__ float2 cmul_conj(float2 a, float2 b) {  // a * conj(b)
    return make_float2(a.x * b.x + a.y * b.y, a.y * b.x - a.x * b.y);
}
__device__ __forceinline__ float2 cadd(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ float2 csub(float2 a, float2 b) { return make_float2(a.x - b.x, a.y - b.y); }

// The row passes read or write the transposed spectra in 16-byte pieces (two neighbouring rows of one spectrum
// position); the eight workgroups whose pieces share a 128-byte line should meet in one L2, or every XCD fetches
// (or partially writes) the line for itself.  Workgroups go to the XCDs round robin by their number, so
// workgroup b takes row block (b mod 8) * ceil(blocks / 8) + b / 8: an XCD gets a run of neighbouring rows.
// Returns -1 for the surplus workgroups of the rounded-up launch.
constexpr int kXcds = 8;
__device__ __forceinline__ int xcd_row_block(int b, int blocks) {
    const int per = (blocks + kXcds - 1) / kXcds;
    const int logical = (b % kXcds) * per + b / kXcds;
    return (b / kXcds < per && logical < blocks) ? logical : -1;
}
inline int xcd_launch_blocks(int blocks) { return kXcds * ((blocks + kXcds - 1) / kXcds); }

// The transforms of length 1024 are five in-place radix-4 passes over the LDS (sub-transform lengths 1024, 256, 64,
// 16, 4 forwards - decimation in frequency, natural order in, base-4 digit-reversed order out - and the same
// backwards for the inverse, decimation in time), 256 butterflies per transform and pass, a barrier after each.
//
// A transform occupies its 1024 LDS slots in a swizzled order: element i sits in slot pad(i), which exchanges
// bits among the low five of i (bit 4 is added into bits 0 and 2, bit 5 into bits 1 and 3, bit 6 into bit 4), so
// that the strides the passes use (256, 64, 16, 4 and 1 elements between the butterflies of neighbouring lanes,
// 8-byte elements) fall on different banks, whether the LDS serves 16 or 32 lanes of an 8-byte access at a time.
// With a plain layout the lanes of the 16- and 4-point passes hit each bank eight deep (forward row pass
// 17 -> 15 us, column pass 22 -> 21 us, inverse row pass 17 -> 13.5 us at 390 rows; 5-8 % of the whole fit of
// 5000 to 60000 points, where the chain of dependent launches is what a step costs).
//
// The twiddles come straight from memory (an 8 KB table that every CU keeps in its L1).
//
// Measured and not kept: passes 1024+256 and 64+16 fused (a thread holding 16 elements in registers, three trips
// through the LDS instead of five): only 64 threads per transform have work in a fused pass, and the passes
// came out 10-15 % slower than five passes that keep every thread busy.  The thread's fifteen twiddles loaded
// once into registers ahead of the data (they are the same for every transform it visits): 1-2 us slower per
// pass than loading them where they are used.
constexpr int kFftPad = kFft;  // slots per transform
__device__ __forceinline__ int pad(int i) {
    return i ^ (((i >> 4) & 1) * 5) ^ (((i >> 5) & 1) * 10) ^ (((i >> 6) & 1) << 4);
}

// Radix-4 butterflies on four registers: decimation in frequency forwards (twiddles after the sums), decimation in
// time for the inverse (conjugate twiddles first).
__device__ __forceinline__ void butterfly_forward(float2 &x0, float2 &x1, float2 &x2, float2 &x3, const float2 (&w)[3]) {
    const float2 t0 = cadd(x0, x2), t1 = csub(x0, x2), t2 = cadd(x1, x3), t3 = csub(x1, x3);
    x0 = cadd(t0, t2);
    x1 = cmul(make_float2(t1.x + t3.y, t1.y - t3.x), w[0]);
    x2 = cmul(csub(t0, t2), w[1]);
    x3 = cmul(make_float2(t1.x - t3.y, t1.y + t3.x), w[2]);
}
__device__ __forceinline__ void butterfly_inverse(float2 &x0, float2 &x1, float2 &x2, float2 &x3, const float2 (&w)[3]) {
    const float2 a1 = cmul_conj(x1, w[0]), a2 = cmul_conj(x2, w[1]), a3 = cmul_conj(x3, w[2]);
    const float2 u0 = cadd(x0, a2), u1 = csub(x0, a2), u2 = cadd(a1, a3), u3 = csub(a1, a3);
    x0 = cadd(u0, u2);
    x1 = make_float2(u1.x - u3.y, u1.y + u3.x);
    x2 = csub(u0, u2);
    x3 = make_float2(u1.x + u3.y, u1.y - u3.x);
}

// One pass (sub-transform length L = 2^log2L) over `nfft` transforms stored kFftPad slots apart.
template <bool INVERSE>
__device__ __forceinline__ void radix4_pass(float2 *s, int nfft, int log2L, const float2 *tw, int tid, int nthreads) {
    const int L = 1 << log2L, q4 = L >> 2, log2q4 = log2L - 2, stride = kFft >> log2L;
    for (int id = tid; id < nfft * (kFft / 4); id += nthreads) {
        const int f = id >> 8, q = id & 255;
        const int k = q & (q4 - 1), b = q >> log2q4;
        float2 *base = s + f * kFftPad;
        const int i0 = b * L + k;
        const float2 w[3] = {tw[k * stride], tw[2 * k * stride], tw[3 * k * stride]};
        float2 x0 = base[pad(i0)], x1 = base[pad(i0 + q4)], x2 = base[pad(i0 + 2 * q4)], x3 = base[pad(i0 + 3 * q4)];
        if (!INVERSE)
            butterfly_forward(x0, x1, x2, x3, w);
        else
            butterfly_inverse(x0, x1, x2, x3, w);
        base[pad(i0)] = x0;
        base[pad(i0 + q4)] = x1;
        base[pad(i0 + 2 * q4)] = x2;
        base[pad(i0 + 3 * q4)] = x3;
    }
}

// Grids of up to 400 nodes per side (133 boxes; the default 130 gives 390) need 799 points of padding, and get
// transforms of 800 = 8 * 10 * 10 points: 0.61 of the 1024 x 1024 transform's points, in three in-place passes
// (forwards: radix 8 over the whole transform, radix 10 over its eight parts of 100, radix 10 over the tens);
// position p = 100 j1 + 10 j2 + j3 then holds frequency j1 + 8 j2 + 80 j3, and the inverse runs the same passes
// backwards.  Plain layout, no swizzle.
template <int R, bool INVERSE>
__device__ __forceinline__ void small_dft(float2 (&x)[R]) {
    if constexpr (R == 2) {
        const float2 a = x[0], b = x[1];
        x[0] = cadd(a, b);
        x[1] = csub(a, b);
    } else if constexpr (R == 4) {
        const float2 t0 = cadd(x[0], x[2]), t1 = csub(x[0], x[2]), t2 = cadd(x[1], x[3]), t3 = csub(x[1], x[3]);
        x[0] = cadd(t0, t2);
        x[2] = csub(t0, t2);
        if (!INVERSE) {
            x[1] = make_float2(t1.x + t3.y, t1.y - t3.x);
            x[3] = make_float2(t1.x - t3.y, t1.y + t3.x);
        } else {
            x[1] = make_float2(t1.x - t3.y, t1.y + t3.x);
            x[3] = make_float2(t1.x + t3.y, t1.y - t3.x);
        }
    } else if constexpr (R == 8) {
        // Even and odd elements as two transforms of four, then w8^k = exp(-+ i pi k / 4) on the odd half.
        float2 e[4] = {x[0], x[2], x[4], x[6]}, o[4] = {x[1], x[3], x[5], x[7]};
        small_dft<4, INVERSE>(e);
        small_dft<4, INVERSE>(o);
        constexpr float h = 0.70710678118654752f;
        const float sg = INVERSE ? -1.0f : 1.0f;  // forwards: w8 = (1 - i) / sqrt 2
        const float2 o1 = make_float2(h * (o[1].x + sg * o[1].y), h * (o[1].y - sg * o[1].x));
        const float2 o2 = make_float2(sg * o[2].y, -sg * o[2].x);
        const float2 o3 = make_float2(h * (-o[3].x + sg * o[3].y), h * (-o[3].y - sg * o[3].x));
        x[0] = cadd(e[0], o[0]);
        x[4] = csub(e[0], o[0]);
        x[1] = cadd(e[1], o1);
        x[5] = csub(e[1], o1);
        x[2] = cadd(e[2], o2);
        x[6] = csub(e[2], o2);
        x[3] = cadd(e[3], o3);
        x[7] = csub(e[3], o3);
    } else if constexpr (R == 10) {
        // Even and odd elements as two transforms of five, then w10^k = exp(-+ i pi k / 5) on the odd half.
        float2 e[5] = {x[0], x[2], x[4], x[6], x[8]}, o[5] = {x[1], x[3], x[5], x[7], x[9]};
        small_dft<5, INVERSE>(e);
        small_dft<5, INVERSE>(o);
        constexpr float wr[5] = {1.0f, 0.80901699437494745f, 0.30901699437494745f, -0.30901699437494745f,
                                 -0.80901699437494745f};
        constexpr float wi[5] = {0.0f, 0.58778525229247314f, 0.95105651629515353f, 0.95105651629515353f,
                                 0.58778525229247314f};  // -Im w10^k forwards
#pragma unroll
        for (int k = 0; k < 5; ++k) {
            const float2 w = make_float2(wr[k], INVERSE ? wi[k] : -wi[k]);
            const float2 t = k == 0 ? o[0] : cmul(o[k], w);
            x[k] = cadd(e[k], t);
            x[k + 5] = csub(e[k], t);
        }
    } else {
        static_assert(R == 5, "radix");
        // cos(2 pi / 5) and cos(4 pi / 5) are -1/4 +- sqrt(5)/4: written so, the part of an output that cancels for
        // smooth data carries exact coefficients, and the rounded constant meets a difference only.
        constexpr float r5 = 0.55901699437494742f;                               // sqrt(5) / 4
        constexpr float s1 = 0.95105651629515353f, s2 = 0.58778525229247314f;   // sin(2 pi / 5), sin(4 pi / 5)
        const float2 t1 = cadd(x[1], x[4]), t2 = cadd(x[2], x[3]), t3 = csub(x[1], x[4]), t4 = csub(x[2], x[3]);
        const float2 t5 = cadd(t1, t2);
        const float2 m0 = make_float2(x[0].x - 0.25f * t5.x, x[0].y - 0.25f * t5.y);
        const float2 t6 = make_float2(r5 * (t1.x - t2.x), r5 * (t1.y - t2.y));
        const float2 a1 = cadd(m0, t6), a2 = csub(m0, t6);
        float2 b1 = make_float2(s1 * t3.x + s2 * t4.x, s1 * t3.y + s2 * t4.y);
        float2 b2 = make_float2(s2 * t3.x - s1 * t4.x, s2 * t3.y - s1 * t4.y);
        if (INVERSE) {
            b1 = make_float2(-b1.x, -b1.y);
            b2 = make_float2(-b2.x, -b2.y);
        }
        x[0] = cadd(x[0], t5);
        x[1] = make_float2(a1.x + b1.y, a1.y - b1.x);  // a1 - i b1
        x[4] = make_float2(a1.x - b1.y, a1.y + b1.x);
        x[2] = make_float2(a2.x + b2.y, a2.y - b2.x);
        x[3] = make_float2(a2.x - b2.y, a2.y + b2.x);
    }
}

// One pass of radix R over the sub-transforms of length L of `nfft` transforms of N points, N slots apart:
// decimation in frequency forwards (twiddles after the sums), decimation in time for the inverse.
// load(f, i, j) delivers element i of transform f (the j-th of its butterfly, a compile-time number once the loop
// is unrolled), store(f, i, j, v) takes it back: the LDS in the middle of a transform, memory at either end of it
// where a kernel fuses its loads and stores into the first and last pass.
template <int N, int L, int R, bool INVERSE, class Load, class Store>
__device__ __forceinline__ void mixed_pass_io(int nfft, const float2 *tw, int tid, int nthreads, Load load,
                                              Store store) {
    constexpr int Q = L / R, B = N / R, STRIDE = N / L;
    for (int id = tid; id < nfft * B; id += nthreads) {
        const int f = id / B, q = id - f * B;
        const int b = q / Q, k = q - b * Q;
        const int i0 = b * L + k;
        float2 x[R];
#pragma unroll
        for (int j = 0; j < R; ++j) x[j] = load(f, i0 + j * Q, j);
        if constexpr (INVERSE && Q > 1) {
#pragma unroll
            for (int j = 1; j < R; ++j) x[j] = cmul_conj(x[j], tw[j * k * STRIDE]);
        }
        small_dft<R, INVERSE>(x);
        if constexpr (!INVERSE && Q > 1) {
#pragma unroll
            for (int j = 1; j < R; ++j) x[j] = cmul(x[j], tw[j * k * STRIDE]);
        }
#pragma unroll
        for (int j = 0; j < R; ++j) store(f, i0 + j * Q, j, x[j]);
    }
}
template <int N, int L, int R, bool INVERSE>
__device__ __forceinline__ void mixed_pass(float2 *s, int nfft, const float2 *tw, int tid, int nthreads) {
    mixed_pass_io<N, L, R, INVERSE>(
        nfft, tw, tid, nthreads, [s](int f, int i, int) { return s[f * N + i]; },
        [s](int f, int i, int, float2 v) { s[f * N + i] = v; });
    __syncthreads();
}

// What the convolution's kernels need of a transform length: the slot of element i within a transform's N LDS
// slots, the frequency held at a position of the forward transform's output, and the transforms themselves
// (every pass ends with a barrier).
template <int N>
struct Transform;

template <>
struct Transform<kFft> {
    static __device__ __forceinline__ int slot(int i) { return pad(i); }
    static __device__ __forceinline__ int frequency(int pos) { return rev4(pos); }
    static __device__ __forceinline__ void forward(float2 *s, int nfft, const float2 *tw, int tid, int nthreads) {
#pragma unroll
        for (int l = kLog2Fft; l >= 2; l -= 2) {
            radix4_pass<false>(s, nfft, l, tw, tid, nthreads);
            __syncthreads();
        }
    }
    static __device__ __forceinline__ void inverse(float2 *s, int nfft, const float2 *tw, int tid, int nthreads) {
#pragma unroll
        for (int l = 2; l <= kLog2Fft; l += 2) {
            radix4_pass<true>(s, nfft, l, tw, tid, nthreads);
            __syncthreads();
        }
    }
};

template <>
struct Transform<kFftShort> {
    static constexpr int N = kFftShort;
    static_assert(N == 800, "the passes below factor 800");
    static __device__ __forceinline__ int slot(int i) { return i; }
    static __device__ __forceinline__ int frequency(int pos) {
        const int j1 = pos / 100, r1 = pos - j1 * 100;
        const int j2 = r1 / 10, j3 = r1 - j2 * 10;
        return j1 + 8 * j2 + 80 * j3;
    }
    static __device__ __forceinline__ void forward(float2 *s, int nfft, const float2 *tw, int tid, int nthreads) {
        mixed_pass<N, 800, 8, false>(s, nfft, tw, tid, nthreads);
        mixed_pass<N, 100, 10, false>(s, nfft, tw, tid, nthreads);
        mixed_pass<N, 10, 10, false>(s, nfft, tw, tid, nthreads);
    }
    static __device__ __forceinline__ void inverse(float2 *s, int nfft, const float2 *tw, int tid, int nthreads) {
        mixed_pass<N, 10, 10, true>(s, nfft, tw, tid, nthreads);
        mixed_pass<N, 100, 10, true>(s, nfft, tw, tid, nthreads);
        mixed_pass<N, 800, 8, true>(s, nfft, tw, tid, nthreads);
    }
};

struct Bounds {
    float lo, box_width, h;
};
__device__ __forceinline__ Bounds load_bounds(const LoopScalars *sc, int slot, int n_boxes) {
#pragma clang fp contract(off)
    Bounds b;
    b.lo = ordered_to_float(sc->min_enc[slot]);
    const float hi = ordered_to_float(sc->max_enc[slot]);
    b.box_width = (hi - b.lo) / (float)n_boxes;  // src/fit_tsne.cu:442
    b.h = b.box_width / (float)kInterp;          // src/kernels/nbodyfft.cu:270
    return b;
}

// 1 / m^2 with m the largest absolute coordinate: brings the r^2 charge plane
// to the magnitude of the unit charge plane it shares a transform with.
__device__ __forceinline__ float r2_plane_scale(const LoopScalars *sc, int slot) {
    const float lo = ordered_to_float(sc->min_enc[slot]);
    const float hi = ordered_to_float(sc->max_enc[slot]);
    const float m2 = fmaxf(lo * lo, hi * hi);
    return m2 > 0.0f ? 1.0f / m2 : 1.0f;
}

// Box index (clamped), in-box coordinate and the three Lagrange basis values of
// one coordinate (src/kernels/nbodyfft.cu:43-105,205-227), with the fp32
// operations kept in the reference's order and never contracted.
__device__ __forceinline__ void bin_and_weights(float v, const Bounds &bd, int n_boxes, const LagrangeConsts &lc,
                                                int &box, float *L) {
#pragma clang fp contract(off)
    int b = (int)((v - bd.lo) / bd.box_width);
    b = max(0, b);
    b = min(n_boxes - 1, b);
    box = b;
    const float lower = b * bd.box_width + bd.lo;
    const float t = (v - lower) / bd.box_width;
    const float d0 = t - lc.spacing[0], d1 = t - lc.spacing[1], d2 = t - lc.spacing[2];
    L[0] = (d1 * d2) / lc.denom[0];
    L[1] = (d0 * d2) / lc.denom[1];
    L[2] = (d0 * d1) / lc.denom[2];
}

// ---------------------------------------------------------------------------
// Bounds of the embedding: one scalar min and max over all 2N coordinates
// (src/fit_tsne.cu:430-432), kept on the device in an order-preserving integer
// encoding so that blocks can combine with integer atomics.
// ---------------------------------------------------------------------------
__global__ void bounds_reset_kernel(LoopScalars *sc, int slot, int new_embedding) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        sc->min_enc[slot] = 0xffffffffu;
        sc->max_enc[slot] = 0u;
        if (new_embedding) sc->reuse_sort = 0;  // whatever grouping by tile the plan holds is not this embedding's
    }
}

__global__ __launch_bounds__(256) void bounds_kernel(const float *__restrict__ v, int64_t n, LoopScalars *sc,
                                                     int slot) {
    float lo = INFINITY, hi = -INFINITY;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += (int64_t)gridDim.x * blockDim.x) {
        const float x = v[t];
        lo = fminf(lo, x);
        hi = fmaxf(hi, x);
    }
    __shared__ float wlo[256 / kWave], whi[256 / kWave];
    lo = group_min<kWave>(lo);
    hi = group_max<kWave>(hi);
    if ((threadIdx.x & (kWave - 1)) == 0) {
        wlo[threadIdx.x / kWave] = lo;
        whi[threadIdx.x / kWave] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < 256 / kWave; ++k) {
            lo = fminf(lo, wlo[k]);
            hi = fmaxf(hi, whi[k]);
        }
        // Atomics on one address are performed one after the other (~12 ns each): a workgroup first looks whether
        // its extremes would change anything (the values only move one way, so a stale look costs at most a
        // superfluous atomic).
        const unsigned int lo_enc = float_to_ordered(lo), hi_enc = float_to_ordered(hi);
        if (lo_enc < __hip_atomic_load(&sc->min_enc[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMin(&sc->min_enc[slot], lo_enc);
        if (hi_enc > __hip_atomic_load(&sc->max_enc[slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMax(&sc->max_enc[slot], hi_enc);
    }
}

// ---------------------------------------------------------------------------
// Spread: w[node][t] += Lx_a * Ly_b * q[t] (src/kernels/nbodyfft.cu:107-139).
// The row index of the node grid is the x node.
//
// The reference issues 36 global atomics per point.  Nodes belong to exactly
// one box, so here the points are first grouped by tile of kTileBoxes x
// kTileBoxes (5 x 5) boxes with a counting sort (count, scan, scatter:
// positions only, the P matrix keeps its order); then a workgroup takes up to
// 1024 points of one tile, accumulates their moments per box in a private LDS
// tile with (integer) LDS atomics, and adds the box moments to the grid's with
// one 64-bit integer atomic each.  The forward row pass forms the node sums
// from the moments.  Every sum between a point and the node charges is an
// integer sum, so the charges do not depend on how the points were grouped or
// on the order in which workgroups arrive: two runs give the same bits.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int box_of(float v, const Bounds &bd, int n_boxes) {
#pragma clang fp contract(off)
    int b = (int)((v - bd.lo) / bd.box_width);  // same expression as bin_and_weights
    b = max(0, b);
    return min(n_boxes - 1, b);
}

__device__ __forceinline__ int tile_of(float x, float y, const Bounds &bd, int n_boxes, int tiles_per_dim) {
    return (box_of(y, bd, n_boxes) / kTileBoxes) * tiles_per_dim + box_of(x, bd, n_boxes) / kTileBoxes;
}

constexpr int kRankBits = 21;  // a point's code: tile << kRankBits | rank (a workgroup counts fewer than 2 M points)
static_assert(kMaxTiles <= (1 << (32 - kRankBits)), "tile numbers must fit the code's upper bits");

// hist[t] += 1 for every active lane of the wave; returns the value the lane's own increment found (its
// rank).  Neighbouring points of the locality-ordered numbering lie close together in the embedding too,
// so most lanes of a wave name the same one or two tiles: 64 LDS atomics on one address would be
// performed one after the other.  Up to four groups of at least eight lanes that share a tile are
// therefore counted by one lane each (ballot + population count); whatever is left adds on its own.
__device__ __forceinline__ int wave_tile_add(int *hist, int t, bool active) {
    const int lane = threadIdx.x & (kWave - 1);
    const unsigned long long below = (1ull << lane) - 1ull;
    unsigned long long remaining = __ballot(active);
    int rank = 0;
    for (int round = 0; round < 4 && remaining; ++round) {
        const int leader = __builtin_amdgcn_readfirstlane(__ffsll((long long)remaining) - 1);
        const int tl = __builtin_amdgcn_readlane(t, leader);
        const bool mine = active && t == tl && ((remaining >> lane) & 1ull);
        const unsigned long long group = __ballot(mine);
        const int members = __popcll(group);
        if (members < 8) break;
        int first = 0;
        if (lane == leader) first = atomicAdd(&hist[tl], members);
        first = __builtin_amdgcn_readlane(first, leader);
        if (mine) rank = first + __popcll(group & below);
        remaining &= ~group;
    }
    if ((remaining >> lane) & 1ull) rank = atomicAdd(&hist[t], 1);
    return rank;
}

// Exclusive scan of the tile counts and of the chunk counts by one workgroup of 1024
// threads: write cursors, every tile cut into chunks of at most kChunkPoints points.
// Two tiles per thread (kMaxTiles <= 2 * 1024).  Leaves the counters at zero for the
// next step.
__device__ __forceinline__ void scan_tiles(int *__restrict__ tile_count, int n_tiles, int *__restrict__ tile_cursor,
                                           int4 *__restrict__ chunks, int *__restrict__ num_chunks, int *pts,
                                           int *chk) {
    static_assert(kMaxTiles <= 2048, "the scan handles two tiles per thread");
    const int t = threadIdx.x;
    int cnt[2], nchunk[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int tile = 2 * t + k;
        // The counts were produced by other workgroups' atomics: read them where atomics live.
        cnt[k] = tile < n_tiles ? atomicExch(&tile_count[tile], 0) : 0;
        nchunk[k] = (cnt[k] + kChunkPoints - 1) / kChunkPoints;
    }
    pts[t] = cnt[0] + cnt[1];
    chk[t] = nchunk[0] + nchunk[1];
    __syncthreads();
    // Hillis-Steele inclusive scans over 1024 slots.
    for (int off = 1; off < 1024; off <<= 1) {
        const int a = t >= off ? pts[t - off] : 0;
        const int b = t >= off ? chk[t - off] : 0;
        __syncthreads();
        pts[t] += a;
        chk[t] += b;
        __syncthreads();
    }
    int first_point = pts[t] - cnt[0] - cnt[1], first_chunk = chk[t] - nchunk[0] - nchunk[1];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int tile = 2 * t + k;
        if (tile < n_tiles) {
            tile_cursor[tile] = first_point;
            for (int c = 0; c < nchunk[k]; ++c)
                chunks[first_chunk + c] =
                    make_int4(tile, first_point + c * kChunkPoints, min(kChunkPoints, cnt[k] - c * kChunkPoints), 0);
        }
        first_point += cnt[k];
        first_chunk += nchunk[k];
    }
    if (t == 1023) *num_chunks = chk[t];
}

// First kernel of a step's repulsive chain.  Counts the points per tile; the workgroup that
// finishes last (a ticket counter tells) scans the counts.  Its first thread also clears Z and
// the bounds slot the coming update will fill.  tile_count is all zero on entry and on exit.
__global__ __launch_bounds__(1024) void tile_count_kernel(const float *__restrict__ emb, int N, LoopScalars *sc,
                                                         int slot, int next_slot, int n_boxes,
                                                         int *__restrict__ tile_count,
                                                         int *__restrict__ tile_cursor, int4 *__restrict__ chunks,
                                                         int *__restrict__ num_chunks, int *__restrict__ ticket,
                                                         unsigned int *__restrict__ point_code,
                                                         int *__restrict__ wg_tile_base, int keep_grouping) {
    __shared__ int hist[kMaxTiles];
    __shared__ int pts[1024], chk[1024];
    __shared__ int last;
    const int tiles_per_dim = (n_boxes + kTileBoxes - 1) / kTileBoxes;
    const int n_tiles = tiles_per_dim * tiles_per_dim;
    // The grouping of the step before is kept (nobody writes the flag while this kernel runs).
    if (keep_grouping && sc->reuse_sort) return;
    for (int b = threadIdx.x; b < n_tiles; b += blockDim.x) hist[b] = 0;
    __syncthreads();
    const Bounds bd = load_bounds(sc, slot, n_boxes);
    // (whole waves enter the loop body together: the bound is rounded up to the wave)
    for (int i0 = blockIdx.x * blockDim.x + (threadIdx.x & ~(kWave - 1)); i0 < N; i0 += gridDim.x * blockDim.x) {
        const int i = i0 + (threadIdx.x & (kWave - 1));
        const bool active = i < N;
        const int t = active ? tile_of(emb[i], emb[N + i], bd, n_boxes, tiles_per_dim) : 0;
        const int rank = wave_tile_add(hist, t, active);
        // The scatter kernel needs no histogram of its own: tile and rank travel with the point.
        if (active) point_code[i] = ((unsigned int)t << kRankBits) | (unsigned int)rank;
    }
    __syncthreads();
    // The counters live where device-scope atomics are performed, so no cache maintenance is needed
    // to publish them (a device-wide fence would write back and invalidate the L2 of every XCD, once
    // per wave): an atomic that has returned its old value has been performed, and the ticket is
    // taken after all of this workgroup's atomics have returned.
    for (int b = threadIdx.x; b < n_tiles; b += blockDim.x) {
        if (hist[b]) {
            // what the counter held before: where this workgroup's points start inside the tile's run
            wg_tile_base[(size_t)blockIdx.x * kMaxTiles + b] = atomicAdd(&tile_count[b], hist[b]);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) last = atomicAdd(ticket, 1) == (int)gridDim.x - 1;
    __syncthreads();
    if (!last) return;
    scan_tiles(tile_count, n_tiles, tile_cursor, chunks, num_chunks, pts, chk);
    if (threadIdx.x == 0) *ticket = 0;
}

// Same point-to-workgroup assignment as tile_count_kernel, which left every point's tile and its rank
// among the workgroup's points of that tile: position = start of the tile's run + start of the
// workgroup's part of it + rank.  A streaming pass without atomics.
__global__ __launch_bounds__(1024) void tile_scatter_kernel(const float *__restrict__ emb, int N, int n_tiles,
                                                           const int *__restrict__ tile_cursor,
                                                           const unsigned int *__restrict__ point_code,
                                                           const int *__restrict__ wg_tile_base,
                                                           float2 *__restrict__ tile_xy, int *__restrict__ tile_perm,
                                                           const LoopScalars *sc, int keep_grouping) {
    __shared__ int base[kMaxTiles];
    if (keep_grouping && sc->reuse_sort) return;
    // (entries of wg_tile_base for tiles this workgroup has no point in are never read)
    for (int b = threadIdx.x; b < n_tiles; b += blockDim.x)
        base[b] = tile_cursor[b] + wg_tile_base[(size_t)blockIdx.x * kMaxTiles + b];
    __syncthreads();
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < N; i += gridDim.x * blockDim.x) {
        const unsigned int code = point_code[i];
        const int pos = base[code >> kRankBits] + (int)(code & ((1u << kRankBits) - 1u));
        tile_xy[pos] = make_float2(emb[i], emb[N + i]);
        tile_perm[pos] = i;
    }
}

constexpr int kSpreadThreads = 512;  // two points of a 1024-point chunk per thread

// v * scale rounded to a 64-bit integer (|v * scale| < 2^51).
__device__ __forceinline__ unsigned long long to_fixed_bits(float v, double scale) {
    const double magic = 6755399441055744.0;  // 1.5 * 2^52: adding it rounds a double to an integer
    const double r = fma((double)v, scale, magic);
    return (unsigned long long)(__double_as_longlong(r) - __double_as_longlong(magic));
}
// 64-bit fixed-point add of v * scale to an LDS (or global) word.
__device__ __forceinline__ void add_fixed(unsigned long long *dst, float v, double scale) {
    atomicAdd(dst, to_fixed_bits(v, scale));
}

// LDS float atomic adds cost ~190 clocks per wave instruction on gfx950 while
// 64-bit integer LDS atomics are about 25x faster, so the private tile is kept
// in 64-bit fixed point (which also makes the sums independent of the order of
// the additions) and converted when it is flushed.
//
// A workgroup takes a contiguous range of the chunk list (the chunks are in tile
// order): while it spreads one chunk the points of the next are already on their
// way, consecutive chunks of one tile share the LDS tile, and the tile goes to
// global memory (integer atomics: neighbouring workgroups may hold parts of the same
// tile) when the tile changes, after kChunksPerFlush chunks (the fixed-point sums
// have room for 8192 contributions of at most 1) and at the end of the range.
constexpr int kChunksPerFlush = 4;
static_assert(kChunkPoints == 2 * kSpreadThreads, "a thread spreads two points of a chunk");
static_assert(kChunksPerFlush * kChunkPoints <= 4096, "a box's fixed-point sums must stay below 2^62");

// In-box coordinate of one embedding coordinate: box as in bin_and_weights, t in [0, 1].
__device__ __forceinline__ void bin_and_coord(float v, const Bounds &bd, int n_boxes, int &box, float &t) {
#pragma clang fp contract(off)
    int b = (int)((v - bd.lo) / bd.box_width);
    b = max(0, b);
    b = min(n_boxes - 1, b);
    box = b;
    const float lower = b * bd.box_width + bd.lo;
    t = (v - lower) / bd.box_width;
}

// Lower edge of a box, rounded as the binning rounds it.
__device__ __forceinline__ float box_lower(int b, const Bounds &bd) {
#pragma clang fp contract(off)
    return b * bd.box_width + bd.lo;
}

// What a point adds to the nine nodes of its box, L_a(u) L_b(v) (1, x, y, x^2 + y^2) with u, v its
// in-box coordinates, is a polynomial in (u, v): the three Lagrange weights are quadratics in their
// coordinate and x = x_box + w u, y = y_box + w v (w the box width).  So the 36 node sums of a box follow
// from the 21 moments sum u^i v^j with (i <= 4, j <= 2) or (i <= 2, j <= 4), and a point costs 21 LDS
// atomics, not 36; the moments lie in [0, 1], so one fixed-point scale (at most 2^50, and small enough
// for a box that holds every point) serves them all and up to 4096 of them sum below 2^62.  The node sums are
// formed from the moments of the whole box in fp64 by the forward row pass, which is exact to fp64 rounding
// where the per-point products were rounded to fp32.
// The moments of a tile are kept for a region of the tile's 5 x 5 boxes plus a rim of kHalo boxes: when the
// grouping by tile is carried over from an earlier step, the points of a tile have moved a little, and the region
// is placed where the tile's points are now (the box of the chunk's first point minus the offset that point had
// when the grouping was made).  Points that have left even the rim ("strays") add their 21 moments to the grid's
// with global atomics - the same integers that the LDS region would have received - and are counted; too many of
// them and the next step groups the points afresh.
constexpr int kHalo = 1;
constexpr int kRegionBoxes = kTileBoxes + 2 * kHalo;
constexpr int kRegionBoxes2 = kRegionBoxes * kRegionBoxes;
constexpr int kMaxSortAge = 32;  // steps a grouping is kept at most
constexpr int kStrayShift = 10;  // ... and only while at most N / 2^10 points strayed in the last step (36 global atomics each),
constexpr int kStrayFloor = 128; // or 128 of a small problem's
__device__ __forceinline__ constexpr int moment_index(int i, int j) { return j <= 2 ? j * 5 + i : 15 + (j - 3) * 3 + i; }

// (At most 128 registers, whatever the compiler would like: beside the attractive kernel's sixteen waves of 64
// registers a compute unit has room for eight waves of 128, one workgroup of this kernel, and for none of more.)
__global__ __launch_bounds__(kSpreadThreads, 4) void spread_kernel(const float2 *__restrict__ tile_xy,
                                                     const int *__restrict__ tile_perm,
                                                     const float2 *__restrict__ yxy, int4 *chunks,
                                                     const int *__restrict__ num_chunks, LoopScalars *sc,
                                                     int slot, int next_slot, int n_boxes, double to_fixed,
                                                     unsigned long long *__restrict__ moments, int keep_grouping) {
    __shared__ unsigned long long acc[kMoments * kRegionBoxes2];  // one plane per moment
    __shared__ int origin[2];
    // The step's resets: the partial sums of z (the gather kernel at the chain's end adds to them) and the
    // bounds slot the coming update will fill.
    if (blockIdx.x == 0 && threadIdx.x < kZParts) sc->z_part[threadIdx.x] = 0ll;
    if (blockIdx.x == 0 && threadIdx.x == 0 && next_slot >= 0) {
        sc->min_enc[next_slot] = 0xffffffffu;
        sc->max_enc[next_slot] = 0u;
    }
    const int nc = *num_chunks;
    // Neighbouring stretches of the chunk list (tiles next to each other) go to workgroups of one XCD: the
    // points of a region of the embedding tend to have numbers from one range, which that XCD's L2 then serves.
    const int share = xcd_row_block(blockIdx.x, gridDim.x);  // (the grid is a multiple of the XCD count)
    const int c0 = (int)((long long)share * nc / gridDim.x);
    const int c1 = (int)((long long)(share + 1) * nc / gridDim.x);
    if (share < 0 || c0 >= c1) return;
    const bool reuse = keep_grouping && sc->reuse_sort;
    const int tid = threadIdx.x;
    for (int e = tid; e < kMoments * kRegionBoxes2; e += kSpreadThreads) acc[e] = 0ull;
    const int tiles_per_dim = (n_boxes + kTileBoxes - 1) / kTileBoxes;
    const Bounds bd = load_bounds(sc, slot, n_boxes);
    // Unconditional, clamped loads: a chunk holds at least one point.  With a grouping carried over, the
    // positions are the current ones of the points the grouping lists (the interleaved copy the update keeps):
    // a chunk's list of points is fetched two chunks ahead, its positions one chunk ahead, so that neither load
    // is waited for where it is issued.
    const float2 *src = reuse ? yxy : tile_xy;
    auto fetch_index = [&](const int4 &ch, int (&idx)[2]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int pos = ch.y + min(tid + u * kSpreadThreads, ch.z - 1);
            idx[u] = reuse ? tile_perm[pos] : pos;
        }
    };
    auto fetch = [&](const int (&idx)[2], float2 (&pt)[2]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) pt[u] = src[idx[u]];
    };
    int4 ch = chunks[c0];
    int4 next_ch = c0 + 1 < c1 ? chunks[c0 + 1] : ch;
    float2 pt[2];
    int next_idx[2];
    {
        int idx[2];
        fetch_index(ch, idx);
        fetch_index(next_ch, next_idx);
        fetch(idx, pt);
    }
    int cur_tile = ch.x, in_tile = 0;
    bool new_run = true;
    unsigned int strays = 0u;
    int ox0 = 0, oy0 = 0;
    for (int c = c0; c < c1; ++c) {
        const bool last = c + 1 == c1;
        float2 next_pt[2] = {pt[0], pt[1]};
        int4 after_ch = next_ch;
        int after_idx[2] = {next_idx[0], next_idx[1]};
        if (!last) {
            fetch(next_idx, next_pt);
            if (c + 2 < c1) {
                after_ch = chunks[c + 2];
                fetch_index(after_ch, after_idx);
            }
        }
        int pbx[2], pby[2];
        float pcu[2], pcv[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            bin_and_coord(pt[u].x, bd, n_boxes, pbx[u], pcu[u]);
            bin_and_coord(pt[u].y, bd, n_boxes, pby[u], pcv[u]);
        }
        // The chunk's anchor: the summed box coordinates of its first 64 points (the clamped loads make that 64
        // whatever the chunk holds).  Stored relative to the region when the grouping is made; on later steps the
        // region goes where the same points' sum puts it, i.e. it follows the mean movement of those points.
        if ((new_run || !reuse) && tid < kWave) {
            int sx = pbx[0], sy = pby[0];
#pragma unroll
            for (int m = kWave / 2; m >= 1; m >>= 1) {
                sx += __shfl_xor(sx, m, kWave);
                sy += __shfl_xor(sy, m, kWave);
            }
            if (tid == 0) {
                const int fx = (cur_tile % tiles_per_dim) * kTileBoxes - kHalo;
                const int fy = (cur_tile / tiles_per_dim) * kTileBoxes - kHalo;
                if (!reuse) {
                    origin[0] = fx;
                    origin[1] = fy;
                    reinterpret_cast<int *>(chunks)[4 * c + 3] = ((sx - kWave * fx) << 16) | (sy - kWave * fy);
                } else {
                    // floor((sum now - sum then) / 64 + 1/2), for either sign
                    origin[0] = (sx - (ch.w >> 16) + kWave / 2 + kWave * 1024) / kWave - 1024;
                    origin[1] = (sy - (ch.w & 0xffff) + kWave / 2 + kWave * 1024) / kWave - 1024;
                }
            }
        }
        if (new_run) {
            __syncthreads();  // the region's place is known (and the region is zero)
            ox0 = origin[0];
            oy0 = origin[1];
            new_run = false;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            bool stray = false;
            if (tid + u * kSpreadThreads < ch.z) {
                const int bx = pbx[u], by = pby[u];
                float pu[5], pv[5];
                pu[0] = pv[0] = 1.0f;
                pu[1] = pcu[u];
                pv[1] = pcv[u];
                const int lx = bx - ox0, ly = by - oy0;
#pragma unroll
                for (int k = 2; k < 5; ++k) {
                    pu[k] = pu[k - 1] * pu[1];
                    pv[k] = pv[k - 1] * pv[1];
                }
                if ((unsigned int)lx < (unsigned int)kRegionBoxes && (unsigned int)ly < (unsigned int)kRegionBoxes) {
                    unsigned long long *dst = acc + lx * kRegionBoxes + ly;
#pragma unroll
                    for (int j = 0; j < 5; ++j)
#pragma unroll
                        for (int i = 0; i < 5; ++i)
                            if (j <= 2 || i <= 2)
                                add_fixed(dst + moment_index(i, j) * kRegionBoxes2, pu[i] * pv[j], to_fixed);
                } else {
                    // A stray: the same 21 integers, straight to the grid's moments.
                    stray = true;
                    unsigned long long *dst = moments + (size_t)bx * kMoments * n_boxes + by;
#pragma unroll
                    for (int j = 0; j < 5; ++j)
#pragma unroll
                        for (int i = 0; i < 5; ++i)
                            if (j <= 2 || i <= 2)
                                add_fixed(dst + (size_t)moment_index(i, j) * n_boxes, pu[i] * pv[j], to_fixed);
                }
            }
            strays += stray ? 1u : 0u;
        }
        ++in_tile;
        if (last || next_ch.x != cur_tile || in_tile == kChunksPerFlush) {
            __syncthreads();
            // The region's moments to the grid's, and the region back to zero.  Neighbouring lanes take neighbouring
            // boxes of one moment (no two lanes on one LDS bank, runs of seven neighbouring words in memory).
            for (int e = tid; e < kMoments * kRegionBoxes2; e += kSpreadThreads) {
                const unsigned long long v = acc[e];
                if (v == 0ull) continue;
                acc[e] = 0ull;
                const int m = e / kRegionBoxes2, box = e % kRegionBoxes2;
                const int bxg = ox0 + box / kRegionBoxes, byg = oy0 + box % kRegionBoxes;
                // (boxes with points lie inside the grid)
                if ((unsigned int)bxg < (unsigned int)n_boxes && (unsigned int)byg < (unsigned int)n_boxes)
                    atomicAdd(moments + ((size_t)bxg * kMoments + m) * n_boxes + byg, v);
            }
            // (the barrier of the next run's start, or the kernel's end, follows)
            cur_tile = next_ch.x;
            in_tile = 0;
            new_run = true;
        }
        ch = next_ch;
        pt[0] = next_pt[0];
        pt[1] = next_pt[1];
        next_ch = after_ch;
        next_idx[0] = after_idx[0];
        next_idx[1] = after_idx[1];
    }
    // Strays are rare: one atomic per wave that met any.
    const unsigned long long any = __ballot(strays != 0u);
    if (any) {
        unsigned int total = strays;
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) total += __shfl_xor(total, m, kWave);
        if ((tid & (kWave - 1)) == 0) atomicAdd(&sc->strays, total);
    }
}

// ---------------------------------------------------------------------------
// Kernel rows: for node offsets a in [0, G) transform the even sequence
// b -> k(a, |b|) = (1 + (a h)^2 + (b h)^2)^-2 (src/kernels/nbodyfft.cu:175-203)
// along b.  Two rows share one complex transform (both spectra are real).
// Output kernel_rows[v][a] for frequencies v in [0, n / 2], n the transform length.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float kernel_value(float lo, float h, int a, int b) {
#pragma clang fp contract(off)
    const float base = lo + h / 2;
    const float ya = base + a * h;
    const float xb = base + b * h;
    const float da = base - ya;
    const float db = base - xb;
    const double s = 1.0 + (double)da * (double)da + (double)db * (double)db;
    return (float)(1.0 / (s * s));
}

// Kernel values of 4 * PAIRS rows of the grid (two rows packed into one complex transform) and their transforms.
template <int THREADS, int PAIRS, int NFFT>
__device__ __forceinline__ void kernel_rows_block(int block, const LoopScalars *sc, int slot, int n_boxes,
                                                  const float2 *__restrict__ tw, float *__restrict__ kernel_rows,
                                                  float2 (*s)[NFFT]) {
    using T = Transform<NFFT>;
    constexpr int kTransforms = 2 * PAIRS;
    const int tid = threadIdx.x;
    const int G = n_boxes * kInterp;
    const Bounds bd = load_bounds(sc, slot, n_boxes);
    const int a0 = block * 2 * kTransforms;
    for (int e = tid; e < kTransforms * NFFT; e += THREADS) {
        const int f = e / NFFT, m = e - f * NFFT;
        const int b = m < NFFT / 2 ? m : NFFT - m;
        const int ra = a0 + 2 * f;
        float2 v = make_float2(0.f, 0.f);
        if (b < G) {
            if (ra < G) v.x = kernel_value(bd.lo, bd.h, ra, b);
            if (ra + 1 < G) v.y = kernel_value(bd.lo, bd.h, ra + 1, b);
        }
        s[f][T::slot(m)] = v;
    }
    __syncthreads();
    T::forward(&s[0][0], kTransforms, tw, tid, THREADS);
    for (int e = tid; e < kTransforms * NFFT; e += THREADS) {
        const int f = e / NFFT, pos = e - f * NFFT;
        const int v = T::frequency(pos);
        const int ra = a0 + 2 * f;
        if (v <= NFFT / 2 && ra < kNodePad) {
            const float2 val = s[f][T::slot(pos)];
            *reinterpret_cast<float2 *>(kernel_rows + (size_t)v * kNodePad + ra) = val;
        }
    }
}

// ---------------------------------------------------------------------------
// Row pass: transforms ROWS grid rows (x nodes m0 ...), both plane pairs, along the y-node axis.  The charges
// of a node, w[node][t] = sum over the points of its box of L_a(u) L_b(v) q_t, are formed here from the box's
// moments: with L_a(u) = sum_i ca_i u^i, L_b(v) = sum_j cb_j v^j, x = x_box + w u and y = y_box + w v (w the box
// width), the four terms are combinations of the five sums s_kl = sum_ij ca_i cb_j M(i + k, j + l),
// (k, l) = (0,0), (1,0), (0,1), (2,0), (0,2), taken in fp64.  Output is transposed:
// row_spectra[pair][pos][m], pos = digit-reversed frequency position.
//
// Two rows per workgroup (512 threads, 32 KB of LDS) is what the loop uses: one such workgroup fits into the 34 KB
// of LDS (27 allocation units of 1280 bytes) that a workgroup of the attractive kernel leaves on a compute unit,
// provided those are in one piece (the loop enqueues the attractive kernel first for that reason).  One row per
// workgroup (256 threads, 16 KB) measured 21 us against 17 us alone and 2 % fewer iterations per second.
// ---------------------------------------------------------------------------
template <int ROWS, int NFFT>
__global__ __launch_bounds__(256 * ROWS) void conv_rows_forward_kernel(const unsigned long long *__restrict__ moments,
                                                                       double from_fixed, LagrangeMonomials mono,
                                                                       float4 *__restrict__ charges_out, int G,
                                                                       int n_boxes, const LoopScalars *sc, int slot,
                                                                       const float2 *__restrict__ twiddles,
                                                                       float2 *__restrict__ row_spectra,
                                                                       float *__restrict__ kernel_rows) {
    using T = Transform<NFFT>;
    constexpr int kThreads = 256 * ROWS;
    __shared__ float2 s[2 * ROWS][NFFT];  // [row * 2 + pair]
    const float2 *tw = twiddles;
    const int tid = threadIdx.x;
    // The workgroups past the rows produce the kernel's row spectra (needed by the column
    // pass only): the two jobs are independent and share the launch.
    const int row_blocks = (G + ROWS - 1) / ROWS;
    const int launched = kXcds * ((row_blocks + kXcds - 1) / kXcds);
    if ((int)blockIdx.x >= launched) {
        kernel_rows_block<kThreads, ROWS, NFFT>(blockIdx.x - launched, sc, slot, n_boxes, tw, kernel_rows, s);
        return;
    }
    const int row_block = xcd_row_block(blockIdx.x, row_blocks);
    if (row_block < 0) return;
    const int m0 = row_block * ROWS;
    const float s3 = r2_plane_scale(sc, slot);
    const Bounds bd = load_bounds(sc, slot, n_boxes);
    for (int e = tid; e < ROWS * NFFT; e += kThreads) {
        const int r = e / NFFT, n = e - r * NFFT;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (n < G && m0 + r < G) {
            const int gx = m0 + r;
            const int bx = gx / kInterp, a = gx % kInterp, by = n / kInterp, b = n % kInterp;
            const unsigned long long *src = moments + (size_t)bx * kMoments * n_boxes + by;
            if (src[0] != 0ull) {  // moment (0, 0) counts the points of the box
                double M[kMoments];
#pragma unroll
                for (int m = 0; m < kMoments; ++m) M[m] = (double)(long long)src[(size_t)m * n_boxes] * from_fixed;
                double ca[3], cb[3];
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    ca[i] = a == 0 ? mono.c[0][i] : (a == 1 ? mono.c[1][i] : mono.c[2][i]);
                    cb[i] = b == 0 ? mono.c[0][i] : (b == 1 ? mono.c[1][i] : mono.c[2][i]);
                }
                double s00 = 0.0, s10 = 0.0, s01 = 0.0, s20 = 0.0, s02 = 0.0;
#pragma unroll
                for (int i = 0; i < 3; ++i)
#pragma unroll
                    for (int j = 0; j < 3; ++j) {
                        const double cc = ca[i] * cb[j];
                        s00 += cc * M[moment_index(i, j)];
                        s10 += cc * M[moment_index(i + 1, j)];
                        s01 += cc * M[moment_index(i, j + 1)];
                        s20 += cc * M[moment_index(i + 2, j)];
                        s02 += cc * M[moment_index(i, j + 2)];
                    }
                const double bw = bd.box_width;
                const double xl = box_lower(bx, bd), yl = box_lower(by, bd);
                v.x = (float)s00;
                v.y = (float)(xl * s00 + bw * s10);
                v.z = (float)(yl * s00 + bw * s01);
                v.w = (float)((xl * xl + yl * yl) * s00 + 2.0 * bw * (xl * s10 + yl * s01) + bw * bw * (s20 + s02));
            }
            if (charges_out) charges_out[(size_t)gx * G + n] = v;
        }
        s[r * 2 + 0][T::slot(n)] = make_float2(v.x, v.w * s3);  // planes 1 and r^2 / m^2
        s[r * 2 + 1][T::slot(n)] = make_float2(v.y, v.z);       // planes x and y
    }
    __syncthreads();
    T::forward(&s[0][0], 2 * ROWS, tw, tid, kThreads);
    for (int e = tid; e < 2 * NFFT; e += kThreads) {
        const int pair = e / NFFT, pos = e - pair * NFFT;
        float2 *dst = row_spectra + ((size_t)pair * NFFT + pos) * kNodePad + m0;
        if (ROWS == 2) {
            const float2 r0 = s[0 + pair][T::slot(pos)], r1 = s[2 + pair][T::slot(pos)];
            *reinterpret_cast<float4 *>(dst) = make_float4(r0.x, r0.y, r1.x, r1.y);
        } else {
            *dst = s[pair][T::slot(pos)];
        }
    }
}

// ---------------------------------------------------------------------------
// Column pass for two spectrum positions: forward transform along the x-node
// axis, multiply by the kernel spectrum, inverse transform.  The kernel
// spectrum column of each position is produced here from kernel_rows (one more
// packed transform) so it never travels through memory.
// ---------------------------------------------------------------------------
// The two plane pairs go through the transforms together: half as many passes one after the other as with one
// pair at a time (24 KB of LDS: 1 % slower at a million points, 3-4 % slower per step from 5000 to 800000).
//
// SLIM = false: the kernel's columns are transformed with the data, as a fifth transform (40 KB of LDS).
// SLIM = true: they are transformed first, on their own, and their spectrum kept in registers (a thread multiplies
// the same two positions of every transform), so the workgroup holds four transforms: 32 KB, the 26 allocation
// units of LDS that fit beside a workgroup of the attractive kernel (27 free), where 40 KB do not.  The extra pass
// has work for half the threads and costs 1.5 us alone.
template <bool SLIM, int NFFT>
__global__ __launch_bounds__(512) void conv_columns_kernel(const float2 *__restrict__ row_spectra, int G,
                                                           const float *__restrict__ kernel_rows,
                                                           const float2 *__restrict__ twiddles,
                                                           float2 *__restrict__ col_results,
                                                           unsigned long long *__restrict__ moments,
                                                           int moment_words) {
    // The forward row pass has consumed the box moments: back to zero for the next step's spread.
    for (int e = blockIdx.x * 512 + threadIdx.x; e < moment_words; e += gridDim.x * 512) moments[e] = 0ull;
    // Layout: [pair in flight][col], then (SLIM = false) the kernel columns; every transform swizzled, see pad().
    constexpr int kPairsInFlight = 2;
    constexpr int kData = 2 * kPairsInFlight;  // transforms of data per round
    constexpr int kKernelSlot = SLIM ? 0 : kData;
    using T = Transform<NFFT>;
    static_assert(!SLIM || NFFT == 2 * 512, "the slim form keeps positions tid and tid + 512 of the kernel's spectrum");
    __shared__ float2 s[SLIM ? kData : kData + 1][NFFT];
    const float2 *tw = twiddles;
    const int tid = threadIdx.x;
    const int c0 = blockIdx.x * 2;
    {
        int v0 = T::frequency(c0), v1 = T::frequency(c0 + 1);
        v0 = min(v0, NFFT - v0);
        v1 = min(v1, NFFT - v1);
        for (int m = tid; m < NFFT; m += 512) {
            const int a = m < NFFT / 2 ? m : NFFT - m;
            float2 v = make_float2(0.f, 0.f);
            if (a < G) {
                v.x = kernel_rows[(size_t)v0 * kNodePad + a];
                v.y = kernel_rows[(size_t)v1 * kNodePad + a];
            }
            s[kKernelSlot][T::slot(m)] = v;
        }
    }
    float2 kk_reg[2] = {make_float2(0.f, 0.f), make_float2(0.f, 0.f)};  // SLIM: the kernel's spectrum at tid, tid + 512
    if constexpr (SLIM) {
        __syncthreads();
        T::forward(&s[0][0], 1, tw, tid, 512);
        kk_reg[0] = s[0][T::slot(tid)];
        kk_reg[1] = s[0][T::slot(tid + 512)];
        __syncthreads();
    }
    for (int pair0 = 0; pair0 < 2; pair0 += kPairsInFlight) {
        for (int e = tid; e < kData * NFFT; e += 512) {
            const int t = e / NFFT, m = e - t * NFFT;  // t = pair in flight * 2 + col
            float2 v = make_float2(0.f, 0.f);
            if (m < G) v = row_spectra[((size_t)(pair0 + (t >> 1)) * NFFT + c0 + (t & 1)) * kNodePad + m];
            s[t][T::slot(m)] = v;
        }
        __syncthreads();
        // (SLIM = false: the kernel columns are transformed with the first round)
        T::forward(&s[0][0], !SLIM && pair0 == 0 ? kData + 1 : kData, tw, tid, 512);
#pragma unroll
        for (int r = 0; r < (kData * NFFT + 511) / 512; ++r) {
            const int e = tid + r * 512;
            if (kData * NFFT % 512 != 0 && e >= kData * NFFT) break;
            const int t = e / NFFT, m = e - t * NFFT;  // (1024 points: m = tid + 512 (r & 1))
            const float2 kk = SLIM ? kk_reg[r & 1] : s[kKernelSlot][T::slot(m)];
            const float kv = (t & 1) ? kk.y : kk.x;
            float2 v = s[t][T::slot(m)];
            v.x *= kv;
            v.y *= kv;
            s[t][T::slot(m)] = v;
        }
        __syncthreads();
        T::inverse(&s[0][0], kData, tw, tid, 512);
        for (int e = tid; e < kData * NFFT; e += 512) {
            const int t = e / NFFT, m = e - t * NFFT;
            if (m < G)
                col_results[((size_t)(pair0 + (t >> 1)) * NFFT + c0 + (t & 1)) * kNodePad + m] = s[t][T::slot(m)];
        }
        __syncthreads();
    }
}

// The column pass on 800-point transforms, with the ends of the transforms in memory: the first forward pass takes
// its elements straight from the row spectra (and the kernel's column from kernel_rows), the first inverse pass
// multiplies by the kernel's spectrum as it loads, and the last inverse pass stores the G rows that are wanted:
// five trips through the LDS per element instead of eight, three barriers fewer.
// SLIM = false: the kernel's two columns ride along as a fifth transform (32000 bytes of LDS).
// SLIM = true: they are transformed first, alone, and every thread keeps the ten values its butterfly of the
// first inverse pass multiplies by: four transforms, 25600 bytes, like the row passes - the 20 allocation units
// of 1280 bytes that are left in one piece on a compute unit that holds a workgroup of the attractive kernel
// (101 units) and one of the spreading kernel (7), whichever of the two was placed first.
template <bool SLIM>
__global__ __launch_bounds__(512) void conv_columns_short_kernel(const float2 *__restrict__ row_spectra, int G,
                                                                 const float *__restrict__ kernel_rows,
                                                                 const float2 *__restrict__ tw,
                                                                 float2 *__restrict__ col_results,
                                                                 unsigned long long *__restrict__ moments,
                                                                 int moment_words) {
    constexpr int N = kFftShort;
    using T = Transform<N>;
    for (int e = blockIdx.x * 512 + threadIdx.x; e < moment_words; e += gridDim.x * 512) moments[e] = 0ull;
    constexpr int kKernelSlot = SLIM ? 0 : 4;
    __shared__ float2 s[SLIM ? 4 : 5][N];  // [pair * 2 + col]; SLIM = false: then the kernel's two columns
    const int tid = threadIdx.x;
    const int c0 = blockIdx.x * 2;
    int v0 = T::frequency(c0), v1 = T::frequency(c0 + 1);
    v0 = min(v0, N - v0);
    v1 = min(v1, N - v1);
    const float *k0 = kernel_rows + (size_t)v0 * kNodePad, *k1 = kernel_rows + (size_t)v1 * kNodePad;
    auto lds_load = [&](int f, int i, int) { return s[f][i]; };
    auto lds_store = [&](int f, int i, int, float2 v) { s[f][i] = v; };
    auto kernel_column = [&](int m) {
        const int a = m < N / 2 ? m : N - m;
        return a < G ? make_float2(k0[a], k1[a]) : make_float2(0.f, 0.f);
    };
    auto data_column = [&](int f, int m) {
        return m < G ? row_spectra[((size_t)(f >> 1) * N + c0 + (f & 1)) * kNodePad + m] : make_float2(0.f, 0.f);
    };
    float kreg[10] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if constexpr (SLIM) {
        mixed_pass_io<N, 800, 8, false>(1, tw, tid, 512, [&](int, int m, int) { return kernel_column(m); }, lds_store);
        __syncthreads();
        mixed_pass<N, 100, 10, false>(&s[0][0], 1, tw, tid, 512);
        mixed_pass<N, 10, 10, false>(&s[0][0], 1, tw, tid, 512);
        if (tid < 4 * (N / 10)) {  // the thread's butterfly of the first inverse pass: transform tid / 80, tens tid % 80
            const int f = tid / (N / 10), b = tid - f * (N / 10);
#pragma unroll
            for (int j = 0; j < 10; ++j) {
                const float2 kk = s[0][10 * b + j];
                kreg[j] = (f & 1) ? kk.y : kk.x;
            }
        }
        __syncthreads();
        mixed_pass_io<N, 800, 8, false>(4, tw, tid, 512, [&](int f, int m, int) { return data_column(f, m); },
                                        lds_store);
    } else {
        mixed_pass_io<N, 800, 8, false>(
            5, tw, tid, 512, [&](int f, int m, int) { return f < 4 ? data_column(f, m) : kernel_column(m); },
            lds_store);
    }
    __syncthreads();
    mixed_pass<N, 100, 10, false>(&s[0][0], SLIM ? 4 : 5, tw, tid, 512);
    mixed_pass<N, 10, 10, false>(&s[0][0], SLIM ? 4 : 5, tw, tid, 512);
    mixed_pass_io<N, 10, 10, true>(
        4, tw, tid, 512,
        [&](int f, int i, int j) {
            const float2 v = s[f][i];
            float kv;
            if constexpr (SLIM) {
                kv = kreg[j];
            } else {
                const float2 kk = s[kKernelSlot][i];
                kv = (f & 1) ? kk.y : kk.x;
            }
            return make_float2(v.x * kv, v.y * kv);
        },
        lds_store);
    __syncthreads();
    mixed_pass<N, 100, 10, true>(&s[0][0], 4, tw, tid, 512);
    mixed_pass_io<N, 800, 8, true>(4, tw, tid, 512, lds_load, [&](int f, int m, int, float2 v) {
        if (m < G) col_results[((size_t)(f >> 1) * N + c0 + (f & 1)) * kNodePad + m] = v;
    });
}

// ---------------------------------------------------------------------------
// Inverse row pass for x nodes m0, m0+1: consumes digit-reversed positions,
// produces node potentials in natural order, scaled by 1 / (transform length)^2.
// ---------------------------------------------------------------------------
template <int NFFT>
__global__ __launch_bounds__(kRowThreads) void conv_rows_inverse_kernel(const float2 *__restrict__ col_results, int G,
                                                                const LoopScalars *sc, int slot,
                                                                const float2 *__restrict__ twiddles,
                                                                float4 *__restrict__ node_potentials) {
    using T = Transform<NFFT>;
    __shared__ float2 s[4][NFFT];  // [row * 2 + pair]
    const float2 *tw = twiddles;
    const int tid = threadIdx.x;
    const int row_block = xcd_row_block(blockIdx.x, (G + 1) / 2);
    if (row_block < 0) return;
    const int m0 = row_block * 2;
    for (int e = tid; e < 2 * NFFT; e += kRowThreads) {
        const int pair = e / NFFT, pos = e - pair * NFFT;
        const float4 v =
            *reinterpret_cast<const float4 *>(col_results + ((size_t)pair * NFFT + pos) * kNodePad + m0);
        s[0 + pair][T::slot(pos)] = make_float2(v.x, v.y);
        s[2 + pair][T::slot(pos)] = make_float2(v.z, v.w);
    }
    __syncthreads();
    T::inverse(&s[0][0], 4, tw, tid, kRowThreads);
    const float scale = 1.0f / ((float)NFFT * (float)NFFT);
    const float scale3 = scale / r2_plane_scale(sc, slot);
    for (int e = tid; e < 2 * NFFT; e += kRowThreads) {
        const int r = e / NFFT, n = e - r * NFFT;
        if (n < G && m0 + r < G) {
            const float2 p0 = s[r * 2 + 0][T::slot(n)], p1 = s[r * 2 + 1][T::slot(n)];
            node_potentials[(size_t)(m0 + r) * G + n] =
                make_float4(p0.x * scale, p1.x * scale, p1.y * scale, p0.y * scale3);
        }
    }
}

// ---------------------------------------------------------------------------
// Gather + force assembly: phi_i = sum_{a,b} Lx_a Ly_b y~[node] then
// rep = (x phi1 - phi2, y phi1 - phi3), z_i = (1+x^2+y^2) phi1 - 2(x phi2 + y phi3) + phi4
// (src/kernels/nbodyfft.cu:141-173, src/kernels/rep_forces.cu:3-31).  Block
// partial sums of z_i go to the device scalar with one atomic per block.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gather_forces_kernel(const float *__restrict__ emb, int N,
                                                            const LoopScalars *sc_in, int slot, int n_boxes,
                                                            LagrangeConsts lc,
                                                            const float4 *__restrict__ node_potentials,
                                                            float *__restrict__ rep, float *__restrict__ phi_out,
                                                            LoopScalars *sc, int keep_grouping, double z_scale) {
    __shared__ float partial[256 / kWave];
    // Last kernel of the chain: whether the next step keeps this step's grouping of the points by tile.  (The
    // spread kernel has finished counting; the chain's kernels of this step have all read the flag.)
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        const bool reused = keep_grouping && sc->reuse_sort;
        const int age = reused ? sc->sort_age + 1 : 0;
        const unsigned int strays = sc->strays;
        sc->strays = 0u;
        sc->sort_age = age;
        sc->chain_runs += 1u;
        sc->chain_sorts += reused ? 0u : 1u;
        sc->strays_total += strays;
        sc->reuse_sort = (keep_grouping && strays <= (unsigned int)max(N >> kStrayShift, kStrayFloor) && age < kMaxSortAge) ? 1 : 0;
    }
    const Bounds bd = load_bounds(sc_in, slot, n_boxes);
    const int G = n_boxes * kInterp;
    float z = 0.0f;
    // Grid-stride: the workgroup count stays small because every workgroup ends with an atomic on
    // the one Z accumulator, and same-address atomics serialise.
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < N; i += gridDim.x * blockDim.x) {
        const float x = emb[i], y = emb[N + i];
        int bx, by;
        float Lx[kInterp], Ly[kInterp];
        bin_and_weights(x, bd, n_boxes, lc, bx, Lx);
        bin_and_weights(y, bd, n_boxes, lc, by, Ly);
        float4 phi = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int a = 0; a < kInterp; ++a) {
#pragma unroll
            for (int b = 0; b < kInterp; ++b) {
                const float lw = Lx[a] * Ly[b];
                const float4 yt = node_potentials[(size_t)(bx * kInterp + a) * G + (by * kInterp + b)];
                phi.x += lw * yt.x;
                phi.y += lw * yt.y;
                phi.z += lw * yt.z;
                phi.w += lw * yt.w;
            }
        }
        z += (1 + x * x + y * y) * phi.x - 2 * (x * phi.y + y * phi.z) + phi.w;
        rep[i] = x * phi.x - phi.y;
        rep[N + i] = y * phi.x - phi.z;
        if (phi_out) reinterpret_cast<float4 *>(phi_out)[i] = phi;
    }
    z = group_sum<kWave>(z);
    if ((threadIdx.x & (kWave - 1)) == 0) partial[threadIdx.x / kWave] = z;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < 256 / kWave; ++k) t += partial[k];
        // (a workgroup's own sum is taken in a fixed order; the sums over workgroups are integer sums)
        atomicAdd(reinterpret_cast<unsigned long long *>(&sc->z_part[blockIdx.x % kZParts]),
                  (unsigned long long)__double2ll_rn((double)t * z_scale));
    }
}

__global__ void finish_z_kernel(const LoopScalars *sc, int N, double z_inv_scale, float *out) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        long long z = 0ll;
        for (int k = 0; k < kZParts; ++k) z += sc->z_part[k];
        *out = (float)((double)z * z_inv_scale) - (float)N;  // src/kernels/rep_forces.cu:54
    }
}

}  // namespace

int launch_finish_z(tsne_hip_plan *p, float *normalization, hipStream_t s) {
    finish_z_kernel<<<1, 64, 0, s>>>(p->scalars, p->num_points, 1.0 / p->z_scale, normalization);
    TSNE_LAUNCHED(s);
    return 0;
}

int launch_bounds_reset(tsne_hip_plan *p, int slot, hipStream_t s, bool new_embedding) {
    bounds_reset_kernel<<<1, 64, 0, s>>>(p->scalars, slot, new_embedding ? 1 : 0);
    TSNE_LAUNCHED(s);
    return 0;
}

int launch_bounds(tsne_hip_plan *p, const float *embedding, int slot, hipStream_t s, bool new_embedding) {
    if (launch_bounds_reset(p, slot, s, new_embedding)) return 1;
    const int64_t n = 2 * (int64_t)p->num_points;
    // (few workgroups: each ends with up to two atomics on the same two words; 2048 of them took 47 us at two
    // million coordinates, nearly all of it those atomics)
    const int blocks = (int)std::min<int64_t>(div_up(n, 256 * 4), 256);
    bounds_kernel<<<blocks, 256, 0, s>>>(embedding, n, p->scalars, slot);
    TSNE_LAUNCHED(s);
    return 0;
}

// All kernels of one repulsive-force evaluation.  Expects the bounds of
// `embedding` in `slot`; leaves sum_i z_i in scalars->z_part and resets the other
// bounds slot.  charges_out (optional) receives a copy of the node charges.
int launch_repulsive(tsne_hip_plan *p, const float *embedding, int slot, float *rep, float *point_potentials,
                     float *charges_out, hipStream_t s, bool keep_grouping) {
    const int keep = keep_grouping && p->keep_grouping ? 1 : 0;
    const int N = p->num_points, G = p->n_nodes, nb = p->n_boxes;
    const int tiles_per_dim = (nb + kTileBoxes - 1) / kTileBoxes;
    // Few, large workgroups: every workgroup ends with one global atomic per tile counter, and
    // same-address atomics serialise (about a thousand per counter cost ~20 us).
    // (one point per thread until that many workgroups are in use)
    const int sort_blocks = std::min(div_up(N, 1024), kSortBlocks);
    if (profile_mark(p, kKernelTileCount, s)) return 1;
    TSNE_LOOP_KERNEL(p, (tile_count_kernel), sort_blocks, 1024, 0, s, embedding, N, p->scalars, slot, slot ^ 1, nb, p->tile_count,
                                                   p->tile_cursor, p->chunks, p->num_chunks, p->num_chunks + 1,
                                                   p->point_code, p->wg_tile_base, keep);
    TSNE_LAUNCHED(s);
    if (profile_mark(p, kKernelTileScatter, s)) return 1;
    TSNE_LOOP_KERNEL(p, (tile_scatter_kernel), sort_blocks, 1024, 0, s, embedding, N, tiles_per_dim * tiles_per_dim, p->tile_cursor,
                                                     p->point_code, p->wg_tile_base, p->tile_xy, p->tile_perm,
                                                     p->scalars, keep);
    TSNE_LAUNCHED(s);
    if (profile_mark(p, kKernelSpread, s)) return 1;
    // Resident workgroups share the chunk list (its length is only known on the device; with fewer chunks
    // than workgroups the surplus ones exit at once).
    const int spread_blocks =
        xcd_launch_blocks(std::min(N / kChunkPoints + tiles_per_dim * tiles_per_dim + 1, p->spread_grid));
    TSNE_LOOP_KERNEL(p, (spread_kernel), spread_blocks, kSpreadThreads, 0, s, p->tile_xy, p->tile_perm, p->yxy, p->chunks,
                                                           p->num_chunks, p->scalars, slot, slot ^ 1, nb,
                                                           p->moment_scale, p->box_moments, keep);
    TSNE_LAUNCHED(s);
    // Transform length: 800 points where the padded grid (2 G - 1) fits, else 1024 (TSNE_FFT=1024 forces the latter).
    const char *fft_env = getenv("TSNE_FFT");  // (read on every call, like the column pass's switch below)
    const bool long_only = fft_env && atoi(fft_env) == kFft;
    const bool short_fft = 2 * G - 1 <= kFftShort && !long_only;
    const int row_grid = xcd_launch_blocks(div_up(G, 2));
    const double from_fixed = 1.0 / p->moment_scale;
    float4 *charges4 = reinterpret_cast<float4 *>(charges_out);
    if (profile_mark(p, kKernelConvRowsForward, s)) return 1;
    if (short_fft)
        TSNE_LOOP_KERNEL(p, (conv_rows_forward_kernel<2, kFftShort>), row_grid + div_up(G, 8), 512, 0, s, p->box_moments, from_fixed, p->monomials, charges4, G, nb, p->scalars, slot, p->twiddles_short,
            p->row_spectra, p->kernel_rows);
    else
        TSNE_LOOP_KERNEL(p, (conv_rows_forward_kernel<2, kFft>), row_grid + div_up(G, 8), 512, 0, s, p->box_moments, from_fixed, p->monomials, charges4, G, nb, p->scalars, slot, p->twiddles, p->row_spectra,
            p->kernel_rows);
    TSNE_LAUNCHED(s);
    if (profile_mark(p, kKernelConvColumns, s)) return 1;
    const char *slim_env = getenv("TSNE_SLIM_COLUMNS");
    const int slim_mode = slim_env ? atoi(slim_env) : -1;
    const bool slim = slim_mode < 0 ? (p->blocked_ready && p->strip_rows >= 1024) : slim_mode == 1;
    const int moment_words = kMoments * nb * nb;
    if (short_fft && slim)
        TSNE_LOOP_KERNEL(p, (conv_columns_short_kernel<true>), kFftShort / 2, 512, 0, s, p->row_spectra, G, p->kernel_rows, p->twiddles_short, p->col_results, p->box_moments, moment_words);
    else if (short_fft)
        TSNE_LOOP_KERNEL(p, (conv_columns_short_kernel<false>), kFftShort / 2, 512, 0, s, p->row_spectra, G, p->kernel_rows, p->twiddles_short, p->col_results, p->box_moments, moment_words);
    else if (slim)
        TSNE_LOOP_KERNEL(p, (conv_columns_kernel<true, kFft>), kFft / 2, 512, 0, s, p->row_spectra, G, p->kernel_rows, p->twiddles,
                                                                 p->col_results, p->box_moments, moment_words);
    else
        TSNE_LOOP_KERNEL(p, (conv_columns_kernel<false, kFft>), kFft / 2, 512, 0, s, p->row_spectra, G, p->kernel_rows, p->twiddles,
                                                                  p->col_results, p->box_moments, moment_words);
    TSNE_LAUNCHED(s);
    if (profile_mark(p, kKernelConvRowsInverse, s)) return 1;
    if (short_fft)
        TSNE_LOOP_KERNEL(p, (conv_rows_inverse_kernel<kFftShort>), row_grid, kRowThreads, 0, s, p->col_results, G, p->scalars, slot,
                                                                            p->twiddles_short, p->node_potentials);
    else
        TSNE_LOOP_KERNEL(p, (conv_rows_inverse_kernel<kFft>), row_grid, kRowThreads, 0, s, p->col_results, G, p->scalars, slot,
                                                                       p->twiddles, p->node_potentials);
    TSNE_LAUNCHED(s);
    if (profile_mark(p, kKernelGather, s)) return 1;
    TSNE_LOOP_KERNEL(p, (gather_forces_kernel), std::min(div_up(N, 256), 1024), 256, 0, s, embedding, N, p->scalars, slot, nb, p->lagrange,
                                                        p->node_potentials, rep, point_potentials, p->scalars, keep,
                                                        p->z_scale);
    TSNE_LAUNCHED(s);
    return 0;
}

}  // namespace tsnehip
