// CPU restatement of the tsne-cuda FIt-SNE pipeline.  TEST INFRASTRUCTURE ONLY.
//
// This file is the parity oracle and the reported CPU baseline.  It is never
// linked into, loaded by, or called from the shipped library: only the tests,
// the smoke check and the benchmark's cpu_baseline leg may load it.
//
// Every function restates one stage of the reference (paths are relative to the
// reference checkout) with the same data layouts and the same stage boundaries:
//
//   oracle_knn            exact kNN that stands in for the FAISS call at
//                         src/util/distance_utils.cu:79-121 (definition below)
//   oracle_knn_ivf        the library's approximate (inverted-file) search, structured as the FAISS call above
//   oracle_max_normalize  src/util/math_utils.cu:66-74
//   oracle_perplexity     src/kernels/perplexity_search.cu:10-141
//   oracle_symmetrize     src/util/math_utils.cu:269-308
//   oracle_attractive     src/kernels/attr_forces.cu:129-184
//   oracle_repulsive      src/kernels/rep_forces.cu:3-92, src/kernels/nbodyfft.cu:3-442,
//                         src/fit_tsne.cu:246-323,430-467
//   oracle_update         src/kernels/apply_forces.cu:11-57
//   oracle_init           src/fit_tsne.cu:184-204 (random initial embeddings)
//   oracle_fit            src/fit_tsne.cu:84-624 (schedule, state, outputs)
//   oracle_kl             build-defined evaluator (the reference never computes KL)
//
// Pinning status (what fixes each function independently of this file):
//   knn         brute force over numpy float32 arithmetic + sklearn brute kNN
//   knn_ivf     a numpy restatement of the candidate rule on small inputs; with every list probed it must
//               reduce to the exact search; recall against the exact search
//   max_norm    closed form
//   perplexity  row sums, entropy target, uniform closed form, sklearn bisection;
//               its exp / log against double-precision exp / log (<= 2 units in the last place),
//               its row-sum order against an exact (fsum) sum
//   symmetrize  dense (A + A^T)/2N masked to the pattern; the full (CSR) form against the dense
//               matrix and scipy.sparse
//   attractive  dense O(N^2) sum
//   repulsive   direct node-to-node convolution on reduced grids, numpy FFT at
//               full size, exact O(N^2) sums to interpolation accuracy
//   update      hand-computed single-coordinate cases
//   init        the std:: engine and distributions themselves (oracle_init_std), moments of the draws
//   The reference's own tests hold no golden vectors for this path and its kNN
//   lives in un-vendored FAISS (v1.9.0, approximate IVF): kNN parity against the
//   reference's *values* is unpinned; it is pinned against the exact definition.
//
// Floating point: fp32 wherever the reference is fp32, no implicit contraction
// (build with -ffp-contract=off); fused multiply-adds appear only where written.

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <complex>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---------------------------------------------------------------------------
// Exact kNN definition.  For a query i the candidates are all j != i; the
// squared distance is accumulated in fp32 over ascending dimension with one
// fused multiply-add per dimension: acc = fma(x_id - x_jd, x_id - x_jd, acc).
// The K-1 smallest by (distance, index) follow (i, 0.0f) which is forced into
// slot 0 (the reference relies on self being neighbour 0 with distance 0,
// src/kernels/perplexity_search.cu:30-32).
// ---------------------------------------------------------------------------
struct Cand {
    float d;
    int j;
};
inline bool cand_less(const Cand &a, const Cand &b) { return a.d < b.d || (a.d == b.d && a.j < b.j); }

// Query rows rows[0 .. n_rows); output row r belongs to query rows[r].
void knn_rows(const float *X, const float *Xt, int N, int D, int K, const int *rows, int n_rows, int *idx,
              float *d2) {
    const int JB = 2048;
#pragma omp parallel
    {
        std::vector<float> acc(JB);
        std::vector<Cand> heap;
        heap.reserve(K);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < n_rows; ++r) {
            const int i = rows[r];
            heap.clear();
            const int want = K - 1;
            const float *xi = X + (size_t)i * D;
            for (int j0 = 0; j0 < N; j0 += JB) {
                const int jn = std::min(JB, N - j0);
                for (int t = 0; t < jn; ++t) acc[t] = 0.0f;
                for (int d = 0; d < D; ++d) {
                    const float xv = xi[d];
                    const float *col = Xt + (size_t)d * N + j0;
                    for (int t = 0; t < jn; ++t) {
                        const float df = xv - col[t];
                        acc[t] = std::fmaf(df, df, acc[t]);
                    }
                }
                if (want <= 0) continue;
                for (int t = 0; t < jn; ++t) {
                    const int j = j0 + t;
                    if (j == i) continue;
                    Cand c{acc[t], j};
                    if ((int)heap.size() < want) {
                        heap.push_back(c);
                        std::push_heap(heap.begin(), heap.end(), cand_less);
                    } else if (cand_less(c, heap.front())) {
                        std::pop_heap(heap.begin(), heap.end(), cand_less);
                        heap.back() = c;
                        std::push_heap(heap.begin(), heap.end(), cand_less);
                    }
                }
            }
            std::sort(heap.begin(), heap.end(), cand_less);
            int *oi = idx + (size_t)r * K;
            float *od = d2 + (size_t)r * K;
            oi[0] = i;
            od[0] = 0.0f;
            for (int s = 1; s < K; ++s) {
                oi[s] = heap[s - 1].j;
                od[s] = heap[s - 1].d;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Radix-2 complex FFT in double, used for the circulant convolution.  The
// reference evaluates the same convolution with 780-point cuFFT transforms in
// fp32 (src/kernels/nbodyfft.cu:289,404,415); any transform length >= 2G-1
// yields the identical linear convolution, so the oracle pads to a power of two
// and works in double so that its own round-off is negligible.
// ---------------------------------------------------------------------------
typedef std::complex<double> cplx;

void fft_inplace(cplx *a, int n, bool inverse, const std::vector<cplx> &tw) {
    for (int i = 1, j = 0; i < n; ++i) {
        int bit = n >> 1;
        for (; j & bit; bit >>= 1) j ^= bit;
        j ^= bit;
        if (i < j) std::swap(a[i], a[j]);
    }
    for (int len = 2; len <= n; len <<= 1) {
        const int step = n / len;
        for (int i = 0; i < n; i += len) {
            for (int k = 0; k < len / 2; ++k) {
                cplx w = tw[(size_t)k * step];
                if (inverse) w = std::conj(w);
                const cplx u = a[i + k];
                const cplx v = a[i + k + len / 2] * w;
                a[i + k] = u + v;
                a[i + k + len / 2] = u - v;
            }
        }
    }
}

void fft2d(std::vector<cplx> &a, int n, bool inverse) {
    std::vector<cplx> tw(n / 2);
    for (int k = 0; k < n / 2; ++k) tw[k] = std::polar(1.0, -2.0 * M_PI * k / n);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < n; ++r) fft_inplace(a.data() + (size_t)r * n, n, inverse, tw);
#pragma omp parallel
    {
        std::vector<cplx> col(n);
#pragma omp for schedule(static)
        for (int c = 0; c < n; ++c) {
            for (int r = 0; r < n; ++r) col[r] = a[(size_t)r * n + c];
            fft_inplace(col.data(), n, inverse, tw);
            for (int r = 0; r < n; ++r) a[(size_t)r * n + c] = col[r];
        }
    }
}

int next_pow2(int v) {
    int n = 1;
    while (n < v) n <<= 1;
    return n;
}

// Kernel value at node offset (a, b): src/kernels/nbodyfft.cu:175-203.  The
// reference forms both node coordinates in fp32 from (coord_min + h/2) and
// subtracts them in fp32 before the double-precision powers.
inline float kernel_tilde_value(float coord_min, float h, int a, int b) {
    const float base = coord_min + h / 2;
    const float ya = base + a * h;
    const float xb = base + b * h;
    const float da = base - ya;
    const float db = base - xb;
    const double s = 1.0 + (double)da * (double)da + (double)db * (double)db;
    return (float)(1.0 / (s * s));
}

struct Grid {
    int nb, p, G;
    float coord_min, coord_max, box_width, h;
    float spacing[8], denom[8];
};

// src/fit_tsne.cu:303-321 (node positions and Lagrange denominators, fp32) and
// src/fit_tsne.cu:430-442 (one scalar min and max over all 2N coordinates).
Grid make_grid(const float *Y, int N, int nb, int p) {
    Grid g;
    g.nb = nb;
    g.p = p;
    g.G = nb * p;
    float lo = Y[0], hi = Y[0];
    for (size_t t = 0; t < (size_t)2 * N; ++t) {
        lo = std::min(lo, Y[t]);
        hi = std::max(hi, Y[t]);
    }
    g.coord_min = lo;
    g.coord_max = hi;
    g.box_width = (hi - lo) / (float)nb;
    g.h = g.box_width / (float)p;
    const float hs = 1 / (float)p;
    g.spacing[0] = hs / 2;
    for (int i = 1; i < p; ++i) g.spacing[i] = g.spacing[i - 1] + hs;
    for (int i = 0; i < p; ++i) {
        g.denom[i] = 1;
        for (int j = 0; j < p; ++j)
            if (i != j) g.denom[i] *= g.spacing[i] - g.spacing[j];
    }
    return g;
}

// src/kernels/nbodyfft.cu:43-105,205-227: box index (clamped), in-box
// coordinate and the p Lagrange basis values for one coordinate.
inline void bin_and_weights(const Grid &g, float v, int &box, float *L) {
    int b = (int)((v - g.coord_min) / g.box_width);
    b = std::max(0, b);
    b = std::min(g.nb - 1, b);
    box = b;
    const float lower = b * g.box_width + g.coord_min;
    const float t = (v - lower) / g.box_width;
    for (int j = 0; j < g.p; ++j) {
        float val = 1;
        for (int k = 0; k < g.p; ++k)
            if (j != k) val *= t - g.spacing[k];
        L[j] = val / g.denom[j];
    }
}

}  // namespace

extern "C" {

int oracle_num_threads() {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// Rows [row_begin, row_end) of the exact kNN of X (N x D row-major); outputs are
// (row_end-row_begin) x K, row-major, int32 indices and fp32 squared distances.
void oracle_knn_row_list(const float *X, int N, int D, int K, const int *rows, int n_rows, int *idx, float *d2) {
    std::vector<float> Xt((size_t)N * D);
#pragma omp parallel for schedule(static)
    for (int d = 0; d < D; ++d)
        for (int i = 0; i < N; ++i) Xt[(size_t)d * N + i] = X[(size_t)i * D + d];
    knn_rows(X, Xt.data(), N, D, K, rows, n_rows, idx, d2);
}

void oracle_knn_rows(const float *X, int N, int D, int K, int row_begin, int row_end, int *idx, float *d2) {
    std::vector<int> rows(row_end - row_begin);
    for (int i = row_begin; i < row_end; ++i) rows[i - row_begin] = i;
    oracle_knn_row_list(X, N, D, K, rows.data(), (int)rows.size(), idx, d2);
}

void oracle_knn(const float *X, int N, int D, int K, int *idx, float *d2) {
    oracle_knn_rows(X, N, D, K, 0, N, idx, d2);
}

// Approximate neighbours through an inverted file: the library's approximate mode, which keeps the structure
// and parameters of the reference's FAISS IndexIVFFlat search (src/util/distance_utils.cu:85-120: nlist lists,
// nprobe probed, L2) - FAISS itself is not among the reference's sources (un-vendored, v1.9.0), so this restates
// the library's documented rule, and what it is held to is that rule plus its recall against the exact search:
//   * every point is filed under its nearest centroid, by (distance, list number), distances accumulated as in
//     the exact search (one fma per dimension);
//   * a list probes the nprobe lists whose centroids are nearest to its own centroid (same order; itself
//     first), and a point probes what its list probes;
//   * the points are renumbered list by list, old numbers ascending inside a list; tiles are runs of 128
//     consecutive new numbers;
//   * the candidates of a query are the points of its tile's 8 neighbours either side in the numbering and of
//     every tile that overlaps a list probed by the list of some query of its tile;
//   * among them the K - 1 nearest by (distance, new number), the query itself first.
// Output in the caller's (old) numbering.  list_out (optional): N list numbers; list_probes_out (optional):
// nlist x nprobe.
void oracle_knn_ivf(const float *X, int N, int D, int K, const float *centroids, int nlist, int nprobe, int *idx_out,
                    float *d2_out, int *list_out, int *list_probes_out) {
    auto nearest = [&](const float *q, int count, int *out) {
        std::vector<Cand> all(nlist);
        for (int c = 0; c < nlist; ++c) {
            float acc = 0.0f;
            for (int d = 0; d < D; ++d) {
                const float df = q[d] - centroids[(size_t)c * D + d];
                acc = std::fmaf(df, df, acc);
            }
            all[c] = Cand{acc, c};
        }
        std::partial_sort(all.begin(), all.begin() + count, all.end(), cand_less);
        for (int r = 0; r < count; ++r) out[r] = all[r].j;
    };
    std::vector<int> list_of(N), lprobes((size_t)nlist * nprobe);
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; ++i) nearest(X + (size_t)i * D, 1, &list_of[i]);
#pragma omp parallel for schedule(static)
    for (int l = 0; l < nlist; ++l) nearest(centroids + (size_t)l * D, nprobe, &lprobes[(size_t)l * nprobe]);
    if (list_out) std::memcpy(list_out, list_of.data(), list_of.size() * sizeof(int));
    if (list_probes_out) std::memcpy(list_probes_out, lprobes.data(), lprobes.size() * sizeof(int));
    std::vector<int> order(N);
    for (int i = 0; i < N; ++i) order[i] = i;
    std::stable_sort(order.begin(), order.end(),
                     [&](int a, int b) { return list_of[a] < list_of[b]; });
    std::vector<int> list_start(nlist + 1, 0);
    for (int i = 0; i < N; ++i) list_start[list_of[i] + 1] += 1;
    for (int l = 0; l < nlist; ++l) list_start[l + 1] += list_start[l];
    const int T = (N + 127) / 128;
#pragma omp parallel
    {
        std::vector<char> probed(nlist), visit(T);
        std::vector<Cand> cands;
#pragma omp for schedule(dynamic, 1)
        for (int qt = 0; qt < T; ++qt) {
            std::fill(probed.begin(), probed.end(), 0);
            std::fill(visit.begin(), visit.end(), 0);
            const int q0 = qt * 128, q1 = std::min(N, q0 + 128);
            for (int r = q0; r < q1; ++r)
                for (int s = 0; s < nprobe; ++s) probed[lprobes[(size_t)list_of[order[r]] * nprobe + s]] = 1;
            for (int t = std::max(0, qt - 8); t <= std::min(T - 1, qt + 8); ++t) visit[t] = 1;
            for (int l = 0; l < nlist; ++l)
                if (probed[l] && list_start[l + 1] > list_start[l])
                    for (int t = list_start[l] / 128; t <= (list_start[l + 1] - 1) / 128; ++t) visit[t] = 1;
            for (int r = q0; r < q1; ++r) {
                const float *xq = X + (size_t)order[r] * D;
                cands.clear();
                for (int t = 0; t < T; ++t) {
                    if (!visit[t]) continue;
                    for (int c = t * 128; c < std::min(N, t * 128 + 128); ++c) {
                        if (c == r) continue;
                        const float *xc = X + (size_t)order[c] * D;
                        float acc = 0.0f;
                        for (int d = 0; d < D; ++d) {
                            const float df = xq[d] - xc[d];
                            acc = std::fmaf(df, df, acc);
                        }
                        cands.push_back(Cand{acc, c});
                    }
                }
                const int keep = std::min<int>(K - 1, (int)cands.size());
                std::partial_sort(cands.begin(), cands.begin() + keep, cands.end(), cand_less);
                int *oi = idx_out + (size_t)order[r] * K;
                float *od = d2_out + (size_t)order[r] * K;
                oi[0] = order[r];
                od[0] = 0.0f;
                for (int s = 1; s < K; ++s) {
                    oi[s] = s - 1 < keep ? order[cands[s - 1].j] : -1;
                    od[s] = s - 1 < keep ? cands[s - 1].d : INFINITY;
                }
            }
        }
    }
}

// src/util/math_utils.cu:66-74: divide every entry by the largest absolute value.
float oracle_max_normalize(float *d2, int64_t n) {
    float m = 0.0f;
    for (int64_t t = 0; t < n; ++t) m = std::max(m, std::fabs(d2[t]));
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < n; ++t) d2[t] = d2[t] / m;
    return m;
}

// exp and log as fixed sequences of correctly rounded single-precision operations (any machine that
// follows the sequence gets the same bits), accurate to about one unit in the last place.  The perplexity
// search stops on |H - ln perplexity| < eps, so the last bit of an exponential can move a row's stopping
// point by a whole bisection step; the reference's __expf / __logf (perplexity_search.cu:32,
// thrust_transform_functions.h:34) cannot be reproduced bit for bit anywhere but on its own GPU, and any
// exp/log this accurate is as good a restatement.  These two are pinned against double-precision
// exp / log in tests/test_oracle.py.
static inline float bits_to_float(uint32_t u) {
    float f;
    std::memcpy(&f, &u, sizeof(f));
    return f;
}
static inline uint32_t float_to_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, sizeof(u));
    return u;
}

// e^x: n = round(x log2 e) by the 1.5 * 2^23 trick, r = x - n ln2 with a split ln2, degree-7 Taylor
// polynomial (Horner, fused multiply-adds), scaling by 2^n in two exact power-of-two factors.
float oracle_expf(float x) {
    if (x != x) return x;
    if (!(x > -104.0f)) return 0.0f;
    if (x > 88.72f) return bits_to_float(0x7f800000u);
    const float t = std::fmaf(x, 1.44269504f, 12582912.0f);
    const float n = t - 12582912.0f;
    float r = std::fmaf(n, -0.693145752f, x);
    r = std::fmaf(n, -1.42860677e-6f, r);
    float p = 1.0f / 5040.0f;
    p = std::fmaf(p, r, 1.0f / 720.0f);
    p = std::fmaf(p, r, 1.0f / 120.0f);
    p = std::fmaf(p, r, 1.0f / 24.0f);
    p = std::fmaf(p, r, 1.0f / 6.0f);
    p = std::fmaf(p, r, 0.5f);
    p = std::fmaf(p, r, 1.0f);
    p = std::fmaf(p, r, 1.0f);
    const int ni = (int)n;
    const int half = ni / 2;
    const float a = bits_to_float((uint32_t)(half + 127) << 23);
    const float b = bits_to_float((uint32_t)(ni - half + 127) << 23);
    return (p * a) * b;
}

// ln v: v = m 2^e, m in [sqrt(1/2), sqrt(2)); f = m - 1, s = f / (2 + f), z = s^2,
// ln m = f - s (f - R), R = z (2/3 + z (2/5 + z (2/7 + z (2/9 + z 2/11)))); ln v = e ln2_hi + (ln m + e ln2_lo).
float oracle_logf(float v) {
    if (v != v) return v;
    if (v < 0.0f) return bits_to_float(0x7fc00000u);
    if (v == 0.0f) return bits_to_float(0xff800000u);
    uint32_t bits = float_to_bits(v);
    if (bits == 0x7f800000u) return v;
    int e = 0;
    if (bits < 0x00800000u) {  // subnormal
        v = v * 33554432.0f;
        bits = float_to_bits(v);
        e = -25;
    }
    bits += 0x3f800000u - 0x3f3504f3u;
    e += (int)(bits >> 23) - 127;
    bits = (bits & 0x007fffffu) + 0x3f3504f3u;
    const float f = bits_to_float(bits) - 1.0f;
    const float s = f / (2.0f + f);
    const float z = s * s;
    float R = 2.0f / 11.0f;
    R = std::fmaf(R, z, 2.0f / 9.0f);
    R = std::fmaf(R, z, 2.0f / 7.0f);
    R = std::fmaf(R, z, 2.0f / 5.0f);
    R = std::fmaf(R, z, 2.0f / 3.0f);
    R = R * z;
    const float ef = (float)e;
    float res = std::fmaf(ef, 1.42860677e-6f, -(s * (f - R)));
    res = res + f;
    return std::fmaf(ef, 0.693145752f, res);
}

// Row sum in the stated order of the search: 64 interleaved partial sums (partial c takes slots c, c + 64,
// c + 128, ... in ascending order, starting from +0), then a balanced tree, partial[c] + partial[c ^ m] for
// m = 32, 16, 8, 4, 2, 1.  (The reference sums a row with cublasSgemv, reduce_utils.cu:24-27, whose order is
// not documented; a pairwise order is what a GPU reduction does and it is one a GPU kernel can follow.)
static inline float ordered_row_sum(const float *v, int K) {
    float part[64];
    for (int c = 0; c < 64; ++c) part[c] = 0.0f;
    for (int s = 0; s < K; ++s) part[s & 63] += v[s];
    for (int m = 32; m > 0; m >>= 1)
        for (int c = 0; c < m; ++c) part[c] = part[c] + part[c + m];
    return part[0];
}

// Array forms of the three helpers above, for the tests that pin them.
void oracle_expf_array(const float *x, int64_t n, float *out) {
    for (int64_t t = 0; t < n; ++t) out[t] = oracle_expf(x[t]);
}
void oracle_logf_array(const float *v, int64_t n, float *out) {
    for (int64_t t = 0; t < n; ++t) out[t] = oracle_logf(v[t]);
}
float oracle_row_sum(const float *v, int K) { return ordered_row_sum(v, K); }

// src/kernels/perplexity_search.cu:81-141.  Rows are independent: the
// reference iterates all rows in lock-step and freezes converged rows, which is
// the same as running each row until it converges or 200 evaluations are done.
// Outputs the row-normalised conditional probabilities of the last evaluated
// beta; beta_out / iters_out (optional) receive that beta and the number of
// evaluations.
void oracle_perplexity(const float *d2, int N, int K, float perplexity, float eps, float *p, float *beta_out,
                       int *iters_out) {
    const float log_target = oracle_logf(perplexity);
#pragma omp parallel
    {
        std::vector<float> row(K), ent_terms(K);
#pragma omp for schedule(static)
        for (int i = 0; i < N; ++i) {
            const float *d = d2 + (size_t)i * K;
            float beta = 1.0f, lo = -FLT_MAX, hi = FLT_MAX;
            float used_beta = beta, sum = 0.0f;
            int it = 0;
            for (;;) {
                for (int s = 0; s < K; ++s) {
                    // perplexity_search.cu:32
                    const float v = (s == 0 && d[s] == 0.0f) ? 0.0f : oracle_expf(-beta * d[s]);
                    row[s] = v;
                    // thrust_transform_functions.h:32-37
                    float e = v * oracle_logf(v);
                    if (e != e || std::isinf(e)) e = 0.0f;
                    ent_terms[s] = e;
                }
                sum = ordered_row_sum(row.data(), K);
                const float ent = ordered_row_sum(ent_terms.data(), K);
                used_beta = beta;
                ++it;
                const float neg_ent = -ent;
                const float H = (neg_ent / sum) + oracle_logf(sum);
                const float diff = H - log_target;
                const bool found = (diff < eps && -diff < eps);
                if (found || it >= 200) break;
                if (diff > 0) {
                    lo = beta;
                    beta = (hi == FLT_MAX || hi == -FLT_MAX) ? beta * 2.0f : (beta + hi) / 2.0f;
                } else {
                    hi = beta;
                    beta = (lo == -FLT_MAX || lo == FLT_MAX) ? beta / 2.0f : (beta + lo) / 2.0f;
                }
            }
            for (int s = 0; s < K; ++s) p[(size_t)i * K + s] = row[s] / sum;
            if (beta_out) beta_out[i] = used_beta;
            if (iters_out) iters_out[i] = it;
        }
    }
}

// ---------------------------------------------------------------------------
// Initial embedding, src/fit_tsne.cu:184-204 (and src/util/random_utils.cu:17-35 for UNIFORM).
// The reference draws from std::default_random_engine(opt.random_seed) with
// std::normal_distribution<float>(0, 1): first 2N values that only feed an unused noise vector
// (x 0.001), then, for GAUSSIAN, the next 2N values x 0.0001 (a double product stored as float), or,
// for UNIFORM, 2N values of std::uniform_real_distribution<float>(-5, 5) from the same engine.
//
// oracle_init spells those std:: components out (libstdc++'s algorithms):
//   engine        minstd_rand0, x <- 16807 x mod (2^31 - 1), seeded with (seed as uint64) mod (2^31 - 1) (1 if that is 0)
//   canonical     one engine call per float: float(x - 1) / 2147483646.0f, clamped below 1
//   normal        Marsaglia's polar method: u, v = 2 c - 1 (double subtraction, stored as float), retried
//                 until 0 < r2 = u u + v v <= 1; m = sqrt(-2 ln r2 / r2); returns v m now and u m at the
//                 next call
//   uniform(a,b)  c (b - a) + a in float
// oracle_init_std calls the std:: classes themselves; tests/test_oracle.py holds the two against each other.
// kind: 0 = UNIFORM, 1 = GAUSSIAN (the TSNE_INIT encodings of src/include/options.h:37-42).
// ---------------------------------------------------------------------------
namespace {
struct MinStd {
    uint32_t x;
    // The engine's seed type is a 64-bit unsigned integer here: an int seed is sign-extended on the way in.
    explicit MinStd(int seed) {
        x = (uint32_t)((uint64_t)(int64_t)seed % 2147483647u);
        if (x == 0) x = 1;
    }
    uint32_t next() {
        x = (uint32_t)(((uint64_t)x * 16807u) % 2147483647u);
        return x;
    }
    float canonical() {
        const float sum = (float)(next() - 1u) * 1.0f;
        const float tmp = 1.0f * 2147483646.0f;  // engine range as a float (rounds to 2^31)
        float ret = sum / tmp;
        if (ret >= 1.0f) ret = std::nextafter(1.0f, 0.0f);
        return ret;
    }
};
struct PolarNormal {
    bool saved_available = false;
    float saved = 0.0f;
    float draw(MinStd &g) {
        float ret;
        if (saved_available) {
            saved_available = false;
            ret = saved;
        } else {
            float u, v, r2;
            do {
                u = (float)(2.0f * g.canonical() - 1.0);
                v = (float)(2.0f * g.canonical() - 1.0);
                r2 = u * u + v * v;
            } while (r2 > 1.0 || r2 == 0.0);
            const float mult = std::sqrt(-2 * std::log(r2) / r2);
            saved = u * mult;
            saved_available = true;
            ret = v * mult;
        }
        return ret * 1.0f + 0.0f;
    }
};
}  // namespace

void oracle_init(int N, int kind, int seed, float *Y) {
    MinStd g(seed);
    PolarNormal normal;
    const size_t n2 = (size_t)2 * N;
    for (size_t i = 0; i < n2; ++i) Y[i] = (float)(0.001 * normal.draw(g));  // the unused noise vector
    if (kind == 0) {
        for (size_t i = 0; i < n2; ++i) Y[i] = g.canonical() * (5.0f - (-5.0f)) + (-5.0f);
    } else {
        for (size_t i = 0; i < n2; ++i) Y[i] = (float)(0.0001 * normal.draw(g));
    }
}

}  // extern "C"
#include <random>
extern "C" {
void oracle_init_std(int N, int kind, int seed, float *Y) {
    std::default_random_engine generator(seed);
    std::normal_distribution<float> distribution1(0.0, 1.0);
    const size_t n2 = (size_t)2 * N;
    for (size_t i = 0; i < n2; ++i) Y[i] = 0.001 * distribution1(generator);
    if (kind == 0) {
        std::uniform_real_distribution<float> distribution(-5, 5);
        for (size_t i = 0; i < n2; ++i) Y[i] = distribution(generator);
    } else {
        for (size_t i = 0; i < n2; ++i) Y[i] = 0.0001 * distribution1(generator);
    }
}

// src/util/math_utils.cu:269-291: symmetrisation restricted to the N x K pattern.
void oracle_symmetrize(const float *p, const int *idx, int N, int K, float *P) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; ++i) {
        for (int s = 0; s < K; ++s) {
            const size_t t = (size_t)i * K + s;
            const int j = idx[t];
            float acc = p[t];
            for (int u = 0; u < K; ++u) acc += (idx[(size_t)j * K + u] == i) ? p[(size_t)j * K + u] : 0.0f;
            P[t] = (float)(acc / (2.0 * N));
        }
    }
}

// Full symmetrisation (A + A^T) / 2N with the union pattern, CSR with ascending columns: what the reference
// holds as a commented-out cuSPARSE routine (src/util/math_utils.cu:76-225: csrsort, csr2csc, csrgeam with
// alpha = beta = 1 / (2N)) and the library offers as an option.  A[i, idx[i,s]] = p[i,s]; an entry's value is
// the fp32 sum of what A and A^T hold there (own entry first), divided by 2.0 * N in double, rounded to float -
// the arithmetic of oracle_symmetrize.  row_ptr: N + 1; col_idx / values: room for 2 N K.  Returns the count.
int64_t oracle_symmetrize_full(const float *p, const int *idx, int N, int K, int *row_ptr, int *col_idx,
                               float *values) {
    struct Item {
        int col;
        float v;
    };
    // The triples are taken entry by entry, (i, j) then (j, i); rows are filled in that order and sorted stably,
    // so equal (row, column) pairs are summed in the order in which they were generated.
    std::vector<std::vector<Item>> rows(N);
    for (int i = 0; i < N; ++i)
        for (int s = 0; s < K; ++s) {
            const size_t t = (size_t)i * K + s;
            const int j = idx[t];
            rows[i].push_back({j, p[t]});
            rows[j].push_back({i, p[t]});
        }
    int64_t out = 0;
    for (int i = 0; i < N; ++i) {
        auto &r = rows[i];
        std::stable_sort(r.begin(), r.end(), [](const Item &a, const Item &b) { return a.col < b.col; });
        row_ptr[i] = (int)out;
        for (size_t a = 0; a < r.size();) {
            float sum = r[a].v;
            size_t b = a + 1;
            for (; b < r.size() && r[b].col == r[a].col; ++b) sum += r[b].v;
            col_idx[out] = r[a].col;
            values[out] = (float)((double)sum / (2.0 * N));
            ++out;
            a = b;
        }
    }
    row_ptr[N] = (int)out;
    return out;
}

// Attractive forces over a CSR pattern (same terms as oracle_attractive, row by row in stored order).
void oracle_attractive_csr(const int *row_ptr, const int *col_idx, const float *values, const float *Y, int N,
                           float *attr) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; ++i) {
        const float ix = Y[i], iy = Y[N + i];
        float ax = 0.0f, ay = 0.0f;
        for (int e = row_ptr[i]; e < row_ptr[i + 1]; ++e) {
            const int j = col_idx[e];
            const float dx = ix - Y[j];
            const float dy = iy - Y[N + j];
            const float w = values[e] / (1 + dx * dx + dy * dy);
            ax += w * dx;
            ay += w * dy;
        }
        attr[i] = ax;
        attr[N + i] = ay;
    }
}

// src/kernels/attr_forces.cu:129-184.  Y is N xs followed by N ys.
void oracle_attractive(const float *P, const int *idx, const float *Y, int N, int K, float *attr) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; ++i) {
        const float ix = Y[i], iy = Y[N + i];
        float ax = 0.0f, ay = 0.0f;
        for (int s = 0; s < K; ++s) {
            const size_t t = (size_t)i * K + s;
            const int j = idx[t];
            const float dx = ix - Y[j];
            const float dy = iy - Y[N + j];
            const float w = P[t] / (1 + dx * dx + dy * dy);
            ax += w * dx;
            ay += w * dy;
        }
        attr[i] = ax;
        attr[N + i] = ay;
    }
}

// Repulsive forces through the interpolation grid.
//   nb, p      boxes per dimension and interpolation nodes per box
//              (130 and 3 in the reference, src/fit_tsne.cu:246-272)
//   rep        2N  (xs then ys): x*phi1 - phi2, y*phi1 - phi3
//   Z_out      sum_i z_i - N                     (rep_forces.cu:18-54)
//   w_out      optional, G*G*4 node charges      (nbodyfft.cu:107-139)
//   yt_out     optional, G*G*4 node potentials   (nbodyfft.cu:23-41)
//   phi_out    optional, N*4 point potentials    (nbodyfft.cu:141-173)
//   direct     non-zero: evaluate the node-to-node sums directly (O(G^4)),
//              no FFT; used to pin the FFT path on reduced grids
void oracle_repulsive(const float *Y, int N, int nb, int p, float *rep, float *Z_out, float *w_out, float *yt_out,
                      float *phi_out, int direct) {
    const Grid g = make_grid(Y, N, nb, p);
    const int G = g.G;
    const int T = 4;
    std::vector<float> w((size_t)G * G * T, 0.0f);
    std::vector<int> bx(N), by(N);
    std::vector<float> Lx((size_t)N * p), Ly((size_t)N * p);

    for (int i = 0; i < N; ++i) {
        bin_and_weights(g, Y[i], bx[i], &Lx[(size_t)i * p]);
        bin_and_weights(g, Y[N + i], by[i], &Ly[(size_t)i * p]);
    }
    // Spread (nbodyfft.cu:107-139): row index of the node grid is the x node.
    for (int i = 0; i < N; ++i) {
        const float x = Y[i], y = Y[N + i];
        const float q[4] = {1.0f, x, y, x * x + y * y};  // rep_forces.cu:57-76
        for (int a = 0; a < p; ++a)
            for (int b = 0; b < p; ++b) {
                const size_t node = (size_t)(bx[i] * p + a) * G + (by[i] * p + b);
                const float lw = Lx[(size_t)i * p + a] * Ly[(size_t)i * p + b];
                for (int t = 0; t < T; ++t) w[node * T + t] += lw * q[t];
            }
    }

    std::vector<float> yt((size_t)G * G * T, 0.0f);
    if (direct) {
        std::vector<float> kt((size_t)G * G);
        for (int a = 0; a < G; ++a)
            for (int b = 0; b < G; ++b) kt[(size_t)a * G + b] = kernel_tilde_value(g.coord_min, g.h, a, b);
#pragma omp parallel for schedule(static)
        for (int m = 0; m < G; ++m)
            for (int n = 0; n < G; ++n) {
                double acc[4] = {0, 0, 0, 0};
                for (int c = 0; c < G; ++c)
                    for (int d = 0; d < G; ++d) {
                        const double kv = kt[(size_t)std::abs(m - c) * G + std::abs(n - d)];
                        const float *wv = &w[((size_t)c * G + d) * T];
                        for (int t = 0; t < T; ++t) acc[t] += kv * wv[t];
                    }
                for (int t = 0; t < T; ++t) yt[((size_t)m * G + n) * T + t] = (float)acc[t];
            }
    } else {
        // Circulant embedding (nbodyfft.cu:3-41,175-203,395-424) at a padded size.
        const int F = next_pow2(2 * G);
        std::vector<cplx> kf((size_t)F * F, cplx(0, 0));
        for (int a = -(G - 1); a < G; ++a)
            for (int b = -(G - 1); b < G; ++b)
                kf[(size_t)((a + F) % F) * F + ((b + F) % F)] =
                    kernel_tilde_value(g.coord_min, g.h, std::abs(a), std::abs(b));
        fft2d(kf, F, false);
        // Two real charge planes ride in one complex transform: the kernel is
        // real and even so its spectrum is real and the planes do not mix.
        for (int pair = 0; pair < 2; ++pair) {
            std::vector<cplx> a((size_t)F * F, cplx(0, 0));
            for (int m = 0; m < G; ++m)
                for (int n = 0; n < G; ++n) {
                    const float *wv = &w[((size_t)m * G + n) * T];
                    a[(size_t)m * F + n] = cplx(wv[2 * pair], wv[2 * pair + 1]);
                }
            fft2d(a, F, false);
            for (size_t t = 0; t < a.size(); ++t) a[t] *= kf[t].real();
            fft2d(a, F, true);
            const double scale = 1.0 / ((double)F * F);
            for (int m = 0; m < G; ++m)
                for (int n = 0; n < G; ++n) {
                    const cplx v = a[(size_t)m * F + n] * scale;
                    yt[((size_t)m * G + n) * T + 2 * pair] = (float)v.real();
                    yt[((size_t)m * G + n) * T + 2 * pair + 1] = (float)v.imag();
                }
        }
    }

    // Gather (nbodyfft.cu:141-173) and force assembly (rep_forces.cu:3-31).
    float zsum = 0.0f;
    std::vector<float> zvec(N);
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; ++i) {
        float phi[4] = {0, 0, 0, 0};
        for (int a = 0; a < p; ++a)
            for (int b = 0; b < p; ++b) {
                const size_t node = (size_t)(bx[i] * p + a) * G + (by[i] * p + b);
                const float lw = Lx[(size_t)i * p + a] * Ly[(size_t)i * p + b];
                for (int t = 0; t < T; ++t) phi[t] += lw * yt[node * T + t];
            }
        const float x = Y[i], y = Y[N + i];
        zvec[i] = (1 + x * x + y * y) * phi[0] - 2 * (x * phi[1] + y * phi[2]) + phi[3];
        rep[i] = x * phi[0] - phi[1];
        rep[N + i] = y * phi[0] - phi[2];
        if (phi_out)
            for (int t = 0; t < T; ++t) phi_out[(size_t)i * T + t] = phi[t];
    }
    // thrust::reduce is a tree reduction; pairwise summation in fp32 models it.
    {
        std::vector<float> buf(zvec);
        size_t n = buf.size();
        while (n > 1) {
            const size_t half = (n + 1) / 2;
            for (size_t t = 0; t + half < n; ++t) buf[t] += buf[t + half];
            n = half;
        }
        zsum = buf[0];
    }
    *Z_out = zsum - N;
    if (w_out) std::memcpy(w_out, w.data(), w.size() * sizeof(float));
    if (yt_out) std::memcpy(yt_out, yt.data(), yt.size() * sizeof(float));
}

// src/kernels/apply_forces.cu:11-57, all 2N coordinates.  attr and rep are
// zeroed as the reference does.
void oracle_update(float *Y, float *attr, float *rep, float *gains, float *old_forces, int N, float eta,
                   float normalization, float momentum, float exaggeration) {
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < (int64_t)2 * N; ++c) {
        float u = old_forces[c];
        float gn = gains[c];
        const float d = exaggeration * attr[c] - (rep[c] / normalization);
        gn = (std::signbit(d) != std::signbit(u)) ? (float)(gn + 0.2) : (float)(gn * 0.8);
        gn = (gn < 0.01) ? (float)0.01 : gn;
        u = momentum * u - eta * gn * d;
        Y[c] += u;
        attr[c] = 0.0f;
        rep[c] = 0.0f;
        old_forces[c] = u;
        gains[c] = gn;
    }
}

// Gradient loop of src/fit_tsne.cu:402-580 on a fixed (P, idx) and a given
// initial embedding (VECTOR init).  Y is updated in place.  Returns the last Z.
// gains and old_forces may be null (fresh state: gains 1, momentum buffer 0).
// recenter (not in the reference, whose loop never re-centres; the library's option): every step subtracts
// from the new positions the centre (mean x, mean y) the embedding had before the step.
float oracle_iterate(const float *P, const int *idx, float *Y, float *gains, float *old_forces, int N, int K,
                     int step_begin, int step_end, int force_magnify_iters, float eta, float pre_momentum,
                     float post_momentum, float early_exaggeration, int nb, int p, int recenter) {
    std::vector<float> attr((size_t)2 * N, 0.0f), rep((size_t)2 * N, 0.0f);
    std::vector<float> g_local, u_local;
    if (!gains) {
        g_local.assign((size_t)2 * N, 1.0f);
        gains = g_local.data();
    }
    if (!old_forces) {
        u_local.assign((size_t)2 * N, 0.0f);
        old_forces = u_local.data();
    }
    float Z = 0.0f;
    for (int step = step_begin; step < step_end; ++step) {
        const bool late = step >= force_magnify_iters;
        const float momentum = late ? post_momentum : pre_momentum;
        const float exag = late ? 1.0f : early_exaggeration;
        double cx = 0.0, cy = 0.0;
        if (recenter) {
            for (int i = 0; i < N; ++i) {
                cx += Y[i];
                cy += Y[N + i];
            }
        }
        oracle_repulsive(Y, N, nb, p, rep.data(), &Z, nullptr, nullptr, nullptr, 0);
        oracle_attractive(P, idx, Y, N, K, attr.data());
        oracle_update(Y, attr.data(), rep.data(), gains, old_forces, N, eta, Z, momentum, exag);
        if (recenter) {
            const float mx = (float)(cx / N), my = (float)(cy / N);
            for (int i = 0; i < N; ++i) {
                Y[i] = Y[i] - mx;
                Y[N + i] = Y[N + i] - my;
            }
        }
    }
    return Z;
}

// Whole fit: kNN -> max-norm -> perplexity -> symmetrise -> gradient loop
// (src/fit_tsne.cu:84-624) from an explicit initial embedding.
float oracle_fit(const float *X, int N, int D, int num_neighbors, float perplexity, float eps, float *Y,
                 int iterations, int force_magnify_iters, float eta, float pre_momentum, float post_momentum,
                 float early_exaggeration, int *idx_out, float *P_out) {
    const int K = std::min(num_neighbors, N);
    std::vector<int> idx((size_t)N * K);
    std::vector<float> d2((size_t)N * K), p((size_t)N * K), P((size_t)N * K);
    oracle_knn(X, N, D, K, idx.data(), d2.data());
    oracle_max_normalize(d2.data(), (int64_t)N * K);
    oracle_perplexity(d2.data(), N, K, perplexity, eps, p.data(), nullptr, nullptr);
    oracle_symmetrize(p.data(), idx.data(), N, K, P.data());
    if (idx_out) std::memcpy(idx_out, idx.data(), idx.size() * sizeof(int));
    if (P_out) std::memcpy(P_out, P.data(), P.size() * sizeof(float));
    return oracle_iterate(P.data(), idx.data(), Y, nullptr, nullptr, N, K, 0, iterations, force_magnify_iters, eta,
                          pre_momentum, post_momentum, early_exaggeration, 130, 3, 0);
}

// KL-style objective on the stored pattern:
//   sum_{P>0} P * (ln P + ln(1 + |y_i - y_j|^2) + ln Z)
// with Z = sum_{i != j} 1/(1 + |y_i - y_j|^2) evaluated exactly (O(N^2)) when
// Z_in <= 0, otherwise Z_in is used.
double oracle_kl(const float *P, const int *idx, const float *Y, int N, int K, double Z_in) {
    double Z = Z_in;
    if (Z <= 0) {
        double acc = 0;
#pragma omp parallel for reduction(+ : acc) schedule(dynamic, 64)
        for (int i = 0; i < N; ++i) {
            double a = 0;
            for (int j = 0; j < N; ++j) {
                if (j == i) continue;
                const double dx = (double)Y[i] - Y[j], dy = (double)Y[N + i] - Y[N + j];
                a += 1.0 / (1.0 + dx * dx + dy * dy);
            }
            acc += a;
        }
        Z = acc;
    }
    const double lz = std::log(Z);
    double kl = 0;
#pragma omp parallel for reduction(+ : kl) schedule(static)
    for (int i = 0; i < N; ++i) {
        double a = 0;
        for (int s = 0; s < K; ++s) {
            const size_t t = (size_t)i * K + s;
            const double pv = P[t];
            if (pv <= 0) continue;
            const int j = idx[t];
            const double dx = (double)Y[i] - Y[j], dy = (double)Y[N + i] - Y[N + j];
            a += pv * (std::log(pv) + std::log1p(dx * dx + dy * dy) + lz);
        }
        kl += a;
    }
    return kl;
}

}  // extern "C"
