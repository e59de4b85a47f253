"""The error bound of the kNN sweep on bf16 terms, checked on the CPU.

The sweep (tsne-cuda_amd/csrc/knn.hip, knn_mfma_sweep_kernel<STEPS, true>) stores
every candidate relative to the centre m of its 128-point tile, splits each
coordinate into two bf16 terms, accumulates high x high, high x low, low x high
and keeps as a candidate's key
    product + |q - m|^2 (1 - (D + 4) 2^-24) - (|q| ga + gb)
with the per-tile coefficients of pack_tile_centres_kernel.  The re-rank's proof
that nothing outside the candidate list belongs to the answer needs that key to
be a LOWER bound of the true squared distance.  This file restates the arithmetic
in numpy (the split and the dropped low x low term exactly; the accumulation in
fp32 in a random order, which the bound's factor of four has to cover with room
to spare) and checks the inequality on clustered, far-from-origin, tiny and mixed
scale data; it also checks that the bound is not vacuous (a small fraction of
the neighbour distances on benchmark-like data), which is what makes the sweep
verify at all.
"""
import numpy as np
import pytest

EPS = 2.0 ** -24


def bf16(x):
    """Nearest bf16 (ties to even) of float32 values, as float32."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


def split(x):
    hi = bf16(x)
    lo = bf16((np.asarray(x, np.float32) - hi).astype(np.float32))
    return hi, lo


def fp32_sum_random_order(terms, rng):
    """Sum of float64 terms accumulated in float32 in a random order (one row per result)."""
    acc = np.zeros(terms.shape[0], np.float32)
    for j in rng.permutation(terms.shape[1]):
        acc = (acc + terms[:, j].astype(np.float32)).astype(np.float32)
    return acc


def keys_for_tile(Q, C, rng, from_terms=False):
    """Keys the sweep would store for queries Q against one candidate tile C (both float32, rows = points).
    from_terms: the chunked sweep's way (more than 126 dimensions): |q - m|^2 from the query's two bf16
    terms, -(high + low) / 2 for q, with 2.1 * 2^-16 |q| |q - m| taken off the key for what they miss."""
    D = C.shape[1]
    m = (C.sum(0, dtype=np.float32) / np.float32(len(C))).astype(np.float32)      # tile_balls_kernel's centre
    delta = (C - m).astype(np.float32)
    r = np.float32(np.sqrt((delta.astype(np.float64) ** 2).sum(1).max()) * (1 + 1e-3) + 1e-30)
    mlen = np.float32(np.sqrt((m.astype(np.float64) ** 2).sum()) * (1 + 1e-6))
    c_split, c_acc = np.float32(6.2 / 65536.0), np.float32(4.0 * (3 * D + 6) * EPS)
    ga = np.float32(1.01) * (c_split + np.float32(2) * c_acc) * r
    gb = np.float32(1.01) * c_acc * (r * r + np.float32(2) * mlen * r) + np.float32(1e-30)
    # beta = |delta|^2 + 2 m.delta as the pack kernel forms it (fp32 fma chains), in three bf16 terms
    sq = np.zeros(len(C), np.float32)
    dot = np.zeros(len(C), np.float32)
    for d in range(D):
        sq = (delta[:, d].astype(np.float64) * delta[:, d] + sq).astype(np.float32)
        dot = (np.float64(m[d]) * delta[:, d] + dot).astype(np.float32)
    beta = (2.0 * dot.astype(np.float64) + sq).astype(np.float32)
    b0 = bf16(beta)
    b1 = bf16((beta - b0).astype(np.float32))
    b2 = bf16((beta - b0 - b1).astype(np.float32))
    dh, dl = split(delta)
    keys = np.empty((len(Q), len(C)), np.float32)
    for i, q in enumerate(Q):
        wh, wl = split((-2.0 * q).astype(np.float32))
        terms = np.concatenate([dh.astype(np.float64) * wh, dl.astype(np.float64) * wh, dh.astype(np.float64) * wl,
                                b0[:, None].astype(np.float64), b1[:, None].astype(np.float64),
                                b2[:, None].astype(np.float64)], axis=1)
        product = fp32_sum_random_order(terms, rng)
        f = np.float32(0)
        q_used = (np.float32(-0.5) * (wh + wl).astype(np.float32)).astype(np.float32) if from_terms else q
        for d in range(D):
            diff = np.float32(q_used[d] - m[d])
            f = np.float32(np.float64(diff) * diff + f)
        q_len = np.float32(np.sqrt(np.float32((q.astype(np.float64) ** 2).sum())) * (1 + 1e-6))
        off = np.float32(f * np.float32(1.0 - (D + 4) * EPS)) - np.float32(q_len * ga + gb)
        if from_terms:
            off = np.float32(off - np.float32(2.1 / 65536.0) * q_len * np.float32(np.sqrt(f)))
        keys[i] = (product + np.float32(off)).astype(np.float32)
    return keys, float(ga), float(gb)


def true_sq_dist(Q, C):
    return ((Q[:, None, :].astype(np.float64) - C[None, :, :].astype(np.float64)) ** 2).sum(2)


@pytest.mark.parametrize("name,d,center,sigma", [
    ("benchmark-like", 50, 10.0, 1.0),      # |x| ~ 70, tile radius ~ 10
    ("far from the origin", 16, 300.0, 1e-2),
    ("tiny", 8, 1e-3, 1e-4),
    ("large", 30, 2e3, 50.0),
    ("few dimensions", 3, 5.0, 2.0),
    ("many dimensions", 125, 4.0, 1.0),
])
def test_keys_are_lower_bounds(name, d, center, sigma):
    rng = np.random.default_rng(len(name) * 7 + d)
    mu = rng.standard_normal(d) * center
    C = (mu + rng.standard_normal((128, d)) * sigma).astype(np.float32)
    Q = np.concatenate([(mu + rng.standard_normal((6, d)) * sigma),              # queries of the same cluster
                        (rng.standard_normal((3, d)) * center),                   # of another one
                        C[:3]]).astype(np.float32)                                # and candidates themselves
    keys, ga, gb = keys_for_tile(Q, C, rng)
    exact = true_sq_dist(Q, C)
    assert (keys.astype(np.float64) <= exact).all(), name
    # what the bound gives away stays of the order of |q| ga + gb
    q_len = np.sqrt((Q.astype(np.float64) ** 2).sum(1))[:, None]
    assert (exact - keys <= 2.5 * (q_len * ga + gb) + 1e-3 * exact + 1e-30).all(), name


@pytest.mark.parametrize("d,center,sigma", [(200, 3.0, 1.0), (784, 3.0, 1.0), (130, 200.0, 0.05)])
def test_keys_are_lower_bounds_with_the_query_from_its_terms(d, center, sigma):
    rng = np.random.default_rng(d)
    mu = rng.standard_normal(d) * center
    C = (mu + rng.standard_normal((128, d)) * sigma).astype(np.float32)
    Q = np.concatenate([(mu + rng.standard_normal((4, d)) * sigma), (rng.standard_normal((2, d)) * center),
                        C[:2]]).astype(np.float32)
    keys, ga, gb = keys_for_tile(Q, C, rng, from_terms=True)
    exact = true_sq_dist(Q, C)
    assert (keys.astype(np.float64) <= exact).all()
    q_len = np.sqrt((Q.astype(np.float64) ** 2).sum(1))[:, None]
    assert (exact - keys <= 2.5 * (q_len * ga + gb) + 2e-3 * exact + 1e-30).all()


def test_mixed_scale_tile():
    """A tile that straddles two clusters (large radius): the bound grows with the radius and still holds."""
    rng = np.random.default_rng(5)
    d = 50
    a, b = rng.standard_normal(d) * 10.0, rng.standard_normal(d) * 10.0
    C = np.concatenate([a + rng.standard_normal((64, d)), b + rng.standard_normal((64, d))]).astype(np.float32)
    Q = np.concatenate([a + rng.standard_normal((4, d)), b + rng.standard_normal((4, d))]).astype(np.float32)
    keys, ga, gb = keys_for_tile(Q, C, rng)
    assert (keys.astype(np.float64) <= true_sq_dist(Q, C)).all()


def test_bound_is_small_on_benchmark_like_data():
    """50-dimensional unit clusters 70 from the origin: the keys are within half a percent of the neighbour
    distances (about 100), far inside the gap between the 89th and the 133rd neighbour that the sweep's
    verification lives on; the same split on the raw coordinates would give away about 1.5."""
    rng = np.random.default_rng(9)
    d = 50
    mu = rng.standard_normal(d) * 10.0
    C = (mu + rng.standard_normal((128, d))).astype(np.float32)
    Q = (mu + rng.standard_normal((8, d))).astype(np.float32)
    keys, ga, gb = keys_for_tile(Q, C, rng)
    exact = true_sq_dist(Q, C)
    slack = exact - keys
    assert slack.max() < 0.5 and slack.max() < 0.005 * np.median(exact)
