"""Shared parity checks between the HIP path and the CPU oracle."""
import numpy as np

DIST_RTOL = 1e-4  # north-star bound: hybrid distances within 1e-4 relative


def assert_dist_close(got, want, what=""):
    """|got - want| <= 1e-4 * max(1, |want|): relative to the size of the inner product,
    absolute near zero (a distance is 1 - IP, so IP close to 1 makes it cancel)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want) / np.maximum(1.0, np.abs(want))
    assert err.max() <= DIST_RTOL, f"{what}: max rel err {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}"


def assert_topk_match(ids_a, dist_a, ids_b, dist_b, k, what=""):
    """Rows of top-k ids agree as sets, except where the ids that differ sit at a
    distance tie (within DIST_RTOL) with the k-th distance of the other side."""
    nq = ids_a.shape[0]
    exact = 0
    for q in range(nq):
        a, b = ids_a[q, :k], ids_b[q, :k]
        if np.array_equal(a, b):
            exact += 1
            continue
        sa, sb = set(a.tolist()), set(b.tolist())
        for x in sa - sb:
            da = float(dist_a[q, list(a).index(x)])
            kth = float(dist_b[q, k - 1])
            assert abs(da - kth) <= DIST_RTOL * max(1.0, abs(kth)), f"{what}: query {q} id {x} at {da} vs kth {kth}"
        for x in sb - sa:
            db = float(dist_b[q, list(b).index(x)])
            kth = float(dist_a[q, k - 1])
            assert abs(db - kth) <= DIST_RTOL * max(1.0, abs(kth)), f"{what}: query {q} id {x} at {db} vs kth {kth}"
        # same set in a different order is allowed only between near-tied distances
        if sa == sb:
            for i in range(k):
                if a[i] != b[i]:
                    j = list(b).index(a[i])
                    assert abs(float(dist_b[q, j]) - float(dist_b[q, i])) <= DIST_RTOL * max(1.0, abs(float(dist_b[q, i]))), \
                        f"{what}: query {q} order differs beyond a tie"
    return exact / max(nq, 1)


def recall_at_k(found, truth, k):
    hit = 0
    for f, t in zip(found, truth):
        hit += len(set(f[:k].tolist()) & set(t[:k].tolist()))
    return hit / (len(truth) * k)
