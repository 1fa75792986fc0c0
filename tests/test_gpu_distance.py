"""HIP fused hybrid distance / norms against the CPU oracle (through the C-ABI)."""
import numpy as np
import pytest

from parity import assert_dist_close

pytestmark = pytest.mark.gpu

WEIGHTS = [(1, 1, 1), (1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 0.5, 2), (0, 1, 1), (1, 0, 1), (1, 1, 0), (3.5, 0.25, 1e-6)]


@pytest.mark.parametrize("w3", WEIGHTS)
def test_distance_batch_matches_oracle(gpu_world, w3):
    import apoe
    import oracle as O
    w = gpu_world
    rng = np.random.default_rng(3)
    ids = rng.integers(0, w["C"].n, size=(w["Q"].n, 96), dtype=np.uint32)
    ids[:, 0] = np.arange(w["Q"].n) % w["C"].n
    got = apoe.distance_batch(w["ctx"], w["gc"], w["gq"], w3, ids)
    want = O.distance_batch(w["C"], w["Q"], w3, ids)
    assert_dist_close(got, want, f"weights {w3}")


def test_distance_batch_out_of_range_id(gpu_world):
    import apoe
    w = gpu_world
    ids = np.full((w["Q"].n, 3), w["C"].n + 5, np.uint32)
    ids[:, 1] = 0
    got = apoe.distance_batch(w["ctx"], w["gc"], w["gq"], (1, 1, 1), ids)
    assert np.all(got[:, 0] == apoe.INF_DIS) and np.all(got[:, 2] == apoe.INF_DIS) and np.all(got[:, 1] < apoe.INF_DIS)


def test_distance_pairs_matches_oracle(gpu_world):
    import apoe
    import oracle as O
    w = gpu_world
    rng = np.random.default_rng(4)
    a = rng.integers(0, w["C"].n, size=3000, dtype=np.uint32)
    b = rng.integers(0, w["C"].n, size=3000, dtype=np.uint32)
    b[:50] = a[:50]  # identical vectors: dist = 1 - norm
    for scale in (7.0, 1.0):
        got = apoe.distance_pairs(w["ctx"], w["gc"], scale, a, b)
        want = O.distance_pairs(w["C"], scale, a, b)
        assert_dist_close(got, want, f"scale {scale}")
        nrm = apoe.norms(w["ctx"], w["gc"], scale)
        assert_dist_close(1.0 - nrm[a[:50]], got[:50], "self distance = 1 - norm")
        # symmetry of the metric
        assert_dist_close(apoe.distance_pairs(w["ctx"], w["gc"], scale, b, a), got, "symmetry")


def test_norms_match_oracle(gpu_world):
    import apoe
    import oracle as O
    w = gpu_world
    for scale in (7.0, 1.0):
        assert_dist_close(apoe.norms(w["ctx"], w["gc"], scale), O.norms(w["C"], scale), f"norms scale {scale}")


def test_corpus_info(gpu_world):
    w = gpu_world
    info = w["gc"].info()
    assert info[0] == w["C"].n and info[1] == 1024
    assert info[2] == int(np.diff(w["C"].s_off).max()) and info[3] == int(np.diff(w["C"].b_off).max())


def test_ragged_rows(gpu_ctx):
    """Empty sparse rows, a single shared term, disjoint term sets, long rows."""
    import apoe
    import oracle as O
    rng = np.random.default_rng(9)
    n = 12
    dense = rng.standard_normal((n, 1024)).astype(np.float32)
    s_rows = [[], [5], [5, 9], list(range(0, 900, 3)), [7], [], [1, 2, 3], [30000], [5], list(range(1, 700)), [2], [9]]
    b_rows = [[5], [], [5], [5, 6, 7], list(range(100, 500)), [], [33000], [5], [], [4, 5], [5], list(range(2, 900, 2))]

    def csr(rows_):
        off = np.zeros(len(rows_) + 1, np.uint32)
        off[1:] = np.cumsum([len(r) for r in rows_])
        idx = np.array([t for r in rows_ for t in r], np.uint32)
        val = rng.uniform(0.5, 2.0, len(idx)).astype(np.float32)
        return off, idx, val

    arrays = (dense,) + csr(s_rows) + csr(b_rows)
    C = O.HybridSet(*arrays)
    gc = apoe.Corpus(gpu_ctx, *arrays)
    gq = apoe.Queries(gpu_ctx, *arrays)
    ids = np.tile(np.arange(n, dtype=np.uint32), (n, 1))
    for w3 in [(1, 1, 1), (0, 1, 0), (0, 0, 1), (0, 1, 1)]:
        assert_dist_close(apoe.distance_batch(gpu_ctx, gc, gq, w3, ids), O.distance_batch(C, C, w3, ids), f"ragged {w3}")
    a, b = np.meshgrid(np.arange(n, dtype=np.uint32), np.arange(n, dtype=np.uint32))
    assert_dist_close(apoe.distance_pairs(gpu_ctx, gc, 7.0, a.ravel(), b.ravel()), O.distance_pairs(C, 7.0, a.ravel(), b.ravel()), "ragged pairs")
    assert_dist_close(apoe.norms(gpu_ctx, gc, 7.0), O.norms(C, 7.0), "ragged norms")
