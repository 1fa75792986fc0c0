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


@pytest.mark.parametrize("top_id", [65535, 65536])
def test_pair_format_boundary(gpu_ctx, top_id):
    """Term id 65535 is the last one a narrow record holds; one id of 65536 anywhere in the corpus turns every
    record wide. Query terms beyond 65535 never match a narrow corpus. Distances, norms and a search on a ring
    graph agree with the oracle on both sides of the boundary, and rows that do not hold the top id do not change."""
    import apoe
    import oracle as O
    rng = np.random.default_rng(31)
    n, d = 40, 4
    dense = (rng.standard_normal((n, 1024)) / 32).astype(np.float32)

    def csr(rows_):
        off = np.zeros(len(rows_) + 1, np.uint32)
        off[1:] = np.cumsum([len(r) for r in rows_])
        idx = np.array([t for r in rows_ for t in r], np.uint32)
        val = rng.uniform(0.5, 2.0, len(idx)).astype(np.float32)
        return off, idx, val

    s_rows = [sorted(set(rng.integers(0, 65000, 30).tolist())) for _ in range(n)]
    b_rows = [sorted(set(rng.integers(0, 65000, 12).tolist())) for _ in range(n)]
    s_rows[3].append(top_id)   # SPLADE side
    b_rows[5].append(top_id)   # BM25 side
    b_rows[6].append(65535)
    corpus = (dense,) + csr(s_rows) + csr(b_rows)
    # queries: copies of some docs plus terms beyond 16 bits that no narrow record can hold
    q_s = [s_rows[3] + [70000, 131071 + 65536], s_rows[8], [65535, 65536], []]
    q_b = [b_rows[5] + [65536 + 5], b_rows[6], [65535, 65536, 70000], [top_id]]
    queries = (dense[:4].copy(),) + csr(q_s) + csr(q_b)
    C, Q = O.HybridSet(*corpus), O.HybridSet(*queries)
    gc, gq = apoe.Corpus(gpu_ctx, *corpus), apoe.Queries(gpu_ctx, *queries)
    assert gc.pair_bytes() == (6 if top_id == 65535 else 8)
    ids = np.tile(np.arange(n, dtype=np.uint32), (4, 1))
    for w3 in [(1, 1, 1), (0, 1, 0), (0, 0, 1), (1, 0, 2)]:
        assert_dist_close(apoe.distance_batch(gpu_ctx, gc, gq, w3, ids), O.distance_batch(C, Q, w3, ids), f"boundary {top_id} {w3}")
    a, b = np.meshgrid(np.arange(n, dtype=np.uint32), np.arange(n, dtype=np.uint32))
    assert_dist_close(apoe.distance_pairs(gpu_ctx, gc, 7.0, a.ravel(), b.ravel()), O.distance_pairs(C, 7.0, a.ravel(), b.ravel()), "boundary pairs")
    assert_dist_close(apoe.norms(gpu_ctx, gc, 7.0), O.norms(C, 7.0), "boundary norms")
    rows = np.zeros((n, d + 8), np.uint32)
    for v in range(n):
        rows[v, :d] = [(v + 1) % n, (v - 1) % n, (v + 7) % n, (v + 13) % n]
    entry = np.array([0, 20], np.uint32)
    gg = apoe.Graph(gpu_ctx, rows, entry)
    for w3 in [(1, 1, 1), (0, 1, 1)]:
        got, gd, _ = apoe.search(gpu_ctx, gc, gq, gg, w3, 16)
        want, wd, _ = O.search(C, Q, rows, entry, w3, 16)
        assert np.array_equal(got, want)
        assert_dist_close(gd, wd, f"boundary search {top_id} {w3}")
    gg.close()
    gq.close()
    gc.close()


def test_term_id_with_bit_31_is_rejected(gpu_ctx):
    """Bit 31 of a stored term id is the path bit of the device records: a corpus that uses it is refused."""
    import apoe
    dense = np.zeros((2, 1024), np.float32)
    off = np.array([0, 1, 2], np.uint32)
    val = np.ones(2, np.float32)
    ok_idx = np.array([5, 0x7FFFFFFE], np.uint32)
    c = apoe.Corpus(gpu_ctx, dense, off, ok_idx, val, off, ok_idx, val)
    assert c.pair_bytes() == 8
    c.close()
    with pytest.raises(apoe.ApoeError, match="31 bits"):
        apoe.Corpus(gpu_ctx, dense, off, np.array([5, 0x80000001], np.uint32), val, off, ok_idx, val)


def test_query_sparse_term_with_bit_31_is_rejected(gpu_ctx):
    """Bit 31 marks a required keyword on a BM25 query term; a SPLADE query term must not carry it."""
    import apoe
    dense = np.zeros((1, 1024), np.float32)
    off = np.array([0, 1], np.uint32)
    val = np.ones(1, np.float32)
    q = apoe.Queries(gpu_ctx, dense, off, np.array([7], np.uint32), val, off, np.array([0x80000007], np.uint32), val)
    q.close()
    with pytest.raises(apoe.ApoeError, match="31 bits"):
        apoe.Queries(gpu_ctx, dense, off, np.array([0x80000007], np.uint32), val, off, np.array([7], np.uint32), val)
