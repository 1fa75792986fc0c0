"""A corpus in which some documents have no SPLADE pairs, some no BM25 pairs and some no sparse pairs at all
(the reference's loaders accept such rows: a CSR row of length zero, utils.cuh:361-398). The build kernels keep a
row's pairs in registers with the row's shape (pair counts) as the only description: a shape of zero pairs must
behave as a row that contributes nothing, not as a row that is not there."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match

pytestmark = pytest.mark.gpu

N = 2000


def _drop_rows(off, idx, val, keep):
    """CSR with the rows where keep is False emptied."""
    cnt = np.diff(off.astype(np.int64)) * keep
    new_off = np.zeros(len(off), np.uint32)
    new_off[1:] = np.cumsum(cnt)
    mask = np.repeat(keep, np.diff(off.astype(np.int64)))
    return new_off, idx[mask], val[mask]


@pytest.fixture(scope="module")
def holes_world(gpu_ctx):
    import apoe
    import apoe_synth as S
    import oracle as O
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(S.corpus(N, seed=71, device="cpu"))
    v = np.arange(N)
    keep_s = ~((v % 7 == 0) | (v % 11 == 0))   # no SPLADE pairs
    keep_b = ~((v % 5 == 0) | (v % 11 == 0))   # no BM25 pairs; multiples of 11 have no sparse pairs at all
    s_off, s_idx, s_val = _drop_rows(s_off, s_idx, s_val, keep_s)
    b_off, b_idx, b_val = _drop_rows(b_off, b_idx, b_val, keep_b)
    corpus = (dense, s_off, s_idx, s_val, b_off, b_idx, b_val)
    queries = S.to_numpy(S.queries(100, seed=72, device="cpu"))
    C, Q = O.HybridSet(*corpus), O.HybridSet(*queries)
    rows, entry, knn_ids, knn_dist = O.build_index(C, dense_scale=7.0, K=64, iters=6, d=32, seed=5, return_knn=True)
    gc = apoe.Corpus(gpu_ctx, *corpus)
    gq = apoe.Queries(gpu_ctx, *queries)
    return dict(ctx=gpu_ctx, C=C, Q=Q, gc=gc, gq=gq, rows=rows, entry=entry, knn_ids=knn_ids, knn_dist=knn_dist)


@pytest.mark.parametrize("join", [0, 1, 2])
def test_nn_descent_stores_the_metric(holes_world, join):
    import apoe
    import oracle as O
    w = holes_world
    knn = apoe.Knn(w["ctx"], w["gc"], 64, 7.0)
    knn.set_join(join)
    knn.init(9)
    for it in range(5):
        knn.iterate(last=(it == 4))
    knn.merge_reverse()
    ids, dist = knn.download()
    knn.close()
    assert np.all(np.diff(dist, axis=1) >= 0) and ids.max() < N
    rows_ = np.repeat(np.arange(N, dtype=np.uint32), 64)
    assert_dist_close(dist.ravel(), O.distance_pairs(w["C"], 7.0, rows_, ids.ravel()), "stored distance == recomputed distance")


def test_prune_matches_oracle_on_the_same_knn_graph(holes_world):
    import apoe
    import oracle as O
    w = holes_world
    knn = apoe.Knn(w["ctx"], w["gc"], 64, 7.0)
    knn.upload(w["knn_ids"], w["knn_dist"])
    knn.prune(32)
    g_fwd, g_det, g_cnt, g_kw = knn.prune_download()
    graph = knn.finalize()
    rows, entry = graph.download()
    graph.close()
    knn.close()
    c_fwd, c_det, c_cnt, c_kw = O.prune(w["C"], 7.0, O.norms(w["C"], 7.0), w["knn_ids"], w["knn_dist"], 32)
    same = np.all(g_fwd == c_fwd, axis=1)
    assert same.mean() >= 0.995, same.mean()
    assert np.array_equal(g_det[same], c_det[same]) and np.array_equal(g_cnt[same], c_cnt[same])
    assert np.all(g_kw == c_kw, axis=1)[same].mean() >= 0.995
    assert (rows == w["rows"]).all(axis=1).mean() >= 0.99
    # entry points: the documents of smallest hybrid norm. The documents without sparse pairs all have the norm of their
    # unit dense row times the build scale, equal up to rounding, so the choice among them is a tie: the norms must agree
    nrm = O.norms(w["C"], 7.0)
    assert len(set(entry.tolist())) == len(entry)
    assert nrm[entry].max() <= np.sort(nrm)[len(entry) - 1] * (1 + 1e-5)


def test_search_matches_oracle(holes_world):
    import apoe
    import oracle as O
    w = holes_world
    g = apoe.Graph(w["ctx"], w["rows"], w["entry"])
    for w3 in ((1.0, 1.0, 1.0), (0.0, 1.0, 1.0), (1.0, 0.0, 1.0)):
        ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], g, w3, 64)
        oid, odist, _ = O.search(w["C"], w["Q"], w["rows"], w["entry"], w3, 64)
        assert assert_topk_match(ids, dist, oid, odist, 10, f"rows without pairs, weights {w3}") > 0.97
        same = ids == oid
        assert_dist_close(dist[same], odist[same], "pool distances")
    g.close()


def test_queries_without_pairs_match_oracle(holes_world):
    """Queries that have no SPLADE pairs, no BM25 pairs or no sparse pairs at all (a dense-only query in a hybrid batch):
    their LDS term tables are empty, every probe misses."""
    import apoe
    import apoe_synth as S
    import oracle as O
    w = holes_world
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(S.queries(120, seed=73, device="cpu"))
    q = np.arange(120)
    s_off, s_idx, s_val = _drop_rows(s_off, s_idx, s_val, ~((q % 3 == 0) | (q % 12 == 0)))
    b_off, b_idx, b_val = _drop_rows(b_off, b_idx, b_val, ~((q % 4 == 0) | (q % 12 == 0)))
    queries = (dense, s_off, s_idx, s_val, b_off, b_idx, b_val)
    Q = O.HybridSet(*queries)
    gq = apoe.Queries(w["ctx"], *queries)
    g = apoe.Graph(w["ctx"], w["rows"], w["entry"])
    for w3 in ((1.0, 1.0, 1.0), (0.0, 1.0, 1.0), (1.0, 0.5, 2.0)):
        ids, dist, _ = apoe.search(w["ctx"], w["gc"], gq, g, w3, 64)
        oid, odist, _ = O.search(w["C"], Q, w["rows"], w["entry"], w3, 64)
        assert assert_topk_match(ids, dist, oid, odist, 10, f"queries without pairs, weights {w3}") > 0.97
        same = ids == oid
        assert_dist_close(dist[same], odist[same], "pool distances")
    g.close()
    gq.close()
