"""The plumbing configuration at its stated size: 10 000 docs, 1 000 queries, degree 32, cands 128, top-10, weights
1/1/1 (K = 64, 10 NN-Descent steps). Small enough for the oracle on every query and every node: the prune and the
final rows on the oracle's own K-NN lists, every query's top-10 on the oracle-built and on the GPU-built graph, and
recall@10 of the GPU builds (three seeds, expansion step and local join) against the oracle builds."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match, recall_at_k

pytestmark = pytest.mark.gpu

N_DOCS, N_QUERIES, DEGREE, CANDS, STEPS = 10_000, 1_000, 32, 128, 10
W3 = (1.0, 1.0, 1.0)
SEEDS = (5, 6, 7)


@pytest.fixture(scope="module")
def world(gpu_ctx):
    import apoe
    import apoe_synth as S
    import oracle as O
    corpus = S.to_numpy(S.corpus(N_DOCS, seed=301, device="cpu"))
    queries = S.to_numpy(S.queries(N_QUERIES, seed=302, device="cpu"))
    C, Q = O.HybridSet(*corpus), O.HybridSet(*queries)
    truth, _ = O.bruteforce_topk(C, Q, W3, 10)
    builds = [O.build_index(C, dense_scale=7.0, K=64, iters=STEPS, d=DEGREE, seed=s, return_knn=True) for s in SEEDS]
    gc, gq = apoe.Corpus(gpu_ctx, *corpus), apoe.Queries(gpu_ctx, *queries)
    yield dict(ctx=gpu_ctx, C=C, Q=Q, gc=gc, gq=gq, truth=truth, builds=builds)
    gq.close()
    gc.close()


def test_every_query_on_the_oracle_built_graph(world):
    import apoe
    import oracle as O
    w = world
    rows, entry = w["builds"][0][:2]
    gg = apoe.Graph(w["ctx"], rows, entry)
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], gg, W3, CANDS)
    oid, odist, cnt = O.search(w["C"], w["Q"], rows, entry, W3, CANDS)
    assert ids.shape == (N_QUERIES, CANDS)
    assert assert_topk_match(ids, dist, oid, odist, 10, "config 0, oracle-built graph") > 0.98
    same = ids == oid
    assert same.mean() > 0.97
    assert_dist_close(dist[same], odist[same], "pool distances")
    assert abs(int(st.evaluations) - int(cnt[:, 1].sum())) <= 0.01 * cnt[:, 1].sum()
    assert int(st.expansions) == int(cnt[:, 0].sum())
    gg.close()


def test_prune_and_final_rows_on_the_oracle_lists(world):
    import apoe
    import oracle as O
    w = world
    rows, entry, knn_ids, knn_dist = w["builds"][0]
    knn = apoe.Knn(w["ctx"], w["gc"], 64, 7.0)
    knn.upload(knn_ids, knn_dist)
    knn.prune(DEGREE)
    g = knn.prune_download()
    c = O.prune(w["C"], 7.0, O.norms(w["C"], 7.0), knn_ids, knn_dist, DEGREE)
    same = np.all(g[0] == c[0], axis=1)
    assert same.mean() >= 0.995
    assert np.array_equal(g[1][same], c[1][same]) and np.array_equal(g[2][same], c[2][same])
    assert np.all(g[3] == c[3], axis=1)[same].mean() >= 0.995
    graph = knn.finalize()
    g_rows, g_entry = graph.download()
    assert np.array_equal(g_rows, O.final_graph(*g))
    assert np.array_equal(g_entry, entry)
    assert (np.all(g_rows == rows, axis=1)).mean() >= 0.99  # the whole rows, reverse halves included
    graph.close()
    knn.close()


@pytest.mark.parametrize("join", [0, 1])
def test_gpu_build_and_every_query_on_it(world, join):
    import apoe
    import oracle as O
    w = world
    graphs = [apoe.build_graph(w["ctx"], w["gc"], K=64, iters=STEPS, degree=DEGREE, dense_scale=7.0, seed=s, join=join)[0] for s in SEEDS]
    r_gpu = []
    for g in graphs:
        ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], g, W3, CANDS)
        r_gpu.append(recall_at_k(ids, w["truth"], 10))
    r_orc = []
    for rows, entry, _, _ in w["builds"]:
        gg = apoe.Graph(w["ctx"], rows, entry)
        ids, _, _ = apoe.search(w["ctx"], w["gc"], w["gq"], gg, W3, CANDS)
        r_orc.append(recall_at_k(ids, w["truth"], 10))
        gg.close()
    print(f"config 0, join={join}: recall@10 at cands {CANDS}: gpu-built {np.round(r_gpu, 4)}, oracle-built {np.round(r_orc, 4)}")
    assert np.mean(r_gpu) >= np.mean(r_orc) - 0.005
    # the oracle walks the GPU-built graph: the same top-10 for every query
    rows, entry = graphs[0].download()
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], graphs[0], W3, CANDS)
    oid, odist, _ = O.search(w["C"], w["Q"], rows, entry, W3, CANDS)
    assert assert_topk_match(ids, dist, oid, odist, 10, "config 0, GPU-built graph") > 0.98
    assert np.array_equal(entry, w["builds"][0][1])
    for g in graphs:
        g.close()
