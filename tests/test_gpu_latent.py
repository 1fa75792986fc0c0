"""A corpus whose rows have neighbours (apoe_synth.latent_corpus), 100 000 docs: searched under the metric the graph is
built for, the path reaches recall@10 >= 0.95 with a pool of 128, the oracle walks the GPU-built graph to the same top-10,
and the bound on the dense part changes no result although most evaluations now read their dense row."""
import numpy as np
import pytest

from parity import assert_topk_match, recall_at_k

pytestmark = pytest.mark.gpu

N_DOCS, N_QUERIES, DEGREE = 100_000, 2_000, 32
W_BUILD = (49.0, 1.0, 1.0)  # index.cu:836-840: dense x 7 on both sides of a pair


@pytest.fixture(scope="module")
def world(gpu_ctx):
    import torch
    import apoe
    import apoe_synth as S
    corpus = S.latent_corpus(N_DOCS, seed=501, world=503, device="cuda:0")
    queries = S.latent_queries(N_QUERIES, seed=502, world=503, device="cuda:0")
    torch.cuda.synchronize()
    gc, gq = apoe.Corpus(gpu_ctx, *corpus), apoe.Queries(gpu_ctx, *queries)
    yield dict(ctx=gpu_ctx, corpus=corpus, queries=queries, gc=gc, gq=gq)
    gq.close()
    gc.close()


@pytest.mark.parametrize("join", [0, 1])
def test_recall_target_is_reached_where_rows_have_neighbours(world, join):
    import apoe
    import apoe_bruteforce as B
    import apoe_synth as S
    import oracle as O
    w = world
    graph, _ = apoe.build_graph(w["ctx"], w["gc"], K=64, iters=10, degree=DEGREE, seed=3, join=join)
    nq = 500
    truth, _ = B.hybrid_topk(w["corpus"], w["queries"], W_BUILD, 10, nq=nq)
    rec = {}
    for cands in (32, 128):
        ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], graph, W_BUILD, cands, q_count=nq)
        rec[cands] = recall_at_k(ids, truth, 10)
    print(f"latent corpus, join={join}: recall@10 {rec}")
    assert rec[128] >= 0.95 and rec[32] < rec[128]
    # the bound never changes a result
    ids2, dist2, st2 = apoe.search(w["ctx"], w["gc"], w["gq"], graph, W_BUILD, 128, q_count=nq, variant=0x100)
    assert np.array_equal(ids, ids2) and np.array_equal(dist, dist2) and st.dense_rows <= st2.dense_rows == st2.evaluations
    # the oracle on the same graph
    rows, entry = graph.download()
    C = O.HybridSet(*S.to_numpy(w["corpus"]))
    Q = O.HybridSet(*S.to_numpy(w["queries"])).head(100)
    oid, odist, _ = O.search(C, Q, rows, entry, W_BUILD, 128)
    assert assert_topk_match(ids[:100], dist[:100], oid, odist, 10, "latent corpus, GPU-built graph") > 0.97
    # under the user weights 1/1/1 the terms decide, and they carry no structure: the graph helps little
    truth1, _ = B.hybrid_topk(w["corpus"], w["queries"], (1.0, 1.0, 1.0), 10, nq=nq)
    ids1, _, _ = apoe.search(w["ctx"], w["gc"], w["gq"], graph, (1.0, 1.0, 1.0), 128, q_count=nq)
    assert recall_at_k(ids1, truth1, 10) < rec[128]
    graph.close()


def test_kg_and_keyword_search_match_the_oracle_where_every_evaluation_reads_its_dense_row(world):
    """Knowledge-graph and keyword-filter search on this corpus (the bound on the dense part rejects nothing here, so
    every candidate goes through the second stage) against the oracle on the GPU-built graph."""
    import apoe
    import apoe_synth as S
    import oracle as O
    w = world
    nq = 100
    graph, _ = apoe.build_graph(w["ctx"], w["gc"], K=64, iters=10, degree=DEGREE, seed=4, join=1)
    rows, entry = graph.download()
    corpus_np, queries_np = S.to_numpy(w["corpus"]), S.to_numpy(w["queries"])
    C, Q = O.HybridSet(*corpus_np), O.HybridSet(*queries_np).head(nq)
    kg = S.to_numpy(S.knowledge_graph(20000, N_DOCS, N_QUERIES, seed=22, device="cpu"))
    gkg = apoe.KnowledgeGraph(w["ctx"], *kg)
    okg = O.Kg(kg[0], kg[1], kg[2], kg[3], kg[4][:nq + 1], kg[5][:kg[4][nq]])
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], graph, W_BUILD, 128, kg=gkg, kg_weight=40.0, q_count=nq)
    oid, odist, _ = O.search(C, Q, rows, entry, W_BUILD, 128, kg=okg, kg_weight=40.0)
    assert assert_topk_match(ids, dist, oid, odist, 10, "latent corpus, knowledge graph") > 0.97
    assert st.dense_rows > 0.9 * st.evaluations
    gkg.close()
    # keyword filter: the rarest BM25 term of each query is required
    b_off, b_idx = queries_np[4], queries_np[5].copy()
    df = np.bincount(corpus_np[5], minlength=int(max(corpus_np[5].max(), b_idx.max())) + 1)
    for q in range(nq):
        t = b_idx[b_off[q]:b_off[q + 1]]
        ok = np.where(df[t] > 0)[0] if len(t) else []
        if len(ok):
            b_idx[b_off[q] + ok[np.argmin(df[t][ok])]] |= 0x80000000
    qk = queries_np[:5] + (b_idx,) + queries_np[6:]
    gqk = apoe.Queries(w["ctx"], *qk)
    kid, kdist, _ = apoe.search(w["ctx"], w["gc"], gqk, graph, W_BUILD, 128, keyword_filter=True, q_count=nq)
    okid, okdist, _ = O.search(C, O.HybridSet(*qk).head(nq), rows, entry, W_BUILD, 128, keyword_filter=True)
    assert (kid == okid).all(axis=1).mean() > 0.97
    assert (okid != 0x7FFFFFFF).any()
    gqk.close()
    graph.close()


def test_k128_degree64_and_the_wide_pair_format_on_this_corpus(world):
    """Lists of 128 pruned to degree 64 (the gather-once prune by tiles, the join with two tiles per row block) and the
    8-byte pair format, where every evaluation reads its dense row: recall, the oracle on the same graph, and the same
    rows from narrow and wide records."""
    import torch
    import apoe
    import apoe_bruteforce as B
    import apoe_synth as S
    import oracle as O
    w = world
    nq = 300
    graph, _ = apoe.build_graph(w["ctx"], w["gc"], K=128, iters=10, degree=64, seed=5, join=1)
    truth, _ = B.hybrid_topk(w["corpus"], w["queries"], W_BUILD, 10, nq=nq)
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], graph, W_BUILD, 64, q_count=nq)
    assert recall_at_k(ids, truth, 10) >= 0.97
    rows, entry = graph.download()
    assert rows.shape == (N_DOCS, 64 + 8)
    C = O.HybridSet(*S.to_numpy(w["corpus"]))
    Q = O.HybridSet(*S.to_numpy(w["queries"])).head(100)
    oid, odist, _ = O.search(C, Q, rows, entry, W_BUILD, 64)
    assert assert_topk_match(ids[:100], dist[:100], oid, odist, 10, "latent corpus, K = 128 / degree 64") > 0.97
    shift = 70000
    corpus_w = tuple(w["corpus"][:5]) + (w["corpus"][5] + shift,) + tuple(w["corpus"][6:])
    queries_w = tuple(w["queries"][:5]) + (w["queries"][5] + shift,) + tuple(w["queries"][6:])
    torch.cuda.synchronize()
    gc2, gq2 = apoe.Corpus(w["ctx"], *corpus_w), apoe.Queries(w["ctx"], *queries_w)
    assert w["gc"].pair_bytes() == 6 and gc2.pair_bytes() == 8
    ids2, dist2, _ = apoe.search(w["ctx"], gc2, gq2, graph, W_BUILD, 64, q_count=nq)
    assert np.array_equal(ids, ids2)
    assert np.allclose(dist, dist2, rtol=1e-5, atol=1e-5)
    gq2.close()
    gc2.close()
    graph.close()
