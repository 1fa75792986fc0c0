"""The whole path at 100 000 docs and 10 000 queries (degree 32, K = 64, 10 NN-Descent steps, cands 128): the oracle
checks a sample, the whole batch is checked through properties that do not depend on the size."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match, recall_at_k

pytestmark = pytest.mark.gpu

N_DOCS, N_QUERIES, DEGREE, CANDS = 100_000, 10_000, 32, 128
EMPTY_ID = 0x7FFFFFFF


@pytest.fixture(scope="module")
def world(gpu_ctx):
    import torch
    import apoe
    import apoe_synth as S
    corpus = S.corpus(N_DOCS, seed=101, device="cuda:0")
    queries = S.queries(N_QUERIES, seed=102, device="cuda:0")
    torch.cuda.synchronize()
    gc = apoe.Corpus(gpu_ctx, *corpus)
    gq = apoe.Queries(gpu_ctx, *queries)
    graph, ms = apoe.build_graph(gpu_ctx, gc, K=64, iters=10, degree=DEGREE, seed=3)
    rows, entry = graph.download()
    yield dict(ctx=gpu_ctx, corpus=corpus, queries=queries, gc=gc, gq=gq, graph=graph, rows=rows, entry=entry, build_ms=ms)
    graph.close()
    gq.close()
    gc.close()


def test_graph_rows_are_well_formed(world):
    rows, entry = world["rows"], world["entry"]
    assert rows.shape == (N_DOCS, DEGREE + 8) and len(entry) == DEGREE
    nb = rows[:, :DEGREE]
    assert nb.max() < N_DOCS
    assert not (nb == np.arange(N_DOCS, dtype=np.uint32)[:, None]).all(axis=1).any()
    # the forward half of a row holds distinct documents
    half = np.sort(nb[:, :DEGREE // 2], axis=1)
    assert (np.diff(half.astype(np.int64), axis=1) != 0).mean() > 0.999
    cnt = rows[:, DEGREE]
    assert cnt.max() <= 7
    kw = rows[:, DEGREE + 1:]
    assert np.all(kw[np.arange(7)[None, :] >= cnt[:, None]] == 0)
    assert kw.max() < N_DOCS
    assert len(set(entry.tolist())) == DEGREE


def test_search_rows_sorted_unique_and_distances_are_the_metric(world):
    import apoe
    w = world
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], (1, 1, 1), CANDS)
    assert np.all(np.diff(dist, axis=1) >= 0)
    real = ids != EMPTY_ID
    assert real[:, :10].all()
    for q in range(0, N_QUERIES, 97):
        r = ids[q][real[q]]
        assert len(set(r.tolist())) == len(r)
    # every reported distance is the fused metric of that pair (an independent kernel computes it)
    safe = np.where(real, ids, 0).astype(np.uint32)
    again = apoe.distance_batch(w["ctx"], w["gc"], w["gq"], (1, 1, 1), safe)
    assert_dist_close(dist[real], again[real], "search distances vs distance_batch")
    # the bound never changes a result: reading every dense row gives the same rows
    ids2, dist2, st2 = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], (1, 1, 1), CANDS, variant=0x100)
    assert np.array_equal(ids, ids2) and np.array_equal(dist, dist2)
    assert st.evaluations == st2.evaluations and st.dense_rows < st2.dense_rows == st2.evaluations
    # launch shapes agree
    ids3, dist3, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], (1, 1, 1), CANDS, variant=2)
    assert assert_topk_match(ids, dist, ids3, dist3, 10, "launch shapes") > 0.99


def test_sample_matches_oracle_on_the_gpu_built_graph(world):
    import apoe_synth as S
    import oracle as O
    import apoe
    w = world
    C = O.HybridSet(*S.to_numpy(w["corpus"]))
    nq = 200
    Q = O.HybridSet(*S.to_numpy(w["queries"])).head(nq)
    for w3 in ((1.0, 1.0, 1.0), (1.0, 0.5, 2.0)):
        ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], w3, CANDS, q_count=nq)
        oid, odist, _ = O.search(C, Q, w["rows"], w["entry"], w3, CANDS)
        assert assert_topk_match(ids, dist, oid, odist, 10, f"100k docs, weights {w3}") > 0.97
        same = ids == oid
        assert same.mean() > 0.95
        assert_dist_close(dist[same], odist[same], "pool distances")
    # entry points and norms as the oracle derives them from the same corpus
    assert np.array_equal(w["entry"], O.entry_points(O.norms(C, 7.0), DEGREE))


def test_recall_grows_with_the_pool_and_beats_a_random_graph(world):
    import torch
    import apoe
    import apoe_bruteforce as B
    w = world
    nq = 500
    truth, _ = B.hybrid_topk(w["corpus"], w["queries"], (1.0, 1.0, 1.0), 10, nq=nq)
    rec = []
    for cands in (32, 128, 512):
        ids, _, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], (1, 1, 1), cands, q_count=nq)
        rec.append(recall_at_k(ids, truth, 10))
    assert rec == sorted(rec) and rec[-1] > rec[0] + 0.05, rec
    rng = np.random.default_rng(0)
    rnd_rows = w["rows"].copy()
    rnd_rows[:, :DEGREE] = rng.integers(0, N_DOCS, (N_DOCS, DEGREE))
    g2 = apoe.Graph(w["ctx"], rnd_rows, w["entry"])
    ids, _, _ = apoe.search(w["ctx"], w["gc"], w["gq"], g2, (1, 1, 1), 128, q_count=nq)
    assert recall_at_k(ids, truth, 10) < rec[1]
    g2.close()


def test_pair_format_does_not_change_results(world):
    """The same corpus with its BM25 terms relabelled past 65 535 (8-byte pairs on the device instead of 6-byte ones)
    gives the same search rows on the same graph, and K-NN lists of the same quality after one NN-Descent step."""
    import torch
    import apoe
    w = world
    shift = 70000
    corpus_w = tuple(w["corpus"][:5]) + (w["corpus"][5] + shift,) + tuple(w["corpus"][6:])
    queries_w = tuple(w["queries"][:5]) + (w["queries"][5] + shift,) + tuple(w["queries"][6:])
    torch.cuda.synchronize()
    gc2 = apoe.Corpus(w["ctx"], *corpus_w)
    gq2 = apoe.Queries(w["ctx"], *queries_w)
    assert w["gc"].pair_bytes() == 6 and gc2.pair_bytes() == 8
    for w3 in ((1, 1, 1), (0, 0, 1)):
        a, ad, sa = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], w3, CANDS, q_count=1000)
        b, bd, sb = apoe.search(w["ctx"], gc2, gq2, w["graph"], w3, CANDS, q_count=1000)
        assert np.array_equal(a, b)
        assert_dist_close(ad, bd, f"narrow vs wide pairs, weights {w3}")
        assert sa.evaluations == sb.evaluations and sa.dense_rows == sb.dense_rows

    def one_step(gc):
        knn = apoe.Knn(w["ctx"], gc, 64, 7.0)
        knn.init(3)
        knn.iterate(last=True)
        knn.merge_reverse()
        ids, dist = knn.download()
        knn.close()
        return ids, dist

    i1, d1 = one_step(w["gc"])
    i2, d2 = one_step(gc2)
    # a step reads lists that other workgroups are rewriting, so no two runs give the same lists; they are equally good
    assert abs(float(d1.mean()) - float(d2.mean())) < 0.01 * abs(float(d1.mean()))
    import apoe_synth as S
    import oracle as O
    C = O.HybridSet(*S.to_numpy(w["corpus"]))
    rng = np.random.default_rng(4)
    r, c = rng.integers(0, N_DOCS, 3000), rng.integers(0, 64, 3000)
    assert_dist_close(d2[r, c], O.distance_pairs(C, 7.0, r.astype(np.uint32), i2[r, c]), "wide pairs: stored distance == metric")
    gq2.close()
    gc2.close()


def test_kg_and_keyword_samples_match_oracle(world):
    """Knowledge-graph and keyword-filter search at this size against the oracle on the GPU-built graph (200 queries)."""
    import apoe
    import apoe_synth as S
    import oracle as O
    w = world
    nq = 200
    corpus_np = S.to_numpy(w["corpus"])
    queries_np = S.to_numpy(w["queries"])
    C = O.HybridSet(*corpus_np)
    Q = O.HybridSet(*queries_np).head(nq)
    kg = S.to_numpy(S.knowledge_graph(20000, N_DOCS, N_QUERIES, seed=21, device="cpu"))
    gkg = apoe.KnowledgeGraph(w["ctx"], *kg)
    okg = O.Kg(kg[0], kg[1], kg[2], kg[3], kg[4][:nq + 1], kg[5][:kg[4][nq]])
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], (1, 1, 1), CANDS, kg=gkg, kg_weight=40.0, q_count=nq)
    oid, odist, _ = O.search(C, Q, w["rows"], w["entry"], (1, 1, 1), CANDS, kg=okg, kg_weight=40.0)
    assert assert_topk_match(ids, dist, oid, odist, 10, "100k docs, knowledge graph") > 0.97
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
    kid, kdist, _ = apoe.search(w["ctx"], w["gc"], gqk, w["graph"], (1, 1, 1), CANDS, keyword_filter=True, q_count=nq)
    okid, okdist, _ = O.search(C, O.HybridSet(*qk).head(nq), w["rows"], w["entry"], (1, 1, 1), CANDS, keyword_filter=True)
    assert (kid == okid).all(axis=1).mean() > 0.97
    assert (okid != EMPTY_ID).any()
    gqk.close()
