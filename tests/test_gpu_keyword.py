"""HIP keyword-filter search against the CPU oracle and closed forms (through the C-ABI)."""
import numpy as np
import pytest

from keyword_worlds import EMPTY_ID, KW, chain_world, make_world
from parity import assert_dist_close

pytestmark = pytest.mark.gpu


def flag_keywords(world, rule):
    """Copy of the world's queries with bit 31 set on one BM25 term per query: the rarest of the
    query's terms ('rare'), the most frequent one ('common'), or none ('none')."""
    corpus, queries = world["corpus"], world["queries"]
    b_off, b_idx = queries[4], queries[5].copy()
    df = np.bincount(corpus[5], minlength=int(max(corpus[5].max(), b_idx.max())) + 1)
    for q in range(len(b_off) - 1):
        terms = b_idx[b_off[q]:b_off[q + 1]]
        if len(terms) == 0 or rule == "none":
            continue
        f = df[terms]
        present = np.where(f > 0)[0]
        if len(present) == 0:
            continue
        j = present[np.argmin(f[present])] if rule == "rare" else int(np.argmax(f))
        b_idx[b_off[q] + j] |= KW
    return queries[:5] + (b_idx,) + queries[6:]


def to_gpu(ctx, C, Q, rows, entry):
    import apoe
    return apoe.Corpus(ctx, *C.arrays()), apoe.Queries(ctx, *Q.arrays()), apoe.Graph(ctx, rows, entry)


def rows_match(ids, dist, oid, odist, what):
    """Rows equal, except where an order differs between distances that tie within 1e-4."""
    same = np.all(ids == oid, axis=1)
    for q in np.where(~same)[0]:
        a, b = ids[q], oid[q]
        assert sorted(a.tolist()) == sorted(b.tolist()), f"{what}: query {q} holds different documents"
        for i in np.where(a != b)[0]:
            j = list(b).index(a[i])
            assert abs(float(odist[q, j]) - float(odist[q, i])) <= 1e-4 * max(1.0, abs(float(odist[q, i]))), f"{what}: query {q}"
    return same.mean()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("cands,rule", [(64, "rare"), (16, "common"), (128, "common"), (32, "rare")])
def test_keyword_search_matches_oracle(gpu_world, cands, rule, variant):
    import apoe
    import oracle as O
    w = gpu_world
    qa = flag_keywords(w, rule)
    Q = O.HybridSet(*qa)
    gq = apoe.Queries(w["ctx"], *qa)
    w3 = (1.0, 1.0, 1.0)
    ids, dist, st = apoe.search(w["ctx"], w["gc"], gq, w["gg"], w3, cands, variant=variant, keyword_filter=True)
    oid, odist, cnt = O.search(w["C"], Q, w["rows"], w["entry"], w3, cands, keyword_filter=True)
    frac = rows_match(ids, dist, oid, odist, f"{rule} cands {cands}")
    assert frac > 0.97
    real = (ids == oid) & (oid != EMPTY_ID)
    assert real.sum() > 0
    assert_dist_close(dist[real], odist[real], "reported distances")
    assert abs(int(st.evaluations) - int(cnt[:, 1].sum())) <= 0.01 * cnt[:, 1].sum()
    # rows hold only documents with the query's keyword
    corpus = w["corpus"]
    for q in range(0, Q.n, 17):
        req = {int(t & 0x7FFFFFFF) for t in Q.b_idx[Q.b_off[q]:Q.b_off[q + 1]] if t & KW}
        for doc in ids[q][ids[q] != EMPTY_ID].tolist():
            assert req & set(corpus[5][corpus[4][doc]:corpus[4][doc + 1]].tolist())


def test_every_dense_row_variant_gives_the_same_rows(gpu_world):
    import apoe
    w = gpu_world
    gq = apoe.Queries(w["ctx"], *flag_keywords(w, "rare"))
    a, ad, sa = apoe.search(w["ctx"], w["gc"], gq, w["gg"], (1, 1, 1), 64, keyword_filter=True)
    b, bd, sb = apoe.search(w["ctx"], w["gc"], gq, w["gg"], (1, 1, 1), 64, keyword_filter=True, variant=0x100)
    assert np.array_equal(a, b) and np.array_equal(ad, bd)
    assert sa.dense_rows < sb.dense_rows == sb.evaluations


def test_no_flagged_term_gives_empty_rows_and_flags_do_not_change_plain_search(gpu_world):
    import apoe
    w = gpu_world
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 32, keyword_filter=True)
    assert np.all(ids == EMPTY_ID) and np.all(dist == np.float32(1000000.0))
    gq = apoe.Queries(w["ctx"], *flag_keywords(w, "common"))
    a, ad, _ = apoe.search(w["ctx"], w["gc"], gq, w["gg"], (1, 1, 1), 32)
    b, bd, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 32)
    assert np.array_equal(a, b) and np.array_equal(ad, bd)


def test_zero_weights_still_run_all_three_paths(gpu_world):
    """The keyword kernel is the three-path loop whatever the weights: a zero BM25 weight still finds the hits."""
    import apoe
    import oracle as O
    w = gpu_world
    qa = flag_keywords(w, "rare")
    gq = apoe.Queries(w["ctx"], *qa)
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], gq, w["gg"], (1.0, 0.0, 0.0), 64, keyword_filter=True)
    oid, odist, _ = O.search(w["C"], O.HybridSet(*qa), w["rows"], w["entry"], (1.0, 0.0, 0.0), 64, keyword_filter=True)
    assert rows_match(ids, dist, oid, odist, "zero sparse weights") > 0.97
    assert (ids != EMPTY_ID).any()


@pytest.mark.parametrize("variant", [0, 1, 3])
def test_ring_closed_form(gpu_ctx, variant):
    """Chain world: the pool ends as docs 299..260, the ring as the last 32 evicted hits 258..196."""
    import apoe
    C, queries, rows, entry = chain_world()
    gc, gq, gg = to_gpu(gpu_ctx, C, queries(True), rows, entry)
    ids, dist, st = apoe.search(gpu_ctx, gc, gq, gg, (1, 1, 1), 40, keyword_filter=True, variant=variant)
    assert st.evaluations == 300
    assert ids[0].tolist() == list(range(298, 218, -2))
    assert np.all(np.diff(dist[0]) > 0)
    ids, dist, st = apoe.search(gpu_ctx, gc, gq, gg, (1, 1, 1), 70, keyword_filter=True, variant=variant)
    assert ids[0].tolist() == list(range(298, 228, -2)) + list(range(228, 164, -2)) + [EMPTY_ID] * 3
    assert np.all(dist[0][-3:] == np.float32(1000000.0))


def test_keyword_edge_is_the_only_route(gpu_ctx):
    import apoe
    n, d = 60, 4
    C, queries, rows, entry = make_world(n=n, kw_docs={50, 7})
    for v in range(n):
        rows[v, :d] = [(v + 1) % 40, (v - 1) % 40, v, v]
    rows[5, d] = 1000  # clamped to the 7 slots a row has
    rows[5, d + 1] = 50
    rows[5, d + 2:] = 0x7FFFFFF0  # not a document: skipped
    entry = np.array([0], np.uint32)
    gc, gq, gg = to_gpu(gpu_ctx, C, queries(True), rows, entry)
    ids, _, _ = apoe.search(gpu_ctx, gc, gq, gg, (1, 1, 1), 64, keyword_filter=True)
    assert sorted(ids[0][ids[0] != EMPTY_ID].tolist()) == [7, 50]
    _, gqp, _ = to_gpu(gpu_ctx, C, queries(False), rows, entry)
    plain, _, _ = apoe.search(gpu_ctx, gc, gqp, gg, (1, 1, 1), 64)
    assert 50 not in plain[0].tolist()


def test_random_graphs_match_oracle(gpu_ctx):
    import apoe
    import oracle as O
    for seed in range(4):
        rng = np.random.default_rng(100 + seed)
        n, d = 80, 6
        kw_docs = set(rng.choice(n, 30, replace=False).tolist())
        C, queries, rows, entry = make_world(n=n, seed=seed, kw_docs=kw_docs, d=d)
        rows[:, :d] = rng.integers(0, n, (n, d))
        rows[:, d] = rng.integers(0, 4, n)
        rows[:, d + 1:] = rng.integers(0, n, (n, 7))
        gc, gq, gg = to_gpu(gpu_ctx, C, queries(True), rows, entry)
        for cands in (3, 8, 40):
            ids, dist, _ = apoe.search(gpu_ctx, gc, gq, gg, (1, 1, 1), cands, keyword_filter=True)
            oid, odist, _ = O.search(C, queries(True), rows, entry, (1, 1, 1), cands, keyword_filter=True)
            assert np.array_equal(ids, oid), (seed, cands)
            assert_dist_close(dist[oid != EMPTY_ID], odist[oid != EMPTY_ID], "tiny world distances")


def test_keyword_filter_with_knowledge_graph_is_rejected(gpu_world):
    import apoe
    w = gpu_world
    empty = (np.zeros(2, np.uint32), np.zeros(0, np.uint32), np.zeros(2, np.uint32), np.zeros(0, np.uint32),
             np.zeros(w["Q"].n + 1, np.uint32), np.zeros(0, np.uint32))
    kg = apoe.KnowledgeGraph(w["ctx"], *empty)
    with pytest.raises(RuntimeError, match="knowledge graph"):
        apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 32, kg=kg, kg_weight=1.0, keyword_filter=True)
