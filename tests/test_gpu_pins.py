"""The hand-built worlds of tests/pin_worlds.py and the reverse merge on the GPU, through the C-ABI: the keyword
flag of the prune (index.cu:128-153,637,651-666), a fresh graph neighbour that is also a logical neighbour
(query.cu:1699-1715), and apoe_nnd_merge_reverse against the oracle on the GPU's own pre-merge state
(index.cu:386-478)."""
import numpy as np
import pytest

import pin_worlds as P

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("K,form", [(64, 0), (64, 1), (128, 0), (128, 1)])  # form 0: the gather-once prunes (Gram matrix in LDS / by tiles), 1: table-probing kernel
@pytest.mark.parametrize("term_shift", [0, 70000])  # narrow and wide pair format of the device records
def test_keyword_flag_world(gpu_ctx, K, form, term_shift):
    import apoe
    import oracle as O
    arrays, ids, dist, expect = P.keyword_flag_world(K=K, term_shift=term_shift)
    gc = apoe.Corpus(gpu_ctx, *arrays)
    assert gc.pair_bytes() == (8 if term_shift else 6)
    knn = apoe.Knn(gpu_ctx, gc, K, 7.0)
    knn.set_prune_form(form)
    knn.upload(ids, dist)
    knn.prune(expect["d"])
    fwd, det, cnt, kw = knn.prune_download()
    assert fwd[0].tolist() == expect["fwd0"]
    assert cnt[0] == expect["cnt0"]
    assert kw[0, 0] == len(expect["kw0"]) and kw[0, 1:1 + kw[0, 0]].tolist() == expect["kw0"]
    assert np.all(kw[1:, 0] == 0)
    C = O.HybridSet(*arrays)
    o = O.prune(C, 7.0, O.norms(C, 7.0), ids, dist, expect["d"])
    for got, want in zip((fwd, det, cnt, kw), o):
        assert np.array_equal(got, want)
    knn.close()
    gc.close()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5])
def test_kg_fresh_neighbour_world(gpu_ctx, variant):
    import apoe
    import oracle as O
    corpus, queries, rows, entry, kg, expect = P.kg_fresh_neighbour_world()
    gc = apoe.Corpus(gpu_ctx, *corpus)
    gq = apoe.Queries(gpu_ctx, *queries)
    gg = apoe.Graph(gpu_ctx, rows, entry)
    gkg = apoe.KnowledgeGraph(gpu_ctx, *kg)
    ids, dist, _ = apoe.search(gpu_ctx, gc, gq, gg, (1.0, 0.0, 0.0), expect["cands"], kg=gkg, kg_weight=expect["kg_weight"], variant=variant)
    plain = 1.0 - corpus[0].astype(np.float64) @ queries[0][0].astype(np.float64)
    P.check_kg_fresh_neighbour(ids[0], dist[0], plain, expect)
    oid, odist, _ = O.search(O.HybridSet(*corpus), O.HybridSet(*queries), rows, entry, (1.0, 0.0, 0.0), expect["cands"], kg=O.Kg(*kg),
                             kg_weight=expect["kg_weight"])
    assert np.array_equal(ids, oid)
    assert np.allclose(dist, odist, atol=1e-4)
    for h in (gkg, gg, gq, gc):
        h.close()


def _oracle_state(n, K, ids, dist, rev, rev_dist, rev_cnt):
    import oracle as O
    st = O.KnnState(n, K)
    st.ids[:], st.dist[:], st.rev[:], st.rev_dist[:], st.rev_cnt[:] = ids, dist, rev, rev_dist, rev_cnt
    return st


@pytest.mark.parametrize("join,steps", [(0, 1), (0, 3), (1, 1), (1, 4), (2, 3)])
def test_merge_reverse_matches_oracle_on_the_gpu_state(gpu_world, join, steps):
    """The lists and reverse lists that the GPU's own steps leave go to the oracle's merge and to the closed form
    (first K of list + registered reverse entries); the GPU merge of the same state must give the same rows."""
    import apoe
    import oracle as O
    w = gpu_world
    n, K = w["C"].n, 64
    knn = apoe.Knn(w["ctx"], w["gc"], K, 7.0)
    knn.set_join(join)
    knn.init(31)
    for it in range(steps):
        knn.iterate(last=(it == steps - 1))
    ids, dist = knn.download()
    rev, rev_dist, rev_cnt = knn.download_reverse()
    assert rev_cnt.max() > 0 and np.any(rev != 0xFFFFFFFF)
    st = _oracle_state(n, K, ids, dist, rev, rev_dist, rev_cnt)
    want_ids, want_dist = P.merge_reverse_closed_form(n, K, ids, dist, rev, rev_dist, rev_cnt)
    O.nnd_merge_reverse(st)
    assert np.array_equal(st.ids, want_ids) and np.array_equal(st.dist, want_dist)
    changed = np.any(want_ids != ids, axis=1)
    assert changed.mean() > 0.3, "the state must give the merge something to do"
    knn.merge_reverse()
    got_ids, got_dist = knn.download()
    assert np.array_equal(got_ids, want_ids)
    assert np.array_equal(got_dist, want_dist)
    _, _, cnt_after = knn.download_reverse()
    assert not cnt_after.any()  # reset_reverse_num, index.cu:899
    knn.close()


def test_merge_reverse_special_cases(gpu_world):
    """An uploaded state: the node itself, an id the list holds, an empty slot, one id twice (the closer copy counts),
    an entry exactly as far as a list entry (goes in front of it), a counter beyond K, a counter below the written slots."""
    import apoe
    import oracle as O
    w = gpu_world
    n, K = w["C"].n, 64
    nxt = (np.arange(n, dtype=np.uint32) + 1) % n
    ids = np.repeat(nxt[:, None], K, axis=1)
    dist = np.full((n, K), P.INF_DIS, np.float32)
    rev = np.full((n, K), 0xFFFFFFFF, np.uint32)
    rev_dist = np.full((n, K), P.INF_DIS, np.float32)
    rev_cnt = np.zeros(n, np.uint32)
    u, v = 7, 9
    ids[u, :4] = [20, 21, 22, 23]
    dist[u, :4] = [0.1, 0.2, 0.3, 0.4]
    rev[u, :8] = [7, 21, 0xFFFFFFFF, 30, 30, 31, 32, 33]
    rev_dist[u, :8] = [0.0, 0.02, P.INF_DIS, 0.25, 0.15, 0.3, 0.35, 5.0]
    rev_cnt[u] = 200
    ids[v, :1] = [40]
    dist[v, :1] = [0.5]
    rev[v, :3] = [41, 42, 43]
    rev_dist[v, :3] = [0.7, 0.6, 0.1]
    rev_cnt[v] = 2
    knn = apoe.Knn(w["ctx"], w["gc"], K, 7.0)
    knn.upload(ids, dist)
    knn.upload_reverse(rev, rev_dist, rev_cnt)
    back = knn.download_reverse()
    assert np.array_equal(back[0], rev) and np.array_equal(back[1], rev_dist) and np.array_equal(back[2], rev_cnt)
    knn.merge_reverse()
    got_ids, got_dist = knn.download()
    assert got_ids[u, :8].tolist() == [20, 30, 21, 31, 22, 32, 23, 33]
    assert np.allclose(got_dist[u, :8], [0.1, 0.15, 0.2, 0.3, 0.3, 0.35, 0.4, 5.0])
    assert np.all(got_dist[u, 8:] == P.INF_DIS)
    assert got_ids[v, :3].tolist() == [40, 42, 41] and got_dist[v, 3] == P.INF_DIS
    st = _oracle_state(n, K, ids, dist, rev, rev_dist, rev_cnt)
    O.nnd_merge_reverse(st)
    assert np.array_equal(got_ids, st.ids) and np.array_equal(got_dist, st.dist)
    # an id that names no document is refused
    bad = rev.copy()
    bad[3, 0] = n + 5
    with pytest.raises(apoe.ApoeError):
        knn.upload_reverse(bad, rev_dist, rev_cnt)
    knn.close()
