"""A corpus with a few very long sparse rows among ordinary ones: the table overflow lists, the loop over rows
longer than the register window and the union-table retry of the prune all run, and must not change a result."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match

pytestmark = pytest.mark.gpu

N, HEAVY_EVERY = 2000, 50  # every 50th doc is heavy: 450 SPLADE + 260 BM25 terms more than the others


@pytest.fixture(scope="module", params=[0, 70000], ids=["narrow_pairs", "wide_pairs"])
def heavy_world(request, gpu_ctx):
    import apoe
    import apoe_synth as S
    import oracle as O
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(S.corpus(N, seed=61, device="cpu"))
    rng = np.random.default_rng(7)

    def inflate(off, idx, val, n_terms, lo, hi):
        rows_i, rows_v = [], []
        for v in range(N):
            i, x = idx[off[v]:off[v + 1]], val[off[v]:off[v + 1]]
            if v % HEAVY_EVERY == 0:
                extra = np.setdiff1d(rng.choice(30000, n_terms, replace=False).astype(np.uint32), i)
                i = np.concatenate([i, extra])
                x = np.concatenate([x, rng.uniform(lo, hi, len(extra)).astype(np.float32)])
                o = np.argsort(i)
                i, x = i[o], x[o]
            rows_i.append(i)
            rows_v.append(x)
        new_off = np.zeros(N + 1, np.uint32)
        new_off[1:] = np.cumsum([len(r) for r in rows_i])
        return new_off, np.concatenate(rows_i).astype(np.uint32), np.concatenate(rows_v).astype(np.float32)

    s_off, s_idx, s_val = inflate(s_off, s_idx, s_val, 450, 0.2, 2.0)
    b_off, b_idx, b_val = inflate(b_off, b_idx, b_val, 260, 0.5, 8.0)
    b_idx = b_idx + np.uint32(request.param)  # relabelled BM25 terms past 65535 force 8-byte pairs on the device
    corpus = (dense, s_off, s_idx, s_val, b_off, b_idx, b_val)
    queries = S.to_numpy(S.queries(100, seed=62, device="cpu"))
    queries = queries[:5] + (queries[5] + np.uint32(request.param),) + queries[6:]
    C, Q = O.HybridSet(*corpus), O.HybridSet(*queries)
    rows, entry, knn_ids, knn_dist = O.build_index(C, dense_scale=7.0, K=64, iters=6, d=32, seed=5, return_knn=True)
    gc = apoe.Corpus(gpu_ctx, *corpus)
    gq = apoe.Queries(gpu_ctx, *queries)
    assert gc.pair_bytes() == (8 if request.param else 6)
    info = gc.info()
    assert info[2] > 400 and info[3] > 250  # the heavy rows are there
    return dict(ctx=gpu_ctx, C=C, Q=Q, gc=gc, gq=gq, rows=rows, entry=entry, knn_ids=knn_ids, knn_dist=knn_dist)


def test_pair_distances_with_heavy_pivots_and_candidates(heavy_world):
    import apoe
    import oracle as O
    w = heavy_world
    rng = np.random.default_rng(3)
    heavy = np.arange(0, N, HEAVY_EVERY, dtype=np.uint32)
    a = np.concatenate([rng.choice(heavy, 300), rng.integers(0, N, 300).astype(np.uint32), rng.choice(heavy, 300)]).astype(np.uint32)
    b = np.concatenate([rng.integers(0, N, 300).astype(np.uint32), rng.choice(heavy, 300), rng.choice(heavy, 300)]).astype(np.uint32)
    got = apoe.distance_pairs(w["ctx"], w["gc"], 7.0, a, b)
    assert_dist_close(got, O.distance_pairs(w["C"], 7.0, a, b), "pairs with heavy rows")


@pytest.mark.parametrize("join", [0, 1, 2])
def test_nn_descent_stores_the_metric(heavy_world, join):
    """Every stored distance is the metric of that pair. Expansion step: heavy pivots go through the overflow list of
    the four-entry bucket table, heavy candidates through the loop over more than 192 pairs. Join tiles: a heavy row
    among the pickers makes the rank table take its group in passes of fewer pivots, a heavy column is read beyond
    the register window of 256 pairs."""
    import apoe
    import oracle as O
    w = heavy_world
    knn = apoe.Knn(w["ctx"], w["gc"], 64, 7.0)
    knn.set_join(join)
    knn.init(9)
    for it in range(4):
        knn.iterate(last=(it == 3))
    knn.merge_reverse()
    ids, dist = knn.download()
    knn.close()
    assert np.all(np.diff(dist, axis=1) >= 0) and ids.max() < N
    heavy = np.arange(0, N, HEAVY_EVERY)
    rows_ = np.concatenate([np.repeat(heavy, 64), np.random.default_rng(1).integers(0, N, 3000)])
    cols_ = np.concatenate([np.tile(np.arange(64), len(heavy)), np.random.default_rng(2).integers(0, 64, 3000)])
    want = O.distance_pairs(w["C"], 7.0, rows_.astype(np.uint32), ids[rows_, cols_])
    assert_dist_close(dist[rows_, cols_], want, "stored distance == recomputed distance")
    # ... and where a heavy row is the stored neighbour (a candidate with more than 192 pairs)
    hr, hc = np.nonzero(np.isin(ids, heavy))
    assert len(hr) > 1000
    want = O.distance_pairs(w["C"], 7.0, hr[:4000].astype(np.uint32), ids[hr[:4000], hc[:4000]])
    assert_dist_close(dist[hr[:4000], hc[:4000]], want, "stored distance of a heavy neighbour")


def test_prune_matches_oracle_on_the_same_knn_graph(heavy_world):
    import apoe
    import oracle as O
    w = heavy_world
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
    assert np.array_equal(entry, w["entry"])


@pytest.mark.parametrize("w3", [(1.0, 1.0, 1.0), (0.0, 1.0, 1.0)])
def test_search_matches_oracle(heavy_world, w3):
    import apoe
    import oracle as O
    w = heavy_world
    g = apoe.Graph(w["ctx"], w["rows"], w["entry"])
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], g, w3, 64)
    oid, odist, cnt = O.search(w["C"], w["Q"], w["rows"], w["entry"], w3, 64)
    assert assert_topk_match(ids, dist, oid, odist, 10, f"heavy rows, weights {w3}") > 0.97
    same = ids == oid
    assert_dist_close(dist[same], odist[same], "pool distances")
    ids2, dist2, _ = apoe.search(w["ctx"], w["gc"], w["gq"], g, w3, 64, variant=0x100)
    assert np.array_equal(ids, ids2) and np.array_equal(dist, dist2)
    g.close()


def test_join_refuses_rows_longer_than_its_table(gpu_ctx):
    """One document with more sparse terms than the join tile's LDS table holds (APOE_JOIN_MAX_ROW_TERMS = 2304): the
    join is refused with a message when it is chosen, instead of evaluating that row without its sparse part."""
    import apoe
    import apoe_synth as S
    n = 200
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(S.corpus(n, seed=63, device="cpu"))
    rng = np.random.default_rng(9)

    def with_long_row(off, idx, val, row, terms):
        cnt = np.diff(off.astype(np.int64))
        keep = np.repeat(np.arange(n) != row, cnt)
        new_i = np.sort(rng.choice(30000, terms, replace=False)).astype(np.uint32)
        new_v = rng.uniform(0.5, 2.0, terms).astype(np.float32)
        at = int(off[row] - 0)  # rows before `row` keep their place; its pairs are replaced
        i2, v2 = idx[keep], val[keep]
        i2 = np.concatenate([i2[:at], new_i, i2[at:]])
        v2 = np.concatenate([v2[:at], new_v, v2[at:]])
        cnt[row] = terms
        o2 = np.zeros(n + 1, np.uint32)
        o2[1:] = np.cumsum(cnt)
        return o2, i2, v2

    s_off, s_idx, s_val = with_long_row(s_off, s_idx, s_val, 17, 1500)
    b_off, b_idx, b_val = with_long_row(b_off, b_idx, b_val, 17, 900)
    gc = apoe.Corpus(gpu_ctx, dense, s_off, s_idx, s_val, b_off, b_idx, b_val)
    assert gc.info()[2] + gc.info()[3] > 2304
    knn = apoe.Knn(gpu_ctx, gc, 64, 7.0)
    with pytest.raises(RuntimeError, match="expansion step"):
        knn.set_join(1)
    knn.close()
    gc.close()


def test_wide_corpus_with_a_row_of_two_thousand_terms_builds(gpu_ctx, tmp_path, capfd):
    """Term ids past 65535 (the wide pair format hashes a row's terms into the join tile's table) and one document of about
    2000 terms: the join chosen by hand either runs or ends with a call-sequence error that names the expansion step, never
    with lists that lack a sparse part; build_index with its default step builds the index either way."""
    import apoe
    import apoe_synth as S
    import hybrid_search
    import oracle as O
    n = 300
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(S.corpus(n, seed=64, device="cpu"))
    rng = np.random.default_rng(10)
    cnt = np.diff(s_off.astype(np.int64))
    row, terms = 23, 1400
    keep = np.repeat(np.arange(n) != row, cnt)
    new_i = np.sort(rng.choice(3_000_000, terms, replace=False)).astype(np.uint32) + np.uint32(70000)
    new_v = rng.uniform(0.5, 2.0, terms).astype(np.float32)
    at = int(s_off[row])
    s_idx = np.concatenate([s_idx[keep][:at], new_i, s_idx[keep][at:]])
    s_val = np.concatenate([s_val[keep][:at], new_v, s_val[keep][at:]])
    cnt[row] = terms
    s_off = np.zeros(n + 1, np.uint32)
    s_off[1:] = np.cumsum(cnt)
    bcnt = np.diff(b_off.astype(np.int64))
    bkeep = np.repeat(np.arange(n) != row, bcnt)
    nb_i = np.sort(rng.choice(3_000_000, 600, replace=False)).astype(np.uint32) + np.uint32(70000)
    bat = int(b_off[row])
    b_idx = np.concatenate([b_idx[bkeep][:bat], nb_i, b_idx[bkeep][bat:]])
    b_val = np.concatenate([b_val[bkeep][:bat], rng.uniform(0.5, 8.0, 600).astype(np.float32), b_val[bkeep][bat:]])
    bcnt[row] = 600
    b_off = np.zeros(n + 1, np.uint32)
    b_off[1:] = np.cumsum(bcnt)
    corpus = (dense, s_off, s_idx, s_val, b_off, b_idx, b_val)
    gc = apoe.Corpus(gpu_ctx, *corpus)
    assert gc.pair_bytes() == 8 and 1024 < gc.info()[2] + gc.info()[3] <= 2304
    C = O.HybridSet(*corpus)
    knn = apoe.Knn(gpu_ctx, gc, 64, 7.0)
    knn.set_join(1)
    knn.init(3)
    try:
        for it in range(3):
            knn.iterate(last=(it == 2))
        ids, dist = knn.download()
        real = dist < apoe.INF_DIS
        a = np.repeat(np.arange(n, dtype=np.uint32), 64).reshape(-1, 64)[real]
        assert_dist_close(dist[real], O.distance_pairs(C, 7.0, a, ids[real]), "stored distance of the join on the wide corpus")
    except apoe.ApoeError as e:
        assert "status -3" in str(e) and "expansion step" in str(e)
    knn.close()
    gc.close()
    p = {k: str(tmp_path / k) for k in ("dense.fvecs", "sparse.bin", "bm25.bin", "index.poe")}
    O.write_fvecs(p["dense.fvecs"], dense)
    O.write_csr(p["sparse.bin"], s_off, s_idx, s_val)
    O.write_csr(p["bm25.bin"], b_off, b_idx, b_val)
    hybrid_search.build_index(dense_data_path=p["dense.fvecs"], sparse_data_path=p["sparse.bin"], bm25_data_path=p["bm25.bin"],
                              output_graph_path=p["index.poe"], nnd_iters=4)
    rows, entry = O.read_poe(p["index.poe"])
    assert rows.shape == (n, 40) and rows[:, :32].max() < n
    assert "Indexing time" in capfd.readouterr().out
