"""The hybrid_search Python module end to end on the GPU: files in, .poe out, search."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def files(tmp_path_factory, small_world):
    import apoe_synth as S
    import oracle as O
    d = tmp_path_factory.mktemp("poe")
    n = 1500
    C = small_world["C"].head(n)
    Q = small_world["Q"]
    p = {k: str(d / k) for k in ("dense.fvecs", "sparse.bin", "bm25.bin", "qdense.fvecs", "qsparse.bin", "qbm25.bin", "index.poe",
                                 "qrels.txt", "kg.bin", "e2d.bin", "qe.bin")}
    O.write_fvecs(p["dense.fvecs"], C.dense)
    O.write_csr(p["sparse.bin"], C.s_off, C.s_idx, C.s_val)
    O.write_csr(p["bm25.bin"], C.b_off, C.b_idx, C.b_val)
    O.write_fvecs(p["qdense.fvecs"], Q.dense)
    O.write_csr(p["qsparse.bin"], Q.s_off, Q.s_idx, Q.s_val)
    O.write_csr(p["qbm25.bin"], Q.b_off, Q.b_idx, Q.b_val)
    kg = S.to_numpy(S.knowledge_graph(500, n, Q.n, seed=31, device="cpu", mean_out=5.0))
    O.write_kg(p["kg.bin"], kg[0], kg[1])
    O.write_kg(p["e2d.bin"], kg[2], kg[3])
    O.write_kg(p["qe.bin"], kg[4], kg[5])
    return dict(paths=p, C=C, Q=Q, kg=kg, n=n)


def test_build_and_search_roundtrip(files, capfd):
    import hybrid_search
    import oracle as O
    p, C, Q = files["paths"], files["C"], files["Q"]
    hybrid_search.build_index(dense_data_path=p["dense.fvecs"], sparse_data_path=p["sparse.bin"], bm25_data_path=p["bm25.bin"],
                              output_graph_path=p["index.poe"], nnd_iters=8)
    out = capfd.readouterr().out
    for line in ("Loading dense data from", "Non zero num:", f"Points: {files['n']}, Dim: 1024", "Max sparse dim:", "Indexing time:"):
        assert line in out, out
    rows, entry = O.read_poe(p["index.poe"])
    assert rows.shape == (files["n"], 40) and len(entry) == 32
    assert os.path.getsize(p["index.poe"]) == 8 + 4 * 32 + files["n"] * 41 * 4
    assert np.array_equal(entry, O.entry_points(O.norms(C, 7.0), 32))

    w_user = (1.0, 1.0, 1.0)
    w_eff = O.calibrate(C, Q, 100, w_user)
    truth, _ = O.bruteforce_topk(C, Q.head(100), w_eff, 10)
    with open(p["qrels.txt"], "w") as f:
        for row in truth:
            f.write(" ".join(str(x) for x in row[:3]) + "\n")
    common = dict(dense_data_path=p["dense.fvecs"], dense_query_path=p["qdense.fvecs"], sparse_data_path=p["sparse.bin"],
                  sparse_query_path=p["qsparse.bin"], bm25_data_path=p["bm25.bin"], bm25_query_path=p["qbm25.bin"], keyword_id_path="",
                  graph_path=p["index.poe"], ground_truth_path=p["qrels.txt"], top_k=10, cands=128, sparse_weight=1.0, bm25_weight=1.0,
                  dense_weight=1.0)
    r = hybrid_search.search(knowledge_path="", entity2doc_path="", query_entity_path="", kg_weight=0.0, **common)
    out = capfd.readouterr().out
    for line in ("query num: 100", "Dense weight: 1, Sparse weight: 1, BM25 weight: 1, KG weight: 0", "Degree: 40,num: 1500", "Begin search",
                 "Search with dense + sparse + bm25", "Query time:", "nDCG@10:"):
        assert line in out, out
    assert r["ids"].shape == (100, 128)
    assert np.allclose(r["weights"], w_eff, rtol=1e-4)
    oid, odist, _ = O.search(C, Q.head(100), rows, entry, r["weights"], 128)
    assert (r["ids"][:, :10] == oid[:, :10]).mean() > 0.97
    want_ndcg, want_recall = O.ndcg(r["ids"][:, :10], [t[:3].tolist() for t in truth])
    assert abs(r["ndcg"] - want_ndcg) < 1e-5 and abs(r["recall"] - want_recall) < 1e-5
    assert r["ndcg"] > 0.5

    # the same search walking on half-precision rows: same rows (the dense part is a small share here), exact distances
    rh = hybrid_search.search(knowledge_path="", entity2doc_path="", query_entity_path="", kg_weight=0.0, half_rows=True, **common)
    capfd.readouterr()
    same = rh["ids"] == r["ids"]
    assert same.mean() > 0.98 and np.array_equal(rh["dist"][same], r["dist"][same])

    # dense-only dispatch and the print-only entry point
    hybrid_search.search_index(knowledge_path="", entity2doc_path="", query_entity_path="", kg_weight=0.0,
                               **{**common, "sparse_weight": 0.0, "bm25_weight": 0.0})
    out = capfd.readouterr().out
    assert "Search with dense\n" in out

    # knowledge-graph path (example.py:14-30 calls it with kg_weight=40)
    rk = hybrid_search.search(knowledge_path=p["kg.bin"], entity2doc_path=p["e2d.bin"], query_entity_path=p["qe.bin"], kg_weight=40.0, **common)
    out = capfd.readouterr().out
    assert "Entity num: 501" in out and "KG Copy end" in out and "Search with dense + sparse + bm25 + kg" in out
    kg = files["kg"]
    okg = O.Kg(kg[0], kg[1], kg[2], kg[3], kg[4][:101], kg[5][:kg[4][100]])
    kid, kdist, _ = O.search(C, Q.head(100), rows, entry, rk["weights"], 128, kg=okg, kg_weight=40.0)
    assert (rk["ids"][:, :10] == kid[:, :10]).mean() > 0.97


def test_keyword_file_search(files, capfd):
    """keyword_id_path: line i lists term ids; those that are BM25 terms of query i become required keywords
    (query.cu:1828-1843) and the keyword-filter search runs (query.cu:2005-2007)."""
    import hybrid_search
    import oracle as O
    p, C, Q = files["paths"], files["C"], files["Q"]
    if not os.path.exists(p["index.poe"]):
        hybrid_search.build_index(dense_data_path=p["dense.fvecs"], sparse_data_path=p["sparse.bin"], bm25_data_path=p["bm25.bin"],
                                  output_graph_path=p["index.poe"], nnd_iters=8)
    rows, entry = O.read_poe(p["index.poe"])
    df = np.bincount(C.b_idx, minlength=int(max(C.b_idx.max(), Q.b_idx.max())) + 2)
    kw_path = os.path.join(os.path.dirname(p["index.poe"]), "keywords.txt")
    flagged = Q.b_idx.copy()
    n_flag = 0
    with open(kw_path, "w") as f:
        for q in range(100):
            terms = Q.b_idx[Q.b_off[q]:Q.b_off[q + 1]]
            present = [int(t) for t in terms if df[t] > 0]
            # the rarest term of the query that some document holds, plus an id no query has
            pick = min(present, key=lambda t: df[t]) if present else None
            f.write(" ".join(str(x) for x in ([pick] if pick is not None else []) + [4000000]) + "\n")
            if pick is not None:
                flagged[Q.b_off[q] + list(terms).index(pick)] |= 0x80000000
                n_flag += 1
    with open(p["qrels.txt"], "w") as f:
        for q in range(100):
            f.write("0\n")
    r = hybrid_search.search(dense_data_path=p["dense.fvecs"], dense_query_path=p["qdense.fvecs"], sparse_data_path=p["sparse.bin"],
                             sparse_query_path=p["qsparse.bin"], bm25_data_path=p["bm25.bin"], bm25_query_path=p["qbm25.bin"],
                             keyword_id_path=kw_path, knowledge_path="", entity2doc_path="", query_entity_path="", graph_path=p["index.poe"],
                             ground_truth_path=p["qrels.txt"], top_k=10, cands=64, sparse_weight=1.0, bm25_weight=1.0, dense_weight=1.0,
                             kg_weight=0.0, calibrate=False)
    out = capfd.readouterr().out
    assert f"keywords: {n_flag}" in out and "Search with dense + sparse + bm25 + keyword" in out
    assert out.index("query num: 100") < out.index("keywords:") < out.index("Dense weight:")
    Qk = O.HybridSet(Q.dense, Q.s_off, Q.s_idx, Q.s_val, Q.b_off, flagged, Q.b_val).head(100)
    oid, odist, _ = O.search(C, Qk, rows, entry, (1.0, 1.0, 1.0), 64, keyword_filter=True)
    assert (r["ids"] == oid).all(axis=1).mean() > 0.97
    assert (oid != 0x7FFFFFFF).any()


def test_knn_graph_save_and_reprune(files, capfd):
    """The K-NN graph saved between NN-Descent and the prune rebuilds the same index without NN-Descent,
    and re-prunes to another degree."""
    import hybrid_search
    import oracle as O
    p = files["paths"]
    d = os.path.dirname(p["index.poe"])
    knn_path, a_path, b_path, c_path = (os.path.join(d, x) for x in ("graph.knn", "a.poe", "b.poe", "c.poe"))
    common = dict(dense_data_path=p["dense.fvecs"], sparse_data_path=p["sparse.bin"], bm25_data_path=p["bm25.bin"])
    hybrid_search.build_index(output_graph_path=a_path, nnd_iters=6, knn_save_path=knn_path, **common)
    n = files["n"]
    assert os.path.getsize(knn_path) == 12 + n * 64 * 8
    head = np.fromfile(knn_path, np.uint32, 3)
    assert head.tolist() == [0x4E4B5041, n, 64]
    ids = np.fromfile(knn_path, np.uint32, n * 64, offset=12).reshape(n, 64)
    dist = np.fromfile(knn_path, np.float32, n * 64, offset=12 + n * 64 * 4).reshape(n, 64)
    assert ids.max() < n and np.all(np.diff(dist, axis=1) >= 0)
    hybrid_search.build_index(output_graph_path=b_path, nnd_iters=0, knn_load_path=knn_path, **common)
    ra, ea = O.read_poe(a_path)
    rb, eb = O.read_poe(b_path)
    assert np.array_equal(ra, rb) and np.array_equal(ea, eb)
    hybrid_search.build_index(output_graph_path=c_path, degree=16, knn_load_path=knn_path, **common)
    rc, ec = O.read_poe(c_path)
    assert rc.shape == (n, 24) and len(ec) == 16
    # the oracle prunes the saved graph to the same rows
    C = files["C"]
    fwd, det, cnt, kw = O.prune(C, 7.0, O.norms(C, 7.0), ids, dist, 16)
    want = O.final_graph(fwd, det, cnt, kw)
    assert (rc == want).all(axis=1).mean() > 0.995
    capfd.readouterr()
    with pytest.raises(RuntimeError, match="K-NN graph"):
        hybrid_search.build_index(output_graph_path=c_path, nnd_k=128, knn_load_path=knn_path, **common)


def test_build_on_half_precision_rows(files, capfd):
    """build_index(half_rows=True): the saved K-NN lists carry fp32 distances and the index file passes the checker."""
    import hybrid_search
    import oracle as O
    p = files["paths"]
    d = os.path.dirname(p["index.poe"])
    knn_path, h_path = os.path.join(d, "half.knn"), os.path.join(d, "half.poe")
    hybrid_search.build_index(dense_data_path=p["dense.fvecs"], sparse_data_path=p["sparse.bin"], bm25_data_path=p["bm25.bin"],
                              output_graph_path=h_path, nnd_iters=6, knn_save_path=knn_path, half_rows=True)
    capfd.readouterr()
    n = files["n"]
    ids = np.fromfile(knn_path, np.uint32, n * 64, offset=12).reshape(n, 64)
    dist = np.fromfile(knn_path, np.float32, n * 64, offset=12 + n * 64 * 4).reshape(n, 64)
    assert ids.max() < n and np.all(np.diff(dist, axis=1) >= 0)
    rng = np.random.default_rng(2)
    r, c = rng.integers(0, n, 3000), rng.integers(0, 64, 3000)
    want = O.distance_pairs(files["C"], 7.0, r.astype(np.uint32), ids[r, c])
    assert np.allclose(dist[r, c], want, rtol=1e-4, atol=1e-4)
    rep = hybrid_search.validate_graph(h_path, n)
    assert rep["ok"] and rep["degree"] == 32


def test_errors_raise(files):
    import hybrid_search
    p = files["paths"]
    with pytest.raises(RuntimeError, match="open file error"):
        hybrid_search.build_index("/nonexistent.fvecs", p["sparse.bin"], p["bm25.bin"], "/tmp/x.poe")
    with pytest.raises(RuntimeError):
        hybrid_search.build_index(p["dense.fvecs"], p["sparse.bin"], p["bm25.bin"], "/tmp/x.poe", degree=33)
    with pytest.raises(RuntimeError, match="knowledge_path"):
        hybrid_search.search_index(p["dense.fvecs"], p["qdense.fvecs"], p["sparse.bin"], p["qsparse.bin"], p["bm25.bin"], p["qbm25.bin"], "",
                                   "", "", "", p["index.poe"], p["qrels.txt"], 10, 64, 1.0, 1.0, 1.0, 40.0)
