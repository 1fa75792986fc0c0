"""File formats against the example data files of the reference checkout (fixtures in
tests/golden/, data only) -- both the oracle's numpy readers and the C++ host loaders
of the hybrid_search module -- and the BM25-only anchor they allow (CPU)."""
import os

import numpy as np
import pytest

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_bm25_queries_header():
    import oracle as O
    off, idx, val = O.read_csr(os.path.join(G, "2wiki_bm25_queries.bin"))
    assert len(idx) == 6763 and len(off) == 1001
    assert off[:5].tolist() == [0, 5, 12, 17, 21]
    ln = np.diff(off)
    assert (ln.min(), ln.max()) == (2, 18) and abs(ln.mean() - 6.76) < 0.01
    assert idx.max() == 33285
    for i in range(1000):
        assert np.all(np.diff(idx[off[i]:off[i + 1]].astype(np.int64)) > 0)


def test_bm25_corpus_header():
    import oracle as O
    off, idx, val = O.read_csr(os.path.join(G, "2wiki_bm25_corpus.bin"))
    assert len(idx) == 225576 and len(off) == 6120
    ln = np.diff(off)
    assert (ln.min(), ln.max()) == (2, 347) and abs(ln.mean() - 36.9) < 0.05
    assert idx.max() == 33356
    n2 = np.add.reduceat(val.astype(np.float64) ** 2, off[:-1].astype(np.int64))
    assert abs(n2.min() - 6.2) < 0.1 and abs(n2.max() - 54.1) < 0.1


def test_kg_headers():
    import oracle as O
    off, idx = O.read_kg(os.path.join(G, "2wiki_kg.bin"))
    assert len(off) == 30485 and len(idx) == 60788
    deg = np.diff(off)
    assert (deg.min(), deg.max()) == (0, 89) and abs(deg.mean() - 1.99) < 0.01
    assert os.path.getsize(os.path.join(G, "2wiki_kg.bin")) == 8 + 4 * 30485 + 4 * 60788
    off, idx = O.read_kg(os.path.join(G, "2wiki_entity2doc.bin"))
    assert len(off) == 30485 and len(idx) == 39852 and idx.max() == 6118
    d = np.diff(off)
    assert (d.min(), d.max()) == (1, 96)
    off, idx = O.read_kg(os.path.join(G, "2wiki_query_kg.bin"))
    assert len(off) == 101 and len(idx) == 148
    d = np.diff(off)
    assert (d.min(), d.max()) == (1, 2)


def test_dense_and_sparse_query_heads():
    import oracle as O
    q = O.read_fvecs(os.path.join(G, "2wiki_dense_queries_head8.fvecs"))
    assert q.shape == (8, 1024)
    assert abs(np.linalg.norm(q[0]) - 1.0002) < 1e-3
    assert np.allclose(q[0, :3], [-0.015411, 0.000314, -0.039612], atol=1e-6)
    off, idx, val = O.read_csr(os.path.join(G, "2wiki_sparse_queries_head16.bin"))
    assert off[:5].tolist() == [0, 62, 113, 181, 249] and len(off) == 17


def test_qrels():
    import oracle as O
    q = O.read_id_lines(os.path.join(G, "2wiki_qrels.txt"))
    assert len(q) == 1000
    assert sum(len(r) == 2 for r in q) == 765 and sum(len(r) == 4 for r in q) == 235
    assert max(max(r) for r in q) == 6115


def test_bm25_only_anchor():
    """Brute-force BM25-only top-10 of the first 100 example queries scores nDCG@10 = 0.7149
    and recall 0.6850 against the example qrels under the reference's nDCG formula."""
    import oracle as O
    coff, cidx, cval = O.read_csr(os.path.join(G, "2wiki_bm25_corpus.bin"))
    qoff, qidx, qval = O.read_csr(os.path.join(G, "2wiki_bm25_queries.bin"))
    n, nq = len(coff) - 1, 100
    zs = (np.zeros(n + 1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    zq = (np.zeros(nq + 1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    C = O.HybridSet(np.zeros((n, 1024), np.float32), *zs, coff, cidx, cval)
    Q = O.HybridSet(np.zeros((nq, 1024), np.float32), *zq, qoff[:nq + 1], qidx[:qoff[nq]], qval[:qoff[nq]])
    ids, dist = O.bruteforce_topk(C, Q, (0, 0, 1), 10)
    gt = O.read_id_lines(os.path.join(G, "2wiki_qrels.txt"), 100)
    nd, rec = O.ndcg(ids, gt)
    assert abs(nd - 0.7149) < 5e-4 and abs(rec - 0.6850) < 5e-4, (nd, rec)


def test_poe_roundtrip_and_size(tmp_path):
    import oracle as O
    rng = np.random.default_rng(0)
    for n, d in ((10, 32), (257, 48), (3, 64)):
        rows = rng.integers(0, n, (n, d + 8), dtype=np.uint32)
        entry = rng.integers(0, n, d, dtype=np.uint32)
        p = str(tmp_path / f"g{n}.poe")
        O.write_poe(p, rows, entry)
        assert os.path.getsize(p) == 8 + 4 * d + n * (d + 8 + 1) * 4
        raw = np.fromfile(p, np.uint32)
        assert raw[0] == d + 8 and raw[1] == d and raw[2 + d] == d + 8
        r2, e2 = O.read_poe(p)
        assert np.array_equal(r2, rows) and np.array_equal(e2, entry)


# ---- the C++ host loaders of the shipped module read the same bytes ----

def test_validate_graph_reports_what_is_wrong(tmp_path):
    """hybrid_search.validate_graph on a good file and on files broken one way each (host code only, no GPU)."""
    import hybrid_search as hs
    rng = np.random.default_rng(5)
    n, d = 50, 6
    rows = rng.integers(0, n, (n, d + 8)).astype(np.uint32)
    rows[:, d] = rng.integers(0, 8, n)
    rows[3, 2] = 3  # a self loop is legal padding
    entry = np.arange(d, dtype=np.uint32)
    good = str(tmp_path / "good.poe")
    hs._write_poe(good, rows, entry)
    r = hs.validate_graph(good, n)
    assert r["ok"] and r["message"] == "ok"
    assert (r["width"], r["degree"], r["num"], r["n_entry"]) == (d + 8, d, n, d)
    assert r["file_bytes"] == 8 + 4 * d + n * (d + 9) * 4 and r["trailing_bytes"] == 0
    assert r["keyword_edges"] == int(rows[:, d].sum()) and r["self_loops"] == int((rows[:, :d] == np.arange(n)[:, None]).sum()) >= 1
    assert not hs.validate_graph(good, n + 1)["ok"]

    def broken(name, change_rows=None, change_entry=None, tail=b""):
        r2, e2 = rows.copy(), entry.copy()
        if change_rows:
            change_rows(r2)
        if change_entry:
            change_entry(e2)
        path = str(tmp_path / name)
        hs._write_poe(path, r2, e2)
        if tail:
            with open(path, "ab") as f:
                f.write(tail)
        return hs.validate_graph(path)

    r = broken("nbr.poe", change_rows=lambda x: x.__setitem__((7, 1), n + 5))
    assert not r["ok"] and r["bad_neighbours"] == 1 and "neighbour" in r["message"]

    def bad_kw(x):
        x[9, d] = 2
        x[9, d + 2] = 1000
        x[9, d + 3] = 1000  # beyond the count: not looked at

    r = broken("kw.poe", change_rows=bad_kw)
    assert not r["ok"] and r["bad_keyword_edges"] == 1
    r = broken("cnt.poe", change_rows=lambda x: x.__setitem__((4, d), 40))
    assert r["keyword_counts_over_7"] == 1 and r["ok"]  # the search clamps the count to the 7 slots
    r = broken("ep.poe", change_entry=lambda e: e.__setitem__(0, n))
    assert not r["ok"] and r["bad_entry_points"] == 1
    r = broken("tail.poe", tail=b"\0" * 12)
    assert not r["ok"] and r["trailing_bytes"] == 12
    # a wrong width word inside the file
    path = str(tmp_path / "width.poe")
    hs._write_poe(path, rows, entry)
    with open(path, "r+b") as f:
        f.seek(8 + 4 * d + 5 * (d + 9) * 4)
        f.write(np.uint32(d + 7).tobytes())
    r = hs.validate_graph(path)
    assert not r["ok"] and r["bad_width_words"] == 1
    with pytest.raises(RuntimeError):
        hs.validate_graph(str(tmp_path / "missing.poe"))


def test_host_loaders_match(tmp_path, capfd):
    import hybrid_search as hs
    import oracle as O
    q = hs._read_fvecs(os.path.join(G, "2wiki_dense_queries_head8.fvecs"))
    assert np.array_equal(q, O.read_fvecs(os.path.join(G, "2wiki_dense_queries_head8.fvecs")))
    off, idx, val = hs._read_csr(os.path.join(G, "2wiki_bm25_queries.bin"), 1000)
    out = capfd.readouterr().out
    assert "Non zero num: 6763" in out
    ooff, oidx, oval = O.read_csr(os.path.join(G, "2wiki_bm25_queries.bin"))
    assert np.array_equal(off, ooff) and np.array_equal(idx, oidx) and np.array_equal(val, oval)
    koff, kidx = hs._read_kg(os.path.join(G, "2wiki_kg.bin"))
    out = capfd.readouterr().out
    assert "Entity num: 30485, Non zero num: 60788" in out
    o2, i2 = O.read_kg(os.path.join(G, "2wiki_kg.bin"))
    assert np.array_equal(koff, o2) and np.array_equal(kidx, i2)
    lines = hs._read_id_lines(os.path.join(G, "2wiki_qrels.txt"), 100)
    assert lines == O.read_id_lines(os.path.join(G, "2wiki_qrels.txt"), 100)
    assert hs._read_id_lines("/nonexistent/qrels.txt", 3) == [[], [], []]
    rng = np.random.default_rng(1)
    rows = rng.integers(0, 50, (50, 40), dtype=np.uint32)
    entry = rng.integers(0, 50, 32, dtype=np.uint32)
    p1, p2 = str(tmp_path / "a.poe"), str(tmp_path / "b.poe")
    hs._write_poe(p1, rows, entry)
    O.write_poe(p2, rows, entry)
    assert open(p1, "rb").read() == open(p2, "rb").read()
    r, e = hs._read_poe(p2)
    assert "Degree: 40,num: 50" in capfd.readouterr().out
    assert np.array_equal(r, rows) and np.array_equal(e, entry)


def test_host_ndcg_matches_oracle():
    import hybrid_search as hs
    import oracle as O
    rng = np.random.default_rng(3)
    res = np.array([rng.permutation(50)[:10] for _ in range(20)], np.uint32)
    gt = [rng.permutation(50)[:rng.integers(1, 6)].tolist() for _ in range(20)]
    a = hs._ndcg(res.tolist(), gt)
    b = O.ndcg(res, gt)
    assert abs(a[0] - b[0]) < 1e-6 and abs(a[1] - b[1]) < 1e-6


def test_host_loader_errors(tmp_path):
    import hybrid_search as hs
    with pytest.raises(RuntimeError, match="open file error"):
        hs._read_fvecs(str(tmp_path / "missing.fvecs"))
    p = str(tmp_path / "short.bin")
    np.array([100, 0, 1], np.uint32).tofile(p)
    with pytest.raises(RuntimeError, match="truncated"):
        hs._read_csr(p, 10)
