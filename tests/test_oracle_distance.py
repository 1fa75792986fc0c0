"""Pins the oracle's hybrid metric (D1-D4, N0) against library routines and closed forms (CPU)."""
import numpy as np
import scipy.sparse as sp


def _csr(off, idx, val, n, vocab):
    return sp.csr_matrix((val.astype(np.float64), idx.astype(np.int64), off.astype(np.int64)), shape=(n, vocab))


def test_distance_equals_dense_gemv_plus_csr_products(small_world):
    import apoe_synth as S
    import oracle as O
    C, Q = small_world["C"], small_world["Q"]
    Cs, Cb = _csr(C.s_off, C.s_idx, C.s_val, C.n, S.VOCAB), _csr(C.b_off, C.b_idx, C.b_val, C.n, S.VOCAB)
    Qs, Qb = _csr(Q.s_off, Q.s_idx, Q.s_val, Q.n, S.VOCAB), _csr(Q.b_off, Q.b_idx, Q.b_val, Q.n, S.VOCAB)
    dense = Q.dense.astype(np.float64) @ C.dense.astype(np.float64).T
    spl = (Qs @ Cs.T).toarray()
    bm = (Qb @ Cb.T).toarray()
    ids = np.tile(np.arange(C.n, dtype=np.uint32), (Q.n, 1))
    for w in [(1, 1, 1), (1, 0.5, 2), (0, 1, 0), (0, 0, 1), (1, 0, 0), (3, 1e-6, 2)]:
        on = [x >= 1e-5 for x in w]
        want = 1 - (w[0] * dense * on[0] + w[1] * spl * on[1] + w[2] * bm * on[2])
        got = O.distance_batch(C, Q, w, ids)
        assert np.max(np.abs(got - want) / np.maximum(1, np.abs(want))) < 1e-6, w
    # per-path parts (compute_hybrid_dis)
    p = O.ip_parts(C, 7, Q, 3)
    assert np.allclose(p, [dense[3, 7], spl[3, 7], bm[3, 7]], rtol=1e-5, atol=1e-6)
    # brute-force top-k = argsort of the closed form
    want = 1 - (dense + spl + bm)
    bi, bd = O.bruteforce_topk(C, Q, (1, 1, 1), 10)
    assert np.array_equal(bi, np.argsort(want, axis=1, kind="stable")[:, :10])


def test_build_metric_and_norms(small_world):
    import apoe_synth as S
    import oracle as O
    C = small_world["C"]
    Cs, Cb = _csr(C.s_off, C.s_idx, C.s_val, C.n, S.VOCAB), _csr(C.b_off, C.b_idx, C.b_val, C.n, S.VOCAB)
    rng = np.random.default_rng(0)
    a = rng.integers(0, C.n, 500).astype(np.uint32)
    b = rng.integers(0, C.n, 500).astype(np.uint32)
    d64 = C.dense.astype(np.float64)
    want = 1 - (49.0 * np.einsum("ij,ij->i", d64[a], d64[b]) + np.asarray(Cs[a].multiply(Cs[b]).sum(1)).ravel()
                + np.asarray(Cb[a].multiply(Cb[b]).sum(1)).ravel())
    got = O.distance_pairs(C, 7.0, a, b)
    assert np.max(np.abs(got - want) / np.maximum(1, np.abs(want))) < 1e-6
    nrm = O.norms(C, 7.0)
    self_d = O.distance_pairs(C, 7.0, a, a)
    assert np.allclose(1 - nrm[a], self_d, rtol=1e-6)
    # dense rows are unit length: norm = 49 + |s|^2 + |b|^2
    s2 = np.asarray(Cs.multiply(Cs).sum(1)).ravel()
    b2 = np.asarray(Cb.multiply(Cb).sum(1)).ravel()
    assert np.allclose(nrm, 49.0 * (d64 ** 2).sum(1) + s2 + b2, rtol=1e-6)


def test_special_cases():
    import oracle as O
    dense = np.zeros((3, 1024), np.float32)
    dense[0, 0] = 1.0
    dense[1, 0] = 0.5
    dense[2, 1] = 2.0
    s_off = np.array([0, 2, 4, 5], np.uint32)
    s_idx = np.array([3, 9, 9, 11, 4], np.uint32)
    s_val = np.array([2.0, 3.0, 5.0, 7.0, 1.0], np.float32)
    b_off = np.array([0, 1, 1, 2], np.uint32)
    b_idx = np.array([9, 9], np.uint32)  # same id as a SPLADE term: the two vocabularies never mix
    b_val = np.array([10.0, 4.0], np.float32)
    C = O.HybridSet(dense, s_off, s_idx, s_val, b_off, b_idx, b_val)
    ids = np.tile(np.arange(3, dtype=np.uint32), (3, 1))
    got = O.distance_batch(C, C, (1, 1, 1), ids)
    # doc0.doc1: dense 0.5, single shared SPLADE term 9 -> 15, no BM25 overlap
    assert got[0, 1] == np.float32(1 - (0.5 + 15.0))
    # doc0.doc2: disjoint SPLADE sets, BM25 term 9 shared -> 40, dense orthogonal
    assert got[0, 2] == np.float32(1 - 40.0)
    # doc1.doc2: nothing shared at all
    assert got[1, 2] == np.float32(1.0)
    assert np.allclose(got, got.T)
    assert got[0, 0] == np.float32(1 - (1 + 4 + 9 + 100))
