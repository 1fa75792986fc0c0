"""Oracle keyword-filter search pinned on hand-built cases, on what it must reduce to, and on an
independent list-based simulation of the reference's loop (CPU)."""
import numpy as np

from keyword_worlds import EMPTY_ID, chain_world, make_world, simulate


def test_no_required_keyword_gives_empty_rows():
    import oracle as O
    C, queries, rows, entry = make_world(kw_docs=range(0, 60, 3))
    ids, dist, _ = O.search(C, queries(False), rows, entry, (1, 1, 1), 16, keyword_filter=True)
    assert np.all(ids == EMPTY_ID) and np.all(dist == np.float32(O.INF_DIS))


def test_every_doc_hits_reduces_to_plain_search():
    """All docs hold the keyword and no row has keyword edges: the row starts with the plain search's pool."""
    import oracle as O
    C, queries, rows, entry = make_world(kw_docs=range(60))
    for cands in (8, 16, 64):
        ids, dist, cnt = O.search(C, queries(True), rows, entry, (1, 1, 1), cands, keyword_filter=True)
        pid, pdist, pcnt = O.search(C, queries(False), rows, entry, (1, 1, 1), cands)
        real = pid[0] != EMPTY_ID
        assert np.array_equal(ids[0][real], pid[0][real]) and np.array_equal(dist[0][real], pdist[0][real])
        assert np.array_equal(cnt, pcnt)


def test_rows_hold_only_hits_sorted_with_metric_distances():
    import oracle as O
    kw_docs = set(range(0, 60, 4)) | {13, 27}
    C, queries, rows, entry = make_world(kw_docs=kw_docs)
    Q = queries(True)
    ids, dist, _ = O.search(C, Q, rows, entry, (1, 0.5, 2), 8, keyword_filter=True)
    real = ids[0] != EMPTY_ID
    got = ids[0][real]
    assert len(got) > 0 and set(got.tolist()) <= kw_docs
    assert len(set(got.tolist())) == len(got)
    assert np.all(np.diff(dist[0][real]) >= 0)
    assert real[:real.sum()].all()  # empty slots only at the end
    Qp = queries(False)
    want = O.distance_batch(C, Qp, (1, 0.5, 2), got[None, :])[0]
    assert np.allclose(dist[0][real], want, atol=1e-6)


def test_evicted_hits_survive_whatever_their_id_parity():
    """The reference tests `id & 0x40000000 != 0`, i.e. id & 1: even-id hits would be lost and odd-id
    non-hits kept. With a pool of 4 on a connected 60-doc graph nearly every hit is evicted at some point."""
    import oracle as O
    kw_docs = {2, 4, 10, 16, 22, 31, 44, 58}
    C, queries, rows, entry = make_world(kw_docs=kw_docs, seed=9)
    ids, dist, cnt = O.search(C, queries(True), rows, entry, (1, 1, 1), 4, keyword_filter=True)
    got = set(ids[0][ids[0] != EMPTY_ID].tolist())
    assert got <= kw_docs
    # every hit that was evaluated and ever entered the pool is reported (fewer than 32 exist)
    sim = simulate(C, queries(True), rows, entry, (1, 1, 1), 4)
    assert [i for i, _ in sim] == ids[0][:len(sim)].tolist()
    assert any(i % 2 == 0 for i in got)


def test_keyword_edge_is_the_only_route():
    """Doc 50 is in no graph row; node 5's row lists it as keyword edge and has a duplicate slot."""
    import oracle as O
    n, d = 60, 4
    C, queries, rows, entry = make_world(n=n, kw_docs={50, 7})
    for v in range(n):  # ring over 0..39 only, slots 2,3 = self (always visited: recyclable)
        rows[v, :d] = [(v + 1) % 40, (v - 1) % 40, v, v]
    rows[5, d] = 1
    rows[5, d + 1] = 50
    entry = np.array([0], np.uint32)
    ids, _, _ = O.search(C, queries(True), rows, entry, (1, 1, 1), 64, keyword_filter=True)
    assert 50 in ids[0].tolist() and 7 in ids[0].tolist()
    plain, _, _ = O.search(C, queries(False), rows, entry, (1, 1, 1), 64)
    assert 50 not in plain[0].tolist()
    # without a duplicate slot in the row the keyword edge is not taken
    rows2 = rows.copy()
    rows2[5, :d] = [6, 4, 45, 46]
    rows2[45, :d] = 45
    rows2[46, :d] = 46
    ids2, _, _ = O.search(C, queries(True), rows2, np.array([5], np.uint32), (1, 1, 1), 64, keyword_filter=True, max_iter=1)
    assert 50 not in ids2[0].tolist()
    # a count beyond 7 is clamped to the 7 slots the row has
    rows3 = rows.copy()
    rows3[5, d] = 1000
    ids3, _, _ = O.search(C, queries(True), rows3, entry, (1, 1, 1), 64, keyword_filter=True)
    assert 50 in ids3[0].tolist()


def test_matches_list_simulation_on_random_graphs():
    import oracle as O
    for seed in range(6):
        rng = np.random.default_rng(100 + seed)
        n, d = 80, 6
        kw_docs = set(rng.choice(n, 30, replace=False).tolist())
        C, queries, rows, entry = make_world(n=n, seed=seed, kw_docs=kw_docs, d=d)
        rows[:, :d] = rng.integers(0, n, (n, d))
        rows[:, d] = rng.integers(0, 4, n)
        rows[:, d + 1:] = rng.integers(0, n, (n, 7))
        for cands in (3, 8, 40):
            ids, dist, _ = O.search(C, queries(True), rows, entry, (1, 1, 1), cands, keyword_filter=True)
            sim = simulate(C, queries(True), rows, entry, (1, 1, 1), cands)
            k = len(sim)
            assert ids[0][:k].tolist() == [i for i, _ in sim], (seed, cands)
            assert np.allclose(dist[0][:k], [x for _, x in sim], atol=1e-6)
            assert np.all(ids[0][k:] == EMPTY_ID)


def test_ring_keeps_the_closest_32():
    """Pool of 40 on the chain: docs 0..259 enter at the top and fall off the end one by one, 130 of
    them hits. Closed form: the pool ends as docs 299..260 (hits 298, 296, ..., 260), the ring as the
    last 32 evicted hits 258, 256, ..., 196, of which the row has room for 20."""
    import oracle as O
    C, queries, rows, entry = chain_world()
    ids, dist, cnt = O.search(C, queries(True), rows, entry, (1, 1, 1), 40, keyword_filter=True)
    assert cnt[0, 1] == 300
    assert ids[0].tolist() == list(range(298, 218, -2))
    assert np.all(np.diff(dist[0]) > 0)
    # a pool of 70 leaves room for the whole ring: 35 pool hits, 32 ring entries, 3 empty slots
    ids, dist, cnt = O.search(C, queries(True), rows, entry, (1, 1, 1), 70, keyword_filter=True)
    assert ids[0].tolist() == list(range(298, 228, -2)) + list(range(228, 164, -2)) + [EMPTY_ID] * 3
