"""Pins the oracle's build stages (N1-N3, P1-P3, S5, nDCG) with brute force and invariants (CPU)."""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def tiny():
    import apoe_synth as S
    import oracle as O
    arrays = S.to_numpy(S.corpus(1200, seed=101, device="cpu"))
    C = O.HybridSet(*arrays)
    st = O.nnd_init(C.n, 64, 9)
    init_ids = st.ids.copy()
    inserted = []
    for it in range(8):
        inserted.append(O.nnd_iterate(C, 7.0, st, threads=1))
        if it < 7:
            st.rev_cnt[:] = 0
    before = (st.ids.copy() & 0x7FFFFFFF, st.dist.copy())
    O.nnd_merge_reverse(st)
    ids, dist = st.ids & 0x7FFFFFFF, st.dist.copy()
    exact = O.bruteforce_knn_self(C, 7.0, 64)
    nrm = O.norms(C, 7.0)
    pr = O.prune(C, 7.0, nrm, ids, dist, 32)
    rows = O.final_graph(*pr)
    return dict(C=C, init_ids=init_ids, inserted=inserted, before=before, ids=ids, dist=dist, exact=exact, norms=nrm, prune=pr, rows=rows)


def test_init_is_deterministic_and_in_range(tiny):
    import oracle as O
    st = O.nnd_init(tiny["C"].n, 64, 9)
    assert np.array_equal(st.ids, tiny["init_ids"])
    assert st.ids.max() < tiny["C"].n
    assert st.ids[3, 5] == O.lib().orc_rand_id(9, 3 * 64 + 5, tiny["C"].n)
    other = O.nnd_init(tiny["C"].n, 64, 10)
    assert not np.array_equal(other.ids, st.ids)


def test_single_thread_iteration_is_deterministic(tiny):
    import oracle as O
    C = tiny["C"]
    a, b = O.nnd_init(C.n, 64, 9), O.nnd_init(C.n, 64, 9)
    ia, ib = O.nnd_iterate(C, 7.0, a, threads=1), O.nnd_iterate(C, 7.0, b, threads=1)
    assert ia == ib and np.array_equal(a.ids, b.ids) and np.array_equal(a.dist, b.dist)


def test_nnd_invariants_and_recall(tiny):
    import oracle as O
    C = tiny["C"]
    for ids, dist in (tiny["before"], (tiny["ids"], tiny["dist"])):
        assert np.all(np.diff(dist, axis=1) >= 0)
        assert not np.any(ids == np.arange(C.n, dtype=np.uint32)[:, None])
        srt = np.sort(ids, axis=1)
        assert not np.any(srt[:, 1:] == srt[:, :-1])
        a = np.repeat(np.arange(C.n, dtype=np.uint32), 64)
        assert np.allclose(dist.ravel(), O.distance_pairs(C, 7.0, a, ids.ravel()), rtol=1e-6)
    assert np.all(tiny["dist"] <= tiny["before"][1])
    truth = tiny["exact"][0]
    rec = np.mean([len(set(tiny["ids"][i, :10].tolist()) & set(truth[i, :10].tolist())) / 10 for i in range(C.n)])
    assert rec > 0.95, rec
    ins = tiny["inserted"]
    assert ins[0] == C.n * 64 and ins[-1] < ins[1]


def test_detour_counts_match_bruteforce(tiny):
    ids, dist = tiny["ids"], tiny["dist"]
    fwd, det, cnt, kw = tiny["prune"]
    for u in (0, 17, 600, 1199):
        want = {}
        for s in range(64):
            c = 0
            for r in range(s):
                lr = ids[ids[u, r]].tolist()
                if ids[u, s] in lr and dist[ids[u, r], lr.index(ids[u, s])] < dist[u, s]:
                    c += 1
            want[int(ids[u, s])] = c
        for j in range(cnt[u]):
            assert det[u, j] == want[int(fwd[u, j])]


def test_prune_selection_rules(tiny):
    """Re-derive the selection of a few nodes from the metric alone."""
    import oracle as O
    C, ids, nrm = tiny["C"], tiny["ids"], tiny["norms"]
    fwd, det, cnt, kw = tiny["prune"]
    n = C.n
    assert np.all(cnt == 32)  # 64 candidates, few dominated pairs on this data
    for u in (1, 250, 777):
        # detour order (stable) of the candidates
        detour = {}
        for s in range(64):
            c = 0
            for r in range(s):
                lr = ids[ids[u, r]].tolist()
                if ids[u, s] in lr and tiny["dist"][ids[u, r], lr.index(ids[u, s])] < tiny["dist"][u, s]:
                    c += 1
            detour[s] = c
        order = sorted(range(64), key=lambda s: (detour[s], s))
        cand = [int(ids[u, s]) for s in order]
        def bm(i):
            return set(C.b_idx[C.b_off[i]:C.b_off[i + 1]].tolist())

        sel, live, flagged = [cand[0]], [True], [False]
        for c in cand[1:]:
            reject, all_flag = False, True
            for i, s in enumerate(sel):
                if not live[i]:
                    continue
                p = np.float32(1.0) - O.distance_pairs(C, 7.0, np.array([c], np.uint32), np.array([s], np.uint32))[0]
                if not ((bm(s) & bm(u)) - bm(c)):  # no term that the member shares with u and the candidate lacks
                    all_flag = False
                if nrm[c] < p:
                    reject = True
                if nrm[s] < p:
                    live[i] = False
            if not reject:
                sel.append(c)
                live.append(True)
                flagged.append(all_flag)
        survivors = [s for s, l in zip(sel, live) if l]
        assert fwd[u].tolist() == survivors[:32]
        alive = [(s, f) for s, l, f in zip(sel, live, flagged) if l]
        want_kw = [s for s, f in alive[32:] if f][:32]
        assert kw[u, 1:1 + kw[u, 0]].tolist() == want_kw
    # surviving pairs satisfy <s1,s2> <= min(norm) among the first rows
    for u in range(0, n, 97):
        r = fwd[u, :cnt[u]]
        a, b = np.meshgrid(r, r)
        ip = 1.0 - O.distance_pairs(C, 7.0, a.ravel().astype(np.uint32), b.ravel().astype(np.uint32)).reshape(len(r), len(r))
        lim = np.minimum(nrm[a], nrm[b])
        off_diag = ~np.eye(len(r), dtype=bool)
        assert np.all(ip[off_diag] <= lim[off_diag] * (1 + 1e-5))


def test_final_rows_layout(tiny):
    fwd, det, cnt, kw = tiny["prune"]
    rows = tiny["rows"]
    n, d = fwd.shape
    assert rows.shape == (n, d + 8)
    assert np.array_equal(rows[:, :d // 2], fwd[:, :d // 2])
    assert np.all(rows[:, d] <= 7)
    # reverse half: in-neighbours by (detour, id), not in the first half
    inn = {v: [] for v in range(n)}
    for u in range(n):
        for j in range(cnt[u]):
            inn[int(fwd[u, j])].append((int(det[u, j]), u))
    for v in range(0, n, 29):
        first = set(rows[v, :d // 2].tolist())
        want = [u for _, u in sorted(inn[v]) if u not in first][:d // 2]
        got = rows[v, d // 2:d // 2 + len(want)].tolist()
        assert got == want
        body = [x for x in rows[v, :d].tolist() if x != v]
        assert len(set(body)) == len(body)
        c = rows[v, d]
        assert np.all(rows[v, d + 1 + c:] == 0)
        assert not (set(rows[v, d + 1:d + 1 + c].tolist()) & set(rows[v, d // 2:d].tolist()))
        assert set(rows[v, d + 1:d + 1 + c].tolist()) <= set(kw[v, 1:1 + kw[v, 0]].tolist())


def test_entry_points_are_smallest_norms(tiny):
    import oracle as O
    nrm = tiny["norms"]
    ep = O.entry_points(nrm, 32)
    assert np.array_equal(ep, np.lexsort((np.arange(len(nrm)), nrm))[:32])


def test_calibration_closed_form(small_world):
    import oracle as O
    C, Q = small_world["C"], small_world["Q"]
    mx = np.full(3, -np.inf)
    for i in range(100):
        for j in range(100):
            mx = np.maximum(mx, O.ip_parts(C, i, Q, j))
    w = O.calibrate(C, Q, Q.n, (1.0, 2.0, 0.5))
    big = int(np.argmax(mx))
    want = np.array([1.0, 2.0, 0.5], np.float64)
    for p in range(3):
        if p != big:
            want[p] *= mx[big] / mx[p]
    assert np.allclose(w, want, rtol=1e-5)
    # a zero user weight stays zero and switches the path off
    w0 = O.calibrate(C, Q, Q.n, (0.0, 1.0, 1.0))
    assert w0[0] == 0.0


def test_ndcg_hand_examples():
    import oracle as O
    # one query, 2 relevant docs, found at ranks 1 and 3 of 4
    res = np.array([[7, 1, 9, 4]], np.uint32)
    nd, rec = O.ndcg(res, [[7, 9]])
    idcg = 1 / np.log2(2) + 1 / np.log2(3)
    dcg = 1 / np.log2(2) + 1 / np.log2(4)
    assert abs(nd - dcg / idcg) < 1e-6 and rec == 1.0
    nd, rec = O.ndcg(res, [[5, 6]])
    assert nd == 0.0 and rec == 0.0
    # IDCG runs over ALL ground-truth ids even beyond k (query.cu:116-119)
    nd, rec = O.ndcg(np.array([[1, 2]], np.uint32), [[1, 2, 3, 4]])
    idcg = sum(1 / np.log2(j + 2) for j in range(4))
    assert abs(nd - (1 / np.log2(2) + 1 / np.log2(3)) / idcg) < 1e-6 and rec == 0.5
