"""Hand-built worlds that pin single branches of the prune and of the knowledge-graph search
(shared by the CPU oracle tests and the GPU parity tests). Every expected value below is
worked out by hand in the comments, not computed by the code under test."""
import numpy as np

INF_DIS = 1000000.0


def _csr(rows):
    off, idx, val = [0], [], []
    for r in rows:
        for t in sorted(r):
            idx.append(t)
            val.append(r[t])
        off.append(len(idx))
    return np.array(off, np.uint32), np.array(idx, np.uint32), np.array(val, np.float32)


def keyword_flag_world(K=64, term_shift=0):
    """12 documents; node 0 is the centre u with the hand-made list 1,2,3,4,10,6,7,11,9,5,8 (ascending
    made-up distances), every other list is empty, so every detour count is 0 and the selection
    (index.cu:612-692) visits the candidates in list order. Dense rows are 0.1 * e_i: no dense overlap,
    49 * 0.01 = 0.49 of squared norm under the x7 build scale. No SPLADE terms. BM25 rows
    (term: value); u = doc 0 holds the terms 100..103:

        0: 100 101 102 103 (1 each), 900:3          norm 0.49 + 4 + 9
        1: 100:1, 901:3                              norm 10.49
        2: 101:1, 902:3
        3: 100:1, 101:1, 903:3
        4: 102:1, 904:3
        5: 905:3                                     no term of u
        6: 100:1, 101:1, 102:1, 906:3, 910:2         <6,10> = 2 > norm(10) = 1.49: tombstones 10
        7: 100:1, 907:3
        8: 103:1, 908:3
        9: 103:1, 909:3
        10: 910:1                                    norm 1.49, no term of u
        11: 901:1                                    norm 1.49; <11,1> = 3 > 1.49: rejected

    All other inner products are at most 2 against norms of at least 9.49, so nothing else is
    rejected or tombstoned. Degree d = 4: the row is 1,2,3,4; what lives beyond it, in order: 6,7,9,5,8.
    Keyword flag of c (index.cu:128-153,637,651-666) = every selected member s that is live when c is
    compared has a BM25 term that u holds and c lacks:
        10: flagged (members 1..4 each hold one of 100..102), but it dies, so it is not emitted
        6:  member 1 holds only 100 of u's terms and 6 has it            -> not flagged
        7:  member 1 again                                               -> not flagged
        9:  live members 1,2,3,4,6,7 (10 is dead: it holds no term of u and would veto) all
            hold one of 100..102, 9 holds only 103                       -> FLAGGED
        5:  live members 1,2,3,4,6,7,9 hold 100..103, 5 holds none       -> FLAGGED
        8:  member 9 holds only 103 of u's terms and 8 has it            -> not flagged
    Expected: fwd[0] = 1,2,3,4; cnt[0] = 4; kw[0] = (2; 9, 5).

    What a wrong flag rule gives instead: "any member" flags 7 too; candidate and member swapped drops 5;
    dead members counted drops 9 and 5; u's term set ignored flags 8 as well.
    term_shift relabels every BM25 term (past 65535: the wide pair format of the device records)."""
    n = 12
    dense = np.zeros((n, 1024), np.float32)
    for i in range(n):
        dense[i, i] = 0.1
    bm = [
        {100: 1, 101: 1, 102: 1, 103: 1, 900: 3},
        {100: 1, 901: 3},
        {101: 1, 902: 3},
        {100: 1, 101: 1, 903: 3},
        {102: 1, 904: 3},
        {905: 3},
        {100: 1, 101: 1, 102: 1, 906: 3, 910: 2},
        {100: 1, 907: 3},
        {103: 1, 908: 3},
        {103: 1, 909: 3},
        {910: 1},
        {901: 1},
    ]
    bm = [{t + term_shift: v for t, v in r.items()} for r in bm]
    empty = (np.zeros(n + 1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    arrays = (dense,) + empty + _csr(bm)
    order = [1, 2, 3, 4, 10, 6, 7, 11, 9, 5, 8]
    ids = np.empty((n, K), np.uint32)
    for v in range(n):
        ids[v, :] = (v + 1) % n  # a valid id at INF_DIS = an empty slot
    dist = np.full((n, K), INF_DIS, np.float32)
    ids[0, :len(order)] = order
    dist[0, :len(order)] = 0.01 * np.arange(1, len(order) + 1, dtype=np.float32)
    expect = dict(fwd0=[1, 2, 3, 4], cnt0=4, kw0=[9, 5], d=4)
    return arrays, ids, dist, expect


def kg_fresh_neighbour_world():
    """40 documents with random unit dense rows and no sparse terms; the query is doc 3's dense row.
    Graph: a ring over docs 0..19 (slots 0,1 = next, previous; slots 2,3 = the node itself), docs
    20..39 are not in the graph. One entry point, doc 10. Entities:

        query -> entity 0;  e2doc[0] = {5}
        e2e[0] = (1, 2)     e2doc[1] = {6}   e2doc[2] = {6}
        e2e[1] = (3)        e2doc[3] = {7, 30}
        e2e[2] = (4)        e2doc[4] = {31}

    Walk (kg_weight 10 dwarfs every plain distance, which lies in (-0.2, 1.2)):
      seeds: doc 5 (entity 0, hop 0, bonus 10) and the entry point 10 (no entity).
      expand 5: row = 6, 4, 5, 5. Docs 6 and 4 are fresh graph neighbours at hop 1. Branch (i)
        (query.cu:1699-1715): 6 is a document of entity 1 AND of entity 2, both neighbours of the
        parent's entity 0: it is a logical neighbour, gets the bonus 10/1, and carries the FIRST
        linking entity, 1. Doc 4 is a document of no neighbour entity: plain distance, no entity.
        The two slots that repeat 5 are recycled (ii): entity 1 offers {6}, entity 2 offers {6},
        both visited: nothing.
      expand 6 (entity 1, hop 1): row = 7, 5, 6, 6. Doc 7 is fresh and a document of entity 3, the
        neighbour of entity 1: bonus 10/2, entity 3. First recycled slot -> entity 3 -> its first
        unvisited document 30: bonus 10/2. (Had 6 carried entity 2, the walk would tag nothing here and
        reach 31 through entity 4 instead of 30.)
      expand 7 and 30 (entity 3, hop 2): entity 3 has no neighbours. Doc 8 follows at hop 3 with no
        entity, and so on round the ring.
    Expected with cands 32: dist(6) = plain - 10, dist(7) = plain - 5, dist(30) = plain - 5,
    dist(4) = plain, 31 absent."""
    rng = np.random.default_rng(5)
    n = 40
    dense = rng.standard_normal((n, 1024)).astype(np.float32)
    dense /= np.linalg.norm(dense, axis=1, keepdims=True)
    empty = (np.zeros(n + 1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    corpus = (dense,) + empty + empty
    eq = (np.zeros(2, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    queries = (dense[3:4].copy(),) + eq + eq
    d, W = 4, 12
    rows = np.zeros((n, W), np.uint32)
    for v in range(n):
        rows[v, :d] = v
    for v in range(20):
        rows[v, 0] = (v + 1) % 20
        rows[v, 1] = (v - 1) % 20
    entry = np.array([10], np.uint32)
    e2e_off = np.array([0, 2, 3, 4, 4, 4], np.uint32)
    e2e_idx = np.array([1, 2, 3, 4], np.uint32)
    e2d_off = np.array([0, 1, 2, 3, 5, 6], np.uint32)
    e2d_idx = np.array([5, 6, 6, 7, 30, 31], np.uint32)
    q2e_off = np.array([0, 1], np.uint32)
    q2e_idx = np.array([0], np.uint32)
    kg = (e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx)
    # doc -> bonus divisor (0 = no bonus); 5 is a seed of the query's own entity (bonus kg_weight)
    expect = dict(bonus={5: 1.0, 6: 1.0, 7: 2.0, 30: 2.0, 4: 0.0, 8: 0.0, 10: 0.0}, absent=[31], kg_weight=10.0, cands=32)
    return corpus, queries, rows, entry, kg, expect


def check_kg_fresh_neighbour(ids, dist, plain, expect):
    """ids/dist: the result row of the one query; plain[doc] = hybrid distance without any bonus."""
    got = ids.tolist()
    for doc, div in expect["bonus"].items():
        assert doc in got, f"doc {doc} missing from the row"
        want = plain[doc] - (expect["kg_weight"] / div if div else 0.0)
        assert abs(float(dist[got.index(doc)]) - want) < 1e-4, (doc, float(dist[got.index(doc)]), want)
    for doc in expect["absent"]:
        assert doc not in got, f"doc {doc} reached"


def merge_reverse_closed_form(n, K, ids, dist, rev, rev_dist, rev_cnt):
    """index.cu:386-478 as a closed form: a node's new list = the first K of (its list) + (its registered
    reverse entries: the first min(K, count) slots, without the node itself, ids out of range, ids the
    list already holds, and repeats of an id, of which the closest stays), ordered by distance with the
    reverse entries before list entries on equal distance and by id among themselves. ids carry the
    sampled flag in bit 31, which list entries keep and new ones lack."""
    out_ids, out_dist = ids.copy(), dist.copy()
    for u in range(n):
        have = set((ids[u] & 0x7FFFFFFF).tolist())
        best = {}
        for j in range(min(K, int(rev_cnt[u]))):
            r = int(rev[u, j])
            if r == 0xFFFFFFFF or r >= n or r == u or r in have:
                continue
            if r not in best or rev_dist[u, j] < best[r]:
                best[r] = rev_dist[u, j]
        if not best:
            continue
        entries = [(float(dd), 1, j, int(i)) for j, (i, dd) in enumerate(zip(ids[u], dist[u]))]
        entries += [(float(dd), 0, r, r) for r, dd in best.items()]
        entries.sort(key=lambda e: (e[0], e[1], e[2]))
        out_ids[u] = [e[3] for e in entries[:K]]
        out_dist[u] = [e[0] for e in entries[:K]]
    return out_ids, out_dist
