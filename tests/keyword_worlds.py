"""Small hand-built worlds for the keyword-filter search tests (shared by the CPU and GPU suites)."""
import numpy as np

KW = 0x80000000
EMPTY_ID = 0x7FFFFFFF


def make_world(n=60, seed=3, kw_docs=(), d=4):
    """Random dense rows; every doc has BM25 terms {1 + (v % 7)} (value 0.1), docs in kw_docs also
    term 40. Query: BM25 terms 3 and 40, term 40 flagged as required keyword."""
    import oracle as O
    rng = np.random.default_rng(seed)
    dense = rng.standard_normal((n, 1024)).astype(np.float32)
    dense /= np.linalg.norm(dense, axis=1, keepdims=True)
    b_off, b_idx, b_val = [0], [], []
    for v in range(n):
        terms = [1 + (v % 7)] + ([40] if v in kw_docs else [])
        b_idx += terms
        b_val += [0.1] * len(terms)
        b_off.append(len(b_idx))
    empty = (np.zeros(n + 1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    C = O.HybridSet(dense, *empty, np.array(b_off, np.uint32), np.array(b_idx, np.uint32), np.array(b_val, np.float32))
    q = rng.standard_normal((1, 1024)).astype(np.float32)
    q /= np.linalg.norm(q)
    eq = (np.zeros(2, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))

    def queries(flag):
        return O.HybridSet(q, *eq, np.array([0, 2], np.uint32), np.array([3, 40 | (KW if flag else 0)], np.uint32),
                           np.array([0.5, 0.25], np.float32))
    W = d + 8
    rows = np.zeros((n, W), np.uint32)
    for v in range(n):
        rows[v, :d] = [(v + 1) % n, (v - 1) % n, (v + 7) % n, (v * 3 + 1) % n, (v + 11) % n, (v * 5 + 2) % n][:d]
    entry = np.array([0, n // 2], np.uint32)
    return C, queries, rows, entry


def simulate(C, Q, rows, entry, w3, cands, max_iter=1000):
    """The loop of query.cu:1271-1483 with plain Python lists: visited set, pool as a list of
    dicts kept sorted by re-sorting (stable, new entries placed before old ones on equal
    distance), evicted hits appended worst first to a list of which the last 32 survive."""
    import oracle as O
    n, W = rows.shape
    d = W - 8
    q_idx = Q.b_idx[Q.b_off[0]:Q.b_off[1]]
    required = {int(t & 0x7FFFFFFF) for t in q_idx if t & KW}
    Qp = O.HybridSet(Q.dense, Q.s_off, Q.s_idx, Q.s_val, Q.b_off, Q.b_idx & 0x7FFFFFFF, Q.b_val)
    all_d = O.distance_batch(C, Qp, w3, np.arange(n, dtype=np.uint32)[None, :])[0]

    def hit(c):
        return bool(required & set(C.b_idx[C.b_off[c]:C.b_off[c + 1]].tolist()))
    visited, pool, evicted = set(), [], []

    def merge(fresh):
        nonlocal pool
        fresh = sorted(fresh, key=lambda e: (e["dist"], e["id"]))
        merged = sorted([dict(e, new=0) for e in fresh] + [dict(e, new=1) for e in pool], key=lambda e: (e["dist"], e["new"]))
        keep, drop = merged[:cands], merged[cands:]
        for e in reversed([e for e in drop if e["new"] == 1 and e["hit"]]):  # worst first
            evicted.append(e)
        pool = [{k: e[k] for k in ("id", "dist", "hit", "done")} for e in keep]

    fresh = []
    for e in entry.tolist():
        if e < n and e not in visited:
            visited.add(e)
            fresh.append(dict(id=e, dist=float(all_d[e]), hit=hit(e), done=False))
    merge(fresh)
    for _ in range(max_iter):
        nxt = next((e for e in pool if not e["done"]), None)
        if nxt is None:
            break
        nxt["done"] = True
        row = rows[nxt["id"]]
        fresh, dup = [], 0
        for c in row[:d].tolist():
            if c >= n or c in visited:
                dup += 1
                continue
            visited.add(c)
            fresh.append(dict(id=c, dist=float(all_d[c]), hit=hit(c), done=False))
        for t in range(min(dup, min(int(row[d]), 7))):
            c = int(row[d + 1 + t])
            if c >= n or c in visited:
                continue
            visited.add(c)
            fresh.append(dict(id=c, dist=float(all_d[c]), hit=hit(c), done=False))
        merge(fresh)
    out = [(e["id"], e["dist"]) for e in pool if e["hit"]]
    out += sorted([(e["id"], e["dist"]) for e in evicted[-32:]], key=lambda t: (t[1], t[0]))
    return out[:cands]


def chain_world(n=300):
    """Doc v lies at dense inner product 0.1*v with the query and links to v+1, so the search walks
    0, 1, 2, ... and every new doc is better than everything seen before. Even docs hold the keyword."""
    import oracle as O
    C, queries, rows, entry = make_world(n=n, kw_docs=range(0, n, 2), seed=21)
    dense = np.zeros((n, 1024), np.float32)
    dense[:, 0] = 0.1 * np.arange(n)
    C = O.HybridSet(dense, C.s_off, C.s_idx, C.s_val, C.b_off, C.b_idx, C.b_val)
    q = np.zeros((1, 1024), np.float32)
    q[0, 0] = 1.0

    def chain_queries(flag):
        Q = queries(flag)
        return O.HybridSet(q, Q.s_off, Q.s_idx, Q.s_val, Q.b_off, Q.b_idx, Q.b_val)
    for v in range(n):
        rows[v, :4] = [min(v + 1, n - 1), max(v - 1, 0), v, v]
    return C, chain_queries, rows, np.array([0], np.uint32)
