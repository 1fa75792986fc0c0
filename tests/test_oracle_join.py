"""Pins the oracle's local-join NN-Descent step (orc_join_iterate) with an independent Python restatement,
determinism across thread counts, invariants and brute-force recall (CPU)."""
import numpy as np
import pytest

FLAG = 0x80000000
EMPTY = 0xFFFFFFFF
M64 = (1 << 64) - 1


def mix64(z):
    z = (z + 0x9E3779B97F4A7C15) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def py_join_step(O, C, scale, st, P, symmetric):
    """One step, written from the definition in apoe_oracle.h with dictionaries and lists."""
    n, K = st.ids.shape
    ids, dist = st.ids.copy(), st.dist.copy()
    rev, rev_dist, rev_cnt = st.rev.copy(), st.rev_dist.copy(), st.rev_cnt.copy()
    start_ids = ids & ~np.uint32(FLAG)
    picks = []
    for u in range(n):
        slots = []
        for g in range(4):
            s = g
            while s < K and ids[u, s] & FLAG:
                s += 1
            if s >= K:
                s = 0
            else:
                ids[u, s] |= FLAG
            if s not in slots:
                slots.append(s)
        picks.append([int(ids[u, s] & ~np.uint32(FLAG)) for s in slots])
    pairs = []
    for u in range(n):
        for v in picks[u]:
            cand = set(int(x) for x in start_ids[v]) | set(int(x) for x in rev[v] if x != EMPTY)
            for c in sorted(cand):
                if c != u and c < n:
                    pairs.append((u, c))
    pa = np.array(pairs, dtype=np.uint32)
    d = O.distance_pairs(C, scale, pa[:, 0], pa[:, 1])
    own = [set(int(x) for x in start_ids[u]) for u in range(n)]
    worst = dist[:, K - 1].copy()
    prop = {}

    def offer(node, cid, dv):
        key = (node, (mix64(cid) >> 40) & (P - 1))
        if key not in prop or (dv, cid) < prop[key]:
            prop[key] = (dv, cid)

    for (u, c), dv in zip(pairs, d):
        if c not in own[u] and dv < worst[u]:
            offer(u, c, dv)
        if symmetric and dv < worst[c]:
            offer(c, u, dv)
    inserted = 0
    for x in range(n):
        fresh = sorted(v for (node, _), v in prop.items() if node == x and v[1] != x and v[1] not in own[x])
        if not fresh:
            continue
        old = [(dist[x, j], int(ids[x, j])) for j in range(K)]
        merged, i, j = [], 0, 0
        while len(merged) < K:
            if i < len(fresh) and (j >= K or fresh[i][0] <= old[j][0]):
                merged.append((fresh[i][0], fresh[i][1], True))
                i += 1
            else:
                merged.append((old[j][0], old[j][1], False))
                j += 1
        ins = sum(1 for m in merged if m[2])
        inserted += ins
        for t, m in enumerate(merged):
            dist[x, t], ids[x, t] = m[0], m[1]
        if ins:
            for m in merged:
                if not m[2]:
                    continue  # an entry registers once, when it enters the list
                v = m[1] & ~FLAG
                slot = int(rev_cnt[v])
                rev_cnt[v] += 1
                if slot < K or m[0] < rev_dist[v, slot % K]:
                    rev[v, slot % K], rev_dist[v, slot % K] = x, m[0]
    return inserted, ids, dist, rev, rev_dist, rev_cnt


@pytest.fixture(scope="module")
def world():
    import apoe_synth as S
    import oracle as O
    return O.HybridSet(*S.to_numpy(S.corpus(260, seed=77, device="cpu")))


@pytest.mark.parametrize("symmetric", [False, True])
def test_two_steps_equal_the_python_restatement(world, symmetric):
    import oracle as O
    C = world
    st = O.nnd_init(C.n, 16, 3)
    for step in range(2):  # the second step has reverse lists to read
        want = py_join_step(O, C, 7.0, st, 16, symmetric)
        ins, evals = O.join_iterate(C, 7.0, st, slots=16, symmetric=symmetric, threads=1)
        assert ins == want[0] and evals > 0
        assert np.array_equal(st.ids, want[1]) and np.array_equal(st.dist, want[2])
        assert np.array_equal(st.rev_cnt, want[5])
        assert np.array_equal(st.rev, want[3]) and np.array_equal(st.rev_dist, want[4])  # the reverse lists are kept over the steps


def test_first_step_does_not_depend_on_the_thread_count(world):
    import oracle as O
    C = world
    a, b = O.nnd_init(C.n, 16, 5), O.nnd_init(C.n, 16, 5)
    ia, _ = O.join_iterate(C, 7.0, a, slots=16, symmetric=True, threads=1)
    ib, _ = O.join_iterate(C, 7.0, b, slots=16, symmetric=True, threads=8)
    assert ia == ib and np.array_equal(a.ids, b.ids) and np.array_equal(a.dist, b.dist)
    # the same registrations were made (which of them a full reverse list keeps follows arrival order, as in the reference)
    assert np.array_equal(a.rev_cnt, b.rev_cnt)


@pytest.mark.parametrize("symmetric", [False, True])
def test_join_lists_invariants_and_recall(symmetric):
    import apoe_synth as S
    import oracle as O
    C = O.HybridSet(*S.to_numpy(S.corpus(1200, seed=101, device="cpu")))
    n = C.n
    st, se = O.nnd_init(n, 64, 9), O.nnd_init(n, 64, 9)
    for it in range(8):
        O.join_iterate(C, 7.0, st, slots=64, symmetric=symmetric)
        O.nnd_iterate(C, 7.0, se)
        if it < 7:
            se.rev_cnt[:] = 0  # the expansion step starts its reverse lists again with every step (index.cu:896), the join keeps them
    O.nnd_merge_reverse(st)
    O.nnd_merge_reverse(se)
    ids, dist = st.ids & 0x7FFFFFFF, st.dist
    assert np.all(np.diff(dist, axis=1) >= 0)
    assert not np.any(ids == np.arange(n, dtype=np.uint32)[:, None])
    srt = np.sort(ids, axis=1)
    assert not np.any(srt[:, 1:] == srt[:, :-1])
    a = np.repeat(np.arange(n, dtype=np.uint32), 64)
    assert np.allclose(dist.ravel(), O.distance_pairs(C, 7.0, a, ids.ravel()), rtol=1e-6)
    truth, _ = O.bruteforce_knn_self(C, 7.0, 64)

    def rec(x):
        return float(np.mean([len(set(x[i, :10].tolist()) & set(truth[i, :10].tolist())) / 10 for i in range(n)]))
    r_join, r_exp = rec(ids), rec(se.ids & 0x7FFFFFFF)
    # the join meets the pairs that the reference's expansion step meets: its lists are as good
    assert r_join > 0.95 and r_join >= r_exp - 0.005, (r_join, r_exp)
