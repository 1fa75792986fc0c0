"""Corpora smaller than, or barely larger than, a neighbour list (K = 64): the random lists then hold repeats and the
node itself, and a document that already sits in a list as a random entry (distance at the empty mark) is never offered
again (index.cu:262-283 drops candidates that are in the list), so with n <= K the steps have nothing to evaluate and
the lists keep their empty marks: that is the algorithm, the oracle does the same. Build, prune, final rows and search
must run on such corpora with every step kind, give rows that name documents only, and agree with the oracle."""
import numpy as np
import pytest

from parity import assert_topk_match

pytestmark = pytest.mark.gpu

INF = np.float32(1.0e5)  # stored distances of empty slots are 1e6
STEPS = 12


def _world(ctx, n, nq=20):
    import apoe
    import apoe_synth as S
    import oracle as O
    corpus = S.to_numpy(S.corpus(n, seed=900 + n, device="cpu"))
    queries = S.to_numpy(S.queries(nq, seed=950 + n, device="cpu"))
    return dict(C=O.HybridSet(*corpus), Q=O.HybridSet(*queries), gc=apoe.Corpus(ctx, *corpus), gq=apoe.Queries(ctx, *queries))


def _oracle_lists(C, join):
    import oracle as O
    st = O.nnd_init(C.n, 64, 3)
    for it in range(STEPS):
        if join:
            O.join_iterate(C, 7.0, st, slots=128, symmetric=(join == 2))
        else:
            O.nnd_iterate(C, 7.0, st)
            if it < STEPS - 1:
                st.rev_cnt[:] = 0  # index.cu:896
    O.nnd_merge_reverse(st)
    return st.ids & 0x7FFFFFFF, st.dist


@pytest.mark.parametrize("join", [0, 1, 2])
@pytest.mark.parametrize("n", [2, 3, 40, 65, 130, 300])
def test_build_and_search_on_a_tiny_corpus(gpu_ctx, n, join):
    import apoe
    import oracle as O
    w = _world(gpu_ctx, n)
    knn = apoe.Knn(gpu_ctx, w["gc"], 64, 7.0)
    knn.set_join(join)
    knn.init(3)
    for it in range(STEPS):
        knn.iterate(last=(it == STEPS - 1))
    knn.merge_reverse()
    ids, dist = knn.download()
    valid = dist < INF
    for i in range(n):
        mine = ids[i][valid[i]]
        assert len(set(mine.tolist())) == len(mine) and i not in mine and (mine < n).all(), (n, i)
        assert np.all(np.diff(dist[i][valid[i]]) >= 0)
    assert ids.max() < n
    # as many evaluated neighbours per list as the oracle's run of the same steps finds (the steps are asynchronous:
    # counts, not rows)
    oids, odist = _oracle_lists(w["C"], join)
    got, want = valid.sum(axis=1).mean(), (odist < INF).sum(axis=1).mean()
    print(f"n {n} step kind {join}: evaluated neighbours per list {got:.1f} (oracle {want:.1f})")
    assert abs(got - want) <= max(2.0, 0.15 * want), (got, want)
    if n >= 130:
        k = 10
        ex_ids, _ = O.bruteforce_knn_self(w["C"], 7.0, k)
        hit = np.mean([len(set(ids[i, :k].tolist()) & set(ex_ids[i].tolist())) / k for i in range(n)])
        ohit = np.mean([len(set(oids[i, :k].tolist()) & set(ex_ids[i].tolist())) / k for i in range(n)])
        print(f"  list recall@10 {hit:.3f} (oracle {ohit:.3f})")
        assert hit >= ohit - 0.05
    # prune, final rows, search: rows name documents only; the search agrees with the oracle on the same rows
    knn.prune(32)
    graph = knn.finalize()
    knn.close()
    rows, entry = graph.download()
    assert rows[:, :32].max() < n and entry.max() < n
    gi, gd, _ = apoe.search(gpu_ctx, w["gc"], w["gq"], graph, (1.0, 1.0, 1.0), 64)
    oi, od, _ = O.search(w["C"], w["Q"], rows, entry, (1.0, 1.0, 1.0), 64)
    assert_topk_match(gi, gd, oi, od, min(10, n), f"n {n}")
    graph.close()
    w["gq"].close()
    w["gc"].close()
