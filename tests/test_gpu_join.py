"""The local-join NN-Descent step on the GPU (apoe_knn_set_join) against its oracle restatement and against the
reference-shaped expansion step."""
import numpy as np
import pytest

from parity import assert_dist_close

pytestmark = pytest.mark.gpu


def knn_recall(ids, truth, k):
    return float(np.mean([len(set(ids[i, :k].tolist()) & set(truth[i, :k].tolist())) / k for i in range(len(truth))]))


@pytest.fixture(scope="module")
def exact_knn(small_world):
    import oracle as O
    return O.bruteforce_knn_self(small_world["C"], 7.0, 64)


@pytest.mark.parametrize("K", [64, 128])
@pytest.mark.parametrize("mode", [1, 2])
def test_first_join_step_equals_the_oracle_step(gpu_world, mode, K):
    """From the same random lists (reverse lists empty) a join step is a function of its input: the GPU's lists are
    the oracle's, row for row, except where two float sums that differ in their last bits decide a comparison."""
    import apoe
    import oracle as O
    w = gpu_world
    knn = apoe.Knn(w["ctx"], w["gc"], K, 7.0)
    knn.set_join(mode)
    knn.init(77)
    ins = knn.iterate(last=True)
    ids, dist = knn.download()
    st = O.nnd_init(w["C"].n, K, 77)
    oins, _ = O.join_iterate(w["C"], 7.0, st, slots=2 * K, symmetric=(mode == 2))
    oids = st.ids & 0x7FFFFFFF
    same = np.all(ids == oids, axis=1)
    print(f"mode {mode} K {K}: inserted {ins} (oracle {oins}); identical rows {same.mean():.4f}")
    assert abs(ins - oins) <= 0.001 * oins
    assert same.mean() >= 0.99
    m = ids == oids
    assert_dist_close(dist[m], st.dist[m], "stored distances")
    knn.close()


def test_later_join_steps_follow_the_oracle_steps(gpu_world):
    """K = 128: from the second step on a tile block has its second tile (what the reverse list adds to the list). The first
    step already registers as many reverse entries as the lists hold, so the reverse lists wrap and which entries share a
    slot follows arrival order: the lists are no longer the oracle's row for row, but they insert as much and are as close."""
    import apoe
    import oracle as O
    w = gpu_world
    K = 128
    knn = apoe.Knn(w["ctx"], w["gc"], K, 7.0)
    knn.set_join(1)
    knn.init(78)
    st = O.nnd_init(w["C"].n, K, 78)
    for step in range(3):
        ins = knn.iterate(last=(step == 2))
        oins, _ = O.join_iterate(w["C"], 7.0, st, slots=2 * K)
        ids, dist = knn.download()
        oids = st.ids & 0x7FFFFFFF
        shared = np.mean([len(np.intersect1d(ids[i], oids[i])) / K for i in range(0, len(ids), 7)])
        print(f"K 128 step {step}: inserted {ins} (oracle {oins}); ids shared with the oracle's rows {shared:.4f}; "
              f"mean distance {dist.mean():.4f} (oracle {st.dist.mean():.4f})")
        assert abs(ins - oins) <= 0.02 * oins
        assert shared >= (0.999 if step == 0 else 0.9)
        assert abs(dist.mean() - st.dist.mean()) <= 0.01 * abs(st.dist.mean())
    rev, rev_dist, rev_cnt = knn.download_reverse()
    assert rev_cnt.max() > K  # the reverse lists did wrap
    knn.close()


@pytest.mark.parametrize("K", [64, 128])
@pytest.mark.parametrize("mode", [1, 2])
def test_join_lists_invariants_and_recall(gpu_world, exact_knn, mode, K):
    import apoe
    import oracle as O
    w = gpu_world
    C, n = w["C"], w["C"].n
    knn = apoe.Knn(w["ctx"], w["gc"], K, 7.0)
    knn.set_join(mode)
    knn.init(5)
    ins = [knn.iterate(last=(it == 7)) for it in range(8)]
    knn.merge_reverse()
    ids, dist = knn.download()
    knn.close()
    assert ins[0] > ins[-1] > 0
    assert ids.max() < n and not np.any(ids == np.arange(n)[:, None])
    assert np.all(np.diff(dist, axis=1) >= 0)
    srt = np.sort(ids, axis=1)
    assert not np.any(srt[:, 1:] == srt[:, :-1])
    rows = np.repeat(np.arange(n, dtype=np.uint32), K)
    assert_dist_close(dist.ravel(), O.distance_pairs(C, 7.0, rows, ids.ravel()), "stored = recomputed")
    # list quality: against the oracle's join and against the oracle's expansion step (the reference's algorithm)
    st = O.nnd_init(n, K, 5)
    for it in range(8):
        O.join_iterate(C, 7.0, st, slots=2 * K, symmetric=(mode == 2))  # the join keeps its reverse lists over the steps
    O.nnd_merge_reverse(st)
    se = O.nnd_init(n, K, 5)
    for it in range(8):
        O.nnd_iterate(C, 7.0, se)
        if it < 7:
            se.rev_cnt[:] = 0
    O.nnd_merge_reverse(se)
    ex_ids, _ = exact_knn
    r_g, r_j, r_e = (knn_recall(x, ex_ids, 10) for x in (ids, st.ids & 0x7FFFFFFF, se.ids & 0x7FFFFFFF))
    print(f"mode {mode} K {K}: kNN recall@10 gpu join {r_g:.4f}, oracle join {r_j:.4f}, oracle expansion {r_e:.4f}")
    assert r_g >= r_j - 0.005 and r_g >= r_e - 0.005
