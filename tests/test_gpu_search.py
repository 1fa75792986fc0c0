"""HIP beam search against the CPU oracle on an identical graph (through the C-ABI)."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match, recall_at_k

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5])
@pytest.mark.parametrize("cands", [32, 128])
def test_search_matches_oracle(gpu_world, cands, variant):
    import apoe
    import oracle as O
    w = gpu_world
    w3 = (1.0, 1.0, 1.0)
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], w3, cands, variant=variant)
    oid, odist, cnt = O.search(w["C"], w["Q"], w["rows"], w["entry"], w3, cands)
    frac = assert_topk_match(ids, dist, oid, odist, 10, f"cands {cands}")
    assert frac > 0.97
    # reported distances are the oracle's distances of those ids
    same = ids == oid
    assert same.mean() > 0.95
    assert_dist_close(dist[same], odist[same], "pool distances")
    # traversal counters agree up to near-tie reorderings
    assert abs(int(st.expansions) - int(cnt[:, 0].sum())) <= 0.01 * cnt[:, 0].sum()
    assert abs(int(st.evaluations) - int(cnt[:, 1].sum())) <= 0.01 * cnt[:, 1].sum()


@pytest.mark.parametrize("w3", [(1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 0.5, 2), (1, 1, 0), (0, 1, 1), (1, 0, 1)])
def test_weight_sweep_without_rebuild(gpu_world, w3):
    import apoe
    import oracle as O
    w = gpu_world
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], w3, 64)
    oid, odist, cnt = O.search(w["C"], w["Q"], w["rows"], w["entry"], w3, 64)
    assert assert_topk_match(ids, dist, oid, odist, 10, f"weights {w3}") > 0.95


def test_rows_sorted_and_unique(gpu_world):
    import apoe
    w = gpu_world
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 128)
    assert np.all(np.diff(dist, axis=1) >= 0)
    for row in ids:
        real = row[row != 0x7FFFFFFF]
        assert len(set(real.tolist())) == len(real)
    assert ids.max() < w["C"].n


def test_recall_monotone_in_cands(gpu_world):
    import apoe
    import oracle as O
    w = gpu_world
    truth, _ = O.bruteforce_topk(w["C"], w["Q"], (1, 1, 1), 10)
    rec = []
    for cands in (16, 64, 256, 512):
        ids, _, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), cands)
        rec.append(recall_at_k(ids, truth, 10))
    assert rec == sorted(rec) and rec[-1] > 0.9, rec


def test_query_range_and_max_iter(gpu_world):
    import apoe
    import oracle as O
    w = gpu_world
    full, fd, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 64)
    part, pd, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 64, q_begin=37, q_count=50)
    assert np.array_equal(part, full[37:87])
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 64, max_iter=5)
    oid, odist, cnt = O.search(w["C"], w["Q"], w["rows"], w["entry"], (1, 1, 1), 64, max_iter=5)
    assert int(st.expansions) == int(cnt[:, 0].sum()) == 5 * w["Q"].n
    assert assert_topk_match(ids, dist, oid, odist, 10, "max_iter 5") > 0.95


def test_bad_graph_ids_are_skipped(gpu_world):
    """Rows holding ids >= n, self loops and duplicates must not fault or repeat."""
    import apoe
    import oracle as O
    w = gpu_world
    rows = w["rows"].copy()
    rows[:, 3] = 0xFFFFFFFF
    rows[:, 4] = rows[:, 5]
    rows[:, 6] = np.arange(rows.shape[0])
    g = apoe.Graph(w["ctx"], rows, w["entry"])
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], g, (1, 1, 1), 64)
    oid, odist, _ = O.search(w["C"], w["Q"], rows, w["entry"], (1, 1, 1), 64)
    assert assert_topk_match(ids, dist, oid, odist, 10, "bad ids") > 0.95
    g.close()


@pytest.mark.parametrize("cands", [1, 7, 100, 2048])
def test_pool_sizes_at_the_edges(gpu_world, cands):
    """Pools of one entry, of sizes that are no multiple of a wave, and of the largest size the library takes
    (more than the 1 000 iterations can explore) against the oracle; one more is refused."""
    import apoe
    import oracle as O
    w = gpu_world
    nq = 60
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), cands, q_count=nq)
    oid, odist, cnt = O.search(w["C"], w["Q"].head(nq), w["rows"], w["entry"], (1, 1, 1), cands)
    assert ids.shape == (nq, cands)
    k = min(10, cands)
    assert assert_topk_match(ids, dist, oid, odist, k, f"cands {cands}") > 0.95
    assert np.all(np.diff(dist, axis=1) >= 0)
    assert abs(int(st.evaluations) - int(cnt[:, 1].sum())) <= 0.01 * cnt[:, 1].sum()
    if cands == 2048:
        with pytest.raises(apoe.ApoeError, match="cands"):
            apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), cands + 1, q_count=nq)


def test_large_pool_picks_its_shape_and_unknown_shapes_are_refused(gpu_world):
    """With the default shape a pool of 2048 entries runs with four waves per query (fewer queries fit a CU): the rows
    are those of the two-wave launch. A shape code that does not exist is an error, not a silent default."""
    import apoe
    w = gpu_world
    a = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 1.0, 1.0), 2048, max_iter=4096, variant=0)
    b = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 1.0, 1.0), 2048, max_iter=4096, variant=4)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    assert a[2].evaluations == b[2].evaluations
    with pytest.raises(RuntimeError, match="launch shape"):
        apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 1.0, 1.0), 32, variant=9)
