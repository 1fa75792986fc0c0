"""HIP knowledge-graph search (seeding + logical-edge expansion) against the CPU oracle."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kg_world(gpu_world):
    import apoe
    import apoe_synth as S
    import oracle as O
    w = gpu_world
    kg = S.to_numpy(S.knowledge_graph(1500, w["C"].n, w["Q"].n, seed=21, device="cpu", mean_out=6.0))
    out = dict(w)
    out["kg_arrays"] = kg
    out["okg"] = O.Kg(*kg)
    out["gkg"] = apoe.KnowledgeGraph(w["ctx"], *kg)
    return out


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("cands,kg_weight", [(64, 40.0), (128, 5.0), (32, 400.0)])
def test_kg_search_matches_oracle(kg_world, cands, kg_weight, variant):
    import apoe
    import oracle as O
    w = kg_world
    w3 = (1.0, 1.0, 1.0)
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], w3, cands, kg=w["gkg"], kg_weight=kg_weight, variant=variant)
    oid, odist, cnt = O.search(w["C"], w["Q"], w["rows"], w["entry"], w3, cands, kg=w["okg"], kg_weight=kg_weight)
    frac = assert_topk_match(ids, dist, oid, odist, 10, f"kg cands {cands}")
    assert frac > 0.97
    same = ids == oid
    assert same.mean() > 0.95
    assert_dist_close(dist[same], odist[same], "kg pool distances")
    assert abs(int(st.evaluations) - int(cnt[:, 1].sum())) <= 0.01 * cnt[:, 1].sum()


def test_kg_bonus_changes_results(kg_world):
    """The KG bonus must matter: entity documents of a query appear in its results."""
    import apoe
    w = kg_world
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 64, kg=w["gkg"], kg_weight=1000.0)
    e2d_off, e2d_idx, q2e_off, q2e_idx = w["kg_arrays"][2], w["kg_arrays"][3], w["kg_arrays"][4], w["kg_arrays"][5]
    hit = 0
    for q in range(w["Q"].n):
        docs = set()
        for e in q2e_idx[q2e_off[q]:q2e_off[q + 1]]:
            docs |= set(e2d_idx[e2d_off[e]:e2d_off[e + 1]].tolist())
        hit += len(docs & set(ids[q].tolist())) == len(docs)
    assert hit >= 0.99 * w["Q"].n


def test_kg_without_entities_equals_plain_search(kg_world):
    import apoe
    w = kg_world
    nq = w["Q"].n
    empty = (np.zeros(2, np.uint32), np.zeros(0, np.uint32), np.zeros(2, np.uint32), np.zeros(0, np.uint32),
             np.zeros(nq + 1, np.uint32), np.zeros(0, np.uint32))
    gkg = apoe.KnowledgeGraph(w["ctx"], *empty)
    a, ad, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 64, kg=gkg, kg_weight=40.0)
    b, bd, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1, 1, 1), 64)
    assert np.array_equal(a, b) and np.array_equal(ad, bd)
    gkg.close()
