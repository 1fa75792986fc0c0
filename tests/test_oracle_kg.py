"""Oracle KG search pinned on a hand-built knowledge graph (CPU)."""
import numpy as np


def tiny_world():
    import oracle as O
    rng = np.random.default_rng(5)
    n = 40
    dense = rng.standard_normal((n, 1024)).astype(np.float32)
    dense /= np.linalg.norm(dense, axis=1, keepdims=True)
    empty = (np.zeros(n + 1, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    C = O.HybridSet(dense, *empty, *empty)
    q = dense[3:4] * 1.0
    eq = (np.zeros(2, np.uint32), np.zeros(0, np.uint32), np.zeros(0, np.float32))
    Q = O.HybridSet(q, *eq, *eq)
    # graph: a ring over docs 0..19 only (degree 2 padded with self), docs 20..39 unreachable
    d, W = 4, 12
    rows = np.zeros((n, W), np.uint32)
    for v in range(n):
        rows[v, :d] = v
    for v in range(20):
        rows[v, 0] = (v + 1) % 20
        rows[v, 1] = (v - 1) % 20
    entry = np.array([10], np.uint32)
    return C, Q, rows, entry


def test_logical_edge_is_the_only_route():
    """doc 30 is outside the graph; the only route is query entity 0 -> doc 5, entity 0 -> entity 1 -> doc 30."""
    import oracle as O
    C, Q, rows, entry = tiny_world()
    e2e_off = np.array([0, 1, 1], np.uint32)
    e2e_idx = np.array([1], np.uint32)
    e2d_off = np.array([0, 1, 2], np.uint32)
    e2d_idx = np.array([5, 30], np.uint32)
    q2e_off = np.array([0, 1], np.uint32)
    q2e_idx = np.array([0], np.uint32)
    kg = O.Kg(e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx)
    ids, dist, _ = O.search(C, Q, rows, entry, (1, 0, 0), 16, kg=kg, kg_weight=10.0)
    plain, pdist, _ = O.search(C, Q, rows, entry, (1, 0, 0), 16)
    assert 30 not in plain[0].tolist()
    got = ids[0].tolist()
    assert 5 in got and 30 in got
    # closed forms: seed bonus = kg_weight, logical edge at hop 1 = kg_weight / 1
    base = O.distance_batch(C, Q, (1, 0, 0), np.array([[5, 30]], np.uint32))[0]
    assert abs(dist[0][got.index(5)] - (base[0] - 10.0)) < 1e-5
    assert abs(dist[0][got.index(30)] - (base[1] - 10.0 / 1.0)) < 1e-5


def test_hop_limit_and_bonus_decay():
    """chain entity0 -> 1 -> 2 -> 3 -> 4 with docs 21..25: hops 1..3 are reached with bonus kg/hop, hop 4 is not."""
    import oracle as O
    C, Q, rows, entry = tiny_world()
    ne = 5
    e2e_off = np.array([0, 1, 2, 3, 4, 4], np.uint32)
    e2e_idx = np.array([1, 2, 3, 4], np.uint32)
    e2d_off = np.arange(ne + 1, dtype=np.uint32)
    e2d_idx = np.array([21, 22, 23, 24, 25], np.uint32)
    kg = O.Kg(e2e_off, e2e_idx, e2d_off, e2d_idx, np.array([0, 1], np.uint32), np.array([0], np.uint32))
    # graph rows of docs 21.. hold only self loops, i.e. every slot is a recyclable duplicate
    ids, dist, _ = O.search(C, Q, rows, entry, (1, 0, 0), 32, kg=kg, kg_weight=100.0)
    got = ids[0].tolist()
    base = O.distance_batch(C, Q, (1, 0, 0), np.array([[21, 22, 23, 24]], np.uint32))[0]
    assert abs(dist[0][got.index(21)] - (base[0] - 100.0)) < 1e-4
    for doc, hop, b in ((22, 1, base[1]), (23, 2, base[2]), (24, 3, base[3])):
        assert doc in got
        assert abs(dist[0][got.index(doc)] - (b - 100.0 / hop)) < 1e-4
    assert 25 not in got


def test_tiny_kg_weight_without_entities_equals_plain():
    import oracle as O
    C, Q, rows, entry = tiny_world()
    kg = O.Kg(np.zeros(2, np.uint32), np.zeros(0, np.uint32), np.zeros(2, np.uint32), np.zeros(0, np.uint32),
              np.zeros(2, np.uint32), np.zeros(0, np.uint32))
    a, ad, _ = O.search(C, Q, rows, entry, (1, 0, 0), 8, kg=kg, kg_weight=1e-3)
    b, bd, _ = O.search(C, Q, rows, entry, (1, 0, 0), 8)
    assert np.array_equal(a, b) and np.array_equal(ad, bd)
