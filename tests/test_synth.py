"""The synthetic-world generator (CPU): one seed is one world, whatever back end or chunking makes it."""
import numpy as np
import pytest

import apoe_synth as S


def _same(a, b):
    assert len(a) == len(b)
    for x, y in zip(a, b):
        x, y = x.numpy(), y.numpy()
        assert x.dtype == y.dtype and x.shape == y.shape
        assert np.array_equal(x.view(np.uint32) if x.dtype == np.float32 else x, y.view(np.uint32) if y.dtype == np.float32 else y)


def test_numpy_and_torch_integer_arithmetic_give_the_same_bits():
    _same(S.corpus(700, seed=3, force_backend="numpy"), S.corpus(700, seed=3, device="cpu", force_backend="torch"))
    _same(S.queries(300, seed=4, force_backend="numpy"), S.queries(300, seed=4, device="cpu", force_backend="torch"))
    _same(S.knowledge_graph(5000, 700, 300, seed=5, force_backend="numpy"), S.knowledge_graph(5000, 700, 300, seed=5, device="cpu", force_backend="torch"))


def test_mix64_matches_the_python_integer_definition():
    X = S.backend("cpu", "numpy")
    idx = np.array([0, 1, 2, 0xFFFFFFFFFFFFFFFF, 0x123456789ABCDEF0], dtype=np.uint64)
    want = [S.mix64_int(int(i)) for i in idx]
    assert [int(v) for v in X.mix(idx)] == want
    # known answers of splitmix64 seeded with 0: its outputs are mix(0), mix(gamma), mix(2 * gamma) with the golden gamma
    assert want[0] == 0xE220A8397B1DCDAF
    assert S.mix64_int(0x9E3779B97F4A7C15) == 0x6E789E6AA1B965F4


def test_a_world_does_not_depend_on_the_chunking():
    a = S.sparse_rows(1000, 60, "bm25", 9, chunk=1 << 18)
    b = S.sparse_rows(1000, 60, "bm25", 9, chunk=137)
    _same(a, b)
    _same((S.dense_rows(300, 9, chunk=1 << 14),), (S.dense_rows(300, 9, chunk=77),))
    # a prefix of a larger world is the smaller world
    big, small = S.corpus(500, seed=21), S.corpus(200, seed=21)
    assert np.array_equal(big[0][:200].numpy(), small[0].numpy())
    e = int(small[1][-1])
    assert np.array_equal(big[2][:e].numpy(), small[2].numpy()) and np.array_equal(big[3][:e].numpy(), small[3].numpy())


def test_distributions():
    n = 20000
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(S.corpus(n, seed=1))
    assert np.allclose(np.linalg.norm(dense.astype(np.float64), axis=1), 1.0, atol=1e-6)
    x = dense[:2000].ravel().astype(np.float64) * 32.0           # components ~ N(0, 1/1024)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1.0) < 0.01
    assert abs(np.mean(np.abs(x) > 1.96) - 0.05) < 0.003          # normal tails, not a uniform sum
    nnz_s, nnz_b = np.diff(s_off.astype(np.int64)), np.diff(b_off.astype(np.int64))
    assert abs(nnz_s.mean() - 120) < 2 and abs(nnz_b.mean() - 60) < 1.5
    for off, idx in ((s_off, s_idx), (b_off, b_idx)):
        rows = np.repeat(np.arange(n), np.diff(off.astype(np.int64)))
        key = rows.astype(np.int64) * S.VOCAB + idx
        assert np.all(np.diff(key) > 0) and idx.max() < S.VOCAB  # ascending and distinct inside every row
    # Zipf(1.1): a draw is term r with probability p_r, so a row of m draws holds it with probability 1 - (1 - p_r)^m
    p, _ = S.zipf_tables()
    m = S.draws_for_unique(60)
    df = np.bincount(b_idx, minlength=S.VOCAB) / n
    for r in (0, 5, 50, 500):
        want = 1 - (1 - p[r]) ** m
        assert abs(df[r] - want) < 0.02 + 0.1 * want, (r, df[r], want)
    logs = np.log(s_val.astype(np.float64))
    assert abs(logs.mean()) < 0.01 and abs(logs.std() - 0.5) < 0.01  # log-normal(0, 0.5)
    assert b_val.min() >= 0.5 and b_val.max() <= 8.0 and abs(b_val.mean() - 4.25) < 0.02
    q = S.to_numpy(S.queries(5000, seed=2))
    assert abs(np.diff(q[1].astype(np.int64)).mean() - 30) < 1 and abs(np.diff(q[4].astype(np.int64)).mean() - 8) < 0.5


def test_latent_world_has_the_structure_it_names():
    n = 3000
    a = S.latent_corpus(n, seed=41, world=43, force_backend="numpy")
    _same(a, S.latent_corpus(n, seed=41, world=43, device="cpu", force_backend="torch"))
    _same(S.latent_queries(300, seed=42, world=43, force_backend="numpy"), S.latent_queries(300, seed=42, world=43, device="cpu", force_backend="torch"))
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = S.to_numpy(a)
    assert np.allclose(np.linalg.norm(dense.astype(np.float64), axis=1), 1.0, atol=1e-6)
    hid = S.hidden_of_rows(S.backend("cpu", "numpy"), 41, 0, n).astype(np.float64)
    assert hid.shape == (n, S.LATENT_DIM) and abs(hid.std() - 16.0) < 0.5
    hn = hid / np.linalg.norm(hid, axis=1)[:, None]
    iu = np.triu_indices(n, 1)
    cos_h, cos_d = (hn @ hn.T)[iu], (dense.astype(np.float64) @ dense.astype(np.float64).T)[iu]
    assert np.corrcoef(cos_h, cos_d)[0, 1] > 0.9                   # the dense row follows the hidden vector ...
    near = cos_h > 0.8
    assert near.sum() > 20 and 0.3 < cos_d[near].mean() < 0.6      # ... at about half its cosine: the other half is the row's own noise
    assert abs(cos_d[np.abs(cos_h) < 0.05].mean()) < 0.01
    # the terms are those of the structureless corpus of the same seed; their values follow the rarity of the term
    plain = S.to_numpy(S.corpus(n, seed=41))
    assert np.array_equal(s_off, plain[1]) and np.array_equal(s_idx, plain[2]) and np.array_equal(b_off, plain[4]) and np.array_equal(b_idx, plain[5])
    f = S.rarity_table(60, "bm25")
    assert f[0] < 1e-3 < 0.5 < f[1000] < f[20000] and np.all(b_val <= f[b_idx] * (1 + 1e-6)) and np.all(b_val >= 0.3 * f[b_idx] * (1 - 1e-6))
    assert np.all(S.rarity_table(120, "splade") <= S.LATENT_SCALE * (1 + 1e-6))
    # without a world the generator stays the structureless one
    assert not np.array_equal(S.to_numpy(S.corpus(50, seed=41))[0], dense[:50])


def test_knowledge_graph_shape():
    e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx = S.to_numpy(S.knowledge_graph(50000, 10000, 2000, seed=8))
    deg = np.diff(e2e_off.astype(np.int64))
    assert deg.min() >= 1 and deg.max() <= 4096 and 3.0 < deg.mean() < 9.0   # heavy tail: the sample mean sits below 8
    assert np.mean(deg == 1) > 0.4 and np.mean(deg >= 100) > 1e-4
    ddeg = np.diff(e2d_off.astype(np.int64))
    assert ddeg.min() >= 1 and abs(ddeg.mean() - 3.0) < 0.05
    qdeg = np.diff(q2e_off.astype(np.int64))
    assert set(np.unique(qdeg)) == {1, 2, 3}
    assert e2e_idx.max() < 50000 and e2d_idx.max() < 10000 and q2e_idx.max() < 50000


@pytest.mark.gpu
def test_gpu_world_is_the_host_world():
    """float64 sqrt and divide are correctly rounded on the GPU too: the device-made world has the host-made bits."""
    _same(S.corpus(3000, seed=31), [t.cpu() for t in S.corpus(3000, seed=31, device="cuda:0")])
    _same(S.queries(500, seed=32), [t.cpu() for t in S.queries(500, seed=32, device="cuda:0")])
    _same(S.knowledge_graph(20000, 3000, 500, seed=33), [t.cpu() for t in S.knowledge_graph(20000, 3000, 500, seed=33, device="cuda:0")])
    _same(S.latent_corpus(2000, seed=34, world=35), [t.cpu() for t in S.latent_corpus(2000, seed=34, world=35, device="cuda:0")])
