"""Small worlds drawn at random (size, graph degree, pair format, pool, weights, launch shape): prune + final rows on
the oracle's lists and searches on the oracle's graph must agree with the oracle whatever the draw. The fixed worlds of
the other tests pin degree 32 and a few pools; this one walks the parameter space (index.cu:539-807, query.cu:488-563)."""
import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("trial", range(8))
def test_random_world_matches_oracle(gpu_ctx, trial):
    import apoe
    import apoe_synth as S
    import oracle as O
    rng = np.random.default_rng(4200 + trial)
    n = int(rng.integers(300, 3000))
    d = int([8, 16, 32, 48, 64, 24, 40, 56][trial])
    seed = int(rng.integers(1, 10 ** 6))
    wide = trial % 2 == 1
    corpus = list(S.to_numpy(S.corpus(n, seed=seed, device="cpu")))
    queries = list(S.to_numpy(S.queries(50, seed=seed + 1, device="cpu")))
    if wide:  # BM25 terms relabelled past 65535: 8-byte pairs on the device
        corpus[5] = corpus[5] + np.uint32(70000)
        queries[5] = queries[5] + np.uint32(70000)
    C, Q = O.HybridSet(*corpus), O.HybridSet(*queries)
    rows, entry, kids, kdist = O.build_index(C, dense_scale=7.0, K=64, iters=5, d=d, seed=seed, return_knn=True)
    gc = apoe.Corpus(gpu_ctx, *corpus)
    gq = apoe.Queries(gpu_ctx, *queries)
    print(f"n {n} degree {d} wide pairs {wide} seed {seed}")

    knn = apoe.Knn(gpu_ctx, gc, 64, 7.0)
    knn.upload(kids, kdist)
    knn.prune(d)
    g_fwd, g_det, g_cnt, _ = knn.prune_download()
    graph = knn.finalize()
    grow, _ = graph.download()
    graph.close()
    knn.close()
    c_fwd, c_det, c_cnt, _ = O.prune(C, 7.0, O.norms(C, 7.0), kids, kdist, d)
    same = np.all(g_fwd == c_fwd, axis=1)
    assert same.mean() >= 0.995, same.mean()
    assert np.array_equal(g_det[same], c_det[same]) and np.array_equal(g_cnt[same], c_cnt[same])
    assert (grow == rows).all(axis=1).mean() >= 0.99

    g = apoe.Graph(gpu_ctx, rows, entry)
    for _ in range(3):
        cands = int(rng.choice([1, 7, 32, 100, 256, 600]))
        w3 = tuple(float(x) for x in rng.choice([0.0, 0.5, 1.0, 2.0], 3))
        if max(w3) < 1e-5:
            w3 = (1.0, 1.0, 1.0)
        variant = int(rng.choice([0, 1, 2, 3])) | (0x100 if rng.integers(0, 4) == 0 else 0)
        ids, dist, _ = apoe.search(gpu_ctx, gc, gq, g, w3, cands, variant=variant)
        oid, odist, _ = O.search(C, Q, rows, entry, w3, cands)
        what = f"cands {cands} weights {w3} variant {variant:#x}"
        assert assert_topk_match(ids, dist, oid, odist, min(10, cands), what) > 0.9, what
        m = ids == oid
        assert_dist_close(dist[m], odist[m], "pool distances, " + what)
    g.close()
    gq.close()
    gc.close()
