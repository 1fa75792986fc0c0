"""The benchmark configurations at their full sizes (one MI355X): 1 M docs / degree 48 with the pool sweep and the
query-time weight sweep, the same world with a 200 k-entity knowledge graph, and 8 M docs / degree 64 / 100 k queries.
The oracle checks a query sample on the GPU-built graph; everything else goes through properties that do not depend
on the size: rows sorted and free of repeats, every reported distance recomputed by the independent distance kernel,
the bounded evaluation bit-equal to reading every dense row, launch shapes in agreement."""
import gc as pygc

import numpy as np
import pytest

from parity import assert_dist_close, assert_topk_match

pytestmark = pytest.mark.gpu

EMPTY_ID = 0x7FFFFFFF
WEIGHTS = ((1.0, 0.0, 0.0), (0.0, 1.0, 0.0), (0.0, 0.0, 1.0), (1.0, 1.0, 1.0), (1.0, 0.5, 2.0))


def _free():
    import torch
    pygc.collect()
    torch.cuda.empty_cache()


def _check_rows(ids_t, dist_t, n_docs):
    """Properties of result rows held as torch tensors on the GPU: ascending distances, ids in range, no id twice."""
    import torch
    assert bool((dist_t[:, 1:] >= dist_t[:, :-1]).all())
    real = ids_t != EMPTY_ID
    assert bool(real[:, :10].all())
    assert int(ids_t[real].max()) < n_docs
    srt, _ = torch.sort(torch.where(real, ids_t, torch.arange(ids_t.shape[1], device=ids_t.device)[None, :] + (1 << 30)), dim=1)
    assert bool((srt[:, 1:] != srt[:, :-1]).all())


def _search_dev(apoe, w, w3, cands, **kw):
    import torch
    nq = kw.get("q_count") or w["gq"].n
    ids = torch.empty((nq, cands), dtype=torch.int32, device="cuda:0")
    dist = torch.empty((nq, cands), dtype=torch.float32, device="cuda:0")
    _, _, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], w3, cands, out_ids=ids, out_dist=dist, **kw)
    return ids, dist, st


# ---- config 2 and 3: 1 M docs, degree 48 ----

@pytest.fixture(scope="module")
def world1m(gpu_ctx):
    import torch
    import apoe
    import apoe_synth as S
    n, nq = 1_000_000, 10_000
    corpus = S.corpus(n, device="cuda:0")
    queries = S.queries(nq, device="cuda:0")
    torch.cuda.synchronize()
    gc = apoe.Corpus(gpu_ctx, *corpus)
    gq = apoe.Queries(gpu_ctx, *queries)
    graph, ms = apoe.build_graph(gpu_ctx, gc, K=64, iters=10, degree=48, seed=1, join=1)
    w = dict(ctx=gpu_ctx, n=n, corpus=corpus, queries=queries, gc=gc, gq=gq, graph=graph, build_ms=ms)
    yield w
    graph.close()
    gq.close()
    gc.close()
    w.clear()
    del corpus, queries
    _free()


def test_config2_graph_is_well_formed(world1m):
    w = world1m
    rows, entry = w["graph"].download()
    w["rows"], w["entry"] = rows, entry
    assert rows.shape == (w["n"], 56) and len(entry) == 48 and len(set(entry.tolist())) == 48
    nb = rows[:, :48]
    assert nb.max() < w["n"]
    assert rows[:, 48].max() <= 7 and rows[:, 49:].max() < w["n"]
    half = np.sort(nb[:, :24], axis=1)
    assert (np.diff(half.astype(np.int64), axis=1) != 0).mean() > 0.999
    print(f"1M docs, degree 48: build {w['build_ms'] / 1e3:.2f} s of GPU time")


@pytest.mark.parametrize("cands", [64, 128, 256])
def test_config2_pool_and_weight_sweep_properties(world1m, cands):
    import torch
    import apoe
    w = world1m
    for w3 in WEIGHTS:
        ids, dist, st = _search_dev(apoe, w, w3, cands)
        _check_rows(ids, dist, w["n"])
        ids2, dist2, st2 = _search_dev(apoe, w, w3, cands, variant=0x100)
        assert torch.equal(ids, ids2) and torch.equal(dist, dist2), f"bounded evaluation changed a row, weights {w3}"
        assert st.evaluations == st2.evaluations and st.dense_rows <= st2.dense_rows
        # reported distances against the independent distance kernel, on a slice of the batch
        sl = slice(0, 256)
        got_i, got_d = ids[sl].cpu().numpy().view(np.uint32), dist[sl].cpu().numpy()
        real = got_i != EMPTY_ID
        q256 = apoe.Queries(w["ctx"], *_head(w["queries"], 256))
        again = apoe.distance_batch(w["ctx"], w["gc"], q256, w3, np.where(real, got_i, 0).astype(np.uint32))
        q256.close()
        assert_dist_close(got_d[real], again[real], f"cands {cands}, weights {w3}")
    ids, dist, _ = _search_dev(apoe, w, (1.0, 1.0, 1.0), cands)
    ids4, dist4, _ = _search_dev(apoe, w, (1.0, 1.0, 1.0), cands, variant=2)
    agree = assert_topk_match(ids[:500].cpu().numpy().view(np.uint32), dist[:500].cpu().numpy(), ids4[:500].cpu().numpy().view(np.uint32),
                              dist4[:500].cpu().numpy(), 10, "launch shapes")
    assert agree > 0.99


def _head(arrays, k):
    """The first k rows of a hybrid set of torch tensors."""
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = arrays
    se, be = int(s_off[k]), int(b_off[k])
    return (dense[:k], s_off[:k + 1], s_idx[:se], s_val[:se], b_off[:k + 1], b_idx[:be], b_val[:be])


def test_config2_oracle_sample(world1m):
    import apoe
    import apoe_synth as S
    import oracle as O
    w = world1m
    if "rows" not in w:
        w["rows"], w["entry"] = w["graph"].download()
    C = O.HybridSet(*S.to_numpy(w["corpus"]))
    w["C"] = C
    nq = 100
    Q = O.HybridSet(*S.to_numpy(_head(w["queries"], nq)))
    for w3, cands in (((1.0, 1.0, 1.0), 128), ((1.0, 0.5, 2.0), 256), ((0.0, 0.0, 1.0), 64)):
        ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], w3, cands, q_count=nq)
        oid, odist, _ = O.search(C, Q, w["rows"], w["entry"], w3, cands)
        assert assert_topk_match(ids, dist, oid, odist, 10, f"1M docs, weights {w3}") > 0.97
        same = ids == oid
        assert same.mean() > 0.95
        assert_dist_close(dist[same], odist[same], "pool distances")


def test_config3_knowledge_graph_200k_entities(world1m):
    import torch
    import apoe
    import apoe_synth as S
    import oracle as O
    w = world1m
    kg = S.knowledge_graph(200_000, w["n"], w["gq"].n, device="cuda:0")
    gkg = apoe.KnowledgeGraph(w["ctx"], *kg)
    cands = 128
    ids = torch.empty((w["gq"].n, cands), dtype=torch.int32, device="cuda:0")
    dist = torch.empty((w["gq"].n, cands), dtype=torch.float32, device="cuda:0")
    _, _, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["graph"], (1.0, 1.0, 1.0), cands, kg=gkg, kg_weight=40.0, out_ids=ids, out_dist=dist)
    _check_rows(ids, dist, w["n"])
    assert st.evaluations > 0
    # the knowledge graph changes what is found: documents of the query's entities carry the bonus
    ids_p, dist_p, _ = _search_dev(apoe, w, (1.0, 1.0, 1.0), cands)
    assert float((dist[:, 0] <= dist_p[:, 0]).float().mean()) > 0.9
    # oracle on a sample
    if "rows" not in w:
        w["rows"], w["entry"] = w["graph"].download()
    C = w.get("C") or O.HybridSet(*S.to_numpy(w["corpus"]))
    nq = 100
    Q = O.HybridSet(*S.to_numpy(_head(w["queries"], nq)))
    kg_np = S.to_numpy(kg)
    q2e_off, q2e_idx = kg_np[4], kg_np[5]
    okg = O.Kg(kg_np[0], kg_np[1], kg_np[2], kg_np[3], q2e_off[:nq + 1].copy(), q2e_idx[:int(q2e_off[nq])].copy())
    oid, odist, _ = O.search(C, Q, w["rows"], w["entry"], (1.0, 1.0, 1.0), cands, kg=okg, kg_weight=40.0)
    got_i, got_d = ids[:nq].cpu().numpy().view(np.uint32), dist[:nq].cpu().numpy()
    assert assert_topk_match(got_i, got_d, oid, odist, 10, "KG search, 1M docs") > 0.95
    gkg.close()


# ---- config 4: 8 M docs, degree 64, 100 k queries, cands 256 ----

def test_config4_8m_docs_degree64(gpu_ctx):
    import torch
    import apoe
    import apoe_synth as S
    _free()
    n, nq, cands = 8_000_000, 100_000, 256
    corpus = S.corpus(n, seed=808, device="cuda:0")
    queries = S.queries(nq, seed=809, device="cuda:0")
    torch.cuda.synchronize()
    gc = apoe.Corpus(gpu_ctx, *corpus)
    assert gc.bytes() > 40e9  # record offsets beyond 32 bits are in use
    del corpus
    _free()
    gq = apoe.Queries(gpu_ctx, *queries)
    graph, ms = apoe.build_graph(gpu_ctx, gc, K=64, iters=10, degree=64, seed=1, join=1, expansion_first=1)
    print(f"8M docs, degree 64: build {ms / 1e3:.1f} s of GPU time")
    w = dict(ctx=gpu_ctx, gc=gc, gq=gq, graph=graph, queries=queries)
    ids, dist, st = _search_dev(apoe, w, (1.0, 1.0, 1.0), cands)
    print(f"8M docs: {nq} queries at cands {cands}: {st.kernel_ms:.0f} ms, {st.evaluations / nq:.0f} evaluations per query")
    _check_rows(ids, dist, n)
    ids2, dist2, st2 = _search_dev(apoe, w, (1.0, 1.0, 1.0), cands, variant=0x100, q_count=20_000)
    assert torch.equal(ids[:20_000], ids2) and torch.equal(dist[:20_000], dist2)
    got_i, got_d = ids[:128].cpu().numpy().view(np.uint32), dist[:128].cpu().numpy()
    q128 = apoe.Queries(gpu_ctx, *_head(queries, 128))
    again = apoe.distance_batch(gpu_ctx, gc, q128, (1.0, 1.0, 1.0), got_i)
    q128.close()
    assert_dist_close(got_d, again, "8M docs: reported distances")
    # documents from all over the corpus are found, the last million included
    assert int(ids.max()) > 7_000_000
    # the static workspace of apoe_search_noalloc is sized for 2 M documents: a larger corpus is refused
    with pytest.raises(apoe.ApoeError, match="up to"):
        apoe.search_noalloc(gpu_ctx, gc, gq, graph, (1.0, 1.0, 1.0), 64, ids[:, :64].contiguous(), dist[:, :64].contiguous())
    rows, entry = graph.download()
    assert rows.shape == (n, 72) and rows[:, :64].max() < n
    graph.close()
    gq.close()
    gc.close()
    del ids, dist, ids2, dist2, rows
    _free()
