"""Where recall@10 is lost on the synthetic corpus: K-NN list quality against prune + search.

Build order under test: NN-Descent lists -> reverse merge -> RNG-IP prune -> final rows (index.cu:894-903), then the
beam search (query.cu:488-563). Two measurements separate the stages:
  * the lists NN-Descent leaves, against the exact hybrid 64-NN (brute force, build metric 49/1/1) of a node sample,
    at 100 k and 1 M docs;
  * at 100 k docs the exact 64-NN lists of ALL nodes, uploaded and sent through the same prune and the same search:
    what the search reaches on a perfect K-NN graph is the share of the loss that belongs to prune + search.
The figures are printed, and written to $APOE_TEST_REPORT_DIR/recall_split.json when that variable is set; the assertions pin the ordering of the
stages (exact lists are never worse than NN-Descent's, more steps never hurt the lists, every step variant stays in
the band of the others), not absolute values."""
import gc as pygc
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

K = 64


def _list_recall(ids, truth, k):
    return float(np.mean([len(set(ids[i, :k].tolist()) & set(truth[i, :k].tolist())) / k for i in range(len(truth))]))


def _record(key, value):
    out = os.environ.get("APOE_TEST_REPORT_DIR")
    if not out or not os.path.isdir(out):
        return
    path = os.path.join(out, "recall_split.json")
    data = json.load(open(path)) if os.path.exists(path) else {}
    data[key] = value
    json.dump(data, open(path, "w"), indent=1)


def _world(ctx, n, nq):
    import torch
    import apoe
    import apoe_synth as S
    corpus = S.corpus(n, device="cuda:0")
    queries = S.queries(nq, device="cuda:0")
    torch.cuda.synchronize()
    return dict(ctx=ctx, n=n, corpus=corpus, queries=queries, gc=apoe.Corpus(ctx, *corpus), gq=apoe.Queries(ctx, *queries))


def _close(w):
    import torch
    w["gq"].close()
    w["gc"].close()
    w.clear()
    pygc.collect()
    torch.cuda.empty_cache()


def _sample_truth(w, sample):
    """Exact K-NN (build metric) of `sample` nodes drawn without repeats."""
    import torch
    import apoe_bruteforce as B
    g = torch.Generator(device="cpu")
    g.manual_seed(7)
    samp = torch.sort(torch.randperm(w["n"], generator=g)[:sample])[0].to("cuda:0")
    ex, _ = B.hybrid_topk(w["corpus"], B.rows_as_queries(w["corpus"], samp), (49.0, 1.0, 1.0), K, self_ids=samp.cpu().numpy())
    return samp.cpu().numpy(), ex


def _nnd_lists(w, iters, join):
    import apoe
    knn = apoe.Knn(w["ctx"], w["gc"], K, 7.0)
    knn.set_join(join)
    knn.init(1)
    for it in range(iters):
        knn.iterate(last=(it == iters - 1))
    ms = knn.elapsed_ms()
    knn.merge_reverse()
    return knn, ms


def _search_recall(w, graph, truth, pools):
    import apoe
    import apoe_bruteforce as B
    out = {}
    for cands in pools:
        # four expansions per pool entry: the pool, not the reference's 1000-expansion cap, ends the walk
        ids, _, st = apoe.search(w["ctx"], w["gc"], w["gq"], graph, (1.0, 1.0, 1.0), cands, q_count=len(truth), max_iter=4 * cands)
        out[cands] = dict(recall_at_10=B.recall_at_k(ids, truth, 10), evaluations_per_query=st.evaluations / len(truth))
    return out


def test_recall_split_100k(gpu_ctx):
    import apoe
    import apoe_bruteforce as B
    n, degree, pools = 100_000, 32, (128, 512, 2048)
    w = _world(gpu_ctx, n, 2000)
    truth, _ = B.hybrid_topk(w["corpus"], w["queries"], (1.0, 1.0, 1.0), 10, nq=2000)
    samp, ex = _sample_truth(w, 2000)
    res = {}
    for name, iters, join in (("expansion, 10 steps", 10, 0), ("expansion, 25 steps", 25, 0), ("join, 10 steps", 10, 1), ("join, 25 steps", 25, 1),
                              ("symmetric join, 10 steps", 10, 2)):
        knn, ms = _nnd_lists(w, iters, join)
        ids, _ = knn.download()
        knn.prune(degree)
        graph = knn.finalize()
        knn.close()
        res[name] = dict(nnd_seconds=ms / 1e3, list_recall_at_10=_list_recall(ids[samp], ex, 10), list_recall_at_64=_list_recall(ids[samp], ex, K),
                         search=_search_recall(w, graph, truth, pools))
        graph.close()
    # exact lists of all nodes through the same prune and search
    ex_i, ex_d = B.hybrid_topk(w["corpus"], w["corpus"], (49.0, 1.0, 1.0), K, self_ids=np.arange(n), q_block=4096, d_chunk=2048)
    knn = apoe.Knn(gpu_ctx, w["gc"], K, 7.0)
    knn.upload(ex_i.astype(np.uint32), ex_d.astype(np.float32))
    knn.prune(degree)
    graph = knn.finalize()
    knn.close()
    res["exact lists"] = dict(list_recall_at_10=1.0, list_recall_at_64=1.0, search=_search_recall(w, graph, truth, pools))
    graph.close()
    _record("100k docs, degree 32", res)
    print(json.dumps(res))
    _close(w)

    for step in ("expansion", "join"):
        assert res[f"{step}, 25 steps"]["list_recall_at_10"] >= res[f"{step}, 10 steps"]["list_recall_at_10"] - 0.005
    for name, r in res.items():
        for cands in pools:
            # a perfect K-NN graph is the ceiling of every NN-Descent build (one point of sampling noise allowed)
            assert res["exact lists"]["search"][cands]["recall_at_10"] >= r["search"][cands]["recall_at_10"] - 0.01, (name, cands)
        assert r["search"][2048]["recall_at_10"] >= r["search"][512]["recall_at_10"] >= r["search"][128]["recall_at_10"]
    # the join forms the pairs of the expansion step: its lists are as good after the same number of steps
    assert res["join, 10 steps"]["list_recall_at_10"] >= res["expansion, 10 steps"]["list_recall_at_10"] - 0.03
    assert res["symmetric join, 10 steps"]["list_recall_at_10"] >= res["expansion, 10 steps"]["list_recall_at_10"] - 0.03


def test_list_recall_1m(gpu_ctx):
    n = 1_000_000
    w = _world(gpu_ctx, n, 100)
    samp, ex = _sample_truth(w, 2000)
    res = {}
    for name, iters, join in (("expansion, 10 steps", 10, 0), ("join, 10 steps", 10, 1), ("join, 15 steps", 15, 1)):
        knn, ms = _nnd_lists(w, iters, join)
        ids, _ = knn.download()
        knn.close()
        res[name] = dict(nnd_seconds=ms / 1e3, list_recall_at_10=_list_recall(ids[samp], ex, 10), list_recall_at_64=_list_recall(ids[samp], ex, K))
        del ids
    _record("1M docs", res)
    print(json.dumps(res))
    _close(w)
    assert res["join, 10 steps"]["list_recall_at_10"] >= res["expansion, 10 steps"]["list_recall_at_10"] - 0.03
    assert res["join, 15 steps"]["list_recall_at_10"] >= res["join, 10 steps"]["list_recall_at_10"]
    # the lists are far from converged at this size after ten steps (about 0.47 measured): a wide band around that
    assert 0.3 < res["join, 10 steps"]["list_recall_at_10"] < 0.8
