import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "allan-poe_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def small_world():
    """4 000 synthetic docs, 200 queries, and an index built by the CPU oracle."""
    import apoe_synth as S
    import oracle as O
    corpus = S.to_numpy(S.corpus(4000, seed=11, device="cpu"))
    queries = S.to_numpy(S.queries(200, seed=12, device="cpu"))
    C = O.HybridSet(*corpus)
    Q = O.HybridSet(*queries)
    rows, entry, knn_ids, knn_dist = O.build_index(C, dense_scale=7.0, K=64, iters=8, d=32, seed=5, return_knn=True)
    return dict(corpus=corpus, queries=queries, C=C, Q=Q, rows=rows, entry=entry, knn_ids=knn_ids, knn_dist=knn_dist)


@pytest.fixture(scope="session")
def gpu_ctx():
    import apoe
    ctx = apoe.Context(0)
    yield ctx
    ctx.close()


@pytest.fixture(scope="session", params=["narrow_pairs", "wide_pairs"])
def gpu_world(request, small_world, gpu_ctx):
    """The small world on the GPU, once per pair format of the device records. The wide form is forced by
    relabelling every BM25 term (corpus and queries alike) past 65535: distances, graphs and searches are
    the same, term for term, so the oracle-built index of the small world serves both."""
    import apoe
    import oracle as O
    w = dict(small_world)
    if request.param == "wide_pairs":
        shift = np.uint32(70000)
        w["corpus"] = w["corpus"][:5] + (w["corpus"][5] + shift,) + w["corpus"][6:]
        w["queries"] = w["queries"][:5] + (w["queries"][5] + shift,) + w["queries"][6:]
        w["C"] = O.HybridSet(*w["corpus"])
        w["Q"] = O.HybridSet(*w["queries"])
    w["ctx"] = gpu_ctx
    w["gc"] = apoe.Corpus(gpu_ctx, *w["corpus"])
    assert w["gc"].pair_bytes() == (8 if request.param == "wide_pairs" else 6)
    w["gq"] = apoe.Queries(gpu_ctx, *w["queries"])
    w["gg"] = apoe.Graph(gpu_ctx, small_world["rows"], small_world["entry"])
    return w
