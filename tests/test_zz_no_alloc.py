"""apoe_search_noalloc (static device workspace, no allocation) against apoe_search, through the C-ABI (needs the GPU).

Two calls in a row on the same GPU, the second with a smaller input: the workspace keeps what the first call left
there, so the second call shows that everything that must start at zero is cleared. Results must be bit-equal:
both entry points run the same kernels on the same graph, and a query's walk does not depend on the grid."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def world(small_world, gpu_ctx):
    """The small world on the GPU (not the parametrized session fixture: pytest would move these tests up
    to run them with that fixture's first parameter, and they are meant to run last)."""
    import apoe
    w = dict(small_world)
    w["ctx"] = gpu_ctx
    w["gc"] = apoe.Corpus(gpu_ctx, *w["corpus"])
    w["gq"] = apoe.Queries(gpu_ctx, *w["queries"])
    w["gg"] = apoe.Graph(gpu_ctx, small_world["rows"], small_world["entry"])
    yield w
    for k in ("gg", "gq", "gc"):
        w[k].close()


def _both(w, cands, q_begin, q_count, **kw):
    import torch
    import apoe
    ids, dist, st = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 1.0, 1.0), cands, q_begin=q_begin, q_count=q_count, **kw)
    nq = ids.shape[0]
    out_ids = torch.full((nq, cands), -1, dtype=torch.int32, device="cuda:0")
    out_dist = torch.full((nq, cands), -1.0, dtype=torch.float32, device="cuda:0")
    st2 = apoe.search_noalloc(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 1.0, 1.0), cands, out_ids, out_dist, q_begin=q_begin, q_count=q_count, **kw)
    return ids, dist, st, out_ids.cpu().numpy().view(np.uint32), out_dist.cpu().numpy(), st2


def test_noalloc_equals_search_twice_in_a_row(world):
    w = world
    ids, dist, st, ids2, dist2, st2 = _both(w, 128, 0, 0)
    assert np.array_equal(ids, ids2) and np.array_equal(dist.view(np.uint32), dist2.view(np.uint32))
    assert (st.expansions, st.evaluations, st.dense_rows, st.algo_bytes) == (st2.expansions, st2.evaluations, st2.dense_rows, st2.algo_bytes)
    # second call, smaller input: fewer queries, a smaller pool
    ids, dist, st, ids2, dist2, st2 = _both(w, 32, 50, 40)
    assert ids2.shape == (40, 32)
    assert np.array_equal(ids, ids2) and np.array_equal(dist.view(np.uint32), dist2.view(np.uint32))
    assert (st.expansions, st.evaluations) == (st2.expansions, st2.evaluations)


def test_noalloc_without_stats_runs_on_the_stream(world):
    import torch
    import apoe
    w = world
    ids, dist, _ = apoe.search(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 0.5, 2.0), 64)
    out_ids = torch.zeros((ids.shape[0], 64), dtype=torch.int32, device="cuda:0")
    out_dist = torch.zeros((ids.shape[0], 64), dtype=torch.float32, device="cuda:0")
    assert apoe.search_noalloc(w["ctx"], w["gc"], w["gq"], w["gg"], (1.0, 0.5, 2.0), 64, out_ids, out_dist, want_stats=False) is None
    w["ctx"].synchronize()
    assert np.array_equal(ids, out_ids.cpu().numpy().view(np.uint32))
    assert np.array_equal(dist.view(np.uint32), out_dist.cpu().numpy().view(np.uint32))


def test_noalloc_refuses_host_outputs(world):
    import ctypes as C
    import apoe
    w = world
    ids = np.empty((w["gq"].n, 16), np.uint32)
    dist = np.empty((w["gq"].n, 16), np.float32)
    p = apoe.SearchParams(1.0, 1.0, 1.0, 0.0, 16, 0, 0, 0, 0, 0)
    st = apoe.lib().apoe_search_noalloc(w["ctx"].h, w["gc"].h, w["gq"].h, w["gg"].h, C.c_void_p(0), C.byref(p), C.c_void_p(ids.ctypes.data),
                                        C.c_void_p(dist.ctypes.data), C.c_void_p(0))
    assert st == -1 and b"device memory" in apoe.lib().apoe_last_error_string()


def test_noalloc_refuses_a_query_range_that_wraps(world):
    import ctypes as C
    import torch
    import apoe
    w = world
    out_ids = torch.zeros((1, 16), dtype=torch.int32, device="cuda:0")
    out_dist = torch.zeros((1, 16), dtype=torch.float32, device="cuda:0")
    p = apoe.SearchParams(1.0, 1.0, 1.0, 0.0, 16, 0, 3, 0xFFFFFFFE, 0, 0)
    st = apoe.lib().apoe_search_noalloc(w["ctx"].h, w["gc"].h, w["gq"].h, w["gg"].h, C.c_void_p(0), C.byref(p), C.c_void_p(out_ids.data_ptr()),
                                        C.c_void_p(out_dist.data_ptr()), C.c_void_p(0))
    assert st == -1 and b"beyond" in apoe.lib().apoe_last_error_string()
