"""Large pageable host arrays go to the device through the pinned double-buffered pipeline (apoe_corpus_create,
apoe_queries_create): the corpus made from host arrays is the corpus made from device arrays, bit for bit."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_corpus_from_host_arrays_equals_corpus_from_device_arrays(gpu_ctx):
    import torch
    import apoe
    import apoe_synth as S
    n = 40_000  # 160 MB of dense rows: above the size from which uploads are streamed
    dev = S.corpus(n, seed=77, device="cuda:0")
    host = S.to_numpy(dev)
    assert host[0].nbytes >= 128 << 20
    g_dev = apoe.Corpus(gpu_ctx, *dev)
    t0 = time.perf_counter()
    g_host = apoe.Corpus(gpu_ctx, *host)
    dt = time.perf_counter() - t0
    print(f"corpus of {g_host.bytes() / 1e6:.0f} MB from pageable host arrays in {dt * 1e3:.0f} ms ({g_host.bytes() / 1e9 / dt:.1f} GB/s, repacking included)")
    assert g_host.bytes() == g_dev.bytes() and g_host.info() == g_dev.info()
    assert np.array_equal(apoe.norms(gpu_ctx, g_host, 7.0).view(np.uint32), apoe.norms(gpu_ctx, g_dev, 7.0).view(np.uint32))
    q = S.to_numpy(S.queries(64, seed=78))
    gq = apoe.Queries(gpu_ctx, *q)
    rng = np.random.default_rng(5)
    ids = rng.integers(0, n, (64, 500)).astype(np.uint32)
    ids[:, -1] = n - 1  # the last record: the tail of the last chunk arrived
    a = apoe.distance_batch(gpu_ctx, g_host, gq, (1.0, 1.0, 1.0), ids)
    b = apoe.distance_batch(gpu_ctx, g_dev, gq, (1.0, 1.0, 1.0), ids)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # a non-contiguous slice of a larger array is copied to contiguous memory by the binding first
    g_odd = apoe.Corpus(gpu_ctx, np.ascontiguousarray(host[0][:n - 3]), host[1][:n - 2], host[2][:host[1][n - 3]], host[3][:host[1][n - 3]],
                        host[4][:n - 2], host[5][:host[4][n - 3]], host[6][:host[4][n - 3]])
    assert g_odd.info()[0] == n - 3
    for g in (g_odd, g_host, g_dev, gq):
        g.close()
    del dev
    torch.cuda.empty_cache()
