"""Synthetic hybrid corpora, queries and knowledge graphs.

Distributions: dense rows i.i.d. N(0,1) in 1024 dims, L2-normalised; SPLADE-like CSR
over a 30 522-term vocabulary with Zipf(1.1) term ids and log-normal(0, 0.5) values;
BM25-like CSR over the same vocabulary with Zipf term ids and U[0.5, 8] values.
Everything is produced with torch on the requested device from one seed, so a run is
reproducible for a given device type. Arrays come back as torch tensors: dense
float32 [n, 1024]; CSR = (off int32 [n+1], idx int32 [nnz], val float32 [nnz]) with
ids ascending inside a row (the layout of utils.cuh:380-398).
"""
import math

import torch

VOCAB = 30522
DIM = 1024
ZIPF_S = 1.1


def _zipf_cdf(vocab, s, device):
    r = torch.arange(1, vocab + 1, dtype=torch.float64, device=device)
    p = r.pow(-s)
    p = p / p.sum()
    return p, torch.cumsum(p, 0)


def _draws_for_unique(p, target):
    """Number of i.i.d. Zipf draws whose expected count of distinct terms is `target`."""
    lo, hi = float(target), float(target) * 64
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        exp_unique = float((1.0 - torch.pow(1.0 - p, mid)).sum())
        if exp_unique < target:
            lo = mid
        else:
            hi = mid
    return 0.5 * (lo + hi)


def sparse_rows(n, mean_nnz, kind, gen, device, vocab=VOCAB, chunk=1 << 18):
    """CSR with about mean_nnz distinct Zipf terms per row. kind: 'splade' | 'bm25'."""
    p, cdf = _zipf_cdf(vocab, ZIPF_S, device)
    draws = _draws_for_unique(p, mean_nnz)
    cdf32 = cdf.to(torch.float32)
    counts, idx_parts = [], []
    for r0 in range(0, n, chunk):
        rows = min(chunk, n - r0)
        # per-row draw count ~ N(draws, draws/4), at least 2
        m = torch.clamp((torch.randn(rows, generator=gen, device=device) * (draws / 4) + draws).round(), min=2).to(torch.int64)
        total = int(m.sum())
        row_of = torch.repeat_interleave(torch.arange(rows, device=device, dtype=torch.int64), m)
        u = torch.rand(total, generator=gen, device=device)
        term = torch.searchsorted(cdf32, u).clamp_(max=vocab - 1)
        key = torch.unique(row_of * vocab + term)  # sorted: by row, then term id
        counts.append(torch.bincount(key // vocab, minlength=rows))
        idx_parts.append((key % vocab).to(torch.int32))
    cnt = torch.cat(counts)
    idx = torch.cat(idx_parts)
    off = torch.zeros(n + 1, dtype=torch.int64, device=device)
    off[1:] = torch.cumsum(cnt, 0)
    nnz = int(off[-1])
    if kind == "splade":
        val = torch.exp(torch.randn(nnz, generator=gen, device=device) * 0.5)
    else:
        val = torch.rand(nnz, generator=gen, device=device) * 7.5 + 0.5
    return off.to(torch.int32), idx, val.to(torch.float32)


def dense_rows(n, gen, device, chunk=1 << 17):
    out = torch.empty(n, DIM, dtype=torch.float32, device=device)
    for r0 in range(0, n, chunk):
        x = torch.randn(min(chunk, n - r0), DIM, generator=gen, device=device)
        out[r0:r0 + x.shape[0]] = x / x.norm(dim=1, keepdim=True)
    return out


def hybrid_set(n, nnz_splade, nnz_bm25, seed, device="cpu"):
    """(dense, s_off, s_idx, s_val, b_off, b_idx, b_val) for n rows."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    dense = dense_rows(n, gen, device)
    s = sparse_rows(n, nnz_splade, "splade", gen, device)
    b = sparse_rows(n, nnz_bm25, "bm25", gen, device)
    return (dense,) + s + b


def corpus(n, seed=20251125, device="cpu"):
    return hybrid_set(n, 120, 60, seed, device)


def queries(n, seed=20251126, device="cpu"):
    return hybrid_set(n, 30, 8, seed, device)


def _csr_from_degrees(deg, targets_n, gen, device):
    off = torch.zeros(deg.numel() + 1, dtype=torch.int64, device=device)
    off[1:] = torch.cumsum(deg, 0)
    idx = torch.randint(0, targets_n, (int(off[-1]),), generator=gen, device=device, dtype=torch.int64)
    return off.to(torch.int32), idx.to(torch.int32)


def knowledge_graph(n_entities, n_docs, n_queries, seed=20251127, device="cpu", mean_out=8.0, alpha=2.1, docs_per_entity=3.0):
    """(e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx): entity graph with power-law
    out-degree (exponent alpha, mean about mean_out), entity->doc lists with about
    docs_per_entity uniform docs, and 1-3 uniform entities per query."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    # Pareto tail with density exponent alpha: x = xm * U^(-1/(alpha-1)); E[x] = xm*(alpha-1)/(alpha-2)
    xm = mean_out * (alpha - 2.0) / (alpha - 1.0)
    u = torch.rand(n_entities, generator=gen, device=device, dtype=torch.float64).clamp_(min=1e-12)
    deg = torch.clamp((xm * u.pow(-1.0 / (alpha - 1.0))).round(), max=min(n_entities - 1, 4096)).to(torch.int64)
    e2e = _csr_from_degrees(deg, n_entities, gen, device)
    ddeg = 1 + torch.poisson(torch.full((n_entities,), docs_per_entity - 1.0, device=device), generator=gen).to(torch.int64)
    e2d = _csr_from_degrees(ddeg, n_docs, gen, device)
    qdeg = torch.randint(1, 4, (n_queries,), generator=gen, device=device, dtype=torch.int64)
    q2e = _csr_from_degrees(qdeg, n_entities, gen, device)
    return e2e + e2d + q2e


def to_numpy(arrays):
    """Torch tensors -> numpy (int32 offsets/ids viewed as uint32)."""
    import numpy as np
    out = []
    for a in arrays:
        a = a.detach().cpu().numpy()
        out.append(a.view(np.uint32) if a.dtype == np.int32 else a)
    return tuple(out)
