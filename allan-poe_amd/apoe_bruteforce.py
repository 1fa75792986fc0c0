"""Exact hybrid top-k by plain torch on the GPU: the ground truth of recall figures.

A CHECKER for tests and bench.py, independent of the library's kernels (dense part: matmul; sparse parts: a dense
[2 * vocab, queries] matrix of the query terms that the corpus pairs gather from). The library never imports it."""
import torch

import apoe_synth as S


def hybrid_topk(corpus, queries, w3, k, nq=None, self_ids=None, q_block=4096, d_chunk=4096, vocab=S.VOCAB):
    """Top-k ids and distances 1 - (w_d <dense> + w_s <splade> + w_b <bm25>) of the first nq query rows against
    every corpus row. corpus / queries: (dense, s_off, s_idx, s_val, b_off, b_idx, b_val) torch tensors on one
    device. self_ids[i] (optional): a corpus row that query i must not return (a document as its own query).
    Returns (ids int64 [nq, k], dist float32 [nq, k]) on the CPU as numpy arrays."""
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = corpus
    qd, qs_off, qs_idx, qs_val, qb_off, qb_idx, qb_val = queries
    dev = dense.device
    n = dense.shape[0]
    nq = qd.shape[0] if nq is None else nq
    out_i = torch.empty((nq, k), dtype=torch.long)
    out_d = torch.empty((nq, k), dtype=torch.float32)
    for q0 in range(0, nq, q_block):
        q1 = min(nq, q0 + q_block)
        m = q1 - q0
        Qt = torch.zeros(2 * vocab, m, device=dev)
        for off, idx, val, base, w in ((qs_off, qs_idx, qs_val, 0, w3[1]), (qb_off, qb_idx, qb_val, vocab, w3[2])):
            if w < 1e-5:
                continue
            e0, e1 = int(off[q0]), int(off[q1])
            cnt = (off[q0 + 1:q1 + 1] - off[q0:q1]).long()
            cols = torch.repeat_interleave(torch.arange(m, device=dev), cnt)
            Qt[(idx[e0:e1].long() & 0x7FFFFFFF) + base, cols] = val[e0:e1] * w
        qdw = qd[q0:q1] * w3[0]
        best_d = torch.full((m, k), float("inf"), device=dev)
        best_i = torch.zeros((m, k), dtype=torch.long, device=dev)
        sid = None if self_ids is None else torch.as_tensor(self_ids[q0:q1], device=dev).long()
        for r0 in range(0, n, d_chunk):
            r1 = min(n, r0 + d_chunk)
            ip = torch.zeros(r1 - r0, m, device=dev)
            if w3[0] >= 1e-5:
                ip += dense[r0:r1] @ qdw.T
            for off, idx, val, base, w in ((s_off, s_idx, s_val, 0, w3[1]), (b_off, b_idx, b_val, vocab, w3[2])):
                if w < 1e-5:
                    continue
                e0, e1 = int(off[r0]), int(off[r1])
                if e1 == e0:
                    continue
                cnt = (off[r0 + 1:r1 + 1] - off[r0:r1]).long()
                rows = torch.repeat_interleave(torch.arange(r1 - r0, device=dev), cnt)
                ip.index_add_(0, rows, Qt.index_select(0, idx[e0:e1].long() + base) * val[e0:e1, None])
            dist = (1.0 - ip).T  # [m, chunk]
            if sid is not None:
                inside = (sid >= r0) & (sid < r1)
                dist[torch.nonzero(inside)[:, 0], sid[inside] - r0] = float("inf")
            cat_d = torch.cat([best_d, dist], 1)
            cat_i = torch.cat([best_i, torch.arange(r0, r1, device=dev).expand(m, -1)], 1)
            best_d, sel = torch.topk(cat_d, k, dim=1, largest=False)
            best_i = torch.gather(cat_i, 1, sel)
        out_i[q0:q1] = best_i.cpu()
        out_d[q0:q1] = best_d.cpu()
    return out_i.numpy(), out_d.numpy()


def rows_as_queries(corpus, ids):
    """The corpus rows `ids` (ascending torch long tensor on the corpus' device) as a query set."""
    dense, s_off, s_idx, s_val, b_off, b_idx, b_val = corpus
    out = [dense[ids]]
    for off, idx, val in ((s_off, s_idx, s_val), (b_off, b_idx, b_val)):
        o = off.long()
        cnt = o[ids + 1] - o[ids]
        new_off = torch.zeros(ids.numel() + 1, dtype=torch.long, device=dense.device)
        new_off[1:] = torch.cumsum(cnt, 0)
        pos = torch.arange(int(new_off[-1]), device=dense.device)
        row = torch.repeat_interleave(torch.arange(ids.numel(), device=dense.device), cnt)
        src = o[ids][row] + (pos - new_off[row])
        out += [new_off.to(torch.int32), idx[src], val[src]]
    return tuple(out)


def recall_at_k(found, truth, k):
    hit = 0
    for f, t in zip(found, truth):
        hit += len(set(f[:k].tolist()) & set(t[:k].tolist()))
    return hit / (len(truth) * k)
