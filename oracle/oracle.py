"""ctypes front end of the CPU oracle (oracle/liboracle.so) and numpy restatements of
the reference's file formats.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py. Nothing shipped imports this module.

File formats (little-endian u32/f32), as the reference reads and writes them:
  fvecs          utils.cuh:361-378   per row [dim][dim x f32]
  sparse CSR     utils.cuh:380-398   [nnz][off x (rows+1)][idx x nnz][val x nnz]
  KG CSR         query.cu:89-108     [rows+1][nnz][off x (rows+1)][idx x nnz]
  qrels/keywords query.cu:65-86      text, line i = ids of query i
  .poe           index.cu:927-939, query.cu:35-62
                 [W][n_ep][ep x n_ep] then per node [W][row x W]
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

INF_DIS = 1000000.0
EMPTY = 0xFFFFFFFF
KW_SLOTS = 8
KW_CAND = 32

u32p = C.POINTER(C.c_uint32)
f32p = C.POINTER(C.c_float)
u64p = C.POINTER(C.c_uint64)


class OrcSet(C.Structure):
    _fields_ = [("n", C.c_uint32), ("dim", C.c_uint32), ("dense", f32p), ("s_off", u32p), ("s_idx", u32p),
                ("s_val", f32p), ("b_off", u32p), ("b_idx", u32p), ("b_val", f32p)]


class OrcKg(C.Structure):
    _fields_ = [("n_entities", C.c_uint32), ("e2e_off", u32p), ("e2e_idx", u32p), ("e2d_off", u32p),
                ("e2d_idx", u32p), ("q2e_off", u32p), ("q2e_idx", u32p)]


def build(force=False):
    """Compile oracle/liboracle.so with the Makefile beside this file."""
    so = os.path.join(_HERE, "liboracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return so


def lib():
    global _LIB
    if _LIB is None:
        # APOE_ORACLE_LIB names another build of the same sources (the sanitizer build of `make asan`)
        so = os.environ.get("APOE_ORACLE_LIB") or os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        _LIB = C.CDLL(so)
        _LIB.orc_rand_id.restype = C.c_uint32
        _LIB.orc_rand_id.argtypes = [C.c_uint64, C.c_uint64, C.c_uint32]
        _LIB.orc_nnd_iterate.restype = C.c_uint64
    return _LIB


def max_threads():
    """omp_get_max_threads() of the oracle library: what threads=0 uses."""
    lib().orc_max_threads.restype = C.c_int
    return int(lib().orc_max_threads())


def _u32(a):
    a = np.ascontiguousarray(a, dtype=np.uint32)
    return a, a.ctypes.data_as(u32p)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(f32p)


class HybridSet:
    """dense [n, dim] f32 + two CSR triples; keeps the arrays alive for the C side."""

    def __init__(self, dense, s_off, s_idx, s_val, b_off, b_idx, b_val):
        self.dense, pd = _f32(dense)
        self.s_off, pso = _u32(s_off)
        self.s_idx, psi = _u32(s_idx)
        self.s_val, psv = _f32(s_val)
        self.b_off, pbo = _u32(b_off)
        self.b_idx, pbi = _u32(b_idx)
        self.b_val, pbv = _f32(b_val)
        self.n, self.dim = self.dense.shape
        assert len(self.s_off) == self.n + 1 and len(self.b_off) == self.n + 1
        self.c = OrcSet(self.n, self.dim, pd, pso, psi, psv, pbo, pbi, pbv)

    def ref(self):
        return C.byref(self.c)

    def arrays(self):
        return (self.dense, self.s_off, self.s_idx, self.s_val, self.b_off, self.b_idx, self.b_val)

    def head(self, n):
        """First n rows as a new set."""
        return HybridSet(self.dense[:n], self.s_off[:n + 1], self.s_idx[:self.s_off[n]], self.s_val[:self.s_off[n]],
                         self.b_off[:n + 1], self.b_idx[:self.b_off[n]], self.b_val[:self.b_off[n]])


class Kg:
    def __init__(self, e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx):
        self.e2e_off, a = _u32(e2e_off)
        self.e2e_idx, b = _u32(e2e_idx)
        self.e2d_off, c = _u32(e2d_off)
        self.e2d_idx, d = _u32(e2d_idx)
        self.q2e_off, e = _u32(q2e_off)
        self.q2e_idx, f = _u32(q2e_idx)
        self.n_entities = len(self.e2e_off) - 1
        assert len(self.e2d_off) == self.n_entities + 1
        self.c = OrcKg(self.n_entities, a, b, c, d, e, f)

    def ref(self):
        return C.byref(self.c)


def _w3(w):
    a = np.asarray(w, dtype=np.float32).copy()
    assert a.shape == (3,)
    return a, a.ctypes.data_as(f32p)


def ip_parts(a, i, b, j):
    out = np.zeros(3, np.float32)
    lib().orc_ip_parts(a.ref(), C.c_uint32(i), b.ref(), C.c_uint32(j), out.ctypes.data_as(f32p))
    return out


def distance_batch(corpus, queries, w3, ids, threads=0):
    ids, pi = _u32(ids)
    assert ids.shape[0] == queries.n
    out = np.empty(ids.shape, np.float32)
    w, pw = _w3(w3)
    lib().orc_distance_batch(corpus.ref(), queries.ref(), pw, pi, C.c_uint32(ids.shape[1]), out.ctypes.data_as(f32p), threads)
    return out


def distance_pairs(corpus, dense_scale, a, b, threads=0):
    a, pa = _u32(a)
    b, pb = _u32(b)
    out = np.empty(len(a), np.float32)
    lib().orc_distance_pairs(corpus.ref(), C.c_float(dense_scale), pa, pb, C.c_uint32(len(a)), out.ctypes.data_as(f32p), threads)
    return out


def norms(corpus, dense_scale, threads=0):
    out = np.empty(corpus.n, np.float32)
    lib().orc_norms(corpus.ref(), C.c_float(dense_scale), out.ctypes.data_as(f32p), threads)
    return out


def bruteforce_topk(corpus, queries, w3, k, threads=0):
    ids = np.empty((queries.n, k), np.uint32)
    dist = np.empty((queries.n, k), np.float32)
    w, pw = _w3(w3)
    lib().orc_bruteforce_topk(corpus.ref(), queries.ref(), pw, C.c_uint32(k), ids.ctypes.data_as(u32p), dist.ctypes.data_as(f32p), threads)
    return ids, dist


def bruteforce_knn_self(corpus, dense_scale, k, threads=0):
    ids = np.empty((corpus.n, k), np.uint32)
    dist = np.empty((corpus.n, k), np.float32)
    lib().orc_bruteforce_knn_self(corpus.ref(), C.c_float(dense_scale), C.c_uint32(k), ids.ctypes.data_as(u32p), dist.ctypes.data_as(f32p), threads)
    return ids, dist


def merge_top(pool_ids, pool_dist, new_ids, new_dist):
    pi, ppi = _u32(np.array(pool_ids, dtype=np.uint32))
    pd, ppd = _f32(np.array(pool_dist, dtype=np.float32))
    ni, pni = _u32(new_ids)
    nd, pnd = _f32(new_dist)
    lib().orc_merge_top(ppi, ppd, C.c_uint32(len(pi)), pni, pnd, C.c_uint32(len(ni)))
    return pi, pd


def search(corpus, queries, rows, entry, w3, cands, max_iter=1000, kg=None, kg_weight=0.0, threads=0, keyword_filter=False):
    rows, pr = _u32(rows)
    entry, pe = _u32(entry)
    n, W = rows.shape
    assert n == corpus.n
    ids = np.empty((queries.n, cands), np.uint32)
    dist = np.empty((queries.n, cands), np.float32)
    counters = np.zeros((queries.n, 4), np.uint64)
    w, pw = _w3(w3)
    if keyword_filter:
        assert kg is None
        lib().orc_search_keyword(corpus.ref(), queries.ref(), pr, C.c_uint32(W), pe, C.c_uint32(len(entry)), pw, C.c_uint32(cands),
                                 C.c_uint32(max_iter), ids.ctypes.data_as(u32p), dist.ctypes.data_as(f32p),
                                 counters.ctypes.data_as(u64p), threads)
    elif kg is None:
        lib().orc_search(corpus.ref(), queries.ref(), pr, C.c_uint32(W), pe, C.c_uint32(len(entry)), pw, C.c_uint32(cands),
                         C.c_uint32(max_iter), ids.ctypes.data_as(u32p), dist.ctypes.data_as(f32p), counters.ctypes.data_as(u64p), threads)
    else:
        lib().orc_search_kg(corpus.ref(), queries.ref(), kg.ref(), pr, C.c_uint32(W), pe, C.c_uint32(len(entry)), pw,
                            C.c_float(kg_weight), C.c_uint32(cands), C.c_uint32(max_iter), ids.ctypes.data_as(u32p),
                            dist.ctypes.data_as(f32p), counters.ctypes.data_as(u64p), threads)
    return ids, dist, counters


class KnnState:
    def __init__(self, n, K):
        self.n, self.K = n, K
        self.ids = np.empty((n, K), np.uint32)
        self.dist = np.empty((n, K), np.float32)
        self.rev = np.empty((n, K), np.uint32)
        self.rev_dist = np.empty((n, K), np.float32)
        self.rev_cnt = np.zeros(n, np.uint32)

    def _p(self):
        return (self.ids.ctypes.data_as(u32p), self.dist.ctypes.data_as(f32p), self.rev.ctypes.data_as(u32p),
                self.rev_dist.ctypes.data_as(f32p), self.rev_cnt.ctypes.data_as(u32p))


def nnd_init(n, K, seed):
    st = KnnState(n, K)
    lib().orc_nnd_init(C.c_uint32(n), C.c_uint32(K), C.c_uint64(seed), *st._p())
    return st


def nnd_iterate(corpus, dense_scale, st, threads=0):
    return int(lib().orc_nnd_iterate(corpus.ref(), C.c_float(dense_scale), C.c_uint32(st.K), *st._p(), threads))


class JoinParams(C.Structure):
    _fields_ = [("slots", C.c_uint32), ("symmetric", C.c_uint32)]


def join_iterate(corpus, dense_scale, st, slots=64, symmetric=False, threads=0):
    """One step as a local join around the picked neighbours; returns (inserted, distance evaluations)."""
    prm = JoinParams(slots, 1 if symmetric else 0)
    ev = C.c_uint64(0)
    lib().orc_join_iterate.restype = C.c_uint64
    ins = lib().orc_join_iterate(corpus.ref(), C.c_float(dense_scale), C.c_uint32(st.K), *st._p(), C.byref(prm), C.byref(ev), threads)
    return int(ins), int(ev.value)


def nnd_merge_reverse(st, threads=0):
    lib().orc_nnd_merge_reverse(C.c_uint32(st.n), C.c_uint32(st.K), *st._p(), threads)


def prune(corpus, dense_scale, norms_, ids, dist, d, threads=0):
    ids, pi = _u32(ids)
    dist, pd = _f32(dist)
    nrm, pn = _f32(norms_)
    n, K = ids.shape
    fwd = np.empty((n, d), np.uint32)
    det = np.empty((n, d), np.uint32)
    cnt = np.empty(n, np.uint32)
    kw = np.empty((n, 1 + KW_CAND), np.uint32)
    lib().orc_prune(corpus.ref(), C.c_float(dense_scale), pn, C.c_uint32(K), pi, pd, C.c_uint32(d), fwd.ctypes.data_as(u32p),
                    det.ctypes.data_as(u32p), cnt.ctypes.data_as(u32p), kw.ctypes.data_as(u32p), threads)
    return fwd, det, cnt, kw


def final_graph(fwd, det, cnt, kw):
    fwd, pf = _u32(fwd)
    det, pdt = _u32(det)
    cnt, pc = _u32(cnt)
    kw, pk = _u32(kw)
    n, d = fwd.shape
    rows = np.empty((n, d + KW_SLOTS), np.uint32)
    lib().orc_final_graph(C.c_uint32(n), C.c_uint32(d), pf, pdt, pc, pk, rows.ctypes.data_as(u32p))
    return rows


def entry_points(norms_, d):
    nrm, pn = _f32(norms_)
    out = np.empty(d, np.uint32)
    lib().orc_entry_points(pn, C.c_uint32(len(nrm)), C.c_uint32(d), out.ctypes.data_as(u32p))
    return out


def calibrate(corpus, queries, n_queries, w3):
    w, pw = _w3(w3)
    lib().orc_calibrate(corpus.ref(), queries.ref(), C.c_uint32(n_queries), pw)
    return w


def ndcg(res, gt_lists):
    res, pr = _u32(res)
    nq, k = res.shape
    off = np.zeros(nq + 1, np.uint32)
    off[1:] = np.cumsum([len(g) for g in gt_lists[:nq]])
    idx = np.concatenate([np.asarray(g, np.uint32) for g in gt_lists[:nq]]) if nq else np.zeros(0, np.uint32)
    off, po = _u32(off)
    idx, pi = _u32(idx)
    out = np.zeros(2, np.float64)
    lib().orc_ndcg(pr, C.c_uint32(nq), C.c_uint32(k), po, pi, out.ctypes.data_as(C.POINTER(C.c_double)))
    return float(out[0]), float(out[1])


def build_index(corpus, dense_scale=7.0, K=64, iters=25, d=32, seed=1, threads=0, return_knn=False):
    n = corpus.n
    rows = np.empty((n, d + KW_SLOTS), np.uint32)
    entry = np.empty(d, np.uint32)
    knn_ids = np.empty((n, K), np.uint32)
    knn_dist = np.empty((n, K), np.float32)
    lib().orc_build(corpus.ref(), C.c_float(dense_scale), C.c_uint32(K), C.c_uint32(iters), C.c_uint32(d), C.c_uint64(seed),
                    rows.ctypes.data_as(u32p), entry.ctypes.data_as(u32p), knn_ids.ctypes.data_as(u32p),
                    knn_dist.ctypes.data_as(f32p), threads)
    if return_knn:
        return rows, entry, knn_ids, knn_dist
    return rows, entry


# ---------------------------------------------------------------- file formats

def read_fvecs(path):
    raw = np.fromfile(path, dtype=np.uint32)
    dim = int(raw[0])
    n = raw.size // (dim + 1)
    return raw[:n * (dim + 1)].reshape(n, dim + 1)[:, 1:].view(np.float32).copy()


def write_fvecs(path, a):
    a = np.ascontiguousarray(a, np.float32)
    n, dim = a.shape
    out = np.empty((n, dim + 1), np.uint32)
    out[:, 0] = dim
    out[:, 1:] = a.view(np.uint32)
    out.tofile(path)


def read_csr(path, rows=None):
    raw = np.fromfile(path, dtype=np.uint32)
    nnz = int(raw[0])
    if rows is None:
        rows = raw.size - 1 - 2 * nnz - 1
    off = raw[1:2 + rows].copy()
    idx = raw[2 + rows:2 + rows + nnz].copy()
    val = raw[2 + rows + nnz:2 + rows + 2 * nnz].view(np.float32).copy()
    return off, idx, val


def write_csr(path, off, idx, val):
    with open(path, "wb") as f:
        np.array([len(idx)], np.uint32).tofile(f)
        np.ascontiguousarray(off, np.uint32).tofile(f)
        np.ascontiguousarray(idx, np.uint32).tofile(f)
        np.ascontiguousarray(val, np.float32).tofile(f)


def read_kg(path):
    raw = np.fromfile(path, dtype=np.uint32)
    num, nnz = int(raw[0]), int(raw[1])  # num = rows + 1
    return raw[2:2 + num].copy(), raw[2 + num:2 + num + nnz].copy()


def write_kg(path, off, idx):
    with open(path, "wb") as f:
        np.array([len(off), len(idx)], np.uint32).tofile(f)
        np.ascontiguousarray(off, np.uint32).tofile(f)
        np.ascontiguousarray(idx, np.uint32).tofile(f)


def read_id_lines(path, n=None):
    out = []
    with open(path) as f:
        for line in f:
            out.append([int(t) for t in line.split()])
            if n is not None and len(out) >= n:
                break
    return out


def write_poe(path, rows, entry):
    rows = np.ascontiguousarray(rows, np.uint32)
    n, W = rows.shape
    with open(path, "wb") as f:
        np.array([W, len(entry)], np.uint32).tofile(f)
        np.ascontiguousarray(entry, np.uint32).tofile(f)
        body = np.empty((n, W + 1), np.uint32)
        body[:, 0] = W
        body[:, 1:] = rows
        body.tofile(f)


def read_poe(path):
    raw = np.fromfile(path, dtype=np.uint32)
    W, n_ep = int(raw[0]), int(raw[1])
    entry = raw[2:2 + n_ep].copy()
    n = (raw.size - 2 - n_ep) // (W + 1)
    rows = raw[2 + n_ep:2 + n_ep + n * (W + 1)].reshape(n, W + 1)[:, 1:].copy()
    return rows, entry
