"""ctypes binding of libapoe.so (the C-ABI declared in include/apoe.h).

Arrays may be numpy arrays (host) or torch tensors (host or the context's GPU); the
library copies as needed. There is no CPU fallback: if the HIP library is missing or a
call fails, an exception is raised.
"""
import ctypes as C
import os
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libapoe.so")

INF_DIS = 1000000.0
KW_SLOTS = 8
KW_CAND = 32

_lib = None


class ApoeError(RuntimeError):
    pass


class SearchParams(C.Structure):
    _fields_ = [("w_dense", C.c_float), ("w_sparse", C.c_float), ("w_bm25", C.c_float), ("kg_weight", C.c_float),
                ("cands", C.c_uint32), ("max_iter", C.c_uint32), ("q_begin", C.c_uint32), ("q_count", C.c_uint32),
                ("variant", C.c_uint32), ("keyword_filter", C.c_uint32)]


class SearchStats(C.Structure):
    _fields_ = [("kernel_ms", C.c_float), ("expansions", C.c_uint64), ("evaluations", C.c_uint64),
                ("nnz_sparse", C.c_uint64), ("nnz_bm25", C.c_uint64), ("dense_rows", C.c_uint64), ("algo_bytes", C.c_uint64)]


EXPORTS = [
    "apoe_last_error_string", "apoe_ctx_create", "apoe_ctx_destroy", "apoe_ctx_synchronize", "apoe_corpus_create",
    "apoe_corpus_destroy", "apoe_corpus_info", "apoe_corpus_bytes", "apoe_corpus_pair_bytes", "apoe_corpus_make_half_rows", "apoe_queries_create", "apoe_queries_destroy",
    "apoe_kg_create", "apoe_kg_destroy", "apoe_calibrate_weights", "apoe_hybrid_distance_batch", "apoe_hybrid_distance_pairs", "apoe_norms",
    "apoe_knn_create", "apoe_knn_destroy", "apoe_knn_use_half_rows", "apoe_knn_set_join", "apoe_nnd_init", "apoe_nnd_iterate", "apoe_nnd_merge_reverse",
    "apoe_knn_download", "apoe_knn_upload", "apoe_knn_download_reverse", "apoe_knn_upload_reverse", "apoe_knn_set_prune_form", "apoe_prune", "apoe_prune_download", "apoe_finalize_graph",
    "apoe_knn_elapsed_ms", "apoe_knn_counters", "apoe_graph_create", "apoe_graph_destroy", "apoe_graph_info", "apoe_graph_download",
    "apoe_search", "apoe_search_noalloc",
]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ApoeError(f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}`")
        # PyTorch wheels bring their own copy of the HIP runtime. A process that loads this library
        # first and PyTorch second ends up with two runtimes, and the second one finds no device:
        # let PyTorch (if it is installed) load its copy first, libapoe.so then binds to the same one.
        if "torch" not in sys.modules:
            try:
                import torch  # noqa: F401
            except ImportError:
                pass
        _lib = C.CDLL(LIB_PATH)
        _lib.apoe_last_error_string.restype = C.c_char_p
        _lib.apoe_corpus_bytes.restype = C.c_uint64
        _lib.apoe_corpus_bytes.argtypes = [C.c_void_p]
        _lib.apoe_corpus_pair_bytes.restype = C.c_uint32
        _lib.apoe_corpus_pair_bytes.argtypes = [C.c_void_p]
        _lib.apoe_knn_elapsed_ms.restype = C.c_float
        _lib.apoe_knn_elapsed_ms.argtypes = [C.c_void_p]
        for name in ("apoe_ctx_destroy", "apoe_corpus_destroy", "apoe_queries_destroy", "apoe_kg_destroy",
                     "apoe_knn_destroy", "apoe_graph_destroy"):
            getattr(_lib, name).restype = None
            getattr(_lib, name).argtypes = [C.c_void_p]
    return _lib


def _check(status):
    if status != 0:
        raise ApoeError(f"apoe status {status}: {lib().apoe_last_error_string().decode()}")


def _ptr(a, dtype):
    """(keepalive, void*) of a numpy array or torch tensor of the given numpy dtype."""
    if a is None:
        return None, C.c_void_p(0)
    if isinstance(a, np.ndarray):
        if a.dtype != dtype or not a.flags.c_contiguous:
            a = np.ascontiguousarray(a, dtype=dtype)
        return a, C.c_void_p(a.ctypes.data)
    import torch
    want = {np.dtype(np.float32): torch.float32, np.dtype(np.uint32): (torch.int32, torch.uint32)}[np.dtype(dtype)]
    if isinstance(want, tuple):
        assert a.dtype in want, a.dtype
    else:
        assert a.dtype == want, a.dtype
    a = a.contiguous()
    return a, C.c_void_p(a.data_ptr())


class Context:
    def __init__(self, device=0):
        self.h = C.c_void_p()
        _check(lib().apoe_ctx_create(C.c_int(device), C.byref(self.h)))
        self.device = device

    def synchronize(self):
        _check(lib().apoe_ctx_synchronize(self.h))

    def close(self):
        if self.h:
            lib().apoe_ctx_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Corpus:
    def __init__(self, ctx, dense, s_off, s_idx, s_val, b_off, b_idx, b_val):
        self.ctx = ctx
        n, dim = dense.shape
        keep = [_ptr(dense, np.float32), _ptr(s_off, np.uint32), _ptr(s_idx, np.uint32), _ptr(s_val, np.float32),
                _ptr(b_off, np.uint32), _ptr(b_idx, np.uint32), _ptr(b_val, np.float32)]
        self.h = C.c_void_p()
        _check(lib().apoe_corpus_create(ctx.h, C.c_uint32(n), C.c_uint32(dim), *[k[1] for k in keep], C.byref(self.h)))
        self.n, self.dim = n, dim

    def info(self):
        out = (C.c_uint32 * 4)()
        _check(lib().apoe_corpus_info(self.h, out))
        return list(out)

    def bytes(self):
        return int(lib().apoe_corpus_bytes(self.h))

    def pair_bytes(self):
        return int(lib().apoe_corpus_pair_bytes(self.h))

    def make_half_rows(self):
        """Half-precision copy of the dense rows, for searches with variant | 0x200."""
        _check(lib().apoe_corpus_make_half_rows(self.ctx.h, self.h))

    def close(self):
        if self.h:
            lib().apoe_corpus_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Queries:
    def __init__(self, ctx, dense, s_off, s_idx, s_val, b_off, b_idx, b_val):
        self.ctx = ctx
        n, dim = dense.shape
        keep = [_ptr(dense, np.float32), _ptr(s_off, np.uint32), _ptr(s_idx, np.uint32), _ptr(s_val, np.float32),
                _ptr(b_off, np.uint32), _ptr(b_idx, np.uint32), _ptr(b_val, np.float32)]
        self.h = C.c_void_p()
        _check(lib().apoe_queries_create(ctx.h, C.c_uint32(n), C.c_uint32(dim), *[k[1] for k in keep], C.byref(self.h)))
        self.n, self.dim = n, dim

    def close(self):
        if self.h:
            lib().apoe_queries_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class KnowledgeGraph:
    def __init__(self, ctx, e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx):
        self.ctx = ctx
        keep = [_ptr(a, np.uint32) for a in (e2e_off, e2e_idx, e2d_off, e2d_idx)]
        keepq = [_ptr(a, np.uint32) for a in (q2e_off, q2e_idx)]
        self.h = C.c_void_p()
        _check(lib().apoe_kg_create(ctx.h, C.c_uint32(len(e2e_off) - 1), *[k[1] for k in keep], C.c_uint32(len(q2e_off) - 1),
                                    *[k[1] for k in keepq], C.byref(self.h)))

    def close(self):
        if self.h:
            lib().apoe_kg_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Graph:
    def __init__(self, ctx, rows=None, entry=None, handle=None):
        self.ctx = ctx
        if handle is not None:
            self.h = handle
        else:
            n, W = rows.shape
            kr, ke = _ptr(rows, np.uint32), _ptr(entry, np.uint32)
            self.h = C.c_void_p()
            _check(lib().apoe_graph_create(ctx.h, C.c_uint32(n), C.c_uint32(W), kr[1], ke[1], C.c_uint32(len(entry)), C.byref(self.h)))
        info = (C.c_uint32 * 3)()
        _check(lib().apoe_graph_info(self.h, info))
        self.n, self.width, self.n_entry = info[0], info[1], info[2]

    def download(self):
        rows = np.empty((self.n, self.width), np.uint32)
        entry = np.empty(self.n_entry, np.uint32)
        _check(lib().apoe_graph_download(self.h, C.c_void_p(rows.ctypes.data), C.c_void_p(entry.ctypes.data)))
        return rows, entry

    def close(self):
        if self.h:
            lib().apoe_graph_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Knn:
    """NN-Descent state and the build steps of index.cu:889-903."""

    def __init__(self, ctx, corpus, K=64, dense_scale=7.0):
        self.ctx, self.corpus, self.K = ctx, corpus, K
        self.h = C.c_void_p()
        _check(lib().apoe_knn_create(ctx.h, corpus.h, C.c_uint32(K), C.c_float(dense_scale), C.byref(self.h)))
        self.degree = None

    def use_half_rows(self, on=True):
        """NN-Descent steps on the half-precision rows; merge_reverse() then recomputes the stored distances in fp32."""
        _check(lib().apoe_knn_use_half_rows(self.h, C.c_int(1 if on else 0)))

    def set_join(self, mode):
        """0: the reference's expansion step; 1: local join around the picked neighbour; 2: the same, both endpoints updated."""
        _check(lib().apoe_knn_set_join(self.h, C.c_int(mode)))

    def init(self, seed):
        _check(lib().apoe_nnd_init(self.h, C.c_uint64(seed)))

    def iterate(self, last=False):
        ins = C.c_uint64(0)
        _check(lib().apoe_nnd_iterate(self.h, C.c_int(1 if last else 0), C.byref(ins)))
        return ins.value

    def merge_reverse(self):
        _check(lib().apoe_nnd_merge_reverse(self.h))

    def download(self):
        ids = np.empty((self.corpus.n, self.K), np.uint32)
        dist = np.empty((self.corpus.n, self.K), np.float32)
        _check(lib().apoe_knn_download(self.h, C.c_void_p(ids.ctypes.data), C.c_void_p(dist.ctypes.data)))
        return ids, dist

    def upload(self, ids, dist):
        ki, kd = _ptr(ids, np.uint32), _ptr(dist, np.float32)
        _check(lib().apoe_knn_upload(self.h, ki[1], kd[1]))

    def download_reverse(self):
        """(rev_ids [n][K], rev_dist [n][K], rev_cnt [n]): the reverse lists as they stand."""
        ids = np.empty((self.corpus.n, self.K), np.uint32)
        dist = np.empty((self.corpus.n, self.K), np.float32)
        cnt = np.empty(self.corpus.n, np.uint32)
        _check(lib().apoe_knn_download_reverse(self.h, C.c_void_p(ids.ctypes.data), C.c_void_p(dist.ctypes.data), C.c_void_p(cnt.ctypes.data)))
        return ids, dist, cnt

    def upload_reverse(self, rev_ids, rev_dist, rev_cnt):
        ri, rd, rc = _ptr(rev_ids, np.uint32), _ptr(rev_dist, np.float32), _ptr(rev_cnt, np.uint32)
        _check(lib().apoe_knn_upload_reverse(self.h, ri[1], rd[1], rc[1]))

    def set_prune_form(self, form):
        """0: the gather-once forms of the prune where they apply (default); 1: the table-probing kernel."""
        _check(lib().apoe_knn_set_prune_form(self.h, C.c_int(form)))

    def prune(self, degree):
        _check(lib().apoe_prune(self.h, C.c_uint32(degree)))
        self.degree = degree

    def prune_download(self):
        n, d = self.corpus.n, self.degree
        fwd = np.empty((n, d), np.uint32)
        det = np.empty((n, d), np.uint32)
        cnt = np.empty(n, np.uint32)
        kw = np.empty((n, 1 + KW_CAND), np.uint32)
        _check(lib().apoe_prune_download(self.h, *[C.c_void_p(a.ctypes.data) for a in (fwd, det, cnt, kw)]))
        return fwd, det, cnt, kw

    def finalize(self):
        h = C.c_void_p()
        _check(lib().apoe_finalize_graph(self.h, C.byref(h)))
        return Graph(self.ctx, handle=h)

    def elapsed_ms(self):
        return float(lib().apoe_knn_elapsed_ms(self.h))

    def counters(self):
        """(evaluations, dense rows read) of the NN-Descent steps since init."""
        out = (C.c_uint64 * 2)()
        _check(lib().apoe_knn_counters(self.h, out))
        return int(out[0]), int(out[1])

    def close(self):
        if self.h:
            lib().apoe_knn_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def build_graph(ctx, corpus, K=64, iters=25, degree=32, dense_scale=7.0, seed=1, half_rows=False, join=0, expansion_first=0):
    """NN-Descent + reverse merge + prune + final assembly; returns (Graph, gpu_ms). With a join mode, the first
    `expansion_first` steps are expansion steps all the same (on very large corpora one such step gets the lists going)."""
    knn = Knn(ctx, corpus, K, dense_scale)
    if half_rows:
        corpus.make_half_rows()
        knn.use_half_rows()
    knn.init(seed)
    for it in range(iters):
        if join:
            knn.set_join(0 if it < expansion_first else join)
        knn.iterate(last=(it == iters - 1))
    knn.merge_reverse()
    knn.prune(degree)
    g = knn.finalize()
    ms = knn.elapsed_ms()
    knn.close()
    return g, ms


def distance_batch(ctx, corpus, queries, w3, ids):
    ids = np.ascontiguousarray(ids, np.uint32)
    assert ids.shape[0] == queries.n
    out = np.empty(ids.shape, np.float32)
    w = (C.c_float * 3)(*w3)
    _check(lib().apoe_hybrid_distance_batch(ctx.h, corpus.h, queries.h, w, C.c_void_p(ids.ctypes.data), C.c_uint32(ids.shape[1]),
                                            C.c_void_p(out.ctypes.data)))
    return out


def distance_pairs(ctx, corpus, dense_scale, a, b):
    a = np.ascontiguousarray(a, np.uint32)
    b = np.ascontiguousarray(b, np.uint32)
    out = np.empty(len(a), np.float32)
    _check(lib().apoe_hybrid_distance_pairs(ctx.h, corpus.h, C.c_float(dense_scale), C.c_void_p(a.ctypes.data),
                                            C.c_void_p(b.ctypes.data), C.c_uint32(len(a)), C.c_void_p(out.ctypes.data)))
    return out


def norms(ctx, corpus, dense_scale):
    out = np.empty(corpus.n, np.float32)
    _check(lib().apoe_norms(ctx.h, corpus.h, C.c_float(dense_scale), C.c_void_p(out.ctypes.data)))
    return out


def calibrate_weights(ctx, corpus, queries, w3, n_queries=None):
    """Effective (dense, sparse, bm25) weights after the reference's calibration step."""
    w = (C.c_float * 3)(*w3)
    _check(lib().apoe_calibrate_weights(ctx.h, corpus.h, queries.h, C.c_uint32(queries.n if n_queries is None else n_queries), w))
    return (float(w[0]), float(w[1]), float(w[2]))


def search(ctx, corpus, queries, graph, w3, cands, kg=None, kg_weight=0.0, max_iter=0, q_begin=0, q_count=0, variant=0,
           out_ids=None, out_dist=None, keyword_filter=False):
    """Returns (ids [q, cands] u32, dist [q, cands] f32, SearchStats). w3 = (dense, sparse, bm25).
    keyword_filter: rows hold only documents with a BM25 term that the query flags (bit 31 of the
    query's BM25 term id) as a required keyword."""
    nq = q_count if q_count else queries.n - q_begin
    if q_begin > queries.n or nq > queries.n - q_begin:
        raise ApoeError(f"query range of {nq} from {q_begin} beyond {queries.n} queries")
    if out_ids is None:
        out_ids = np.empty((nq, cands), np.uint32)
        out_dist = np.empty((nq, cands), np.float32)
    for arr, dt, name in ((out_ids, np.uint32, "out_ids"), (out_dist, np.float32, "out_dist")):
        # the library writes into these: a copy made here would be filled and thrown away
        if isinstance(arr, np.ndarray):
            if arr.dtype != dt or not arr.flags.c_contiguous or arr.shape != (nq, cands):
                raise ApoeError(f"{name} must be a C-contiguous {np.dtype(dt).name} array of shape {(nq, cands)}")
        elif not arr.is_contiguous() or tuple(arr.shape) != (nq, cands):
            raise ApoeError(f"{name} must be a contiguous tensor of shape {(nq, cands)}")
    ki, kd = _ptr(out_ids, np.uint32), _ptr(out_dist, np.float32)
    p = SearchParams(w3[0], w3[1], w3[2], kg_weight, cands, max_iter, q_begin, q_count, variant, 1 if keyword_filter else 0)
    st = SearchStats()
    _check(lib().apoe_search(ctx.h, corpus.h, queries.h, graph.h, kg.h if kg is not None else C.c_void_p(0), C.byref(p), ki[1], kd[1],
                             C.byref(st)))
    return out_ids, out_dist, st


def search_noalloc(ctx, corpus, queries, graph, w3, cands, out_ids, out_dist, kg=None, kg_weight=0.0, max_iter=0, q_begin=0, q_count=0,
                   variant=0, keyword_filter=False, want_stats=True):
    """apoe_search_noalloc: the search with a static device workspace; out_ids / out_dist are device tensors
    [q, cands] that the kernels write in place. Without stats the call does not wait for the GPU."""
    nq = q_count if q_count else queries.n - q_begin
    assert tuple(out_ids.shape) == (nq, cands) and tuple(out_dist.shape) == (nq, cands) and out_ids.is_contiguous() and out_dist.is_contiguous()
    ki, kd = _ptr(out_ids, np.uint32), _ptr(out_dist, np.float32)
    p = SearchParams(w3[0], w3[1], w3[2], kg_weight, cands, max_iter, q_begin, q_count, variant, 1 if keyword_filter else 0)
    st = SearchStats() if want_stats else None
    _check(lib().apoe_search_noalloc(ctx.h, corpus.h, queries.h, graph.h, kg.h if kg is not None else C.c_void_p(0), C.byref(p), ki[1], kd[1],
                                     C.byref(st) if want_stats else C.c_void_p(0)))
    return st
