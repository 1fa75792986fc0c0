"""Synthetic hybrid corpora, queries and knowledge graphs from a counter-based generator.

Distributions: dense rows i.i.d. N(0,1) in 1024 dims, L2-normalised; SPLADE-like CSR
over a 30 522-term vocabulary with Zipf(1.1) term ids and log-normal(0, 0.5) values;
BM25-like CSR over the same vocabulary with Zipf term ids and U[0.5, 8] values.

Every random number is a pure function of (seed, stream, index): splitmix64 applied
twice to a 64-bit counter. Nothing depends on a library's generator, on the device or
on how the work is cut into chunks, so one seed names ONE world wherever it is made:
with numpy on the host (device="cpu") or with torch integer arithmetic on the GPU
(device="cuda:0") -- the two give the same bits. To keep it that way the samplers use
only operations that are exact or correctly rounded everywhere: 64-bit integer
arithmetic, table look-ups, binary search in a float64 table, and float64
add / multiply / divide / sqrt. Transcendental functions are evaluated once, on the
host, into tables (normal quantiles, log-normal values, the Zipf and degree
distribution functions) that both back ends index.

Arrays come back as torch tensors on the requested device: dense float32 [n, 1024];
CSR = (off int32 [n+1], idx int32 [nnz], val float32 [nnz]) with ids ascending inside
a row (the layout of utils.cuh:380-398).
"""
import functools

import numpy as np

VOCAB = 30522
DIM = 1024
ZIPF_S = 1.1
MAX_DRAWS = 4096          # per sparse row: index stride of the draw counters
GAUSS_BITS = 20           # normal quantile table: 2^20 levels, fixed point with 20 fractional bits
LOGN_BITS = 16            # log-normal value table: 2^16 levels

_M64 = (1 << 64) - 1
_GOLD = 0x9E3779B97F4A7C15
_C1 = 0xBF58476D1CE4E5B9
_C2 = 0x94D049BB133111EB

# streams: one per array of a set
S_DENSE, S_S_COUNT, S_S_TERM, S_S_VAL, S_B_COUNT, S_B_TERM, S_B_VAL = range(1, 8)
S_KG_DEG, S_KG_E2E, S_KG_DDEG, S_KG_E2D, S_KG_QDEG, S_KG_Q2E = range(16, 22)
S_L_ROW, S_L_DENSE = range(32, 34)

LATENT_DIM = 16           # latent sets: dimension of the hidden vector behind a dense row
LATENT_NOISE = 4          # dense row = image of the hidden vector + LATENT_NOISE x own normal vector (in units of the hidden vector's scale)
LATENT_SCALE = 0.3        # sparse values times this: under 49 x dense + sparse + bm25 the dense part then carries about three quarters


def mix64_int(z):
    """splitmix64 finaliser on a Python int."""
    z = (z + _GOLD) & _M64
    z = ((z ^ (z >> 30)) * _C1) & _M64
    z = ((z ^ (z >> 27)) * _C2) & _M64
    return z ^ (z >> 31)


def stream_key(seed, stream):
    return mix64_int((seed & _M64) ^ mix64_int(stream))


class _Numpy:
    """uint64 arrays: arithmetic wraps."""
    name = "numpy"

    def __init__(self, device=None):
        pass

    def arange(self, a, b):
        return np.arange(a, b, dtype=np.uint64)

    def mix(self, z):
        z = z + np.uint64(_GOLD)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(_C1)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(_C2)
        return z ^ (z >> np.uint64(31))

    def rnd(self, key, idx):
        return self.mix(np.uint64(key) ^ self.mix(idx))

    def top_bits(self, h, bits):
        return (h >> np.uint64(64 - bits)).astype(np.int64)

    def unit53(self, h):
        return (h >> np.uint64(11)).astype(np.float64) * (2.0 ** -53)

    def mod(self, h, n):
        return ((h >> np.uint64(1)) % np.uint64(n)).astype(np.int64)

    def table(self, t):
        return t

    def take(self, t, i):
        return t[i]

    def searchsorted(self, t, u):
        return np.searchsorted(t, u, side="left").astype(np.int64)

    def shr_signed(self, x, s):
        return x >> s

    def repeat_rows(self, counts):
        return np.repeat(np.arange(len(counts), dtype=np.int64), counts)

    def cumsum0(self, c):
        out = np.zeros(len(c) + 1, dtype=np.int64)
        np.cumsum(c, out=out[1:])
        return out

    def unique(self, k):
        return np.unique(k)

    def bincount(self, x, n):
        return np.bincount(x, minlength=n).astype(np.int64)

    def cat(self, parts, dtype):
        return np.concatenate(parts).astype(dtype) if parts else np.zeros(0, dtype)

    def f64(self, x):
        return x.astype(np.float64)

    def f32(self, x):
        return x.astype(np.float32)

    def i32(self, x):
        return x.astype(np.int32)

    def u64(self, x):
        return x.astype(np.uint64)

    def rint_clamp(self, x, lo, hi):
        return np.clip(np.rint(x), lo, hi).astype(np.int64)

    def sqrt(self, x):
        return np.sqrt(x)

    def empty_f32(self, n, d):
        return np.empty((n, d), np.float32)

    def to_torch(self, x):
        import torch
        return torch.from_numpy(np.ascontiguousarray(x))


class _Torch:
    """int64 tensors stand for uint64: add, multiply and xor are the same bits; a logical shift right is an
    arithmetic one with the copied sign bits masked off."""
    name = "torch"

    def __init__(self, device):
        import torch
        self.t = torch
        self.dev = device

    @staticmethod
    def _s(c):  # a 64-bit constant as the signed value of the same bits
        c &= _M64
        return c - (1 << 64) if c >> 63 else c

    def arange(self, a, b):
        return self.t.arange(a, b, dtype=self.t.int64, device=self.dev)

    def _shr(self, z, s):
        return (z >> s) & ((1 << (64 - s)) - 1)

    def mix(self, z):
        z = z + self._s(_GOLD)
        z = (z ^ self._shr(z, 30)) * self._s(_C1)
        z = (z ^ self._shr(z, 27)) * self._s(_C2)
        return z ^ self._shr(z, 31)

    def rnd(self, key, idx):
        return self.mix(self.mix(idx) ^ self._s(key))

    def top_bits(self, h, bits):
        return self._shr(h, 64 - bits)

    def unit53(self, h):
        return self._shr(h, 11).to(self.t.float64) * (2.0 ** -53)

    def mod(self, h, n):
        return self._shr(h, 1) % n

    def table(self, t):
        return self.t.from_numpy(t).to(self.dev)

    def take(self, t, i):
        return t[i]

    def searchsorted(self, t, u):
        return self.t.searchsorted(t, u, right=False)

    def shr_signed(self, x, s):
        return x >> s

    def repeat_rows(self, counts):
        return self.t.repeat_interleave(self.t.arange(counts.numel(), dtype=self.t.int64, device=self.dev), counts)

    def cumsum0(self, c):
        out = self.t.zeros(c.numel() + 1, dtype=self.t.int64, device=self.dev)
        out[1:] = self.t.cumsum(c, 0)
        return out

    def unique(self, k):
        return self.t.unique(k)

    def bincount(self, x, n):
        return self.t.bincount(x, minlength=n)

    def cat(self, parts, dtype):
        td = {np.int32: self.t.int32, np.float32: self.t.float32, np.int64: self.t.int64}[dtype]
        return self.t.cat(parts).to(td) if parts else self.t.zeros(0, dtype=td, device=self.dev)

    def f64(self, x):
        return x.to(self.t.float64)

    def f32(self, x):
        return x.to(self.t.float32)

    def i32(self, x):
        return x.to(self.t.int32)

    def u64(self, x):
        return x.to(self.t.int64)

    def rint_clamp(self, x, lo, hi):
        return self.t.clamp(self.t.round(x), lo, hi).to(self.t.int64)

    def sqrt(self, x):
        return self.t.sqrt(x)

    def empty_f32(self, n, d):
        return self.t.empty((n, d), dtype=self.t.float32, device=self.dev)

    def to_torch(self, x):
        return x


def backend(device="cpu", force=None):
    kind = force or ("numpy" if str(device) == "cpu" else "torch")
    return _Numpy() if kind == "numpy" else _Torch(device)


# ---- host-side tables (float64 / integer; every back end indexes the same numbers) ----

@functools.lru_cache(maxsize=None)
def gauss_table_fixed():
    """Normal quantiles at (k + 1/2) / 2^20 as fixed point with 20 fractional bits (int64)."""
    from scipy.special import ndtri
    k = np.arange(1 << GAUSS_BITS, dtype=np.float64)
    return np.rint(ndtri((k + 0.5) / (1 << GAUSS_BITS)) * (1 << 20)).astype(np.int64)


@functools.lru_cache(maxsize=None)
def lognormal_table():
    """exp(0.5 * z) at the normal quantiles z of (k + 1/2) / 2^16, float32."""
    from scipy.special import ndtri
    k = np.arange(1 << LOGN_BITS, dtype=np.float64)
    return np.exp(0.5 * ndtri((k + 0.5) / (1 << LOGN_BITS))).astype(np.float32)


@functools.lru_cache(maxsize=None)
def zipf_tables(vocab=VOCAB, s=ZIPF_S):
    r = np.arange(1, vocab + 1, dtype=np.float64)
    p = r ** (-s)
    p /= p.sum()
    cdf = np.cumsum(p)
    cdf[-1] = 1.0
    return p, cdf


@functools.lru_cache(maxsize=None)
def draws_for_unique(target, vocab=VOCAB):
    """Number of i.i.d. Zipf draws whose expected count of distinct terms is `target`."""
    p, _ = zipf_tables(vocab)
    lo, hi = float(target), float(target) * 64
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        if float((1.0 - np.power(1.0 - p, mid)).sum()) < target:
            lo = mid
        else:
            hi = mid
    return 0.5 * (lo + hi)


# ---- samplers ----

@functools.lru_cache(maxsize=None)
def rarity_table(mean_nnz, kind, vocab=VOCAB):
    """Latent sets weight a term by how rare it is, as BM25 and learned sparse encoders do: idf(t) = ln(1 / df(t))
    with df(t) the share of rows of mean_nnz terms that hold t. BM25-like values are LATENT_SCALE x idf x U[0.3, 1],
    SPLADE-like values LATENT_SCALE x min(1, idf / 4) x log-normal. The factor in front of the random part, float32."""
    p, _ = zipf_tables(vocab)
    df = 1.0 - np.power(1.0 - p, draws_for_unique(mean_nnz, vocab))
    idf = np.log(1.0 / df)
    return (LATENT_SCALE * (idf if kind == "bm25" else np.minimum(1.0, idf / 4.0))).astype(np.float32)


def sparse_rows(n, mean_nnz, kind, seed, device="cpu", vocab=VOCAB, chunk=1 << 18, force_backend=None, by_rarity=False):
    """CSR with about mean_nnz distinct Zipf terms per row. kind: 'splade' | 'bm25'. Row r draws
    m_r ~ round(N(draws, draws/4)) terms (2 <= m_r < 4096), keeps the distinct ones in ascending order; the value
    of term t in row r depends on (r, t) only. by_rarity: values carry the term's rarity_table() factor."""
    X = backend(device, force_backend)
    rarity = X.table(rarity_table(mean_nnz, kind, vocab)) if by_rarity else None
    s_count, s_term, s_val = (S_S_COUNT, S_S_TERM, S_S_VAL) if kind == "splade" else (S_B_COUNT, S_B_TERM, S_B_VAL)
    k_count, k_term, k_val = stream_key(seed, s_count), stream_key(seed, s_term), stream_key(seed, s_val)
    _, cdf_h = zipf_tables(vocab)
    cdf = X.table(cdf_h)
    gauss = X.table(gauss_table_fixed())
    logn = X.table(lognormal_table())
    draws = draws_for_unique(mean_nnz, vocab)
    counts, idx_parts, val_parts = [], [], []
    for r0 in range(0, n, chunk):
        rows = min(chunk, n - r0)
        g = X.f64(X.take(gauss, X.top_bits(X.rnd(k_count, X.arange(r0, r0 + rows)), GAUSS_BITS))) * (2.0 ** -20)
        m = X.rint_clamp(g * (draws / 4) + draws, 2, MAX_DRAWS - 1)
        start = X.cumsum0(m)
        total = int(start[-1])
        row_of = X.repeat_rows(m)                                   # local row of every draw
        j = X.arange(0, total) - X.u64(X.take(start, row_of))       # its number inside the row
        h = X.rnd(k_term, (X.u64(row_of) + r0) * MAX_DRAWS + j)
        term = X.searchsorted(cdf, X.unit53(h))
        key = X.unique(row_of * vocab + term)                       # sorted: by row, then term id
        krow, kterm = key // vocab, key % vocab
        counts.append(X.bincount(krow, rows))
        idx_parts.append(X.i32(kterm))
        hv = X.rnd(k_val, (X.u64(krow) + r0) * 65536 + X.u64(kterm))
        if kind == "splade":
            val = X.take(logn, X.top_bits(hv, LOGN_BITS))
        elif not by_rarity:
            val = X.f32((X.f64(X.top_bits(hv, 24)) + 0.5) * (7.5 / (1 << 24)) + 0.5)
        else:
            val = X.f32((X.f64(X.top_bits(hv, 24)) + 0.5) * (0.7 / (1 << 24)) + 0.3)
        val_parts.append(val * X.take(rarity, kterm) if by_rarity else val)
    cnt = X.cat(counts, np.int64)
    off = X.i32(X.cumsum0(cnt))
    return X.to_torch(off), X.to_torch(X.cat(idx_parts, np.int32)), X.to_torch(X.cat(val_parts, np.float32))


def hidden_of_rows(X, seed, r0, r1):
    """The hidden vectors of rows r0..r1-1 of the latent set that `seed` names: [r1 - r0, LATENT_DIM] normal integers
    with 4 fractional bits (standard deviation 16)."""
    g = X.take(X.table(gauss_table_fixed()), X.top_bits(X.rnd(stream_key(seed, S_L_ROW), X.arange(r0 * LATENT_DIM, r1 * LATENT_DIM)), GAUSS_BITS))
    return X.shr_signed(g, 16).reshape(r1 - r0, LATENT_DIM)


def dense_rows(n, seed, device="cpu", chunk=1 << 14, force_backend=None, world=None):
    """Rows of 1024 normal values at 2^-20 resolution, L2-normalised: the sum of squares is an exact integer,
    its square root and the division are float64 operations, the result is rounded to float32 once. With `world`
    (a seed that names a 16 x 1024 normal map shared by every set of that world) a row is the image of its 16 hidden
    values under the map plus LATENT_NOISE x its own normal vector: two rows have about half the cosine of their
    hidden vectors."""
    X = backend(device, force_backend)
    key = stream_key(seed, S_DENSE)
    gauss = X.table(gauss_table_fixed())
    out = X.empty_f32(n, DIM)
    if world is not None:
        spread = X.take(gauss, X.top_bits(X.rnd(stream_key(world, S_L_DENSE), X.arange(0, LATENT_DIM * DIM)), GAUSS_BITS)).reshape(LATENT_DIM, DIM)
    for r0 in range(0, n, chunk):
        rows = min(chunk, n - r0)
        g = X.take(gauss, X.top_bits(X.rnd(key, X.arange(r0 * DIM, (r0 + rows) * DIM)), GAUSS_BITS)).reshape(rows, DIM)
        if world is not None:
            hid = hidden_of_rows(X, seed, r0, r0 + rows)              # 4 fractional bits: LATENT_NOISE counts in sixteenths
            g = g * (16 * LATENT_NOISE)
            for k in range(LATENT_DIM):                               # integers: exact, whatever the order
                g = g + spread[k][None, :] * hid[:, k][:, None]
            g = X.shr_signed(g, 10)                                   # room for the exact sum of squares
        norm = X.sqrt(X.f64((g * g).sum(1)))
        out[r0:r0 + rows] = X.f32(X.f64(g) / norm[:, None])
    return X.to_torch(out)


def hybrid_set(n, nnz_splade, nnz_bm25, seed, device="cpu", force_backend=None):
    """(dense, s_off, s_idx, s_val, b_off, b_idx, b_val) for n rows."""
    dense = dense_rows(n, seed, device, force_backend=force_backend)
    s = sparse_rows(n, nnz_splade, "splade", seed, device, force_backend=force_backend)
    b = sparse_rows(n, nnz_bm25, "bm25", seed, device, force_backend=force_backend)
    return (dense,) + s + b


def latent_set(n, nnz_splade, nnz_bm25, seed, world, device="cpu", force_backend=None):
    dense = dense_rows(n, seed, device, force_backend=force_backend, world=world)
    s = sparse_rows(n, nnz_splade, "splade", seed, device, force_backend=force_backend, by_rarity=True)
    b = sparse_rows(n, nnz_bm25, "bm25", seed, device, force_backend=force_backend, by_rarity=True)
    return (dense,) + s + b


def latent_corpus(n, seed=20251125, world=20251201, device="cpu", force_backend=None):
    """A hybrid corpus in which a graph has something to find: a hidden 16-dimensional normal vector per row steers
    its dense vector, so rows have neighbours at every scale, as embedded text has; the terms are drawn as in corpus()
    (they carry no structure of their own) but valued by rarity and scaled so that the dense part carries about three
    quarters of a pair's score under 49 x dense + sparse + bm25. Not the distribution of corpus(): it stands next to the
    structureless one."""
    return latent_set(n, 120, 60, seed, world, device, force_backend)


def latent_queries(n, seed=20251126, world=20251201, device="cpu", force_backend=None):
    return latent_set(n, 30, 8, seed, world, device, force_backend)


def corpus(n, seed=20251125, device="cpu", force_backend=None):
    return hybrid_set(n, 120, 60, seed, device, force_backend)


def queries(n, seed=20251126, device="cpu", force_backend=None):
    return hybrid_set(n, 30, 8, seed, device, force_backend)


def _csr_from_degrees(X, deg, targets_n, key):
    off = X.cumsum0(deg)
    total = int(off[-1])
    idx = X.mod(X.rnd(key, X.arange(0, total)), targets_n)
    return X.to_torch(X.i32(off)), X.to_torch(X.i32(idx))


def knowledge_graph(n_entities, n_docs, n_queries, seed=20251127, device="cpu", mean_out=8.0, alpha=2.1, docs_per_entity=3.0,
                    force_backend=None):
    """(e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx): entity graph with power-law
    out-degree (exponent alpha, mean about mean_out), entity->doc lists with about
    docs_per_entity uniform docs, and 1-3 uniform entities per query."""
    X = backend(device, force_backend)
    # Pareto tail with density exponent alpha, x = xm * U^(-1/(alpha-1)), rounded to an integer degree:
    # P(degree <= d) = 1 - (xm / (d + 1/2))^(alpha-1); E[x] = xm*(alpha-1)/(alpha-2)
    xm = mean_out * (alpha - 2.0) / (alpha - 1.0)
    dmax = min(n_entities - 1, 4096)
    d = np.arange(0, dmax, dtype=np.float64)
    deg_cdf = np.where(d + 0.5 > xm, 1.0 - np.power(xm / (d + 0.5), alpha - 1.0), 0.0)  # searchsorted -> degree in [0, dmax]
    deg = X.searchsorted(X.table(deg_cdf), X.unit53(X.rnd(stream_key(seed, S_KG_DEG), X.arange(0, n_entities))))
    e2e = _csr_from_degrees(X, deg, n_entities, stream_key(seed, S_KG_E2E))
    # 1 + Poisson(docs_per_entity - 1) documents per entity
    lam = docs_per_entity - 1.0
    pk = [np.exp(-lam)]
    for k in range(1, 64):
        pk.append(pk[-1] * lam / k)
    pois_cdf = np.cumsum(np.array(pk, dtype=np.float64))
    ddeg = 1 + X.searchsorted(X.table(pois_cdf), X.unit53(X.rnd(stream_key(seed, S_KG_DDEG), X.arange(0, n_entities))))
    e2d = _csr_from_degrees(X, ddeg, n_docs, stream_key(seed, S_KG_E2D))
    qdeg = 1 + X.mod(X.rnd(stream_key(seed, S_KG_QDEG), X.arange(0, n_queries)), 3)
    q2e = _csr_from_degrees(X, qdeg, n_entities, stream_key(seed, S_KG_Q2E))
    return e2e + e2d + q2e


def to_numpy(arrays):
    """Torch tensors -> numpy (int32 offsets/ids viewed as uint32)."""
    out = []
    for a in arrays:
        a = a.detach().cpu().numpy()
        out.append(a.view(np.uint32) if a.dtype == np.int32 else a)
    return tuple(out)
