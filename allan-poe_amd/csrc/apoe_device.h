// Device-side building blocks shared by every kernel: the packed corpus record,
// wave64 reductions and sorts, the LDS term hash that a pivot's sparse terms are
// scattered into, and the wave-cooperative hybrid inner product.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace apoe {

constexpr int WAVE = 64;
constexpr uint32_t EMPTY = 0xFFFFFFFFu;
constexpr uint32_t FLAG = 0x80000000u;     // "explored"/"sampled" bit on a doc id
constexpr uint32_t BM25_BIT = 0x80000000u; // unified term key: bit31 set = BM25 term
constexpr uint32_t KW_HIT = 0x40000000u;   // keyword-filter search: pool id of a document that holds a required keyword
constexpr uint32_t ID_MASK = 0x3FFFFFFFu;  // doc id without the two flag bits
constexpr float INF_DIS = 1000000.0f;
constexpr int DIM = 1024;
constexpr int DENSE_BYTES = DIM * 4;
constexpr int NV = DIM / (4 * WAVE); // float4 loads per lane for one dense row

// Descriptor of one document: record offset (16-byte units) and the two pair counts.
constexpr int DESC_OFF_BITS = 36;
constexpr int DESC_NNZ_BITS = 14;
constexpr uint32_t DESC_NNZ_MAX = (1u << DESC_NNZ_BITS) - 1;
constexpr uint64_t DESC_OFF_MASK = (1ull << DESC_OFF_BITS) - 1;

__host__ __device__ inline uint64_t make_desc(uint64_t off16, uint32_t nnz_s, uint32_t nnz_b) {
    return off16 | ((uint64_t)nnz_s << DESC_OFF_BITS) | ((uint64_t)nnz_b << (DESC_OFF_BITS + DESC_NNZ_BITS));
}
__host__ __device__ inline uint64_t desc_off(uint64_t d) { return d & DESC_OFF_MASK; }
__host__ __device__ inline uint32_t desc_nnz_s(uint64_t d) { return (uint32_t)(d >> DESC_OFF_BITS) & DESC_NNZ_MAX; }
__host__ __device__ inline uint32_t desc_nnz_b(uint64_t d) { return (uint32_t)(d >> (DESC_OFF_BITS + DESC_NNZ_BITS)) & DESC_NNZ_MAX; }

// Record = [DIM floats][pairs], pairs = nnz_s SPLADE terms then nnz_b BM25 terms.
// Wide pairs:   nnz x (term | path bit, value), two 32-bit words each.
// Narrow pairs: nnz x value (f32), then nnz x term (u16); the path of pair j follows from j >= nnz_s.
// A corpus is narrow when every term id of both paths is below 65536 (6 instead of 8 bytes a pair).
// Records start on a 128-byte boundary, and so does the term array of a narrow record: a read of
// a row, of its values or of its terms then starts at a memory line and only its last line is partial.
constexpr uint32_t REC_ALIGN = 128;
struct CorpusView {
    const uint64_t* desc;
    const char* recs;
    const float* dnorm; // Euclidean norm of each dense row (bounds the dense inner product)
    uint32_t n;
    uint32_t narrow;
};

__host__ __device__ inline uint32_t narrow_keys_offset(uint32_t nnz) { // of the term array, from the first value
    return (4u * nnz + REC_ALIGN - 1) & ~(REC_ALIGN - 1);
}
__host__ __device__ inline uint64_t record_units(uint32_t nnz, bool narrow) { // 16-byte units of one record
    const uint64_t bytes = (uint64_t)DENSE_BYTES + (narrow ? (uint64_t)narrow_keys_offset(nnz) + 2ull * nnz : 8ull * nnz);
    return (bytes + REC_ALIGN - 1) / REC_ALIGN * (REC_ALIGN / 16);
}

struct SetView { // a set kept in CSR form on the device (queries)
    const float* dense;
    const uint32_t* s_off;
    const uint32_t* s_idx;
    const float* s_val;
    const uint32_t* b_off;
    const uint32_t* b_idx;
    const float* b_val;
    uint32_t n;
};

#ifdef __HIPCC__

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

// The path bit of pair j of a record with ns SPLADE pairs: narrow records do not store it.
__device__ __forceinline__ uint32_t pair_flag(uint32_t narrow, uint32_t ns, uint32_t j) { return narrow && j >= ns ? 0x80000000u : 0u; }

// The pair array of one record; [j] gives (term | path bit, value bits) whatever the format.
// `narrow` is the same for every record of a corpus, so the branch on it is uniform (the hot
// kernels make it a compile-time constant). raw(j) is the load alone: a kernel that wants the loads
// of several rows in flight takes raw pairs and ORs pair_flag() in where it consumes them, because
// an OR next to the load makes the wave wait for the load there.
struct Pairs {
    const char* base; // first byte after the dense row
    uint32_t ns, nnz; // SPLADE pairs, all pairs
    uint32_t narrow;
    __device__ __forceinline__ uint2 raw(uint32_t j) const {
        if (narrow) return make_uint2(reinterpret_cast<const uint16_t*>(base + narrow_keys_offset(nnz))[j], reinterpret_cast<const uint32_t*>(base)[j]);
        return reinterpret_cast<const uint2*>(base)[j];
    }
    __device__ __forceinline__ uint32_t key(uint32_t j) const {
        if (narrow) return (uint32_t) reinterpret_cast<const uint16_t*>(base + narrow_keys_offset(nnz))[j] | pair_flag(1, ns, j);
        return reinterpret_cast<const uint2*>(base)[j].x;
    }
    __device__ __forceinline__ uint2 operator[](uint32_t j) const {
        uint2 kv = raw(j);
        kv.x |= pair_flag(narrow, ns, j);
        return kv;
    }
};
__device__ __forceinline__ Pairs record_pairs(const CorpusView& C, const char* rec, uint32_t ns, uint32_t nb) {
    Pairs p;
    p.base = rec + DENSE_BYTES;
    p.ns = ns;
    p.nnz = ns + nb;
    p.narrow = C.narrow;
    return p;
}
__device__ __forceinline__ Pairs record_pairs(const CorpusView& C, uint64_t desc) {
    return record_pairs(C, C.recs + desc_off(desc) * 16, desc_nnz_s(desc), desc_nnz_b(desc));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// Sum over the wave with DPP adds inside each 16-lane row and four lane reads across rows;
// every lane gets the total.
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));  // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));  // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false)); // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false)); // row_mirror
    const int iv = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
}

// Total order on floats as unsigned integers (negative distances are common: 1 - IP).
__device__ __forceinline__ uint32_t float_key(float f) {
    uint32_t u = __float_as_uint(f);
    return u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ uint64_t dist_id_key(float d, uint32_t id) {
    return ((uint64_t)float_key(d) << 32) | id;
}

__device__ __forceinline__ uint64_t shfl_xor64(uint64_t v, int m) {
    uint32_t lo = __shfl_xor((uint32_t)v, m, WAVE), hi = __shfl_xor((uint32_t)(v >> 32), m, WAVE);
    return ((uint64_t)hi << 32) | lo;
}

// ---- LDS term hash: (key, value-bits) slots, open addressing, linear probing ----

__device__ __forceinline__ uint32_t term_hash(uint32_t key, uint32_t mask) {
    return ((key * 2654435761u) >> 12) & mask;
}

__device__ __forceinline__ void term_table_clear(uint2* tab, uint32_t slots, int tid, int nthreads) {
    for (uint32_t i = tid; i < slots; i += nthreads) tab[i] = make_uint2(EMPTY, 0u);
}

// Keys inserted into one table are distinct; the table has at least twice as many slots as keys.
__device__ __forceinline__ void term_table_insert(uint2* tab, uint32_t mask, uint32_t key, float val) {
    uint32_t h = term_hash(key, mask);
    while (true) {
        uint32_t old = atomicCAS(&tab[h].x, EMPTY, key);
        if (old == EMPTY || old == key) { tab[h].y = __float_as_uint(val); return; }
        h = (h + 1) & mask;
    }
}

// Returns true and adds value*stored on a hit.
__device__ __forceinline__ bool term_table_probe(const uint2* tab, uint32_t mask, uint32_t key, float val, float& acc) {
    uint32_t h = term_hash(key, mask);
    while (true) {
        uint2 e = tab[h];
        if (e.x == key) { acc = fmaf(val, __uint_as_float(e.y), acc); return true; }
        if (e.x == EMPTY) return false;
        h = (h + 1) & mask;
    }
}

// ---- pivot: the vector every candidate is compared with ----
// Dense part lives in registers (lane l owns float4 number l + 64*i of the row),
// sparse part lives in the LDS term table.
struct PivotDense {
    float4 v[NV];
};

__device__ __forceinline__ void pivot_dense_load(PivotDense& p, const float* row, float scale) {
    const float4* r = reinterpret_cast<const float4*>(row);
    const int lane = lane_id();
#pragma unroll
    for (int i = 0; i < NV; i++) {
        float4 x = r[lane + WAVE * i];
        p.v[i] = make_float4(x.x * scale, x.y * scale, x.z * scale, x.w * scale);
    }
}

// Insert the sparse part of a packed document record (all pairs, both paths).
__device__ __forceinline__ void pivot_terms_from_record(uint2* tab, uint32_t mask, const Pairs& sp, int tid, int nthreads) {
    for (uint32_t j = tid; j < sp.nnz; j += nthreads) {
        uint2 kv = sp[j];
        term_table_insert(tab, mask, kv.x, __uint_as_float(kv.y));
    }
}

// Insert the sparse part of CSR query q, values multiplied by the path weights; a
// path that is switched off inserts nothing.
__device__ __forceinline__ void pivot_terms_from_query(uint2* tab, uint32_t mask, const SetView& Q, uint32_t q, float w_s, float w_b,
                                                        bool use_s, bool use_b, int tid, int nthreads) {
    if (use_s)
        for (uint32_t j = Q.s_off[q] + tid; j < Q.s_off[q + 1]; j += nthreads) term_table_insert(tab, mask, Q.s_idx[j], Q.s_val[j] * w_s);
    if (use_b)
        for (uint32_t j = Q.b_off[q] + tid; j < Q.b_off[q + 1]; j += nthreads)
            term_table_insert(tab, mask, Q.b_idx[j] | BM25_BIT, Q.b_val[j] * w_b);
}

struct EvalOut {
    float ip;        // dense_mul * <dense> + <sparse pairs that hit the table>
    uint32_t nnz_s;  // SPLADE pairs read
    uint32_t nnz_b;  // BM25 pairs read
};

constexpr uint32_t PATH_DENSE = 1, PATH_SPARSE = 2, PATH_BM25 = 4;

// Read-only probe of a plain id set (keys only).
__device__ __forceinline__ bool id_set_contains(const uint32_t* set, uint32_t mask, uint32_t key) {
    uint32_t h = term_hash(key, mask);
    while (true) {
        const uint32_t e = set[h];
        if (e == key) return true;
        if (e == EMPTY) return false;
        h = (h + 1) & mask;
    }
}

// Insert into a plain id set; false if the key was already there.
__device__ __forceinline__ bool id_set_insert(uint32_t* set, uint32_t mask, uint32_t id) {
    uint32_t h = term_hash(id, mask);
    while (true) {
        uint32_t old = atomicCAS(&set[h], EMPTY, id);
        if (old == EMPTY) return true;
        if (old == id) return false;
        h = (h + 1) & mask;
    }
}

// One pair of the candidate against the pivot's table. With KW, a BM25 term of the
// candidate that the pivot lacks but the centre node's term set holds raises `kw`
// (the test of the build-time cal_bm25_dist, index.cu:128-153).
template <bool KW>
__device__ __forceinline__ void probe_pair(const uint2* tab, uint32_t mask, uint2 kv, float& acc, const uint32_t* uset, uint32_t umask, bool& kw) {
    const bool hit = term_table_probe(tab, mask, kv.x, __uint_as_float(kv.y), acc);
    if (KW) {
        if (!hit && (kv.x & BM25_BIT) && id_set_contains(uset, umask, kv.x)) kw = true;
    }
}

// Wave-cooperative hybrid inner product between the pivot and document `id`
// (wave-uniform). All 64 lanes must call it; every lane gets the result.
template <bool KW = false>
__device__ __forceinline__ EvalOut eval_wave(const CorpusView& C, uint32_t id, const PivotDense& pv, const uint2* tab, uint32_t mask,
                                             uint32_t paths, float dense_mul, const uint32_t* uset = nullptr, uint32_t umask = 0,
                                             bool* kw_any = nullptr) {
    const int lane = lane_id();
    const uint64_t desc = C.desc[id];
    const char* rec = C.recs + desc_off(desc) * 16;
    const uint32_t ns = desc_nnz_s(desc), nb = desc_nnz_b(desc);
    const uint32_t begin = (paths & PATH_SPARSE) ? 0u : ns;
    const uint32_t end = (paths & PATH_BM25) ? ns + nb : ns;
    const Pairs sp = record_pairs(C, rec, ns, nb);
    float4 x[NV];
    if (paths & PATH_DENSE) {
        const float4* r = reinterpret_cast<const float4*>(rec);
#pragma unroll
        for (int i = 0; i < NV; i++) x[i] = r[lane + WAVE * i];
    }
    // first three chunks of pairs are requested before anything is consumed
    uint2 kv0 = make_uint2(0, 0), kv1 = kv0, kv2 = kv0;
    const uint32_t j0 = begin + lane, j1 = j0 + WAVE, j2 = j1 + WAVE;
    if (j0 < end) kv0 = sp[j0];
    if (j1 < end) kv1 = sp[j1];
    if (j2 < end) kv2 = sp[j2];
    float acc = 0.f;
    if (paths & PATH_DENSE) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            acc = fmaf(x[i].x, pv.v[i].x, acc);
            acc = fmaf(x[i].y, pv.v[i].y, acc);
            acc = fmaf(x[i].z, pv.v[i].z, acc);
            acc = fmaf(x[i].w, pv.v[i].w, acc);
        }
        acc *= dense_mul;
    }
    bool kw = false;
    if (j0 < end) probe_pair<KW>(tab, mask, kv0, acc, uset, umask, kw);
    if (j1 < end) probe_pair<KW>(tab, mask, kv1, acc, uset, umask, kw);
    if (j2 < end) probe_pair<KW>(tab, mask, kv2, acc, uset, umask, kw);
    for (uint32_t j = j2 + WAVE; j < end; j += WAVE) probe_pair<KW>(tab, mask, sp[j], acc, uset, umask, kw);
    EvalOut o;
    o.ip = wave_sum(acc);
    o.nnz_s = (paths & PATH_SPARSE) ? ns : 0u;
    o.nnz_b = (paths & PATH_BM25) ? nb : 0u;
    if (KW) *kw_any = __ballot(kw) != 0;
    return o;
}

// ---- two-stage evaluation ----
// Stage 1 reads the candidate's descriptor, dense norm and pairs and forms the sparse sum.
// |<pivot_d, doc_d>| <= |pivot_d| * |doc_d|, so 1 - (sparse + dense_mul*|p|*|d|) - bonus is a lower
// bound of the distance: if even that is above `thr` (the value the caller would reject anyway: the
// worst entry of a full pool / list), the dense row is not read and INF_DIS is reported. Otherwise
// stage 2 reads the row. thr = +inf always gives the exact distance. The stages are separate calls
// so that a wave can have the loads of several candidates in flight before it consumes the first.
struct PendingEval {
    const char* rec;
    uint2 kv0, kv1, kv2; // raw pairs: the consumer adds pair_flag()
    uint32_t ns, nb, begin, end;
    float dub;
};

// desc / dnorm are the candidate's descriptor and dense norm (wave-uniform).
__device__ __forceinline__ void eval_issue_desc(PendingEval& p, const CorpusView& C, uint64_t desc, float dnorm, float pv_norm, uint32_t paths,
                                                float dense_mul) {
    const int lane = lane_id();
    p.rec = C.recs + desc_off(desc) * 16;
    p.ns = desc_nnz_s(desc);
    p.nb = desc_nnz_b(desc);
    p.begin = (paths & PATH_SPARSE) ? 0u : p.ns;
    p.end = (paths & PATH_BM25) ? p.ns + p.nb : p.ns;
    p.dub = (paths & PATH_DENSE) ? dense_mul * pv_norm * dnorm : 0.f;
    const Pairs sp = record_pairs(C, p.rec, p.ns, p.nb);
    const uint32_t j0 = p.begin + lane, j1 = j0 + WAVE, j2 = j1 + WAVE;
    p.kv0 = p.kv1 = p.kv2 = make_uint2(0, 0);
    // no per-lane branches: a lane past the end of the row loads the row's last pair again and the
    // consumer masks it (it tests j < end anyway)
    if (p.begin < p.end) {
        const uint32_t last = p.end - 1;
        p.kv0 = sp.raw(min(j0, last));
        p.kv1 = sp.raw(min(j1, last));
        p.kv2 = sp.raw(min(j2, last));
    }
}

// Lane `src` of a 64-bit / float register as a wave-uniform value (src is wave-uniform).
__device__ __forceinline__ uint64_t readlane64(uint64_t v, uint32_t src) {
    const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)v, src), hi = __builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), src);
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ float readlane_f32(float v, uint32_t src) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src));
}

// ---- query term tables for the search kernels ----
// One table per path (SPLADE first, BM25 second, each sized for the longest row of its path), two (key, value)
// entries per 16-byte bucket, so a lookup is ONE ds_read_b128 and no probe loop: every lane can issue
// the reads for all its pairs (of several candidates) back to back instead of walking a chain of
// dependent LDS reads whose length is set by the unluckiest lane. Keys are stored the way the record
// loads deliver them ("raw": without the path bit for narrow records, with it for wide ones), so a
// probe needs no operation on the loaded key besides the hash; the table is picked by the pair's
// path. A term whose bucket is already full goes to an overflow list that holds up to every term of
// the row (with at least twice as many buckets as terms it is empty for most rows); its length is
// wave-uniform and the list is only walked when it is not zero.
struct QueryTabs {
    uint4* b;        // [(mask_s + 1) + (mask_b + 1)] buckets: (key0, value0, key1, value1)
    uint2* ovf;      // overflow entries: (term | path bit, value)
    uint32_t* n_ovf; // their number
    uint32_t mask_s, mask_b; // buckets of the SPLADE / BM25 table - 1
};

// Hash of a raw key. The 24-bit multiply is a full-rate instruction (the 32-bit one is not).
template <bool NARROW>
__device__ __forceinline__ uint32_t query_hash(uint32_t raw) {
    if (NARROW) return __umul24(raw, 0x9E3779u) >> 10;
    const uint32_t k = raw & 0x7FFFFFFFu;
    return __umul24(k ^ (k >> 16), 0x9E3779u) >> 10;
}

__device__ __forceinline__ void query_tabs_clear(const QueryTabs& T, int tid, int nthreads) {
    for (uint32_t i = tid; i < T.mask_s + T.mask_b + 2; i += nthreads) T.b[i] = make_uint4(EMPTY, 0u, EMPTY, 0u);
    if (tid == 0) *T.n_ovf = 0;
}

// key carries the path bit; keys inserted into one table are distinct.
template <bool NARROW>
__device__ __forceinline__ void query_tabs_insert(const QueryTabs& T, uint32_t key, float val) {
    const uint32_t raw = NARROW ? key & ~BM25_BIT : key;
    const uint32_t h = query_hash<NARROW>(raw);
    uint4* e = T.b + ((key & BM25_BIT) ? T.mask_s + 1 + (h & T.mask_b) : (h & T.mask_s));
    if (atomicCAS(&e->x, EMPTY, raw) == EMPTY) { e->y = __float_as_uint(val); return; }
    if (atomicCAS(&e->z, EMPTY, raw) == EMPTY) { e->w = __float_as_uint(val); return; }
    T.ovf[atomicAdd(T.n_ovf, 1u)] = make_uint2(key, __float_as_uint(val));
}

template <bool NARROW>
__device__ __forceinline__ void query_tabs_fill(const QueryTabs& T, const SetView& Q, uint32_t q, float w_s, float w_b, bool use_s, bool use_b,
                                                int tid, int nthreads) {
    if (use_s)
        for (uint32_t j = Q.s_off[q] + tid; j < Q.s_off[q + 1]; j += nthreads) query_tabs_insert<NARROW>(T, Q.s_idx[j], Q.s_val[j] * w_s);
    if (use_b)
        for (uint32_t j = Q.b_off[q] + tid; j < Q.b_off[q + 1]; j += nthreads)
            query_tabs_insert<NARROW>(T, Q.b_idx[j] | BM25_BIT, Q.b_val[j] * w_b);
}

// The pairs of one candidate row on their way to a probe: three chunks of 64, raw keys and value
// bits per lane, and what the wave knows about the row. The loads are not clamped to the row (no
// address arithmetic per lane beyond lane * size): a lane past the end reads whatever follows the
// row (the record buffer ends with slack for that) and the probe masks it.
struct RowLoad {
    uint32_t k[3], v[3];
};
struct RowInfo { // wave-uniform
    const char* rec;
    uint32_t ns, nb;
    uint32_t begin; // first pair of the paths in use
    uint32_t n;     // pairs of the paths in use (0 for a candidate that is not there)
    uint32_t nsr;   // SPLADE pairs among them
};
constexpr uint32_t ROW_LOAD_SLACK = 3 * WAVE * 8; // bytes a row load may read past the last record

template <bool NARROW>
__device__ __forceinline__ void row_issue(RowLoad& r, RowInfo& s, const CorpusView& C, uint64_t desc, bool live, uint32_t paths) {
    const int lane = lane_id();
    s.rec = C.recs + desc_off(desc) * 16;
    s.ns = desc_nnz_s(desc);
    s.nb = desc_nnz_b(desc);
    s.begin = (paths & PATH_SPARSE) ? 0u : s.ns;
    const uint32_t end = (paths & PATH_BM25) ? s.ns + s.nb : s.ns;
    s.n = live ? end - s.begin : 0u;
    s.nsr = s.ns - s.begin;
    // a dense-only search reads no pairs: its (masked) loads all go to the first record and stay in the cache
    const char* from = (paths & (PATH_SPARSE | PATH_BM25)) ? s.rec : C.recs;
    if (NARROW) {
        const uint32_t* vals = reinterpret_cast<const uint32_t*>(from + DENSE_BYTES) + s.begin;
        const uint16_t* keys = reinterpret_cast<const uint16_t*>(from + DENSE_BYTES + narrow_keys_offset(s.ns + s.nb)) + s.begin;
#pragma unroll
        for (int c = 0; c < 3; c++) {
            r.k[c] = keys[lane + WAVE * c];
            r.v[c] = vals[lane + WAVE * c];
        }
    } else {
        const uint2* pairs = reinterpret_cast<const uint2*>(from + DENSE_BYTES) + s.begin;
#pragma unroll
        for (int c = 0; c < 3; c++) {
            const uint2 kv = pairs[lane + WAVE * c];
            r.k[c] = kv.x;
            r.v[c] = kv.y;
        }
    }
}

template <bool NARROW, bool KWD>
__device__ __forceinline__ void query_match(const uint4 e, uint32_t raw, uint32_t val_bits, bool valid, bool bm25, float& acc, const uint32_t* kwset,
                                            uint32_t kwmask, bool& hit) {
    const bool m0 = e.x == raw, m1 = e.z == raw;
    const float v = __uint_as_float(m0 ? e.y : e.w);
    const bool found = valid && (m0 || m1);
    const float next = fmaf(__uint_as_float(val_bits), v, acc);
    acc = found ? next : acc;
    if (KWD) {
        if (found && bm25 && id_set_contains(kwset, kwmask, raw | BM25_BIT)) hit = true;
    }
}

template <bool NARROW, bool KWD>
__device__ __forceinline__ void query_overflow(const QueryTabs& T, uint32_t n_ovf, uint32_t raw, uint32_t val_bits, bool valid, bool bm25, float& acc,
                                               const uint32_t* kwset, uint32_t kwmask, bool& hit) {
    const uint32_t key = NARROW ? raw | (bm25 ? BM25_BIT : 0u) : raw;
    for (uint32_t i = 0; i < n_ovf; i++) {
        const uint2 o = T.ovf[i];
        if (valid && o.x == key) {
            acc = fmaf(__uint_as_float(val_bits), __uint_as_float(o.y), acc);
            if (KWD) {
                if (bm25 && id_set_contains(kwset, kwmask, key)) hit = true;
            }
        }
    }
}

// The per-lane part of stage 1: this lane's pairs of the candidate against the query's tables.
// Straight-line code on purpose: the three bucket reads of a candidate are issued back to back.
// n_ovf is the (wave-uniform) overflow count read after the tables were built.
template <bool NARROW, bool KWD>
__device__ __forceinline__ float row_probe(const CorpusView& C, const RowLoad& r, const RowInfo& s, const QueryTabs& T, uint32_t n_ovf,
                                           const uint32_t* kwset, uint32_t kwmask, bool& hit) {
    const int lane = lane_id();
    float acc = 0.f;
    bool in[3], bm[3];
    uint4 e[3];
    const uint4* tab_s = T.b;
    const uint4* tab_b = T.b + T.mask_s + 1;
#pragma unroll
    for (int c = 0; c < 3; c++) {
        in[c] = lane < (int)s.n - WAVE * c;
        bm[c] = NARROW ? lane >= (int)s.nsr - WAVE * c : (int)r.k[c] < 0;
        e[c] = (bm[c] ? tab_b : tab_s)[query_hash<NARROW>(r.k[c]) & (bm[c] ? T.mask_b : T.mask_s)];
    }
    // keep the three reads together: nothing below may be scheduled between them
    asm volatile("" : "+v"(e[0].x), "+v"(e[1].x), "+v"(e[2].x));
#pragma unroll
    for (int c = 0; c < 3; c++) query_match<NARROW, KWD>(e[c], r.k[c], r.v[c], in[c], bm[c], acc, kwset, kwmask, hit);
    if (n_ovf) {
#pragma unroll
        for (int c = 0; c < 3; c++) query_overflow<NARROW, KWD>(T, n_ovf, r.k[c], r.v[c], in[c], bm[c], acc, kwset, kwmask, hit);
    }
    if (s.n > 3 * WAVE) { // rows with more than 192 pairs
        Pairs sp = record_pairs(C, s.rec, s.ns, s.nb);
        sp.narrow = NARROW ? 1u : 0u;
        for (uint32_t j = s.begin + 3 * WAVE + lane; j < s.begin + s.n; j += WAVE) {
            const uint2 kv = sp.raw(j);
            const bool b = NARROW ? j >= s.ns : (int)kv.x < 0;
            query_match<NARROW, KWD>((b ? tab_b : tab_s)[query_hash<NARROW>(kv.x) & (b ? T.mask_b : T.mask_s)], kv.x, kv.y, true, b, acc, kwset, kwmask,
                                     hit);
            query_overflow<NARROW, KWD>(T, n_ovf, kv.x, kv.y, true, b, acc, kwset, kwmask, hit);
        }
    }
    return acc;
}

// Sum inside each row of 16 lanes (every lane of a row gets its row's sum): four DPP adds.
__device__ __forceinline__ float row_sum_dpp(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));  // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));  // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false)); // row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false)); // row_mirror
    return v;
}

// The wave-level part of stage 1: reduce, then decide whether the dense row is needed at all.
struct SparseOut {
    float v;      // decided: the distance to report (INF_DIS if the bound rejects); else the sparse sum
    bool decided; // no dense row needed
};

__device__ __forceinline__ SparseOut sparse_decide(const PendingEval& p, float acc, uint32_t paths, float bonus, float thr) {
    SparseOut o;
    float ssum = 0.f;
    if (paths & (PATH_SPARSE | PATH_BM25)) {
        ssum = wave_sum_dpp(acc);
        if (!(paths & PATH_DENSE)) {
            o.v = 1.0f - ssum - bonus;
            o.decided = true;
            return o;
        }
        const float lb = 1.0f - (ssum + p.dub) - bonus;
        if (lb > thr + 1e-5f * (fabsf(ssum) + p.dub + fabsf(bonus) + 1.0f)) {
            o.v = INF_DIS;
            o.decided = true;
            return o;
        }
    }
    o.v = ssum;
    o.decided = false;
    return o;
}

struct DenseRow {
    float4 x[NV];
};
__device__ __forceinline__ void dense_issue(DenseRow& d, const char* rec) {
    const float4* r = reinterpret_cast<const float4*>(rec);
    const int lane = lane_id();
#pragma unroll
    for (int i = 0; i < NV; i++) d.x[i] = r[lane + WAVE * i];
}
// dense_mul * <row, pivot> with the pivot's dense row in LDS (float4 number l + 64*i belongs to lane l,
// as in PivotDense): frees 64 registers per lane for kernels that need the occupancy more.
__device__ __forceinline__ float dense_finish_lds(const DenseRow& d, const float4* pivot, float dense_mul) {
    const int lane = lane_id();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const float4 p = pivot[lane + WAVE * i];
        acc = fmaf(d.x[i].x, p.x, acc);
        acc = fmaf(d.x[i].y, p.y, acc);
        acc = fmaf(d.x[i].z, p.z, acc);
        acc = fmaf(d.x[i].w, p.w, acc);
    }
    return dense_mul * wave_sum_dpp(acc);
}
// The same with the row taken from the half-precision copy of the dense rows (2 KB instead of 4 KB): lane l
// loads the four halves that stand where its float4 number l + 64*i stands in the fp32 row, so the pivot is read
// from LDS exactly as above. Products and sums stay fp32.
struct DenseRowHalf {
    uint2 h[NV];
};
__device__ __forceinline__ void dense_issue_half(DenseRowHalf& d, const uint16_t* row) {
    const uint2* r = reinterpret_cast<const uint2*>(row);
    const int lane = lane_id();
#pragma unroll
    for (int i = 0; i < NV; i++) d.h[i] = r[lane + WAVE * i];
}
__device__ __forceinline__ float half_bits_to_float(uint32_t bits16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16); }
__device__ __forceinline__ float dense_finish_lds_half(const DenseRowHalf& d, const float4* pivot, float dense_mul) {
    const int lane = lane_id();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const float4 p = pivot[lane + WAVE * i];
        acc = fmaf(half_bits_to_float(d.h[i].x & 0xFFFFu), p.x, acc);
        acc = fmaf(half_bits_to_float(d.h[i].x >> 16), p.y, acc);
        acc = fmaf(half_bits_to_float(d.h[i].y & 0xFFFFu), p.z, acc);
        acc = fmaf(half_bits_to_float(d.h[i].y >> 16), p.w, acc);
    }
    return dense_mul * wave_sum_dpp(acc);
}
__device__ __forceinline__ float pivot_dense_norm_lds(const float4* pivot) {
    const int lane = lane_id();
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const float4 p = pivot[lane + WAVE * i];
        a += p.x * p.x + p.y * p.y + p.z * p.z + p.w * p.w;
    }
    return sqrtf(wave_sum_dpp(a));
}

// ---- four-entry bucket table: a document's terms as pivot (NN-Descent) ----
// Same idea as QueryTabs with 32-byte buckets (two ds_read_b128 per lookup), which keeps the table
// at 8 bytes per slot for rows of several hundred terms. A term whose bucket is full goes to the
// overflow list (wave-uniform length, walked only when not empty); should even that list be full,
// lookups fall back to scanning the pivot's own pair array in global memory (correct, slow, and
// not reachable with a hash that spreads the row's terms).
struct Bucket4Tab {
    uint4* b;        // [2 * (mask + 1)]: bucket i is b[2i], b[2i+1] = (k0, v0, k1, v1), (k2, v2, k3, v3)
    uint2* ovf;      // [ovf_cap]
    uint32_t* n_ovf; // terms that found their bucket full (may exceed ovf_cap)
    uint32_t mask, ovf_cap;
};

__device__ __forceinline__ void bucket4_clear(const Bucket4Tab& T, int tid, int nthreads) {
    for (uint32_t i = tid; i < 2 * (T.mask + 1); i += nthreads) T.b[i] = make_uint4(EMPTY, 0u, EMPTY, 0u);
    if (tid == 0) *T.n_ovf = 0;
}

__device__ __forceinline__ void bucket4_insert(const Bucket4Tab& T, uint32_t key, uint32_t val_bits) {
    uint4* e = T.b + 2 * term_hash(key, T.mask);
    if (atomicCAS(&e[0].x, EMPTY, key) == EMPTY) { e[0].y = val_bits; return; }
    if (atomicCAS(&e[0].z, EMPTY, key) == EMPTY) { e[0].w = val_bits; return; }
    if (atomicCAS(&e[1].x, EMPTY, key) == EMPTY) { e[1].y = val_bits; return; }
    if (atomicCAS(&e[1].z, EMPTY, key) == EMPTY) { e[1].w = val_bits; return; }
    const uint32_t at = atomicAdd(T.n_ovf, 1u);
    if (at < T.ovf_cap) T.ovf[at] = make_uint2(key, val_bits);
}

__device__ __forceinline__ void bucket4_terms_from_record(const Bucket4Tab& T, const Pairs& sp, int tid, int nthreads) {
    for (uint32_t j = tid; j < sp.nnz; j += nthreads) {
        const uint2 kv = sp[j];
        bucket4_insert(T, kv.x, kv.y);
    }
}

__device__ __forceinline__ bool bucket4_match(const uint4 e0, const uint4 e1, uint2 kv, bool valid, float& acc) {
    const bool m0 = e0.x == kv.x, m1 = e0.z == kv.x, m2 = e1.x == kv.x, m3 = e1.z == kv.x;
    const float v = __uint_as_float(m0 ? e0.y : m1 ? e0.w : m2 ? e1.y : e1.w);
    const bool found = valid && (m0 || m1 || m2 || m3);
    const float next = fmaf(__uint_as_float(kv.y), v, acc);
    acc = found ? next : acc;
    return found;
}

// Terms that are not in their bucket: the overflow list, or the pivot's pair array if the list overflowed.
__device__ __forceinline__ void bucket4_overflow(const Bucket4Tab& T, uint32_t n_ovf, const Pairs& pivot_pairs, uint2 kv, bool pending, float& acc) {
    if (n_ovf <= T.ovf_cap) {
        for (uint32_t i = 0; i < n_ovf; i++) {
            const uint2 o = T.ovf[i];
            if (pending && o.x == kv.x) acc = fmaf(__uint_as_float(kv.y), __uint_as_float(o.y), acc);
        }
    } else {
        for (uint32_t i = 0; i < pivot_pairs.nnz; i++) {
            const uint2 o = pivot_pairs[i];
            if (pending && o.x == kv.x) acc = fmaf(__uint_as_float(kv.y), __uint_as_float(o.y), acc);
        }
    }
}

// Per-lane part of stage 1 against a document pivot (all paths on).
__device__ __forceinline__ float doc_sparse_probe(const CorpusView& C, const PendingEval& p, const Bucket4Tab& T, uint32_t n_ovf,
                                                  const Pairs& pivot_pairs) {
    const int lane = lane_id();
    float acc = 0.f;
    const uint32_t j0 = p.begin + lane, j1 = j0 + WAVE, j2 = j1 + WAVE;
    const bool in0 = j0 < p.end, in1 = j1 < p.end, in2 = j2 < p.end;
    const uint2 kv0 = make_uint2(p.kv0.x | pair_flag(C.narrow, p.ns, j0), p.kv0.y);
    const uint2 kv1 = make_uint2(p.kv1.x | pair_flag(C.narrow, p.ns, j1), p.kv1.y);
    const uint2 kv2 = make_uint2(p.kv2.x | pair_flag(C.narrow, p.ns, j2), p.kv2.y);
    const uint4* b0 = T.b + 2 * term_hash(kv0.x, T.mask);
    const uint4* b1 = T.b + 2 * term_hash(kv1.x, T.mask);
    const uint4* b2 = T.b + 2 * term_hash(kv2.x, T.mask);
    uint4 e00 = b0[0], e01 = b0[1], e10 = b1[0], e11 = b1[1], e20 = b2[0], e21 = b2[1];
    // keep the six reads together: nothing below may be scheduled between them
    asm volatile("" : "+v"(e00.x), "+v"(e01.x), "+v"(e10.x), "+v"(e11.x), "+v"(e20.x), "+v"(e21.x));
    const bool f0 = bucket4_match(e00, e01, kv0, in0, acc);
    const bool f1 = bucket4_match(e10, e11, kv1, in1, acc);
    const bool f2 = bucket4_match(e20, e21, kv2, in2, acc);
    if (n_ovf) {
        bucket4_overflow(T, n_ovf, pivot_pairs, kv0, in0 && !f0, acc);
        bucket4_overflow(T, n_ovf, pivot_pairs, kv1, in1 && !f1, acc);
        bucket4_overflow(T, n_ovf, pivot_pairs, kv2, in2 && !f2, acc);
    }
    if (p.begin + 3 * WAVE < p.end) { // rows with more than 192 pairs
        const Pairs sp = record_pairs(C, p.rec, p.ns, p.nb);
        for (uint32_t j = j2 + WAVE; j < p.end; j += WAVE) {
            const uint2 kv = sp[j];
            const uint4* bb = T.b + 2 * term_hash(kv.x, T.mask);
            const bool f = bucket4_match(bb[0], bb[1], kv, true, acc);
            if (n_ovf) bucket4_overflow(T, n_ovf, pivot_pairs, kv, !f, acc);
        }
    }
    return acc;
}

// splitmix64 finaliser (random initial neighbours).
__host__ __device__ inline uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

#endif // __HIPCC__

} // namespace apoe
