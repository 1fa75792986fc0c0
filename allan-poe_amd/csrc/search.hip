// Greedy beam search over the hybrid graph: one workgroup per query; the candidate pool, the
// query's dense row, its sparse-term tables and the fresh-neighbour list in LDS; an exact
// visited bitmap per workgroup in HBM.
#include <mutex>

#include "apoe_internal.h"

namespace apoe {

constexpr int MAX_NEW = 64;   // fresh candidates per step: one lane each in wave 0
// Tuning constants: the measured best on MI355X.
#define APOE_SEARCH_WAVES_PER_EU 6 // plain search: 12 queries per CU fit its LDS; the other modes need more LDS per query and stay at 5 (a macro: it sits in an attribute)
constexpr int EVAL_BATCH = 3;  // candidates whose sparse parts a wave keeps in flight together
constexpr int DENSE_BATCH = 1; // dense rows a wave keeps in flight together
constexpr int MERGE_ROUNDS = 4; // 64-element rounds of the pool that the merge moves per LDS round trip
constexpr int RING = 32;      // keyword-filter search: evicted keyword hits kept beside the pool (query.cu:18)

// What the kernel does on top of the plain beam search.
enum SearchMode { MODE_PLAIN = 0, MODE_KG = 1, MODE_KEYWORD = 2 };

// Arguments that a query needs once (when it starts or ends) stay in device memory and are read
// where they are used; the rest travels by value. Scalar registers are the scarce resource of this
// kernel: every argument held in one for the whole launch pushes loop state into vector registers.
struct SearchCold {
    SetView Q;
    const uint32_t* entry;
    uint32_t n_entry;
    float w_d, w_s, w_b;
    uint32_t q_begin;
    uint32_t* out_ids;
    float* out_dist;
    const uint32_t *q2e_off, *q2e_idx;
};

struct SearchArgs {
    CorpusView C;
    const SearchCold* cold;
    const uint32_t* graph;
    uint32_t W, degree;
    uint32_t paths;
    uint32_t cands, max_iter, q_count;
    uint32_t* bitmaps;     // one visited bitmap per workgroup
    uint32_t bitmap_words; // multiple of 4
    unsigned long long* work; // [0] next query, [1] expansions, [2] evaluations, [3] nnz splade, [4] nnz bm25, [5] dense rows read,
                              // [6] pool entries evaluated again in fp32, [7] their pairs
    uint32_t full_eval;       // 1: read the dense row of every candidate (no bound test)
    const uint16_t* half;     // not null: the walk takes dense parts from the half-precision rows, the final pool is evaluated again in fp32
    uint32_t slots_s, slots_b, ovf_cap; // buckets of the query's SPLADE / BM25 term table, entries of the overflow list
    // knowledge graph (KG kernels only)
    const uint32_t *e2e_off, *e2e_idx, *e2d_off, *e2d_idx;
    uint32_t n_entities;
    float kg_weight;
    uint32_t kw_slots; // keyword-filter kernels only: slots of the per-query keyword term set
};

// LDS carve-up shared by host (size) and device (pointers).
struct SearchLds {
    uint32_t qd, stat, part, tab, ovf, pool_id, pool_dist, pool_ent, pool_hop, new_lb, new_id, new_dist, new_ent, new_hop, seed_id, seed_ent, seed_dist, link, ring_id,
        ring_dist, kwset, ctl, total;
    __host__ __device__ SearchLds(uint32_t slots_s, uint32_t slots_b, uint32_t ovf_cap, uint32_t cands, int mode, uint32_t kw_slots) {
        const bool kg = mode == MODE_KG, kwd = mode == MODE_KEYWORD;
        // fixed-size arrays first: their offsets are compile-time constants
        uint32_t o = 0;
        qd = o; o += DENSE_BYTES;       // the query's dense row, weight applied
        ctl = o; o += 16 * 4;
        stat = o; o += 8 * 8;           // the workgroup's counters (work[1..7]), sent once when it leaves
        part = o; o += MAX_NEW * 16;    // sparse sum of a fresh candidate as four partial sums (one per 16 lanes)
        new_lb = o; o += MAX_NEW * 4;
        new_id = o; o += MAX_NEW * 4;
        new_dist = o; o += MAX_NEW * 4;
        new_ent = o; o += kg || kwd ? MAX_NEW * 4 : 0; // KG: linking entity; keyword search: the hit flag of a fresh candidate
        new_hop = o; o += kg ? MAX_NEW * 4 : 0;
        link = o; o += kg ? MAX_NEW * 4 : 0;
        ring_id = o; o += kwd ? RING * 4 : 0;
        ring_dist = o; o += kwd ? RING * 4 : 0;
        tab = o; o += (slots_s + slots_b) * 16; // two tables (SPLADE, BM25) of buckets of two (key, value) entries; twice as many
                                                // buckets as the longest row of the path has terms keep overflows rare
        ovf = o; o += ovf_cap * 8;              // overflow entries: up to every term of the longest query row
        pool_id = o; o += cands * 4;
        pool_dist = o; o += cands * 4;
        pool_ent = o; o += kg ? cands * 4 : 0;
        pool_hop = o; o += kg ? cands * 4 : 0;
        seed_id = o; o += kg ? (cands + MAX_NEW) * 4 : 0;
        seed_ent = o; o += kg ? (cands + MAX_NEW) * 4 : 0;
        seed_dist = o; o += kg ? (cands + MAX_NEW) * 4 : 0;
        kwset = o; o += kwd ? kw_slots * 4 : 0;
        total = o;
    }
};

enum { CTL_QUERY = 0, CTL_PARENT = 1, CTL_NNEW = 2, CTL_NSEED = 3, CTL_NOVF = 4 };

struct Pool {
    uint32_t* id;   // [cands], ascending distance
    float* dist;    // [cands]
    uint32_t* ent;  // KG only
    uint32_t* hop;  // KG only
    uint32_t* lb;   // [MAX_NEW] scratch of the merge
    uint32_t cands;
};

// Keyword-filter search: pool entries that carry KW_HIT and fall off the pool. Entries are
// appended merge by merge, within one merge from the worst to the best, and slot (count % RING)
// is overwritten, so the ring holds the RING most recent ones: distances never grow along that
// sequence, which makes them the closest evicted hits (query.cu:244-248 appends in atomic order).
struct Ring {
    uint32_t* id;
    float* dist;
    uint32_t n; // appended so far (wave-uniform, wave 0)
};

__device__ __forceinline__ void wave_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Wave 0 only. Orders the n (<= 64) new candidates by (distance, id) and merges them into the
// sorted pool in place: a pool element keeps rank pos + #{new <= it}, a new element takes rank
// pos + #{pool < it}, so on equal distance the new one goes first (query.cu:181-224); ranks >=
// cands fall off. With lb_i = #{pool < new_i}: new_i <= pool[p]  <=>  lb_i <= p, so a pool element
// moves up by the number of new elements whose lb is <= its position, and nothing below lb_0
// moves at all -- only the 64-element rounds from the top down to lb_0 are touched (each round
// is read into registers before anything at or above it is written). Returns the lowest rank a
// new element took (cands if none entered).
// Keyword-filter search: nent[i] != 0 says that new candidate i holds a required keyword; it
// enters the pool with KW_HIT set on its id (ordering uses the plain id).
template <int MODE>
__device__ __forceinline__ uint32_t sort_merge(const Pool& P, uint32_t* nid, float* ndist, uint32_t* nent, uint32_t* nhop, uint32_t n, Ring& R) {
    constexpr bool KG = MODE == MODE_KG, KWD = MODE == MODE_KEYWORD;
    const int lane = lane_id();
    const uint32_t cands = P.cands;
    if (n == 0) return cands;
    // a candidate beyond the pool's worst entry cannot enter (with a full pool that is most of them:
    // everything the bound rejected, and more): only the others are ordered and merged
    float d = INF_DIS;
    uint32_t id = EMPTY, ent = EMPTY, hop = 0, rank = 0;
    if (lane < (int)n) d = ndist[lane];
    const bool keep = lane < (int)n && d <= P.dist[cands - 1];
    const uint64_t kept = __ballot(keep);
    if (kept == 0) return cands;
    // order by counting: rank = #{kept (d, id) pairs below mine}; ids are distinct
    if (keep) {
        id = nid[lane];
        if (KG) { ent = nent[lane]; hop = nhop[lane]; }
        if (KWD) ent = nent[lane];
    }
    for (uint64_t rest = kept; rest; rest &= rest - 1) {
        const uint32_t i = __builtin_ctzll(rest); // wave-uniform
        const float di = ndist[i];
        const uint32_t ii = nid[i];
        rank += (di < d) || (di == d && ii < id);
    }
    wave_fence();
    if (keep) {
        ndist[rank] = d;
        nid[rank] = id;
        if (KG) { nent[rank] = ent; nhop[rank] = hop; }
        if (KWD) nent[rank] = ent;
    }
    n = __popcll(kept);
    wave_fence();
    // lane i now takes the i-th smallest
    uint32_t lb = cands;
    if (lane < (int)n) {
        d = ndist[lane];
        id = nid[lane];
        if (KG) { ent = nent[lane]; hop = nhop[lane]; }
        if (KWD) id |= nent[lane] ? KW_HIT : 0u;
        if (d <= P.dist[cands - 1]) {
            uint32_t lo = 0, len = cands;
            while (len > 0) {
                const uint32_t half = len >> 1;
                if (P.dist[lo + half] < d) { lo += half + 1; len -= half + 1; } else len = half;
            }
            lb = lo;
        }
        P.lb[lane] = lb;
    }
    const bool enters = lane < (int)n && lb + lane < cands;
    const uint32_t n_in = __popcll(__ballot(enters)); // ranks grow with the lane: the first n_in enter
    if (n_in == 0) return cands;
    wave_fence();
    if (KWD) {
        // exactly the last n_in pool entries fall off; lane l looks at the l-th from the end
        uint32_t eid = EMPTY;
        float ed = 0.f;
        if ((uint32_t)lane < n_in) { eid = P.id[cands - 1 - lane]; ed = P.dist[cands - 1 - lane]; }
        const bool hit = eid != EMPTY && (eid & KW_HIT);
        const uint64_t hb = __ballot(hit);
        const uint32_t cnt = __popcll(hb), rank = __popcll(hb & ((1ull << lane) - 1));
        if (hit && rank + RING >= cnt) {
            const uint32_t slot = (R.n + rank) % RING;
            R.id[slot] = eid & ID_MASK;
            R.dist[slot] = ed;
        }
        R.n += cnt;
        wave_fence();
    }
    const uint32_t lo0 = uniform(P.lb[0]);
    // MERGE_ROUNDS rounds are read before any of them is written: one LDS round trip per group, and a
    // group only writes at or above its own positions (into rounds that were moved before it)
    for (int top = (int)((cands - 1) & ~(uint32_t)(WAVE - 1)); top >= 0 && (uint32_t)top + WAVE > lo0; top -= WAVE * MERGE_ROUNDS) {
        float v[MERGE_ROUNDS];
        uint32_t pid[MERGE_ROUNDS], pent[MERGE_ROUNDS], phop[MERGE_ROUNDS], dst[MERGE_ROUNDS];
#pragma unroll
        for (int r = 0; r < MERGE_ROUNDS; r++) {
            const int base = top - r * WAVE;
            const uint32_t p = (uint32_t)(base + lane);
            const bool act = base >= 0 && (uint32_t)base + WAVE > lo0 && p >= lo0 && p < cands;
            dst[r] = cands; // nothing to write
            v[r] = 0.f;
            pid[r] = pent[r] = phop[r] = 0;
            if (act) {
                v[r] = P.dist[p];
                pid[r] = P.id[p];
                if (KG) { pent[r] = P.ent[p]; phop[r] = P.hop[p]; }
                uint32_t shift = 0;
                for (uint32_t i = 0; i < n_in; i++) shift += (uint32_t)__builtin_amdgcn_readlane((int)lb, i) <= p;
                dst[r] = p + shift;
            }
        }
        wave_fence();
#pragma unroll
        for (int r = 0; r < MERGE_ROUNDS; r++) {
            if (dst[r] < cands) {
                P.dist[dst[r]] = v[r];
                P.id[dst[r]] = pid[r];
                if (KG) { P.ent[dst[r]] = pent[r]; P.hop[dst[r]] = phop[r]; }
            }
        }
        wave_fence();
    }
    if (enters) {
        P.dist[lb + lane] = d;
        P.id[lb + lane] = id;
        if (KG) { P.ent[lb + lane] = ent; P.hop[lb + lane] = hop; }
    }
    wave_fence();
    return lo0;
}

template <int NW, int MODE, bool NARROW, bool HALF>
__global__ __launch_bounds__(NW* WAVE) __attribute__((amdgpu_waves_per_eu(MODE == MODE_PLAIN && !HALF ? APOE_SEARCH_WAVES_PER_EU : 5, 8))) void search_kernel(SearchArgs a) {
    constexpr bool KG = MODE == MODE_KG, KWD = MODE == MODE_KEYWORD;
    a.C.narrow = NARROW ? 1u : 0u; // the pair format as a compile-time constant: no branch at the loads
    extern __shared__ __align__(16) char smem[];
    const SearchLds L(a.slots_s, a.slots_b, a.ovf_cap, a.cands, MODE, a.kw_slots);
    volatile uint32_t* ctl = reinterpret_cast<volatile uint32_t*>(smem + L.ctl);
    float4* qd = reinterpret_cast<float4*>(smem + L.qd);
    float* part = reinterpret_cast<float*>(smem + L.part);
    QueryTabs T;
    T.b = reinterpret_cast<uint4*>(smem + L.tab);
    T.ovf = reinterpret_cast<uint2*>(smem + L.ovf);
    T.n_ovf = const_cast<uint32_t*>(&ctl[CTL_NOVF]);
    T.mask_s = a.slots_s - 1;
    T.mask_b = a.slots_b - 1;
    Pool P;
    P.id = reinterpret_cast<uint32_t*>(smem + L.pool_id);
    P.dist = reinterpret_cast<float*>(smem + L.pool_dist);
    P.ent = reinterpret_cast<uint32_t*>(smem + L.pool_ent);
    P.hop = reinterpret_cast<uint32_t*>(smem + L.pool_hop);
    P.lb = reinterpret_cast<uint32_t*>(smem + L.new_lb);
    P.cands = a.cands;
    uint32_t* new_id = reinterpret_cast<uint32_t*>(smem + L.new_id);
    float* new_dist = reinterpret_cast<float*>(smem + L.new_dist);
    uint32_t* new_ent = reinterpret_cast<uint32_t*>(smem + L.new_ent);
    uint32_t* new_hop = reinterpret_cast<uint32_t*>(smem + L.new_hop);
    uint32_t* seed_id = reinterpret_cast<uint32_t*>(smem + L.seed_id);
    uint32_t* seed_ent = reinterpret_cast<uint32_t*>(smem + L.seed_ent);
    float* seed_dist = reinterpret_cast<float*>(smem + L.seed_dist);
    uint32_t* link = reinterpret_cast<uint32_t*>(smem + L.link);
    uint32_t* kwset = reinterpret_cast<uint32_t*>(smem + L.kwset);
    Ring R;
    R.id = reinterpret_cast<uint32_t*>(smem + L.ring_id);
    R.dist = reinterpret_cast<float*>(smem + L.ring_dist);
    R.n = 0;

    const int tid = threadIdx.x, wave = (int)uniform(tid / WAVE), lane = lane_id();
    const uint32_t cands = a.cands;
    uint32_t* bitmap = a.bitmaps + (size_t)blockIdx.x * a.bitmap_words;
    const uint64_t lane_lt = (1ull << lane) - 1;

    unsigned long long* stat = reinterpret_cast<unsigned long long*>(smem + L.stat);
    if (tid < 8) stat[tid] = 0;
    while (true) {
        __syncthreads();
        if (tid == 0) ctl[CTL_QUERY] = (uint32_t)atomicAdd(a.work, 1ull);
        __syncthreads();
        const uint32_t qi = uniform(ctl[CTL_QUERY]);
        if (qi >= a.q_count) break;
        const uint32_t q = a.cold->q_begin + qi;

        // ---- reset per-query state ----
        {
            uint4* b4 = reinterpret_cast<uint4*>(bitmap);
            for (uint32_t i = tid; i < a.bitmap_words / 4; i += NW * WAVE) b4[i] = make_uint4(0, 0, 0, 0);
        }
        query_tabs_clear(T, tid, NW * WAVE);
        if (KWD) {
            for (uint32_t i = tid; i < a.kw_slots; i += NW * WAVE) kwset[i] = EMPTY;
            R.n = 0;
        }
        for (uint32_t i = tid; i < cands; i += NW * WAVE) {
            P.id[i] = EMPTY;
            P.dist[i] = INF_DIS;
            if (KG) { P.ent[i] = EMPTY; P.hop[i] = 0; }
        }
        {
            const float4* src = reinterpret_cast<const float4*>(a.cold->Q.dense + (size_t)q * DIM);
            for (uint32_t i = tid; i < DIM / 4; i += NW * WAVE) {
                const float4 x = src[i];
                qd[i] = make_float4(x.x * a.cold->w_d, x.y * a.cold->w_d, x.z * a.cold->w_d, x.w * a.cold->w_d);
            }
        }
        __threadfence();
        __syncthreads();
        query_tabs_fill<NARROW>(T, a.cold->Q, q, a.cold->w_s, a.cold->w_b, a.paths & PATH_SPARSE, a.paths & PATH_BM25, tid, NW * WAVE);
        if (KWD) {
            // required keywords: BM25 query terms whose id arrives with bit 31 set (query.cu:1828-1843)
            for (uint32_t j = a.cold->Q.b_off[q] + tid; j < a.cold->Q.b_off[q + 1]; j += NW * WAVE) {
                const uint32_t t = a.cold->Q.b_idx[j];
                if (t & BM25_BIT) id_set_insert(kwset, a.kw_slots - 1, t);
            }
        }

        __syncthreads();
        const float pv_norm = pivot_dense_norm_lds(qd);
        uint64_t st_exp = 0, st_eval = 0, st_dense = 0, st_again = 0, st_again_pairs = 0; // wave-uniform counters
        uint32_t ln_s = 0, ln_b = 0;                    // pairs read for the candidates this lane decided
        uint32_t hint = 0;                                       // wave 0: every pool slot below hint is explored

        // ---- seeds ----
        if (!KG) {
            // entry points (query.cu:440-485)
            if (wave == 0) {
                uint32_t c = lane < (int)a.cold->n_entry ? a.cold->entry[lane] : EMPTY;
                bool fresh = false;
                if (c < a.C.n) {
                    const uint32_t bit = 1u << (c & 31);
                    fresh = !(atomicOr(&bitmap[c >> 5], bit) & bit);
                }
                const uint64_t b = __ballot(fresh);
                if (fresh) new_id[__popcll(b & lane_lt)] = c;
                if (lane == 0) { ctl[CTL_NNEW] = __popcll(b); ctl[CTL_PARENT] = 0; }
            }
            __syncthreads();
        } else {
            // documents of the query's entities first, entry points only if those do not
            // fill the pool (query.cu:1577-1604); at most cands + degree seeds
            if (wave == 0) {
                const uint32_t seed_cap = cands + a.degree;
                uint32_t n_seed = 0;
                const uint32_t qe0 = uniform(a.cold->q2e_off[q]), qe1 = uniform(a.cold->q2e_off[q + 1]);
                for (uint32_t i = qe0; i < qe1; i++) {
                    const uint32_t e = uniform(a.cold->q2e_idx[i]);
                    if (e >= a.n_entities) continue;
                    const uint32_t d0 = uniform(a.e2d_off[e]), d1 = uniform(a.e2d_off[e + 1]);
                    for (uint32_t b0 = d0; b0 < d1; b0 += WAVE) {
                        const uint32_t doc = b0 + lane < d1 ? a.e2d_idx[b0 + lane] : EMPTY;
                        bool fresh = false;
                        if (doc < a.C.n) {
                            const uint32_t bit = 1u << (doc & 31);
                            fresh = !(atomicOr(&bitmap[doc >> 5], bit) & bit);
                        }
                        const uint64_t b = __ballot(fresh);
                        const uint32_t pos = n_seed + __popcll(b & lane_lt);
                        if (fresh && pos < seed_cap) { seed_id[pos] = doc; seed_ent[pos] = e; }
                        n_seed = min(seed_cap, n_seed + (uint32_t)__popcll(b));
                    }
                }
                if (n_seed < cands) {
                    const uint32_t c = lane < (int)a.cold->n_entry ? a.cold->entry[lane] : EMPTY;
                    bool fresh = false;
                    if (c < a.C.n) {
                        const uint32_t bit = 1u << (c & 31);
                        fresh = !(atomicOr(&bitmap[c >> 5], bit) & bit);
                    }
                    const uint64_t b = __ballot(fresh);
                    const uint32_t pos = n_seed + __popcll(b & lane_lt);
                    if (fresh && pos < seed_cap) { seed_id[pos] = c; seed_ent[pos] = EMPTY; }
                    n_seed = min(seed_cap, n_seed + (uint32_t)__popcll(b));
                }
                if (lane == 0) ctl[CTL_NSEED] = n_seed;
            }
            __syncthreads();
            const uint32_t n_seed = uniform(ctl[CTL_NSEED]);
            const uint32_t n_ovf_seed = uniform(ctl[CTL_NOVF]);
            for (uint32_t j = wave; j < n_seed; j += NW) {
                const uint32_t id = uniform(seed_id[j]);
                const float bonus = seed_ent[j] != EMPTY ? a.kg_weight : 0.0f; // query.cu:1637-1638
                RowLoad rl;
                RowInfo ri;
                row_issue<NARROW>(rl, ri, a.C, a.C.desc[id], true, a.paths);
                bool hit = false;
                const float acc = row_probe<NARROW, false>(a.C, rl, ri, T, n_ovf_seed, nullptr, 0, hit);
                const float ssum = (a.paths & (PATH_SPARSE | PATH_BM25)) ? wave_sum_dpp(acc) : 0.f;
                float dist = 1.0f - ssum - bonus;
                if (a.paths & PATH_DENSE) { // seeds are never dropped by the bound
                    DenseRow row;
                    dense_issue(row, ri.rec);
                    dist = 1.0f - (dense_finish_lds(row, qd, 1.0f) + ssum) - bonus;
                    st_dense++;
                }
                st_eval++;
                if (lane == 0) {
                    ln_s += (a.paths & PATH_SPARSE) ? ri.ns : 0u;
                    ln_b += (a.paths & PATH_BM25) ? ri.nb : 0u;
                    seed_dist[j] = dist;
                }
            }
            __syncthreads();
            if (wave == 0) {
                for (uint32_t b0 = 0; b0 < n_seed; b0 += WAVE) {
                    const uint32_t nb = min((uint32_t)WAVE, n_seed - b0);
                    if (lane < (int)nb) {
                        new_id[lane] = seed_id[b0 + lane];
                        new_dist[lane] = seed_dist[b0 + lane];
                        new_ent[lane] = seed_ent[b0 + lane];
                        new_hop[lane] = 0;
                    }
                    wave_fence();
                    sort_merge<MODE>(P, new_id, new_dist, new_ent, new_hop, nb, R);
                }
                if (lane == 0) { ctl[CTL_NNEW] = 0; ctl[CTL_PARENT] = 0; }
            }
            __syncthreads();
        }

        for (uint32_t it = 0; it <= a.max_iter; it++) {
            // ---- evaluate the fresh candidates: one wave per candidate ----
            const uint32_t n_new = uniform(ctl[CTL_NNEW]);
            if (uniform(ctl[CTL_PARENT]) == EMPTY) break;
            // a candidate that provably cannot enter the (full) pool is dropped after its sparse part:
            // it is reported as INF_DIS and falls off the end of the merge like any other loser
            const float thr = a.full_eval ? __builtin_inff() : P.dist[cands - 1];
            const float thr_eff = thr < INF_DIS ? thr : __builtin_inff();
            const uint32_t n_ovf = uniform(ctl[CTL_NOVF]);
            // descriptors and dense norms of all fresh candidates in one gather: lane l holds candidate l's
            uint64_t my_desc = 0;
            float my_dn = 0.f;
            if ((uint32_t)lane < n_new) {
                const uint32_t cid = new_id[lane];
                my_desc = a.C.desc[cid];
                my_dn = a.C.dnorm[cid];
            }
            // stage 1: the sparse parts of this wave's candidates (wave + k * NW), EVAL_BATCH of them in flight.
            // No branch on whether a candidate of the batch exists: one that does not is a row of no pairs,
            // so the loads of the whole batch are issued back to back.
            for (uint32_t j = wave; j < n_new; j += NW * EVAL_BATCH) {
                RowLoad rl[EVAL_BATCH];
                RowInfo ri[EVAL_BATCH];
#pragma unroll
                for (int b = 0; b < EVAL_BATCH; b++) {
                    const uint32_t jj = j + b * NW;
                    row_issue<NARROW>(rl[b], ri[b], a.C, readlane64(my_desc, jj & (WAVE - 1)), jj < n_new, a.paths);
                }
                float acc[EVAL_BATCH];
                bool hit[EVAL_BATCH];
#pragma unroll
                for (int b = 0; b < EVAL_BATCH; b++) {
                    hit[b] = false;
                    acc[b] = row_probe<NARROW, KWD>(a.C, rl[b], ri[b], T, n_ovf, kwset, a.kw_slots - 1, hit[b]);
                }
#pragma unroll
                for (int b = 0; b < EVAL_BATCH; b++) {
                    const uint32_t jj = j + b * NW;
                    const float rs = row_sum_dpp(acc[b]);
                    if (jj < n_new) {
                        if ((lane & 15) == 0) part[jj * 4 + (lane >> 4)] = rs;
                        if (KWD) {
                            const bool kw_hit = __ballot(hit[b]) != 0;
                            if (lane == 0) new_ent[jj] = kw_hit ? 1u : 0u;
                        }
                    }
                }
            }
            wave_fence();
            // the decision for all of the wave's candidates at once, lane l for candidate l: a candidate whose
            // sparse part plus the bound of its dense part cannot reach the pool is reported as INF_DIS
            uint64_t need; // bit l: candidate l still needs its dense row
            {
                const bool mine = (uint32_t)lane < n_new && (uint32_t)(lane & (NW - 1)) == (uint32_t)wave;
                bool undecided = false;
                if (mine) {
                    float bonus = 0.f;
                    if (KG) {
                        if (new_ent[lane] != EMPTY) bonus = a.kg_weight / (float)new_hop[lane]; // query.cu:1759-1760
                    }
                    float ssum = 0.f, v = 0.f;
                    undecided = true;
                    if (a.paths & (PATH_SPARSE | PATH_BM25)) {
                        const float4 p4 = reinterpret_cast<const float4*>(part)[lane];
                        ssum = p4.x + p4.y + p4.z + p4.w; // the order wave_sum_dpp adds its four rows in
                        v = ssum;
                        if (!(a.paths & PATH_DENSE)) {
                            v = 1.0f - ssum - bonus;
                            undecided = false;
                        } else {
                            const float dub = pv_norm * my_dn; // |<query_d, doc_d>| <= |query_d| * |doc_d|
                            const float lb = 1.0f - (ssum + dub) - bonus;
                            if (lb > thr_eff + 1e-5f * (fabsf(ssum) + dub + fabsf(bonus) + 1.0f)) {
                                v = INF_DIS;
                                undecided = false;
                            }
                        }
                    }
                    new_dist[lane] = v;
                    ln_s += (a.paths & PATH_SPARSE) ? desc_nnz_s(my_desc) : 0u;
                    ln_b += (a.paths & PATH_BM25) ? desc_nnz_b(my_desc) : 0u;
                }
                st_eval += __popcll(__ballot(mine));
                need = __ballot(undecided);
            }
            wave_fence();
            // stage 2: the dense rows of the survivors, DENSE_BATCH rows in flight (two of the half-precision rows)
            while (HALF && need) {
                DenseRowHalf row[2];
                uint32_t jj[2];
#pragma unroll
                for (int b = 0; b < 2; b++) {
                    jj[b] = EMPTY;
                    if (need) {
                        jj[b] = __builtin_ctzll(need);
                        need &= need - 1;
                        dense_issue_half(row[b], a.half + (size_t)uniform(new_id[jj[b]]) * DIM);
                    }
                }
#pragma unroll
                for (int b = 0; b < 2; b++) {
                    if (jj[b] != EMPTY) {
                        const float dsum = dense_finish_lds_half(row[b], qd, 1.0f);
                        st_dense++;
                        if (lane == 0) new_dist[jj[b]] = 1.0f - (dsum + new_dist[jj[b]]) - 0.f;
                    }
                }
            }
            while (!HALF && need) {
                DenseRow row[DENSE_BATCH];
                uint32_t jj[DENSE_BATCH];
#pragma unroll
                for (int b = 0; b < DENSE_BATCH; b++) {
                    jj[b] = EMPTY;
                    if (need) {
                        jj[b] = __builtin_ctzll(need);
                        need &= need - 1;
                        dense_issue(row[b], a.C.recs + desc_off(readlane64(my_desc, jj[b])) * 16);
                    }
                }
#pragma unroll
                for (int b = 0; b < DENSE_BATCH; b++) {
                    if (jj[b] != EMPTY) {
                        float bonus = 0.f;
                        if (KG) {
                            if (new_ent[jj[b]] != EMPTY) bonus = a.kg_weight / (float)new_hop[jj[b]];
                        }
                        const float dsum = dense_finish_lds(row[b], qd, 1.0f);
                        st_dense++;
                        if (lane == 0) new_dist[jj[b]] = 1.0f - (dsum + new_dist[jj[b]]) - bonus;
                    }
                }
            }
            __syncthreads();
            // ---- wave 0: merge, pick the next parent, fetch its neighbours ----
            if (wave == 0) {
                hint = min(hint, sort_merge<MODE>(P, new_id, new_dist, new_ent, new_hop, n_new, R));
                uint32_t parent = EMPTY, slot = 0, n_next = 0;
                if (it < a.max_iter) {
                    for (uint32_t base = hint & ~(uint32_t)(WAVE - 1); base < cands; base += WAVE) {
                        const uint32_t id = base + lane < cands ? P.id[base + lane] : EMPTY;
                        const uint64_t b = __ballot((id & FLAG) == 0);
                        if (b) {
                            const int l = __ffsll((unsigned long long)b) - 1;
                            slot = base + l;
                            parent = __shfl(id, l, WAVE);
                            break;
                        }
                    }
                    hint = parent != EMPTY ? slot + 1 : cands;
                }
                if (parent != EMPTY) {
                    uint32_t p_ent = EMPTY, p_hop = 0;
                    if (KG) { p_ent = P.ent[slot]; p_hop = P.hop[slot]; }
                    if (lane == 0) P.id[slot] = parent | FLAG;
                    if (KWD) parent &= ID_MASK;
                    st_exp++;
                    uint32_t c = lane < (int)a.degree ? a.graph[(size_t)parent * a.W + lane] : EMPTY;
                    bool fresh = false;
                    if (c < a.C.n) {
                        const uint32_t bit = 1u << (c & 31);
                        fresh = !(atomicOr(&bitmap[c >> 5], bit) & bit);
                    }
                    bool alive = fresh;
                    uint32_t ent = EMPTY;
                    if (KWD) {
                        // slots whose graph neighbour was already visited (or invalid) are recycled with
                        // the parent's keyword edges: the t-th such slot takes keyword edge t
                        // (query.cu:1397-1409; which slot gets which edge does not matter)
                        const bool dup = lane < (int)a.degree && !fresh;
                        const uint32_t t = __popcll(__ballot(dup) & lane_lt);
                        const uint32_t n_kw = min(uniform(a.graph[(size_t)parent * a.W + a.degree]), (uint32_t)APOE_KW_SLOTS - 1u);
                        if (dup && t < n_kw) {
                            const uint32_t c2 = a.graph[(size_t)parent * a.W + a.degree + 1 + t];
                            if (c2 < a.C.n) {
                                const uint32_t bit = 1u << (c2 & 31);
                                if (!(atomicOr(&bitmap[c2 >> 5], bit) & bit)) { c = c2; alive = true; }
                            }
                        }
                    }
                    if (KG) {
                        // logical edges: parent's entity -> neighbour entity -> document
                        if (p_hop < 3 && p_ent < a.n_entities) {
                            uint32_t* slot_id = seed_id; // scratch, free after seeding
                            uint32_t* prop = seed_ent;
                            const uint32_t e0 = uniform(a.e2e_off[p_ent]), e1 = uniform(a.e2e_off[p_ent + 1]);
                            slot_id[lane] = fresh ? c : EMPTY;
                            link[lane] = EMPTY;
                            wave_fence();
                            // (i) a fresh graph neighbour that is also a logical neighbour is
                            //     tagged with the first linking entity (query.cu:1699-1715)
                            for (uint32_t jb = e0; jb < e1; jb += WAVE) {
                                const uint32_t j = jb + lane;
                                if (j < e1) {
                                    const uint32_t e2 = a.e2e_idx[j];
                                    if (e2 < a.n_entities) {
                                        for (uint32_t k = a.e2d_off[e2]; k < a.e2d_off[e2 + 1]; k++) {
                                            const uint32_t doc = a.e2d_idx[k];
                                            for (uint32_t t = 0; t < a.degree; t++)
                                                if (slot_id[t] == doc) atomicMin(&link[t], j - e0);
                                        }
                                    }
                                }
                            }
                            wave_fence();
                            if (fresh && link[lane] != EMPTY) ent = a.e2e_idx[e0 + link[lane]];
                            // (ii) slots whose graph neighbour was already visited (or invalid) are
                            //      recycled: the t-th such slot takes the first unvisited document
                            //      of the t-th neighbour entity (query.cu:1718-1735). A document
                            //      claimed by several slots in one round goes to the lowest slot;
                            //      the others move on to their next document.
                            const bool recyc = lane < (int)a.degree && !fresh;
                            const uint64_t rb = __ballot(recyc);
                            const uint32_t t = __popcll(rb & lane_lt);
                            bool unresolved = recyc && t < e1 - e0;
                            uint32_t e2 = EMPTY, k = 0, k1 = 0;
                            if (unresolved) {
                                e2 = a.e2e_idx[e0 + t];
                                if (e2 < a.n_entities) { k = a.e2d_off[e2]; k1 = a.e2d_off[e2 + 1]; }
                                else unresolved = false;
                            }
                            while (__any(unresolved)) {
                                uint32_t doc = EMPTY;
                                if (unresolved) {
                                    while (k < k1) {
                                        const uint32_t x = a.e2d_idx[k];
                                        if (x != parent && x < a.C.n) {
                                            const uint32_t word = __hip_atomic_load(&bitmap[x >> 5], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            if (!(word & (1u << (x & 31)))) { doc = x; break; }
                                        }
                                        k++;
                                    }
                                    if (doc == EMPTY) unresolved = false;
                                }
                                prop[lane] = doc;
                                wave_fence();
                                if (unresolved) {
                                    bool lose = false;
                                    for (int l = 0; l < lane; l++) lose |= prop[l] == doc;
                                    if (lose) k++;
                                    else {
                                        atomicOr(&bitmap[doc >> 5], 1u << (doc & 31));
                                        c = doc;
                                        ent = e2;
                                        alive = true;
                                        unresolved = false;
                                    }
                                }
                                wave_fence();
                                __threadfence();
                            }
                        }
                    }
                    const uint64_t b = __ballot(alive);
                    if (alive) {
                        const uint32_t pos = __popcll(b & lane_lt);
                        new_id[pos] = c;
                        if (KG) { new_ent[pos] = ent; new_hop[pos] = p_hop + 1; }
                    }
                    n_next = __popcll(b);
                }
                if (lane == 0) { ctl[CTL_PARENT] = parent; ctl[CTL_NNEW] = n_next; }
            }
            __syncthreads();
        }
        // ---- half-precision walk: every pool entry again with its fp32 row, then the pool in order again ----
        if (HALF) {
            __syncthreads();
            const uint32_t n_ovf = uniform(ctl[CTL_NOVF]);
            for (uint32_t e = wave; e < cands; e += NW) {
                const uint32_t id = uniform(P.id[e]) & ~FLAG;
                if (id >= a.C.n) continue; // empty slot
                RowLoad rl;
                RowInfo ri;
                row_issue<NARROW>(rl, ri, a.C, a.C.desc[id], true, a.paths);
                bool hit = false;
                const float acc = row_probe<NARROW, false>(a.C, rl, ri, T, n_ovf, nullptr, 0, hit);
                const float ssum = (a.paths & (PATH_SPARSE | PATH_BM25)) ? wave_sum_dpp(acc) : 0.f;
                // the same expressions as in the walk, so an entry gets the bits the default search gives it
                float dist = 1.0f - ssum - 0.f;
                if (a.paths & PATH_DENSE) {
                    DenseRow row;
                    dense_issue(row, ri.rec);
                    dist = 1.0f - (dense_finish_lds(row, qd, 1.0f) + ssum) - 0.f;
                }
                if (lane == 0) P.dist[e] = dist;
                st_again++;
                st_again_pairs += ri.n;
            }
            __syncthreads();
            if (wave == 0) {
                // nearly sorted already: odd-even transposition until a double pass moves nothing (stable)
                bool moved = true;
                while (moved) {
                    moved = false;
                    for (uint32_t phase = 0; phase < 2; phase++) {
                        bool sw = false;
                        for (uint32_t i = phase + 2 * lane; i + 1 < cands; i += 2 * WAVE) {
                            const float d0 = P.dist[i], d1 = P.dist[i + 1];
                            if (d1 < d0) {
                                const uint32_t i0 = P.id[i], i1 = P.id[i + 1];
                                P.dist[i] = d1;
                                P.dist[i + 1] = d0;
                                P.id[i] = i1;
                                P.id[i + 1] = i0;
                                sw = true;
                            }
                        }
                        wave_fence();
                        moved |= __any(sw) != 0;
                    }
                }
            }
            __syncthreads();
        }
        // ---- results (query.cu:566-569) ----
        if (!KWD) {
            for (uint32_t i = tid; i < cands; i += NW * WAVE) {
                a.cold->out_ids[(size_t)qi * cands + i] = P.id[i] & ~FLAG;
                a.cold->out_dist[(size_t)qi * cands + i] = P.dist[i];
            }
        } else if (wave == 0) {
            // pool entries that hold a required keyword, in pool order, then the evicted hits by
            // (distance, id); the rest of the row is empty (query.cu:1464-1481)
            uint32_t* oid = a.cold->out_ids + (size_t)qi * cands;
            float* od = a.cold->out_dist + (size_t)qi * cands;
            uint32_t kn = 0;
            for (uint32_t base = 0; base < cands; base += WAVE) {
                const uint32_t id = base + lane < cands ? P.id[base + lane] : EMPTY;
                const bool hit = id != EMPTY && (id & KW_HIT);
                const uint64_t hb = __ballot(hit);
                if (hit) {
                    const uint32_t pos = kn + __popcll(hb & lane_lt);
                    oid[pos] = id & ID_MASK;
                    od[pos] = P.dist[base + lane];
                }
                kn += __popcll(hb);
            }
            const uint32_t m = min(R.n, (uint32_t)RING);
            if ((uint32_t)lane < m) {
                const float d = R.dist[lane];
                const uint32_t id = R.id[lane];
                uint32_t rank = 0;
                for (uint32_t i = 0; i < m; i++) {
                    const float di = R.dist[i];
                    const uint32_t ii = R.id[i];
                    rank += (di < d) || (di == d && ii < id);
                }
                if (kn + rank < cands) { oid[kn + rank] = id; od[kn + rank] = d; }
            }
            for (uint32_t i = kn + m + lane; i < cands; i += WAVE) { oid[i] = EMPTY & ~FLAG; od[i] = INF_DIS; }
        }
        uint32_t st_ns = ln_s, st_nb = ln_b;
#pragma unroll
        for (int o = WAVE / 2; o > 0; o >>= 1) {
            st_ns += __shfl_xor(st_ns, o, WAVE);
            st_nb += __shfl_xor(st_nb, o, WAVE);
        }
        if (lane == 0) { // summed in LDS over the workgroup's queries: seven atomics per query on one memory line would queue up
            if (st_exp) atomicAdd(stat + 1, (unsigned long long)st_exp);
            if (st_eval) atomicAdd(stat + 2, (unsigned long long)st_eval);
            if (st_ns) atomicAdd(stat + 3, (unsigned long long)st_ns);
            if (st_nb) atomicAdd(stat + 4, (unsigned long long)st_nb);
            if (st_dense) atomicAdd(stat + 5, (unsigned long long)st_dense);
            if (st_again) atomicAdd(stat + 6, (unsigned long long)st_again);
            if (st_again_pairs) atomicAdd(stat + 7, (unsigned long long)st_again_pairs);
        }
    }
    __syncthreads();
    if (tid >= 1 && tid < 8 && stat[tid]) atomicAdd(a.work + tid, stat[tid]);
}

// Counters and once-per-query arguments of a launch, written on the stream (no host copy from a stack frame,
// no memset node for a caller that records the stream).
__global__ void search_setup_kernel(unsigned long long* work, SearchCold* dst, SearchCold cold) {
    if (threadIdx.x < 8) work[threadIdx.x] = 0ull;
    if (threadIdx.x == 0) *dst = cold;
}

// Workspace of apoe_search_noalloc: counters, once-per-query arguments and the visited bitmaps of as many
// workgroups as fit. One copy per GPU, held until the process ends; every call on a GPU uses it, so calls
// that overlap on one GPU race. Host code never uses the array's name as an address: the device address is
// asked for once per device (search_static_workspace) and kept.
static __device__ __align__(256) unsigned char search_scratch[APOE_NOALLOC_WS_BYTES];

constexpr int MAX_DEVICES = 64;
static std::mutex scratch_mutex;
static char* scratch_ptr[MAX_DEVICES]; // per device: address of search_scratch on that GPU, null until asked for

int search_static_workspace(int device, char** out) {
    APOE_REQUIRE(device >= 0 && device < MAX_DEVICES, "device %d outside [0,%d)", device, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[device]) {
        APOE_HIP(hipSetDevice(device));
        void* p = nullptr;
        APOE_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(search_scratch)));
        APOE_REQUIRE(p != nullptr, "no device address for the static search workspace on device %d", device);
        scratch_ptr[device] = static_cast<char*>(p);
    }
    *out = scratch_ptr[device];
    return APOE_OK;
}

template <int NW, int MODE, bool NARROW, bool HALF = false>
static int launch_format(apoe_ctx* ctx, const SearchArgs& a, uint32_t grid, size_t lds, int* per_cu) {
    if constexpr (MODE == MODE_PLAIN && !HALF) {
        if (a.half) return launch_format<NW, MODE, NARROW, true>(ctx, a, grid, lds, per_cu);
    }
    const void* fn = reinterpret_cast<const void*>(&search_kernel<NW, MODE, NARROW, HALF>);
    APOE_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    if (per_cu) { // occupancy query only
        APOE_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(per_cu, fn, NW * WAVE, lds));
        return APOE_OK;
    }
    search_kernel<NW, MODE, NARROW, HALF><<<grid, NW * WAVE, lds, ctx->stream>>>(a);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

template <int NW, int MODE>
static int launch_variant(apoe_ctx* ctx, const SearchArgs& a, uint32_t grid, size_t lds, int* per_cu) {
    return a.C.narrow ? launch_format<NW, MODE, true>(ctx, a, grid, lds, per_cu) : launch_format<NW, MODE, false>(ctx, a, grid, lds, per_cu);
}

template <int MODE>
static int launch_shape(apoe_ctx* ctx, int nw, const SearchArgs& a, uint32_t grid, size_t lds, int* per_cu) {
    switch (nw) {
        case 1: return launch_variant<1, MODE>(ctx, a, grid, lds, per_cu);
        case 4: return launch_variant<4, MODE>(ctx, a, grid, lds, per_cu);
        case 8: return launch_variant<8, MODE>(ctx, a, grid, lds, per_cu);
        case 16: return launch_variant<16, MODE>(ctx, a, grid, lds, per_cu);
        default: return launch_variant<2, MODE>(ctx, a, grid, lds, per_cu);
    }
}

static int launch_mode(apoe_ctx* ctx, int mode, int nw, const SearchArgs& a, uint32_t grid, size_t lds, int* per_cu) {
    switch (mode) {
        case MODE_KG: return launch_shape<MODE_KG>(ctx, nw, a, grid, lds, per_cu);
        case MODE_KEYWORD: return launch_shape<MODE_KEYWORD>(ctx, nw, a, grid, lds, per_cu);
        default: return launch_shape<MODE_PLAIN>(ctx, nw, a, grid, lds, per_cu);
    }
}

// static_ws: null, or the device address of this GPU's search_scratch: then nothing is allocated, the grid is cut to
// the bitmaps that fit, and a call without `stats` returns with the work still running on the context's stream.
int launch_search(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const apoe_graph* g, const apoe_kg* kg,
                  const apoe_search_params* p, uint32_t* out_ids_dev, float* out_dist_dev, apoe_search_stats* stats, char* static_ws) {
    APOE_REQUIRE(p->cands >= 1 && p->cands <= APOE_MAX_CANDS, "cands must be in 1..%d, got %u", APOE_MAX_CANDS, p->cands);
    APOE_REQUIRE(g->width > APOE_KW_SLOTS && g->width - APOE_KW_SLOTS <= MAX_NEW, "graph degree must be in 1..64, got width %u", g->width);
    APOE_REQUIRE(g->n == c->n, "graph has %u nodes but the corpus has %u documents", g->n, c->n);
    APOE_REQUIRE(p->q_begin <= q->n, "q_begin %u beyond %u queries", p->q_begin, q->n);
    const uint32_t q_count = p->q_count ? p->q_count : q->n - p->q_begin;
    APOE_REQUIRE(q_count <= q->n - p->q_begin, "query range of %u from %u beyond %u queries", q_count, p->q_begin, q->n);
    if (stats) *stats = apoe_search_stats{};
    if (q_count == 0) return APOE_OK;

    SearchArgs a{};
    SearchCold cold{};
    a.C = c->view();
    cold.Q = q->view();
    a.graph = g->rows.p;
    a.W = g->width;
    a.degree = g->width - APOE_KW_SLOTS;
    cold.entry = g->entry.p;
    cold.n_entry = std::min<uint32_t>(g->n_entry, MAX_NEW);
    cold.w_d = p->w_dense;
    cold.w_s = p->w_sparse;
    cold.w_b = p->w_bm25;
    a.paths = (!(p->w_dense < 1e-5f) ? PATH_DENSE : 0) | (!(p->w_sparse < 1e-5f) ? PATH_SPARSE : 0) | (!(p->w_bm25 < 1e-5f) ? PATH_BM25 : 0);
    a.cands = p->cands;
    a.max_iter = p->max_iter ? p->max_iter : 1000;
    cold.q_begin = p->q_begin;
    a.q_count = q_count;
    cold.out_ids = out_ids_dev;
    cold.out_dist = out_dist_dev;
    a.slots_s = next_pow2(std::max(16u, 2 * q->max_nnz_s));
    a.slots_b = next_pow2(std::max(16u, 2 * q->max_nnz_b));
    a.ovf_cap = (q->max_nnz + 7u) & ~7u;
    a.kg_weight = p->kg_weight;
    a.full_eval = (p->variant & 0x100u) ? 1u : 0u;
    a.half = nullptr;
    if (p->variant & 0x200u) {
        APOE_REQUIRE(c->half.p != nullptr, "variant 0x200 needs the half-precision rows: call apoe_corpus_make_half_rows first");
        APOE_REQUIRE(kg == nullptr && !p->keyword_filter, "variant 0x200 (half-precision rows) is for the plain search only");
        a.half = c->half.p;
    }

    const bool use_kg = kg != nullptr;
    const bool use_kw = p->keyword_filter != 0;
    APOE_REQUIRE(!(use_kg && use_kw), "keyword-filter search cannot be combined with a knowledge graph");
    const int mode = use_kg ? MODE_KG : use_kw ? MODE_KEYWORD : MODE_PLAIN;
    if (use_kw) {
        APOE_REQUIRE(c->n < (1u << 30), "keyword-filter search keeps two flag bits on a document id: %u documents are too many", c->n);
        a.paths = PATH_DENSE | PATH_SPARSE | PATH_BM25; // query.cu:2005-2007: always the three-path loop
        a.kw_slots = next_pow2(std::max(64u, 2 * q->max_keywords));
    }
    if (use_kg) {
        APOE_REQUIRE(kg->n_queries >= p->q_begin + q_count, "knowledge graph holds entities for %u queries, %u needed", kg->n_queries, p->q_begin + q_count);
        a.e2e_off = kg->e2e_off.p;
        a.e2e_idx = kg->e2e_idx.p;
        a.e2d_off = kg->e2d_off.p;
        a.e2d_idx = kg->e2d_idx.p;
        cold.q2e_off = kg->q2e_off.p;
        cold.q2e_idx = kg->q2e_idx.p;
        a.n_entities = kg->n_entities;
    }
    const SearchLds L(a.slots_s, a.slots_b, a.ovf_cap, a.cands, mode, a.kw_slots);
    APOE_REQUIRE(L.total <= 64 * 1024, "search needs %u bytes of LDS (query rows with up to %u sparse terms)", L.total, q->max_nnz);

    a.bitmap_words = ((c->n + 31) / 32 + 3) & ~3u;
    // workspace: [counters: 8 x u64][once-per-query arguments][visited bitmaps]
    const size_t cold_at = 8 * sizeof(unsigned long long), bitmaps_at = (cold_at + sizeof(SearchCold) + 255) & ~(size_t)255;
    const size_t bitmap_bytes = (size_t)a.bitmap_words * sizeof(uint32_t);
    size_t fit = SIZE_MAX; // workgroups whose visited bitmaps fit the workspace
    if (static_ws) {
        fit = (APOE_NOALLOC_WS_BYTES - bitmaps_at) / bitmap_bytes;
        APOE_REQUIRE(fit >= 1, "the static workspace of %u bytes holds no visited bitmap of %zu bytes", (unsigned)APOE_NOALLOC_WS_BYTES, bitmap_bytes);
    }

    // Launch shape (waves per query). 1, 2, 3, 4, 5: one, four, eight, two, sixteen waves, as the caller says. 0, the default:
    //  * a batch that is resident all at once is bound by the time of ONE query, and that falls with the waves it has
    //    (alone, cands 256: 4.2 / 2.9 / 2.0 / 1.7 ms with 2 / 4 / 8 / 16 waves): sixteen waves while every query has a
    //    CU of its own (256), eight while all queries still fit the machine that way (768 at 3 per CU), else four while
    //    they fit (1 536), e.g. 100 queries at cands 256 in 2.4 instead of 7.9 ms, 1 024 in 5.6 instead of 8.8 ms; four also for batches of up to two rounds of the two-wave
    //    grid (6 144 queries), whose second round ends sooner that way (4-9 % at 4 096 to 6 144 queries, cands 64-512);
    //  * a longer batch is bound by the memory system and runs best with two waves per query and as many queries as fit
    //    (12 per CU) - unless the pool is so large that LDS leaves room for at most 8 queries on a CU: then four waves
    //    per query keep twice the loads in flight (1 M docs: 167 against 191 ms at cands 1500, 234 against 290 ms at
    //    2048, the same at 1024, where 9 queries fit; knowledge-graph search: 66 against 77 ms at cands 512, 150
    //    against 195 ms at 1024; the keyword search measures the same or worse with four and stays at two).
    int nw = 2;
    const uint32_t shape = p->variant & 0xFFu;
    if (shape == 1) nw = 1;
    else if (shape == 2) nw = 4;
    else if (shape == 3) nw = 8;
    else if (shape == 5) nw = 16;
    else APOE_REQUIRE(shape == 0 || shape == 4, "launch shape %u is not one of 0 (default), 1, 2, 3, 4, 5 (one, four, eight, two, sixteen waves per query)", shape);
    auto resident_per_cu = [&](int waves, int* out) -> int {
        *out = 1;
        APOE_TRY(launch_mode(ctx, mode, waves, a, 0, L.total, out));
        if (*out < 1) *out = 1;
        return APOE_OK;
    };
    int per_cu = 1;
    if (shape == 0) {
        const size_t at_once = std::min<size_t>(q_count, fit); // queries in flight if every one of them had a workgroup
        int pc16 = 1, pc8 = 1, pc4 = 1;
        APOE_TRY(resident_per_cu(16, &pc16));
        APOE_TRY(resident_per_cu(8, &pc8));
        APOE_TRY(resident_per_cu(4, &pc4));
        APOE_TRY(resident_per_cu(2, &per_cu));
        if (at_once <= (size_t)pc16 * ctx->num_cus) { nw = 16; per_cu = pc16; }
        else if (at_once <= (size_t)pc8 * ctx->num_cus) { nw = 8; per_cu = pc8; }
        else if (at_once <= (size_t)pc4 * ctx->num_cus || at_once <= 2 * (size_t)per_cu * ctx->num_cus) { nw = 4; per_cu = pc4; }
        else if (per_cu <= 8 && mode != MODE_KEYWORD && pc4 * 4 > per_cu * 2) { nw = 4; per_cu = pc4; }
    } else {
        APOE_TRY(resident_per_cu(nw, &per_cu));
    }
    // persistent grid: as many workgroups as can be resident, never more than queries or bitmaps
    const uint32_t grid = (uint32_t)std::min<size_t>(std::min<size_t>(q_count, fit), (size_t)per_cu * (size_t)ctx->num_cus);
    char* ws = static_ws;
    if (!static_ws) APOE_TRY(ctx->search_workspace(bitmaps_at + (size_t)grid * bitmap_bytes, &ws));
    unsigned long long* work = reinterpret_cast<unsigned long long*>(ws);
    search_setup_kernel<<<1, WAVE, 0, ctx->stream>>>(work, reinterpret_cast<SearchCold*>(ws + cold_at), cold);
    APOE_HIP(hipGetLastError());
    a.cold = reinterpret_cast<const SearchCold*>(ws + cold_at);
    a.bitmaps = reinterpret_cast<uint32_t*>(ws + bitmaps_at);
    a.work = work;

    if (static_ws && !stats) return launch_mode(ctx, mode, nw, a, grid, L.total, nullptr);
    float ms = 0.f;
    APOE_TRY(timed(ctx, &ms, [&]() { return launch_mode(ctx, mode, nw, a, grid, L.total, nullptr); }));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    if (stats) {
        unsigned long long h[8];
        APOE_HIP(hipMemcpy(h, work, sizeof(h), hipMemcpyDeviceToHost));
        stats->kernel_ms = ms;
        stats->expansions = h[1];
        stats->evaluations = h[2];
        stats->nnz_sparse = h[3];
        stats->nnz_bm25 = h[4];
        stats->dense_rows = h[5];
        // dense rows actually needed + pairs + descriptor and dense norm (12 B per evaluation)
        uint64_t bytes = h[5] * (uint64_t)(a.half ? DENSE_BYTES / 2 : DENSE_BYTES);
        bytes += (c->narrow ? 6 : 8) * (h[3] + h[4]) + 12 * h[2];
        bytes += h[6] * (uint64_t)(DENSE_BYTES + 8) + (c->narrow ? 6 : 8) * h[7]; // the pool evaluated again in fp32
        bytes += h[1] * 4ull * a.W;
        uint64_t qbytes = (uint64_t)q_count * DENSE_BYTES + 8 * (q->h_s_off[p->q_begin + q_count] - q->h_s_off[p->q_begin]) +
                          8 * (q->h_b_off[p->q_begin + q_count] - q->h_b_off[p->q_begin]);
        bytes += qbytes + (uint64_t)q_count * a.cands * 8;
        stats->algo_bytes = bytes;
    }
    return APOE_OK;
}

} // namespace apoe
