// NN-Descent on the GPU: random initial lists, the per-node expansion step, and the
// final merge with the reverse lists. One workgroup (4 waves) per node.
#include <algorithm>
#include <memory>

#include "apoe_internal.h"

namespace apoe {

constexpr int NND_THREADS = 256;
constexpr int NND_PICKS = 4; // neighbours sampled per node and step (index.cu:157,171-181)
constexpr int NND_EVAL_BATCH = 4;  // candidates whose sparse parts a wave keeps in flight
constexpr int NND_DENSE_BATCH = 2; // dense rows a wave keeps in flight
constexpr uint32_t ALLP = PATH_DENSE | PATH_SPARSE | PATH_BM25;

__device__ __forceinline__ float key_dist(uint64_t key) {
    uint32_t u = (uint32_t)(key >> 32);
    u ^= (u >> 31) ? 0x80000000u : 0xFFFFFFFFu;
    return __uint_as_float(u);
}

__global__ __launch_bounds__(256) void nnd_init_kernel(uint32_t n, uint32_t K, uint64_t seed, uint32_t* ids, float* dist,
                                                       unsigned long long* rev, uint32_t* rev_cnt) {
    const uint64_t total = (uint64_t)n * K;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) {
        ids[t] = (uint32_t)(mix64(seed ^ mix64(t)) % n);
        dist[t] = INF_DIS;
        rev[t] = ~0ull; // (distance key, id) in one word: id part reads as EMPTY
        if (t < n) rev_cnt[t] = 0;
    }
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* p, uint64_t count, uint32_t v) {
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < count; t += (uint64_t)gridDim.x * blockDim.x) p[t] = v;
}

// Merge of a node's sorted list (o_id with flag bits, o_dist) with survivors given as
// distinct 64-bit (distance, id) keys. The best min(n_surv, K) survivors are sorted by
// counting ranks, then old and new elements take their merged ranks: an old element
// keeps rank pos + #{new <= it}, a new one takes pos + #{old < it} (new first on
// ties, index.cu:333-351). m_id/m_dist receive the K best. Returns via *n_ins the
// number of new elements kept. All threads of the block must call it.
__device__ void block_merge(const uint32_t* o_id, const float* o_dist, uint32_t K, const uint64_t* surv, uint32_t n_surv,
                            uint64_t* new_sorted, uint32_t* m_id, float* m_dist, uint32_t* n_ins, int tid, int nthreads) {
    if (tid == 0) *n_ins = 0;
    for (uint32_t i = tid; i < n_surv; i += nthreads) {
        const uint64_t k = surv[i];
        uint32_t r = 0;
        for (uint32_t j = 0; j < n_surv; j++) r += surv[j] < k;
        if (r < K) new_sorted[r] = k;
    }
    __syncthreads();
    const uint32_t n_new = min(n_surv, K);
    for (uint32_t t = tid; t < K + n_new; t += nthreads) {
        if (t < K) {
            const float v = o_dist[t];
            uint32_t lo = 0, len = n_new;
            while (len > 0) {
                uint32_t half = len >> 1;
                if (key_dist(new_sorted[lo + half]) <= v) { lo += half + 1; len -= half + 1; } else len = half;
            }
            const uint32_t rank = t + lo;
            if (rank < K) { m_id[rank] = o_id[t]; m_dist[rank] = v; }
        } else {
            const uint32_t i = t - K;
            const uint64_t k = new_sorted[i];
            const float v = key_dist(k);
            uint32_t lo = 0, len = K;
            while (len > 0) {
                uint32_t half = len >> 1;
                if (o_dist[lo + half] < v) { lo += half + 1; len -= half + 1; } else len = half;
            }
            const uint32_t rank = i + lo;
            if (rank < K) { m_id[rank] = (uint32_t)k; m_dist[rank] = v; atomicAdd(n_ins, 1u); }
        }
    }
    __syncthreads();
}

struct NndLds {
    uint32_t tab, seen, cand_id, cand_dist, surv, new_sorted, own_id, own_dist, m_id, m_dist, ctl, total;
    __host__ __device__ NndLds(uint32_t term_slots, uint32_t seen_slots, uint32_t K) {
        const uint32_t max_cand = NND_PICKS * 2 * K;
        uint32_t o = 0;
        tab = o; o += term_slots * 8;
        surv = o; o += max_cand * 8;
        new_sorted = o; o += K * 8;
        seen = o; o += seen_slots * 4;
        cand_id = o; o += max_cand * 4;
        cand_dist = o; o += max_cand * 4;
        own_id = o; o += K * 4;
        own_dist = o; o += K * 4;
        m_id = o; o += K * 4;
        m_dist = o; o += K * 4;
        ctl = o; o += 16 * 4;
        total = o;
    }
};

// One expansion step for node u = blockIdx.x (index.cu:156-376): sample up to four
// not-yet-sampled neighbours, gather their forward and reverse lists, drop self,
// duplicates and ids already in u's list, evaluate the rest against u, merge those
// closer than u's current worst into the list, and register u with every member of
// the merged list when the list changed.
// NARROW: the pair format of the corpus as a compile-time constant (no branch at the loads).
// HALF: the dense part of a candidate comes from the half-precision copy of the rows (`half`, [n][DIM]).
template <bool NARROW, bool HALF>
__global__ __launch_bounds__(NND_THREADS) void nnd_iterate_kernel(CorpusView C, float dense_mul, uint32_t K, uint32_t* ids, float* dist,
                                                                  unsigned long long* rev, uint32_t* rev_cnt, uint32_t term_slots,
                                                                  uint32_t seen_slots, unsigned long long* inserted, const uint16_t* half) {
    C.narrow = NARROW ? 1u : 0u;
    extern __shared__ __align__(16) char smem[];
    const NndLds L(term_slots, seen_slots, K);
    // the dedupe set is dead once the candidates are gathered: the pivot's dense row and the overflow
    // list of its term table take its place; the survivor array doubles as the list of candidates
    // that need their dense row
    float4* qd = reinterpret_cast<float4*>(smem + L.seen);
    unsigned long long* need = reinterpret_cast<unsigned long long*>(smem + L.surv);
    uint64_t* surv = reinterpret_cast<uint64_t*>(smem + L.surv);
    uint64_t* new_sorted = reinterpret_cast<uint64_t*>(smem + L.new_sorted);
    uint32_t* seen = reinterpret_cast<uint32_t*>(smem + L.seen);
    uint32_t* cand_id = reinterpret_cast<uint32_t*>(smem + L.cand_id);
    float* cand_dist = reinterpret_cast<float*>(smem + L.cand_dist);
    uint32_t* own_id = reinterpret_cast<uint32_t*>(smem + L.own_id);
    float* own_dist = reinterpret_cast<float*>(smem + L.own_dist);
    uint32_t* m_id = reinterpret_cast<uint32_t*>(smem + L.m_id);
    float* m_dist = reinterpret_cast<float*>(smem + L.m_dist);
    uint32_t* ctl = reinterpret_cast<uint32_t*>(smem + L.ctl); // [0..3] picks, [4] n_picks, [5] n_cand, [6] n_surv, [7] n_ins

    const int tid = threadIdx.x, wave = (int)uniform(tid / WAVE), lane = lane_id();
    const uint32_t u = blockIdx.x, smask = seen_slots - 1;
    Bucket4Tab T;
    T.b = reinterpret_cast<uint4*>(smem + L.tab);
    T.ovf = reinterpret_cast<uint2*>(smem + L.seen + DENSE_BYTES);
    T.n_ovf = &ctl[8];
    T.mask = term_slots / 4 - 1;
    T.ovf_cap = min(term_slots / 8, (seen_slots * 4 - DENSE_BYTES) / 8);
    const size_t base = (size_t)u * K;

    for (uint32_t i = tid; i < K; i += NND_THREADS) { own_id[i] = ids[base + i]; own_dist[i] = dist[base + i]; }
    bucket4_clear(T, tid, NND_THREADS);
    for (uint32_t i = tid; i < seen_slots; i += NND_THREADS) seen[i] = EMPTY;
    if (tid < 8) ctl[tid] = 0;
    if (tid == 9) ctl[9] = 0;
    __syncthreads();

    // 1. picks: group g takes the first unsampled slot >= g; none left -> slot 0
    if (wave == 0) {
        uint64_t m0 = __ballot(!(own_id[lane] & FLAG));
        uint64_t m1 = K > 64 ? __ballot(!(own_id[64 + lane] & FLAG)) : 0ull;
        if (lane == 0) {
            uint32_t np = 0;
            for (uint32_t g = 0; g < NND_PICKS; g++) {
                const uint64_t a = m0 & ~((1ull << g) - 1);
                uint32_t s;
                if (a) { s = __ffsll((unsigned long long)a) - 1; m0 &= ~(1ull << s); }
                else if (m1) { s = 64 + __ffsll((unsigned long long)m1) - 1; m1 &= ~(1ull << (s - 64)); }
                else s = EMPTY;
                if (s != EMPTY) { own_id[s] |= FLAG; ids[base + s] = own_id[s]; }
                else s = 0;
                bool dup = false;
                for (uint32_t t = 0; t < np; t++) dup |= ctl[t] == s;
                if (!dup) ctl[np++] = s;
            }
            ctl[4] = np;
        }
    }
    // own ids and u itself are never candidates
    for (uint32_t i = tid; i < K; i += NND_THREADS) id_set_insert(seen, smask, own_id[i] & ~FLAG);
    if (tid == NND_THREADS - 1) id_set_insert(seen, smask, u);
    __syncthreads();

    // 2./3. gather forward and reverse lists of the picked neighbours, deduplicated
    const uint32_t np = ctl[4];
    for (uint32_t t = tid; t < np * 2 * K; t += NND_THREADS) {
        const uint32_t p = t / (2 * K), r = t % (2 * K);
        const uint32_t v = own_id[ctl[p]] & ~FLAG;
        uint32_t c;
        if (r < K) c = ids[(size_t)v * K + r] & ~FLAG;
        else c = (uint32_t)rev[(size_t)v * K + (r - K)];
        if (c < C.n && id_set_insert(seen, smask, c)) cand_id[atomicAdd(&ctl[5], 1u)] = c;
    }
    __syncthreads();
    // pivot = u: dense row into LDS (float4 number l + 64*i belongs to lane l), terms into the bucket table
    const uint64_t du = C.desc[u];
    const char* rec = C.recs + desc_off(du) * 16;
    const Pairs u_pairs = record_pairs(C, du);
    {
        const float4* src = reinterpret_cast<const float4*>(rec);
        for (uint32_t i = tid; i < DIM / 4; i += NND_THREADS) qd[i] = src[i];
    }
    bucket4_terms_from_record(T, u_pairs, tid, NND_THREADS);
    __syncthreads();

    // 4. distances; only those below the current worst matter (step 5), so a candidate whose
    //    sparse part plus the bound of its dense part cannot get there is not read in full.
    //    Stage 1 settles the sparse parts (EVAL_BATCH candidates of a wave in flight), stage 2 reads
    //    the dense rows of the rest (DENSE_BATCH rows in flight), shared out again over the waves.
    constexpr int NW = NND_THREADS / WAVE;
    const uint32_t n_cand = ctl[5];
    const float worst = own_dist[K - 1];
    const float thr = worst < INF_DIS ? worst : __builtin_inff();
    const float pv_norm = pivot_dense_norm_lds(qd);
    const uint32_t n_ovf = uniform(ctl[8]);
    for (uint32_t c0 = 0; c0 * NW < n_cand; c0 += WAVE) {
        // lane l fetches descriptor and dense norm of the wave's (c0 + l)-th candidate
        uint64_t my_desc = 0;
        float my_dn = 0.f;
        {
            const uint32_t jl = wave + (c0 + lane) * NW;
            if (jl < n_cand) {
                const uint32_t cid = cand_id[jl];
                my_desc = C.desc[cid];
                my_dn = C.dnorm[cid];
            }
        }
        for (uint32_t t = 0; t < WAVE && wave + (c0 + t) * NW < n_cand; t += NND_EVAL_BATCH) {
            PendingEval pe[NND_EVAL_BATCH];
            float acc[NND_EVAL_BATCH];
#pragma unroll
            for (int b = 0; b < NND_EVAL_BATCH; b++) {
                const uint32_t jj = wave + (c0 + t + b) * NW;
                if (t + b < WAVE && jj < n_cand) eval_issue_desc(pe[b], C, readlane64(my_desc, t + b), readlane_f32(my_dn, t + b), pv_norm, ALLP, dense_mul);
            }
#pragma unroll
            for (int b = 0; b < NND_EVAL_BATCH; b++) {
                const uint32_t jj = wave + (c0 + t + b) * NW;
                acc[b] = 0.f;
                if (t + b < WAVE && jj < n_cand) acc[b] = doc_sparse_probe(C, pe[b], T, n_ovf, u_pairs);
            }
#pragma unroll
            for (int b = 0; b < NND_EVAL_BATCH; b++) {
                const uint32_t jj = wave + (c0 + t + b) * NW;
                if (t + b < WAVE && jj < n_cand) {
                    const SparseOut so = sparse_decide(pe[b], acc[b], ALLP, 0.f, thr);
                    if (lane == 0) {
                        cand_dist[jj] = so.v;
                        // what stage 2 needs to find the row: the record offset, or the document id for the half-precision copy
                        if (!so.decided)
                            need[atomicAdd(&ctl[9], 1u)] = ((unsigned long long)jj << 40) | (HALF ? (uint64_t)cand_id[jj] : desc_off(readlane64(my_desc, t + b)));
                    }
                }
            }
        }
    }
    __syncthreads();
    const uint32_t n_need = ctl[9];
    for (uint32_t t = wave; HALF && t < n_need; t += NW * NND_DENSE_BATCH * 2) {
        DenseRowHalf row[NND_DENSE_BATCH * 2];
        uint32_t jj[NND_DENSE_BATCH * 2];
#pragma unroll
        for (int b = 0; b < NND_DENSE_BATCH * 2; b++) {
            const uint32_t tt = t + b * NW;
            jj[b] = EMPTY;
            if (tt < n_need) {
                const unsigned long long e = need[tt];
                const uint32_t lo = uniform((uint32_t)e), hi = uniform((uint32_t)(e >> 32));
                jj[b] = hi >> 8;
                dense_issue_half(row[b], half + (size_t)lo * DIM);
            }
        }
#pragma unroll
        for (int b = 0; b < NND_DENSE_BATCH * 2; b++) {
            if (jj[b] != EMPTY) {
                const float dsum = dense_finish_lds_half(row[b], qd, dense_mul);
                if (lane == 0) cand_dist[jj[b]] = 1.0f - (dsum + cand_dist[jj[b]]) - 0.f;
            }
        }
    }
    for (uint32_t t = wave; !HALF && t < n_need; t += NW * NND_DENSE_BATCH) {
        DenseRow row[NND_DENSE_BATCH];
        uint32_t jj[NND_DENSE_BATCH];
#pragma unroll
        for (int b = 0; b < NND_DENSE_BATCH; b++) {
            const uint32_t tt = t + b * NW;
            jj[b] = EMPTY;
            if (tt < n_need) {
                const unsigned long long e = need[tt];
                const uint32_t lo = uniform((uint32_t)e), hi = uniform((uint32_t)(e >> 32));
                jj[b] = hi >> 8;
                dense_issue(row[b], C.recs + ((((uint64_t)(hi & 0xFFu)) << 32) | lo) * 16);
            }
        }
#pragma unroll
        for (int b = 0; b < NND_DENSE_BATCH; b++) {
            if (jj[b] != EMPTY) {
                const float dsum = dense_finish_lds(row[b], qd, dense_mul);
                if (lane == 0) cand_dist[jj[b]] = 1.0f - (dsum + cand_dist[jj[b]]) - 0.f;
            }
        }
    }
    const unsigned long long n_dense = wave == 0 ? n_need : 0;
    if (lane == 0 && n_dense) atomicAdd(inserted + 3, n_dense);
    if (tid == 0) atomicAdd(inserted + 2, (unsigned long long)n_cand);
    __syncthreads();

    // 5. survivors: closer than the current worst
    for (uint32_t j = tid; j < n_cand; j += NND_THREADS)
        if (cand_dist[j] < worst) surv[atomicAdd(&ctl[6], 1u)] = dist_id_key(cand_dist[j], cand_id[j]);
    __syncthreads();
    const uint32_t n_surv = ctl[6];
    if (n_surv == 0) return;
    block_merge(own_id, own_dist, K, surv, n_surv, new_sorted, m_id, m_dist, &ctl[7], tid, NND_THREADS);

    // 6. write back and register reverse edges (index.cu:358-372)
    for (uint32_t j = tid; j < K; j += NND_THREADS) {
        const uint32_t e = m_id[j];
        const float dv = m_dist[j];
        ids[base + j] = e;
        dist[base + j] = dv;
        const uint32_t v = e & ~FLAG;
        // (distance, u) travels as one 64-bit word, so a slot never holds the id of one writer with
        // the distance of another; beyond K registrations slot (count % K) keeps the closer one
        const uint32_t slot = atomicAdd(&rev_cnt[v], 1u);
        const unsigned long long key = dist_id_key(dv, u);
        unsigned long long* at = rev + (size_t)v * K + (slot % K);
        if (slot < K) *at = key;
        else atomicMin(at, key);
    }
    if (tid == 0) atomicAdd(inserted, (unsigned long long)ctl[7]);
}

// Merge with the reverse neighbours registered in the last step (index.cu:386-478).
__global__ __launch_bounds__(NND_THREADS) void nnd_merge_reverse_kernel(uint32_t n, uint32_t K, uint32_t* ids, float* dist,
                                                                        const unsigned long long* rev, const uint32_t* rev_cnt) {
    extern __shared__ __align__(16) char smem[];
    uint64_t* surv = reinterpret_cast<uint64_t*>(smem);
    uint64_t* new_sorted = surv + K;
    uint32_t* own_id = reinterpret_cast<uint32_t*>(new_sorted + K);
    float* own_dist = reinterpret_cast<float*>(own_id + K);
    uint32_t* m_id = reinterpret_cast<uint32_t*>(own_dist + K);
    float* m_dist = reinterpret_cast<float*>(m_id + K);
    uint32_t* r_id = reinterpret_cast<uint32_t*>(m_dist + K);
    float* r_dist = reinterpret_cast<float*>(r_id + K);
    uint32_t* ctl = reinterpret_cast<uint32_t*>(r_dist + K);
    const int tid = threadIdx.x;
    const uint32_t u = blockIdx.x;
    const size_t base = (size_t)u * K;
    const uint32_t cnt = min(K, rev_cnt[u]);
    for (uint32_t i = tid; i < K; i += NND_THREADS) {
        own_id[i] = ids[base + i];
        own_dist[i] = dist[base + i];
        const unsigned long long rk = i < cnt ? rev[base + i] : ~0ull;
        r_id[i] = (uint32_t)rk;
        r_dist[i] = r_id[i] != EMPTY ? key_dist(rk) : INF_DIS;
    }
    if (tid < 4) ctl[tid] = 0;
    __syncthreads();
    for (uint32_t j = tid; j < cnt; j += NND_THREADS) {
        const uint32_t r = r_id[j];
        const float rd = r_dist[j];
        bool keep = r < n && r != u;
        for (uint32_t t = 0; keep && t < K; t++) keep = (own_id[t] & ~FLAG) != r;
        // a repeated reverse id keeps its closest copy (first one on equal distance)
        for (uint32_t t = 0; keep && t < cnt; t++)
            if (t != j && r_id[t] == r && (r_dist[t] < rd || (r_dist[t] == rd && t < j))) keep = false;
        if (keep) surv[atomicAdd(&ctl[0], 1u)] = dist_id_key(rd, r);
    }
    __syncthreads();
    const uint32_t n_surv = ctl[0];
    if (n_surv == 0) return;
    block_merge(own_id, own_dist, K, surv, n_surv, new_sorted, m_id, m_dist, &ctl[1], tid, NND_THREADS);
    for (uint32_t j = tid; j < K; j += NND_THREADS) { ids[base + j] = m_id[j]; dist[base + j] = m_dist[j]; }
}

static uint32_t doc_term_slots(const apoe_corpus* c) { return next_pow2(std::max(64u, 2 * (c->max_nnz_s + c->max_nnz_b))); }

int launch_nnd_init(apoe_knn* g, uint64_t seed) {
    apoe_ctx* ctx = g->ctx;
    APOE_HIP(hipMemsetAsync(g->counter.p, 0, 4 * sizeof(unsigned long long), ctx->stream));
    const uint64_t total = (uint64_t)g->n * g->K;
    const uint32_t grid = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 20);
    nnd_init_kernel<<<grid, 256, 0, ctx->stream>>>(g->n, g->K, seed, g->ids.p, g->dist.p, g->rev.p, g->rev_cnt.p);
    APOE_HIP(hipGetLastError());
    return launch_norms(ctx, g->corpus, g->dense_scale, g->norms.p);
}

int launch_nnd_iterate(apoe_knn* g, uint64_t* inserted) {
    apoe_ctx* ctx = g->ctx;
    if (g->join) {
        APOE_REQUIRE(!g->half_rows, "the local-join step reads the fp32 rows: switch the half-precision rows off");
        APOE_TRY(launch_nnd_join_iterate(g));
        if (inserted) {
            unsigned long long h = 0;
            APOE_HIP(hipMemcpyAsync(&h, g->counter.p, sizeof(h), hipMemcpyDeviceToHost, ctx->stream));
            APOE_HIP(hipStreamSynchronize(ctx->stream));
            *inserted = h;
        }
        return APOE_OK;
    }
    const uint32_t term_slots = doc_term_slots(g->corpus);
    const uint32_t seen_slots = next_pow2(2 * (NND_PICKS * 2 * g->K + g->K + 1));
    const NndLds L(term_slots, seen_slots, g->K);
    APOE_REQUIRE(L.total <= 64 * 1024, "NN-Descent needs %u bytes of LDS (rows with up to %u sparse terms)", L.total,
                 g->corpus->max_nnz_s + g->corpus->max_nnz_b);
    APOE_HIP(hipMemsetAsync(g->counter.p, 0, sizeof(unsigned long long), ctx->stream)); // [0] inserted; [2], [3] accumulate over the build
    auto kernel = g->half_rows ? (g->corpus->narrow ? &nnd_iterate_kernel<true, true> : &nnd_iterate_kernel<false, true>)
                               : (g->corpus->narrow ? &nnd_iterate_kernel<true, false> : &nnd_iterate_kernel<false, false>);
    APOE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total));
    kernel<<<g->n, NND_THREADS, L.total, ctx->stream>>>(g->corpus->view(), g->dense_scale * g->dense_scale, g->K, g->ids.p, g->dist.p, g->rev.p,
                                                        g->rev_cnt.p, term_slots, seen_slots, g->counter.p, g->half_rows ? g->corpus->half.p : nullptr);
    APOE_HIP(hipGetLastError());
    if (inserted) {
        unsigned long long h = 0;
        APOE_HIP(hipMemcpyAsync(&h, g->counter.p, sizeof(h), hipMemcpyDeviceToHost, ctx->stream));
        APOE_HIP(hipStreamSynchronize(ctx->stream));
        *inserted = h;
    }
    return APOE_OK;
}

// Every stored distance again from the fp32 rows, then each list in (distance, id) order again: what follows a build
// whose steps took the dense parts from the half-precision rows. One workgroup per node: the node is the pivot (dense
// row in registers, terms in the LDS table), each wave takes every fourth list entry.
__global__ __launch_bounds__(NND_THREADS) void knn_refine_kernel(CorpusView C, float dense_mul, uint32_t K, uint32_t* ids, float* dist, uint32_t slots) {
    extern __shared__ __align__(16) char smem[];
    uint2* tab = reinterpret_cast<uint2*>(smem);
    uint32_t* l_id = reinterpret_cast<uint32_t*>(smem + (size_t)slots * 8);
    float* l_dist = reinterpret_cast<float*>(l_id + K);
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    const uint32_t u = blockIdx.x, mask = slots - 1;
    const size_t base = (size_t)u * K;
    term_table_clear(tab, slots, tid, NND_THREADS);
    for (uint32_t j = tid; j < K; j += NND_THREADS) {
        l_id[j] = ids[base + j];
        l_dist[j] = dist[base + j];
    }
    const uint64_t du = C.desc[u];
    const char* rec = C.recs + desc_off(du) * 16;
    PivotDense pv;
    pivot_dense_load(pv, reinterpret_cast<const float*>(rec), 1.0f);
    __syncthreads();
    pivot_terms_from_record(tab, mask, record_pairs(C, du), tid, NND_THREADS);
    __syncthreads();
    for (uint32_t j = wave; j < K; j += NND_THREADS / WAVE) {
        const uint32_t v = l_id[j] & ~FLAG;
        if (v >= C.n || !(l_dist[j] < INF_DIS)) continue; // an empty slot keeps what it holds
        const EvalOut e = eval_wave(C, v, pv, tab, mask, PATH_DENSE | PATH_SPARSE | PATH_BM25, dense_mul);
        if (lane == 0) l_dist[j] = 1.0f - e.ip;
    }
    __syncthreads();
    // counting rank by (distance, id): the flag bit of an id stays where it is
    for (uint32_t j = tid; j < K; j += NND_THREADS) {
        const float d = l_dist[j];
        const uint32_t id = l_id[j];
        uint32_t rank = 0;
        for (uint32_t i = 0; i < K; i++) {
            const float di = l_dist[i];
            const uint32_t ii = l_id[i];
            rank += (di < d) || (di == d && ((ii & ~FLAG) < (id & ~FLAG) || ((ii & ~FLAG) == (id & ~FLAG) && i < j)));
        }
        ids[base + rank] = id;
        dist[base + rank] = d;
    }
}

int launch_knn_refine(apoe_knn* g) {
    apoe_ctx* ctx = g->ctx;
    const uint32_t slots = doc_term_slots(g->corpus);
    const size_t lds = (size_t)slots * 8 + (size_t)g->K * 8;
    APOE_REQUIRE(lds <= 64 * 1024, "document rows with %u sparse terms exceed the LDS term table", g->corpus->max_nnz_s + g->corpus->max_nnz_b);
    knn_refine_kernel<<<g->n, NND_THREADS, lds, ctx->stream>>>(g->corpus->view(), g->dense_scale * g->dense_scale, g->K, g->ids.p, g->dist.p, slots);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

int launch_nnd_merge_reverse(apoe_knn* g) {
    apoe_ctx* ctx = g->ctx;
    const size_t lds = (size_t)g->K * (8 + 8 + 4 * 6) + 16;
    nnd_merge_reverse_kernel<<<g->n, NND_THREADS, lds, ctx->stream>>>(g->n, g->K, g->ids.p, g->dist.p, g->rev.p, g->rev_cnt.p);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

} // namespace apoe

using namespace apoe;

extern "C" {

int apoe_knn_create(apoe_ctx* ctx, const apoe_corpus* c, uint32_t K, float dense_scale, apoe_knn** out) {
    APOE_REQUIRE(ctx && c && out, "null argument");
    *out = nullptr;
    APOE_REQUIRE(K == 64 || K == 128, "K must be 64 or 128, got %u", K);
    APOE_REQUIRE(c->n > 1, "at least two documents are needed");
    APOE_HIP(hipSetDevice(ctx->device));
    std::unique_ptr<apoe_knn> g(new apoe_knn());
    g->ctx = ctx;
    g->corpus = c;
    g->n = c->n;
    g->K = K;
    g->dense_scale = dense_scale;
    const size_t total = (size_t)c->n * K;
    APOE_TRY(g->ids.alloc(total));
    APOE_TRY(g->dist.alloc(total));
    APOE_TRY(g->rev.alloc(total));
    APOE_TRY(g->rev_cnt.alloc(c->n));
    APOE_TRY(g->norms.alloc(c->n));
    APOE_TRY(g->counter.alloc(4));
    *out = g.release();
    return APOE_OK;
}

void apoe_knn_destroy(apoe_knn* g) { delete g; }

int apoe_knn_use_half_rows(apoe_knn* g, int on) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE(!on || g->corpus->half.p != nullptr, "the corpus has no half-precision rows: call apoe_corpus_make_half_rows first");
    g->half_rows = on != 0;
    return APOE_OK;
}

int apoe_knn_set_join(apoe_knn* g, int mode) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE(mode >= 0 && mode <= 2, "join mode must be 0 (expansion step), 1 (local join) or 2 (local join, both endpoints), got %d", mode);
    APOE_REQUIRE(mode == 0 || g->corpus->max_nnz_s + g->corpus->max_nnz_b <= APOE_JOIN_MAX_ROW_TERMS,
                 "the local-join step holds documents of up to %d sparse terms in its table, this corpus has rows of up to %u + %u: use the expansion step (mode 0)",
                 APOE_JOIN_MAX_ROW_TERMS, g->corpus->max_nnz_s, g->corpus->max_nnz_b);
    g->join = mode;
    g->join_symmetric = mode == 2;
    return APOE_OK;
}

int apoe_nnd_init(apoe_knn* g, uint64_t seed) {
    APOE_REQUIRE(g, "null argument");
    APOE_HIP(hipSetDevice(g->ctx->device));
    float ms = 0.f;
    APOE_TRY(timed(g->ctx, &ms, [&]() { return launch_nnd_init(g, seed); }));
    g->elapsed_ms = ms;
    g->ready = true;
    g->pruned = false;
    return APOE_OK;
}

int apoe_nnd_iterate(apoe_knn* g, int last, uint64_t* inserted) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE_STATE(g->ready, "the lists are empty: call apoe_nnd_init or apoe_knn_upload first");
    APOE_HIP(hipSetDevice(g->ctx->device));
    float ms = 0.f;
    APOE_TRY(timed(g->ctx, &ms, [&]() -> int {
        APOE_TRY(launch_nnd_iterate(g, nullptr));
        if (!last && !g->join) { // reset_reverse_num, index.cu:896; the join's reverse lists grow over the steps (join_apply_kernel)
            fill_u32_kernel<<<1024, 256, 0, g->ctx->stream>>>(g->rev_cnt.p, g->n, 0u);
            APOE_HIP(hipGetLastError());
        }
        return APOE_OK;
    }));
    g->elapsed_ms += ms;
    if (inserted) {
        unsigned long long h = 0;
        APOE_HIP(hipMemcpy(&h, g->counter.p, sizeof(h), hipMemcpyDeviceToHost));
        *inserted = h;
    }
    if (g->join) { // a picker row whose terms did not fit the tile's table was evaluated without its sparse part
        unsigned long long c3[3] = {0, 0, 0};
        APOE_TRY(join_step_counters(g, c3));
        if (c3[2]) g->ready = false;
        APOE_REQUIRE_STATE(c3[2] == 0, "the local-join step could not hold the sparse terms of %llu rows in its table (too many terms share table "
                           "slots): the lists of this handle are not valid, build again with the expansion step (apoe_knn_set_join(..., 0))", c3[2]);
    }
    return APOE_OK;
}

int apoe_nnd_merge_reverse(apoe_knn* g) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE_STATE(g->ready, "the lists are empty: call apoe_nnd_init or apoe_knn_upload first");
    APOE_HIP(hipSetDevice(g->ctx->device));
    float ms = 0.f;
    APOE_TRY(timed(g->ctx, &ms, [&]() -> int {
        APOE_TRY(launch_nnd_merge_reverse(g));
        fill_u32_kernel<<<1024, 256, 0, g->ctx->stream>>>(g->rev_cnt.p, g->n, 0u); // index.cu:899
        APOE_HIP(hipGetLastError());
        if (g->half_rows) APOE_TRY(launch_knn_refine(g)); // the lists leave the build with fp32 distances
        return APOE_OK;
    }));
    g->elapsed_ms += ms;
    return APOE_OK;
}

__global__ __launch_bounds__(256) static void strip_flags_kernel(const uint32_t* in, uint32_t* out, uint64_t count) {
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < count; t += (uint64_t)gridDim.x * blockDim.x) out[t] = in[t] & ~FLAG;
}

int apoe_knn_download(apoe_knn* g, uint32_t* ids, float* dist) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE_STATE(g->ready, "the lists are empty: call apoe_nnd_init or apoe_knn_upload first");
    APOE_HIP(hipSetDevice(g->ctx->device));
    const size_t total = (size_t)g->n * g->K;
    if (ids) {
        DevBuf<uint32_t> tmp;
        APOE_TRY(tmp.alloc(total));
        strip_flags_kernel<<<1024, 256, 0, g->ctx->stream>>>(g->ids.p, tmp.p, total);
        APOE_HIP(hipGetLastError());
        APOE_TRY(copy_out(g->ctx, ids, tmp.p, total * sizeof(uint32_t)));
    }
    if (dist) APOE_TRY(copy_out(g->ctx, dist, g->dist.p, total * sizeof(float)));
    return APOE_OK;
}

// How many uploaded neighbour ids do not name a document (flag bits count as such).
__global__ __launch_bounds__(256) static void knn_count_bad_kernel(uint32_t n, uint64_t total, const uint32_t* ids, unsigned long long* bad) {
    unsigned long long mine = 0;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) mine += ids[t] >= n;
    if (mine) atomicAdd(bad, mine);
}

__global__ __launch_bounds__(256) static void rev_reset_kernel(uint32_t n, uint32_t K, unsigned long long* rev, uint32_t* rev_cnt) {
    const uint64_t total = (uint64_t)n * K;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) {
        rev[t] = ~0ull;
        if (t < n) rev_cnt[t] = 0;
    }
}

// The steps index other nodes' lists and reverse lists with whatever a list holds, so an id that names no
// document is refused here; the reverse lists start empty, as after apoe_nnd_init. A refused upload leaves
// the handle as it was.
int apoe_knn_upload(apoe_knn* g, const uint32_t* ids, const float* dist) {
    APOE_REQUIRE(g && ids && dist, "null argument");
    APOE_HIP(hipSetDevice(g->ctx->device));
    hipStream_t st = g->ctx->stream;
    const size_t total = (size_t)g->n * g->K;
    DevBuf<uint32_t> tmp;
    APOE_TRY(tmp.alloc(total));
    APOE_TRY(copy_in(g->ctx, tmp.p, ids, total * sizeof(uint32_t)));
    APOE_HIP(hipMemsetAsync(g->counter.p + 1, 0, sizeof(unsigned long long), st));
    const uint32_t grid = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 16);
    knn_count_bad_kernel<<<grid, 256, 0, st>>>(g->n, total, tmp.p, g->counter.p + 1);
    APOE_HIP(hipGetLastError());
    unsigned long long bad = 0;
    APOE_TRY(copy_out(g->ctx, &bad, g->counter.p + 1, sizeof(bad)));
    APOE_REQUIRE(bad == 0, "%llu uploaded neighbour ids are not below the %u documents of the corpus", bad, g->n);
    APOE_HIP(hipMemcpyAsync(g->ids.p, tmp.p, total * sizeof(uint32_t), hipMemcpyDeviceToDevice, st));
    APOE_TRY(copy_in(g->ctx, g->dist.p, dist, total * sizeof(float)));
    rev_reset_kernel<<<grid, 256, 0, st>>>(g->n, g->K, g->rev.p, g->rev_cnt.p);
    APOE_HIP(hipGetLastError());
    APOE_TRY(launch_norms(g->ctx, g->corpus, g->dense_scale, g->norms.p));
    APOE_HIP(hipStreamSynchronize(st));
    g->ready = true;
    g->pruned = false;
    return APOE_OK;
}

// Reverse lists as (id, distance) arrays: a slot is one 64-bit word (distance key << 32 | id) on the device.
__global__ __launch_bounds__(256) static void rev_unpack_kernel(uint64_t total, const unsigned long long* rev, uint32_t* ids, float* dist) {
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) {
        const unsigned long long k = rev[t];
        const uint32_t id = (uint32_t)k;
        ids[t] = id;
        dist[t] = id != EMPTY ? key_dist(k) : INF_DIS;
    }
}

__global__ __launch_bounds__(256) static void rev_pack_kernel(uint32_t n, uint64_t total, const uint32_t* ids, const float* dist, unsigned long long* rev,
                                                              unsigned long long* bad) {
    unsigned long long mine = 0;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t id = ids[t];
        mine += id >= n && id != EMPTY;
        rev[t] = id < n ? dist_id_key(dist[t], id) : ~0ull;
    }
    if (mine) atomicAdd(bad, mine);
}

int apoe_knn_download_reverse(apoe_knn* g, uint32_t* rev_ids, float* rev_dist, uint32_t* rev_cnt) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE_STATE(g->ready, "the lists are empty: call apoe_nnd_init or apoe_knn_upload first");
    APOE_HIP(hipSetDevice(g->ctx->device));
    const size_t total = (size_t)g->n * g->K;
    if (rev_ids || rev_dist) {
        DevBuf<uint32_t> ti;
        DevBuf<float> td;
        APOE_TRY(ti.alloc(total));
        APOE_TRY(td.alloc(total));
        const uint32_t grid = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 16);
        rev_unpack_kernel<<<grid, 256, 0, g->ctx->stream>>>(total, g->rev.p, ti.p, td.p);
        APOE_HIP(hipGetLastError());
        if (rev_ids) APOE_TRY(copy_out(g->ctx, rev_ids, ti.p, total * sizeof(uint32_t)));
        if (rev_dist) APOE_TRY(copy_out(g->ctx, rev_dist, td.p, total * sizeof(float)));
    }
    if (rev_cnt) APOE_TRY(copy_out(g->ctx, rev_cnt, g->rev_cnt.p, (size_t)g->n * sizeof(uint32_t)));
    return APOE_OK;
}

int apoe_knn_upload_reverse(apoe_knn* g, const uint32_t* rev_ids, const float* rev_dist, const uint32_t* rev_cnt) {
    APOE_REQUIRE(g && rev_ids && rev_dist && rev_cnt, "null argument");
    APOE_REQUIRE_STATE(g->ready, "the lists are empty: call apoe_nnd_init or apoe_knn_upload first");
    APOE_HIP(hipSetDevice(g->ctx->device));
    hipStream_t st = g->ctx->stream;
    const size_t total = (size_t)g->n * g->K;
    DevBuf<uint32_t> ti;
    DevBuf<float> td;
    DevBuf<unsigned long long> packed;
    APOE_TRY(ti.alloc(total));
    APOE_TRY(td.alloc(total));
    APOE_TRY(packed.alloc(total));
    APOE_TRY(copy_in(g->ctx, ti.p, rev_ids, total * sizeof(uint32_t)));
    APOE_TRY(copy_in(g->ctx, td.p, rev_dist, total * sizeof(float)));
    APOE_HIP(hipMemsetAsync(g->counter.p + 1, 0, sizeof(unsigned long long), st));
    const uint32_t grid = (uint32_t)std::min<uint64_t>((total + 255) / 256, 1u << 16);
    rev_pack_kernel<<<grid, 256, 0, st>>>(g->n, total, ti.p, td.p, packed.p, g->counter.p + 1);
    APOE_HIP(hipGetLastError());
    unsigned long long bad = 0;
    APOE_TRY(copy_out(g->ctx, &bad, g->counter.p + 1, sizeof(bad)));
    APOE_REQUIRE(bad == 0, "%llu uploaded reverse ids are neither below the %u documents of the corpus nor the empty slot 0xFFFFFFFF", bad, g->n);
    APOE_HIP(hipMemcpyAsync(g->rev.p, packed.p, total * sizeof(unsigned long long), hipMemcpyDeviceToDevice, st));
    APOE_TRY(copy_in(g->ctx, g->rev_cnt.p, rev_cnt, (size_t)g->n * sizeof(uint32_t)));
    APOE_HIP(hipStreamSynchronize(st));
    return APOE_OK;
}

float apoe_knn_elapsed_ms(const apoe_knn* g) { return g ? g->elapsed_ms : 0.f; }

int apoe_knn_counters(apoe_knn* g, uint64_t* out2) {
    APOE_REQUIRE(g && out2, "null argument");
    APOE_HIP(hipSetDevice(g->ctx->device));
    unsigned long long h[4] = {0, 0, 0, 0};
    APOE_HIP(hipStreamSynchronize(g->ctx->stream));
    APOE_HIP(hipMemcpy(h, g->counter.p, sizeof(h), hipMemcpyDeviceToHost));
    out2[0] = h[2];
    out2[1] = h[3];
    return APOE_OK;
}

} // extern "C"
