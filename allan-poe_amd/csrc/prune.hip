// RNG-IP joint pruning with keyword-aware neighbour recycling, and the final row
// assembly with reverse edges. One workgroup (4 waves) per node for the prune, one
// wave per node for the assembly.
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <memory>

#include "apoe_gram.h"
#include <cmath>

#include "apoe_internal.h"
#include "apoe_ranktab.h"

namespace apoe {

constexpr int PR_THREADS = 256;
constexpr uint32_t ALL_PATHS = PATH_DENSE | PATH_SPARSE | PATH_BM25;

__device__ __forceinline__ void wave_fence_lds() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

struct PruneLds {
    uint32_t tab, idmap, uset, nb_id, nb_dist, det, cid, cdet, sel_id, sel_det, sel_live, sel_kw, o_fwd, o_det, o_kw, ctl, total;
    __host__ __device__ PruneLds(uint32_t term_slots, uint32_t uset_slots, uint32_t map_slots, uint32_t K) {
        uint32_t o = 0;
        tab = o; o += term_slots * 8;
        idmap = o; o += map_slots * 8;
        uset = o; o += uset_slots * 4;
        nb_id = o; o += K * 4;
        nb_dist = o; o += K * 4;
        det = o; o += K * 4;
        cid = o; o += K * 4;
        cdet = o; o += K * 4;
        sel_id = o; o += K * 4;
        sel_det = o; o += K * 4;
        sel_live = o; o += K * 4;
        sel_kw = o; o += K * 4;
        o_fwd = o; o += K * 4;
        o_det = o; o += K * 4;
        o_kw = o; o += (1 + APOE_KW_CAND) * 4;
        ctl = o; o += 16 * 4;
        total = o;
    }
};

enum { PC_M = 0, PC_NSEL = 1, PC_REJECT = 2, PC_ALLFLAG = 3, PC_CNT = 4, PC_FAIL = 5 };

// allan_poe (index.cu:539-714) for node u = blockIdx.x:
//  (a) detour counts over u's sorted list; (b) order by (detour, rank);
//  (c) sequential RNG-IP selection: candidate c is the pivot, each live selected s is
//      evaluated against it by one wave; norm[c] < <c,s> rejects c, norm[s] < <c,s>
//      tombstones s; (d) c carries the keyword flag when every live s it met has a
//      BM25 term that u holds and c lacks; (e) first `d` live selected go to the
//      forward row, flagged live ones beyond become keyword-edge candidates.
__global__ __launch_bounds__(PR_THREADS) void prune_kernel(CorpusView C, float dense_mul, const float* __restrict__ norms, uint32_t K,
                                                           const uint32_t* __restrict__ ids, const float* __restrict__ dist, uint32_t d,
                                                           uint32_t* fwd, uint32_t* det_out, uint32_t* cnt_out, uint32_t* kw_out,
                                                           uint32_t term_slots, uint32_t uset_slots, uint32_t map_slots) {
    extern __shared__ __align__(16) char smem[];
    const PruneLds L(term_slots, uset_slots, map_slots, K);
    uint2* tab = reinterpret_cast<uint2*>(smem + L.tab);
    uint2* idmap = reinterpret_cast<uint2*>(smem + L.idmap);
    uint32_t* uset = reinterpret_cast<uint32_t*>(smem + L.uset);
    uint32_t* nb_id = reinterpret_cast<uint32_t*>(smem + L.nb_id);
    float* nb_dist = reinterpret_cast<float*>(smem + L.nb_dist);
    uint32_t* det = reinterpret_cast<uint32_t*>(smem + L.det);
    uint32_t* cid = reinterpret_cast<uint32_t*>(smem + L.cid);
    uint32_t* cdet = reinterpret_cast<uint32_t*>(smem + L.cdet);
    uint32_t* sel_id = reinterpret_cast<uint32_t*>(smem + L.sel_id);
    uint32_t* sel_det = reinterpret_cast<uint32_t*>(smem + L.sel_det);
    volatile uint32_t* sel_live = reinterpret_cast<volatile uint32_t*>(smem + L.sel_live);
    uint32_t* sel_kw = reinterpret_cast<uint32_t*>(smem + L.sel_kw);
    uint32_t* o_fwd = reinterpret_cast<uint32_t*>(smem + L.o_fwd);
    uint32_t* o_det = reinterpret_cast<uint32_t*>(smem + L.o_det);
    uint32_t* o_kw = reinterpret_cast<uint32_t*>(smem + L.o_kw);
    volatile uint32_t* ctl = reinterpret_cast<volatile uint32_t*>(smem + L.ctl);

    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    const uint32_t u = blockIdx.x, tmask = term_slots - 1, umask = uset_slots - 1, mmask = map_slots - 1;
    const size_t base = (size_t)u * K;
    const uint64_t lane_lt = (1ull << lane) - 1;

    for (uint32_t i = tid; i < map_slots; i += PR_THREADS) idmap[i] = make_uint2(EMPTY, 0u);
    for (uint32_t i = tid; i < uset_slots; i += PR_THREADS) uset[i] = EMPTY;
    for (uint32_t i = tid; i < K; i += PR_THREADS) det[i] = 0;
    if (tid < 16) ctl[tid] = 0;
    __syncthreads();

    // valid list entries, in list order
    if (wave == 0) {
        uint32_t m = 0;
        for (uint32_t b0 = 0; b0 < K; b0 += WAVE) {
            const uint32_t v = ids[base + b0 + lane] & ~FLAG;
            const float dv = dist[base + b0 + lane];
            const bool ok = dv < INF_DIS && v < C.n && v != u;
            const uint64_t b = __ballot(ok);
            if (ok) {
                const uint32_t pos = m + __popcll(b & lane_lt);
                nb_id[pos] = v;
                nb_dist[pos] = dv;
            }
            m += __popcll(b);
        }
        if (lane == 0) ctl[PC_M] = m;
    }
    {   // u's BM25 terms
        const uint64_t du = C.desc[u];
        const Pairs sp = record_pairs(C, du);
        const uint32_t ns = desc_nnz_s(du), nb = desc_nnz_b(du);
        for (uint32_t j = tid; j < nb; j += PR_THREADS) {
            const uint32_t key = sp.key(ns + j);
            uint32_t h = term_hash(key, umask);
            while (true) {
                const uint32_t old = atomicCAS(&uset[h], EMPTY, key);
                if (old == EMPTY || old == key) break;
                h = (h + 1) & umask;
            }
        }
    }
    __syncthreads();
    const uint32_t m = ctl[PC_M];

    // (a) detour counts
    for (uint32_t i = tid; i < m; i += PR_THREADS) {
        const uint32_t key = nb_id[i];
        uint32_t h = term_hash(key, mmask);
        while (true) {
            const uint32_t old = atomicCAS(&idmap[h].x, EMPTY, key);
            if (old == EMPTY) { idmap[h].y = i; break; }
            if (old == key) break;
            h = (h + 1) & mmask;
        }
    }
    __syncthreads();
    for (uint32_t t = tid; t < m * K; t += PR_THREADS) {
        const uint32_t r = t / K, j = t % K;
        const size_t at = (size_t)nb_id[r] * K + j;
        const uint32_t x = ids[at] & ~FLAG;
        const float dx = dist[at];
        uint32_t h = term_hash(x, mmask);
        while (true) {
            const uint2 e = idmap[h];
            if (e.x == x) {
                if (e.y > r && dx < nb_dist[e.y]) atomicAdd(&det[e.y], 1u);
                break;
            }
            if (e.x == EMPTY) break;
            h = (h + 1) & mmask;
        }
    }
    __syncthreads();
    // (b) stable order by detour count
    for (uint32_t i = tid; i < m; i += PR_THREADS) {
        const uint32_t key = (det[i] << 16) | i;
        uint32_t r = 0;
        for (uint32_t j = 0; j < m; j++) r += ((det[j] << 16) | j) < key;
        cid[r] = nb_id[i];
        cdet[r] = det[i];
    }
    if (tid == 0 && m > 0) ctl[PC_ALLFLAG] = 1;
    __syncthreads();
    if (tid == 0 && m > 0) {
        sel_id[0] = cid[0];
        sel_det[0] = cdet[0];
        sel_live[0] = 1;
        sel_kw[0] = 0;
        ctl[PC_NSEL] = 1;
    }
    __syncthreads();

    // (c)+(d) sequential selection
    for (uint32_t t = 1; t < m; t++) {
        const uint32_t c = cid[t];
        term_table_clear(tab, term_slots, tid, PR_THREADS);
        __syncthreads();
        const uint64_t dc = C.desc[c];
        const char* rec = C.recs + desc_off(dc) * 16;
        PivotDense pv;
        pivot_dense_load(pv, reinterpret_cast<const float*>(rec), 1.0f);
        pivot_terms_from_record(tab, tmask, record_pairs(C, dc), tid, PR_THREADS);
        __syncthreads();
        const uint32_t n_sel = ctl[PC_NSEL];
        const float norm_c = norms[c];
        for (uint32_t i = wave; i < n_sel; i += PR_THREADS / WAVE) {
            if (!sel_live[i]) continue;
            const uint32_t s = uniform(sel_id[i]);
            bool kwf = false;
            EvalOut e = eval_wave<true>(C, s, pv, tab, tmask, ALL_PATHS, dense_mul, uset, umask, &kwf);
            if (lane == 0) {
                if (norm_c < e.ip) ctl[PC_REJECT] = 1;
                if (norms[s] < e.ip) sel_live[i] = 0;
                if (!kwf) ctl[PC_ALLFLAG] = 0;
            }
        }
        __syncthreads();
        if (tid == 0) {
            if (!ctl[PC_REJECT]) {
                sel_id[n_sel] = c;
                sel_det[n_sel] = cdet[t];
                sel_live[n_sel] = 1;
                sel_kw[n_sel] = ctl[PC_ALLFLAG];
                ctl[PC_NSEL] = n_sel + 1;
            }
            ctl[PC_REJECT] = 0;
            ctl[PC_ALLFLAG] = 1;
        }
        __syncthreads();
    }

    // (e) emit
    if (tid == 0) {
        const uint32_t n_sel = ctl[PC_NSEL];
        uint32_t cnt = 0, nkw = 0;
        for (uint32_t i = 0; i < n_sel; i++) {
            if (!sel_live[i]) continue;
            if (cnt < d) { o_fwd[cnt] = sel_id[i]; o_det[cnt] = sel_det[i]; cnt++; }
            else if (sel_kw[i] && nkw < APOE_KW_CAND) { o_kw[1 + nkw] = sel_id[i]; nkw++; }
        }
        for (uint32_t t = 0; t < m && cnt < d; t++) {
            const uint32_t c = cid[t];
            bool present = false;
            for (uint32_t j = 0; j < cnt; j++) present |= o_fwd[j] == c;
            if (!present) { o_fwd[cnt] = c; o_det[cnt] = cdet[t]; cnt++; }
        }
        ctl[PC_CNT] = cnt;
        for (; cnt < d; cnt++) { o_fwd[cnt] = u; o_det[cnt] = EMPTY; }
        o_kw[0] = nkw;
        for (uint32_t j = nkw; j < APOE_KW_CAND; j++) o_kw[1 + j] = 0;
    }
    __syncthreads();
    for (uint32_t i = tid; i < d; i += PR_THREADS) {
        fwd[(size_t)u * d + i] = o_fwd[i];
        det_out[(size_t)u * d + i] = o_det[i];
    }
    for (uint32_t i = tid; i < 1 + APOE_KW_CAND; i += PR_THREADS) kw_out[(size_t)u * (1 + APOE_KW_CAND) + i] = o_kw[i];
    if (tid == 0) cnt_out[u] = ctl[PC_CNT];
}

// ---- the prune on a Gram matrix that the tile kernel of join.hip has left in memory (lists of up to 128 entries) ----

constexpr uint32_t PS_MAX = 128;            // longest list
constexpr int PS_THREADS = 256;

struct SelectLds {
    uint32_t F, rdesc, idmap, umap, R, nb_id, nb_dist, nrm, det, order, o_fwd, o_det, o_kw, ctl, total;
    __host__ __device__ SelectLds(uint32_t umap_slots, uint32_t map_slots, uint32_t words) {
        uint32_t o = 0;
        F = o; o += PS_MAX * (PS_MAX / 32) * 4; // keyword-flag matrix: bit s of row c = "s holds a term of u that c lacks"
        o = (o + 7) & ~7u;
        rdesc = o; o += PS_MAX * 8;             // descriptors of the rows
        idmap = o; o += map_slots * 8;
        umap = o; o += umap_slots * 8;
        R = o; o += PS_MAX * words * 4;
        nb_id = o; o += PS_MAX * 4;
        nb_dist = o; o += PS_MAX * 4;
        nrm = o; o += PS_MAX * 4;
        det = o; o += PS_MAX * 4;
        order = o; o += PS_MAX * 4;
        o_fwd = o; o += PS_MAX * 4;
        o_det = o; o += PS_MAX * 4;
        o_kw = o; o += (1 + APOE_KW_CAND) * 4;
        ctl = o; o += 16 * 4;
        total = o;
    }
};

// allan_poe (index.cu:539-714) for node u = node0 + blockIdx.x, as prune_kernel, with every inner product <c, s> read from the
// node's Gram matrix gram[blockIdx.x][i][j] (i <= j: positions in the list of valid entries) instead of being evaluated:
// detour counts and the (detour, rank) order as there; the keyword flag of a pair from bit masks R[i] = the BM25 terms of u
// that row i holds (flag(c, s) = R[s] has a bit that R[c] lacks); the sequential selection by wave 0 alone, two selected
// members per lane (slots `lane` and `lane + 64` of the selection order), every member's product with the NEXT candidate
// requested from the matrix in memory while the current candidate is decided. The workgroup keeps no copy of the matrix:
// several nodes share a CU, and the others cover the selection's waits.
__global__ __launch_bounds__(PS_THREADS) void prune_select_kernel(CorpusView C, const float* __restrict__ norms, uint32_t K, const uint32_t* __restrict__ ids,
                                                                  const float* __restrict__ dist, uint32_t d, uint32_t node0, const float* __restrict__ gram,
                                                                  uint32_t* fwd, uint32_t* det_out, uint32_t* cnt_out, uint32_t* kw_out, uint32_t umap_slots,
                                                                  uint32_t map_slots, uint32_t words) {
    extern __shared__ __align__(16) char smem[];
    const SelectLds L(umap_slots, map_slots, words);
    uint32_t* F = reinterpret_cast<uint32_t*>(smem + L.F);
    uint64_t* rdesc = reinterpret_cast<uint64_t*>(smem + L.rdesc);
    uint2* idmap = reinterpret_cast<uint2*>(smem + L.idmap);
    uint2* umap = reinterpret_cast<uint2*>(smem + L.umap);
    uint32_t* R = reinterpret_cast<uint32_t*>(smem + L.R);
    uint32_t* nb_id = reinterpret_cast<uint32_t*>(smem + L.nb_id);
    float* nb_dist = reinterpret_cast<float*>(smem + L.nb_dist);
    float* nrm = reinterpret_cast<float*>(smem + L.nrm);
    uint32_t* det = reinterpret_cast<uint32_t*>(smem + L.det);
    uint32_t* order = reinterpret_cast<uint32_t*>(smem + L.order);
    uint32_t* o_fwd = reinterpret_cast<uint32_t*>(smem + L.o_fwd);
    uint32_t* o_det = reinterpret_cast<uint32_t*>(smem + L.o_det);
    uint32_t* o_kw = reinterpret_cast<uint32_t*>(smem + L.o_kw);
    volatile uint32_t* ctl = reinterpret_cast<volatile uint32_t*>(smem + L.ctl);

    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    constexpr uint32_t NWV = PS_THREADS / WAVE;
    const uint32_t u = node0 + blockIdx.x, umask = umap_slots - 1, mmask = map_slots - 1;
    const size_t base = (size_t)u * K;
    const uint64_t lane_lt = (1ull << lane) - 1;
    const float* gu = gram + (size_t)blockIdx.x * PS_MAX * PS_MAX;

    for (uint32_t i = tid; i < map_slots; i += PS_THREADS) idmap[i] = make_uint2(EMPTY, 0u);
    for (uint32_t i = tid; i < umap_slots; i += PS_THREADS) umap[i] = make_uint2(EMPTY, 0u);
    for (uint32_t i = tid; i < PS_MAX * words; i += PS_THREADS) R[i] = 0;
    for (uint32_t i = tid; i < PS_MAX; i += PS_THREADS) det[i] = 0;
    if (tid < 16) ctl[tid] = 0;
    __syncthreads();
    // valid list entries, in list order (the rows and columns of the Gram matrix)
    if (wave == 0) {
        uint32_t m = 0;
        for (uint32_t b0 = 0; b0 < K; b0 += WAVE) {
            const uint32_t v = ids[base + b0 + lane] & ~FLAG;
            const float dv = dist[base + b0 + lane];
            const bool ok = dv < INF_DIS && v < C.n && v != u;
            const uint64_t b = __ballot(ok);
            if (ok) {
                const uint32_t pos = m + __popcll(b & lane_lt);
                nb_id[pos] = v;
                nb_dist[pos] = dv;
                nrm[pos] = norms[v];
                rdesc[pos] = C.desc[v];
            }
            m += __popcll(b);
        }
        if (lane == 0) ctl[PC_M] = m;
    }
    {   // u's BM25 terms -> their index in u's row
        const uint64_t du = C.desc[u];
        const Pairs sp = record_pairs(C, du);
        const uint32_t ns = desc_nnz_s(du), nb = desc_nnz_b(du);
        for (uint32_t j = tid; j < nb; j += PS_THREADS) {
            const uint32_t key = sp.key(ns + j);
            uint32_t h = term_hash(key, umask);
            while (true) {
                const uint32_t old = atomicCAS(&umap[h].x, EMPTY, key);
                if (old == EMPTY) { umap[h].y = j; break; }
                if (old == key) break;
                h = (h + 1) & umask;
            }
        }
    }
    __syncthreads();
    const uint32_t m = ctl[PC_M];
    // (a) detour counts
    for (uint32_t i = tid; i < m; i += PS_THREADS) {
        const uint32_t key = nb_id[i];
        uint32_t h = term_hash(key, mmask);
        while (true) {
            const uint32_t old = atomicCAS(&idmap[h].x, EMPTY, key);
            if (old == EMPTY) { idmap[h].y = i; break; }
            if (old == key) break;
            h = (h + 1) & mmask;
        }
    }
    // R[r] = bits of u's BM25 terms that row r holds too: one wave per row, lanes over its BM25 pairs; the first 128 BM25 terms
    // of four rows are requested before the first of them is looked up
    auto mark = [&](uint32_t r, uint32_t key) {
        uint32_t h = term_hash(key, umask);
        while (true) {
            const uint2 e = umap[h];
            if (e.x == key) { atomicOr(&R[r * words + (e.y >> 5)], 1u << (e.y & 31)); break; }
            if (e.x == EMPTY) break;
            h = (h + 1) & umask;
        }
    };
    for (uint32_t r0 = wave; r0 < m; r0 += 4 * NWV) {
        uint32_t key[4][2], nbs[4];
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t r = r0 + b * NWV;
            nbs[b] = 0;
            key[b][0] = key[b][1] = EMPTY;
            if (r < m) {
                const uint64_t dr = rdesc[r];
                const Pairs sp = record_pairs(C, dr);
                const uint32_t ns = desc_nnz_s(dr);
                nbs[b] = desc_nnz_b(dr);
                if ((uint32_t)lane < nbs[b]) key[b][0] = sp.key(ns + lane);
                if ((uint32_t)lane + WAVE < nbs[b]) key[b][1] = sp.key(ns + lane + WAVE);
            }
        }
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const uint32_t r = r0 + b * NWV;
            if ((uint32_t)lane < nbs[b]) mark(r, key[b][0]);
            if ((uint32_t)lane + WAVE < nbs[b]) mark(r, key[b][1]);
            if (nbs[b] > 2 * WAVE) { // a longer row: the rest as it comes
                const uint64_t dr = rdesc[r];
                const Pairs sp = record_pairs(C, dr);
                const uint32_t ns = desc_nnz_s(dr);
                for (uint32_t j = 2 * WAVE + lane; j < nbs[b]; j += WAVE) mark(r, sp.key(ns + j));
            }
        }
    }
    __syncthreads();
    // sixteen list entries of this thread are requested before the first of them is looked up
    for (uint32_t t0 = 0; t0 < m * K; t0 += 16 * PS_THREADS) {
        uint32_t xs[16];
        float dxs[16];
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const uint32_t t = t0 + tid + k * PS_THREADS;
            xs[k] = EMPTY;
            dxs[k] = 0.f;
            if (t < m * K) {
                const size_t at = (size_t)nb_id[t / K] * K + t % K;
                xs[k] = ids[at] & ~FLAG;
                dxs[k] = dist[at];
            }
        }
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const uint32_t r = (t0 + tid + k * PS_THREADS) / K, x = xs[k];
            if (x == EMPTY) continue;
            uint32_t h = term_hash(x, mmask);
            while (true) {
                const uint2 e = idmap[h];
                if (e.x == x) {
                    if (e.y > r && dxs[k] < nb_dist[e.y]) atomicAdd(&det[e.y], 1u);
                    break;
                }
                if (e.x == EMPTY) break;
                h = (h + 1) & mmask;
            }
        }
    }
    __syncthreads();
    // (b) stable order by detour count
    for (uint32_t i = tid; i < m; i += PS_THREADS) {
        const uint32_t key = (det[i] << 16) | i;
        uint32_t r = 0;
        for (uint32_t j = 0; j < m; j++) r += ((det[j] << 16) | j) < key;
        order[r] = i;
    }
    // keyword flags of all pairs at once (index.cu:637,651-654): flag(c, s) = (R[s] & ~R[c]) != 0. A thread takes one row c and
    // half of the columns: its own mask stays in registers (the first four words), the lanes of a wave read the same R[s]
    {
        static_assert(PS_THREADS == 2 * PS_MAX && PS_MAX == 128, "one row and two flag words per thread");
        const uint32_t c = tid % PS_MAX, half = tid / PS_MAX;
        uint32_t rc[4];
#pragma unroll
        for (int w = 0; w < 4; w++) rc[w] = (uint32_t)w < words && c < m ? R[c * words + w] : 0u;
#pragma unroll
        for (int q2 = 0; q2 < 2; q2++) {
            const uint32_t q = half * 2 + q2;
            uint32_t word = 0;
            for (uint32_t b = 0; b < 32 && q * 32 + b < m; b++) {
                const uint32_t sidx = q * 32 + b;
                uint32_t any = 0;
#pragma unroll
                for (int w = 0; w < 4; w++)
                    if ((uint32_t)w < words) any |= R[sidx * words + w] & ~rc[w];
                for (uint32_t w = 4; w < words; w++) any |= R[sidx * words + w] & ~(c < m ? R[c * words + w] : 0u);
                word |= (any != 0 ? 1u : 0u) << b;
            }
            F[c * (PS_MAX / 32) + q] = c < m ? word : 0u;
        }
    }
    __syncthreads();
    // (c)+(d) sequential selection, wave 0: member k of the selection order lives in slot k / 64 of lane k % 64; what a step
    // needs of its candidate (Gram index, norm, flag row) is read one step ahead
    if (wave == 0) {
        uint32_t gi[2] = {0, 0}, kw[2] = {0, 0}; // Gram index (position in the list) and keyword flag of the member
        bool live[2] = {false, false};
        float mn[2] = {0.f, 0.f};
        uint32_t n_sel = 0;
        if (m > 0) {
            const uint32_t c0 = order[0];
            if (lane == 0) { gi[0] = c0; live[0] = true; mn[0] = nrm[c0]; }
            n_sel = 1;
        }
        uint32_t c_next = m > 1 ? order[1] : 0u;
        float norm_next = nrm[c_next];
        uint4 f_next = *reinterpret_cast<const uint4*>(&F[c_next * (PS_MAX / 32)]);
        auto product = [&](uint32_t a, uint32_t b) { return gu[(size_t)min(a, b) * PS_MAX + max(a, b)]; };
        float p_next[2] = {0.f, 0.f}; // <member, next candidate>
        if (m > 1 && lane == 0) p_next[0] = product(gi[0], c_next);
        for (uint32_t t = 1; t < m; t++) {
            const uint32_t c = c_next;
            const float norm_c = norm_next;
            const uint4 fc = f_next;
            const float p_cur[2] = {p_next[0], p_next[1]};
            if (t + 1 < m) {
                c_next = order[t + 1];
                norm_next = nrm[c_next];
                f_next = *reinterpret_cast<const uint4*>(&F[c_next * (PS_MAX / 32)]);
#pragma unroll
                for (int s = 0; s < 2; s++) { // also for the slot that c takes if it is accepted
                    const uint32_t slot = (uint32_t)lane + 64u * s;
                    if (slot < n_sel && live[s]) p_next[s] = product(gi[s], c_next);
                    else if (slot == n_sel) p_next[s] = product(c, c_next);
                }
            }
            bool rej = false, noflag = false;
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const bool act = (uint32_t)lane + 64u * s < n_sel && live[s];
                if (act) {
                    const float p = p_cur[s];
                    const uint32_t q = gi[s] >> 5, fw = q == 0 ? fc.x : q == 1 ? fc.y : q == 2 ? fc.z : fc.w;
                    rej |= norm_c < p;
                    if (mn[s] < p) live[s] = false;
                    noflag |= !((fw >> (gi[s] & 31)) & 1u);
                }
            }
            const bool reject = __ballot(rej) != 0;
            const bool allflag = __ballot(noflag) == 0;
            if (!reject) {
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    if ((uint32_t)lane + 64u * s == n_sel) { gi[s] = c; live[s] = true; mn[s] = norm_c; kw[s] = allflag ? 1u : 0u; }
                }
                n_sel++;
            }
        }
        // (e) emit: live members in selection order fill the row, flagged ones beyond d become keyword candidates
        uint32_t seen_live = 0, seen_kw = 0;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const bool lv = (uint32_t)lane + 64u * s < n_sel && live[s];
            const uint64_t lb = __ballot(lv);
            const uint32_t pos = seen_live + __popcll(lb & lane_lt);
            if (lv && pos < d) { o_fwd[pos] = nb_id[gi[s]]; o_det[pos] = det[gi[s]]; }
            const bool kwc = lv && pos >= d && kw[s];
            const uint64_t kb = __ballot(kwc);
            const uint32_t kpos = seen_kw + __popcll(kb & lane_lt);
            if (kwc && kpos < APOE_KW_CAND) o_kw[1 + kpos] = nb_id[gi[s]];
            seen_live += __popcll(lb);
            seen_kw += __popcll(kb);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (lane == 0) {
            uint32_t cnt = min(seen_live, d);
            const uint32_t nkw = min(seen_kw, (uint32_t)APOE_KW_CAND);
            // fewer survivors than the row has slots: the remaining neighbours in order, each id once, then the node itself
            for (uint32_t t = 0; t < m && cnt < d; t++) {
                const uint32_t cidx = order[t], cid = nb_id[cidx];
                bool present = false;
                for (uint32_t j = 0; j < cnt; j++) present |= o_fwd[j] == cid;
                if (!present) { o_fwd[cnt] = cid; o_det[cnt] = det[cidx]; cnt++; }
            }
            ctl[PC_CNT] = cnt;
            for (; cnt < d; cnt++) { o_fwd[cnt] = u; o_det[cnt] = EMPTY; }
            o_kw[0] = nkw;
            for (uint32_t j = nkw; j < APOE_KW_CAND; j++) o_kw[1 + j] = 0;
        }
    }
    __syncthreads();
    for (uint32_t i = tid; i < d; i += PS_THREADS) {
        fwd[(size_t)u * d + i] = o_fwd[i];
        det_out[(size_t)u * d + i] = o_det[i];
    }
    for (uint32_t i = tid; i < 1 + APOE_KW_CAND; i += PS_THREADS) kw_out[(size_t)u * (1 + APOE_KW_CAND) + i] = o_kw[i];
    if (tid == 0) cnt_out[u] = ctl[PC_CNT];
}

// ---- gather-once form of the prune (K = 64) ----

constexpr int PRUNE_DENSE_NB = 2; // 8-float blocks of the rows a wave requests ahead of the ones it multiplies
constexpr int GRAM_THREADS = 512; // 8 waves share one node's tables: more lookups in flight per byte of LDS

struct GramPruneLds {
    uint32_t G, tabs, ovf_cnt, rowptr, rownnz, umap, R, F, idmap, nb_id, nb_dist, nrm, det, order, o_fwd, o_det, o_kw, ctl, total;
    // union_slots != 0: the table region holds one union table (apoe_gram.h) instead of tgroup pivot tables;
    // rank_slots != 0: it holds a rank table (apoe_ranktab.h) of rank_bits index bits instead
    __host__ __device__ __forceinline__ GramPruneLds(uint32_t term_slots, uint32_t tgroup, uint32_t umap_slots, uint32_t map_slots, uint32_t words,
                                     uint32_t union_slots, uint32_t rank_bits = 0, uint32_t rank_slots = 0, bool narrow = true) {
        uint32_t o = 0;
        G = o; o += GRAM_ROWS * GRAM_STRIDE * 4;
        o = (o + 15) & ~15u;
        tabs = o; o += rank_slots ? RankTabLds(rank_bits, rank_slots, narrow).total
                           : union_slots ? GramUnionLds(union_slots).total : tgroup * (term_slots + GRAM_OVF) * 8;
        o = (o + 15) & ~15u;
        ovf_cnt = o; o += 24 * 4; // also the scratch of the rank table's running counts
        rowptr = o; o += GRAM_ROWS * 8;
        rownnz = o; o += GRAM_ROWS * 4;
        umap = o; o += umap_slots * 8;
        idmap = o; o += map_slots * 8;
        R = o; o += GRAM_ROWS * words * 4;
        F = o; o += GRAM_ROWS * 2 * 4; // keyword-flag matrix: bit s of row c = "s holds a term of u that c lacks"
        nb_id = o; o += GRAM_ROWS * 4;
        nb_dist = o; o += GRAM_ROWS * 4;
        nrm = o; o += GRAM_ROWS * 4;
        det = o; o += GRAM_ROWS * 4;
        order = o; o += GRAM_ROWS * 4;
        o_fwd = o; o += GRAM_ROWS * 4;
        o_det = o; o += GRAM_ROWS * 4;
        o_kw = o; o += (1 + APOE_KW_CAND) * 4;
        ctl = o; o += 16 * 4;
        total = o;
    }
};

// Sparse part of the Gram matrix with the rows in registers (K = 64, eight waves): wave w owns rows w, w + 8, ...
// (own[k] = row w + 8k, shape nnz | ns << 16, 0 where the row does not exist), loaded once. The pivots are taken
// eight at a time, one per wave (group g = rows 8g .. 8g + 7: every wave scatters ITS row own[g] into the rank
// table, apoe_ranktab.h), and every wave then probes the table with its own rows of index >= 8g, two per batch:
// no global memory access in the whole phase but for rows longer than the register window. G[p][b] += <p, b>
// for p < b. A group whose distinct terms exceed the table is done in passes of 4, 2 or 1 pivots.
constexpr int GR_OWN = GRAM_ROWS / 8;
template <bool NARROW>
__device__ __forceinline__ void gram_sparse_rank(const CorpusView& C, uint32_t m, float* G, const RankTab& T, uint32_t* scan,
                                                 const unsigned long long* rowptr, const uint32_t* rownnz, const RtRow<NARROW> (&own)[GR_OWN],
                                                 const uint32_t (&own_shape)[GR_OWN], uint32_t* fail, int tid, int nthreads) {
    const int wave = (int)uniform(tid / WAVE), lane = tid & (WAVE - 1);
    auto row_pairs = [&](uint32_t i) { Pairs p = gram_row(C, rowptr, rownnz, i); p.narrow = NARROW ? 1u : 0u; return p; };
    const uint32_t ng = m >= 2 ? (m - 2) / 8 + 1 : 0; // the last row is never a pivot
    uint32_t shape_lanes = 0; // lane k holds own_shape[k]: a wave-uniform pick by index without an indexed array
#pragma unroll
    for (int k = 0; k < GR_OWN; k++) shape_lanes = lane == k ? own_shape[k] : shape_lanes;
    for (uint32_t g = 0; g < ng; g++) {
        // this wave's pivot of the group: own[g], picked with wave-uniform selects so that own[] stays in registers
        RtRow<NARROW> pr = own[0];
#pragma unroll
        for (int k = 1; k < GR_OWN; k++) rt_row_select(pr, own[k], g == (uint32_t)k);
        const uint32_t pshape = (uint32_t)__builtin_amdgcn_readlane((int)shape_lanes, (int)g);
        const uint32_t prow = 8 * g + wave;
        const Pairs ptail = row_pairs(min(prow, m - 1));
        uint32_t lo = 0, cnt = 8;
        while (lo < 8) {
            const bool mine = (uint32_t)wave >= lo && (uint32_t)wave < lo + cnt && prow < m;
            const uint32_t built = ranktab_build_rows<NARROW>(T, pr, pshape, mine, wave - (int)lo, ptail, scan, tid, nthreads);
            if (built == EMPTY) {
                if (cnt == 1) { // one row alone does not fit: the caller falls back
                    if (tid == 0) *fail = 1;
                    lo += 1;
                } else {
                    cnt >>= 1;
                }
                continue;
            }
            const uint32_t n_ovf = NARROW ? 0u : uniform(min(scan[16], (uint32_t)RT_OVF));
#pragma unroll
            for (int k = 0; k < GR_OWN; k++) {
                if ((uint32_t)k >= g && own_shape[k] != 0) { // wave-uniform: rows of earlier groups have met these pivots as pivots themselves
                    float acc[1][RT_T];
                    RtRow<NARROW> rows[1];
                    uint32_t shape[1];
                    rows[0] = own[k];
                    rows[0].touch();
                    shape[0] = own_shape[k];
                    asm volatile("" : "+s"(shape[0]));
#pragma unroll
                    for (int t = 0; t < RT_T; t++) acc[0][t] = 0.f;
                    ranktab_probe_rows<NARROW, 1>(T, rows, shape, [&](int) { return row_pairs(wave + 8 * k); }, n_ovf, acc, lane);
                    uint32_t t;
                    const float z = wave_sum_1x8(acc[0], lane, &t);
                    const uint32_t b = wave + 8 * k, p = 8 * g + lo + t;
                    if ((lane & 15) < 4 && (lane & 32) == 0 && t < cnt && p < b) G[p * GRAM_STRIDE + b] += z;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            lo += cnt;
            __syncthreads(); // the table is rebuilt next
        }
    }
    for (uint32_t t = tid; t < m * m; t += nthreads) {
        const uint32_t i = t / m, j = t % m;
        if (i > j) G[i * GRAM_STRIDE + j] = G[j * GRAM_STRIDE + i];
    }
    __syncthreads();
}

// Same result as prune_kernel, different traffic: the node's <= 64 neighbour rows are read
// once, their hybrid Gram matrix is built in LDS (dense part on the matrix cores), every
// row's overlap with the centre node's BM25 terms becomes a bit mask, and the sequential
// RNG-IP selection with its keyword flags then runs on LDS only:
//   <c,s> = G[c][s];   flag(c,s) = (R[s] & ~R[c]) != 0   with R[x] = bm25(x) ∩ bm25(u).
template <int NT, bool NARROW>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void prune_gram_kernel(CorpusView C, float dense_mul, const float* __restrict__ norms,
                                                                const uint32_t* __restrict__ ids, const float* __restrict__ dist,
                                                                uint32_t d, uint32_t* fwd, uint32_t* det_out, uint32_t* cnt_out,
                                                                uint32_t* kw_out, uint32_t term_slots, uint32_t tgroup,
                                                                uint32_t umap_slots, uint32_t map_slots, uint32_t words,
                                                                uint32_t union_slots, uint32_t rank_bits, uint32_t rank_slots,
                                                                uint32_t rank_span, unsigned long long* gfail) {
    constexpr uint32_t K = GRAM_ROWS;
    C.narrow = NARROW ? 1u : 0u; // the pair format as a compile-time constant: no branch at the loads
    extern __shared__ __align__(16) char smem[];
    const GramPruneLds L(term_slots, tgroup, umap_slots, map_slots, words, union_slots, rank_bits, rank_slots, NARROW);
    float* G = reinterpret_cast<float*>(smem + L.G);
    uint2* tabs = reinterpret_cast<uint2*>(smem + L.tabs);
    uint32_t* ovf_cnt = reinterpret_cast<uint32_t*>(smem + L.ovf_cnt);
    unsigned long long* rowptr = reinterpret_cast<unsigned long long*>(smem + L.rowptr);
    uint32_t* rownnz = reinterpret_cast<uint32_t*>(smem + L.rownnz);
    uint2* umap = reinterpret_cast<uint2*>(smem + L.umap);
    uint2* idmap = reinterpret_cast<uint2*>(smem + L.idmap);
    uint32_t* R = reinterpret_cast<uint32_t*>(smem + L.R);
    uint32_t* F = reinterpret_cast<uint32_t*>(smem + L.F);
    uint32_t* nb_id = reinterpret_cast<uint32_t*>(smem + L.nb_id);
    float* nb_dist = reinterpret_cast<float*>(smem + L.nb_dist);
    float* nrm = reinterpret_cast<float*>(smem + L.nrm);
    uint32_t* det = reinterpret_cast<uint32_t*>(smem + L.det);
    uint32_t* order = reinterpret_cast<uint32_t*>(smem + L.order);
    uint32_t* o_fwd = reinterpret_cast<uint32_t*>(smem + L.o_fwd);
    uint32_t* o_det = reinterpret_cast<uint32_t*>(smem + L.o_det);
    uint32_t* o_kw = reinterpret_cast<uint32_t*>(smem + L.o_kw);
    volatile uint32_t* ctl = reinterpret_cast<volatile uint32_t*>(smem + L.ctl);

    const int tid = threadIdx.x, wave = (int)uniform(tid / WAVE), lane = lane_id();
    const uint32_t u = blockIdx.x, umask = umap_slots - 1, mmask = map_slots - 1;
    const size_t base = (size_t)u * K;
    const uint64_t lane_lt = (1ull << lane) - 1;

    for (uint32_t i = tid; i < map_slots; i += NT) idmap[i] = make_uint2(EMPTY, 0u);
    for (uint32_t i = tid; i < umap_slots; i += NT) umap[i] = make_uint2(EMPTY, 0u);
    for (uint32_t i = tid; i < K * words; i += NT) R[i] = 0;
    for (uint32_t i = tid; i < K; i += NT) det[i] = 0;
    for (uint32_t i = tid; i < K * 2; i += NT) F[i] = 0;
    if (tid < 16) ctl[tid] = 0;
    __syncthreads();

    if (wave == 0) {
        const uint32_t v = ids[base + lane] & ~FLAG;
        const float dv = dist[base + lane];
        const bool ok = dv < INF_DIS && v < C.n && v != u;
        const uint64_t b = __ballot(ok);
        if (ok) {
            const uint32_t pos = __popcll(b & lane_lt);
            nb_id[pos] = v;
            nb_dist[pos] = dv;
            nrm[pos] = norms[v];
        }
        if (lane == 0) ctl[PC_M] = __popcll(b);
    }
    if (!(NARROW && rank_slots != 0)) {   // u's BM25 terms -> index (the rank path of narrow corpora numbers them through the rank table)
        const uint64_t du = C.desc[u];
        const Pairs sp = record_pairs(C, du);
        const uint32_t ns = desc_nnz_s(du), nb = desc_nnz_b(du);
        for (uint32_t j = tid; j < nb; j += NT) {
            const uint32_t key = sp.key(ns + j);
            uint32_t h = term_hash(key, umask);
            while (true) {
                const uint32_t old = atomicCAS(&umap[h].x, EMPTY, key);
                if (old == EMPTY) { umap[h].y = j; break; }
                if (old == key) break;
                h = (h + 1) & umask;
            }
        }
    }
    __syncthreads();
    const uint32_t m = uniform(ctl[PC_M]);

    const bool rank = rank_slots != 0; // the sparse part runs on the rank table with the rows held in registers
    if (rank) gram_rows_gather(C, nb_id, m, rowptr, rownnz, tid, NT);
    // (a) detour counts (as prune_kernel)
    for (uint32_t i = tid; i < m; i += NT) {
        const uint32_t key = nb_id[i];
        uint32_t h = term_hash(key, mmask);
        while (true) {
            const uint32_t old = atomicCAS(&idmap[h].x, EMPTY, key);
            if (old == EMPTY) { idmap[h].y = i; break; }
            if (old == key) break;
            h = (h + 1) & mmask;
        }
    }
    // R[r] = bits of u's BM25 terms that row r holds too: one wave per row, lanes over its BM25 pairs
    auto mark = [&](uint32_t r, uint32_t key) {
        uint32_t h = term_hash(key, umask);
        while (true) {
            const uint2 e = umap[h];
            if (e.x == key) { atomicOr(&R[r * words + (e.y >> 5)], 1u << (e.y & 31)); break; }
            if (e.x == EMPTY) break;
            h = (h + 1) & umask;
        }
    };
    for (uint32_t r = wave; r < (rank ? 0u : m); r += NT / WAVE) {
        const uint64_t dr = C.desc[nb_id[r]];
        const Pairs sp = record_pairs(C, dr);
        const uint32_t ns = desc_nnz_s(dr), nb = desc_nnz_b(dr);
        for (uint32_t j = lane; j < nb; j += WAVE) {
            const uint32_t key = sp.key(ns + j);
            uint32_t h = term_hash(key, umask);
            while (true) {
                const uint2 e = umap[h];
                if (e.x == key) { atomicOr(&R[r * words + (e.y >> 5)], 1u << (e.y & 31)); break; }
                if (e.x == EMPTY) break;
                h = (h + 1) & umask;
            }
        }
    }
    __syncthreads();
    {   // all list entries of this thread are requested before the first one is looked up
        constexpr uint32_t PER = K * K / NT;
        uint32_t xs[PER];
        float dxs[PER];
#pragma unroll
        for (uint32_t k = 0; k < PER; k++) {
            const uint32_t t = tid + k * NT, r = t / K, j = t % K;
            xs[k] = EMPTY;
            dxs[k] = 0.f;
            if (t < m * K) {
                const size_t at = (size_t)nb_id[r] * K + j;
                xs[k] = ids[at] & ~FLAG;
                dxs[k] = dist[at];
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < PER; k++) {
            const uint32_t r = (tid + k * NT) / K, x = xs[k];
            if (x == EMPTY) continue;
            uint32_t h = term_hash(x, mmask);
            while (true) {
                const uint2 e = idmap[h];
                if (e.x == x) {
                    if (e.y > r && dxs[k] < nb_dist[e.y]) atomicAdd(&det[e.y], 1u);
                    break;
                }
                if (e.x == EMPTY) break;
                h = (h + 1) & mmask;
            }
        }
    }
    __syncthreads();
    // hybrid Gram matrix of the m rows. Only the upper triangle of G is used (the sparse part is added there and the
    // lower triangle is mirrored from it at the end). Every wave takes an eighth of the dimensions and computes the
    // three upper tiles for it from one read of the rows; the partial tiles are added into G in a fixed order
    // (barriers between them): the result does not depend on timing.
    constexpr int NWAVES = NT / WAVE, BLOCKS = DIM / 8;
    static_assert(NWAVES == 8, "dimensions and rows are dealt out to eight waves");
    floatx16 dacc00, dacc01, dacc11;
    gram_dense_upper<PRUNE_DENSE_NB>(C, nb_id, m, lane, wave * (BLOCKS / NWAVES), (wave + 1) * (BLOCKS / NWAVES), dacc00, dacc01, dacc11);
    // this wave's rows w, w + 8, ...: requested as soon as the wave's dense tile is done (its operands need the registers), used from the keyword masks on
    static_assert(NT / WAVE == 8 || NT / WAVE == 4, "rows are dealt out to eight waves");
    RtRow<NARROW> own[GR_OWN];
    uint32_t own_shape[GR_OWN];
#pragma unroll
    for (int k = 0; k < GR_OWN; k++) {
        const uint32_t b = wave + 8 * k;
        own_shape[k] = 0;
        if (rank && b < m) {
            own_shape[k] = uniform(rownnz[b]);
            Pairs sp = gram_row(C, rowptr, rownnz, b);
            sp.narrow = NARROW ? 1u : 0u;
            rt_row_load(own[k], sp, lane);
        }
    }
    // (b) stable order by detour count (LDS only: runs while the rows arrive)
    for (uint32_t i = tid; i < m; i += NT) {
        const uint32_t key = (det[i] << 16) | i;
        uint32_t r = 0;
        for (uint32_t j = 0; j < m; j++) r += ((det[j] << 16) | j) < key;
        order[r] = i;
    }
    for (int ph = 0; ph < NWAVES; ph++) {
        if (wave == ph && m > 0) {
            gram_dense_store(G, 0, lane, dacc00, dense_mul, ph != 0);
            if (m > 32) {
                gram_dense_store(G, 1, lane, dacc01, dense_mul, ph != 0);
                gram_dense_store(G, 3, lane, dacc11, dense_mul, ph != 0);
            }
        }
        if (ph + 1 < NWAVES) __syncthreads();
    }
    if (rank && NARROW) {
        // keyword masks through the rank table: u's BM25 terms alone go into the bitmap (no values), a term's slot -- its
        // rank among them -- is its bit in the masks, and every wave looks the BM25 pairs of its rows up with one 8-byte
        // read each: no hash collisions, no probe loop
        const RankTab T = ranktab_at(reinterpret_cast<char*>(tabs), rank_bits, rank_slots, rank_span, NARROW);
        const uint64_t du = C.desc[u];
        const Pairs up = record_pairs(C, du);
        const uint32_t ns_u = desc_nnz_s(du), nb_u = desc_nnz_b(du);
        ranktab_build_bits<NARROW>(T, [&](auto f) {
            for (uint32_t j = tid; j < nb_u; j += NT) f(up.raw(ns_u + j), true, 0);
        }, ~0u, ovf_cnt, tid, NT);
        __syncthreads();
        auto mark_bit = [&](uint32_t r, uint2 w, uint32_t idx) {
            const uint32_t e = ranktab_slot(w, idx);
            if (e != EMPTY) atomicOr(&R[r * words + (e >> 5)], 1u << (e & 31));
        };
#pragma unroll
        for (int k = 0; k < GR_OWN; k++) {
            const uint32_t nnz = own_shape[k] & 0xFFFFu, ns = own_shape[k] >> 16, r = wave + 8 * k;
            if (nnz > ns) { // wave-uniform: the row has BM25 pairs
                uint32_t idx[RT_CHUNKS];
                uint2 w[RT_CHUNKS];
#pragma unroll
                for (int c = 0; c < RT_CHUNKS; c++) {
                    const uint32_t j = rt_pair(c, lane);
                    idx[c] = ranktab_index<NARROW>(T, own[k].key(c), true);
                    w[c] = T.word[j >= ns && j < nnz ? idx[c] >> 5 : 0u];
                }
#pragma unroll
                for (int c = 0; c < RT_CHUNKS; c++) {
                    const uint32_t j = rt_pair(c, lane);
                    if (j >= ns && j < nnz) mark_bit(r, w[c], idx[c]);
                }
                if (nnz > RT_CHUNKS * WAVE) {
                    Pairs sp = gram_row(C, rowptr, rownnz, r);
                    sp.narrow = NARROW ? 1u : 0u;
                    for (uint32_t j = max(ns, (uint32_t)(RT_CHUNKS * WAVE)) + lane; j < nnz; j += WAVE) {
                        const uint32_t ix = ranktab_index<NARROW>(T, sp.raw(j).x, true);
                        mark_bit(r, T.word[ix >> 5], ix);
                    }
                }
            }
        }
    } else if (rank) {
#pragma unroll
        for (int k = 0; k < GR_OWN; k++) {
            const uint32_t nnz = own_shape[k] & 0xFFFFu, ns = own_shape[k] >> 16, r = wave + 8 * k;
            if (nnz > ns) { // wave-uniform: the row has BM25 pairs
                // the first table slot of all four pairs is read before any is compared; the probe loop is for the
                // pairs whose slot holds another term
                uint32_t key[RT_CHUNKS], h[RT_CHUNKS];
                uint2 e[RT_CHUNKS];
#pragma unroll
                for (int c = 0; c < RT_CHUNKS; c++) {
                    key[c] = own[k].key(c) | (NARROW ? 0x80000000u : 0u);
                    h[c] = term_hash(key[c], umask);
                    e[c] = umap[h[c]];
                }
#pragma unroll
                for (int c = 0; c < RT_CHUNKS; c++) {
                    const uint32_t j = rt_pair(c, lane);
                    if (j >= ns && j < nnz) {
                        if (e[c].x == key[c]) atomicOr(&R[r * words + (e[c].y >> 5)], 1u << (e[c].y & 31));
                        else if (e[c].x != EMPTY) mark(r, key[c]);
                    }
                }
                if (nnz > RT_CHUNKS * WAVE) {
                    Pairs sp = gram_row(C, rowptr, rownnz, r);
                    sp.narrow = NARROW ? 1u : 0u;
                    for (uint32_t j = max(ns, (uint32_t)(RT_CHUNKS * WAVE)) + lane; j < nnz; j += WAVE) mark(r, sp.key(j));
                }
            }
        }
    }
    __syncthreads();
    if (rank) {
        const RankTab T = ranktab_at(reinterpret_cast<char*>(tabs), rank_bits, rank_slots, rank_span, NARROW);
        gram_sparse_rank<NARROW>(C, m, G, T, ovf_cnt, rowptr, rownnz, own, own_shape, (uint32_t*)&ctl[PC_FAIL], tid, NT);
    } else if (union_slots) gram_sparse_union(C, nb_id, m, G, reinterpret_cast<char*>(tabs), union_slots, ovf_cnt, rowptr, rownnz, (uint32_t*)&ctl[PC_FAIL], tid, NT);
    else if (tgroup == 8) gram_sparse_64<8>(C, nb_id, m, G, tabs, term_slots, ovf_cnt, rowptr, rownnz, (uint32_t*)&ctl[PC_FAIL], tid, NT);
    else gram_sparse_64<4>(C, nb_id, m, G, tabs, term_slots, ovf_cnt, rowptr, rownnz, (uint32_t*)&ctl[PC_FAIL], tid, NT);
    // keyword flags of all pairs at once (index.cu:637,651-654): flag(c, s) = (R[s] & ~R[c]) != 0. A thread takes one row c and
    // one of its two flag words: its own mask stays in registers (the first four words), the lanes of a wave read the same R[s]
    if (tid < 2 * (int)K) {
        const uint32_t c = (uint32_t)tid % K, q = (uint32_t)tid / K;
        uint32_t rc[4], word = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) rc[w] = (uint32_t)w < words && c < m ? R[c * words + w] : 0u;
        for (uint32_t b = 0; b < 32 && q * 32 + b < m; b++) {
            const uint32_t sidx = q * 32 + b;
            uint32_t any = 0;
#pragma unroll
            for (int w = 0; w < 4; w++)
                if ((uint32_t)w < words) any |= R[sidx * words + w] & ~rc[w];
            for (uint32_t w = 4; w < words; w++) any |= R[sidx * words + w] & ~(c < m ? R[c * words + w] : 0u);
            word |= (any != 0 ? 1u : 0u) << b;
        }
        F[c * 2 + q] = c < m ? word : 0u;
    }
    __syncthreads();
    // (c)+(d) sequential selection on the Gram matrix: wave 0, lane i keeps selected member i in registers and the
    // candidate at position i of the order (its Gram row, norm and flag word are handed out with readlane); the Gram
    // entries of step t + 1 are requested before step t is decided (the lane that would hold candidate t as a new
    // member asks for its entry too), so a step waits for no memory
    if (wave == 0 && m > 0) {
        const uint32_t ord = (uint32_t)lane < m ? order[lane] : order[0];
        const float nrm_o = nrm[ord];
        const uint32_t f_lo = F[ord * 2], f_hi = F[ord * 2 + 1];
        const uint32_t id_o = nb_id[ord], det_o = det[ord];
        uint32_t n_sel = 1;
        uint32_t my_gi = (uint32_t)__builtin_amdgcn_readlane((int)ord, 0), my_kw = 0;
        bool my_live = lane == 0;
        float my_nrm = readlane_f32(nrm_o, 0);
        float p_next = 0.f;
        if (m > 1) p_next = G[(uint32_t)__builtin_amdgcn_readlane((int)ord, 1) * GRAM_STRIDE + my_gi];
        for (uint32_t t = 1; t < m; t++) {
            const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)ord, (int)t);
            const float norm_c = readlane_f32(nrm_o, t);
            const uint64_t fc = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)f_hi, (int)t) << 32) | (uint32_t)__builtin_amdgcn_readlane((int)f_lo, (int)t);
            const float p = p_next;
            if (t + 1 < m) {
                const uint32_t cn = (uint32_t)__builtin_amdgcn_readlane((int)ord, (int)(t + 1));
                p_next = G[cn * GRAM_STRIDE + ((uint32_t)lane == n_sel ? c : my_gi)];
            }
            const bool act = (uint32_t)lane < n_sel && my_live;
            const bool rej = act && norm_c < p, tomb = act && my_nrm < p, noflag = act && !((fc >> my_gi) & 1ull);
            const bool reject = __ballot(rej) != 0;
            const bool allflag = __ballot(noflag) == 0;
            if (tomb) my_live = false;
            if (!reject) {
                if ((uint32_t)lane == n_sel) { my_gi = c; my_live = true; my_nrm = norm_c; my_kw = allflag ? 1u : 0u; }
                n_sel++;
            }
        }
        // (e) emit: live members in selection order fill the row, flagged ones beyond d become keyword candidates
        const bool live = (uint32_t)lane < n_sel && my_live;
        const uint64_t lb = __ballot(live);
        const uint32_t pos = __popcll(lb & lane_lt);
        const uint32_t my_id = nb_id[my_gi], my_det = det[my_gi];
        if (live && pos < d) { o_fwd[pos] = my_id; o_det[pos] = my_det; }
        uint32_t cnt = min((uint32_t)__popcll(lb), d);
        const bool kwc = live && pos >= d && my_kw;
        const uint64_t kb = __ballot(kwc);
        const uint32_t kpos = __popcll(kb & lane_lt);
        if (kwc && kpos < APOE_KW_CAND) o_kw[1 + kpos] = my_id;
        const uint32_t nkw = min((uint32_t)__popcll(kb), (uint32_t)APOE_KW_CAND);
        if (cnt < d) { // fewer survivors than the row has slots: the remaining neighbours in order, each id once
            bool add = (uint32_t)lane < m;
            for (uint64_t rest = lb; rest; rest &= rest - 1) add = add && (uint32_t)__builtin_amdgcn_readlane((int)my_id, __builtin_ctzll(rest)) != id_o;
            for (uint32_t t = 0; t + 1 < m; t++) add = add && !((uint32_t)lane > t && (uint32_t)__builtin_amdgcn_readlane((int)id_o, (int)t) == id_o);
            const uint64_t ab = __ballot(add);
            const uint32_t at = cnt + __popcll(ab & lane_lt);
            if (add && at < d) { o_fwd[at] = id_o; o_det[at] = det_o; }
            cnt = min(d, cnt + (uint32_t)__popcll(ab));
        }
        if (lane == 0) { ctl[PC_CNT] = cnt; o_kw[0] = nkw; }
        for (uint32_t j = cnt + lane; j < d; j += WAVE) { o_fwd[j] = u; o_det[j] = EMPTY; }
        for (uint32_t j = nkw + lane; j < APOE_KW_CAND; j += WAVE) o_kw[1 + j] = 0;
    }
    if (m == 0 && tid == 0) {
        for (uint32_t j = 0; j < d; j++) { o_fwd[j] = u; o_det[j] = EMPTY; }
        for (uint32_t j = 0; j <= APOE_KW_CAND; j++) o_kw[j] = 0;
        ctl[PC_CNT] = 0;
    }
    __syncthreads();
    for (uint32_t i = tid; i < d; i += NT) {
        fwd[(size_t)u * d + i] = o_fwd[i];
        det_out[(size_t)u * d + i] = o_det[i];
    }
    for (uint32_t i = tid; i < 1 + APOE_KW_CAND; i += NT) kw_out[(size_t)u * (1 + APOE_KW_CAND) + i] = o_kw[i];
    if (tid == 0) {
        cnt_out[u] = ctl[PC_CNT];
        if (ctl[PC_FAIL]) atomicOr(gfail, 1ull);
        // an overflow list was too short: the host redoes the prune with prune_kernel
    }
}

// ---- final rows (index.cu:717-807) ----

__global__ __launch_bounds__(256) void indegree_kernel(uint32_t n, uint32_t d, const uint32_t* __restrict__ fwd, const uint32_t* __restrict__ cnt,
                                                       uint32_t* indeg) {
    const uint64_t total = (uint64_t)n * d;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t u = (uint32_t)(t / d), j = (uint32_t)(t % d);
        if (j >= cnt[u]) continue;
        const uint32_t v = fwd[t];
        if (v < n && v != u) atomicAdd(&indeg[v], 1u);
    }
}

__global__ __launch_bounds__(256) void fill_in_edges_kernel(uint32_t n, uint32_t d, const uint32_t* __restrict__ fwd,
                                                            const uint32_t* __restrict__ det, const uint32_t* __restrict__ cnt,
                                                            const uint32_t* __restrict__ in_off, uint32_t* cursor, uint64_t* in_edges) {
    const uint64_t total = (uint64_t)n * d;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t u = (uint32_t)(t / d), j = (uint32_t)(t % d);
        if (j >= cnt[u]) continue;
        const uint32_t v = fwd[t];
        if (v < n && v != u) in_edges[in_off[v] + atomicAdd(&cursor[v], 1u)] = ((uint64_t)det[t] << 32) | u;
    }
}

__device__ __forceinline__ uint64_t wave_min64(uint64_t v) {
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        const uint64_t other = shfl_xor64(v, o);
        v = other < v ? other : v;
    }
    return v;
}

// One wave per node v. Row = first half of v's forward list, then up to d/2 reverse
// neighbours in (detour, id) order that are not in the first half, topped up from the
// second half of the forward list and finally with v itself; then the keyword slots.
__global__ __launch_bounds__(256) void final_rows_kernel(uint32_t n, uint32_t d, const uint32_t* __restrict__ fwd, const uint32_t* __restrict__ kw,
                                                         const uint32_t* __restrict__ in_off, const uint64_t* __restrict__ in_edges,
                                                         uint32_t* rows) {
    __shared__ uint32_t s_row[4][WAVE + APOE_KW_SLOTS];
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const uint32_t v = blockIdx.x * 4 + wave;
    if (v >= n) return;
    uint32_t* row = s_row[wave];
    const uint32_t W = d + APOE_KW_SLOTS, h = d / 2;
    const uint32_t* fw = fwd + (size_t)v * d;
    if ((uint32_t)lane < h) row[lane] = fw[lane];
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    uint32_t fill = h;
    const uint32_t e0 = in_off[v], e1 = in_off[v + 1];
    {
        // the h smallest (detour, source) keys among the in-edges whose source is not in the first half, in one pass:
        // lanes 0 .. h-1 hold the best keys so far in ascending order; a chunk of 64 in-edges is tested against the
        // largest of them first (after a few chunks almost no key passes: a node with 10^5 in-edges costs one load and
        // one compare per 64 of them), the keys that pass are inserted one at a time
        uint64_t best = ~0ull; // lane i: the i-th smallest key so far (lanes >= h unused)
        for (uint32_t eb = e0; eb < e1; eb += WAVE) {
            const uint32_t e = eb + lane;
            uint64_t k = e < e1 ? in_edges[e] : ~0ull;
            const uint64_t worst = readlane64(best, h - 1);
            bool cand = k < worst;
            if (__ballot(cand) == 0) continue;
            if (cand) {
                const uint32_t uu = (uint32_t)k;
                bool present = false;
                for (uint32_t j = 0; j < h; j++) present |= row[j] == uu;
                cand = !present;
            }
            for (uint64_t rest = __ballot(cand); rest; rest &= rest - 1) {
                const uint64_t x = readlane64(k, (uint32_t)__builtin_ctzll(rest));
                const uint32_t pos = __popcll(__ballot(best < x)); // best is ascending: the lanes below pos keep their keys
                if (pos >= h) continue;
                const uint64_t up = __shfl_up(best, 1, WAVE);
                best = (uint32_t)lane == pos ? x : (uint32_t)lane > pos ? up : best;
            }
        }
        const uint32_t got = min((uint32_t)__popcll(__ballot(best != ~0ull && (uint32_t)lane < h)), h);
        if ((uint32_t)lane < got) row[h + lane] = (uint32_t)best;
        fill = h + got;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (uint32_t j = h; j < d && fill < d; j++) {
        const uint32_t c = fw[j];
        bool present = false;
        for (uint32_t t = lane; t < fill; t += WAVE) present |= row[t] == c;
        if (!__any(present)) {
            if (lane == 0) row[fill] = c;
            fill++;
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
    for (uint32_t j = fill + lane; j < d; j += WAVE) row[j] = v;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // keyword edges
    const uint32_t* kv = kw + (size_t)v * (1 + APOE_KW_CAND);
    const uint32_t nk = min(kv[0], (uint32_t)APOE_KW_CAND);
    if (lane < APOE_KW_SLOTS) row[d + lane] = 0;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    uint32_t c = 0;
    for (uint32_t j = 0; j < nk && c < APOE_KW_SLOTS - 1; j++) {
        const uint32_t x = kv[1 + j];
        bool present = false;
        for (uint32_t t = h + lane; t < d; t += WAVE) present |= row[t] == x;
        if (!__any(present)) {
            if (lane == 0) row[d + 1 + c] = x;
            c++;
        }
    }
    if (lane == 0) row[d] = c;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (uint32_t j = lane; j < W; j += WAVE) rows[(size_t)v * W + j] = row[j];
}

static uint32_t doc_term_slots(const apoe_corpus* c) { return next_pow2(std::max(64u, 2 * (c->max_nnz_s + c->max_nnz_b))); }

int launch_prune(apoe_knn* g, uint32_t degree) {
    apoe_ctx* ctx = g->ctx;
    const uint32_t term_slots = doc_term_slots(g->corpus);
    const uint32_t uset_slots = next_pow2(std::max(64u, 2 * g->corpus->max_nnz_b));
    const uint32_t map_slots = next_pow2(4 * g->K);
    // gather-once form: K = 64 and the BM25 overlap masks fit in LDS
    const uint32_t words = (g->corpus->max_nnz_b + 31) / 32 + (g->corpus->max_nnz_b == 0);
    const uint32_t gram_slots = next_pow2(std::max(64u, 2 * (g->corpus->max_nnz_s + g->corpus->max_nnz_b)));
    // 8 live pivot tables if two workgroups then still share a CU's LDS, else 4
    const uint32_t lds_budget = (uint32_t)std::min<size_t>(ctx->lds_per_block, 80 * 1024);
    uint32_t tgroup = GramPruneLds(gram_slots, 8, uset_slots, map_slots, words, 0).total <= lds_budget ? 8 : 4;
    // one union table for GU_T pivots when it fits: 2.5 slots per term of an average group, and room for the longest row alone
    const double mean_nnz = g->n ? (double)g->corpus->total_pairs / g->n : 0.0;
    uint32_t union_slots = std::max(next_pow2((uint32_t)std::ceil(2.5 * GU_T * mean_nnz)), std::max(512u, gram_slots));
    if (GramPruneLds(gram_slots, tgroup, uset_slots, map_slots, words, union_slots).total > lds_budget) union_slots = 0;
    // rank table for eight pivots when its bitmap leaves room for the values of at least the longest row (and then as many
    // slots as the budget allows, up to eight rows' worth): the sparse part then runs with the rows held in registers
    const bool narrow = g->corpus->narrow;
    const uint32_t rank_span = next_pow2(std::max(g->corpus->max_term + 1, 1024u));
    const uint32_t rank_bits = narrow ? 2 * rank_span : 65536u;
    uint32_t rank_slots = 0;
    {
        const uint32_t longest = g->corpus->max_nnz_s + g->corpus->max_nnz_b;
        const uint32_t fixed = GramPruneLds(gram_slots, tgroup, uset_slots, map_slots, words, 0, rank_bits, 64, narrow).total -
                               RankTabLds(rank_bits, 64, narrow).total + RankTabLds(rank_bits, 0, narrow).total;
        const uint32_t per_slot = RT_T * 4 + (narrow ? 0 : 4);
        if (fixed + 64 < lds_budget) {
            uint32_t fit = ((lds_budget - fixed - 64) / per_slot) & ~63u;
            fit = std::min(fit, (RT_T * longest + 63) & ~63u);
            if (fit >= std::max(longest, 64u)) rank_slots = fit;
        }
    }
    const GramPruneLds GL(gram_slots, tgroup, uset_slots, map_slots, words, union_slots, rank_bits, rank_slots, narrow);
    if (g->K == GRAM_ROWS && GL.total <= lds_budget && !g->force_sequential_prune) {
        APOE_HIP(hipMemsetAsync(g->counter.p + 1, 0, sizeof(unsigned long long), ctx->stream));
        auto kernel = g->corpus->narrow ? &prune_gram_kernel<GRAM_THREADS, true> : &prune_gram_kernel<GRAM_THREADS, false>;
        APOE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GL.total));
        kernel<<<g->n, GRAM_THREADS, GL.total, ctx->stream>>>(g->corpus->view(), g->dense_scale * g->dense_scale, g->norms.p, g->ids.p, g->dist.p, degree,
                                                              g->fwd.p, g->det.p, g->cnt.p, g->kw.p, gram_slots, tgroup, uset_slots, map_slots, words,
                                                              union_slots, rank_bits, rank_slots, rank_span, g->counter.p + 1);
        APOE_HIP(hipGetLastError());
        unsigned long long failed = 0;
        APOE_HIP(hipMemcpyAsync(&failed, g->counter.p + 1, sizeof(failed), hipMemcpyDeviceToHost, ctx->stream));
        APOE_HIP(hipStreamSynchronize(ctx->stream));
        if (!failed) return APOE_OK;
        // a row's terms clustered on the same table slots: redo with the table-probing kernel below
    }
    // lists longer than 64 entries: Gram matrices by the tile kernel of the local join, a batch of nodes at a time, and the
    // selection on them; a row too long for a tile's table sends the whole prune to the table-probing kernel below
    if (g->K > GRAM_ROWS && g->K <= PS_MAX && !g->force_sequential_prune && gram_tiles_fit(g)) {
        const SelectLds SL(uset_slots, map_slots, words);
        if (SL.total <= ctx->lds_per_block) {
            const uint32_t batch = std::min<uint32_t>(g->n, 32768u);
            DevBuf<float> gram;
            APOE_TRY(gram.alloc((size_t)batch * PS_MAX * PS_MAX));
            APOE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&prune_select_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)SL.total));
            unsigned long long unfit = 0;
            for (uint32_t node0 = 0; node0 < g->n && !unfit; node0 += batch) {
                const uint32_t cnt = std::min(batch, g->n - node0);
                APOE_TRY(launch_gram_tiles(g, node0, cnt, gram.p, &unfit));
                if (unfit) break;
                prune_select_kernel<<<cnt, PS_THREADS, SL.total, ctx->stream>>>(g->corpus->view(), g->norms.p, g->K, g->ids.p, g->dist.p, degree, node0, gram.p,
                                                                              g->fwd.p, g->det.p, g->cnt.p, g->kw.p, uset_slots, map_slots, words);
                APOE_HIP(hipGetLastError());
            }
            APOE_HIP(hipStreamSynchronize(ctx->stream)); // the batch buffer is freed on return
            if (!unfit) return APOE_OK;
        }
    }
    const PruneLds L(term_slots, uset_slots, map_slots, g->K);
    APOE_REQUIRE(L.total <= 64 * 1024, "prune needs %u bytes of LDS (rows with up to %u sparse terms)", L.total,
                 g->corpus->max_nnz_s + g->corpus->max_nnz_b);
    APOE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&prune_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total));
    prune_kernel<<<g->n, PR_THREADS, L.total, ctx->stream>>>(g->corpus->view(), g->dense_scale * g->dense_scale, g->norms.p, g->K, g->ids.p,
                                                             g->dist.p, degree, g->fwd.p, g->det.p, g->cnt.p, g->kw.p, term_slots, uset_slots,
                                                             map_slots);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

int launch_final_graph(apoe_knn* g, uint32_t* rows_dev) {
    apoe_ctx* ctx = g->ctx;
    const uint32_t n = g->n, d = g->degree;
    DevBuf<uint32_t> indeg, in_off, cursor;
    DevBuf<uint64_t> in_edges;
    DevBuf<char> temp;
    APOE_TRY(indeg.alloc((size_t)n + 1));
    APOE_TRY(in_off.alloc((size_t)n + 1));
    APOE_TRY(cursor.alloc(n));
    APOE_TRY(in_edges.alloc((size_t)n * d));
    APOE_HIP(hipMemsetAsync(indeg.p, 0, ((size_t)n + 1) * sizeof(uint32_t), ctx->stream));
    APOE_HIP(hipMemsetAsync(cursor.p, 0, (size_t)n * sizeof(uint32_t), ctx->stream));
    const uint32_t grid = (uint32_t)std::min<uint64_t>(((uint64_t)n * d + 255) / 256, 1u << 20);
    indegree_kernel<<<grid, 256, 0, ctx->stream>>>(n, d, g->fwd.p, g->cnt.p, indeg.p);
    APOE_HIP(hipGetLastError());
    size_t temp_bytes = 0;
    APOE_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, temp_bytes, indeg.p, in_off.p, (int)(n + 1), ctx->stream));
    APOE_TRY(temp.alloc(temp_bytes));
    APOE_HIP(hipcub::DeviceScan::ExclusiveSum(temp.p, temp_bytes, indeg.p, in_off.p, (int)(n + 1), ctx->stream));
    fill_in_edges_kernel<<<grid, 256, 0, ctx->stream>>>(n, d, g->fwd.p, g->det.p, g->cnt.p, in_off.p, cursor.p, in_edges.p);
    APOE_HIP(hipGetLastError());
    final_rows_kernel<<<(n + 3) / 4, 256, 0, ctx->stream>>>(n, d, g->fwd.p, g->kw.p, in_off.p, in_edges.p, rows_dev);
    APOE_HIP(hipGetLastError());
    APOE_HIP(hipStreamSynchronize(ctx->stream)); // temporaries are released on return
    return APOE_OK;
}

} // namespace apoe

using namespace apoe;

extern "C" {

int apoe_knn_set_prune_form(apoe_knn* g, int form) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE(form == 0 || form == 1, "prune form must be 0 (gather-once forms where they apply) or 1 (the table-probing kernel), got %d", form);
    g->force_sequential_prune = form == 1;
    return APOE_OK;
}

int apoe_prune(apoe_knn* g, uint32_t degree) {
    APOE_REQUIRE(g, "null argument");
    APOE_REQUIRE(degree >= 2 && degree <= 64 && degree % 2 == 0 && degree <= g->K, "degree must be even, in [2, 64] and <= K, got %u", degree);
    APOE_REQUIRE_STATE(g->ready, "the lists are empty: call apoe_nnd_init or apoe_knn_upload first");
    APOE_HIP(hipSetDevice(g->ctx->device));
    g->degree = degree;
    APOE_TRY(g->fwd.alloc((size_t)g->n * degree));
    APOE_TRY(g->det.alloc((size_t)g->n * degree));
    APOE_TRY(g->cnt.alloc(g->n));
    APOE_TRY(g->kw.alloc((size_t)g->n * (1 + APOE_KW_CAND)));
    float ms = 0.f;
    APOE_TRY(timed(g->ctx, &ms, [&]() { return launch_prune(g, degree); }));
    g->elapsed_ms += ms;
    g->pruned = true;
    return APOE_OK;
}

int apoe_prune_download(apoe_knn* g, uint32_t* fwd, uint32_t* det, uint32_t* cnt, uint32_t* kw) {
    APOE_REQUIRE(g, "null argument");
    if (!g->pruned) {
        set_error("apoe_prune has not run on this handle");
        return APOE_ERR_STATE;
    }
    APOE_HIP(hipSetDevice(g->ctx->device));
    if (fwd) APOE_TRY(copy_out(g->ctx, fwd, g->fwd.p, g->fwd.bytes()));
    if (det) APOE_TRY(copy_out(g->ctx, det, g->det.p, g->det.bytes()));
    if (cnt) APOE_TRY(copy_out(g->ctx, cnt, g->cnt.p, (size_t)g->n * sizeof(uint32_t)));
    if (kw) APOE_TRY(copy_out(g->ctx, kw, g->kw.p, g->kw.bytes()));
    return APOE_OK;
}

int apoe_finalize_graph(apoe_knn* g, apoe_graph** out) {
    APOE_REQUIRE(g && out, "null argument");
    *out = nullptr;
    if (!g->pruned) {
        set_error("apoe_prune has not run on this handle");
        return APOE_ERR_STATE;
    }
    APOE_HIP(hipSetDevice(g->ctx->device));
    std::unique_ptr<apoe_graph> gr(new apoe_graph());
    gr->ctx = g->ctx;
    gr->n = g->n;
    gr->width = g->degree + APOE_KW_SLOTS;
    gr->n_entry = g->degree;
    APOE_TRY(gr->rows.alloc((size_t)gr->n * gr->width));
    APOE_TRY(gr->entry.alloc(gr->n_entry));
    float ms = 0.f;
    APOE_TRY(timed(g->ctx, &ms, [&]() { return launch_final_graph(g, gr->rows.p); }));
    g->elapsed_ms += ms;
    // entry points: the `degree` documents of smallest hybrid norm, ties by id (index.cu:916-925)
    std::vector<float> nrm(g->n);
    APOE_TRY(copy_out(g->ctx, nrm.data(), g->norms.p, (size_t)g->n * sizeof(float)));
    std::vector<std::pair<float, uint32_t>> dp(g->n);
    for (uint32_t i = 0; i < g->n; i++) dp[i] = {nrm[i], i};
    const uint32_t k = std::min(gr->n_entry, g->n);
    std::partial_sort(dp.begin(), dp.begin() + k, dp.end());
    std::vector<uint32_t> ep(gr->n_entry);
    for (uint32_t i = 0; i < gr->n_entry; i++) ep[i] = dp[i % k].second;
    APOE_TRY(copy_in(g->ctx, gr->entry.p, ep.data(), ep.size() * sizeof(uint32_t)));
    *out = gr.release();
    return APOE_OK;
}

} // extern "C"
