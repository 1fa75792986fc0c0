// Hybrid Gram matrix of up to 64 documents, built once per workgroup in LDS:
// dense part on the matrix cores (fp32 MFMA 32x32x2, every wave the three upper 32x32 tiles over its
// share of the dimensions, rows read straight from the packed records), sparse part by scattering a few pivot rows at a time
// into LDS term tables that the later rows look their terms up in (the hashed tables below; the prune's
// default is the rank table of apoe_ranktab.h with the rows held in registers, prune.hip).
#pragma once

#include "apoe_device.h"

namespace apoe {

#ifdef __HIPCC__

typedef float floatx16 __attribute__((ext_vector_type(16)));
constexpr int GRAM_ROWS = 64;
constexpr int GRAM_STRIDE = GRAM_ROWS + 1; // odd stride: column reads do not collide on LDS banks

// Dense part of the Gram matrix on the matrix cores, fp32 in and out.
// MFMA 32x32x2 operand layout: lane l feeds A[l % 32][l / 32] and B[l / 32][l % 32];
// accumulator register v of lane l is C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].
// A lane therefore streams ITS row: float4 number (2 * block + l / 32) of every 8-float block,
// and the four components go into four consecutive MFMAs (the k order inside the sum is free).
// Rows >= m repeat row m - 1 (their entries are never read).
// The three tiles of the upper triangle at once, over the 8-float blocks [b_begin, b_end) of the rows: a wave reads
// its slice of rows 0-31 (operand a) and of rows 32-63 (operand b) once and feeds a x a, a x b and b x b from the same
// registers, so every dense row is read from memory exactly once per node (tile by tile each row block is read
// twice). m <= 32: only a x a. Batches of NB blocks, the next batch requested before the current one is multiplied.
template <int NB>
__device__ __forceinline__ void gram_dense_upper(const CorpusView& C, const uint32_t* ids, uint32_t m, int lane, int b_begin, int b_end,
                                                 floatx16& acc00, floatx16& acc01, floatx16& acc11) {
#pragma unroll
    for (int v = 0; v < 16; v++) { acc00[v] = 0.f; acc01[v] = 0.f; acc11[v] = 0.f; }
    if (m == 0) return;
    const bool has_b = m > 32;
    const uint32_t ra = min((uint32_t)(lane & 31), m - 1), rb = min((uint32_t)(32 + (lane & 31)), m - 1);
    const float4* pa = reinterpret_cast<const float4*>(C.recs + desc_off(C.desc[ids[ra]]) * 16) + (lane >> 5);
    const float4* pb = reinterpret_cast<const float4*>(C.recs + desc_off(C.desc[ids[rb]]) * 16) + (lane >> 5);
    float4 a[2][NB], bb[2][NB];
#pragma unroll
    for (int u = 0; u < NB; u++) {
        a[0][u] = pa[2 * (b_begin + u)];
        bb[0][u] = has_b ? pb[2 * (b_begin + u)] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll 1
    for (int b = b_begin; b < b_end; b += 2 * NB) {
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int nb = b + (half + 1) * NB; // first block of the batch after this one
            if (nb < b_end) {
#pragma unroll
                for (int u = 0; u < NB; u++) {
                    a[half ^ 1][u] = pa[2 * (nb + u)];
                    if (has_b) bb[half ^ 1][u] = pb[2 * (nb + u)];
                }
            }
#pragma unroll
            for (int u = 0; u < NB; u++) {
                const float4 x = a[half][u], y = bb[half][u];
                acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, x.x, acc00, 0, 0, 0);
                acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, x.y, acc00, 0, 0, 0);
                acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, x.z, acc00, 0, 0, 0);
                acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, x.w, acc00, 0, 0, 0);
                if (has_b) {
                    acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, y.x, acc01, 0, 0, 0);
                    acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, y.y, acc01, 0, 0, 0);
                    acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, y.z, acc01, 0, 0, 0);
                    acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, y.w, acc01, 0, 0, 0);
                    acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.x, y.x, acc11, 0, 0, 0);
                    acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.y, y.y, acc11, 0, 0, 0);
                    acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.z, y.z, acc11, 0, 0, 0);
                    acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(y.w, y.w, acc11, 0, 0, 0);
                }
            }
        }
    }
}

__device__ __forceinline__ void gram_dense_store(float* G, int tile, int lane, const floatx16& acc, float dense_mul, bool add) {
    const int ti = tile >> 1, tj = tile & 1;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int i = 8 * (v / 4) + 4 * (lane >> 5) + (v % 4), j = lane & 31;
        float* at = &G[(ti * 32 + i) * GRAM_STRIDE + tj * 32 + j];
        *at = add ? *at + dense_mul * acc[v] : dense_mul * acc[v];
    }
}

// ---- sparse part ----
// Pivots are taken T at a time. Each pivot row is scattered into its own table with THREE
// candidate slots per term (first free one wins; the rare term that finds all three taken
// goes to a short overflow list), so a lookup is three independent 8-byte LDS reads and no
// probe loop: a lane issues the reads for all its terms and all T pivots back to back.
// Every later row is read once per group (pairs in registers, the next row's loads already
// in flight), per-lane partial sums are reduced once per (row, pivot) with DPP adds, and
// lane 0 adds the result to G. Two barriers per group of T pivots; the lower triangle is
// mirrored at the end.
constexpr int GRAM_CHUNKS = 5;  // 64-pair chunks of a row kept in registers (320 pairs)
constexpr int GRAM_OVF = 32;    // overflow entries per pivot table

struct RowPairs { // raw pairs: the consumer adds pair_flag()
    uint2 kv[GRAM_CHUNKS];
};

__device__ __forceinline__ void row_pairs_load(RowPairs& r, const Pairs& sp, int lane) {
#pragma unroll
    for (int c = 0; c < GRAM_CHUNKS; c++) {
        const uint32_t j = c * WAVE + lane;
        r.kv[c] = j < sp.nnz ? sp.raw(j) : make_uint2(EMPTY, 0u);
    }
}
// Chunk c of a prefetched row as (term | path bit, value); a padding lane gives (EMPTY, 0): value 0
// adds nothing, and key EMPTY matches only empty slots, whose value is 0.
__device__ __forceinline__ uint2 row_pairs_get(const RowPairs& r, int c, uint32_t narrow, uint32_t ns, int lane) {
    uint2 kv = r.kv[c];
    if (kv.x == EMPTY) kv.y = 0u;
    else kv.x |= pair_flag(narrow, ns, c * WAVE + lane);
    return kv;
}

// The 64 gathered rows are kept in LDS as the address of the pair array and one word with
// nnz (low half) and nnz_s (high half); nnz <= 2 * DESC_NNZ_MAX fits 16 bits.
__device__ __forceinline__ void gram_rows_gather(const CorpusView& C, const uint32_t* ids, uint32_t m, unsigned long long* rowptr, uint32_t* rownnz,
                                                 int tid, int nthreads) {
    for (uint32_t i = tid; i < m; i += nthreads) {
        const uint64_t d = C.desc[ids[i]];
        rowptr[i] = (unsigned long long)(C.recs + desc_off(d) * 16 + DENSE_BYTES);
        rownnz[i] = (desc_nnz_s(d) + desc_nnz_b(d)) | (desc_nnz_s(d) << 16);
    }
}
__device__ __forceinline__ Pairs gram_row(const CorpusView& C, const unsigned long long* rowptr, const uint32_t* rownnz, uint32_t i) {
    Pairs p;
    p.base = reinterpret_cast<const char*>(rowptr[i]);
    const uint32_t w = rownnz[i];
    p.nnz = w & 0xFFFFu;
    p.ns = w >> 16;
    p.narrow = C.narrow;
    return p;
}

struct Slots3 {
    uint32_t a, b, c;
};
__device__ __forceinline__ Slots3 gram_slots3(uint32_t key, uint32_t mask) {
    const uint32_t k = key ^ (key >> 16); // the BM25 bit must reach the middle bits too
    Slots3 s;
    s.a = ((k * 0x9E3779B1u) >> 11) & mask;
    s.b = (((k ^ 0x5BD1E995u) * 0x85EBCA6Bu) >> 13) & mask;
    s.c = (((k + 0x7F4A7C15u) * 0xC2B2AE35u) >> 9) & mask;
    return s;
}

// tabs: T tables of `slots` entries, then T overflow lists of GRAM_OVF entries; ovf_cnt[T];
// rowptr/rownnz: LDS scratch for 64 rows; *fail is set when an overflow list is too short
// (the caller must then discard G). All threads of the block call it; G must already hold
// the dense part. slots >= 2 x the longest row.
template <int T>
__device__ __forceinline__ void gram_sparse_64(const CorpusView& C, const uint32_t* ids, uint32_t m, float* G, uint2* tabs, uint32_t slots,
                                               uint32_t* ovf_cnt, unsigned long long* rowptr, uint32_t* rownnz, uint32_t* fail, int tid,
                                               int nthreads) {
    const uint32_t mask = slots - 1;
    const int wave = tid / WAVE, lane = tid & (WAVE - 1), nwaves = nthreads / WAVE;
    uint2* ovf = tabs + (size_t)T * slots;
    gram_rows_gather(C, ids, m, rowptr, rownnz, tid, nthreads);
    __syncthreads();
    for (uint32_t a0 = 0; a0 + 1 < m; a0 += T) {
        const uint32_t nt = min((uint32_t)T, m - 1 - a0); // the last row is never a pivot
        for (uint32_t i = tid; i < T * slots; i += nthreads) tabs[i] = make_uint2(EMPTY, 0u);
        if (tid < T) ovf_cnt[tid] = 0;
        __syncthreads();
        for (uint32_t t = 0; t < nt; t++) {
            const Pairs sp = gram_row(C, rowptr, rownnz, a0 + t);
            const uint32_t nnz = sp.nnz;
            uint2* tab = tabs + (size_t)t * slots;
            for (uint32_t j = tid; j < nnz; j += nthreads) {
                const uint2 kv = sp[j];
                const Slots3 s3 = gram_slots3(kv.x, mask);
                uint32_t old = atomicCAS(&tab[s3.a].x, EMPTY, kv.x);
                if (old == EMPTY) { tab[s3.a].y = kv.y; continue; }
                if (old == kv.x) continue;
                old = atomicCAS(&tab[s3.b].x, EMPTY, kv.x);
                if (old == EMPTY) { tab[s3.b].y = kv.y; continue; }
                if (old == kv.x) continue;
                old = atomicCAS(&tab[s3.c].x, EMPTY, kv.x);
                if (old == EMPTY) { tab[s3.c].y = kv.y; continue; }
                if (old == kv.x) continue;
                const uint32_t at = atomicAdd(&ovf_cnt[t], 1u);
                if (at < GRAM_OVF) ovf[t * GRAM_OVF + at] = kv;
                else *fail = 1;
            }
        }
        __syncthreads();
        uint32_t novf[T];
#pragma unroll
        for (int t = 0; t < T; t++) novf[t] = uniform(min(ovf_cnt[t], (uint32_t)GRAM_OVF));
        uint32_t b = a0 + 1 + wave;
        RowPairs cur;
        if (b < m) row_pairs_load(cur, gram_row(C, rowptr, rownnz, b), lane);
        while (b < m) {
            const uint32_t bn = b + nwaves;
            RowPairs nxt;
            if (bn < m) row_pairs_load(nxt, gram_row(C, rowptr, rownnz, bn), lane);
            const uint32_t nnz = rownnz[b] & 0xFFFFu, ns_b = rownnz[b] >> 16;
            const uint32_t np = min(nt, b - a0); // pivots a0 .. a0+np-1 precede row b
            float acc[T];
#pragma unroll
            for (int t = 0; t < T; t++) acc[t] = 0.f;
            auto lookup = [&](uint2 kv) {
                const Slots3 s3 = gram_slots3(kv.x, mask);
                const float val = __uint_as_float(kv.y);
                // all 3*T reads are issued before any compare: the empty asm keeps the compiler
                // from sinking the second and third read behind a branch on the first
                uint2 e[T][3];
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const uint2* tab = tabs + (size_t)t * slots;
                    e[t][0] = tab[s3.a];
                    e[t][1] = tab[s3.b];
                    e[t][2] = tab[s3.c];
                }
#pragma unroll
                for (int t = 0; t < T; t++)
                    asm volatile("" : "+v"(e[t][0].x), "+v"(e[t][0].y), "+v"(e[t][1].x), "+v"(e[t][1].y), "+v"(e[t][2].x), "+v"(e[t][2].y));
#pragma unroll
                for (int t = 0; t < T; t++) {
                    if ((uint32_t)t < np) { // wave-uniform
                        const uint32_t hit = (e[t][0].x == kv.x ? e[t][0].y : 0u) | (e[t][1].x == kv.x ? e[t][1].y : 0u) |
                                             (e[t][2].x == kv.x ? e[t][2].y : 0u);
                        acc[t] = fmaf(val, __uint_as_float(hit), acc[t]);
                        for (uint32_t o = 0; o < novf[t]; o++) { // uniform, almost always zero trips
                            const uint2 ov = ovf[t * GRAM_OVF + o];
                            if (ov.x == kv.x) acc[t] = fmaf(val, __uint_as_float(ov.y), acc[t]);
                        }
                    }
                }
            };
#pragma unroll
            for (int c = 0; c < GRAM_CHUNKS; c++) {
                if (c * WAVE < (int)nnz) { // wave-uniform
                    lookup(row_pairs_get(cur, c, C.narrow, ns_b, lane));
                }
            }
            if (nnz > GRAM_CHUNKS * WAVE) { // rows longer than the register window
                const Pairs sp = gram_row(C, rowptr, rownnz, b);
                for (uint32_t j0 = GRAM_CHUNKS * WAVE; j0 < nnz; j0 += WAVE) {
                    const uint32_t j = j0 + lane;
                    lookup(j < nnz ? sp[j] : make_uint2(EMPTY, 0u));
                }
            }
#pragma unroll
            for (int t = 0; t < T; t++) {
                if ((uint32_t)t < np) {
                    const float sres = wave_sum_dpp(acc[t]);
                    if (lane == 0) G[(a0 + t) * GRAM_STRIDE + b] += sres;
                }
            }
            cur = nxt;
            b = bn;
        }
        __syncthreads();
    }
    for (uint32_t t = tid; t < m * m; t += nthreads) {
        const uint32_t i = t / m, j = t % m;
        if (i > j) G[i * GRAM_STRIDE + j] = G[j * GRAM_STRIDE + i];
    }
    __syncthreads();
}

// ---- sparse part, union-table form ----
// The terms of GU_T pivot rows go into ONE table: a term's slot holds GU_T values, one per pivot
// (zero where the pivot lacks the term). A pair of a later row is then looked up once per group
// instead of once per pivot, and most lookups end at the key compare because most terms of a row
// are in none of the pivots. Keys sit in buckets of 8 (two ds_read_b128), values in float4 slots
// (one ds_read_b128, read with the hit masked into the multiplier, so there is no branch); a term
// whose bucket is full goes to a short overflow list. When the pivots of a group hold more distinct
// terms than the table takes, the group is retried with half as many pivots; one row always fits
// (the host sizes the table for the longest row), else *fail is raised and G must be discarded.
constexpr int GU_T = 4;      // pivots per union table
constexpr int GU_BUCKET = 8; // keys per bucket
constexpr int GU_OVF = 32;   // overflow terms per group

struct GramUnionLds { // byte offsets inside the table region
    uint32_t keys, vals, ovf_key, ovf_val, total;
    __host__ __device__ explicit GramUnionLds(uint32_t slots) {
        uint32_t o = 0;
        keys = o; o += slots * 4;
        vals = o; o += slots * GU_T * 4;
        ovf_key = o; o += GU_OVF * 4;
        ovf_val = o; o += GU_OVF * GU_T * 4;
        total = o;
    }
};

__device__ __forceinline__ uint32_t gu_hash(uint32_t key, uint32_t bucket_mask) {
    const uint32_t k = key ^ (key >> 15); // the BM25 bit must reach the multiplied bits
    return ((k * 0x9E3779B1u) >> 14) & bucket_mask;
}

// ctl2: two LDS words (overflow count, spare). slots: power of two, >= 2 x the longest row.
__device__ __forceinline__ void gram_sparse_union(const CorpusView& C, const uint32_t* ids, uint32_t m, float* G, char* table, uint32_t slots,
                                                  uint32_t* ctl2, unsigned long long* rowptr, uint32_t* rownnz, uint32_t* fail, int tid,
                                                  int nthreads) {
    const GramUnionLds L(slots);
    uint32_t* keys = reinterpret_cast<uint32_t*>(table + L.keys);
    float* vals = reinterpret_cast<float*>(table + L.vals);
    uint32_t* ovf_key = reinterpret_cast<uint32_t*>(table + L.ovf_key);
    float* ovf_val = reinterpret_cast<float*>(table + L.ovf_val);
    const uint4* keys4 = reinterpret_cast<const uint4*>(keys);
    const float4* vals4 = reinterpret_cast<const float4*>(vals);
    const float4* ovf_val4 = reinterpret_cast<const float4*>(ovf_val);
    const uint32_t bmask = slots / GU_BUCKET - 1;
    const int wave = (int)uniform(tid / WAVE), lane = tid & (WAVE - 1), nwaves = nthreads / WAVE;
    gram_rows_gather(C, ids, m, rowptr, rownnz, tid, nthreads);
    __syncthreads();
    uint32_t a0 = 0;
    while (a0 + 1 < m) { // the last row is never a pivot
        uint32_t nt = min((uint32_t)GU_T, m - 1 - a0);
        while (true) {
            for (uint32_t i = tid; i < slots; i += nthreads) keys[i] = EMPTY;
            for (uint32_t i = tid; i < slots * GU_T / 4; i += nthreads) reinterpret_cast<float4*>(vals)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            for (uint32_t i = tid; i < GU_OVF; i += nthreads) ovf_key[i] = EMPTY;
            for (uint32_t i = tid; i < GU_OVF * GU_T; i += nthreads) ovf_val[i] = 0.f;
            if (tid == 0) ctl2[0] = 0;
            __syncthreads();
            // wave w scatters pivot (w % GU_T); waves w and w + GU_T share a pivot
            const uint32_t t = (uint32_t)wave % GU_T;
            if (t < nt) {
                const Pairs sp = gram_row(C, rowptr, rownnz, a0 + t);
                const uint32_t nnz = sp.nnz;
                const uint32_t step = (uint32_t)(nwaves / GU_T > 0 ? nwaves / GU_T : 1) * WAVE;
                for (uint32_t j = (uint32_t)(wave / GU_T) * WAVE + lane; j < nnz; j += step) {
                    const uint2 kv = sp[j];
                    const uint32_t b0 = gu_hash(kv.x, bmask) * GU_BUCKET;
                    uint32_t slot = EMPTY;
                    for (uint32_t s = 0; s < GU_BUCKET; s++) {
                        const uint32_t old = atomicCAS(&keys[b0 + s], EMPTY, kv.x);
                        if (old == EMPTY || old == kv.x) { slot = b0 + s; break; }
                    }
                    if (slot != EMPTY) {
                        vals[slot * GU_T + t] = __uint_as_float(kv.y);
                    } else {
                        uint32_t at = EMPTY;
                        for (uint32_t s = 0; s < GU_OVF; s++) {
                            const uint32_t old = atomicCAS(&ovf_key[s], EMPTY, kv.x);
                            if (old == EMPTY) atomicAdd(&ctl2[0], 1u);
                            if (old == EMPTY || old == kv.x) { at = s; break; }
                        }
                        if (at != EMPTY) ovf_val[at * GU_T + t] = __uint_as_float(kv.y);
                        else atomicAdd(&ctl2[0], GU_OVF + 1u); // the list is full too
                    }
                }
            }
            __syncthreads();
            const uint32_t filled = ctl2[0];
            if (filled <= GU_OVF) break;
            if (nt == 1) { // one row does not fit: the caller falls back
                if (tid == 0) *fail = 1;
                break;
            }
            nt = (nt + 1) / 2;
            __syncthreads();
        }
        const uint32_t novf = uniform(min(ctl2[0], (uint32_t)GU_OVF));
        uint32_t b = a0 + 1 + wave;
        RowPairs cur;
        if (b < m) row_pairs_load(cur, gram_row(C, rowptr, rownnz, b), lane);
        while (b < m) {
            const uint32_t bn = b + nwaves;
            RowPairs nxt;
            if (bn < m) row_pairs_load(nxt, gram_row(C, rowptr, rownnz, bn), lane);
            const uint32_t nnz = uniform(rownnz[b] & 0xFFFFu), ns_b = uniform(rownnz[b] >> 16);
            const uint32_t np = min(nt, b - a0); // pivots a0 .. a0+np-1 precede row b
            float acc[GU_T];
#pragma unroll
            for (int t = 0; t < GU_T; t++) acc[t] = 0.f;
            // one pair against the union table: keys of its bucket, then the value slot of the key that matched
            auto match = [&](const uint4 k0, const uint4 k1, uint32_t bucket, uint2 kv, uint32_t& slot) -> float {
                const uint32_t off = k0.x == kv.x ? 0u : k0.y == kv.x ? 1u : k0.z == kv.x ? 2u : k0.w == kv.x ? 3u : k1.x == kv.x ? 4u
                                     : k1.y == kv.x ? 5u : k1.z == kv.x ? 6u : k1.w == kv.x ? 7u : 8u;
                slot = bucket * GU_BUCKET + (off & 7u);
                return off < 8u ? __uint_as_float(kv.y) : 0.f; // a miss multiplies whatever the slot holds by zero
            };
            auto overflow = [&](uint2 kv) {
                for (uint32_t o = 0; o < novf; o++) { // uniform, almost always zero trips
                    if (ovf_key[o] == kv.x) {
                        const float4 v = ovf_val4[o];
                        const float val = __uint_as_float(kv.y);
                        acc[0] = fmaf(val, v.x, acc[0]);
                        acc[1] = fmaf(val, v.y, acc[1]);
                        acc[2] = fmaf(val, v.z, acc[2]);
                        acc[3] = fmaf(val, v.w, acc[3]);
                    }
                }
            };
            // the first three chunks (192 pairs) as one batch: six key reads, then three value reads
            {
                uint2 kv[3];
                uint32_t bk[3], slot[3];
                uint4 k0[3], k1[3];
#pragma unroll
                for (int c = 0; c < 3; c++) {
                    kv[c] = row_pairs_get(cur, c, C.narrow, ns_b, lane);
                    bk[c] = gu_hash(kv[c].x, bmask);
                    k0[c] = keys4[bk[c] * 2];
                    k1[c] = keys4[bk[c] * 2 + 1];
                }
                asm volatile("" : "+v"(k0[0].x), "+v"(k1[0].x), "+v"(k0[1].x), "+v"(k1[1].x), "+v"(k0[2].x), "+v"(k1[2].x));
                float val[3];
                float4 v[3];
#pragma unroll
                for (int c = 0; c < 3; c++) {
                    val[c] = match(k0[c], k1[c], bk[c], kv[c], slot[c]);
                    v[c] = vals4[slot[c]];
                }
                asm volatile("" : "+v"(v[0].x), "+v"(v[1].x), "+v"(v[2].x));
#pragma unroll
                for (int c = 0; c < 3; c++) {
                    acc[0] = fmaf(val[c], v[c].x, acc[0]);
                    acc[1] = fmaf(val[c], v[c].y, acc[1]);
                    acc[2] = fmaf(val[c], v[c].z, acc[2]);
                    acc[3] = fmaf(val[c], v[c].w, acc[3]);
                }
                if (novf) {
#pragma unroll
                    for (int c = 0; c < 3; c++) overflow(kv[c]);
                }
            }
            auto lookup = [&](uint2 kv) {
                if (kv.x == EMPTY) kv.y = 0u;
                const uint32_t bk = gu_hash(kv.x, bmask);
                uint32_t slot;
                const float val = match(keys4[bk * 2], keys4[bk * 2 + 1], bk, kv, slot);
                const float4 v = vals4[slot];
                acc[0] = fmaf(val, v.x, acc[0]);
                acc[1] = fmaf(val, v.y, acc[1]);
                acc[2] = fmaf(val, v.z, acc[2]);
                acc[3] = fmaf(val, v.w, acc[3]);
                if (novf) overflow(kv);
            };
#pragma unroll
            for (int c = 3; c < GRAM_CHUNKS; c++)
                if (c * WAVE < (int)nnz) lookup(row_pairs_get(cur, c, C.narrow, ns_b, lane)); // wave-uniform
            if (nnz > GRAM_CHUNKS * WAVE) { // rows longer than the register window
                const Pairs sp = gram_row(C, rowptr, rownnz, b);
                for (uint32_t j0 = GRAM_CHUNKS * WAVE; j0 < nnz; j0 += WAVE) {
                    const uint32_t j = j0 + lane;
                    lookup(j < nnz ? sp[j] : make_uint2(EMPTY, 0u));
                }
            }
            // four sums over the wave at once: after two exchange-and-add steps inside each quad, lane l
            // holds pivot t(l) = 2 * (l & 1) + ((l >> 1) & 1) summed over its quad; the rest is one sum per lane
            {
                const bool odd = lane & 1, hi = lane & 2;
                const float keep0 = odd ? acc[2] : acc[0], keep1 = odd ? acc[3] : acc[1];
                const float give0 = odd ? acc[0] : acc[2], give1 = odd ? acc[1] : acc[3];
                const float x0 = keep0 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give0), 0xB1, 0xF, 0xF, false));
                const float x1 = keep1 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give1), 0xB1, 0xF, 0xF, false));
                const float keep = hi ? x1 : x0, give = hi ? x0 : x1;
                float z = keep + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give), 0x4E, 0xF, 0xF, false));
                z += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, z), 0x124, 0xF, 0xF, false)); // row_ror:4
                z += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, z), 0x128, 0xF, 0xF, false)); // row_ror:8
                z += __shfl_xor(z, 16, WAVE);
                z += __shfl_xor(z, 32, WAVE);
                const uint32_t t = 2u * (lane & 1) + ((lane >> 1) & 1);
                if (lane < GU_T && t < np) G[(a0 + t) * GRAM_STRIDE + b] += z;
            }
            cur = nxt;
            b = bn;
        }
        __syncthreads();
        a0 += nt;
    }
    for (uint32_t t = tid; t < m * m; t += nthreads) {
        const uint32_t i = t / m, j = t % m;
        if (i > j) G[i * GRAM_STRIDE + j] = G[j * GRAM_STRIDE + i];
    }
    __syncthreads();
}

#endif // __HIPCC__

} // namespace apoe
