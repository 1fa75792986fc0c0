// Hybrid Gram matrix of up to 64 documents, built once per workgroup in LDS:
// dense part on the matrix cores (fp32 MFMA 32x32x2, one 32x32 tile per wave, rows read
// straight from the packed records), sparse part by scattering a few pivot rows at a time
// into LDS term tables that the later rows look their terms up in.
#pragma once

#include "apoe_device.h"

namespace apoe {

#ifdef __HIPCC__

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int GRAM_ROWS = 64;
constexpr int GRAM_STRIDE = GRAM_ROWS + 1; // odd stride: column reads do not collide on LDS banks

// G[i][j] = dense_mul * <dense_i, dense_j> for i, j < 64; rows >= m repeat row m-1 (their
// entries are never read). Called by 4 waves; wave w owns tile (w >> 1, w & 1).
// MFMA 32x32x2 operand layout: lane l feeds A[l % 32][l / 32] and B[l / 32][l % 32];
// accumulator register v of lane l is C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].
// A lane therefore streams ITS row: float4 number (2 * block + l / 32) of every 8-float block,
// and the four components go into four consecutive MFMAs (the k order inside the sum is free).
__device__ __forceinline__ void gram_dense_64(const CorpusView& C, const uint32_t* ids, uint32_t m, float dense_mul, float* G, int wave,
                                              int lane) {
    const int ti = wave >> 1, tj = wave & 1;
    if ((uint32_t)(ti * 32) >= m || (uint32_t)(tj * 32) >= m) return;
    const uint32_t ra = min((uint32_t)(ti * 32 + (lane & 31)), m - 1), rb = min((uint32_t)(tj * 32 + (lane & 31)), m - 1);
    const float4* pa = reinterpret_cast<const float4*>(C.recs + desc_off(C.desc[ids[ra]]) * 16) + (lane >> 5);
    const float4* pb = reinterpret_cast<const float4*>(C.recs + desc_off(C.desc[ids[rb]]) * 16) + (lane >> 5);
    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.f;
    if (ti == tj) {
        for (int b = 0; b < DIM / 8; b += 4) {
            float4 a[4];
#pragma unroll
            for (int u = 0; u < 4; u++) a[u] = pa[2 * (b + u)];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].x, a[u].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].y, a[u].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].z, a[u].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].w, a[u].w, acc, 0, 0, 0);
            }
        }
    } else {
        for (int b = 0; b < DIM / 8; b += 4) {
            float4 a[4], bb[4];
#pragma unroll
            for (int u = 0; u < 4; u++) { a[u] = pa[2 * (b + u)]; bb[u] = pb[2 * (b + u)]; }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].x, bb[u].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].y, bb[u].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].z, bb[u].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].w, bb[u].w, acc, 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int i = 8 * (v / 4) + 4 * (lane >> 5) + (v % 4), j = lane & 31;
        G[(ti * 32 + i) * GRAM_STRIDE + tj * 32 + j] = dense_mul * acc[v];
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

struct RowPairs {
    uint2 kv[GRAM_CHUNKS];
};

__device__ __forceinline__ void row_pairs_load(RowPairs& r, const uint2* sp, uint32_t nnz, int lane) {
#pragma unroll
    for (int c = 0; c < GRAM_CHUNKS; c++) {
        const uint32_t j = c * WAVE + lane;
        r.kv[c] = j < nnz ? sp[j] : make_uint2(EMPTY, 0u);
    }
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
    for (uint32_t i = tid; i < m; i += nthreads) {
        const uint64_t d = C.desc[ids[i]];
        rowptr[i] = (unsigned long long)(C.recs + desc_off(d) * 16 + DENSE_BYTES);
        rownnz[i] = desc_nnz_s(d) + desc_nnz_b(d);
    }
    __syncthreads();
    for (uint32_t a0 = 0; a0 + 1 < m; a0 += T) {
        const uint32_t nt = min((uint32_t)T, m - 1 - a0); // the last row is never a pivot
        for (uint32_t i = tid; i < T * slots; i += nthreads) tabs[i] = make_uint2(EMPTY, 0u);
        if (tid < T) ovf_cnt[tid] = 0;
        __syncthreads();
        for (uint32_t t = 0; t < nt; t++) {
            const uint2* sp = reinterpret_cast<const uint2*>(rowptr[a0 + t]);
            const uint32_t nnz = rownnz[a0 + t];
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
        if (b < m) row_pairs_load(cur, reinterpret_cast<const uint2*>(rowptr[b]), rownnz[b], lane);
        while (b < m) {
            const uint32_t bn = b + nwaves;
            RowPairs nxt;
            if (bn < m) row_pairs_load(nxt, reinterpret_cast<const uint2*>(rowptr[bn]), rownnz[bn], lane);
            const uint32_t nnz = rownnz[b];
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
                    uint2 kv = cur.kv[c];
                    if (kv.x == EMPTY) kv.y = 0u; // padding lane: value 0 adds nothing, key EMPTY matches only empty slots whose value is 0
                    lookup(kv);
                }
            }
            if (nnz > GRAM_CHUNKS * WAVE) { // rows longer than the register window
                const uint2* sp = reinterpret_cast<const uint2*>(rowptr[b]);
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

#endif // __HIPCC__

} // namespace apoe
