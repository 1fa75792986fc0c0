// Corpus packing, fused hybrid distance (batch and pair forms) and hybrid norms.
#include "apoe_internal.h"

namespace apoe {

// Largest value of an index array (decides whether the corpus can use narrow pairs).
__global__ __launch_bounds__(256) void max_u32_kernel(const uint32_t* __restrict__ a, size_t n, uint32_t* out) {
    uint32_t m = 0;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) m = max(m, a[i]);
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) m = max(m, (uint32_t)__shfl_xor(m, o, WAVE));
    if (lane_id() == 0 && m) atomicMax(out, m);
}

int launch_max_u32(apoe_ctx* ctx, const uint32_t* a_dev, size_t n, uint32_t* out_dev) { // *out_dev must hold 0 (or a running maximum)
    if (n == 0) return APOE_OK;
    const uint32_t grid = (uint32_t)std::min<size_t>((n + 255) / 256, 4096);
    max_u32_kernel<<<grid, 256, 0, ctx->stream>>>(a_dev, n, out_dev);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

// One workgroup per document: dense row, then SPLADE pairs, then BM25 pairs, written as one
// contiguous record in the wide (path bit in the term key) or the narrow pair format.
__global__ __launch_bounds__(256) void pack_kernel(uint32_t n, const float* __restrict__ dense, const uint32_t* __restrict__ s_off,
                                                   const uint32_t* __restrict__ s_idx, const float* __restrict__ s_val,
                                                   const uint32_t* __restrict__ b_off, const uint32_t* __restrict__ b_idx,
                                                   const float* __restrict__ b_val, const uint64_t* __restrict__ desc, char* recs, float* dnorm,
                                                   uint32_t narrow) {
    __shared__ float part[4];
    for (uint32_t doc = blockIdx.x; doc < n; doc += gridDim.x) {
        const uint64_t d = desc[doc];
        char* rec = recs + desc_off(d) * 16;
        const float4* src = reinterpret_cast<const float4*>(dense + (size_t)doc * DIM);
        float4* dst = reinterpret_cast<float4*>(rec);
        float sq = 0.f;
        for (int i = threadIdx.x; i < DIM / 4; i += blockDim.x) {
            const float4 x = src[i];
            dst[i] = x;
            sq += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
        }
        sq = wave_sum_dpp(sq);
        __syncthreads();
        if (lane_id() == 0) part[threadIdx.x / WAVE] = sq;
        __syncthreads();
        if (threadIdx.x == 0) dnorm[doc] = sqrtf(part[0] + part[1] + part[2] + part[3]);
        const uint32_t s0 = s_off[doc], ns = desc_nnz_s(d), b0 = b_off[doc], nb = desc_nnz_b(d), nnz = ns + nb;
        if (narrow) {
            float* vals = reinterpret_cast<float*>(rec + DENSE_BYTES);
            uint16_t* keys = reinterpret_cast<uint16_t*>(rec + DENSE_BYTES + narrow_keys_offset(nnz));
            for (uint32_t j = threadIdx.x; j < ns; j += blockDim.x) {
                vals[j] = s_val[s0 + j];
                keys[j] = (uint16_t)s_idx[s0 + j];
            }
            for (uint32_t j = threadIdx.x; j < nb; j += blockDim.x) {
                vals[ns + j] = b_val[b0 + j];
                keys[ns + j] = (uint16_t)b_idx[b0 + j];
            }
            // fill the two alignment gaps so that a record never holds stale bytes
            for (uint32_t j = nnz + threadIdx.x; j < narrow_keys_offset(nnz) / 4; j += blockDim.x) vals[j] = 0.f;
            const uint32_t key_slots = (uint32_t)(record_units(nnz, true) * 16 - DENSE_BYTES - narrow_keys_offset(nnz)) / 2;
            for (uint32_t j = nnz + threadIdx.x; j < key_slots; j += blockDim.x) keys[j] = 0xFFFFu;
        } else {
            uint2* sp = reinterpret_cast<uint2*>(rec + DENSE_BYTES);
            for (uint32_t j = threadIdx.x; j < ns; j += blockDim.x) sp[j] = make_uint2(s_idx[s0 + j], __float_as_uint(s_val[s0 + j]));
            for (uint32_t j = threadIdx.x; j < nb; j += blockDim.x)
                sp[ns + j] = make_uint2(b_idx[b0 + j] | BM25_BIT, __float_as_uint(b_val[b0 + j]));
            const uint32_t pair_slots = (uint32_t)(record_units(nnz, false) * 16 - DENSE_BYTES) / 8;
            for (uint32_t j = nnz + threadIdx.x; j < pair_slots; j += blockDim.x) sp[j] = make_uint2(EMPTY, 0u);
        }
    }
}

int launch_pack(apoe_ctx* ctx, uint32_t n, const float* dense, const uint32_t* s_off, const uint32_t* s_idx, const float* s_val,
                const uint32_t* b_off, const uint32_t* b_idx, const float* b_val, const uint64_t* desc, char* recs, float* dnorm,
                bool narrow) {
    uint32_t grid = n < 65536u * 16u ? n : 65536u * 16u;
    if (grid == 0) return APOE_OK;
    pack_kernel<<<grid, 256, 0, ctx->stream>>>(n, dense, s_off, s_idx, s_val, b_off, b_idx, b_val, desc, recs, dnorm, narrow ? 1u : 0u);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

// One workgroup (4 waves) per query and candidate chunk. The query's dense part is
// held in registers by every wave, its sparse terms sit in the LDS table; each wave
// takes every 4th candidate.
__global__ __launch_bounds__(256) void distance_batch_kernel(CorpusView C, SetView Q, float w_d, float w_s, float w_b, uint32_t paths,
                                                             const uint32_t* __restrict__ ids, uint32_t M, uint32_t chunk,
                                                             uint32_t slots, float* __restrict__ out) {
    extern __shared__ uint2 tab[];
    const uint32_t q = blockIdx.x, mask = slots - 1;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = lane_id();
    term_table_clear(tab, slots, tid, blockDim.x);
    PivotDense pv;
    pivot_dense_load(pv, Q.dense + (size_t)q * DIM, w_d);
    __syncthreads();
    pivot_terms_from_query(tab, mask, Q, q, w_s, w_b, paths & PATH_SPARSE, paths & PATH_BM25, tid, blockDim.x);
    __syncthreads();
    const uint32_t m0 = blockIdx.y * chunk, m1 = min(M, m0 + chunk);
    for (uint32_t m = m0 + wave; m < m1; m += blockDim.x / WAVE) {
        const uint32_t id = ids[(size_t)q * M + m];
        float dist = INF_DIS;
        if (id < C.n) {
            EvalOut e = eval_wave(C, id, pv, tab, mask, paths, 1.0f);
            dist = 1.0f - e.ip;
        }
        if (lane == 0) out[(size_t)q * M + m] = dist;
    }
}

static uint32_t path_mask(const float* w3) {
    uint32_t p = 0;
    if (!(w3[0] < 1e-5f)) p |= PATH_DENSE;
    if (!(w3[1] < 1e-5f)) p |= PATH_SPARSE;
    if (!(w3[2] < 1e-5f)) p |= PATH_BM25;
    return p;
}

int launch_distance_batch(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const float* w3, const uint32_t* ids_dev,
                          uint32_t M, float* out_dev) {
    if (q->n == 0 || M == 0) return APOE_OK;
    const uint32_t slots = next_pow2(std::max(64u, 2 * q->max_nnz));
    const size_t lds = (size_t)slots * sizeof(uint2);
    APOE_REQUIRE(lds <= 64 * 1024, "query rows with %u sparse terms exceed the LDS term table", q->max_nnz);
    const uint32_t chunk = 1024;
    dim3 grid(q->n, (M + chunk - 1) / chunk);
    distance_batch_kernel<<<grid, 256, lds, ctx->stream>>>(c->view(), q->view(), w3[0], w3[1], w3[2], path_mask(w3), ids_dev, M, chunk,
                                                           slots, out_dev);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

// One wave per pair: document a is the pivot, document b the candidate.
__global__ __launch_bounds__(64) void distance_pairs_kernel(CorpusView C, float dense_mul, const uint32_t* __restrict__ a,
                                                            const uint32_t* __restrict__ b, uint32_t n_pairs, uint32_t slots,
                                                            float* __restrict__ out) {
    extern __shared__ uint2 tab[];
    const uint32_t mask = slots - 1;
    const int lane = lane_id();
    for (uint32_t t = blockIdx.x; t < n_pairs; t += gridDim.x) {
        const uint32_t ia = a[t], ib = b[t];
        float dist = INF_DIS;
        if (ia < C.n && ib < C.n) {
            term_table_clear(tab, slots, lane, WAVE);
            __syncthreads();
            const uint64_t d = C.desc[ia];
            const char* rec = C.recs + desc_off(d) * 16;
            PivotDense pv;
            pivot_dense_load(pv, reinterpret_cast<const float*>(rec), 1.0f);
            pivot_terms_from_record(tab, mask, record_pairs(C, d), lane, WAVE);
            __syncthreads();
            EvalOut e = eval_wave(C, ib, pv, tab, mask, PATH_DENSE | PATH_SPARSE | PATH_BM25, dense_mul);
            dist = 1.0f - e.ip;
            __syncthreads();
        }
        if (lane == 0) out[t] = dist;
    }
}

int launch_distance_pairs(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, const uint32_t* a_dev, const uint32_t* b_dev,
                          uint32_t n_pairs, float* out_dev) {
    if (n_pairs == 0) return APOE_OK;
    const uint32_t slots = next_pow2(std::max(64u, 2 * (c->max_nnz_s + c->max_nnz_b)));
    const size_t lds = (size_t)slots * sizeof(uint2);
    APOE_REQUIRE(lds <= 64 * 1024, "document rows with %u sparse terms exceed the LDS term table", c->max_nnz_s + c->max_nnz_b);
    uint32_t grid = std::min<uint32_t>(n_pairs, 1u << 20);
    distance_pairs_kernel<<<grid, 64, lds, ctx->stream>>>(c->view(), dense_scale * dense_scale, a_dev, b_dev, n_pairs, slots, out_dev);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

// One wave per document: the dense row rounded to half precision (round to nearest even), 2 KB per row.
__global__ __launch_bounds__(256) void half_rows_kernel(CorpusView C, uint16_t* __restrict__ out) {
    const int lane = lane_id();
    const uint32_t waves = gridDim.x * (blockDim.x / WAVE);
    for (uint32_t doc = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE; doc < C.n; doc += waves) {
        const float4* r = reinterpret_cast<const float4*>(C.recs + desc_off(C.desc[doc]) * 16);
        uint2* o = reinterpret_cast<uint2*>(out + (size_t)doc * DIM);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const float4 x = r[lane + WAVE * i];
            const uint32_t a = __builtin_bit_cast(uint16_t, (_Float16)x.x), b = __builtin_bit_cast(uint16_t, (_Float16)x.y);
            const uint32_t c = __builtin_bit_cast(uint16_t, (_Float16)x.z), d = __builtin_bit_cast(uint16_t, (_Float16)x.w);
            o[lane + WAVE * i] = make_uint2(a | (b << 16), c | (d << 16));
        }
    }
}

int launch_half_rows(apoe_ctx* ctx, const apoe_corpus* c, uint16_t* out_dev) {
    if (c->n == 0) return APOE_OK;
    uint32_t grid = std::min<uint32_t>((c->n + 3) / 4, 1u << 16);
    half_rows_kernel<<<grid, 256, 0, ctx->stream>>>(c->view(), out_dev);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

// One wave per document: dense_mul*|dense|^2 + sum of squared pair values.
__global__ __launch_bounds__(256) void norms_kernel(CorpusView C, float dense_mul, float* __restrict__ out) {
    const int lane = lane_id();
    const uint32_t waves = gridDim.x * (blockDim.x / WAVE);
    for (uint32_t doc = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE; doc < C.n; doc += waves) {
        const uint64_t d = C.desc[doc];
        const char* rec = C.recs + desc_off(d) * 16;
        const float4* r = reinterpret_cast<const float4*>(rec);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NV; i++) {
            float4 x = r[lane + WAVE * i];
            acc += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
        }
        acc *= dense_mul;
        const Pairs sp = record_pairs(C, d);
        for (uint32_t j = lane; j < sp.nnz; j += WAVE) {
            float v = __uint_as_float(sp[j].y);
            acc = fmaf(v, v, acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) out[doc] = acc;
    }
}

int launch_norms(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, float* out_dev) {
    if (c->n == 0) return APOE_OK;
    uint32_t grid = std::min<uint32_t>((c->n + 3) / 4, 1u << 16);
    norms_kernel<<<grid, 256, 0, ctx->stream>>>(c->view(), dense_scale * dense_scale, out_dev);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

} // namespace apoe
