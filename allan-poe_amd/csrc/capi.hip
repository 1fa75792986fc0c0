// C-ABI entry points (include/apoe.h): handle life cycle, uploads, and thin
// wrappers that stage caller memory and call the kernel launchers.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <numeric>
#include <system_error>
#include <thread>

#include "apoe_internal.h"

namespace apoe {

static thread_local std::string g_error;

void set_error(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
}

static bool is_device_ptr(const void* p) {
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError(); // plain host memory is reported as an error
        return false;
    }
    return attr.type == hipMemoryTypeDevice;
}

// Device memory of one particular GPU.
static bool is_device_ptr_of(const void* p, int device) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return attr.type == hipMemoryTypeDevice && attr.device == device;
}

constexpr size_t STREAM_CHUNK = 32u << 20;     // bytes per pinned staging buffer
constexpr size_t STREAM_MIN = 4 * STREAM_CHUNK; // smaller uploads go through the plain copy

static int host_copy_threads() {
    const unsigned hw = std::thread::hardware_concurrency();
    return (int)std::min(8u, std::max(1u, hw / 2));
}

// Pageable host memory -> device through the two pinned buffers: while the copy engine moves chunk i out of one buffer,
// host threads fill the other with chunk i + 1 (the reference copies whole arrays with blocking cudaMemcpy from pageable
// memory, index.cu:842-877, query.cu:1901-1980).
static int stream_in(apoe_ctx* ctx, char* dst_dev, const char* src_host, size_t bytes) {
    for (int b = 0; b < 2; b++) {
        if (!ctx->pinned[b]) APOE_HIP(hipHostMalloc(&ctx->pinned[b], STREAM_CHUNK, hipHostMallocDefault));
        if (!ctx->pinned_done[b]) APOE_HIP(hipEventCreateWithFlags(&ctx->pinned_done[b], hipEventDisableTiming));
    }
    const int nt = host_copy_threads();
    bool used[2] = {false, false};
    size_t i = 0;
    for (size_t off = 0; off < bytes; off += STREAM_CHUNK, i++) {
        const int b = (int)(i & 1);
        const size_t len = std::min(STREAM_CHUNK, bytes - off);
        if (used[b]) APOE_HIP(hipEventSynchronize(ctx->pinned_done[b])); // the copy that last read this buffer has finished
        char* stage = static_cast<char*>(ctx->pinned[b]);
        if (nt == 1) {
            std::memcpy(stage, src_host + off, len);
        } else {
            std::thread workers[8];
            const size_t part = ((len + nt - 1) / nt + 4095) & ~(size_t)4095;
            int started = 0;
            for (int t = 0; t < nt; t++) {
                const size_t p0 = (size_t)t * part;
                if (p0 >= len) break;
                const size_t pl = std::min(part, len - p0);
                try {
                    workers[started] = std::thread([=]() { std::memcpy(stage + p0, src_host + off + p0, pl); });
                    started++;
                } catch (const std::system_error&) { // no thread to be had: this part is copied here
                    std::memcpy(stage + p0, src_host + off + p0, pl);
                }
            }
            for (int t = 0; t < started; t++) workers[t].join();
        }
        APOE_HIP(hipMemcpyAsync(dst_dev + off, stage, len, hipMemcpyHostToDevice, ctx->stream));
        APOE_HIP(hipEventRecord(ctx->pinned_done[b], ctx->stream));
        used[b] = true;
    }
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return APOE_OK;
}

int copy_in(apoe_ctx* ctx, void* dst_dev, const void* src_any, size_t bytes) {
    if (bytes == 0) return APOE_OK;
    if (bytes >= STREAM_MIN) {
        hipPointerAttribute_t attr;
        const hipError_t e = hipPointerGetAttributes(&attr, src_any);
        if (e != hipSuccess) (void)hipGetLastError(); // plain host memory is reported as an error
        const bool pageable = e != hipSuccess || attr.type == hipMemoryTypeUnregistered;
        if (pageable) return stream_in(ctx, static_cast<char*>(dst_dev), static_cast<const char*>(src_any), bytes);
    }
    APOE_HIP(hipMemcpyAsync(dst_dev, src_any, bytes, hipMemcpyDefault, ctx->stream));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return APOE_OK;
}

int copy_out(apoe_ctx* ctx, void* dst_any, const void* src_dev, size_t bytes) {
    if (bytes == 0) return APOE_OK;
    APOE_HIP(hipMemcpyAsync(dst_any, src_dev, bytes, hipMemcpyDefault, ctx->stream));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return APOE_OK;
}

// A caller array made readable by kernels: used in place when it already lives on
// the device, staged into a temporary device buffer otherwise.
template <typename T>
struct DevInput {
    DevBuf<T> staged;
    const T* p = nullptr;
    int init(apoe_ctx* ctx, const T* src, size_t count) {
        if (count == 0) { p = nullptr; return APOE_OK; }
        if (is_device_ptr(src)) { p = src; return APOE_OK; }
        APOE_TRY(staged.alloc(count));
        APOE_TRY(copy_in(ctx, staged.p, src, count * sizeof(T)));
        p = staged.p;
        return APOE_OK;
    }
};

// A caller output array: kernels write a device buffer, finish() copies it home.
template <typename T>
struct DevOutput {
    DevBuf<T> staged;
    T* p = nullptr;
    T* home = nullptr;
    size_t count = 0;
    int init(T* dst, size_t n) {
        count = n;
        home = dst;
        if (n == 0) return APOE_OK;
        if (is_device_ptr(dst)) { p = dst; return APOE_OK; }
        APOE_TRY(staged.alloc(n));
        p = staged.p;
        return APOE_OK;
    }
    int finish(apoe_ctx* ctx) {
        if (count && p != home) APOE_TRY(copy_out(ctx, home, p, count * sizeof(T)));
        return APOE_OK;
    }
};

static int check_csr(const std::vector<uint32_t>& off, const char* what) {
    for (size_t i = 1; i < off.size(); i++) APOE_REQUIRE(off[i] >= off[i - 1], "%s offsets decrease at row %zu", what, i - 1);
    return APOE_OK;
}

} // namespace apoe

using namespace apoe;

extern "C" {

const char* apoe_last_error_string(void) { return g_error.c_str(); }

int apoe_ctx_create(int device, apoe_ctx** out) {
    APOE_REQUIRE(out != nullptr, "out is null");
    *out = nullptr;
    int count = 0;
    APOE_HIP(hipGetDeviceCount(&count));
    APOE_REQUIRE(device >= 0 && device < count, "device %d not in [0,%d)", device, count);
    APOE_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    APOE_HIP(hipGetDeviceProperties(&prop, device));
    apoe_ctx* ctx = new apoe_ctx();
    ctx->device = device;
    ctx->num_cus = prop.multiProcessorCount;
    ctx->lds_per_block = prop.sharedMemPerBlock;
    if (search_static_workspace(device, &ctx->static_ws) != APOE_OK) {
        delete ctx;
        return APOE_ERR_HIP;
    }
    if (hipStreamCreate(&ctx->stream) != hipSuccess || hipEventCreate(&ctx->ev0) != hipSuccess || hipEventCreate(&ctx->ev1) != hipSuccess) {
        set_error("could not create the HIP stream/events: %s", hipGetErrorString(hipGetLastError()));
        apoe_ctx_destroy(ctx);
        return APOE_ERR_HIP;
    }
    *out = ctx;
    return APOE_OK;
}

void apoe_ctx_destroy(apoe_ctx* ctx) {
    if (!ctx) return;
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    for (int b = 0; b < 2; b++) {
        if (ctx->pinned_done[b]) (void)hipEventDestroy(ctx->pinned_done[b]);
        if (ctx->pinned[b]) (void)hipHostFree(ctx->pinned[b]);
    }
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

int apoe_ctx_synchronize(apoe_ctx* ctx) {
    APOE_REQUIRE(ctx != nullptr, "ctx is null");
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return APOE_OK;
}

int apoe_corpus_create(apoe_ctx* ctx, uint32_t n, uint32_t dim, const float* dense, const uint32_t* s_off, const uint32_t* s_idx,
                       const float* s_val, const uint32_t* b_off, const uint32_t* b_idx, const float* b_val, apoe_corpus** out) {
    APOE_REQUIRE(ctx && out, "ctx/out is null");
    *out = nullptr;
    APOE_REQUIRE(dim == DIM, "dim must be %d, got %u", DIM, dim);
    APOE_REQUIRE(n >= 1 && n < (1u << 30), "document count %u outside [1, 2^30)", n);
    APOE_REQUIRE(dense && s_off && b_off, "dense/s_off/b_off is null");
    APOE_HIP(hipSetDevice(ctx->device));
    std::vector<uint32_t> hs(n + 1), hb(n + 1);
    APOE_HIP(hipMemcpy(hs.data(), s_off, (n + 1) * sizeof(uint32_t), hipMemcpyDefault));
    APOE_HIP(hipMemcpy(hb.data(), b_off, (n + 1) * sizeof(uint32_t), hipMemcpyDefault));
    APOE_TRY(check_csr(hs, "sparse"));
    APOE_TRY(check_csr(hb, "bm25"));
    APOE_REQUIRE(hs[n] == 0 || (s_idx && s_val), "sparse idx/val is null");
    APOE_REQUIRE(hb[n] == 0 || (b_idx && b_val), "bm25 idx/val is null");
    std::unique_ptr<apoe_corpus> c(new apoe_corpus());
    c->ctx = ctx;
    c->n = n;
    c->dim = dim;
    for (uint32_t i = 0; i < n; i++) {
        const uint32_t ns = hs[i + 1] - hs[i], nb = hb[i + 1] - hb[i];
        APOE_REQUIRE(ns <= DESC_NNZ_MAX && nb <= DESC_NNZ_MAX, "row %u has %u/%u sparse/bm25 terms; at most %u each are supported", i, ns, nb,
                     DESC_NNZ_MAX);
        c->max_nnz_s = std::max(c->max_nnz_s, ns);
        c->max_nnz_b = std::max(c->max_nnz_b, nb);
    }
    {
        DevInput<float> d_dense, d_sval, d_bval;
        DevInput<uint32_t> d_soff, d_sidx, d_boff, d_bidx;
        APOE_TRY(d_sidx.init(ctx, s_idx, hs[n]));
        APOE_TRY(d_bidx.init(ctx, b_idx, hb[n]));
        // the pair format follows from the largest term id of either path
        DevBuf<uint32_t> d_max;
        uint32_t max_term = 0;
        APOE_TRY(d_max.alloc(1));
        APOE_TRY(copy_in(ctx, d_max.p, &max_term, sizeof(uint32_t)));
        APOE_TRY(launch_max_u32(ctx, d_sidx.p, hs[n], d_max.p));
        APOE_TRY(launch_max_u32(ctx, d_bidx.p, hb[n], d_max.p));
        APOE_TRY(copy_out(ctx, &max_term, d_max.p, sizeof(uint32_t)));
        // bit 31 is the path bit of a stored key, and a BM25 key of all ones would read as an empty table slot
        APOE_REQUIRE(max_term < BM25_BIT - 1, "term id %u does not fit 31 bits (the largest usable id is %u)", max_term, BM25_BIT - 2);
        c->narrow = max_term < 65536u;
        c->max_term = max_term;
        std::vector<uint64_t> desc(n);
        uint64_t off16 = 0;
        for (uint32_t i = 0; i < n; i++) {
            const uint32_t ns = hs[i + 1] - hs[i], nb = hb[i + 1] - hb[i];
            desc[i] = make_desc(off16, ns, nb);
            off16 += record_units(ns + nb, c->narrow);
        }
        APOE_REQUIRE(off16 < (1ull << DESC_OFF_BITS), "corpus of %llu bytes exceeds the record address range", (unsigned long long)off16 * 16);
        c->rec_bytes = off16 * 16;
        c->total_pairs = (uint64_t)hs[n] + hb[n];
        APOE_TRY(c->desc.alloc(n));
        APOE_TRY(c->recs.alloc(c->rec_bytes + ROW_LOAD_SLACK)); // unclamped row loads may read past the last record
        APOE_TRY(c->dnorm.alloc(n));
        APOE_TRY(copy_in(ctx, c->desc.p, desc.data(), n * sizeof(uint64_t)));
        APOE_TRY(d_dense.init(ctx, dense, (size_t)n * dim));
        APOE_TRY(d_soff.init(ctx, s_off, n + 1));
        APOE_TRY(d_sval.init(ctx, s_val, hs[n]));
        APOE_TRY(d_boff.init(ctx, b_off, n + 1));
        APOE_TRY(d_bval.init(ctx, b_val, hb[n]));
        APOE_TRY(launch_pack(ctx, n, d_dense.p, d_soff.p, d_sidx.p, d_sval.p, d_boff.p, d_bidx.p, d_bval.p, c->desc.p, c->recs.p, c->dnorm.p,
                             c->narrow));
        APOE_HIP(hipStreamSynchronize(ctx->stream));
    }
    *out = c.release();
    return APOE_OK;
}

int apoe_corpus_make_half_rows(apoe_ctx* ctx, apoe_corpus* c) {
    APOE_REQUIRE(ctx && c, "ctx/corpus is null");
    if (c->half.p) return APOE_OK;
    APOE_HIP(hipSetDevice(ctx->device));
    APOE_TRY(c->half.alloc((size_t)c->n * c->dim));
    APOE_TRY(launch_half_rows(ctx, c, c->half.p));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return APOE_OK;
}

void apoe_corpus_destroy(apoe_corpus* c) { delete c; }

int apoe_corpus_info(const apoe_corpus* c, uint32_t* info4) {
    APOE_REQUIRE(c && info4, "null argument");
    info4[0] = c->n;
    info4[1] = c->dim;
    info4[2] = c->max_nnz_s;
    info4[3] = c->max_nnz_b;
    return APOE_OK;
}

uint32_t apoe_corpus_pair_bytes(const apoe_corpus* c) { return c ? (c->narrow ? 6u : 8u) : 0u; }

uint64_t apoe_corpus_bytes(const apoe_corpus* c) { return c ? c->rec_bytes + (uint64_t)c->n * 12 + c->half.bytes() : 0; }

int apoe_queries_create(apoe_ctx* ctx, uint32_t n, uint32_t dim, const float* dense, const uint32_t* s_off, const uint32_t* s_idx,
                        const float* s_val, const uint32_t* b_off, const uint32_t* b_idx, const float* b_val, apoe_queries** out) {
    APOE_REQUIRE(ctx && out, "ctx/out is null");
    *out = nullptr;
    APOE_REQUIRE(dim == DIM, "dim must be %d, got %u", DIM, dim);
    APOE_REQUIRE(n >= 1, "no queries");
    APOE_REQUIRE(dense && s_off && b_off, "dense/s_off/b_off is null");
    APOE_HIP(hipSetDevice(ctx->device));
    std::unique_ptr<apoe_queries> q(new apoe_queries());
    q->ctx = ctx;
    q->n = n;
    q->dim = dim;
    q->h_s_off.resize(n + 1);
    q->h_b_off.resize(n + 1);
    APOE_HIP(hipMemcpy(q->h_s_off.data(), s_off, (n + 1) * sizeof(uint32_t), hipMemcpyDefault));
    APOE_HIP(hipMemcpy(q->h_b_off.data(), b_off, (n + 1) * sizeof(uint32_t), hipMemcpyDefault));
    APOE_TRY(check_csr(q->h_s_off, "query sparse"));
    APOE_TRY(check_csr(q->h_b_off, "query bm25"));
    const uint32_t nnz_s = q->h_s_off[n], nnz_b = q->h_b_off[n];
    APOE_REQUIRE(nnz_s == 0 || (s_idx && s_val), "sparse idx/val is null");
    APOE_REQUIRE(nnz_b == 0 || (b_idx && b_val), "bm25 idx/val is null");
    for (uint32_t i = 0; i < n; i++) {
        q->max_nnz = std::max(q->max_nnz, (q->h_s_off[i + 1] - q->h_s_off[i]) + (q->h_b_off[i + 1] - q->h_b_off[i]));
        q->max_nnz_s = std::max(q->max_nnz_s, q->h_s_off[i + 1] - q->h_s_off[i]);
        q->max_nnz_b = std::max(q->max_nnz_b, q->h_b_off[i + 1] - q->h_b_off[i]);
    }
    q->total_nnz_s = nnz_s;
    q->total_nnz_b = nnz_b;
    if (nnz_b) {
        std::vector<uint32_t> h_idx(nnz_b);
        APOE_HIP(hipMemcpy(h_idx.data(), b_idx, (size_t)nnz_b * sizeof(uint32_t), hipMemcpyDefault));
        for (uint32_t i = 0; i < n; i++) {
            uint32_t k = 0;
            for (uint32_t j = q->h_b_off[i]; j < q->h_b_off[i + 1]; j++) k += h_idx[j] >> 31;
            q->max_keywords = std::max(q->max_keywords, k);
        }
    }
    APOE_TRY(q->dense.alloc((size_t)n * dim));
    APOE_TRY(q->s_off.alloc(n + 1));
    APOE_TRY(q->b_off.alloc(n + 1));
    APOE_TRY(q->s_idx.alloc(nnz_s));
    APOE_TRY(q->s_val.alloc(nnz_s));
    APOE_TRY(q->b_idx.alloc(nnz_b));
    APOE_TRY(q->b_val.alloc(nnz_b));
    APOE_TRY(copy_in(ctx, q->dense.p, dense, (size_t)n * dim * sizeof(float)));
    APOE_TRY(copy_in(ctx, q->s_off.p, s_off, (n + 1) * sizeof(uint32_t)));
    APOE_TRY(copy_in(ctx, q->b_off.p, b_off, (n + 1) * sizeof(uint32_t)));
    APOE_TRY(copy_in(ctx, q->s_idx.p, s_idx, nnz_s * sizeof(uint32_t)));
    APOE_TRY(copy_in(ctx, q->s_val.p, s_val, nnz_s * sizeof(float)));
    APOE_TRY(copy_in(ctx, q->b_idx.p, b_idx, nnz_b * sizeof(uint32_t)));
    APOE_TRY(copy_in(ctx, q->b_val.p, b_val, nnz_b * sizeof(float)));
    if (nnz_s) { // bit 31 of a BM25 term id is the keyword flag; on a SPLADE term id it would send the term to the BM25 table
        DevBuf<uint32_t> d_max;
        uint32_t max_term = 0;
        APOE_TRY(d_max.alloc(1));
        APOE_TRY(copy_in(ctx, d_max.p, &max_term, sizeof(uint32_t)));
        APOE_TRY(launch_max_u32(ctx, q->s_idx.p, nnz_s, d_max.p));
        APOE_TRY(copy_out(ctx, &max_term, d_max.p, sizeof(uint32_t)));
        APOE_REQUIRE(max_term < BM25_BIT, "query sparse term id %u does not fit 31 bits", max_term);
    }
    *out = q.release();
    return APOE_OK;
}

void apoe_queries_destroy(apoe_queries* q) { delete q; }

int apoe_kg_create(apoe_ctx* ctx, uint32_t n_entities, const uint32_t* e2e_off, const uint32_t* e2e_idx, const uint32_t* e2d_off,
                   const uint32_t* e2d_idx, uint32_t n_queries, const uint32_t* q2e_off, const uint32_t* q2e_idx, apoe_kg** out) {
    APOE_REQUIRE(ctx && out, "ctx/out is null");
    *out = nullptr;
    APOE_REQUIRE(e2e_off && e2d_off && q2e_off, "offset array is null");
    APOE_HIP(hipSetDevice(ctx->device));
    std::unique_ptr<apoe_kg> kg(new apoe_kg());
    kg->ctx = ctx;
    kg->n_entities = n_entities;
    kg->n_queries = n_queries;
    auto upload = [&](DevBuf<uint32_t>& off_d, DevBuf<uint32_t>& idx_d, const uint32_t* off, const uint32_t* idx, uint32_t rows,
                      const char* what) -> int {
        std::vector<uint32_t> h(rows + 1);
        APOE_HIP(hipMemcpy(h.data(), off, (rows + 1) * sizeof(uint32_t), hipMemcpyDefault));
        APOE_TRY(check_csr(h, what));
        APOE_REQUIRE(h[rows] == 0 || idx, "%s idx is null", what);
        APOE_TRY(off_d.alloc(rows + 1));
        APOE_TRY(idx_d.alloc(h[rows]));
        APOE_TRY(copy_in(ctx, off_d.p, off, (rows + 1) * sizeof(uint32_t)));
        APOE_TRY(copy_in(ctx, idx_d.p, idx, (size_t)h[rows] * sizeof(uint32_t)));
        return APOE_OK;
    };
    APOE_TRY(upload(kg->e2e_off, kg->e2e_idx, e2e_off, e2e_idx, n_entities, "entity graph"));
    APOE_TRY(upload(kg->e2d_off, kg->e2d_idx, e2d_off, e2d_idx, n_entities, "entity2doc"));
    APOE_TRY(upload(kg->q2e_off, kg->q2e_idx, q2e_off, q2e_idx, n_queries, "query entities"));
    *out = kg.release();
    return APOE_OK;
}

void apoe_kg_destroy(apoe_kg* kg) { delete kg; }

int apoe_hybrid_distance_batch(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const float* w3, const uint32_t* ids,
                               uint32_t M, float* out) {
    APOE_REQUIRE(ctx && c && q && w3 && ids && out, "null argument");
    APOE_HIP(hipSetDevice(ctx->device));
    DevInput<uint32_t> d_ids;
    DevOutput<float> d_out;
    APOE_TRY(d_ids.init(ctx, ids, (size_t)q->n * M));
    APOE_TRY(d_out.init(out, (size_t)q->n * M));
    APOE_TRY(launch_distance_batch(ctx, c, q, w3, d_ids.p, M, d_out.p));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return d_out.finish(ctx);
}

int apoe_hybrid_distance_pairs(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, const uint32_t* a, const uint32_t* b,
                               uint32_t n_pairs, float* out) {
    APOE_REQUIRE(ctx && c && a && b && out, "null argument");
    APOE_HIP(hipSetDevice(ctx->device));
    DevInput<uint32_t> d_a, d_b;
    DevOutput<float> d_out;
    APOE_TRY(d_a.init(ctx, a, n_pairs));
    APOE_TRY(d_b.init(ctx, b, n_pairs));
    APOE_TRY(d_out.init(out, n_pairs));
    APOE_TRY(launch_distance_pairs(ctx, c, dense_scale, d_a.p, d_b.p, n_pairs, d_out.p));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return d_out.finish(ctx);
}

int apoe_norms(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, float* out) {
    APOE_REQUIRE(ctx && c && out, "null argument");
    APOE_HIP(hipSetDevice(ctx->device));
    DevOutput<float> d_out;
    APOE_TRY(d_out.init(out, c->n));
    APOE_TRY(launch_norms(ctx, c, dense_scale, d_out.p));
    APOE_HIP(hipStreamSynchronize(ctx->stream));
    return d_out.finish(ctx);
}

int apoe_calibrate_weights(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, uint32_t n_queries, float* w3) {
    APOE_REQUIRE(ctx && c && q && w3, "null argument");
    APOE_HIP(hipSetDevice(ctx->device));
    const uint32_t nd = std::min<uint32_t>(c->n, 100), nq = std::min<uint32_t>(std::min(n_queries, q->n), 100);
    if (nd == 0 || nq == 0) return APOE_OK;
    // per-path inner products of the first nd documents with the first nq queries
    std::vector<uint32_t> ids((size_t)q->n * nd);
    for (uint32_t i = 0; i < q->n; i++)
        for (uint32_t j = 0; j < nd; j++) ids[(size_t)i * nd + j] = i < nq ? j : 0xFFFFFFFFu;
    DevBuf<uint32_t> d_ids;
    DevBuf<float> d_out;
    APOE_TRY(d_ids.alloc(ids.size()));
    APOE_TRY(d_out.alloc(ids.size()));
    APOE_TRY(copy_in(ctx, d_ids.p, ids.data(), ids.size() * sizeof(uint32_t)));
    std::vector<float> out(ids.size());
    float mx[3];
    for (int p = 0; p < 3; p++) {
        const float w[3] = {p == 0 ? 1.f : 0.f, p == 1 ? 1.f : 0.f, p == 2 ? 1.f : 0.f};
        APOE_TRY(launch_distance_batch(ctx, c, q, w, d_ids.p, nd, d_out.p));
        APOE_TRY(copy_out(ctx, out.data(), d_out.p, out.size() * sizeof(float)));
        float m = -INFINITY;
        for (uint32_t i = 0; i < nq; i++)
            for (uint32_t j = 0; j < nd; j++) m = std::max(m, 1.0f - out[(size_t)i * nd + j]);
        mx[p] = m;
    }
    // query.cu:1858-1869: the path with the strictly largest maximum is the yardstick
    int big = -1;
    if (mx[1] > mx[2] && mx[1] > mx[0]) big = 1;
    else if (mx[2] > mx[1] && mx[2] > mx[0]) big = 2;
    else if (mx[0] > mx[1] && mx[0] > mx[2]) big = 0;
    if (big < 0) return APOE_OK;
    for (int p = 0; p < 3; p++)
        if (p != big && mx[p] > 0.f) w3[p] *= mx[big] / mx[p];
    return APOE_OK;
}

int apoe_graph_create(apoe_ctx* ctx, uint32_t n, uint32_t width, const uint32_t* rows, const uint32_t* entry, uint32_t n_entry,
                      apoe_graph** out) {
    APOE_REQUIRE(ctx && out && rows && (entry || n_entry == 0), "null argument");
    *out = nullptr;
    APOE_REQUIRE(width > APOE_KW_SLOTS, "graph width %u must exceed the %d keyword slots", width, APOE_KW_SLOTS);
    APOE_HIP(hipSetDevice(ctx->device));
    std::unique_ptr<apoe_graph> g(new apoe_graph());
    g->ctx = ctx;
    g->n = n;
    g->width = width;
    g->n_entry = n_entry;
    APOE_TRY(g->rows.alloc((size_t)n * width));
    APOE_TRY(g->entry.alloc(n_entry));
    APOE_TRY(copy_in(ctx, g->rows.p, rows, (size_t)n * width * sizeof(uint32_t)));
    APOE_TRY(copy_in(ctx, g->entry.p, entry, (size_t)n_entry * sizeof(uint32_t)));
    *out = g.release();
    return APOE_OK;
}

void apoe_graph_destroy(apoe_graph* g) { delete g; }

int apoe_graph_info(const apoe_graph* g, uint32_t* info3) {
    APOE_REQUIRE(g && info3, "null argument");
    info3[0] = g->n;
    info3[1] = g->width;
    info3[2] = g->n_entry;
    return APOE_OK;
}

int apoe_graph_download(const apoe_graph* g, uint32_t* rows, uint32_t* entry) {
    APOE_REQUIRE(g, "null argument");
    APOE_HIP(hipSetDevice(g->ctx->device));
    if (rows) APOE_TRY(copy_out(g->ctx, rows, g->rows.p, (size_t)g->n * g->width * sizeof(uint32_t)));
    if (entry) APOE_TRY(copy_out(g->ctx, entry, g->entry.p, (size_t)g->n_entry * sizeof(uint32_t)));
    return APOE_OK;
}

int apoe_search(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const apoe_graph* g, const apoe_kg* kg,
                const apoe_search_params* p, uint32_t* out_ids, float* out_dist, apoe_search_stats* stats) {
    APOE_REQUIRE(ctx && c && q && g && p && out_ids && out_dist, "null argument");
    APOE_HIP(hipSetDevice(ctx->device));
    APOE_REQUIRE(p->q_begin <= q->n, "q_begin %u beyond %u queries", p->q_begin, q->n);
    const uint32_t q_count = p->q_count ? p->q_count : q->n - p->q_begin;
    // before anything is sized from them
    APOE_REQUIRE(q_count <= q->n - p->q_begin, "query range of %u from %u beyond %u queries", q_count, p->q_begin, q->n);
    APOE_REQUIRE(p->cands >= 1 && p->cands <= APOE_MAX_CANDS, "cands must be in 1..%d, got %u", APOE_MAX_CANDS, p->cands);
    DevOutput<uint32_t> d_ids;
    DevOutput<float> d_dist;
    APOE_TRY(d_ids.init(out_ids, (size_t)q_count * p->cands));
    APOE_TRY(d_dist.init(out_dist, (size_t)q_count * p->cands));
    APOE_TRY(launch_search(ctx, c, q, g, kg, p, d_ids.p, d_dist.p, stats, nullptr));
    APOE_TRY(d_ids.finish(ctx));
    return d_dist.finish(ctx);
}

int apoe_search_noalloc(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const apoe_graph* g, const apoe_kg* kg,
                        const apoe_search_params* p, uint32_t* out_ids, float* out_dist, apoe_search_stats* stats) {
    APOE_REQUIRE(ctx && c && q && g && p && out_ids && out_dist, "null argument");
    APOE_HIP(hipSetDevice(ctx->device));
    APOE_REQUIRE(c->n <= APOE_NOALLOC_MAX_DOCS, "apoe_search_noalloc serves corpora of up to %u documents, this one has %u", (unsigned)APOE_NOALLOC_MAX_DOCS,
                 c->n);
    APOE_REQUIRE(is_device_ptr_of(out_ids, ctx->device) && is_device_ptr_of(out_dist, ctx->device),
                 "apoe_search_noalloc writes its results in place: out_ids and out_dist must be device memory of GPU %d, the context's", ctx->device);
    return launch_search(ctx, c, q, g, kg, p, out_ids, out_dist, stats, ctx->static_ws);
}

} // extern "C"
