// Host-side handle definitions and helpers behind the C-ABI of include/apoe.h.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <string>
#include <vector>

#include "../../include/apoe.h"
#include "apoe_device.h"

namespace apoe {

void set_error(const char* fmt, ...);

#define APOE_HIP(call)                                                                              \
    do {                                                                                            \
        hipError_t e_ = (call);                                                                     \
        if (e_ != hipSuccess) {                                                                     \
            apoe::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            return APOE_ERR_HIP;                                                                    \
        }                                                                                           \
    } while (0)

#define APOE_REQUIRE(cond, ...)              \
    do {                                     \
        if (!(cond)) {                       \
            apoe::set_error(__VA_ARGS__);    \
            return APOE_ERR_ARG;             \
        }                                    \
    } while (0)

#define APOE_REQUIRE_STATE(cond, ...)        \
    do {                                     \
        if (!(cond)) {                       \
            apoe::set_error(__VA_ARGS__);    \
            return APOE_ERR_STATE;           \
        }                                    \
    } while (0)

#define APOE_TRY(expr)              \
    do {                            \
        int s_ = (expr);            \
        if (s_ != APOE_OK) return s_; \
    } while (0)

// Device buffer owned by a handle.
template <typename T>
struct DevBuf {
    T* p = nullptr;
    size_t n = 0;
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    ~DevBuf() { release(); }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        n = 0;
    }
    int alloc(size_t count) {
        release();
        if (count == 0) count = 1;
        APOE_HIP(hipMalloc((void**)&p, count * sizeof(T)));
        n = count;
        return APOE_OK;
    }
    size_t bytes() const { return n * sizeof(T); }
};

inline uint32_t next_pow2(uint32_t v) {
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

} // namespace apoe

struct apoe_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    int num_cus = 0;
    size_t lds_per_block = 0;
    // Search workspace (visited bitmaps, counters, once-per-query arguments): grows to the largest
    // request and is kept until the context is destroyed, so that repeated searches do not pay for
    // a device allocation each. One search at a time per context.
    apoe::DevBuf<char> search_ws;
    char* static_ws = nullptr; // this GPU's copy of the static workspace of apoe_search_noalloc
    // Upload pipeline for large pageable host arrays: two pinned staging buffers that host threads fill while the
    // copy engine drains the other one (created on first use, kept until the context is destroyed).
    void* pinned[2] = {nullptr, nullptr};
    hipEvent_t pinned_done[2] = {nullptr, nullptr};
    int search_workspace(size_t bytes, char** out) {
        if (search_ws.n < bytes) APOE_TRY(search_ws.alloc(bytes));
        *out = search_ws.p;
        return APOE_OK;
    }
};

struct apoe_corpus {
    apoe_ctx* ctx = nullptr;
    uint32_t n = 0, dim = 0, max_nnz_s = 0, max_nnz_b = 0;
    uint32_t max_term = 0; // largest term id of either path
    uint64_t rec_bytes = 0, total_pairs = 0;
    bool narrow = false; // pair format of the records (6 instead of 8 bytes a pair when every term id is below 65536)
    apoe::DevBuf<uint64_t> desc;
    apoe::DevBuf<char> recs;
    apoe::DevBuf<float> dnorm;
    apoe::DevBuf<uint16_t> half; // optional half-precision copy of the dense rows, [n][dim] (apoe_corpus_make_half_rows)
    apoe::CorpusView view() const { return apoe::CorpusView{desc.p, recs.p, dnorm.p, n, narrow ? 1u : 0u}; }
};

struct apoe_queries {
    apoe_ctx* ctx = nullptr;
    uint32_t n = 0, dim = 0, max_nnz = 0; // max over queries of nnz_s + nnz_b
    uint32_t max_nnz_s = 0, max_nnz_b = 0; // ... and of either alone
    uint32_t max_keywords = 0;            // max over queries of BM25 terms flagged as required keyword (bit 31)
    uint64_t total_nnz_s = 0, total_nnz_b = 0;
    std::vector<uint32_t> h_s_off, h_b_off;
    apoe::DevBuf<float> dense, s_val, b_val;
    apoe::DevBuf<uint32_t> s_off, s_idx, b_off, b_idx;
    apoe::SetView view() const { return apoe::SetView{dense.p, s_off.p, s_idx.p, s_val.p, b_off.p, b_idx.p, b_val.p, n}; }
};

struct apoe_kg {
    apoe_ctx* ctx = nullptr;
    uint32_t n_entities = 0, n_queries = 0;
    apoe::DevBuf<uint32_t> e2e_off, e2e_idx, e2d_off, e2d_idx, q2e_off, q2e_idx;
};

struct apoe_graph {
    apoe_ctx* ctx = nullptr;
    uint32_t n = 0, width = 0, n_entry = 0;
    apoe::DevBuf<uint32_t> rows, entry;
};

struct apoe_knn {
    apoe_ctx* ctx = nullptr;
    const apoe_corpus* corpus = nullptr;
    uint32_t n = 0, K = 0, degree = 0;
    float dense_scale = 1.f;
    float elapsed_ms = 0.f;
    bool ready = false;  // lists hold something: apoe_nnd_init or apoe_knn_upload has run
    bool pruned = false;
    bool force_sequential_prune = false; // K = 64 handles use the gather-once prune unless this is set
    bool half_rows = false;              // NN-Descent steps take dense parts from the corpus' half-precision rows
    apoe::DevBuf<uint32_t> ids, rev_cnt;
    apoe::DevBuf<unsigned long long> rev; // [n][K] reverse lists: (distance key << 32 | id) per slot
    apoe::DevBuf<float> dist, norms;
    apoe::DevBuf<unsigned long long> counter;
    // local-join step (apoe_knn_set_join): the picks of a step grouped by the picked node, the tiles, the proposal rows
    int join = 0; // 0: expansion step, 1: local join, 2: local join that offers a pair to both endpoints
    bool join_symmetric = false;
    apoe::DevBuf<uint32_t> picks, pick_cnt, pick_off, pick_fill, pick_src, tile_cnt, tile_off, tile_v;
    apoe::DevBuf<unsigned long long> prop, join_work;
    apoe::DevBuf<char> scan_tmp;
    // prune outputs
    apoe::DevBuf<uint32_t> fwd, det, cnt, kw;
};

namespace apoe {

// Copies between caller memory (host or device) and library device memory.
int copy_in(apoe_ctx* ctx, void* dst_dev, const void* src_any, size_t bytes);
int copy_out(apoe_ctx* ctx, void* dst_any, const void* src_dev, size_t bytes);

// Kernel launchers (one per .hip file).
int launch_pack(apoe_ctx* ctx, uint32_t n, const float* dense, const uint32_t* s_off, const uint32_t* s_idx, const float* s_val,
                const uint32_t* b_off, const uint32_t* b_idx, const float* b_val, const uint64_t* desc, char* recs, float* dnorm,
                bool narrow);
int launch_max_u32(apoe_ctx* ctx, const uint32_t* a_dev, size_t n, uint32_t* out_dev);
int launch_half_rows(apoe_ctx* ctx, const apoe_corpus* c, uint16_t* out_dev);
int launch_distance_batch(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const float* w3, const uint32_t* ids_dev,
                          uint32_t M, float* out_dev);
int launch_distance_pairs(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, const uint32_t* a_dev, const uint32_t* b_dev,
                          uint32_t n_pairs, float* out_dev);
int launch_norms(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, float* out_dev);
int launch_search(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const apoe_graph* g, const apoe_kg* kg,
                  const apoe_search_params* p, uint32_t* out_ids_dev, float* out_dist_dev, apoe_search_stats* stats, char* static_ws);
int search_static_workspace(int device, char** out); // device address of the static search workspace on that GPU
int launch_nnd_init(apoe_knn* g, uint64_t seed);
int launch_nnd_iterate(apoe_knn* g, uint64_t* inserted);
int launch_nnd_join_iterate(apoe_knn* g);
int join_step_counters(apoe_knn* g, unsigned long long* out3);
int launch_gram_tiles(apoe_knn* g, uint32_t node0, uint32_t n_nodes, float* gram, unsigned long long* unfit);
bool gram_tiles_fit(const apoe_knn* g);
int launch_nnd_merge_reverse(apoe_knn* g);
int launch_prune(apoe_knn* g, uint32_t degree);
int launch_final_graph(apoe_knn* g, uint32_t* rows_dev);

// Times `fn` (which enqueues work on ctx->stream) with HIP events; blocks until done.
template <typename F>
int timed(apoe_ctx* ctx, float* ms, F&& fn) {
    APOE_HIP(hipEventRecord(ctx->ev0, ctx->stream));
    APOE_TRY(fn());
    APOE_HIP(hipEventRecord(ctx->ev1, ctx->stream));
    APOE_HIP(hipEventSynchronize(ctx->ev1));
    float t = 0.f;
    APOE_HIP(hipEventElapsedTime(&t, ctx->ev0, ctx->ev1));
    if (ms) *ms = t;
    return APOE_OK;
}

} // namespace apoe
