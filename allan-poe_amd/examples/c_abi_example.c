/*
 * The hot path through the bare C-ABI (include/apoe.h), as a cgo / JNI / FFI binding would drive it: upload a small
 * hybrid corpus, build the index (random lists, NN-Descent steps, reverse merge, RNG-IP prune, final rows), search a
 * batch of queries, print the first ids of every row. Stands where build_index_impl and search_index_impl call their
 * kernels (index.cu:889-925, query.cu:1999-2075).
 *
 *   gcc -std=c99 -O2 -I include allan-poe_amd/examples/c_abi_example.c -L allan-poe_amd -lapoe -Wl,-rpath,$PWD/allan-poe_amd -lm -o c_abi_example
 *   ./c_abi_example [n_docs] [n_queries] [cands]
 *
 * Output: one line per query, "q <index>: <id> <id> <id> <id> <id> | <distance of the first>".
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "apoe.h"

#define DIM 1024
#define CHECK(call)                                                                      \
    do {                                                                                 \
        if ((call) != APOE_OK) {                                                         \
            fprintf(stderr, "%s failed: %s\n", #call, apoe_last_error_string());         \
            return 1;                                                                    \
        }                                                                                \
    } while (0)

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint64_t rnd(void) { /* splitmix64 */
    uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static float unit(void) { return (float)((rnd() >> 40) + 0.5) / 16777216.0f; }

#define CLUSTERS 64
#define W_DENSE 49.0f /* the weights of the search are those of the build metric (dense rows scaled by 7, index.cu:836-840) */
static float centre[CLUSTERS][DIM];

/* n rows around CLUSTERS topics: a unit dense vector near the topic's centre, `per_row` distinct ascending term ids (values in
 * (0.5, 1.5)), two thirds of them from the topic's own block of the vocabulary: rows of one topic are each other's neighbours */
static void make_set(uint32_t n, uint32_t per_row, uint32_t vocab, float* dense, uint32_t* off, uint32_t* idx, float* val) {
    const uint32_t stride = vocab / per_row, block = stride / CLUSTERS;
    for (uint32_t i = 0; i < n; i++) {
        const uint32_t c = (uint32_t)(rnd() % CLUSTERS);
        double norm = 0.0;
        for (int d = 0; d < DIM; d++) {
            const float g = centre[c][d] + 0.4f * sqrtf(-2.0f * logf(unit())) * cosf(6.2831853f * unit());
            dense[(size_t)i * DIM + d] = g;
            norm += (double)g * g;
        }
        for (int d = 0; d < DIM; d++) dense[(size_t)i * DIM + d] /= (float)sqrt(norm);
        off[i] = i * per_row;
        for (uint32_t t = 0; t < per_row; t++) { /* one term per stride: ascending, no repeats */
            const uint32_t in_stride = t % 3 ? c * block + (uint32_t)(rnd() % block) : (uint32_t)(rnd() % stride);
            idx[(size_t)i * per_row + t] = t * stride + in_stride;
            val[(size_t)i * per_row + t] = 0.5f + unit();
        }
    }
    off[n] = n * per_row;
}

/* 1 - (W_DENSE * dense + splade + bm25 inner products) of query q and document v on the host */
static float host_distance(const float* qd, const uint32_t* qo, const uint32_t* qi, const float* qv, const uint32_t* qbo, const uint32_t* qbi,
                           const float* qbv, uint32_t q, const float* dd, const uint32_t* so, const uint32_t* si, const float* sv,
                           const uint32_t* bo, const uint32_t* bi, const float* bv, uint32_t v) {
    double ip = 0.0;
    for (int d = 0; d < DIM; d++) ip += W_DENSE * (double)qd[(size_t)q * DIM + d] * dd[(size_t)v * DIM + d];
    for (uint32_t a = qo[q], b = so[v]; a < qo[q + 1] && b < so[v + 1];) {
        if (qi[a] == si[b]) ip += (double)qv[a++] * sv[b++];
        else if (qi[a] < si[b]) a++;
        else b++;
    }
    for (uint32_t a = qbo[q], b = bo[v]; a < qbo[q + 1] && b < bo[v + 1];) {
        if (qbi[a] == bi[b]) ip += (double)qbv[a++] * bv[b++];
        else if (qbi[a] < bi[b]) a++;
        else b++;
    }
    return (float)(1.0 - ip);
}

int main(int argc, char** argv) {
    const uint32_t n = argc > 1 ? (uint32_t)atoi(argv[1]) : 3000, nq = argc > 2 ? (uint32_t)atoi(argv[2]) : 8;
    const uint32_t cands = argc > 3 ? (uint32_t)atoi(argv[3]) : 64, degree = 32, steps = 8;
    const uint32_t ns = 40, nb = 20, qs = 12, qb = 6, vocab = 30000;

    float* dense = malloc((size_t)n * DIM * sizeof(float));
    uint32_t *s_off = malloc((n + 1) * 4), *s_idx = malloc((size_t)n * ns * 4), *b_off = malloc((n + 1) * 4), *b_idx = malloc((size_t)n * nb * 4);
    float *s_val = malloc((size_t)n * ns * 4), *b_val = malloc((size_t)n * nb * 4);
    float* qdense = malloc((size_t)nq * DIM * sizeof(float));
    uint32_t *qs_off = malloc((nq + 1) * 4), *qs_idx = malloc((size_t)nq * qs * 4), *qb_off = malloc((nq + 1) * 4), *qb_idx = malloc((size_t)nq * qb * 4);
    float *qs_val = malloc((size_t)nq * qs * 4), *qb_val = malloc((size_t)nq * qb * 4);
    if (!dense || !s_off || !s_idx || !b_off || !b_idx || !s_val || !b_val || !qdense || !qs_off || !qs_idx || !qb_off || !qb_idx || !qs_val || !qb_val) return 2;
    for (int c = 0; c < CLUSTERS; c++)
        for (int d = 0; d < DIM; d++) centre[c][d] = sqrtf(-2.0f * logf(unit())) * cosf(6.2831853f * unit());
    const uint64_t corpus_seed = rng_state;
    make_set(n, ns, vocab, dense, s_off, s_idx, s_val);
    { /* BM25 side of the corpus: its own draw, dense rows kept */
        float* scratch = malloc((size_t)n * DIM * sizeof(float));
        if (!scratch) return 2;
        rng_state = corpus_seed; /* the same topics, row by row, as the SPLADE side */
        make_set(n, nb, vocab, scratch, b_off, b_idx, b_val);
        free(scratch);
    }
    const uint64_t query_seed = rng_state;
    make_set(nq, qs, vocab, qdense, qs_off, qs_idx, qs_val);
    {
        float* scratch = malloc((size_t)nq * DIM * sizeof(float));
        if (!scratch) return 2;
        rng_state = query_seed;
        make_set(nq, qb, vocab, scratch, qb_off, qb_idx, qb_val);
        free(scratch);
    }

    apoe_ctx* ctx = NULL;
    apoe_corpus* corpus = NULL;
    apoe_queries* queries = NULL;
    apoe_knn* knn = NULL;
    apoe_graph* graph = NULL;
    CHECK(apoe_ctx_create(0, &ctx));
    CHECK(apoe_corpus_create(ctx, n, DIM, dense, s_off, s_idx, s_val, b_off, b_idx, b_val, &corpus));
    CHECK(apoe_queries_create(ctx, nq, DIM, qdense, qs_off, qs_idx, qs_val, qb_off, qb_idx, qb_val, &queries));

    /* build: index.cu:889-925 */
    CHECK(apoe_knn_create(ctx, corpus, 64, 7.0f, &knn));
    CHECK(apoe_knn_set_join(knn, 1));
    CHECK(apoe_nnd_init(knn, 20251125));
    for (uint32_t it = 0; it < steps; it++) {
        uint64_t inserted = 0;
        CHECK(apoe_nnd_iterate(knn, it + 1 == steps, &inserted));
        fprintf(stderr, "step %u: %llu list entries inserted\n", it, (unsigned long long)inserted);
    }
    CHECK(apoe_nnd_merge_reverse(knn));
    CHECK(apoe_prune(knn, degree));
    CHECK(apoe_finalize_graph(knn, &graph));
    const float build_ms = apoe_knn_elapsed_ms(knn);
    fprintf(stderr, "index of %u documents, degree %u: %.2f ms of GPU time\n", n, degree, build_ms);

    /* search: query.cu:1999-2075 */
    apoe_search_params p = {W_DENSE, 1.0f, 1.0f, 0.0f, 0, 0, 0, 0, 0, 0};
    p.cands = cands;
    uint32_t* ids = malloc((size_t)nq * cands * 4);
    float* dist = malloc((size_t)nq * cands * 4);
    if (!ids || !dist) return 2;
    apoe_search_stats st;
    CHECK(apoe_search(ctx, corpus, queries, graph, NULL, &p, ids, dist, &st));
    fprintf(stderr, "%u queries, pool %u: %.3f ms, %llu evaluations\n", nq, cands, st.kernel_ms, (unsigned long long)st.evaluations);
    for (uint32_t q = 0; q < nq; q++) {
        printf("q %u:", q);
        for (uint32_t k = 0; k < 5 && k < cands; k++) printf(" %u", ids[(size_t)q * cands + k]);
        printf(" | %.5f\n", dist[(size_t)q * cands]);
    }

    /* the closest document by brute force on the host must be in the pool, and the reported distance must be the metric */
    uint32_t found = 0, exact = 0;
    for (uint32_t q = 0; q < nq; q++) {
        uint32_t best = 0;
        float best_d = 1e30f;
        for (uint32_t v = 0; v < n; v++) {
            const float d = host_distance(qdense, qs_off, qs_idx, qs_val, qb_off, qb_idx, qb_val, q, dense, s_off, s_idx, s_val, b_off, b_idx, b_val, v);
            if (d < best_d) { best_d = d; best = v; }
        }
        for (uint32_t k = 0; k < cands; k++) found += ids[(size_t)q * cands + k] == best;
        const uint32_t top = ids[(size_t)q * cands];
        const float again = host_distance(qdense, qs_off, qs_idx, qs_val, qb_off, qb_idx, qb_val, q, dense, s_off, s_idx, s_val, b_off, b_idx, b_val, top);
        exact += fabsf(again - dist[(size_t)q * cands]) <= 1e-4f * fmaxf(1.0f, fabsf(again));
    }
    printf("brute-force best document in the pool for %u of %u queries; reported distance equals the metric for %u of %u\n", found, nq, exact, nq);

    apoe_graph_destroy(graph);
    apoe_knn_destroy(knn);
    apoe_queries_destroy(queries);
    apoe_corpus_destroy(corpus);
    apoe_ctx_destroy(ctx);
    return 0;
}
