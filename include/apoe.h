/*
 * apoe.h -- C-ABI of the MI355X (gfx950) implementation of the Allan-Poe hybrid
 * graph index hot path: fused hybrid distance, NN-Descent, RNG-IP pruning with
 * keyword recycling, final graph assembly, and greedy beam search with optional
 * knowledge-graph expansion.
 *
 * Conventions
 *  - Every function returns APOE_OK (0) or a negative status; the message of the
 *    last failure on the calling thread is apoe_last_error_string(). Nothing here
 *    throws or exits (the reference calls exit() on any failure, index.cu:19-28).
 *  - Bulk input/output pointers may point to host memory or to device memory of
 *    the context's GPU; the library copies with hipMemcpyDefault. The caller owns
 *    them; the library owns everything it allocates on the device.
 *  - All work of a context runs on the context's own HIP stream. A context and
 *    its handles may be used from one thread at a time. There is no global state.
 *  - Sparse matrices are CSR in the reference's file layout: off[rows+1], idx[nnz]
 *    ascending inside a row, val[nnz] (utils.cuh:380-398). Term ids must be < 2^31 - 1 (corpus) and < 2^31 (queries).
 *  - Document ids must be < 2^30 (bits 30/31 are flags inside pools, query.cu:503).
 *  - dim must be 1024 (utils.cuh:31 DIM).
 */
#ifndef APOE_H
#define APOE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define APOE_OK 0
#define APOE_ERR_ARG -1      /* bad argument / unsupported size */
#define APOE_ERR_HIP -2      /* a HIP runtime call failed */
#define APOE_ERR_STATE -3    /* call sequence error (e.g. finalize before prune) */

#define APOE_INF_DIS 1000000.0f /* index.cu:8, query.cu:11 */
#define APOE_KW_SLOTS 8         /* index.cu:15 KEYEDGEFINAL: row width = degree + 8 */
#define APOE_KW_CAND 32         /* index.cu:14 KEYEDGE */
#define APOE_MAX_CANDS 2048     /* pool size limit (the reference stops at 512, query.cu:9) */
#define APOE_JOIN_MAX_ROW_TERMS 2304 /* sparse terms of one document (both paths) that the local-join step's LDS table holds */

typedef struct apoe_ctx apoe_ctx;
typedef struct apoe_corpus apoe_corpus;
typedef struct apoe_queries apoe_queries;
typedef struct apoe_kg apoe_kg;
typedef struct apoe_graph apoe_graph;
typedef struct apoe_knn apoe_knn;

const char* apoe_last_error_string(void);

/* Replaces the implicit "device 0, default stream" of the reference. */
int apoe_ctx_create(int device, apoe_ctx** out);
void apoe_ctx_destroy(apoe_ctx* ctx);
int apoe_ctx_synchronize(apoe_ctx* ctx);

/*
 * Corpus upload. Replaces the cudaMalloc/cudaMemcpy block of build_index_impl
 * (index.cu:842-872) and search_index_impl (query.cu:1909-1934). The rows are
 * repacked on the device into one record per document (dense row followed by the
 * SPLADE and BM25 (id, value) pairs) so that one evaluation is one contiguous read.
 * Term ids must be below 2^31 - 1.
 */
int apoe_corpus_create(apoe_ctx* ctx, uint32_t n, uint32_t dim, const float* dense,
                       const uint32_t* s_off, const uint32_t* s_idx, const float* s_val,
                       const uint32_t* b_off, const uint32_t* b_idx, const float* b_val,
                       apoe_corpus** out);
/* Optional second copy of the dense rows in half precision (IEEE binary16, round to nearest even; 2 KB per
 * row beside the 4 KB fp32 row, which stays). The reference keeps ONLY such a copy and multiplies and adds in
 * half precision (f2h, utils.cuh:78-83; query.cu:459-465); here it is an option for callers that trade
 * exactness during the graph walk for bytes: apoe_search with variant | 0x200 takes the dense part of a
 * candidate from this copy (fp32 products and sums) and re-evaluates the final pool with the fp32 rows.
 * Idempotent. */
int apoe_corpus_make_half_rows(apoe_ctx* ctx, apoe_corpus* c);
void apoe_corpus_destroy(apoe_corpus* c);
/* info4 = {n, dim, max splade nnz per row, max bm25 nnz per row} (index.cu:829-835). */
int apoe_corpus_info(const apoe_corpus* c, uint32_t* info4);
/* Bytes of the device records: the HBM footprint one full scan reads. */
uint64_t apoe_corpus_bytes(const apoe_corpus* c);
/* Bytes one (term, value) pair takes in the device records: 6 when every term id of the corpus
 * (both paths) is below 65536 (values as f32, ids as u16, the path known from the position),
 * else 8. Chosen by apoe_corpus_create from the data; results do not depend on it. */
uint32_t apoe_corpus_pair_bytes(const apoe_corpus* c);

/* Query upload (query.cu:1936-1961). Weights are NOT folded in here; they are
 * applied when a search or distance call loads the query (query.cu:1871-1881). */
int apoe_queries_create(apoe_ctx* ctx, uint32_t n, uint32_t dim, const float* dense,
                        const uint32_t* s_off, const uint32_t* s_idx, const float* s_val,
                        const uint32_t* b_off, const uint32_t* b_idx, const float* b_val,
                        apoe_queries** out);
void apoe_queries_destroy(apoe_queries* q);

/* KG upload (query.cu:1963-1980). Each CSR has rows+1 offsets. */
int apoe_kg_create(apoe_ctx* ctx, uint32_t n_entities, const uint32_t* e2e_off,
                   const uint32_t* e2e_idx, const uint32_t* e2d_off, const uint32_t* e2d_idx,
                   uint32_t n_queries, const uint32_t* q2e_off, const uint32_t* q2e_idx,
                   apoe_kg** out);
void apoe_kg_destroy(apoe_kg* kg);

/*
 * Fused hybrid distance, query side (the per-candidate block of every search
 * kernel, query.cu:536-557): out[q*M+m] = 1 - (w3[0]*dense + w3[1]*splade +
 * w3[2]*bm25) between query q and document ids[q*M+m]; w3 = {dense, splade, bm25};
 * a path with weight < 1e-5 is skipped (query.cu:2004-2041); ids >= n give INF_DIS.
 */
int apoe_hybrid_distance_batch(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q,
                               const float* w3, const uint32_t* ids, uint32_t M, float* out);

/* Build-metric distance between documents a[i] and b[i] (index.cu:248-267):
 * 1 - (dense_scale^2*dense + splade + bm25); dense_scale is the x7 of index.cu:836-840. */
int apoe_hybrid_distance_pairs(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale,
                               const uint32_t* a, const uint32_t* b, uint32_t n_pairs, float* out);

/* Hybrid squared norms (cal_power, index.cu:483-534). out has n floats. */
int apoe_norms(apoe_ctx* ctx, const apoe_corpus* c, float dense_scale, float* out);

/*
 * Query-time weight calibration (query.cu:1847-1869): the largest per-path inner
 * product over the first min(n,100) documents x first min(n_queries,100) queries is
 * taken for each path; the two paths with the smaller maxima have their weights
 * multiplied by max_largest / max_path. w3 = {dense, splade, bm25}, updated in place.
 * Nothing changes on a tie for the largest; a path whose maximum is not positive
 * keeps its weight (the reference divides by it).
 */
int apoe_calibrate_weights(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q,
                           uint32_t n_queries, float* w3);

/* ---- index construction (build_index_impl, index.cu:889-903) ---- */

/* kNN-graph state: ids/dist [n][K], reverse lists, norms. K is 64 or 128 (index.cu:6). */
int apoe_knn_create(apoe_ctx* ctx, const apoe_corpus* c, uint32_t K, float dense_scale,
                    apoe_knn** out);
void apoe_knn_destroy(apoe_knn* g);
/* on != 0: the NN-Descent steps take the dense part of a candidate from the half-precision copy of the rows
 * (apoe_corpus_make_half_rows; 2 KB instead of 4 KB per row read, fp32 products and sums), and
 * apoe_nnd_merge_reverse ends with a pass that computes every stored distance again from the fp32 rows and
 * puts each list in order again, so the prune sees exact distances. Which neighbours the lists hold can
 * differ from the fp32 build's where the rounding (at most 2^-11 dense_scale^2 |a_d| |b_d| per pair) decided.
 * No counterpart in the reference, which has only half-precision rows. */
int apoe_knn_use_half_rows(apoe_knn* g, int on);
/* Which step apoe_nnd_iterate runs (replaces nn_descent_gpu, index.cu:156-376, either way):
 *   0  the reference's expansion step: every node against the forward and reverse lists of the neighbours it
 *      picks, one pivot against many rows (the default);
 *   1  the same pairs as a local join around the picked neighbour: all pickers of a node v are the rows of a
 *      tile, N(v) and R(v) its columns, every row gathered once, the dense part of the tile on the matrix
 *      cores, survivors sent to the row nodes' lists by 64-bit atomicMin on proposal slots and merged by a
 *      second kernel; lists are read as the step found them (the reference reads them while they change); an
 *      entry registers with its node's reverse list once, when it enters, and the reverse lists are kept over
 *      the steps (the reference registers every entry of a changed list and starts them again with every step);
 *   2  as 1, and every pair is offered to the column node as well (insertion into both endpoints' lists, as
 *      the classic NN-Descent join does; the reference's step updates the picking node only).
 * K must be 64 for 1 and 2, and no document may have more than APOE_JOIN_MAX_ROW_TERMS sparse terms (longest SPLADE row +
 * longest BM25 row): a tile keeps the terms of a picker row in an LDS table. May be changed between steps. */
int apoe_knn_set_join(apoe_knn* g, int mode);
/* initialize_graph + cal_power (index.cu:890-892). */
int apoe_nnd_init(apoe_knn* g, uint64_t seed);
/* One nn_descent_gpu + reset_reverse_num step (index.cu:894-897). last != 0 keeps the
 * reverse counts for the following merge. *inserted (optional) = list entries inserted. */
int apoe_nnd_iterate(apoe_knn* g, int last, uint64_t* inserted);
/* merge_reverse_plus (index.cu:898). */
int apoe_nnd_merge_reverse(apoe_knn* g);
/* Copy the kNN graph out / in (ids without flag bits, distances), [n][K] each. */
int apoe_knn_download(apoe_knn* g, uint32_t* ids, float* dist);
int apoe_knn_upload(apoe_knn* g, const uint32_t* ids, const float* dist);
/* The reverse lists as they stand (reverse_graph_dev / reverse_distance / reverse_num, index.cu:90,93,845-846):
 * rev_ids/rev_dist [n][K] (a slot never written holds id 0xFFFFFFFF, distance INF_DIS), rev_cnt [n] = registrations
 * counted so far (may exceed K: later ones replaced slot count % K when closer, index.cu:362-372). Any pointer may
 * be NULL. With the upload they make apoe_nnd_merge_reverse checkable on a state of the caller's making; uploaded
 * ids must name a document or be 0xFFFFFFFF. */
int apoe_knn_download_reverse(apoe_knn* g, uint32_t* rev_ids, float* rev_dist, uint32_t* rev_cnt);
int apoe_knn_upload_reverse(apoe_knn* g, const uint32_t* rev_ids, const float* rev_dist, const uint32_t* rev_cnt);
/* Which form of the prune apoe_prune runs (all replace allan_poe, index.cu:539-714, and give the same rows):
 *   0  (default) the forms that gather every neighbour row once: for K = 64 one workgroup builds the node's hybrid Gram
 *      matrix in LDS and selects on it; for K = 128 the Gram matrices of a batch of nodes are computed by the tile kernel
 *      of the local join (32 rows x up to 128 columns of a list at a time) into device memory and a second kernel selects
 *      on them. A corpus whose rows do not fit the tables of these forms falls back to form 1 by itself;
 *   1  the table-probing kernel: the candidate is the pivot, one wave per live selected member evaluates its product,
 *      rows are read again at every selection step (what the reference does). */
int apoe_knn_set_prune_form(apoe_knn* g, int form);
/* allan_poe (index.cu:539-714): RNG-IP prune to `degree` + keyword-edge candidates. */
int apoe_prune(apoe_knn* g, uint32_t degree);
/* Intermediate result of apoe_prune: fwd/det [n][degree], cnt [n], kw [n][1+APOE_KW_CAND]. */
int apoe_prune_download(apoe_knn* g, uint32_t* fwd, uint32_t* det, uint32_t* cnt, uint32_t* kw);
/* allan_poe_final_graph + entry-point selection (index.cu:717-807, 916-925). */
int apoe_finalize_graph(apoe_knn* g, apoe_graph** out);
/* Milliseconds of GPU time (HIP events on the context stream) spent in the build
 * calls on this handle so far: the reference's "Indexing time" region (index.cu:889-908). */
float apoe_knn_elapsed_ms(const apoe_knn* g);
/* out2 = {hybrid distance evaluations, dense rows read} of the NN-Descent steps since apoe_nnd_init
 * (a candidate whose sparse part plus the bound of its dense part cannot enter the list is not
 * read in full). No counterpart in the reference; used to price the build against the HBM roofline. */
int apoe_knn_counters(apoe_knn* g, uint64_t* out2);

/* ---- graph handle: the .poe payload (index.cu:927-939, query.cu:35-62) ---- */
int apoe_graph_create(apoe_ctx* ctx, uint32_t n, uint32_t width, const uint32_t* rows,
                      const uint32_t* entry, uint32_t n_entry, apoe_graph** out);
void apoe_graph_destroy(apoe_graph* g);
/* info3 = {n, width, n_entry}. */
int apoe_graph_info(const apoe_graph* g, uint32_t* info3);
int apoe_graph_download(const apoe_graph* g, uint32_t* rows, uint32_t* entry);

/* ---- search (search_with_* kernels, query.cu:277-1268, 1541-1779) ---- */
typedef struct {
    float w_dense, w_sparse, w_bm25; /* effective (already calibrated) weights */
    float kg_weight;                 /* used only when kg != NULL */
    uint32_t cands;                  /* pool size, 1..APOE_MAX_CANDS */
    uint32_t max_iter;               /* 0 -> 1000 (query.cu:7 MAX_ITER) */
    uint32_t q_begin, q_count;       /* query range; q_count 0 -> all from q_begin */
    uint32_t variant;                /* low byte: launch shape = waves per query. 0 = default: 16 while every query
                                        has a CU of its own, 8 while the whole batch is resident at once that way,
                                        else 4 up to two rounds of the 2-wave grid (about 6 000 queries), else 2 -
                                        or 4 when the pool is so large that fewer than 9 queries fit a CU (plain
                                        and KG search). 1/2/3/4/5 = 1/4/8/2/16 waves whatever the batch; other
                                        values are refused. Rows do not depend on it.
                                        0x100: read the dense row of every candidate; by
                                        default a candidate whose sparse part plus the Cauchy-Schwarz
                                        bound of its dense part cannot beat the worst entry of the full
                                        pool is dropped without reading its dense row (same results).
                                        0x200: while the graph is walked, the dense part of a candidate is
                                        taken from the half-precision copy of the rows (needs
                                        apoe_corpus_make_half_rows; plain search only); when the walk has
                                        ended every pool entry is evaluated again with its fp32 row and
                                        the pool sorted again, so the reported distances are the exact
                                        ones; an id can differ from the default search's where the
                                        rounding (at most 2^-11 |q_d| |d_d| w_dense per candidate)
                                        changed a decision of the walk */
    uint32_t keyword_filter;         /* 1: keyword-filter search (search_with_keyword, query.cu:1271-1483);
                                        kg must be NULL */
} apoe_search_params;

typedef struct {
    float kernel_ms;      /* HIP-event time of the search kernel on the context stream */
    uint64_t expansions;  /* parents expanded, summed over the queries */
    uint64_t evaluations; /* hybrid distance evaluations */
    uint64_t nnz_sparse;  /* SPLADE pairs read by those evaluations (0 if path off) */
    uint64_t nnz_bm25;    /* BM25 pairs read by those evaluations (0 if path off) */
    uint64_t dense_rows;  /* evaluations that had to read the 4 KB dense row (see variant) */
    uint64_t algo_bytes;  /* algorithmic HBM bytes: dense rows read + pairs + descriptors + graph
                             rows + queries + results */
} apoe_search_stats;

/* out_ids/out_dist are [q_count][cands], ascending distance; top_k is the row
 * prefix (query.cu:2070-2075). Empty slots hold id 0x7FFFFFFF, distance INF_DIS.
 *
 * Keyword-filter search (keyword_filter = 1): a BM25 term id of a QUERY row with bit 31 set is a
 * required keyword (the host sets the bit, query.cu:1828-1843; every search compares term ids
 * under the mask 0x7FFFFFFF, so a flagged term scores like an unflagged one). A document "hits"
 * when one of its BM25 terms is a required keyword of the query. All three paths are computed
 * whatever the weights (the reference runs its three-path loop), slots of a graph row whose
 * neighbour was already visited are refilled from the row's keyword edges, and a result row holds
 * only hits: the hits of the final pool in pool order, then up to 32 hits that were pushed out of
 * the pool (the closest ones, ascending), then empty slots. Needs n < 2^30 documents. */
int apoe_search(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const apoe_graph* g,
                const apoe_kg* kg, const apoe_search_params* p, uint32_t* out_ids, float* out_dist,
                apoe_search_stats* stats);

/*
 * apoe_search without any allocation. No counterpart in the reference: it is for callers that cannot
 * allocate device memory -- tight serving loops, harnesses that forbid hipMalloc. (It still queries the
 * device and the kernel's attributes on every call, so it is not meant to be recorded into a HIP graph.)
 * Same kernels, arguments and results as apoe_search, except that
 *  - out_ids / out_dist must be device memory of the context's GPU (results are written in place);
 *  - the counters, the once-per-query arguments and the visited bitmaps live in one static device array of
 *    APOE_NOALLOC_WS_BYTES that each GPU holds from the first apoe_ctx_create on it until the process
 *    ends; the launch uses as many workgroups as bitmaps of n bits fit there (255 at 1 M documents), so a
 *    large batch runs slower than through apoe_search; corpora above APOE_NOALLOC_MAX_DOCS are refused;
 *  - with stats == NULL the call returns with the search still running on the context's stream
 *    (apoe_ctx_synchronize waits for it); with stats it blocks like apoe_search;
 *  - all calls on one GPU share that array: calls that overlap on a GPU (two contexts, two threads) race.
 */
#define APOE_NOALLOC_WS_BYTES (32u << 20)
#define APOE_NOALLOC_MAX_DOCS (1u << 21)
int apoe_search_noalloc(apoe_ctx* ctx, const apoe_corpus* c, const apoe_queries* q, const apoe_graph* g,
                        const apoe_kg* kg, const apoe_search_params* p, uint32_t* out_ids, float* out_dist,
                        apoe_search_stats* stats);

#ifdef __cplusplus
}
#endif
#endif
