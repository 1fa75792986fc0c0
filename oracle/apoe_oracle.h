/*
 * CPU oracle for the Allan-Poe hybrid graph index hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the checker that the HIP path is
 * compared against; nothing shipped (the C-ABI library, the hybrid_search
 * module) links, imports or calls it. It restates, in plain C++ on the host,
 * the algorithms of the reference's CUDA kernels (file:line citations are
 * relative to the reference checkout), with the reference's undefined or racy
 * behaviours replaced by the defined semantics noted at each function.
 *
 * All matrices are row-major; CSR arrays use the reference's on-disk layout
 * (off[rows+1], idx[nnz] ascending in a row, val[nnz]).
 */
#ifndef APOE_ORACLE_H
#define APOE_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_INF_DIS 1000000.0f /* index.cu:8, query.cu:11 */
#define ORC_EMPTY 0xFFFFFFFFu
#define ORC_FLAG 0x80000000u
#define ORC_KW_SLOTS 8  /* index.cu:15 KEYEDGEFINAL */
#define ORC_KW_CAND 32  /* index.cu:14 KEYEDGE */

/* A hybrid vector set: dense rows + SPLADE CSR + BM25 CSR. */
typedef struct {
    uint32_t n;
    uint32_t dim;
    const float* dense;
    const uint32_t* s_off;
    const uint32_t* s_idx;
    const float* s_val;
    const uint32_t* b_off;
    const uint32_t* b_idx;
    const float* b_val;
} orc_set;

/* KG CSR triple (query.cu:89-108): entity->entity, entity->doc, query->entity. */
typedef struct {
    uint32_t n_entities;
    const uint32_t* e2e_off;
    const uint32_t* e2e_idx;
    const uint32_t* e2d_off;
    const uint32_t* e2d_idx;
    const uint32_t* q2e_off;
    const uint32_t* q2e_idx;
} orc_kg;

/* Per-path inner products of a[i] and b[j]: out3 = {dense, splade, bm25}. */
void orc_ip_parts(const orc_set* a, uint32_t i, const orc_set* b, uint32_t j, float* out3);

/* dist[q][m] = 1 - (w[0]*dense + w[1]*splade + w[2]*bm25) for ids[q*M+m]. */
void orc_distance_batch(const orc_set* corpus, const orc_set* queries, const float* w3,
                        const uint32_t* ids, uint32_t M, float* out, int threads);

/* Pair distances inside one set under the build metric:
 * 1 - (scale^2*dense + splade + bm25). */
void orc_distance_pairs(const orc_set* corpus, float dense_scale, const uint32_t* a,
                        const uint32_t* b, uint32_t n_pairs, float* out, int threads);

/* Hybrid squared norm scale^2*|d|^2 + |s|^2 + |b|^2 (index.cu:483-534). */
void orc_norms(const orc_set* corpus, float dense_scale, float* out, int threads);

/* Exact top-k by hybrid distance (ties by id). Query side (w3) or build metric. */
void orc_bruteforce_topk(const orc_set* corpus, const orc_set* queries, const float* w3,
                         uint32_t k, uint32_t* out_ids, float* out_dist, int threads);
void orc_bruteforce_knn_self(const orc_set* corpus, float dense_scale, uint32_t k,
                             uint32_t* out_ids, float* out_dist, int threads);

/* Rank merge of a sorted pool with a sorted new list, ties new-before-old,
 * truncated to cap (query.cu:181-224). pool arrays are updated in place. */
void orc_merge_top(uint32_t* pool_ids, float* pool_dist, uint32_t cap, const uint32_t* new_ids,
                   const float* new_dist, uint32_t n_new);

/* Greedy beam search (query.cu:414-570). graph is [n][W] with W = degree+8.
 * counters (optional, per query): {expansions, evaluations, sum nnz splade, sum nnz bm25}. */
void orc_search(const orc_set* corpus, const orc_set* queries, const uint32_t* graph, uint32_t W,
                const uint32_t* entry, uint32_t n_entry, const float* w3, uint32_t cands,
                uint32_t max_iter, uint32_t* out_ids, float* out_dist, uint64_t* counters,
                int threads);

/* Keyword-filter beam search (query.cu:1271-1483): query BM25 term ids with bit 31 set are the
 * required keywords; rows hold only documents with such a term (pool hits, then evicted hits). */
void orc_search_keyword(const orc_set* corpus, const orc_set* queries, const uint32_t* graph,
                        uint32_t W, const uint32_t* entry, uint32_t n_entry, const float* w3,
                        uint32_t cands, uint32_t max_iter, uint32_t* out_ids, float* out_dist,
                        uint64_t* counters, int threads);

/* Beam search with KG seeding and logical-edge expansion (query.cu:1541-1779). */
void orc_search_kg(const orc_set* corpus, const orc_set* queries, const orc_kg* kg,
                   const uint32_t* graph, uint32_t W, const uint32_t* entry, uint32_t n_entry,
                   const float* w3, float kg_weight, uint32_t cands, uint32_t max_iter,
                   uint32_t* out_ids, float* out_dist, uint64_t* counters, int threads);

/* omp_get_max_threads(): the thread count every function here uses when its `threads` argument is 0. */
int orc_max_threads(void);

/* NN-Descent (index.cu:99-106, 156-478). ids carry ORC_FLAG = "already sampled". */
uint32_t orc_rand_id(uint64_t seed, uint64_t counter, uint32_t n);
void orc_nnd_init(uint32_t n, uint32_t K, uint64_t seed, uint32_t* ids, float* dist,
                  uint32_t* rev, float* rev_dist, uint32_t* rev_cnt);
uint64_t orc_nnd_iterate(const orc_set* corpus, float dense_scale, uint32_t K, uint32_t* ids,
                         float* dist, uint32_t* rev, float* rev_dist, uint32_t* rev_cnt,
                         int threads);
void orc_nnd_merge_reverse(uint32_t n, uint32_t K, uint32_t* ids, float* dist, const uint32_t* rev,
                           const float* rev_dist, const uint32_t* rev_cnt, int threads);

/*
 * The NN-Descent step as a LOCAL JOIN around the picked neighbour. It stands where
 * orc_nnd_iterate stands (index.cu:156-376) and evaluates the same pairs -- node u against
 * the forward list N(v) and the reverse list R(v) of each neighbour v it picks, by the same
 * picking rule -- but as the GPU's join kernels do it: all pickers of one v form the rows of a
 * tile whose columns are N(v) and R(v), every list is read as it was when the step started,
 * and a row's survivors travel to its list as proposals: slot (mix64(id) >> 40) mod `slots`
 * of the node's proposal row keeps the smallest (distance, id), so a step is deterministic
 * whatever the order of evaluation (the reverse lists keep the reference's arrival order).
 * With `symmetric` a pair (u, c) is also offered to the COLUMN node c (u proposed to c's list
 * when it is closer than c's last entry; whether c already holds u is only looked at when c
 * merges): the classic join's insertion into both endpoints, which the reference's step does
 * not do.
 * Then every node merges its proposals (new before old on equal distance, index.cu:333-351);
 * the entries that are NEW in a list register with the reverse lists of their nodes (slot
 * count mod K, the closer one stays beyond K). The reference registers every entry of a changed
 * list and starts the reverse lists again with every step (index.cu:362-372, :896); the join
 * keeps the reverse lists over the steps -- the caller does not reset rev_cnt between join
 * steps -- so an entry registers once, when it enters.
 */
typedef struct {
    uint32_t slots;      /* proposal slots per node, a power of two */
    uint32_t symmetric;  /* 1: offer every evaluated pair to both endpoints */
} orc_join_params;
/* Returns the number of list entries inserted; *evals (optional) += distances computed. */
uint64_t orc_join_iterate(const orc_set* corpus, float dense_scale, uint32_t K, uint32_t* ids,
                          float* dist, uint32_t* rev, float* rev_dist, uint32_t* rev_cnt,
                          const orc_join_params* prm, uint64_t* evals, int threads);

/* RNG-IP prune + keyword recycling (index.cu:539-714).
 * out_fwd [n][d] ids, out_det [n][d] detour counts, out_cnt [n] real entries,
 * out_kw [n][1+ORC_KW_CAND] = count followed by keyword-edge candidates. */
void orc_prune(const orc_set* corpus, float dense_scale, const float* norms, uint32_t K,
               const uint32_t* ids, const float* dist, uint32_t d, uint32_t* out_fwd,
               uint32_t* out_det, uint32_t* out_cnt, uint32_t* out_kw, int threads);

/* Final row assembly (index.cu:717-807): rows [n][d+8]. */
void orc_final_graph(uint32_t n, uint32_t d, const uint32_t* fwd, const uint32_t* det,
                     const uint32_t* cnt, const uint32_t* kw, uint32_t* rows);

/* d docs of smallest hybrid norm, ties by id (index.cu:916-925). */
void orc_entry_points(const float* norms, uint32_t n, uint32_t d, uint32_t* out);

/* Query-time weight calibration (query.cu:1847-1869). w3 = {dense, splade, bm25} in/out. */
void orc_calibrate(const orc_set* corpus, const orc_set* queries, uint32_t n_queries, float* w3);

/* nDCG@k and recall as cal_precision computes them (query.cu:111-145).
 * res [nq][k]; gt as CSR (gt_off[nq+1], gt_idx). out2 = {nDCG, recall}. */
void orc_ndcg(const uint32_t* res, uint32_t nq, uint32_t k, const uint32_t* gt_off,
              const uint32_t* gt_idx, double* out2);

/* Full build pipeline on host cores, same order as index.cu:889-903. rows [n][d+8],
 * entry [d]. knn_ids/knn_dist (optional, [n][K]) receive the kNN graph after N3. */
void orc_build(const orc_set* corpus, float dense_scale, uint32_t K, uint32_t iters, uint32_t d,
               uint64_t seed, uint32_t* rows, uint32_t* entry, uint32_t* knn_ids, float* knn_dist,
               int threads);

#ifdef __cplusplus
}
#endif
#endif
