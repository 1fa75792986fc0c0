// Host drivers of the hybrid_search module (see host_impl.cpp).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace hs {

struct Csr {
    std::vector<unsigned> off, idx;
    std::vector<float> val;
};

// Knobs that the reference hard-wires; the defaults are the reference's constants.
struct BuildOptions {
    unsigned degree = 32;           // index.cu:888
    unsigned nnd_k = 64;            // index.cu:6
    unsigned nnd_iters = 25;        // index.cu:884
    float dense_build_scale = 7.0f; // index.cu:836-840
    uint64_t seed = 20251125;       // the reference seeds from clock(), index.cu:102
    int device = 0;
    // Intermediate artefact, no counterpart in the reference: the K-NN graph between NN-Descent
    // (after the reverse merge) and the prune. Saving it allows a re-prune to another degree
    // without repeating NN-Descent; loading it skips NN-Descent.
    // File: "APKN", n, K (u32 each), then ids [n][K] u32, then distances [n][K] f32.
    std::string knn_save_path;
    std::string knn_load_path;
    // NN-Descent steps on a half-precision copy of the dense rows (what the reference stores), stored distances
    // recomputed from the fp32 rows before the prune. Off: every step reads fp32 rows.
    bool half_rows = false;
    // 0: the reference's expansion step (index.cu:156-376). 1: the same pairs as a local join around the picked
    // neighbour (rows gathered once per tile, dense part on the matrix cores). 2: the join, both endpoints updated.
    // -1 (default): the join (1) when the handle allows it -- fp32 rows that fit the tile's table -- else the expansion step.
    int nnd_join = -1;
    // With a join: the first nnd_expansion_steps steps are expansion steps all the same. The join's first steps on random
    // lists bring little; on very large corpora (millions of documents) one leading expansion step leaves better lists
    // after the same number of steps (8 M documents, 10 steps: list recall@10 0.30 instead of 0.27, for 1.1 s more).
    unsigned nnd_expansion_steps = 0;
};

struct SearchOptions {
    unsigned max_queries = 100; // query.cu:1825
    bool calibrate = true;      // query.cu:1847-1869
    int device = 0;
    // Plain search only (ignored with keywords or a knowledge graph): walk the graph on a half-precision copy of the
    // dense rows and evaluate the final pool again from the fp32 rows.
    bool half_rows = false;
};

struct SearchResult {
    unsigned query_num = 0, cands = 0;
    std::vector<unsigned> ids; // [query_num][cands]
    std::vector<float> dist;   // [query_num][cands]
    float weights[3] = {0, 0, 0}; // effective dense, sparse, bm25
    float kernel_ms = 0;
    double ndcg = 0, recall = 0;
    uint64_t evaluations = 0, expansions = 0, algo_bytes = 0;
};

void load_fvecs(const std::string& path, std::vector<float>& data, unsigned& num, unsigned& dim);
void load_sparse(const std::string& path, unsigned rows, Csr& out);
void load_kg(const std::string& path, std::vector<unsigned>& off, std::vector<unsigned>& idx, unsigned& num);
void load_txt(const std::string& path, std::vector<std::vector<unsigned>>& results, unsigned query_num);
void write_graph(const std::string& path, const std::vector<unsigned>& rows, unsigned n, unsigned width, const std::vector<unsigned>& entry);
void load_graph(const std::string& path, std::vector<unsigned>& rows, std::vector<unsigned>& entry, unsigned& width, unsigned& num);

// What a .poe file holds, and whether every row is usable by the search kernels: the size formula
// 8 + 4*n_ep + N*(W+1)*4 (index.cu:927-939), the per-row width words, neighbour / keyword-edge /
// entry-point ids below N, keyword counts at most 7 (a larger count is clamped by the search, so it
// is reported, not an error). num_docs = 0 takes N from the file size, as the reader does
// (query.cu:35-62). No counterpart in the reference, which trusts the file.
struct GraphReport {
    unsigned width = 0, degree = 0, num = 0, n_entry = 0;
    uint64_t file_bytes = 0, trailing_bytes = 0; // bytes after the last whole row
    uint64_t bad_width_words = 0;                // rows whose leading width word differs from the header's
    uint64_t bad_neighbours = 0, bad_keyword_edges = 0, bad_entry_points = 0; // ids >= N
    uint64_t self_loops = 0;                     // neighbour slots that hold the row's own id (legal padding)
    uint64_t keyword_counts_over_7 = 0, keyword_edges = 0;
    bool ok = false; // no trailing bytes, no bad width word, no id out of range, N as expected
    std::string message;
};
GraphReport validate_graph(const std::string& path, unsigned num_docs = 0);

void write_knn(const std::string& path, unsigned n, unsigned K, const std::vector<unsigned>& ids, const std::vector<float>& dist);
void load_knn(const std::string& path, unsigned n, unsigned K, std::vector<unsigned>& ids, std::vector<float>& dist);
double ndcg_at_k(const std::vector<std::vector<unsigned>>& res, std::vector<std::vector<unsigned>> gt, double* recall);

void build_index_impl(const std::string& dense_data_path, const std::string& sparse_data_path, const std::string& bm25_data_path,
                      const std::string& output_graph_path, const BuildOptions& opt);

SearchResult search_index_impl(const std::string& dense_data_path, const std::string& dense_query_path, const std::string& sparse_data_path,
                               const std::string& sparse_query_path, const std::string& bm25_data_path, const std::string& bm25_query_path,
                               const std::string& keyword_id_path, const std::string& knowledge_path, const std::string& entity2doc_path,
                               const std::string& query_entity_path, const std::string& graph_path, const std::string& ground_truth_path,
                               int top_k, int cands, float sparse_weight, float bm25_weight, float dense_weight, float kg_weight,
                               const SearchOptions& opt);

} // namespace hs
