// Host drivers behind the hybrid_search Python module: the file loaders, the .poe
// writer/reader, nDCG, and build_index_impl / search_index_impl with the reference's
// argument meaning and stdout lines (index.cu:810-941, query.cu:1781-2081). All GPU
// work goes through the C-ABI of include/apoe.h; failures throw std::runtime_error
// (the reference calls exit()).
#include "host_impl.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <stdexcept>

#include "../../include/apoe.h"

namespace hs {

namespace {

[[noreturn]] void fail(const std::string& what) { throw std::runtime_error(what); }

void check(int status, const char* what) {
    if (status != APOE_OK) fail(std::string(what) + ": " + apoe_last_error_string());
}

size_t file_size(std::ifstream& in) {
    in.seekg(0, std::ios::end);
    size_t s = (size_t)in.tellg();
    in.seekg(0, std::ios::beg);
    return s;
}

template <typename T>
void read_exact(std::ifstream& in, T* dst, size_t count, const std::string& path) {
    in.read(reinterpret_cast<char*>(dst), (std::streamsize)(count * sizeof(T)));
    if ((size_t)in.gcount() != count * sizeof(T)) fail("truncated file: " + path);
}

struct Handles { // RAII over the C-ABI handles of one call
    apoe_ctx* ctx = nullptr;
    apoe_corpus* corpus = nullptr;
    apoe_queries* queries = nullptr;
    apoe_kg* kg = nullptr;
    apoe_graph* graph = nullptr;
    apoe_knn* knn = nullptr;
    ~Handles() {
        apoe_knn_destroy(knn);
        apoe_graph_destroy(graph);
        apoe_kg_destroy(kg);
        apoe_queries_destroy(queries);
        apoe_corpus_destroy(corpus);
        apoe_ctx_destroy(ctx);
    }
};

} // namespace

// utils.cuh:361-378
void load_fvecs(const std::string& path, std::vector<float>& data, unsigned& num, unsigned& dim) {
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) fail("open file error: " + path);
    const size_t fsize = file_size(in);
    if (fsize < 4) fail("truncated file: " + path);
    read_exact(in, &dim, 1, path);
    if (dim == 0) fail("zero dimension in " + path);
    num = (unsigned)(fsize / ((size_t)dim + 1) / 4);
    data.resize((size_t)num * dim);
    in.seekg(0, std::ios::beg);
    std::vector<uint32_t> row((size_t)dim + 1);
    for (size_t i = 0; i < num; i++) {
        read_exact(in, row.data(), (size_t)dim + 1, path);
        std::memcpy(data.data() + i * dim, row.data() + 1, (size_t)dim * 4);
    }
}

// utils.cuh:380-398; rows = number of vectors (the reference passes rows+1)
void load_sparse(const std::string& path, unsigned rows, Csr& out) {
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) fail("open file error: " + path);
    unsigned nnz = 0;
    read_exact(in, &nnz, 1, path);
    std::cout << "Non zero num: " << nnz << std::endl;
    out.off.resize((size_t)rows + 1);
    out.idx.resize(nnz);
    out.val.resize(nnz);
    read_exact(in, out.off.data(), (size_t)rows + 1, path);
    read_exact(in, out.idx.data(), nnz, path);
    read_exact(in, out.val.data(), nnz, path);
    if (out.off[rows] > nnz) fail("offsets exceed the non-zero count in " + path);
}

// query.cu:89-108; the leading count is rows + 1
void load_kg(const std::string& path, std::vector<unsigned>& off, std::vector<unsigned>& idx, unsigned& num) {
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) fail("open file error: " + path);
    unsigned nnz = 0;
    read_exact(in, &num, 1, path);
    read_exact(in, &nnz, 1, path);
    std::cout << "Entity num: " << num << ", Non zero num: " << nnz << std::endl;
    if (num == 0) fail("empty CSR in " + path);
    off.resize(num);
    idx.resize(nnz);
    read_exact(in, off.data(), num, path);
    read_exact(in, idx.data(), nnz, path);
    if (off[num - 1] > nnz) fail("offsets exceed the non-zero count in " + path);
}

// query.cu:65-86: a missing file is reported and leaves the lists empty
void load_txt(const std::string& path, std::vector<std::vector<unsigned>>& results, unsigned query_num) {
    std::ifstream file(path);
    if (!file.is_open()) {
        std::cout << "open file error" << std::endl;
        return;
    }
    std::string line;
    unsigned count = 0;
    while (count < query_num && std::getline(file, line)) {
        std::istringstream iss(line);
        unsigned number;
        while (iss >> number) results[count].push_back(number);
        count++;
    }
}

// index.cu:927-939
void write_graph(const std::string& path, const std::vector<unsigned>& rows, unsigned n, unsigned width, const std::vector<unsigned>& entry) {
    std::ofstream out(path, std::ios::binary | std::ios::out);
    if (!out.is_open()) fail("cannot write " + path);
    const unsigned n_ep = (unsigned)entry.size();
    out.write(reinterpret_cast<const char*>(&width), 4);
    out.write(reinterpret_cast<const char*>(&n_ep), 4);
    out.write(reinterpret_cast<const char*>(entry.data()), (std::streamsize)n_ep * 4);
    for (size_t i = 0; i < n; i++) {
        out.write(reinterpret_cast<const char*>(&width), 4);
        out.write(reinterpret_cast<const char*>(rows.data() + i * width), (std::streamsize)width * 4);
    }
    if (!out.good()) fail("write error on " + path);
}

// query.cu:35-62
void load_graph(const std::string& path, std::vector<unsigned>& rows, std::vector<unsigned>& entry, unsigned& width, unsigned& num) {
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) fail("open file error: " + path);
    const size_t fsize = file_size(in);
    unsigned ent_num = 0;
    read_exact(in, &width, 1, path);
    read_exact(in, &ent_num, 1, path);
    if (width == 0 || fsize < ((size_t)ent_num + 2) * 4) fail("bad graph header in " + path);
    num = (unsigned)((fsize - ((size_t)ent_num + 2) * 4) / ((size_t)width + 1) / 4);
    std::cout << "Degree: " << width << "," << "num: " << num << std::endl;
    entry.resize(ent_num);
    read_exact(in, entry.data(), ent_num, path);
    rows.resize((size_t)num * width);
    unsigned w = 0;
    for (size_t i = 0; i < num; i++) {
        read_exact(in, &w, 1, path);
        read_exact(in, rows.data() + i * width, width, path);
    }
}

GraphReport validate_graph(const std::string& path, unsigned num_docs) {
    GraphReport r;
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) fail("open file error: " + path);
    r.file_bytes = file_size(in);
    if (r.file_bytes < 8) fail("bad graph header in " + path);
    read_exact(in, &r.width, 1, path);
    read_exact(in, &r.n_entry, 1, path);
    if (r.width <= 8 || r.file_bytes < ((uint64_t)r.n_entry + 2) * 4) fail("bad graph header in " + path);
    r.degree = r.width - 8;
    const uint64_t body = r.file_bytes - ((uint64_t)r.n_entry + 2) * 4, row_bytes = ((uint64_t)r.width + 1) * 4;
    r.num = (unsigned)(body / row_bytes);
    r.trailing_bytes = body % row_bytes;
    std::vector<unsigned> entry(r.n_entry), row(r.width);
    read_exact(in, entry.data(), r.n_entry, path);
    for (unsigned e : entry) r.bad_entry_points += e >= r.num;
    for (unsigned v = 0; v < r.num; v++) {
        unsigned w = 0;
        read_exact(in, &w, 1, path);
        read_exact(in, row.data(), r.width, path);
        r.bad_width_words += w != r.width;
        for (unsigned j = 0; j < r.degree; j++) {
            r.bad_neighbours += row[j] >= r.num;
            r.self_loops += row[j] == v;
        }
        const unsigned cnt = row[r.degree];
        r.keyword_counts_over_7 += cnt > 7;
        for (unsigned j = 0; j < std::min(cnt, 7u); j++) r.bad_keyword_edges += row[r.degree + 1 + j] >= r.num;
        r.keyword_edges += std::min(cnt, 7u);
    }
    std::ostringstream msg;
    if (r.trailing_bytes) msg << r.trailing_bytes << " bytes after the last whole row; ";
    if (num_docs && num_docs != r.num) msg << "holds " << r.num << " rows, expected " << num_docs << "; ";
    if (r.bad_width_words) msg << r.bad_width_words << " rows with a wrong width word; ";
    if (r.bad_neighbours) msg << r.bad_neighbours << " neighbour ids out of range; ";
    if (r.bad_keyword_edges) msg << r.bad_keyword_edges << " keyword-edge ids out of range; ";
    if (r.bad_entry_points) msg << r.bad_entry_points << " entry points out of range; ";
    r.message = msg.str();
    r.ok = r.message.empty();
    if (r.ok) r.message = "ok";
    return r;
}

// K-NN graph between NN-Descent and the prune: "APKN", n, K, ids [n][K], distances [n][K].
void write_knn(const std::string& path, unsigned n, unsigned K, const std::vector<unsigned>& ids, const std::vector<float>& dist) {
    std::ofstream out(path, std::ios::binary | std::ios::out);
    if (!out.is_open()) fail("cannot write " + path);
    const unsigned head[3] = {0x4E4B5041u, n, K}; // "APKN"
    out.write(reinterpret_cast<const char*>(head), sizeof(head));
    out.write(reinterpret_cast<const char*>(ids.data()), (std::streamsize)ids.size() * 4);
    out.write(reinterpret_cast<const char*>(dist.data()), (std::streamsize)dist.size() * 4);
    if (!out.good()) fail("write error on " + path);
}

void load_knn(const std::string& path, unsigned n, unsigned K, std::vector<unsigned>& ids, std::vector<float>& dist) {
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) fail("open file error: " + path);
    unsigned head[3] = {0, 0, 0};
    read_exact(in, head, 3, path);
    if (head[0] != 0x4E4B5041u) fail(path + " is not a K-NN graph file");
    if (head[1] != n || head[2] != K) fail("K-NN graph in " + path + " is for " + std::to_string(head[1]) + " points, K = " + std::to_string(head[2]));
    ids.resize((size_t)n * K);
    dist.resize((size_t)n * K);
    read_exact(in, ids.data(), ids.size(), path);
    read_exact(in, dist.data(), dist.size(), path);
    for (unsigned v : ids)
        if (v >= n) fail("K-NN graph in " + path + " names a point beyond the corpus");
}

// query.cu:111-145: IDCG over all ground-truth ids, DCG by position in the result
double ndcg_at_k(const std::vector<std::vector<unsigned>>& res, std::vector<std::vector<unsigned>> gt, double* recall) {
    float all = 0.f, ndcg = 0.f;
    for (size_t i = 0; i < res.size(); i++) {
        if (gt[i].empty()) continue; // the reference divides by zero here
        float idcg = 0.f;
        for (unsigned j = 0; j < gt[i].size(); j++) idcg += 1.f / std::log2((float)(j + 2));
        std::vector<unsigned> r = res[i], v;
        std::sort(r.begin(), r.end());
        std::sort(gt[i].begin(), gt[i].end());
        std::set_intersection(r.begin(), r.end(), gt[i].begin(), gt[i].end(), std::back_inserter(v));
        all += (float)v.size() / (float)gt[i].size();
        float dcg = 0.f;
        for (unsigned x : v)
            for (unsigned it = 0; it < res[i].size(); it++)
                if (res[i][it] == x) { dcg += 1.f / std::log2((float)(it + 2)); break; }
        ndcg += dcg / idcg;
    }
    if (recall) *recall = res.empty() ? 0.0 : all / res.size();
    return res.empty() ? 0.0 : ndcg / res.size();
}

static unsigned max_row(const std::vector<unsigned>& off, unsigned rows) {
    unsigned m = 0;
    for (unsigned i = 0; i < rows; i++) m = std::max(m, off[i + 1] - off[i]);
    return m;
}

void build_index_impl(const std::string& dense_data_path, const std::string& sparse_data_path, const std::string& bm25_data_path,
                      const std::string& output_graph_path, const BuildOptions& opt) {
    std::vector<float> dense;
    unsigned points_num = 0, dim = 0;
    Csr sparse, bm25;
    std::cout << "Loading dense data from " << dense_data_path << std::endl;
    load_fvecs(dense_data_path, dense, points_num, dim);
    load_sparse(sparse_data_path, points_num, sparse);
    load_sparse(bm25_data_path, points_num, bm25);
    std::cout << "Points: " << points_num << ", Dim: " << dim << std::endl;
    std::cout << "Max sparse dim: " << max_row(sparse.off, points_num) << ", Max bm25 dim: " << max_row(bm25.off, points_num) << std::endl;

    Handles h;
    check(apoe_ctx_create(opt.device, &h.ctx), "apoe_ctx_create");
    check(apoe_corpus_create(h.ctx, points_num, dim, dense.data(), sparse.off.data(), sparse.idx.data(), sparse.val.data(), bm25.off.data(),
                             bm25.idx.data(), bm25.val.data(), &h.corpus),
          "apoe_corpus_create");
    // index.cu:889-903; the x7 dense scale of index.cu:836-840 is applied inside the metric
    check(apoe_knn_create(h.ctx, h.corpus, opt.nnd_k, opt.dense_build_scale, &h.knn), "apoe_knn_create");
    if (!opt.knn_load_path.empty()) {
        std::vector<unsigned> ids;
        std::vector<float> dist;
        load_knn(opt.knn_load_path, points_num, opt.nnd_k, ids, dist);
        check(apoe_knn_upload(h.knn, ids.data(), dist.data()), "apoe_knn_upload");
    } else {
        if (opt.half_rows) {
            check(apoe_corpus_make_half_rows(h.ctx, h.corpus), "apoe_corpus_make_half_rows");
            check(apoe_knn_use_half_rows(h.knn, 1), "apoe_knn_use_half_rows");
        }
        unsigned info[4] = {0, 0, 0, 0};
        check(apoe_corpus_info(h.corpus, info), "apoe_corpus_info");
        // nnd_join < 0: the local join where its tile holds every row. A corpus in the wide pair format hashes a row's terms
        // into the tile's table, which takes rows of about a thousand terms safely; beyond that, and if a step still meets a
        // row that it cannot hold, the build runs (again) with the expansion step.
        const unsigned longest = info[2] + info[3]; // longest SPLADE row + longest BM25 row
        const bool wide = apoe_corpus_pair_bytes(h.corpus) == 8;
        const bool rows_fit = longest <= (wide ? 1024u : (unsigned)APOE_JOIN_MAX_ROW_TERMS);
        int join = opt.nnd_join >= 0 ? opt.nnd_join : (!opt.half_rows && rows_fit ? 1 : 0);
        while (true) {
            check(apoe_knn_set_join(h.knn, join), "apoe_knn_set_join"); // refuses what the handle cannot run before any step does
            check(apoe_nnd_init(h.knn, opt.seed), "apoe_nnd_init");
            int status = APOE_OK;
            for (unsigned it = 0; it < opt.nnd_iters && status == APOE_OK; it++) {
                check(apoe_knn_set_join(h.knn, it < opt.nnd_expansion_steps ? 0 : join), "apoe_knn_set_join");
                status = apoe_nnd_iterate(h.knn, it + 1 == opt.nnd_iters, nullptr);
            }
            if (status == APOE_ERR_STATE && join != 0 && opt.nnd_join < 0) { // a row did not fit the join's table
                join = 0;
                continue;
            }
            check(status, "apoe_nnd_iterate");
            break;
        }
        check(apoe_nnd_merge_reverse(h.knn), "apoe_nnd_merge_reverse");
    }
    if (!opt.knn_save_path.empty()) {
        std::vector<unsigned> ids((size_t)points_num * opt.nnd_k);
        std::vector<float> dist((size_t)points_num * opt.nnd_k);
        check(apoe_knn_download(h.knn, ids.data(), dist.data()), "apoe_knn_download");
        write_knn(opt.knn_save_path, points_num, opt.nnd_k, ids, dist);
    }
    check(apoe_prune(h.knn, opt.degree), "apoe_prune");
    check(apoe_finalize_graph(h.knn, &h.graph), "apoe_finalize_graph");
    std::cout << "Indexing time: " << apoe_knn_elapsed_ms(h.knn) / 1000.0f << "s" << std::endl;

    unsigned info[3];
    check(apoe_graph_info(h.graph, info), "apoe_graph_info");
    std::vector<unsigned> rows((size_t)info[0] * info[1]), entry(info[2]);
    check(apoe_graph_download(h.graph, rows.data(), entry.data()), "apoe_graph_download");
    write_graph(output_graph_path, rows, info[0], info[1], entry);
}

SearchResult search_index_impl(const std::string& dense_data_path, const std::string& dense_query_path, const std::string& sparse_data_path,
                               const std::string& sparse_query_path, const std::string& bm25_data_path, const std::string& bm25_query_path,
                               const std::string& keyword_id_path, const std::string& knowledge_path, const std::string& entity2doc_path,
                               const std::string& query_entity_path, const std::string& graph_path, const std::string& ground_truth_path,
                               int top_k, int cands, float sparse_weight, float bm25_weight, float dense_weight, float kg_weight,
                               const SearchOptions& opt) {
    if (top_k < 1 || cands < top_k) fail("need 1 <= top_k <= cands");
    std::vector<float> dense, qdense;
    unsigned points_num = 0, dim = 0, query_num = 0, query_dim = 0;
    Csr sparse, bm25, qsparse, qbm25;
    load_fvecs(dense_data_path, dense, points_num, dim);
    load_fvecs(dense_query_path, qdense, query_num, query_dim);
    if (dim != query_dim) fail("corpus and query dimensions differ");
    load_sparse(sparse_data_path, points_num, sparse);
    load_sparse(bm25_data_path, points_num, bm25);
    load_sparse(sparse_query_path, query_num, qsparse);
    load_sparse(bm25_query_path, query_num, qbm25);

    std::vector<unsigned> kg_off, kg_idx, e2d_off, e2d_idx, qe_off, qe_idx;
    unsigned entity_num = 0, entity_num2 = 0, query_entity_num = 0;
    const bool have_kg = !knowledge_path.empty();
    if (have_kg) {
        load_kg(knowledge_path, kg_off, kg_idx, entity_num);
        load_kg(entity2doc_path, e2d_off, e2d_idx, entity_num2);
        load_kg(query_entity_path, qe_off, qe_idx, query_entity_num);
        if (entity_num2 != entity_num) fail("knowledge graph and entity2doc disagree on the entity count");
    }

    // the reference searches the first 100 queries only (query.cu:1825)
    query_num = std::min(query_num, opt.max_queries);
    std::cout << "query num: " << query_num << std::endl;
    // query.cu:1828-1843: a BM25 term of query i that line i of the keyword file lists becomes a
    // required keyword (bit 31 of its id)
    const bool have_keywords = !keyword_id_path.empty();
    if (have_keywords) {
        std::vector<std::vector<unsigned>> keyword_vec(query_num);
        load_txt(keyword_id_path, keyword_vec, query_num);
        unsigned t_count = 0;
        for (unsigned i = 0; i < query_num; i++)
            for (unsigned j = qbm25.off[i]; j < qbm25.off[i + 1]; j++)
                for (unsigned kw : keyword_vec[i])
                    if (kw == qbm25.idx[j]) {
                        qbm25.idx[j] |= 0x80000000u;
                        t_count += 1;
                    }
        std::cout << "keywords: " << t_count << std::endl;
    }
    if (have_kg && query_entity_num < query_num + 1) fail("query entity file has fewer rows than queries");

    std::cout << "Dense weight: " << dense_weight << ", Sparse weight: " << sparse_weight << ", BM25 weight: " << bm25_weight
              << ", KG weight: " << kg_weight << std::endl;

    std::vector<unsigned> rows, entry;
    unsigned width = 0, graph_num = 0;
    load_graph(graph_path, rows, entry, width, graph_num);
    if (graph_num != points_num) fail("graph and corpus disagree on the number of points");
    std::cout << "Points: " << points_num << ", Dim: " << dim << std::endl;
    std::cout << "Query: " << query_num << ", Dim: " << query_dim << std::endl;
    std::cout << "Max sparse dim: " << max_row(sparse.off, points_num) << ", Max bm25 dim: " << max_row(bm25.off, points_num) << std::endl;
    std::cout << "Max query sparse dim: " << max_row(qsparse.off, query_num) << ", Max query bm25 dim: " << max_row(qbm25.off, query_num)
              << std::endl;

    Handles h;
    check(apoe_ctx_create(opt.device, &h.ctx), "apoe_ctx_create");
    check(apoe_corpus_create(h.ctx, points_num, dim, dense.data(), sparse.off.data(), sparse.idx.data(), sparse.val.data(), bm25.off.data(),
                             bm25.idx.data(), bm25.val.data(), &h.corpus),
          "apoe_corpus_create");
    check(apoe_queries_create(h.ctx, query_num, dim, qdense.data(), qsparse.off.data(), qsparse.idx.data(), qsparse.val.data(),
                              qbm25.off.data(), qbm25.idx.data(), qbm25.val.data(), &h.queries),
          "apoe_queries_create");
    check(apoe_graph_create(h.ctx, points_num, width, rows.data(), entry.data(), (unsigned)entry.size(), &h.graph), "apoe_graph_create");
    if (have_kg) {
        check(apoe_kg_create(h.ctx, entity_num - 1, kg_off.data(), kg_idx.data(), e2d_off.data(), e2d_idx.data(), query_num, qe_off.data(),
                             qe_idx.data(), &h.kg),
              "apoe_kg_create");
        std::cout << "KG Copy end" << std::endl;
    }

    // query.cu:1847-1869
    float w3[3] = {dense_weight, sparse_weight, bm25_weight};
    if (opt.calibrate) check(apoe_calibrate_weights(h.ctx, h.corpus, h.queries, query_num, w3), "apoe_calibrate_weights");

    std::cout << "Begin search" << std::endl;
    const bool on_d = !(w3[0] < 1e-5f), on_s = !(w3[1] < 1e-5f), on_b = !(w3[2] < 1e-5f);
    const bool use_kg = !(kg_weight < 1e-5f);
    // query.cu:2004-2047: the knowledge-graph search wins over the keyword filter, which wins over the weights
    const bool use_keywords = have_keywords && !use_kg;
    if (use_kg) {
        std::cout << "Search with dense + sparse + bm25 + kg" << std::endl;
        if (!have_kg) fail("kg_weight is set but knowledge_path is empty"); // the reference launches nothing here (query.cu:2042-2047)
    } else if (use_keywords) {
        std::cout << "Search with dense + sparse + bm25 + keyword" << std::endl;
    } else {
        if (!on_d && !on_s && !on_b) fail("all three weights are zero"); // the reference launches nothing here
        std::string what;
        for (const char* part : {on_d ? "dense" : "", on_s ? "sparse" : "", on_b ? "bm25" : ""})
            if (*part) what += (what.empty() ? "" : " + ") + std::string(part);
        std::cout << "Search with " << what << std::endl;
    }

    SearchResult res;
    res.query_num = query_num;
    res.cands = (unsigned)cands;
    res.ids.resize((size_t)query_num * cands);
    res.dist.resize((size_t)query_num * cands);
    apoe_search_params p{};
    p.w_dense = w3[0];
    p.w_sparse = w3[1];
    p.w_bm25 = w3[2];
    p.kg_weight = kg_weight;
    p.cands = (unsigned)cands;
    p.keyword_filter = use_keywords ? 1u : 0u;
    if (opt.half_rows && !use_kg && !use_keywords) {
        check(apoe_corpus_make_half_rows(h.ctx, h.corpus), "apoe_corpus_make_half_rows");
        p.variant |= 0x200u;
    }
    apoe_search_stats st{};
    const auto start = std::chrono::high_resolution_clock::now();
    check(apoe_search(h.ctx, h.corpus, h.queries, h.graph, use_kg ? h.kg : nullptr, &p, res.ids.data(), res.dist.data(), &st), "apoe_search");
    const std::chrono::duration<float> duration = std::chrono::high_resolution_clock::now() - start;
    std::cout << "Query time: " << duration.count() << "s" << std::endl;
    res.kernel_ms = st.kernel_ms;
    res.weights[0] = w3[0];
    res.weights[1] = w3[1];
    res.weights[2] = w3[2];
    res.evaluations = st.evaluations;
    res.expansions = st.expansions;
    res.algo_bytes = st.algo_bytes;

    // query.cu:2070-2080
    std::vector<std::vector<unsigned>> results2(query_num), gt(query_num);
    for (unsigned i = 0; i < query_num; i++)
        for (int j = 0; j < top_k; j++) results2[i].push_back(res.ids[(size_t)i * cands + j]);
    load_txt(ground_truth_path, gt, query_num);
    res.ndcg = ndcg_at_k(results2, gt, &res.recall);
    std::cout << "nDCG@10: " << res.ndcg << std::endl;
    return res;
}

} // namespace hs
