// Python module `hybrid_search`: the same two entry points, keyword names and order
// as the reference's bindings (bindings.cpp:7-40). Both print the reference's stdout
// lines and return None. The extra keyword arguments are the reference's hard-wired
// constants made adjustable (their defaults are those constants), and `search` is the
// same call returning the result arrays instead of only printing nDCG.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "host_impl.h"

namespace py = pybind11;

static hs::SearchResult run_search(const std::string& dense_data_path, const std::string& dense_query_path, const std::string& sparse_data_path,
                                   const std::string& sparse_query_path, const std::string& bm25_data_path, const std::string& bm25_query_path,
                                   const std::string& keyword_id_path, const std::string& knowledge_path, const std::string& entity2doc_path,
                                   const std::string& query_entity_path, const std::string& graph_path, const std::string& ground_truth_path,
                                   int top_k, int cands, float sparse_weight, float bm25_weight, float dense_weight, float kg_weight,
                                   unsigned max_queries, bool calibrate, int device, bool half_rows = false) {
    hs::SearchOptions opt;
    opt.max_queries = max_queries;
    opt.calibrate = calibrate;
    opt.device = device;
    opt.half_rows = half_rows;
    py::gil_scoped_release release;
    return hs::search_index_impl(dense_data_path, dense_query_path, sparse_data_path, sparse_query_path, bm25_data_path, bm25_query_path,
                                 keyword_id_path, knowledge_path, entity2doc_path, query_entity_path, graph_path, ground_truth_path, top_k, cands,
                                 sparse_weight, bm25_weight, dense_weight, kg_weight, opt);
}

PYBIND11_MODULE(hybrid_search, m) {
    m.doc() = "Hybrid Search with Allan-Poe";

    m.def(
        "build_index",
        [](const std::string& dense_data_path, const std::string& sparse_data_path, const std::string& bm25_data_path,
           const std::string& output_graph_path, unsigned degree, unsigned nnd_k, unsigned nnd_iters, float dense_build_scale, uint64_t seed,
           int device, const std::string& knn_save_path, const std::string& knn_load_path, bool half_rows, int nnd_join,
           unsigned nnd_expansion_steps) {
            hs::BuildOptions opt;
            opt.degree = degree;
            opt.nnd_k = nnd_k;
            opt.nnd_iters = nnd_iters;
            opt.dense_build_scale = dense_build_scale;
            opt.seed = seed;
            opt.device = device;
            opt.knn_save_path = knn_save_path;
            opt.knn_load_path = knn_load_path;
            opt.half_rows = half_rows;
            opt.nnd_join = nnd_join;
            opt.nnd_expansion_steps = nnd_expansion_steps;
            py::gil_scoped_release release;
            hs::build_index_impl(dense_data_path, sparse_data_path, bm25_data_path, output_graph_path, opt);
        },
        "Build the hybrid index", py::arg("dense_data_path"), py::arg("sparse_data_path"), py::arg("bm25_data_path"),
        py::arg("output_graph_path"), py::arg("degree") = 32, py::arg("nnd_k") = 64, py::arg("nnd_iters") = 25,
        py::arg("dense_build_scale") = 7.0f, py::arg("seed") = 20251125ull, py::arg("device") = 0, py::arg("knn_save_path") = "",
        py::arg("knn_load_path") = "", py::arg("half_rows") = false, py::arg("nnd_join") = -1, py::arg("nnd_expansion_steps") = 0);

    m.def(
        "search_index",
        [](const std::string& a, const std::string& b, const std::string& c, const std::string& d, const std::string& e, const std::string& f,
           const std::string& g, const std::string& h, const std::string& i, const std::string& j, const std::string& k, const std::string& l,
           int top_k, int cands, float sparse_weight, float bm25_weight, float dense_weight, float kg_weight, unsigned max_queries,
           bool calibrate, int device) {
            run_search(a, b, c, d, e, f, g, h, i, j, k, l, top_k, cands, sparse_weight, bm25_weight, dense_weight, kg_weight, max_queries,
                       calibrate, device);
        },
        "Search the hybrid index", py::arg("dense_data_path"), py::arg("dense_query_path"), py::arg("sparse_data_path"),
        py::arg("sparse_query_path"), py::arg("bm25_data_path"), py::arg("bm25_query_path"), py::arg("keyword_id_path"),
        py::arg("knowledge_path"), py::arg("entity2doc_path"), py::arg("query_entity_path"), py::arg("graph_path"),
        py::arg("ground_truth_path"), py::arg("top_k"), py::arg("cands"), py::arg("sparse_weight"), py::arg("bm25_weight"),
        py::arg("dense_weight"), py::arg("kg_weight"), py::arg("max_queries") = 100, py::arg("calibrate") = true, py::arg("device") = 0);

    m.def(
        "search",
        [](const std::string& a, const std::string& b, const std::string& c, const std::string& d, const std::string& e, const std::string& f,
           const std::string& g, const std::string& h, const std::string& i, const std::string& j, const std::string& k, const std::string& l,
           int top_k, int cands, float sparse_weight, float bm25_weight, float dense_weight, float kg_weight, unsigned max_queries,
           bool calibrate, int device, bool half_rows) {
            hs::SearchResult r = run_search(a, b, c, d, e, f, g, h, i, j, k, l, top_k, cands, sparse_weight, bm25_weight, dense_weight,
                                            kg_weight, max_queries, calibrate, device, half_rows);
            py::array_t<uint32_t> ids({(py::ssize_t)r.query_num, (py::ssize_t)r.cands});
            py::array_t<float> dist({(py::ssize_t)r.query_num, (py::ssize_t)r.cands});
            std::copy(r.ids.begin(), r.ids.end(), ids.mutable_data());
            std::copy(r.dist.begin(), r.dist.end(), dist.mutable_data());
            py::dict out;
            out["ids"] = ids;
            out["dist"] = dist;
            out["weights"] = py::make_tuple(r.weights[0], r.weights[1], r.weights[2]);
            out["kernel_ms"] = r.kernel_ms;
            out["ndcg"] = r.ndcg;
            out["recall"] = r.recall;
            out["evaluations"] = r.evaluations;
            out["expansions"] = r.expansions;
            out["algo_bytes"] = r.algo_bytes;
            return out;
        },
        "search_index that also returns {ids, dist, weights (dense, sparse, bm25), kernel_ms, ndcg, recall, ...}", py::arg("dense_data_path"),
        py::arg("dense_query_path"), py::arg("sparse_data_path"), py::arg("sparse_query_path"), py::arg("bm25_data_path"),
        py::arg("bm25_query_path"), py::arg("keyword_id_path"), py::arg("knowledge_path"), py::arg("entity2doc_path"),
        py::arg("query_entity_path"), py::arg("graph_path"), py::arg("ground_truth_path"), py::arg("top_k"), py::arg("cands"),
        py::arg("sparse_weight"), py::arg("bm25_weight"), py::arg("dense_weight"), py::arg("kg_weight"), py::arg("max_queries") = 100,
        py::arg("calibrate") = true, py::arg("device") = 0, py::arg("half_rows") = false);

    // ---- host-side pieces exposed for tests of the file formats and of nDCG ----
    m.def("_read_fvecs", [](const std::string& path) {
        std::vector<float> data;
        unsigned num = 0, dim = 0;
        hs::load_fvecs(path, data, num, dim);
        py::array_t<float> out({(py::ssize_t)num, (py::ssize_t)dim});
        std::copy(data.begin(), data.end(), out.mutable_data());
        return out;
    });
    m.def("_read_csr", [](const std::string& path, unsigned rows) {
        hs::Csr c;
        hs::load_sparse(path, rows, c);
        return py::make_tuple(py::array_t<uint32_t>(c.off.size(), c.off.data()), py::array_t<uint32_t>(c.idx.size(), c.idx.data()),
                              py::array_t<float>(c.val.size(), c.val.data()));
    });
    m.def("_read_kg", [](const std::string& path) {
        std::vector<unsigned> off, idx;
        unsigned num = 0;
        hs::load_kg(path, off, idx, num);
        return py::make_tuple(py::array_t<uint32_t>(off.size(), off.data()), py::array_t<uint32_t>(idx.size(), idx.data()));
    });
    m.def("_read_id_lines", [](const std::string& path, unsigned n) {
        std::vector<std::vector<unsigned>> r(n);
        hs::load_txt(path, r, n);
        return r;
    });
    m.def("_read_poe", [](const std::string& path) {
        std::vector<unsigned> rows, entry;
        unsigned width = 0, num = 0;
        hs::load_graph(path, rows, entry, width, num);
        py::array_t<uint32_t> out({(py::ssize_t)num, (py::ssize_t)width});
        std::copy(rows.begin(), rows.end(), out.mutable_data());
        return py::make_tuple(out, py::array_t<uint32_t>(entry.size(), entry.data()));
    });
    m.def("_write_poe", [](const std::string& path, py::array_t<uint32_t, py::array::c_style | py::array::forcecast> rows,
                           py::array_t<uint32_t, py::array::c_style | py::array::forcecast> entry) {
        std::vector<unsigned> r(rows.data(), rows.data() + rows.size()), e(entry.data(), entry.data() + entry.size());
        hs::write_graph(path, r, (unsigned)rows.shape(0), (unsigned)rows.shape(1), e);
    });
    m.def(
        "validate_graph",
        [](const std::string& path, unsigned num_docs) {
            const hs::GraphReport r = hs::validate_graph(path, num_docs);
            py::dict d;
            d["ok"] = r.ok;
            d["message"] = r.message;
            d["width"] = r.width;
            d["degree"] = r.degree;
            d["num"] = r.num;
            d["n_entry"] = r.n_entry;
            d["file_bytes"] = r.file_bytes;
            d["trailing_bytes"] = r.trailing_bytes;
            d["bad_width_words"] = r.bad_width_words;
            d["bad_neighbours"] = r.bad_neighbours;
            d["bad_keyword_edges"] = r.bad_keyword_edges;
            d["bad_entry_points"] = r.bad_entry_points;
            d["self_loops"] = r.self_loops;
            d["keyword_counts_over_7"] = r.keyword_counts_over_7;
            d["keyword_edges"] = r.keyword_edges;
            return d;
        },
        py::arg("graph_path"), py::arg("num_docs") = 0u,
        "Check a .poe graph file (size formula, width words, id ranges, keyword counts) without a GPU; returns a dict with 'ok' and counts.");
    m.def("_ndcg", [](const std::vector<std::vector<unsigned>>& res, const std::vector<std::vector<unsigned>>& gt) {
        double recall = 0;
        double n = hs::ndcg_at_k(res, gt, &recall);
        return py::make_tuple(n, recall);
    });
}
