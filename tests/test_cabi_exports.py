"""The C-ABI library loads without a GPU and exports every function include/apoe.h declares (CPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "apoe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(apoe_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    import apoe
    lib = ctypes.CDLL(apoe.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(apoe.EXPORTS) == names


def test_errors_are_status_codes_not_exits():
    import apoe
    lib = apoe.lib()
    h = ctypes.c_void_p()
    # no GPU here (or device 99 does not exist on a GPU box): a status and a message, never exit()
    st = lib.apoe_ctx_create(ctypes.c_int(99), ctypes.byref(h))
    assert st < 0 and len(lib.apoe_last_error_string()) > 0
    assert lib.apoe_corpus_info(None, None) == -1
    assert b"null" in lib.apoe_last_error_string()


def test_module_surface_matches_reference():
    import hybrid_search
    assert hybrid_search.__doc__ == "Hybrid Search with Allan-Poe"
    doc = hybrid_search.build_index.__doc__
    for kw in ("dense_data_path", "sparse_data_path", "bm25_data_path", "output_graph_path"):
        assert kw in doc
    doc = hybrid_search.search_index.__doc__
    order = ["dense_data_path", "dense_query_path", "sparse_data_path", "sparse_query_path", "bm25_data_path", "bm25_query_path",
             "keyword_id_path", "knowledge_path", "entity2doc_path", "query_entity_path", "graph_path", "ground_truth_path", "top_k",
             "cands", "sparse_weight", "bm25_weight", "dense_weight", "kg_weight"]
    pos = [doc.index(k + ":") for k in order]
    assert pos == sorted(pos)
