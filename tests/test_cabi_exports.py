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


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """include/apoe.h is the boundary a cgo / JNI / FFI binding compiles against: it must be valid C99 by itself, and a C
    program that calls through it must link against the library and get a status code back."""
    import subprocess
    import apoe
    src = tmp_path / "caller.c"
    src.write_text('#include "apoe.h"\n'
                   "#include <stdio.h>\n"
                   "int main(void) {\n"
                   "    apoe_ctx* ctx = 0;\n"
                   "    int st = apoe_ctx_create(99, &ctx);\n"
                   '    printf("%d %s\\n", st, apoe_last_error_string());\n'
                   "    return st == APOE_OK;\n"
                   "}\n")
    exe = tmp_path / "caller"
    libdir = os.path.dirname(apoe.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                    "-L", libdir, "-lapoe", "-Wl,-rpath," + libdir], check=True, capture_output=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 1)
    assert int(out[0]) < 0 and len(out[1].strip()) > 0
