"""Copies the small example data files of the reference checkout into tests/golden/
as fixtures (data only: binary vectors, CSR files, a qrels text file). The large dense
query file is cut to its first 8 rows. Run once from the repository root:

    python tests/golden/make_fixtures.py /root/reference/example_data
"""
import os
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
COPY = ["2wiki_bm25_queries.bin", "2wiki_query_kg.bin", "2wiki_qrels.txt", "2wiki_bm25_corpus.bin", "2wiki_kg.bin", "2wiki_entity2doc.bin"]


def main(src):
    for name in COPY:
        shutil.copyfile(os.path.join(src, name), os.path.join(HERE, name))
    row = (1024 + 1) * 4
    with open(os.path.join(src, "2wiki_dense_queries.fvecs"), "rb") as f, open(os.path.join(HERE, "2wiki_dense_queries_head8.fvecs"), "wb") as g:
        g.write(f.read(8 * row))
    # the sparse query file is cut to its first 16 rows: [nnz][17 offsets][idx][val]
    import numpy as np
    raw = np.fromfile(os.path.join(src, "2wiki_sparse_queries.bin"), dtype=np.uint32)
    nnz, rows = int(raw[0]), 1000
    off = raw[1:2 + rows]
    idx = raw[2 + rows:2 + rows + nnz]
    val = raw[2 + rows + nnz:2 + rows + 2 * nnz]
    k = int(off[16])
    out = np.concatenate([np.array([k], np.uint32), off[:17], idx[:k], val[:k]])
    out.tofile(os.path.join(HERE, "2wiki_sparse_queries_head16.bin"))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference/example_data")
