"""Pins three branches of the oracle on inputs whose expected output is written out by hand or by a closed
form (CPU): the keyword flag of the prune (index.cu:128-153,637,651-666), the tagging of a fresh graph
neighbour that is also a logical neighbour in the knowledge-graph search (query.cu:1699-1715), and the merge of
the reverse lists (index.cu:386-478). Each check is also run against deliberately broken builds of the oracle
(one textual change each, compiled into a temporary directory) and must fail there."""
import os
import re
import subprocess

import numpy as np
import pytest

import pin_worlds as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------ the checks (take the oracle module as an argument)

def check_keyword_flag(O, term_shift=0):
    arrays, ids, dist, expect = P.keyword_flag_world(term_shift=term_shift)
    C = O.HybridSet(*arrays)
    nrm = O.norms(C, 7.0)
    assert abs(nrm[10] - 1.49) < 1e-5 and abs(nrm[1] - 10.49) < 1e-5  # the arithmetic of the world's docstring
    fwd, det, cnt, kw = O.prune(C, 7.0, nrm, ids, dist, expect["d"])
    assert fwd[0].tolist() == expect["fwd0"]
    assert cnt[0] == expect["cnt0"]
    assert kw[0, 0] == len(expect["kw0"]) and kw[0, 1:1 + kw[0, 0]].tolist() == expect["kw0"]
    assert np.all(kw[1:, 0] == 0)


def check_kg_fresh_neighbour(O):
    corpus, queries, rows, entry, kg, expect = P.kg_fresh_neighbour_world()
    C, Q = O.HybridSet(*corpus), O.HybridSet(*queries)
    ids, dist, _ = O.search(C, Q, rows, entry, (1, 0, 0), expect["cands"], kg=O.Kg(*kg), kg_weight=expect["kg_weight"])
    plain = 1.0 - corpus[0].astype(np.float64) @ queries[0][0].astype(np.float64)
    P.check_kg_fresh_neighbour(ids[0], dist[0], plain, expect)


def reverse_state(O, n=700, steps=3, seed=9):
    import apoe_synth as S
    C = O.HybridSet(*S.to_numpy(S.corpus(n, seed=41, device="cpu")))
    st = O.nnd_init(C.n, 64, seed)
    for it in range(steps):
        O.nnd_iterate(C, 7.0, st, threads=1)
        if it < steps - 1:
            st.rev_cnt[:] = 0
    return st


def check_merge_reverse(O, st=None):
    st = st or reverse_state(O)
    want_ids, want_dist = P.merge_reverse_closed_form(st.n, st.K, st.ids, st.dist, st.rev, st.rev_dist, st.rev_cnt)
    changed = int(np.sum(np.any(want_ids != st.ids, axis=1)))
    assert changed > st.n // 2, "the state must give the merge something to do"
    O.nnd_merge_reverse(st)
    assert np.array_equal(st.ids, want_ids)
    assert np.array_equal(st.dist, want_dist)


def crafted_reverse_state(O):
    """One node whose reverse list holds every special case: the node itself, an id out of range, an id the
    list already holds, an empty slot, the same id twice (the closer copy counts), an entry exactly as far
    as a list entry (goes in front of it), more registrations than K (only K slots exist)."""
    n, K = 80, 64
    st = O.KnnState(n, K)
    st.ids[:] = ((np.arange(n, dtype=np.uint32) + 1) % n)[:, None]  # filler: every slot names the next node at INF_DIS
    st.dist[:] = P.INF_DIS
    st.rev[:] = 0xFFFFFFFF
    st.rev_dist[:] = P.INF_DIS
    st.rev_cnt[:] = 0
    u = 7
    st.ids[u, :4] = [20 | 0x80000000, 21, 22, 23]  # 20 carries the sampled flag
    st.dist[u, :4] = [0.1, 0.2, 0.3, 0.4]
    st.rev[u, :9] = [7, 9999, 21, 0xFFFFFFFF, 30, 30, 31, 32, 33]
    st.rev_dist[u, :9] = [0.0, 0.01, 0.02, 0.03, 0.25, 0.15, 0.3, 0.35, 5.0]
    st.rev_cnt[u] = 200
    v = 8  # a node whose counter says 2 although more slots are written: only the first two count
    st.ids[v, :1] = [40]
    st.dist[v, :1] = [0.5]
    st.rev[v, :3] = [41, 42, 43]
    st.rev_dist[v, :3] = [0.7, 0.6, 0.1]
    st.rev_cnt[v] = 2
    return st, u, v


def check_merge_reverse_crafted(O):
    st, u, v = crafted_reverse_state(O)
    O.nnd_merge_reverse(st)
    assert st.ids[u, :8].tolist() == [20 | 0x80000000, 30, 21, 31, 22, 32, 23, 33]
    assert np.allclose(st.dist[u, :8], [0.1, 0.15, 0.2, 0.3, 0.3, 0.35, 0.4, 5.0])
    assert np.all(st.dist[u, 8:] == P.INF_DIS)
    assert st.ids[v, :3].tolist() == [40, 42, 41] and st.dist[v, 3] == P.INF_DIS


def test_keyword_flag_world():
    import oracle as O
    check_keyword_flag(O)
    check_keyword_flag(O, term_shift=70000)


def test_kg_fresh_neighbour_world():
    import oracle as O
    check_kg_fresh_neighbour(O)


def test_merge_reverse_closed_form():
    import oracle as O
    check_merge_reverse(O)
    check_merge_reverse_crafted(O)


def test_merge_reverse_closed_form_after_a_join_step():
    """The join keeps its reverse lists over the steps and lets the counter pass K."""
    import apoe_synth as S
    import oracle as O
    C = O.HybridSet(*S.to_numpy(S.corpus(700, seed=41, device="cpu")))
    st = O.nnd_init(C.n, 64, 3)
    for _ in range(4):
        O.join_iterate(C, 7.0, st, slots=128, threads=1)
    check_merge_reverse(O, st)


# ------------------------------------------------------------------ broken builds

MUTANTS = {
    # prune keyword flag (orc_prune)
    "kw_any_member": ([(r"bool reject = false, all_flag = true;", "bool reject = false, all_flag = true, any_flag = false;"),
                       (r"if \(!flag\) all_flag = false;", "if (flag) any_flag = true;"),
                       (r"sel\.push_back\(\{c, det\[order\[t\]\], true, all_flag\}\);", "sel.push_back({c, det[order[t]], true, any_flag && all_flag});")],
                      check_keyword_flag),
    "kw_swapped": ([(r"k < sbn && !flag", "k < cbn && !flag"), (r"uint32_t term = sb\[k\];", "uint32_t term = cb[k];"),
                    (r"!std::binary_search\(cb, cb \+ cbn, term\) && std::binary_search\(ub, ub \+ ubn, term\)",
                     "!std::binary_search(sb, sb + sbn, term) && std::binary_search(ub, ub + ubn, term)")], check_keyword_flag),
    "kw_inverted": ([(r"if \(!flag\) all_flag = false;", "if (flag) all_flag = false;")], check_keyword_flag),
    "kw_ignores_centre": ([(r"!std::binary_search\(cb, cb \+ cbn, term\) && std::binary_search\(ub, ub \+ ubn, term\)",
                            "!std::binary_search(cb, cb + cbn, term)")], check_keyword_flag),
    "kw_counts_dead_members": ([(r"if \(!s\.live\) continue;\n(\s+)float p = \(float\)build_ip\(corpus, c, s\.id, dense_scale\);",
                                 r"\1float p = s.live ? (float)build_ip(corpus, c, s.id, dense_scale) : -1e30f;")], check_keyword_flag),
    # knowledge-graph search, branch (i)
    "kg_last_entity_wins": ([(r"if \(s\.state == 0 && s\.id == doc\)", "if (s.state != 2 && s.id == doc)")], check_kg_fresh_neighbour),
    "kg_no_tagging": ([(r"if \(s\.state == 0 && s\.id == doc\) \{ s\.state = 1; s\.ent = e2; \}", "(void)doc;")], check_kg_fresh_neighbour),
    "kg_bonus_without_hop": ([(r"dist -= kg_weight / \(float\)s\.hop;", "dist -= kg_weight;")], check_kg_fresh_neighbour),
    "kg_bonus_for_all": ([(r"if \(s\.state == 1\) dist -= kg_weight / \(float\)s\.hop;", "dist -= kg_weight / (float)s.hop;")], check_kg_fresh_neighbour),
    # reverse merge
    "rev_noop": ([(r"(void orc_nnd_merge_reverse\([^{]*\{)", r"\1 return;")], check_merge_reverse),
    "rev_keeps_far_copy": ([(r"return a\.id < b\.id \|\| \(a\.id == b\.id && a\.dist < b\.dist\);",
                             "return a.id < b.id || (a.id == b.id && a.dist > b.dist);")], check_merge_reverse_crafted),
    "rev_no_list_check": ([(r"if \(!in_list\) fresh\.push_back\(\{rev_dist\[base \+ j\], r, 0, 0\}\);",
                            "fresh.push_back({rev_dist[base + j], r, 0, 0});")], check_merge_reverse_crafted),
    "rev_ignores_count": ([(r"const uint32_t cnt = std::min\(K, rev_cnt\[uu\]\);", "const uint32_t cnt = K; (void)rev_cnt;")], check_merge_reverse_crafted),
    "rev_old_before_new": ([(r"fresh\[f\]\.dist <= pool\[p\]\.dist", "fresh[f].dist < pool[p].dist")], check_merge_reverse_crafted),
    "rev_keeps_self": ([(r"\|\| r >= n \|\| r == \(uint32_t\)uu\) continue;", "|| r >= n) continue;")], check_merge_reverse_crafted),
}


def _load_mutant(name, tmp):
    """A second copy of oracle.py bound to the broken library (its own module object, its own CDLL)."""
    import importlib.util
    mutated = open(os.path.join(ROOT, "oracle", "apoe_oracle.cpp")).read()
    for pattern, repl in MUTANTS[name][0]:
        mutated, count = re.subn(pattern, repl, mutated, count=1)
        assert count == 1, f"mutant {name}: the line to break was not found in the oracle ({pattern})"
    cpp = os.path.join(tmp, f"{name}.cpp")
    so = os.path.join(tmp, f"lib{name}.so")
    with open(cpp, "w") as f:
        f.write(mutated)
    subprocess.check_call(["g++", "-O1", "-march=x86-64-v3", "-fopenmp", "-fPIC", "-std=c++17", "-shared", "-I", os.path.join(ROOT, "oracle"),
                           "-o", so, cpp])
    spec = importlib.util.spec_from_file_location(f"oracle_mutant_{name}", os.path.join(ROOT, "oracle", "oracle.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    os.environ["APOE_ORACLE_LIB"] = so
    try:
        mod.lib()
    finally:
        del os.environ["APOE_ORACLE_LIB"]
    return mod


@pytest.mark.skipif("APOE_ORACLE_LIB" in os.environ, reason="runs its own builds of the oracle")
@pytest.mark.parametrize("name", sorted(MUTANTS))
def test_broken_oracle_fails_its_pin(name, tmp_path):
    mod = _load_mutant(name, str(tmp_path))
    with pytest.raises(AssertionError):
        MUTANTS[name][1](mod)
