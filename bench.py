#!/usr/bin/env python3
"""Headline benchmark: search QPS at recall@10 >= 0.95 and index build seconds on a
synthetic hybrid corpus (dense 1024-d + SPLADE-like CSR + BM25-like CSR), one MI355X.
When no pool of the sweep reaches the recall target the line says so in `metric`,
`config.recall_target_met` and `config.qps_at_recall_target` (null), and `value` is the
rate at the largest configured pool (256).

A "step" is one pass of the beam-search kernel over the whole query batch, inputs
already resident in HBM. The JSON line also carries the roofline of the search kernel
(algorithmic bytes from the kernel's own counters / HIP-event time) and the same
search run by the CPU oracle on the host cores (a reported baseline only).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--docs N] [--queries Q]
"""
import argparse
import json
import os
import re
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "allan-poe_amd"))

HBM_PEAK_GBS = 8000.0

# HBM bytes per search launch, RECORDED from FETCH_SIZE + WRITE_SIZE counter runs (rocprofv3 --pmc, scaled by what the
# counters read for a 1 GiB copy) and not measured by this script: keyed by the workload they were taken on
# (corpus, docs, degree, queries, cands, variant, NN-Descent step) with the profiles/ file that holds the run. Any other
# workload reports null.
RECORDED_TRAFFIC = {
    ("iid", 1_000_000, 48, 10_000, 256, 0, 1): {"default": 1.876e11, "every_dense_row_read": 5.312e11,
                                                 "source": "profiles/bench_1Mdocs_degree48_cands256.md (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from a 1 GiB copy)"},
    ("latent", 1_000_000, 48, 10_000, 80, 0, 1): {"default": 1.872e11, "every_dense_row_read": 1.872e11,
                                                  "source": "profiles/bench_1Mdocs_latent_degree48_cands80.md (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from a 1 GiB copy)"},
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def recall_at_k(found, truth, k):
    hit = 0
    for f, t in zip(found, truth):
        hit += len(set(f[:k].tolist()) & set(t[:k].tolist()))
    return hit / (len(truth) * k)


def build_index(apoe, ctx, gc, args, join, keep_lists=False):
    """NN-Descent + reverse merge + prune + final rows; returns (graph, timings dict, K-NN ids or None)."""
    t0 = time.time()
    knn = apoe.Knn(ctx, gc, args.nnd_k, 7.0)
    knn.init(1)
    for it in range(args.nnd_iters):
        knn.set_join(0 if it < args.nnd_expansion_steps else join)
        knn.iterate(last=(it == args.nnd_iters - 1))
    nnd_ms = knn.elapsed_ms()
    evals, rows = knn.counters()
    knn.merge_reverse()
    lists = knn.download()[0] if keep_lists else None
    knn.prune(args.degree)
    graph = knn.finalize()
    total_ms = knn.elapsed_ms()
    knn.close()
    return graph, dict(nnd_ms=nnd_ms, total_ms=total_ms, wall_s=time.time() - t0, evaluations=evals, rows_read=rows), lists


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--docs", type=int, default=1_000_000)
    ap.add_argument("--queries", type=int, default=10_000)
    ap.add_argument("--degree", type=int, default=48)
    ap.add_argument("--nnd-k", type=int, default=64)
    ap.add_argument("--nnd-iters", type=int, default=10)
    ap.add_argument("--join", type=int, default=1, help="NN-Descent step of the index the searches run on: 0 the reference's expansion step, "
                    "1 the local join around the picked neighbour (same pairs), 2 the join that updates both endpoints")
    ap.add_argument("--nnd-expansion-steps", type=int, default=0, help="with a join: that many leading steps are expansion steps all the same "
                    "(one such step pays on corpora of several million documents)")
    ap.add_argument("--cands", type=str, default="64,128,256,512,1024,2048",
                    help="pool sizes of the recall sweep; 64,128,256 are the configured ones, the larger ones look for the recall target")
    ap.add_argument("--truth-queries", type=int, default=1000)
    ap.add_argument("--cpu-queries", type=int, default=10000)
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-membench", action="store_true", help="do not run bench/membench for roofline.random_read_ceiling")
    ap.add_argument("--no-sweeps", action="store_true", help="skip the query-time weight sweep and the knowledge-graph search (about 10 s)")
    ap.add_argument("--extras", action="store_true",
                    help="also time: the keyword-filter search, a four times longer batch, the corpus handed over as host buffers, "
                         "the half-precision walks and build")
    ap.add_argument("--corpus", choices=("iid", "latent"), default="iid",
                    help="iid: the configured generators (no document has neighbours); latent: apoe_synth.latent_corpus (dense rows steered by a hidden "
                         "16-dimensional vector, terms valued by rarity), searched under the build metric 49/1/1")
    ap.add_argument("--calibrate", action="store_true",
                    help="apply the reference's query-time weight calibration to the 1/1/1 weights (off: the metric is literally 1/1/1)")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run one 1 GiB device-to-device copy (reference point for FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box here has one GPU); run with --gpus 1")

    import numpy as np
    import torch
    import apoe
    import apoe_bruteforce as B
    import apoe_synth as S

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = "cuda:0"
    t0 = time.time()
    latent = args.corpus == "latent"
    gen_corpus, gen_queries = (S.latent_corpus, S.latent_queries) if latent else (S.corpus, S.queries)
    user_weights = (49.0, 1.0, 1.0) if latent else (1.0, 1.0, 1.0)
    corpus = gen_corpus(args.docs, device=dev)
    queries = gen_queries(args.queries, device=dev)
    torch.cuda.synchronize()
    log(f"[bench] generated {args.docs} docs / {args.queries} queries in {time.time() - t0:.1f}s; "
        f"nnz/doc splade {corpus[2].numel() / args.docs:.1f} bm25 {corpus[5].numel() / args.docs:.1f}")

    ctx = apoe.Context(0)
    t0 = time.time()
    gc = apoe.Corpus(ctx, *corpus)
    gq = apoe.Queries(ctx, *queries)
    log(f"[bench] packed corpus: {gc.bytes() / 1e9:.2f} GB of records in {time.time() - t0:.2f}s")

    # ---- index build (NN-Descent + reverse merge + RNG-IP prune + final rows), with both NN-Descent steps ----
    mean_pairs = (corpus[2].numel() + corpus[5].numel()) / args.docs
    row_bytes = 4096 + gc.pair_bytes() * mean_pairs + 12
    builds = {}
    graph = None
    lists = None
    for join in sorted({0, args.join}):
        g, tm, ls = build_index(apoe, ctx, gc, args, join, keep_lists=True)
        if join == 0:
            # expansion step: an evaluation reads pairs + descriptor, and the dense row when the bound does not settle it
            tm["algo_bytes"] = tm["rows_read"] * 4096 + tm["evaluations"] * (gc.pair_bytes() * mean_pairs + 12)
        else:
            # join: every row of a tile is read once, in full
            tm["algo_bytes"] = tm["rows_read"] * row_bytes
        builds[join] = tm
        log(f"[bench] build (NN-Descent step {join}): {tm['total_ms'] / 1e3:.2f}s GPU time ({tm['wall_s']:.2f}s wall); NN-Descent {tm['nnd_ms'] / 1e3:.2f}s, "
            f"{tm['evaluations'] / 1e9:.2f}G pair evaluations, {tm['rows_read'] / 1e9:.3f}G rows read, {tm['algo_bytes'] / (tm['nnd_ms'] / 1e3) / 1e12:.2f} TB/s algorithmic")
        if join == args.join:
            graph, lists = g, ls
        else:
            builds[join]["lists"] = ls
            g.close()
    # K-NN list quality of both builds against exact lists of a node sample (brute force by torch)
    gsamp = torch.Generator(device="cpu")
    gsamp.manual_seed(7)
    samp = torch.sort(torch.randperm(args.docs, generator=gsamp)[:1000])[0].to(dev)
    exact, _ = B.hybrid_topk(corpus, B.rows_as_queries(corpus, samp), (49.0, 1.0, 1.0), 10, self_ids=samp.cpu().numpy())
    samp_np = samp.cpu().numpy()
    for join, tm in builds.items():
        ls = tm.pop("lists", None)
        ls = lists if ls is None else ls
        tm["knn_list_recall_at_10"] = float(np.mean([len(set(ls[samp_np[i], :10].tolist()) & set(exact[i].tolist())) / 10 for i in range(len(samp_np))]))
        log(f"[bench] NN-Descent step {join}: K-NN list recall@10 on 1000 sampled nodes {tm['knn_list_recall_at_10']:.4f}")
    del lists
    bt = builds[args.join]

    # ---- effective weights and exact ground truth on a query subset ----
    w3 = apoe.calibrate_weights(ctx, gc, gq, (1.0, 1.0, 1.0)) if args.calibrate else user_weights
    nq_truth = min(args.truth_queries, args.queries)
    t0 = time.time()
    truth, _ = B.hybrid_topk(corpus, queries, w3, 10, nq=nq_truth)
    log(f"[bench] effective weights dense/sparse/bm25 = {w3}; ground truth for {nq_truth} queries in {time.time() - t0:.1f}s")

    # ---- pool sweep: recall and one launch each ----
    sweep = []

    def iter_cap(c):
        # the reference stops a walk after 1000 expansions (query.cu:7 MAX_ITER), fewer than a pool above 512 has entries:
        # the larger pools of the sweep get four expansions per entry so that the pool, not the cap, ends the walk
        return 0 if c <= 512 else 4 * c

    for cands in [int(c) for c in args.cands.split(",")]:
        apoe.search(ctx, gc, gq, graph, w3, cands, variant=args.variant, max_iter=iter_cap(cands))
        ids, dist, st = apoe.search(ctx, gc, gq, graph, w3, cands, variant=args.variant, max_iter=iter_cap(cands))
        rec = recall_at_k(ids[:nq_truth], truth, 10)
        sweep.append(dict(cands=cands, max_iter=iter_cap(cands) or 1000, recall=rec, ms=st.kernel_ms, qps=args.queries / (st.kernel_ms / 1e3),
                          gbs=st.algo_bytes / (st.kernel_ms / 1e3) / 1e9))
        log(f"[bench] cands={cands}: recall@10={rec:.4f} kernel {st.kernel_ms:.2f} ms -> {sweep[-1]['qps']:.0f} QPS, "
            f"{sweep[-1]['gbs']:.0f} GB/s algorithmic, {st.evaluations / args.queries:.0f} evals/query, "
            f"{st.dense_rows / max(st.evaluations, 1):.2f} of them read the dense row")
    ok = [s for s in sweep if s["recall"] >= 0.95]
    # the smallest pool that reaches the recall target; if none does, the largest configured pool (256) stands in and the
    # line says so: `value` is then NOT a rate at the target
    configured = [s for s in sweep if s["cands"] <= 256] or sweep
    pick = ok[0] if ok else configured[-1]
    cands = pick["cands"]

    out_ids = torch.empty((args.queries, cands), dtype=torch.int32, device=dev)
    out_dist = torch.empty((args.queries, cands), dtype=torch.float32, device=dev)
    for _ in range(args.warmup):
        apoe.search(ctx, gc, gq, graph, w3, cands, variant=args.variant, out_ids=out_ids, out_dist=out_dist, max_iter=iter_cap(cands))
    torch.cuda.synchronize()
    ctx.synchronize()
    kernel_ms, algo_bytes = [], 0
    t0 = time.perf_counter()
    for _ in range(args.steps):
        _, _, st = apoe.search(ctx, gc, gq, graph, w3, cands, variant=args.variant, out_ids=out_ids, out_dist=out_dist, max_iter=iter_cap(cands))
        kernel_ms.append(st.kernel_ms)
        algo_bytes = st.algo_bytes
    ctx.synchronize()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    achieved = algo_bytes / (avg_kernel_ms / 1e3) / 1e9
    # the same launch with the dense row of every candidate read (no bound test): same results, more bytes
    full_ms, full_bytes = [], 0
    for i in range(args.warmup + args.steps):
        _, _, stf = apoe.search(ctx, gc, gq, graph, w3, cands, variant=args.variant | 0x100, out_ids=out_ids, out_dist=out_dist, max_iter=iter_cap(cands))
        if i >= args.warmup:
            full_ms.append(stf.kernel_ms)
            full_bytes = stf.algo_bytes
    full_avg = sum(full_ms) / len(full_ms)
    key = (args.corpus, args.docs, args.degree, args.queries, cands, args.variant, args.join)
    rec_traffic = RECORDED_TRAFFIC.get(key) if not args.calibrate else None
    full_eval = {"kernel_ms": full_avg, "qps": args.queries / (full_avg / 1e3), "achieved": full_bytes / (full_avg / 1e3) / 1e9,
                 "frac": full_bytes / (full_avg / 1e3) / 1e9 / HBM_PEAK_GBS, "algo_bytes_per_launch": full_bytes,
                 "traffic": rec_traffic["every_dense_row_read"] if rec_traffic else None}
    log(f"[bench] timed: {avg_kernel_ms:.2f} ms/launch, {achieved:.0f} GB/s algorithmic; every dense row read: {full_avg:.2f} ms, "
        f"{full_eval['achieved']:.0f} GB/s")

    # ---- the other searches of the configured workloads: query-time weight sweep without rebuild, knowledge graph ----
    weight_sweep, kg_search = None, None
    if not args.no_sweeps:
        weight_sweep = []
        for wx in ((1.0, 0.0, 0.0), (0.0, 1.0, 0.0), (0.0, 0.0, 1.0), (1.0, 1.0, 1.0), (1.0, 0.5, 2.0)):
            tx, _ = B.hybrid_topk(corpus, queries, wx, 10, nq=nq_truth)
            for ec in (64, 128, 256):
                apoe.search(ctx, gc, gq, graph, wx, ec)
                ids_x, _, sx = apoe.search(ctx, gc, gq, graph, wx, ec)
                weight_sweep.append(dict(weights=wx, cands=ec, kernel_ms=sx.kernel_ms, qps=args.queries / (sx.kernel_ms / 1e3),
                                         recall_at_10=recall_at_k(ids_x[:nq_truth], tx, 10), algo_gbs=sx.algo_bytes / (sx.kernel_ms / 1e3) / 1e9))
                log(f"[bench] weights {wx} cands {ec}: {sx.kernel_ms:.2f} ms, recall {weight_sweep[-1]['recall_at_10']:.4f}")
        kg = S.knowledge_graph(200_000, args.docs, args.queries, device=dev)
        gkg = apoe.KnowledgeGraph(ctx, *kg)
        apoe.search(ctx, gc, gq, graph, w3, 128, kg=gkg, kg_weight=40.0)
        ids_k, _, sk = apoe.search(ctx, gc, gq, graph, w3, 128, kg=gkg, kg_weight=40.0)
        # documents of the query's own entities among the top 10: what the logical edges bring in
        q2e_off, q2e_idx, e2d_off, e2d_idx = kg[4].long(), kg[5].long(), kg[2].long(), kg[3].long()
        hits = 0
        for qi in range(nq_truth):
            ents = q2e_idx[q2e_off[qi]:q2e_off[qi + 1]]
            docs = torch.cat([e2d_idx[e2d_off[e]:e2d_off[e + 1]] for e in ents.tolist()]).tolist()
            hits += len(set(docs) & set(ids_k[qi, :10].tolist())) > 0
        kg_search = dict(entities=200_000, cands=128, kg_weight=40.0, kernel_ms=sk.kernel_ms, qps=args.queries / (sk.kernel_ms / 1e3),
                         evaluations=int(sk.evaluations), algo_gbs=sk.algo_bytes / (sk.kernel_ms / 1e3) / 1e9,
                         queries_with_an_entity_document_in_top10=hits / nq_truth)
        log(f"[bench] KG search cands 128: {sk.kernel_ms:.2f} ms, entity document in the top 10 for {hits / nq_truth:.3f} of the queries")
        gkg.close()

    # ---- the reference's own semantics: user weights 1/1/1 go through the query-time calibration (query.cu:1847-1881),
    # ground truth is brute force under the calibrated weights ----
    calibrated = None
    if not args.no_sweeps and not args.calibrate:
        wc = apoe.calibrate_weights(ctx, gc, gq, (1.0, 1.0, 1.0))
        tc, _ = B.hybrid_topk(corpus, queries, wc, 10, nq=nq_truth)
        calibrated = dict(user_weights=(1.0, 1.0, 1.0), effective_weights_dense_sparse_bm25=tuple(float(x) for x in wc), sweep=[])
        for ec in (64, 128, 256):
            apoe.search(ctx, gc, gq, graph, wc, ec)
            ids_c, _, sc = apoe.search(ctx, gc, gq, graph, wc, ec)
            calibrated["sweep"].append(dict(cands=ec, kernel_ms=sc.kernel_ms, qps=args.queries / (sc.kernel_ms / 1e3),
                                            recall_at_10=recall_at_k(ids_c[:nq_truth], tc, 10), algo_gbs=sc.algo_bytes / (sc.kernel_ms / 1e3) / 1e9,
                                            dense_rows_per_evaluation=sc.dense_rows / max(sc.evaluations, 1)))
            log(f"[bench] calibrated weights {tuple(round(float(x), 2) for x in wc)} cands {ec}: {sc.kernel_ms:.2f} ms, recall {calibrated['sweep'][-1]['recall_at_10']:.4f}")

    # ---- the same corpus built with K = 128 lists and degree 64 (the reference's own layout asks for K >= 2 * degree,
    # index.cu:702): build seconds and the recall sweep as a second row beside the configured one ----
    k128 = None
    if not args.no_sweeps and args.nnd_k == 64:
        knn2 = apoe.Knn(ctx, gc, 128, 7.0)
        knn2.set_join(args.join)
        knn2.init(1)
        for it in range(args.nnd_iters):
            knn2.iterate(last=(it == args.nnd_iters - 1))
        nnd2_ms = knn2.elapsed_ms()
        knn2.merge_reverse()
        lists2 = knn2.download()[0]
        knn2.prune(64)
        graph2 = knn2.finalize()
        total2_ms = knn2.elapsed_ms()
        knn2.close()
        k128 = dict(nnd_k=128, degree=64, nnd_iters=args.nnd_iters, build_seconds_gpu=total2_ms / 1e3, nnd_seconds_gpu=nnd2_ms / 1e3,
                    knn_list_recall_at_10=float(np.mean([len(set(lists2[samp_np[i], :10].tolist()) & set(exact[i].tolist())) / 10 for i in range(len(samp_np))])),
                    cands_sweep=[])
        del lists2
        for ec in [int(c) for c in args.cands.split(",")]:
            apoe.search(ctx, gc, gq, graph2, w3, ec, max_iter=iter_cap(ec))
            ids_2, _, s2 = apoe.search(ctx, gc, gq, graph2, w3, ec, max_iter=iter_cap(ec))
            k128["cands_sweep"].append(dict(cands=ec, recall=recall_at_k(ids_2[:nq_truth], truth, 10), ms=s2.kernel_ms, qps=args.queries / (s2.kernel_ms / 1e3),
                                            gbs=s2.algo_bytes / (s2.kernel_ms / 1e3) / 1e9))
        log(f"[bench] K = 128, degree 64: build {total2_ms / 1e3:.2f}s GPU time (NN-Descent {nnd2_ms / 1e3:.2f}s), list recall@10 {k128['knn_list_recall_at_10']:.4f}; " +
            ", ".join(f"cands {x['cands']} recall {x['recall']:.3f} {x['ms']:.1f} ms" for x in k128["cands_sweep"]))
        graph2.close()

    # ---- short batches: the launch shape follows the batch (more waves per query while the whole batch is resident at once) ----
    short_batches = None
    if not args.no_sweeps:
        short_batches = []
        for nq_short in (1, 100, 1000):
            if nq_short > args.queries:
                continue
            apoe.search(ctx, gc, gq, graph, w3, cands, q_count=nq_short)
            ms_short = min(apoe.search(ctx, gc, gq, graph, w3, cands, q_count=nq_short)[2].kernel_ms for _ in range(3))
            short_batches.append(dict(queries=nq_short, cands=cands, kernel_ms=ms_short, qps=nq_short / (ms_short / 1e3)))
            log(f"[bench] {nq_short} queries at cands {cands}: {ms_short:.2f} ms")

    # ---- where the recall target IS reached: the same generators, build and search on smaller corpora ----
    smaller = None
    if not args.no_sweeps:
        smaller = []
        for n_small, deg_small in ((4_000, 32), (30_000, 32), (100_000, 32)):
            if n_small >= args.docs:
                continue
            c_s = gen_corpus(n_small, device=dev)
            gc_s = apoe.Corpus(ctx, *c_s)
            g_s, ms_s = apoe.build_graph(ctx, gc_s, K=args.nnd_k, iters=args.nnd_iters, degree=deg_small, seed=1, join=args.join)
            t_s, _ = B.hybrid_topk(c_s, queries, user_weights, 10, nq=nq_truth)
            row = dict(docs=n_small, degree=deg_small, build_seconds_gpu=ms_s / 1e3, sweep=[], qps_at_recall_target=None, cands_at_recall_target=None)
            for ec in (64, 128, 256, 512, 1024, 2048):
                if ec >= n_small:
                    break
                apoe.search(ctx, gc_s, gq, g_s, user_weights, ec, max_iter=iter_cap(ec))
                ids_s, _, ss = apoe.search(ctx, gc_s, gq, g_s, user_weights, ec, max_iter=iter_cap(ec))
                rec_s = recall_at_k(ids_s[:nq_truth], t_s, 10)
                row["sweep"].append(dict(cands=ec, recall=rec_s, kernel_ms=ss.kernel_ms, qps=args.queries / (ss.kernel_ms / 1e3)))
                if rec_s >= 0.95 and row["cands_at_recall_target"] is None:
                    row["cands_at_recall_target"], row["qps_at_recall_target"] = ec, args.queries / (ss.kernel_ms / 1e3)
                    break
            smaller.append(row)
            log(f"[bench] {n_small} docs, degree {deg_small}: " + ", ".join(f"cands {x['cands']} recall {x['recall']:.3f}" for x in row["sweep"]) +
                (f" -> {row['qps_at_recall_target']:.0f} QPS at recall@10 >= 0.95" if row["qps_at_recall_target"] else " -> target not reached"))
            g_s.close()
            gc_s.close()
            del c_s

    # ---- a corpus of the same size whose rows HAVE neighbours (apoe_synth.latent_corpus: a hidden 16-dimensional vector steers
    # the dense row; terms drawn as in the headline corpus, valued by rarity, the dense part carrying about three quarters of a
    # pair's score), searched under the metric its graph is built for (49 x dense + sparse + bm25, index.cu:836-840); the user
    # weights 1/1/1, raw and through the reference's calibration, beside it ----
    structured = None
    if not args.no_sweeps and not latent:
        c_l = S.latent_corpus(args.docs, device=dev)
        q_l = S.latent_queries(args.queries, device=dev)
        gc_l, gq_l = apoe.Corpus(ctx, *c_l), apoe.Queries(ctx, *q_l)
        g_l, ms_l = apoe.build_graph(ctx, gc_l, K=args.nnd_k, iters=args.nnd_iters, degree=args.degree, seed=1, join=args.join)
        w_l = (49.0, 1.0, 1.0)
        t_l, _ = B.hybrid_topk(c_l, q_l, w_l, 10, nq=nq_truth)
        structured = dict(corpus="apoe_synth.latent_corpus / latent_queries: dense rows with neighbours (16 hidden dimensions + own noise), the headline corpus's "
                                 "terms valued by rarity, all three paths active", docs=args.docs,
                          degree=args.degree, build_seconds_gpu=ms_l / 1e3, weights_dense_sparse_bm25=w_l, weights_are="the build metric",
                          sweep=[], qps_at_recall_target=None, cands_at_recall_target=None, other_weights_at_cands_256=[])
        for ec in (32, 64, 80, 96, 128, 256):
            apoe.search(ctx, gc_l, gq_l, g_l, w_l, ec, max_iter=iter_cap(ec))
            ids_l, _, sl = apoe.search(ctx, gc_l, gq_l, g_l, w_l, ec, max_iter=iter_cap(ec))
            rec_l = recall_at_k(ids_l[:nq_truth], t_l, 10)
            structured["sweep"].append(dict(cands=ec, recall=rec_l, kernel_ms=sl.kernel_ms, qps=args.queries / (sl.kernel_ms / 1e3),
                                            evaluations_per_query=sl.evaluations / args.queries, dense_rows_per_query=sl.dense_rows / args.queries,
                                            algo_gbs=sl.algo_bytes / (sl.kernel_ms / 1e3) / 1e9, frac_of_hbm_peak=sl.algo_bytes / (sl.kernel_ms / 1e3) / 1e9 / HBM_PEAK_GBS))
            if rec_l >= 0.95 and structured["cands_at_recall_target"] is None:
                structured["cands_at_recall_target"], structured["qps_at_recall_target"] = ec, args.queries / (sl.kernel_ms / 1e3)
        if structured["cands_at_recall_target"]:
            # the same walk on half-precision copies of the dense rows, the final pool evaluated again in fp32 (variant | 0x200):
            # here every evaluation reads its dense row, so the narrower row shows
            gc_l.make_half_rows()
            hc = structured["cands_at_recall_target"]
            apoe.search(ctx, gc_l, gq_l, g_l, w_l, hc, max_iter=iter_cap(hc), variant=0x200)
            ids_h, _, sh = apoe.search(ctx, gc_l, gq_l, g_l, w_l, hc, max_iter=iter_cap(hc), variant=0x200)
            structured["half_precision_walk"] = dict(cands=hc, recall=recall_at_k(ids_h[:nq_truth], t_l, 10), kernel_ms=sh.kernel_ms,
                                                     qps=args.queries / (sh.kernel_ms / 1e3), algo_gbs=sh.algo_bytes / (sh.kernel_ms / 1e3) / 1e9)
        for w_o, what in (((1.0, 1.0, 1.0), "1/1/1 as given"), (tuple(float(x) for x in apoe.calibrate_weights(ctx, gc_l, gq_l, (1.0, 1.0, 1.0))), "1/1/1 after the reference's calibration")):
            t_o, _ = B.hybrid_topk(c_l, q_l, w_o, 10, nq=nq_truth)
            ids_o, _, so = apoe.search(ctx, gc_l, gq_l, g_l, w_o, 256)
            structured["other_weights_at_cands_256"].append(dict(weights_dense_sparse_bm25=w_o, what=what, recall=recall_at_k(ids_o[:nq_truth], t_o, 10), kernel_ms=so.kernel_ms))
        log(f"[bench] structured corpus, {args.docs} docs, weights {w_l}: build {ms_l / 1e3:.2f}s, " + ", ".join(f"cands {x['cands']} recall {x['recall']:.3f}" for x in structured["sweep"]) +
            (f" -> {structured['qps_at_recall_target']:.0f} QPS at recall@10 >= 0.95" if structured["qps_at_recall_target"] else " -> target not reached") +
            "; " + ", ".join(f"{x['what']}: {x['recall']:.3f}" for x in structured["other_weights_at_cands_256"]) +
            (f"; half-precision walk at cands {structured['half_precision_walk']['cands']}: recall {structured['half_precision_walk']['recall']:.3f}, "
             f"{structured['half_precision_walk']['qps']:.0f} QPS" if "half_precision_walk" in structured else ""))
        g_l.close()
        gq_l.close()
        gc_l.close()
        del c_l, q_l

    extras = None
    if args.extras:
        extras = {}
        ec = 128
        # the host boundary: the same corpus handed over as host (pageable) buffers, H2D included
        host = S.to_numpy(corpus)
        th = time.perf_counter()
        gch = apoe.Corpus(ctx, *host)
        ctx.synchronize()
        h2d_s = time.perf_counter() - th
        gch.close()
        del host
        extras["corpus handed over as host buffers"] = dict(seconds=h2d_s, gb=gc.bytes() / 1e9, gbs=gc.bytes() / 1e9 / h2d_s)
        log(f"[bench] extras: corpus from host buffers: {h2d_s:.2f}s for {gc.bytes() / 1e9:.2f} GB")
        # a batch four times as long: 10 000 queries are three and a bit rounds of the resident workgroups, and the last
        # round runs on a draining machine
        queries4 = S.queries(4 * args.queries, seed=4321, device=dev)
        torch.cuda.synchronize()
        gq4 = apoe.Queries(ctx, *queries4)
        apoe.search(ctx, gc, gq4, graph, w3, cands, variant=args.variant)
        _, _, s4 = apoe.search(ctx, gc, gq4, graph, w3, cands, variant=args.variant)
        extras[f"{4 * args.queries} queries, cands {cands}"] = dict(kernel_ms=s4.kernel_ms, qps=4 * args.queries / (s4.kernel_ms / 1e3),
                                                                   algo_gbs=s4.algo_bytes / (s4.kernel_ms / 1e3) / 1e9)
        log(f"[bench] extras: {4 * args.queries} queries at cands {cands}: {s4.kernel_ms:.2f} ms = {4 * args.queries / (s4.kernel_ms / 1e3):.0f} QPS, "
            f"{s4.algo_bytes / (s4.kernel_ms / 1e3) / 1e9:.0f} GB/s algorithmic")
        gq4.close()
        del queries4
        # the walk on half-precision dense rows with the final pool evaluated again in fp32 (variant | 0x200)
        gc.make_half_rows()
        for hc, hw in ((ec, w3), (cands, w3), (ec, (1.0, 0.0, 0.0))):
            apoe.search(ctx, gc, gq, graph, hw, hc, variant=0x200 | args.variant)
            ids_h, _, sh = apoe.search(ctx, gc, gq, graph, hw, hc, variant=0x200 | args.variant)
            ids_d, _, sd = apoe.search(ctx, gc, gq, graph, hw, hc, variant=args.variant)
            key_h = f"half-precision rows, weights {hw}, cands {hc}"
            extras[key_h] = dict(kernel_ms=sh.kernel_ms, default_kernel_ms=sd.kernel_ms, same_top10=float((ids_h[:, :10] == ids_d[:, :10]).mean()),
                                 algo_gbs=sh.algo_bytes / (sh.kernel_ms / 1e3) / 1e9)
            log(f"[bench] extras: {key_h}: {sh.kernel_ms:.2f} ms (fp32 rows {sd.kernel_ms:.2f} ms), top-10 ids equal at {extras[key_h]['same_top10']:.4f}")
        # the build with NN-Descent (expansion) steps on the half-precision rows (stored distances recomputed in fp32 before the prune)
        knn_h = apoe.Knn(ctx, gc, args.nnd_k, 7.0)
        knn_h.use_half_rows()
        knn_h.init(20251125)
        for it in range(args.nnd_iters):
            knn_h.iterate(last=(it == args.nnd_iters - 1))
        nnd_h_ms = knn_h.elapsed_ms()
        knn_h.merge_reverse()
        knn_h.prune(args.degree)
        graph_h = knn_h.finalize()
        build_h_ms = knn_h.elapsed_ms()
        knn_h.close()
        ids_gh, _, _ = apoe.search(ctx, gc, gq, graph_h, w3, ec)
        extras["build with half-precision rows"] = dict(build_seconds_gpu=build_h_ms / 1e3, nnd_seconds_gpu=nnd_h_ms / 1e3,
                                                        recall_at_10=recall_at_k(ids_gh[:nq_truth], truth, 10))
        log(f"[bench] extras: build with half-precision rows: {build_h_ms / 1e3:.2f}s (NN-Descent {nnd_h_ms / 1e3:.2f}s); recall@10 at cands {ec}: "
            f"{extras['build with half-precision rows']['recall_at_10']:.4f}")
        graph_h.close()
        # keyword filter: flag the rarest BM25 term of each query (by document frequency)
        qb_off, qb_idx = queries[4].long(), queries[5].long()
        df = torch.bincount(corpus[5].long(), minlength=S.VOCAB)
        cnt = qb_off[1:] - qb_off[:-1]
        rows = torch.repeat_interleave(torch.arange(args.queries, device=dev), cnt)
        f = df[qb_idx].float()
        f[f == 0] = float("inf")
        best = torch.full((args.queries,), float("inf"), device=dev).scatter_reduce(0, rows, f, "amin")
        pos = torch.arange(qb_idx.numel(), device=dev)
        first = torch.full((args.queries,), qb_idx.numel(), device=dev, dtype=torch.long).scatter_reduce(
            0, rows, torch.where(f == best[rows], pos, torch.full_like(pos, qb_idx.numel())), "amin")
        flagged = qb_idx.clone()
        okq = first < qb_idx.numel()
        flagged[first[okq]] |= 0x80000000
        flagged32 = (flagged & 0xFFFFFFFF).to(torch.int64)
        flagged32 = torch.where(flagged32 >= 2 ** 31, flagged32 - 2 ** 32, flagged32).to(torch.int32)
        gqk = apoe.Queries(ctx, *(tuple(queries[:5]) + (flagged32,) + tuple(queries[6:])))
        apoe.search(ctx, gc, gqk, graph, w3, ec, keyword_filter=True)
        ids_k, _, sw = apoe.search(ctx, gc, gqk, graph, w3, ec, keyword_filter=True)
        extras["keyword filter, rarest BM25 term"] = dict(kernel_ms=sw.kernel_ms, qps=args.queries / (sw.kernel_ms / 1e3), evaluations=int(sw.evaluations),
                                                          mean_hits_per_row=float((ids_k != 0x7FFFFFFF).sum(1).mean()),
                                                          algo_gbs=sw.algo_bytes / (sw.kernel_ms / 1e3) / 1e9)
        log(f"[bench] extras: keyword-filter search cands {ec}: {sw.kernel_ms:.2f} ms, {extras['keyword filter, rarest BM25 term']['mean_hits_per_row']:.1f} hits per row")

    if args.copy_calib:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        log("[bench] copy-calib: one 1 GiB device copy issued")
        del src, dst

    # ---- the same search on the host cores (CPU oracle: a reported baseline only) ----
    cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle as O
        ncpu = min(args.cpu_queries, args.queries)
        C_ = O.HybridSet(*S.to_numpy(corpus))
        q_np = S.to_numpy(queries)
        Q_ = O.HybridSet(*q_np).head(ncpu)
        rows, entry = graph.download()
        threads = O.max_threads()  # omp_get_max_threads(): every host core this process is given
        t0 = time.perf_counter()
        oid, odist, _ = O.search(C_, Q_, rows, entry, w3, cands, max_iter=iter_cap(cands) or 1000, threads=threads)
        cpu_s = time.perf_counter() - t0
        agree = float(np.mean(oid[:, :10] == out_ids[:ncpu, :10].cpu().numpy().view(np.uint32)))
        cpu = dict(value=ncpu / cpu_s, unit="queries/s", cores=threads, kind="port",
                   sample=f"first {ncpu} of the {args.queries} queries, same corpus, graph, weights and cands={cands}; "
                          f"{cpu_s:.1f}s on omp_get_max_threads() = {threads} threads (the host shows {os.cpu_count()} logical CPUs); "
                          f"top-10 ids equal to the GPU's at {agree:.4f} of positions")
        log(f"[bench] cpu oracle: {cpu['value']:.0f} QPS on {threads} threads; top-10 agreement {agree:.4f}")

    if ok:
        metric = "search QPS @ recall@10>=0.95 (index build seconds in config)"
    else:
        best = max(sweep, key=lambda s: s["recall"])
        metric = (f"search QPS at cands={cands}, recall@10 {pick['recall']:.3f}: the recall@10>=0.95 point of the configured metric is NOT reached on this corpus "
                  f"(best {best['recall']:.3f} at cands {best['cands']}); index build seconds in config")
        if structured and structured["qps_at_recall_target"]:
            metric += (f"; on a corpus of the same size whose rows have neighbours it is reached at cands {structured['cands_at_recall_target']}: "
                       f"{structured['qps_at_recall_target']:.0f} QPS (config.structured_corpus_same_size)")
    result = {
        "metric": metric,
        "value": args.queries / (ms_per_step / 1e3),
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{args.docs} hybrid docs (dense 1024-d f32 + SPLADE ~120 nnz + BM25 ~60 nnz{'; apoe_synth.latent_corpus: dense rows with neighbours, terms valued by rarity' if latent else ''}), degree {args.degree}, "
                        f"{args.queries} queries, weights dense/sparse/bm25 = {tuple(round(x, 3) for x in w3)}"
                        f"{' (1/1/1 after calibration)' if args.calibrate else ''}, top_k 10",
            "cands": cands,
            "recall_at_10": pick["recall"],
            "recall_target_met": bool(ok),
            "qps_at_recall_target": (args.queries / (ms_per_step / 1e3)) if ok else None,
            "build_seconds_gpu": bt["total_ms"] / 1e3,
            "build_seconds_wall": bt["wall_s"],
            "nnd_step": {0: "expansion (the reference's step)", 1: "local join around the picked neighbour", 2: "local join, both endpoints updated"}[args.join],
            "nnd_k": args.nnd_k,
            "nnd_iters": args.nnd_iters,
            "nnd_leading_expansion_steps": args.nnd_expansion_steps,
            "nnd_seconds_gpu": bt["nnd_ms"] / 1e3,
            "nnd_pair_evaluations": bt["evaluations"],
            "nnd_rows_read": bt["rows_read"],
            "nnd_algo_gbs": bt["algo_bytes"] / (bt["nnd_ms"] / 1e3) / 1e9,
            "knn_list_recall_at_10": bt["knn_list_recall_at_10"],
            **({"build_with_the_reference_expansion_step": {
                "build_seconds_gpu": builds[0]["total_ms"] / 1e3, "nnd_seconds_gpu": builds[0]["nnd_ms"] / 1e3, "nnd_pair_evaluations": builds[0]["evaluations"],
                "nnd_dense_rows_read": builds[0]["rows_read"], "nnd_algo_gbs": builds[0]["algo_bytes"] / (builds[0]["nnd_ms"] / 1e3) / 1e9,
                "knn_list_recall_at_10": builds[0]["knn_list_recall_at_10"]}} if args.join != 0 else {}),
            "cands_sweep": sweep,
            "kernel_ms": avg_kernel_ms,
            **({"weight_sweep_without_rebuild": weight_sweep} if weight_sweep else {}),
            **({"knowledge_graph_search": kg_search} if kg_search else {}),
            **({"reference_semantics_calibrated_weights": calibrated} if calibrated else {}),
            **({"same_corpus_k128_degree64": k128} if k128 else {}),
            **({"short_batches": short_batches} if short_batches else {}),
            **({"same_generators_smaller_corpora": smaller} if smaller else {}),
            **({"structured_corpus_same_size": structured} if structured else {}),
            **({"extras": extras} if extras else {}),
        },
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     # HBM bytes per launch from rocprofv3 counter runs recorded in profiles/ (not measured in this run): null for any other workload
                     "traffic": rec_traffic["default"] if rec_traffic else None,
                     "traffic_source": rec_traffic["source"] if rec_traffic else None,
                     "kernel": "search_kernel", "algo_bytes_per_launch": algo_bytes,
                     "at_recall_target": bool(ok),
                     "mode": "dense row read only when the sparse part plus the bound of the dense part can enter the pool",
                     # the same evaluations priced as the reference prices them (every evaluation reads its dense row), over the
                     # default mode's time: what a kernel without the bound would have to sustain to be as fast
                     "equivalent_if_every_evaluation_read_its_dense_row": {"bytes_per_launch": full_bytes,
                                                                            "gbs": full_bytes / (avg_kernel_ms / 1e3) / 1e9},
                     "every_dense_row_read": full_eval,
                     # what this GPU gives a kernel that does nothing but such loads (bench/membench, run now)
                     "random_read_ceiling": None if args.no_membench else membench()},
        "cpu_baseline": cpu,
    }
    print(json.dumps(result), flush=True)


def membench():
    """GB/s of random 128-byte aligned chunk reads on this GPU, by chunk size, with nothing but the loads in the kernel:
    the ceiling of a gather of records (the search reads about 1.1 KB per evaluation, 5.2 KB when it needs the dense row)."""
    exe = os.path.join(ROOT, "bench", "membench")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe], capture_output=True, text=True, timeout=120).stdout
    except (OSError, subprocess.TimeoutExpired):
        return None
    res = {"unit": "GB/s", "what": "random chunk reads, 3 in flight per wave, 20 waves per CU"}
    for line in out.splitlines():
        m = re.match(r"random reads,\s+(\d+) B chunks, .*:\s+(\d+) GB/s", line)
        if m:
            res[f"{m.group(1)}B"] = float(m.group(2))
        m = re.match(r"random reads,\s+(\d+) B chunks \+ ([\d.]+) returning atomics per chunk:\s+(\d+) GB/s", line)
        if m:
            res[f"{m.group(1)}B+{m.group(2)}atomics"] = float(m.group(3))
        log("[bench] " + line)
    return res


if __name__ == "__main__":
    main()
