"""The benchmark configurations as parity cases: config 2 (the headline: 1M x 200, the builder's graph from 100 000
auxiliary queries, k=100, L in {256, 512} and the beam at which recall@100 reaches 0.90, all 10 000 queries in one batch),
config 1 (100k x 128, exact 32-NN graph, k=10, L=64: the reference's CPU-runnable case),
config 3 (inner product, 1M x 512, k=100, L=256), config 4 (10M x 200, batch sweep) and
config 5 (100M x 200 with 10 % tombstones; skipped where memory is short).
Configs 2-4 search graphs made by the library's own builder from 100 000 auxiliary queries; config 5 uses a
cheap block graph (coral_amd.synth.block_graph; building for 100M nodes would take several minutes): it checks
parity and size handling, not recall."""
import os
import time

import numpy as np
import pytest

from coral_amd import capi, synth, workloads

pytestmark = pytest.mark.gpu
WAVE64 = 3


def check_basic(ids, dists, n, k, larger_is_closer=False):
    assert ((ids >= 0) & (ids < n)).all()
    d = np.diff(dists, axis=1)
    assert (d <= 0).all() if larger_is_closer else (d >= 0).all()
    assert all(len(set(r.tolist())) == k for r in ids[:: max(1, len(ids) // 64)])


def test_config1_reference_cpu_case(orc):
    w = workloads.config1()
    base, q, nbrs, starts, k, L = w["base"], w["queries"], w["nbrs"], w["starts"], 10, 64
    assert starts.size == 1 and (nbrs >= 0).all()
    idx = capi.Index(base, nbrs, starts)
    prob = orc.Problem(base, nbrs, starts)
    gt, _ = orc.bruteforce(base, q, k)
    # the rounds policy: exact against the same-order oracle, tolerance against the reference orders
    ids, dists, st = idx.search(q, k, L)
    cnt = idx.query_counters(q.shape[0])
    oi, od, os_, _ = orc.search_B(prob, q, k, L, start_order=WAVE64, nbr_order=WAVE64)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes() and np.array_equal(cnt, os_)
    ri, rd, _, _ = orc.search_B(prob, q, k, L)
    assert (np.abs(dists - rd)[ids == ri] <= 1e-5 * rd[ids == ri]).all()
    assert (ids == ri).all(1).mean() >= 0.99
    print("config1 rounds: %.0f QPS, recall@10 %.4f" % (q.shape[0] / st.time_s,
                                                          orc.recall_hits(ids, gt, k) / gt.size), flush=True)
    # the reference runs this configuration on its CPU path: best-first, M = 1, AVX-512 order
    ids, dists, st = idx.search(q, k, L, policy=capi.POLICY_BEST_FIRST)
    cnt = idx.query_counters(q.shape[0])
    oi, od, os_, _ = orc.search_A(prob, q, k, L, order=WAVE64)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes() and np.array_equal(cnt, os_)
    ci, cd, cs, _ = orc.search_A(prob, q, k, L)  # the reference's own summation order
    assert (np.abs(dists - cd)[ids == ci] <= 1e-5 * cd[ids == ci]).all()
    assert (ids == ci).all(1).mean() >= 0.99
    r_gpu = orc.recall_hits(ids, gt, k) / gt.size
    r_cpu = orc.recall_hits(ci, gt, k) / gt.size
    assert abs(r_gpu - r_cpu) <= 1e-3
    print("config1 best-first: %.0f QPS, recall@10 %.4f (cpu order %.4f)" % (q.shape[0] / st.time_s, r_gpu, r_cpu),
          flush=True)
    idx.close()


# totals over the 10 000 queries of configuration 2, as bench.py reports them per query (x 10 000): the workload is
# seeded and the traversal is deterministic, so these are constants of the build
CONFIG2_COUNTERS = {  # (policy, L): (expansions, distance evaluations)
    (0, 256): (6488806, 177671509),
    (0, 512): (13082353, 332139154),
    (0, 13312): (306488765, 3472320309),
    (1, 256): (2692843, 77838276),
    (1, 512): (5221889, 144803048),
}


def test_config2_headline_workload(orc):
    """BASELINE's configuration 2 as bench.py runs it (tests/test_search_pipeline.cpp:283-314 of the reference: one
    Search call per L over the whole query file): the graph built by the library's construction path from 100 000
    auxiliary queries, M = 16 entry points from it, all 10 000 queries in one batch, both traversals at L = 256 and
    512 and the expand-all traversal at the beam where bench.py quotes its headline."""
    from util import explain_divergence, near_tie_equal
    w = workloads.config2()
    base, q, nbrs, starts, k = w["base"], w["queries"], w["nbrs"], w["starts"], 100
    n, Q = base.shape[0], q.shape[0]
    assert starts.size == 16 and (nbrs[:, 0] >= 0).all()
    idx = capi.Index(base, nbrs, starts)
    gt, _, _ = idx.bruteforce(q, k, want_dists=False)
    prob = orc.Problem(base, nbrs, starts)
    sub = np.arange(0, Q, 157)  # 64 queries
    kept = {}
    for policy, Ls in ((capi.POLICY_ROUNDS, (256, 512, 13312)), (capi.POLICY_BEST_FIRST, (256, 512))):
        for L in Ls:
            ids, dists, st = idx.search(q, k, L, policy=policy)
            cnt = idx.query_counters(Q)
            kept[(policy, L)] = (ids, dists)
            check_basic(ids, dists, n, k)
            for qi in range(0, Q, 1250):  # the distances are the distances of the ids
                want = ((base[ids[qi]].astype(np.float64) - q[qi].astype(np.float64)) ** 2).sum(1)
                assert np.allclose(dists[qi], want, rtol=1e-5)
            # the totals bench.py divides by Q are the sums of the per-query counters, and constants of the workload
            assert st.expansions == int(cnt[:, 1].astype(np.int64).sum())
            assert st.dist_evals == int(cnt[:, 2].astype(np.int64).sum())
            recall = orc.recall_hits(ids, gt, k) / float(Q * k)
            print("config2 policy %d L=%d: recall@100 %.4f, %.0f QPS, expansions %d, distance evaluations %d, spills %d"
                  % (policy, L, recall, Q / st.kernel_s, st.expansions, st.dist_evals, st.spills), flush=True)
            if (policy, L) in CONFIG2_COUNTERS:
                assert (st.expansions, st.dist_evals) == CONFIG2_COUNTERS[(policy, L)]
            # exact parity on the stride: ids, distance bits, the four counters
            if policy == capi.POLICY_ROUNDS:
                oi, od, os_, _ = orc.search_B(prob, q[sub], k, L, start_order=WAVE64, nbr_order=WAVE64)
                ri, rd, _, _ = orc.search_B(prob, q[sub], k, L)
            else:
                oi, od, os_, _ = orc.search_A(prob, q[sub], k, L, order=WAVE64)
                ri, rd, _, _ = orc.search_A(prob, q[sub], k, L)
            assert np.array_equal(ids[sub], oi) and dists[sub].tobytes() == od.tobytes()
            assert np.array_equal(cnt[sub], os_)
            # against the reference's summation orders: 1e-5 on distances, id lists up to near-tie swaps, recall 0.1 %
            same = ids[sub] == ri
            assert (np.abs(dists[sub] - rd)[same] <= 1e-5 * rd[same]).all()
            bad = [int(sub[i]) for i in range(len(sub)) if not near_tie_equal(ids[sub[i]], dists[sub[i]], ri[i], rd[i])]
            print("  queries of the stride beyond the near-tie rule: %d of %d %s" % (len(bad), len(sub), bad), flush=True)
            # a query beyond the rule must be one whose traversal parts from the reference order's at a pair of nodes
            # within 1e-6 of each other (everything after such a step may differ); shown by replaying both traversals,
            # which the long beam does not afford: none is accepted there
            assert len(bad) == 0 or L <= 512
            if L <= 512:
                for qi in bad:
                    why = explain_divergence(orc, base, nbrs, starts, q[qi], orc.L2, policy, L, k)
                    print("  query %d parts at step %s: %s" % (qi, why and why[0], why and why[1]), flush=True)
                    assert why is not None and all(gap < 1e-6 for _, _, gap in why[1]), why
            r_gpu = orc.recall_hits(ids[sub], gt[sub], k) / float(len(sub) * k)
            r_ref = orc.recall_hits(ri, gt[sub], k) / float(len(sub) * k)
            assert abs(r_gpu - r_ref) <= 1e-3
            if L == 13312:
                assert recall >= 0.90  # the metric's operating point (bench.py finds the same L)
    # size-independent properties on the whole batch: the same call returns the same bytes, a permutation of the
    # batch permutes the answers, a query's answer does not depend on the batch it travels in
    ids, dists = kept[(capi.POLICY_ROUNDS, 256)]
    ids2, dists2, _ = idx.search(q, k, 256)
    assert np.array_equal(ids, ids2) and dists.tobytes() == dists2.tobytes()
    perm = np.random.RandomState(0).permutation(Q)
    ids3, _, _ = idx.search(q[perm], k, 256)
    assert np.array_equal(ids3, ids[perm])
    ids4, dists4, _ = idx.search(q[:777], k, 256)
    assert np.array_equal(ids4, ids[:777]) and dists4.tobytes() == dists[:777].tobytes()
    # the screening of rows on a smaller copy changes no byte of the whole batch's answer and no counter: without it,
    # in half precision and on eight-bit codes (the library's choice above), at the configuration's beam and at the
    # headline's; best-first likewise
    for policy, L in ((capi.POLICY_ROUNDS, 512), (capi.POLICY_ROUNDS, 13312), (capi.POLICY_BEST_FIRST, 512)):
        ids, dists = kept[(policy, L)]
        idx.prepare(Q, L, policy=policy)
        idx.search(q, k, L, policy=policy)
        cnt = idx.query_counters(Q)
        for screening in (-1, 1):
            idx.prepare(Q, L, policy=policy, screening=screening)
            ids5, dists5, _ = idx.search(q, k, L, policy=policy)
            assert np.array_equal(ids5, ids) and dists5.tobytes() == dists.tobytes(), (policy, L, screening)
            assert np.array_equal(idx.query_counters(Q), cnt), (policy, L, screening)
    idx.close()


# the same for the graph of the reference's shipped config.json ("top_hit_num": 5000000): totals over the 10 000 queries
SHIPPED_GRAPH_COUNTERS = {  # L: (expansions, distance evaluations)
    512: (13294172, 244437655),
    22528: (426698680, 2746117307),
}
SHIPPED_GRAPH_RECALL_BEAM = 22528  # the smallest multiple of 512 with recall@100 >= 0.90 on that graph (bench.py's leg)


def test_config2_on_the_graph_of_the_shipped_config(orc):
    """Configuration 2 on the graph that the reference's build driver makes with the config.json it ships:
    "top_hit_num": 5000000 (read at src/index_gpu.cpp:78) sends the most-hit nodes through a second search-and-rewire
    pass after the isolated ones (src/enhance.cu:819-856; capped at n here, where the reference reads past its id
    array).  The headline's graph is built with the code's default of 0.  Expand-all rounds at the configuration's
    L = 512 and at the beam where this graph reaches recall@100 >= 0.90: a 64-query stride exact against the oracle
    (ids, distance bits, counters), the reference's summation orders within the contract's tolerances, the totals
    pinned as constants of the workload."""
    from util import near_tie_equal
    w = workloads.config2()
    base, q, k = w["base"], w["queries"], 100
    nbrs, starts, info = workloads.build_query_aware_graph(base, w["aux"], "l2", top_hit_num=5000000)
    print("shipped-config graph:", info, flush=True)
    assert info["top_hit_nodes"] > 0 and not np.array_equal(nbrs, w["nbrs"])
    n, Q = base.shape[0], q.shape[0]
    idx = capi.Index(base, nbrs, starts)
    gt, _, _ = idx.bruteforce(q, k, want_dists=False)
    prob = orc.Problem(base, nbrs, starts)
    sub = np.arange(0, Q, 157)  # 64 queries
    for L in (512, SHIPPED_GRAPH_RECALL_BEAM):
        ids, dists, st = idx.search(q, k, L)
        cnt = idx.query_counters(Q)
        check_basic(ids, dists, n, k)
        recall = orc.recall_hits(ids, gt, k) / float(Q * k)
        print("shipped-config graph L=%d: recall@100 %.4f, %.0f QPS, expansions %d, distance evaluations %d"
              % (L, recall, Q / st.kernel_s, st.expansions, st.dist_evals), flush=True)
        assert st.expansions == int(cnt[:, 1].astype(np.int64).sum())
        assert st.dist_evals == int(cnt[:, 2].astype(np.int64).sum())
        if L in SHIPPED_GRAPH_COUNTERS:
            assert (st.expansions, st.dist_evals) == SHIPPED_GRAPH_COUNTERS[L]
        oi, od, os_, _ = orc.search_B(prob, q[sub], k, L, start_order=WAVE64, nbr_order=WAVE64)
        assert np.array_equal(ids[sub], oi) and dists[sub].tobytes() == od.tobytes()
        assert np.array_equal(cnt[sub], os_)
        ri, rd, _, _ = orc.search_B(prob, q[sub], k, L)
        same = ids[sub] == ri
        assert (np.abs(dists[sub] - rd)[same] <= 1e-5 * rd[same]).all()
        bad = [int(sub[i]) for i in range(len(sub)) if not near_tie_equal(ids[sub[i]], dists[sub[i]], ri[i], rd[i])]
        print("  queries of the stride beyond the near-tie rule: %d of %d %s" % (len(bad), len(sub), bad), flush=True)
        assert len(bad) == 0
        r_gpu = orc.recall_hits(ids[sub], gt[sub], k) / float(len(sub) * k)
        r_ref = orc.recall_hits(ri, gt[sub], k) / float(len(sub) * k)
        assert abs(r_gpu - r_ref) <= 1e-3
        if L == SHIPPED_GRAPH_RECALL_BEAM:
            assert recall >= 0.90
            # ... and it is the smallest such beam
            ids_b, _, _ = idx.search(q, k, L - 512)
            assert orc.recall_hits(ids_b, gt, k) / float(Q * k) < 0.90
    idx.close()


def test_structured_data_reaches_the_recall_the_metric_names(orc):
    """On data with neighbourhood structure (points near an 8-dimensional subspace) the built graph and both
    traversals reach recall@100 >= 0.90, which the isotropic configurations cannot; parity with the oracle holds
    there as everywhere (a sample of queries, exact)."""
    w = workloads.structured(n=200000, dim=64, latent=8, Q=2000, A=20000)
    base, q, nbrs, starts, k = w["base"], w["queries"], w["nbrs"], w["starts"], 100
    idx = capi.Index(base, nbrs, starts)
    gt, _, _ = idx.bruteforce(q, k, want_dists=False)
    prob = orc.Problem(base, nbrs, starts)
    for policy, L in ((capi.POLICY_ROUNDS, 256), (capi.POLICY_BEST_FIRST, 512)):
        ids, dists, st = idx.search(q, k, L, policy=policy)
        recall = orc.recall_hits(ids, gt, k) / gt.size
        print("structured policy %d L=%d: recall@100 %.4f, %.0f QPS" % (policy, L, recall, q.shape[0] / st.kernel_s),
              flush=True)
        assert recall >= 0.90
        if policy == capi.POLICY_ROUNDS:
            oi, od, _, _ = orc.search_B(prob, q[:200], k, L, start_order=WAVE64, nbr_order=WAVE64)
        else:
            oi, od, _, _ = orc.search_A(prob, q[:200], k, L, order=WAVE64)
        assert np.array_equal(ids[:200], oi) and dists[:200].tobytes() == od.tobytes()
    idx.close()


def test_config3_inner_product_1m_x_512(orc):
    t0 = time.time()
    w = workloads.config3()
    base, q, nbrs, starts, k, L = w["base"], w["queries"], w["nbrs"], w["starts"], 100, 256
    print("config3 prepared in %.0f s: %s" % (time.time() - t0, w["build"]), flush=True)
    n = base.shape[0]
    idx = capi.Index(base, nbrs, starts, capi.IP)
    ids, dists, st = idx.search(q, k, L)
    cnt = idx.query_counters(q.shape[0])
    check_basic(ids, dists, n, k, larger_is_closer=True)
    for qi in range(0, q.shape[0], 1001):  # returned value = raw inner product of the returned id
        want = base[ids[qi]].astype(np.float64) @ q[qi].astype(np.float64)
        assert np.allclose(dists[qi], want, rtol=1e-5, atol=1e-6)
    sub = np.arange(0, q.shape[0], 211)
    prob = orc.Problem(base, nbrs, starts)
    oi, od, os_, _ = orc.search_B(prob, q[sub], k, L, metric=orc.IP, start_order=WAVE64, nbr_order=WAVE64)
    assert np.array_equal(ids[sub], oi) and dists[sub].tobytes() == od.tobytes() and np.array_equal(cnt[sub], os_)
    ri, rd, _, _ = orc.search_B(prob, q[sub], k, L, metric=orc.IP)
    same = ids[sub] == ri
    assert (np.abs(dists[sub] - rd)[same] <= 1e-5 * np.abs(rd[same])).all()
    gt = workloads.ground_truth(base, q[sub], k, "ip")
    r_gpu = orc.recall_hits(ids[sub], gt, k) / gt.size
    r_ref = orc.recall_hits(ri, gt, k) / gt.size
    assert abs(r_gpu - r_ref) <= 1e-3
    B = st.expansions * 128 + st.dist_evals * 2048 + q.shape[0] * (2048 + k * 8)
    print("config3: %.0f QPS, %.0f GB/s algorithmic, recall@100 %.4f, %.0f distance evaluations/query" %
          (q.shape[0] / st.kernel_s, B / st.kernel_s / 1e9, r_gpu, st.dist_evals / q.shape[0]), flush=True)
    idx.close()


def big_case(orc, n, dim, Qs, L, k, tomb_seed=None, built=False):
    t0 = time.time()
    base = workloads.gaussian_base(4001 if n <= 10 ** 7 else 5001, n, dim)
    print("generated %d x %d in %.0f s" % (n, dim, time.time() - t0), flush=True)
    if built:
        aux = synth.shifted_queries(100000, dim, 2002, 2003, 2005)
        nbrs, starts, info = workloads.build_query_aware_graph(base, aux, "l2")
        assert (nbrs[:, 0] >= 0).all()  # the enhancement left no node without neighbours
        print("built graph at %.0f s: %s" % (time.time() - t0, info), flush=True)
    else:
        nbrs = synth.block_graph(base, 32)
        print("block graph at %.0f s" % (time.time() - t0), flush=True)
        starts = (np.arange(16, dtype=np.int64) * (n // 16) + 5).astype(np.int32)
    q = synth.shifted_queries(max(Qs), dim, 2002, 2003, 2004)
    idx = capi.Index(base, nbrs, starts)
    mask = None
    if tomb_seed is not None:
        mask = synth.tombstone_mask(n, tomb_seed, 10)
        idx.set_deleted(mask)
    print("index resident at %.0f s" % (time.time() - t0), flush=True)
    results = {}
    for Q in Qs:
        ids, dists, st = idx.search(q[:Q], k, L, have_delete=mask is not None)
        results[Q] = (ids, dists, idx.query_counters(Q))
        check_basic(ids, dists, n, k)
        B = st.expansions * 128 + st.dist_evals * dim * 4 + Q * (dim * 4 + k * 8)
        print("n=%d Q=%d: %.0f QPS, %.0f GB/s algorithmic, %d spills" %
              (n, Q, Q / st.kernel_s, B / st.kernel_s / 1e9, st.spills), flush=True)
        # beyond 2^24 ids too the visited set of nearly every query stays in LDS: the library sizes the table of
        # 16-bit cells for the displacement a cell has to carry, not for the load alone
        assert st.spills * 20 <= Q or n <= (1 << 24)
    # a query's answer does not depend on the batch it travels in
    small = min(Qs)
    for Q in Qs:
        assert np.array_equal(results[Q][0][:small], results[small][0])
        assert results[Q][1][:small].tobytes() == results[small][1].tobytes()
    ids, dists, cnt = results[small]
    sub = np.arange(0, small, max(1, small // 48))
    prob = orc.Problem(base, nbrs, starts, mask)
    oi, od, os_, _ = orc.search_B(prob, q[sub], k, L, start_order=WAVE64, nbr_order=WAVE64)
    assert np.array_equal(ids[sub], oi) and dists[sub].tobytes() == od.tobytes() and np.array_equal(cnt[sub], os_)
    if mask is not None:
        dead = (mask[ids >> 5] >> (ids & 31).astype(np.uint32)) & 1
        assert not dead.any()
    # the CPU path's traversal at this size (a wavefront per query while n bytes per query slot fit the memory
    # budget, else a workgroup per query)
    Qb = min(max(Qs), 10000)
    ids, dists, st = idx.search(q[:Qb], k, L, policy=capi.POLICY_BEST_FIRST, have_delete=mask is not None)
    cnt = idx.query_counters(Qb)
    B = st.expansions * 128 + st.dist_evals * dim * 4 + Qb * (dim * 4 + k * 8)
    print("n=%d Q=%d best-first: %.0f QPS, %.0f GB/s algorithmic" % (n, Qb, Qb / st.kernel_s, B / st.kernel_s / 1e9),
          flush=True)
    sub = np.arange(0, Qb, max(1, Qb // 48))
    oi, od, os_, _ = orc.search_A(prob, q[sub], k, L, order=WAVE64)
    assert np.array_equal(ids[sub], oi) and dists[sub].tobytes() == od.tobytes() and np.array_equal(cnt[sub], os_)
    idx.close()


def test_config4_10m_batch_sweep(orc):
    big_case(orc, 10 ** 7, 200, (1000, 10000, 100000), 256, 100, built=True)


def _mem_available_gib():
    try:
        for line in open("/proc/meminfo"):
            if line.startswith("MemAvailable:"):
                return int(line.split()[1]) / (1 << 20)
    except OSError:
        pass
    return 0.0


def test_config5_100m_tombstones(orc):
    """80 GB of vectors + 12.8 GB of graph rows resident in HBM, 10 % of the ids tombstoned.
    About a minute on an MI355X box; skipped where host or device memory cannot hold it."""
    import torch
    if os.environ.get("CORAL_SKIP_100M") == "1":
        pytest.skip("CORAL_SKIP_100M=1")
    if _mem_available_gib() < 130:
        pytest.skip("needs about 100 GB of host memory")
    free, _ = torch.cuda.mem_get_info()
    if free < 120 * (1 << 30):
        pytest.skip("needs about 105 GB of device memory")
    big_case(orc, 10 ** 8, 200, (1000, 100000), 256, 100, tomb_seed=5002)
