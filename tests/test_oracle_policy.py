"""Pins the oracle's two traversal policies.

Policy A (best-first, src/search_in_cpu.cpp:23-119): bit equality with the
reference's own queue + distance compiled in place, the committed golden
fixtures written from it, and the invariants below.
Policy B (expand-all rounds, src/search_gpu.cu:347-580): nothing executable
exists for the reference, so it is pinned by what the algorithm fixes: exact kNN
on complete graphs and for L >= N, hand-computed traversals on ring graphs, the
top-L-of-visited invariant, and an independent pure-Python simulator.
"""
import json
import os

import numpy as np
import pytest

import pysim
from util import digest, make_problem, make_queries, ragged, rounds_hand_case

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def signed(orc, q, base, metric, order):
    out = {}
    for i in range(base.shape[0]):
        d = orc.dist(q, base[i], metric, order)
        out[i] = float(np.float32(0.0) - np.float32(d)) if metric == orc.IP else d
    return out


# ----------------------------------------------------------------- policy A

@pytest.mark.parametrize("L,k,M", [(8, 4, 1), (32, 10, 4), (64, 64, 4)])
def test_policy_a_equals_reference_harness(orc, ref, L, k, M):
    base, nbrs, starts = make_problem(600, 36, 12, seed=21, n_start=4, ragged_seed=5)
    q = make_queries(25, 36, 90)
    prob = orc.Problem(base, nbrs, starts)
    a = orc.search_A(prob, q, k, L, M=M)
    b = orc.ref_search_in_cpu(prob, q, k, L, M=M)
    assert np.array_equal(a[0], b[0])
    assert a[1].tobytes() == b[1].tobytes()
    assert np.array_equal(a[2], b[2])


def test_best_first_hand_case_on_the_reference_queue(orc, ref):
    """The hand-worked line of util.rounds_hand_case under the reference's own queue and distance: the answer
    that differs from the rounds policy's (6 instead of 4) is the reference's, not a slip of the restatement."""
    base, nbrs, starts, q, L, k, _ = rounds_hand_case()
    ids, dists, stats, _ = orc.ref_search_in_cpu(orc.Problem(base, nbrs, starts), q, k, L)
    assert ids[0].tolist() == [10, 5, 6] and dists[0].tolist() == [1.0, 36.0, 56.25]
    assert stats[0, :3].tolist() == [1 + 5, 5, 7]


def golden_cases():
    return sorted(f for f in os.listdir(GOLDEN) if f.startswith("policyA_") and f.endswith(".json"))


@pytest.mark.parametrize("name", golden_cases())
def test_policy_a_golden(orc, name):
    case = json.load(open(os.path.join(GOLDEN, name)))
    base, nbrs, starts, q = golden_inputs(case)
    assert digest(base, nbrs, starts, q) == case["input_sha256"]
    prob = orc.Problem(base, nbrs, starts)
    ids, dists, stats, _ = orc.search_A(prob, q, case["k"], case["L"], M=case["M"])
    assert ids.tolist() == case["ids"]
    assert dists.view(np.uint32).tolist() == case["dist_bits"]
    assert stats.tolist() == case["stats"]


def golden_inputs(case):
    if case["kind"] == "gauss":
        base, nbrs, starts = make_problem(case["n"], case["dim"], case["R"], case["seed"],
                                          n_start=case["n_start"], ragged_seed=case.get("ragged_seed"))
        q = make_queries(case["Q"], case["dim"], case["seed"] + 50)
    else:  # integer lattice: many exact distance ties
        side, dim = case["side"], case["dim"]
        grid = np.stack(np.meshgrid(*[np.arange(side)] * dim, indexing="ij"), -1).reshape(-1, dim)
        base = grid.astype(np.float32)
        from coral_amd import synth
        nbrs = synth.exact_knn_graph(base, case["R"])
        starts = np.array(case["starts"], np.int32)
        q = (np.array(case["queries"], np.float32))
    return base, nbrs, starts, q


@pytest.mark.parametrize("policy", ["A", "B"])
@pytest.mark.parametrize("metric", ["l2", "ip"])
def test_traversal_equals_python_simulator(orc, policy, metric):
    m = orc.IP if metric == "ip" else orc.L2
    base, nbrs, starts = make_problem(60, 8, 6, seed=3, metric=metric, n_start=3, ragged_seed=9)
    q = make_queries(6, 8, 40, metric)
    dele = np.zeros(2, np.uint32)
    for i in (1, 5, 17, 33, 40):
        dele[i >> 5] |= np.uint32(1 << (i & 31))
    for use_del in (False, True):
        prob = orc.Problem(base, nbrs, starts, dele if use_del else None)
        dset = frozenset((1, 5, 17, 33, 40)) if use_del else frozenset()
        for L, k in ((4, 2), (8, 8), (16, 5), (64, 10)):
            if policy == "A":
                ids, dists, stats, _ = orc.search_A(prob, q, k, L, metric=m, order=0)
            else:
                ids, dists, stats, _ = orc.search_B(prob, q, k, L, metric=m, start_order=0, nbr_order=0)
            for qi in range(q.shape[0]):
                dist = signed(orc, q[qi], base, m, 0)
                sim = (pysim.policy_best_first if policy == "A" else pysim.policy_rounds)(
                    nbrs.tolist(), starts.tolist(), dist, L, k, dset)
                assert ids[qi].tolist() == sim[0], (policy, metric, use_del, L, k, qi)
                assert stats[qi, 0] == sim[1] and stats[qi, 1] == sim[2] and stats[qi, 2] == sim[3]


# ----------------------------------------------------------------- both policies

def complete_graph(n):
    g = np.empty((n, n - 1), np.int32)
    for i in range(n):
        g[i] = [j for j in range(n) if j != i]
    return g


@pytest.mark.parametrize("metric", ["l2", "ip"])
def test_complete_graph_gives_exact_knn(orc, metric):
    m = orc.IP if metric == "ip" else orc.L2
    n, dim = 24, 12
    from coral_amd import synth
    base = synth.gaussian_matrix(5, n, dim)
    q = make_queries(10, dim, 60, metric)
    if metric == "ip":
        base = synth.normalize_rows(base)
    prob = orc.Problem(base, complete_graph(n), np.array([0], np.int32))
    gt, gd = orc.bruteforce(base, q, 5, m)
    for ids, dists in (orc.search_B(prob, q, 5, 8, metric=m)[:2], orc.search_A(prob, q, 5, 8, metric=m, order=0)[:2]):
        assert np.array_equal(ids, gt)
        assert np.allclose(dists, gd, rtol=1e-5)


def test_beam_not_smaller_than_component_gives_exact_knn_of_component(orc):
    base, nbrs, starts = make_problem(120, 16, 8, seed=8, n_start=2)
    q = make_queries(8, 16, 70)
    prob = orc.Problem(base, nbrs, starts)
    for fn in (lambda: orc.search_B(prob, q, 10, 128), lambda: orc.search_A(prob, q, 10, 128, order=0)):
        ids, dists, stats, _ = fn()
        # reachable set by BFS
        seen, todo = set(starts.tolist()), list(starts.tolist())
        while todo:
            v = todo.pop()
            for w in nbrs[v]:
                if w >= 0 and w not in seen:
                    seen.add(int(w))
                    todo.append(int(w))
        comp = np.array(sorted(seen))
        gt, _ = orc.bruteforce(base[comp], q, 10)
        assert np.array_equal(ids, comp[gt])
        assert (stats[:, 2] == len(comp)).all()  # every reachable node measured exactly once


def test_ring_graph_hand_computed(orc):
    # nodes 0..9 on a line at x = id, each linked to id-1 and id+1 (ring); query at x = 6.2;
    # start at node 0, L = 3.
    n = 10
    base = np.zeros((n, 4), np.float32)
    base[:, 0] = np.arange(n)
    nbrs = np.stack([(np.arange(n) - 1) % n, (np.arange(n) + 1) % n], 1).astype(np.int32)
    q = np.zeros((1, 4), np.float32)
    q[0, 0] = 6.2
    prob = orc.Problem(base, nbrs, np.array([0], np.int32))
    # policy B by hand: round 1 expands 0 -> {9, 1}; beam {9(7.84), 1(27.04), 0(38.44)}
    # round 2 expands 9, 1 -> {8, 2}: overflow, beam {8, 9, 2}... continues until 6,7,5 hold.
    ids, dists, stats, _ = orc.search_B(prob, q, 3, 3, start_order=0, nbr_order=0)
    assert ids[0].tolist() == [6, 7, 5]
    assert np.allclose(dists[0], [0.04, 0.64, 1.44], rtol=1e-5)
    # rounds: r1 {9,1} r2 {8,2} r3 {7,3->rejected? 3 is at 10.24 < thr} ...
    # every node is visited exactly once on a ring: the two search fronts meet
    assert stats[0, 2] <= n
    # policy A by hand: expands 0, 9, 8, 7, 6, 5 (then 4 is visited but not closer than the beam)
    ids, dists, stats, _ = orc.search_A(prob, q, 3, 3, order=0)
    assert ids[0].tolist() == [6, 7, 5]
    # expansions: 0,9,8,7,6,5 and then 4? no: after 6,7,5 are in the beam and expanded the
    # queue holds no unexpanded entry.  0->9,1; 9->8; 8->7; 7->6; 6->5; 5->4(rejected): 6 expansions
    assert stats[0, 1] == 6 and stats[0, 0] == 1 + 6
    assert stats[0, 2] == 8  # 0,9,1,8,7,6,5,4


def test_rounds_policy_hand_computed_counters(orc):
    """Every counter of a traversal worked out by hand (util.rounds_hand_case): the threshold that is not tightened
    when an append fills the beam exactly, the threshold frozen inside a round, the strict comparison, the start id
    that is not a hop -- each of them changes `hops` if it is restated wrongly."""
    base, nbrs, starts, q, L, k, want = rounds_hand_case()
    prob = orc.Problem(base, nbrs, starts)
    for order in (0, 1, 2, 3):
        ids, dists, stats, _ = orc.search_B(prob, q, k, L, start_order=order, nbr_order=order)
        assert ids[0].tolist() == want["ids"] and dists[0].tolist() == want["dists"]
        assert stats[0].tolist() == [want["hops"], want["expansions"], want["dist_evals"], want["rounds"]]
    dist = {i: float(x) ** 2 for i, x in enumerate(base[:, 2])}
    sim = pysim.policy_rounds(nbrs.tolist(), starts.tolist(), dist, L, k)
    assert sim == (want["ids"], want["hops"], want["expansions"], want["dist_evals"])
    # node 5 tombstoned (src/search_gpu.cu:695-725): the traversal and its counters are untouched, the output
    # skips 5 and, the beam exhausted, ends in id -1 with the farthest distance
    dead = orc.Problem(base, nbrs, starts, deleted=np.array([1 << 5], np.uint32))
    ids, dists, stats, _ = orc.search_B(dead, q, k, L, start_order=0, nbr_order=0)
    assert ids[0].tolist() == [10, 4, -1] and dists[0].tolist() == [1.0, 49.0, float(np.finfo(np.float32).max)]
    assert stats[0].tolist() == [want["hops"], want["expansions"], want["dist_evals"], want["rounds"]]
    # the same points under best-first: 0 -> 1, 2; 2 -> 5 (0 leaves the queue); 5 -> 6, 7 (1 and 2 leave);
    # 6 -> 10 (7 leaves, unexpanded); 10 -> nothing new.  Five expansions, seven distances, and a different
    # answer: 4 is never reached, because 1, the only way to it, was dropped unexpanded.
    ids, dists, stats, _ = orc.search_A(prob, q, k, L, order=0)
    assert ids[0].tolist() == [10, 5, 6] and dists[0].tolist() == [1.0, 36.0, 56.25]
    assert stats[0, :3].tolist() == [1 + 5, 5, 7]


@pytest.mark.parametrize("policy", ["A", "B"])
def test_result_is_top_k_of_top_L_of_visited(orc, policy):
    """Invariant: the result equals the k closest of everything whose distance was
    evaluated (the beam can only drop an entry in favour of a closer one)."""
    base, nbrs, starts = make_problem(400, 20, 10, seed=13, n_start=3, ragged_seed=2)
    q = make_queries(12, 20, 80)
    prob = orc.Problem(base, nbrs, starts)
    L, k = 24, 24
    if policy == "A":
        ids, dists, stats, _ = orc.search_A(prob, q, k, L, order=0)
    else:
        ids, dists, stats, _ = orc.search_B(prob, q, k, L, start_order=0, nbr_order=0)
    for qi in range(q.shape[0]):
        # replay: visited = starts + neighbours of every expanded node; a node is expanded
        # only if it was in the beam, so grow the set from the result's own closure
        dist = signed(orc, q[qi], base, orc.L2, 0)
        sim = (pysim.policy_best_first if policy == "A" else pysim.policy_rounds)(
            nbrs.tolist(), starts.tolist(), dist, L, k)
        assert ids[qi].tolist() == sim[0]
        d = [dist[i] for i in ids[qi] if i >= 0]
        assert d == sorted(d)
        assert len(set(ids[qi].tolist())) == k


def test_tombstones_filter_output_not_traversal(orc):
    base, nbrs, starts = make_problem(300, 16, 8, seed=31, n_start=2)
    q = make_queries(10, 16, 95)
    mask = np.zeros((300 + 31) // 32, np.uint32)
    dead = set(range(0, 300, 3))
    for i in dead:
        mask[i >> 5] |= np.uint32(1 << (i & 31))
    plain = orc.Problem(base, nbrs, starts)
    tomb = orc.Problem(base, nbrs, starts, mask)
    for L, k in ((32, 8), (16, 16)):
        full_ids, full_d, full_s, _ = orc.search_B(plain, q, L, L)  # whole beam
        ids, d, s, _ = orc.search_B(tomb, q, k, L)
        assert np.array_equal(s, orc.search_B(plain, q, k, L)[2])  # same traversal
        for qi in range(q.shape[0]):
            live = [i for i in full_ids[qi].tolist() if i >= 0 and i not in dead][:k]
            assert ids[qi].tolist() == live + [-1] * (k - len(live))


def test_rejects_bad_arguments(orc):
    base, nbrs, starts = make_problem(50, 8, 4, seed=2, n_start=2)
    q = make_queries(2, 8, 5)
    dup = orc.Problem(base, nbrs, np.array([3, 3], np.int32))
    with pytest.raises(ValueError):
        orc.search_B(dup, q, 2, 8)
    ok = orc.Problem(base, nbrs, starts)
    with pytest.raises(ValueError):
        orc.search_B(ok, q, 2, 1)  # M > L
    with pytest.raises(ValueError):
        orc.search_A(ok, q, 2, 8, M=3)  # M > number of start ids


def test_recall_hits_is_set_intersection(orc):
    res = np.array([[1, 2, 3], [4, 5, 6]], np.int32)
    gt = np.array([[3, 9, 1, 7], [6, 5, 4, 0]], np.int32)  # rows gt_dim = 4 apart, first k count
    assert orc.recall_hits(res, gt, 3) == 2 + 3
