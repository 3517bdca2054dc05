"""Shared builders for the tests: small seeded problems and comparison helpers."""
import hashlib

import numpy as np

from coral_amd import synth


def ragged(nbrs, seed, keep_min=0):
    """Cut every row to a seeded random degree in [keep_min, R] (rest -1)."""
    rng = np.random.RandomState(seed)
    out = nbrs.copy()
    deg = rng.randint(keep_min, nbrs.shape[1] + 1, nbrs.shape[0])
    for i, d in enumerate(deg):
        out[i, d:] = -1
    return out


def make_problem(n, dim, R, seed, metric="l2", n_start=4, ragged_seed=None):
    base = synth.gaussian_matrix(seed, n, dim)
    if metric == "ip":
        base = synth.normalize_rows(base)
    nbrs = synth.exact_knn_graph(base, R, metric=metric)
    if ragged_seed is not None:
        nbrs = ragged(nbrs, ragged_seed)
    starts = np.random.RandomState(seed + 7).choice(n, n_start, replace=False).astype(np.int32)
    return base, nbrs, starts


def make_queries(Q, dim, seed, metric="l2"):
    q = synth.shifted_queries(Q, dim, seed, seed + 1, seed + 2)
    return synth.normalize_rows(q) if metric == "ip" else q


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def near_tie_equal(ids_a, d_a, ids_b, d_b, rel=1e-6):
    """True when two result lists (closest first, same length) are identical except for permutations or substitutions
    among entries whose distances differ by less than rel * |d|:
      * where the lists hold different ids at a rank, the two distances at that rank are within rel of each other
        (the ids that swapped or replaced one another are a near-tie);
      * an id that both lists hold has the same distance in both up to the summation order (1e-5);
      * an id that only one list holds is within rel of the other list's last entry (a near-tie decided membership)."""
    if np.array_equal(ids_a, ids_b):
        return True
    k = len(ids_a)

    def close(x, y, r):
        return abs(float(x) - float(y)) <= r * max(abs(float(x)), abs(float(y)), 1e-30)

    for i in range(k):
        if ids_a[i] == ids_b[i]:
            if not close(d_a[i], d_b[i], 1e-5):
                return False
            continue
        if not close(d_a[i], d_b[i], rel):
            return False
        for x, mine_d, other_ids, other_d in ((ids_a[i], d_a[i], ids_b, d_b), (ids_b[i], d_b[i], ids_a, d_a)):
            pos = np.where(other_ids == x)[0]
            if pos.size:
                if not close(other_d[pos[0]], mine_d, 1e-5):
                    return False
            elif not close(other_d[k - 1], mine_d, rel):
                return False
    return True


def rounds_hand_case():
    """A traversal of the expand-all-rounds policy (src/search_gpu.cu:412-483, 525-576) worked out by hand.

    Eleven points on a line (distance to the query at the origin = x squared, exact in fp32 in any summation order),
    L = 3, one start id.  Every rule that sets this policy apart from a best-first search decides a counter:

      round 1  expands 0 (100): 1 (81) and 2 (64) pass the initial threshold; beam {0, 1, 2} is exactly full by
               APPENDING, so the threshold stays at the sentinel (:477-483).
      round 2  expands 1 and 2: 3 (400), 4 (49), 5 (36).  3 is farther than everything in the beam and still
               counts as a candidate because the threshold was not tightened.  Overflow: beam {5, 4, 2}, threshold 64.
      round 3  expands 5 then 4: 6 (56.25) passes; 7 (60.0625) passes although it no longer fits beside 6, because
               the threshold is frozen for the round (:412-439); 7 is listed by 4 as well and is measured once;
               8 (72.25) fails; 9 (64) fails: the comparison is strict.  Beam {5, 4, 6}, threshold 56.25.
      round 4  expands 6: 10 (1) passes.  Beam {10, 5, 4}, threshold 49.
      round 5  expands 10: its only neighbour, 0, is visited; no candidate, the search ends.

    hops = candidates = 2 + 3 + 2 + 1 = 8 (start ids are not counted), expansions = 1 + 2 + 2 + 1 + 1 = 7,
    distance evaluations = 1 + 2 + 3 + 4 + 1 = 11, rounds = 5.  With the threshold tightened on the exact fit, or
    moved inside a round, hops is 7; with a non-strict comparison, or the start counted, 9.
    """
    xs = [10, 9, 8, 20, 7, 6, 7.5, 7.75, 8.5, 8, 1]
    base = np.zeros((len(xs), 4), np.float32)
    base[:, 2] = xs
    rows = {0: [1, 2], 1: [3, 4], 2: [5], 4: [7, 8, 9], 5: [6, 7], 6: [10], 10: [0]}
    nbrs = np.full((len(xs), 3), -1, np.int32)
    for i, r in rows.items():
        nbrs[i, :len(r)] = r
    q = np.zeros((1, 4), np.float32)
    expect = dict(ids=[10, 5, 4], dists=[1.0, 36.0, 49.0], hops=8, expansions=7, dist_evals=11, rounds=5)
    return base, nbrs, np.array([0], np.int32), q, 3, 3, expect


def explain_divergence(orc, base, nbrs, starts, q1, metric, policy, L, k, rel=1e-6):
    """Why do the kernel's summation order and the reference's lead one query to different answers?

    Both traversals are replayed step by step (tests/pysim.py) on the distances of every node in the kernel's order
    (ORDER_WAVE64) and in the reference's (policy 0: the warp tree for start ids and the one-thread chain for
    neighbours; policy 1: the AVX-512 order).  Up to the first step at which they part the two have done the same
    work on the same beam, so what they do differently there -- another entry expanded, or another entry kept at the
    beam's boundary -- is a pair of nodes that the two orders rank in opposite ways.  Returns (step, pairs): pairs =
    [(x, y, relative gap of their exact distances)], each x chosen by one order where the other chose y.  The
    contract allows such swaps only for near-ties, gap < 1e-6; None when the traversals never part."""
    import pysim
    n = base.shape[0]
    sign = -1.0 if metric == orc.IP else 1.0

    def all_dists(order):
        ids, d = orc.bruteforce(base, q1[None, :], n, metric, order=order)
        out = np.empty(n, np.float64)
        out[ids[0]] = sign * d[0].astype(np.float64)
        return out

    d_gpu = all_dists(orc.ORDER_WAVE64)
    if policy == 0:
        d_ref = all_dists(orc.ORDER_GPU_SEQ)
        d_ref[starts] = all_dists(orc.ORDER_GPU_WARP32)[starts]
    else:
        d_ref = all_dists(orc.ORDER_CPU_AVX512)
    exact = all_dists(-1)
    sim = pysim.policy_rounds if policy == 0 else pysim.policy_best_first
    rows = [[int(v) for v in r] for r in nbrs]
    ta, tb = [], []
    sim(rows, [int(s) for s in starts], d_gpu, L, k, trace=ta)
    sim(rows, [int(s) for s in starts], d_ref, L, k, trace=tb)
    for step, (a, b) in enumerate(zip(ta, tb)):
        if a == b:
            continue
        # the expanded ids differ, or the beams do; either way the ids on one side only
        only_a = (a[0] - b[0]) or (a[1] - b[1])
        only_b = (b[0] - a[0]) or (b[1] - a[1])
        pairs = []
        for x in sorted(only_a):
            y = min(only_b, key=lambda v: abs(exact[v] - exact[x]))
            pairs.append((x, int(y), abs(exact[x] - exact[y]) / max(abs(exact[x]), 1e-30)))
        return step, pairs
    return None
