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
    """True when two result lists are identical except for swaps or substitutions
    among entries whose distances differ by less than rel * |d|."""
    if np.array_equal(ids_a, ids_b):
        return True
    k = len(ids_a)
    if not np.allclose(d_a, d_b, rtol=1e-5, atol=0):
        return False
    sa, sb = set(ids_a.tolist()), set(ids_b.tolist())
    for i in range(k):
        if ids_a[i] == ids_b[i]:
            continue
        # the entry of a must appear in b at a position of (nearly) the same distance,
        # or sit at the tail where a near-tie decided membership
        for x, other_ids, other_d, mine_d in ((ids_a[i], ids_b, d_b, d_a[i]), (ids_b[i], ids_a, d_a, d_b[i])):
            pos = np.where(other_ids == x)[0]
            if pos.size:
                if abs(other_d[pos[0]] - mine_d) > rel * max(abs(mine_d), 1e-30) * 4:
                    return False
            else:
                # membership differs: only acceptable against the last entry's distance
                if abs(other_d[k - 1] - mine_d) > rel * max(abs(mine_d), 1e-30) * 4:
                    return False
    return len(sa ^ sb) <= 2 * k
