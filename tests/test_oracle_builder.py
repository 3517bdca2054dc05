"""The graph-builder restatement of the oracle (src/upd_gpu.cu:12-303, src/enhance.cu:131-208, 334-575):
hand-computed cases on a line, the invariants of the occlusion rule, and an independent set-based Python
statement of the same two steps on small random inputs.  The Python statement takes its distances from
oracle.dist (pinned elsewhere), so that only the selection logic is under test here."""
import numpy as np
import pytest

from coral_amd import synth

SEQ = 0  # the one-thread-walks-the-row summation order


def line(xs, dim=4):
    """Points on the first coordinate axis: squared distance between two of them is (x - y)^2 exactly."""
    b = np.zeros((len(xs), dim), np.float32)
    b[:, 0] = xs
    return b


# ------------------------------------------------------------------ hand-computed: one cluster on a line

def test_nap_occlusion_on_a_line(orc):
    # ids:      0    1    2    3    4
    base = line([0.0, 1.0, 2.0, 3.0, -1.5])
    knn = np.array([[0, 1, 2, 3, 4]], np.int32)
    # pivot 0: candidates by distance 1 (d=1), 4 (2.25), 2 (4), 3 (9)
    #   1 kept; 4: d(1,4)=6.25 > 2.25 kept; 2: d(1,2)=1 < 4 discarded; 3: d(1,3)=4 < 9 discarded
    st = orc.GraphState(5, 2)
    orc.nap_batch(base, st, knn, need_discard=True)
    assert st.nbrs[0].tolist() == [1, 4] and st.dists[0].tolist() == [1.0, 2.25] and st.deg[0] == 2
    st = orc.GraphState(5, 4)
    orc.nap_batch(base, st, knn, need_discard=True)
    # two kept, two discarded fill the row, in distance order
    assert st.nbrs[0].tolist() == [1, 4, 2, 3] and st.dists[0].tolist() == [1.0, 2.25, 4.0, 9.0]
    # pivot 3 (x=3): 2 (1) kept; 1 (4): d(2,1)=1 < 4 discarded; 0 (9) discarded; 4 (20.25) discarded
    assert st.nbrs[3].tolist() == [2, 1, 0, 4]
    st = orc.GraphState(5, 4)
    orc.nap_batch(base, st, knn, need_discard=False)
    assert st.nbrs[0].tolist() == [1, 4, -1, -1] and st.deg[0] == 2
    assert st.nbrs[3].tolist() == [2, -1, -1, -1] and st.deg[3] == 1
    # pivot 1 (x=1): 0 (1) kept, 2 (1) tie: d(0,2)=4 > 1 kept; ties keep cluster order -> [0, 2]
    assert st.nbrs[1].tolist()[:2] == [0, 2]


def test_nap_inner_product_on_unit_circle(orc):
    # inner product, larger is closer: candidate j is discarded when <i,j> > <p,j> for a kept i
    ang = np.deg2rad([0.0, 10.0, 20.0, 180.0])
    base = np.zeros((4, 4), np.float32)
    base[:, 0], base[:, 1] = np.cos(ang), np.sin(ang)
    st = orc.GraphState(4, 3)
    orc.nap_batch(base, st, np.array([[0, 1, 2, 3]], np.int32), metric=orc.IP, need_discard=False)
    # pivot 0: 1 (cos10) kept; 2: <1,2>=cos10 > <0,2>=cos20 discarded; 3: <1,3>=-cos10 < <0,3>=-1? no: -0.98 > -1 discarded
    assert st.nbrs[0].tolist() == [1, -1, -1]
    # pivot 3 (180 deg): nearest by ip is 2 (cos160), then 1, then 0; <2,1>=cos10 > <3,1> discarded, same for 0
    assert st.nbrs[3].tolist() == [2, -1, -1]


def test_nap_pairs_need_a_side_without_neighbours_and_keep_current_rows(orc):
    base = line([0.0, 1.0, 2.0, 3.0, 10.0, 11.0])
    st = orc.GraphState(6, 3)
    orc.nap_batch(base, st, np.array([[0, 1, 2, 3]], np.int32))
    before = st.copy()
    # the same cluster again: every pair has neighbours on both sides, candidates are the current rows only,
    # and pruning a pruned-and-filled row gives the same row
    orc.nap_batch(base, st, np.array([[0, 1, 2, 3]], np.int32))
    assert np.array_equal(st.nbrs, before.nbrs) and st.dists.tobytes() == before.dists.tobytes()
    # a cluster mixing old nodes (0, 3) with new ones (4, 5): 0 and 3 are not paired with each other, but each
    # is offered 4 and 5 next to its current row; 4 and 5 see all three others
    orc.nap_batch(base, st, np.array([[0, 3, 4, 5]], np.int32))
    assert set(st.nbrs[4].tolist()) - {-1} <= {0, 3, 5} and st.nbrs[4, 0] == 5
    assert st.nbrs[0].tolist() == before.nbrs[0].tolist()  # 1, 2, 3 are all closer than 4 and 5 and R = 3
    # 3 (x=3): 2 (1) kept; 1 (4), 0 (9) discarded by 2; 4 (49): d(2,4)=64 > 49 kept.  Two kept, one filler: the
    # nearest discarded one (1); 0 falls out of the row
    assert before.nbrs[3].tolist() == [2, 1, 0] and st.nbrs[3].tolist() == [2, 1, 4]
    assert np.array_equal(st.nbrs[1], before.nbrs[1]) and np.array_equal(st.nbrs[2], before.nbrs[2])


def test_nap_lowest_pivot_index_wins_and_pivots_read_the_rows_of_before_the_batch(orc):
    base = line([0.0, 1.0, 2.0, 5.0, 6.0, 7.0])
    # id 2 occurs in both clusters: its row comes from cluster 0 (members 0, 1), not from cluster 1
    st = orc.GraphState(6, 4)
    orc.nap_batch(base, st, np.array([[0, 1, 2], [2, 3, 4]], np.int32))
    assert sorted(set(st.nbrs[2].tolist()) - {-1}) == [0, 1]
    # 3 and 4 were offered 2 (cluster 1) although cluster 0 gives 2 neighbours in the same batch
    assert 2 in st.nbrs[3].tolist() and 2 in st.nbrs[4].tolist()
    one = orc.GraphState(6, 4)
    orc.nap_batch(base, one, np.array([[0, 1, 2]], np.int32))
    assert np.array_equal(one.nbrs[:3], st.nbrs[:3])


# ------------------------------------------------------------------ independent statement of one NAP batch

def py_prune(orc, base, pivot_dist_pairs, R, metric, need_discard):
    """pivot_dist_pairs: [(dist to pivot, id)] in column order.  Returns [(id, dist)] of the new row."""
    sign = 1.0 if metric == 0 else -1.0
    order = sorted(range(len(pivot_dist_pairs)), key=lambda t: sign * pivot_dist_pairs[t][0])  # stable
    seen, kept, disc = set(), [], []
    rank = {}
    for pos, t in enumerate(order):
        d, v = pivot_dist_pairs[t]
        if v in seen:
            continue
        seen.add(v)
        if len(kept) == R:
            break
        rank[v] = pos
        if any(sign * orc.dist(base[u], base[v], metric, SEQ) < sign * d for u, _ in kept):
            disc.append((v, d))
        else:
            kept.append((v, d))
    row = kept + (disc[:max(0, R - len(kept))] if need_discard else [])
    return sorted(row, key=lambda e: rank[e[0]])[:R]


def py_nap_batch(orc, base, nbrs, dists, deg, knn, R, metric, need_discard):
    new = {}
    for b, ids in enumerate(knn):
        for r, p in enumerate(ids):
            if p in new:
                continue
            cands = []
            for c, v in enumerate(ids):
                if c != r and (deg[p] == 0 or deg[v] == 0):
                    cands.append((orc.dist(base[p], base[v], metric, SEQ), int(v)))
            cands += [(float(dists[p, j]), int(nbrs[p, j])) for j in range(deg[p])]
            new[p] = py_prune(orc, base, cands, R, metric, need_discard)
    for p, row in new.items():
        nbrs[p], dists[p] = -1, 0
        for j, (v, d) in enumerate(row):
            nbrs[p, j], dists[p, j] = v, d
        deg[p] = len(row)


@pytest.mark.parametrize("metric,need_discard,seed", [(0, 1, 0), (0, 0, 1), (1, 1, 2), (0, 1, 3), (1, 0, 4)])
def test_nap_batches_match_the_python_statement(orc, metric, need_discard, seed):
    rng = np.random.RandomState(seed)
    n, dim, R, kb = 300, 8, 6, 10
    base = synth.gaussian_matrix(100 + seed, n, dim)
    if seed == 3:
        base = np.round(base)  # many exact ties and a few duplicate points
    if metric == 1:
        base = synth.normalize_rows(base + 0.01)
    st = orc.GraphState(n, R)
    nb, ds, dg = st.nbrs.copy(), st.dists.copy(), st.deg.copy()
    for _ in range(6):
        knn = np.stack([rng.choice(n, kb, replace=False) for _ in range(12)]).astype(np.int32)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=need_discard)
        py_nap_batch(orc, base, nb, ds, dg, knn, R, metric, need_discard)
        assert np.array_equal(st.deg, dg)
        assert np.array_equal(st.nbrs, nb)
        assert st.dists.tobytes() == ds.tobytes()


@pytest.mark.parametrize("metric", [0, 1])
def test_nap_rows_satisfy_the_occlusion_invariants(orc, metric):
    rng = np.random.RandomState(11)
    n, dim, R, kb = 2000, 16, 8, 20
    base = synth.gaussian_matrix(7, n, dim)
    if metric == 1:
        base = synth.normalize_rows(base)
    sign = 1.0 if metric == 0 else -1.0
    st = orc.GraphState(n, R)
    for _ in range(5):
        knn = np.stack([rng.choice(n, kb, replace=False) for _ in range(40)]).astype(np.int32)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=False)
    touched = np.where(st.deg > 0)[0]
    assert touched.size > 1000
    for p in touched[::7]:
        row, d = st.nbrs[p, :st.deg[p]], st.dists[p, :st.deg[p]]
        assert (st.nbrs[p, st.deg[p]:] == -1).all()
        assert p not in row and len(set(row.tolist())) == len(row)
        assert (np.diff(sign * d) >= 0).all()  # closest first
        for j in range(len(row)):
            assert d[j] == orc.dist(base[p], base[row[j]], metric, SEQ)  # stored distances are the distances
            for i in range(j):  # no kept neighbour occludes a later kept one
                assert not sign * orc.dist(base[row[i]], base[row[j]], metric, SEQ) < sign * d[j]


# ------------------------------------------------------------------ connectivity enhancement

def state_from_rows(orc, n, R, rows):
    st = orc.GraphState(n, R)
    for p, row in rows.items():
        for j, (v, d) in enumerate(row):
            st.nbrs[p, j], st.dists[p, j] = v, d
        st.deg[p] = len(row)
    return st


def test_enhance_reverse_edge_goes_to_its_sorted_place_when_the_row_has_room(orc):
    #            0    1    2    3     4(iso)
    base = line([0.0, 1.0, 4.0, -3.0, 2.0])
    st = state_from_rows(orc, 5, 4, {0: [(1, 1.0), (3, 9.0), (2, 16.0)], 1: [(0, 1.0)], 2: [(1, 9.0)], 3: [(0, 9.0)]})
    # the search found 1 (d=1), 0 (4), 2 (4) for the isolated node 4
    stats = orc.enhance_batch(base, st, [4], np.array([[1, 0, 2]], np.int32), np.array([[1.0, 4.0, 4.0]], np.float32))
    assert st.nbrs[0].tolist() == [1, 4, 3, 2] and st.dists[0].tolist() == [1.0, 4.0, 9.0, 16.0]  # room: always
    assert st.nbrs[1].tolist() == [4, 0, -1, -1]  # equal distance: goes in front of the entry that was there
    assert st.nbrs[2].tolist() == [4, 1, -1, -1]
    assert stats[0] == 3 and stats[1] == 0
    # own row: 1 kept; 0: d(1,0)=1 < 4 discarded; 2: d(1,2)=9 > 4 kept; filled with 0
    assert st.nbrs[4].tolist() == [1, 0, 2, -1] and st.deg[4] == 3


def test_enhance_full_rows_reject_occluded_newcomers_and_evict_what_the_newcomer_occludes(orc):
    #            0    1    2    3    4     5(iso)
    base = line([0.0, 1.0, 3.0, 5.0, -4.0, 2.0])
    rows = {0: [(1, 1.0), (2, 9.0), (4, 16.0)], 3: [(2, 4.0), (1, 16.0), (0, 25.0)], 4: [(0, 16.0), (1, 25.0), (2, 49.0)]}
    st = state_from_rows(orc, 6, 3, rows)
    knn = np.array([[0, 3, 4]], np.int32)
    kd = np.array([[4.0, 9.0, 36.0]], np.float32)
    stats = orc.enhance_batch(base, st, [5], knn, kd)
    # row of 0 is full; newcomer 5 at distance 4 comes after 1 (d=1): d(1,5)=1 < 4, occluded -> rejected
    assert st.nbrs[0].tolist() == [1, 2, 4]
    # row of 3: newcomer at 9 after 2 (4): d(2,5)=1 < 9 -> rejected
    assert st.nbrs[3].tolist() == [2, 1, 0]
    # row of 4: newcomer at 36 after 0 (16): d(0,5)=4 < 36 occluded -> rejected; all three rejected
    assert st.nbrs[4].tolist() == [0, 1, 2]
    assert stats[0] == 0 and stats[1] == 3
    # a newcomer that nobody occludes: node 6 at x=-1 for the row of 0 = [1 (1), 2 (9), 4 (16)]
    base2 = line([0.0, 1.0, 3.0, 5.0, -4.0, 2.0, -1.0])
    st = state_from_rows(orc, 7, 3, rows)
    orc.enhance_batch(base2, st, [6], np.array([[0]], np.int32), np.array([[1.0]], np.float32))
    # equal to the first entry's distance: position 0; from the back, 4 (16): d(4,6)=9 < 16 is occluded -> evicted
    assert st.nbrs[0].tolist() == [6, 1, 2] and st.dists[0].tolist() == [1.0, 1.0, 9.0]
    # nobody occluded by the newcomer: the last entry goes.  Row of 0 = [1, 2, 3'] with a far third entry
    base3 = line([0.0, 1.0, 3.0, 50.0, -4.0, 2.0, -1.0])
    st = state_from_rows(orc, 7, 3, {0: [(1, 1.0), (2, 9.0), (3, 2500.0)]})
    orc.enhance_batch(base3, st, [6], np.array([[0]], np.int32), np.array([[1.0]], np.float32))
    # from the back: 3 (2500): d(3,6)=2601 > 2500 no; 2 (9): d(2,6)=16 > 9 no; 1 (1): d(1,6)=4 > 1 no -> none:
    # the last one is dropped
    assert st.nbrs[0].tolist() == [6, 1, 2]


def test_enhance_first_claim_in_batch_order_wins_and_minus_one_ends_a_list(orc):
    base = line([0.0, 1.0, 2.0, 3.0, 4.0])
    st = state_from_rows(orc, 5, 4, {0: [(1, 1.0)], 1: [(0, 1.0)]})
    knn = np.array([[1, 0, -1], [0, 1, -1]], np.int32)
    kd = np.array([[1.0, 4.0, 0.0], [9.0, 4.0, 0.0]], np.float32)
    stats = orc.enhance_batch(base, st, [2, 3], knn, kd)
    # both 0 and 1 were claimed by node 2 (the first of the batch); node 3 inserts nowhere
    assert st.nbrs[0].tolist() == [1, 2, -1, -1] and st.nbrs[1].tolist() == [2, 0, -1, -1]
    assert stats[0] == 2
    assert st.nbrs[2].tolist() == [1, 0, -1, -1]  # 0: d(1,0)=1 < 4 discarded, filled back in
    assert st.nbrs[3].tolist() == [1, 0, -1, -1]  # sorted by its own distances: 1 (4), 0 (9)
    # a new batch clears the claims
    orc.enhance_batch(base, st, [4], np.array([[1, -1, -1]], np.int32), np.array([[9.0, 0, 0]], np.float32))
    assert st.nbrs[1].tolist() == [2, 0, 4, -1]


def py_enhance_batch(orc, base, nbrs, dists, deg, iso_ids, knn_ids, knn_dists, R, metric):
    sign = 1.0 if metric == 0 else -1.0
    claimed = set()
    for b, iso in enumerate(iso_ids):
        for v, vd in zip(knn_ids[b], knn_dists[b]):
            v = int(v)
            if v < 0:
                break
            if v in claimed:
                continue
            claimed.add(v)
            row = [(int(nbrs[v, j]), float(dists[v, j])) for j in range(deg[v])]
            ahead = [e for e in row if sign * e[1] < sign * vd]  # rows are sorted: these are its leading entries
            pos = len(ahead)
            occluded = any(sign * orc.dist(base[iso], base[u], metric, SEQ) < sign * vd for u, _ in ahead)
            if len(row) == R:
                if occluded or pos == R:
                    continue
                behind = [j for j in range(pos, R)
                          if sign * orc.dist(base[iso], base[row[j][0]], metric, SEQ) < sign * row[j][1]]
                del row[behind[-1] if behind else R - 1]
            row.insert(pos, (int(iso), float(vd)))
            nbrs[v], dists[v] = -1, 0
            for j, (u, d) in enumerate(row):
                nbrs[v, j], dists[v, j] = u, d
            deg[v] = len(row)
    for b, iso in enumerate(iso_ids):
        cands = [(float(d), int(v)) for v, d in zip(knn_ids[b], knn_dists[b]) if v >= 0]
        row = py_prune(orc, base, cands, R, metric, True)
        nbrs[iso], dists[iso] = -1, 0
        for j, (u, d) in enumerate(row):
            nbrs[iso, j], dists[iso, j] = u, d
        deg[iso] = len(row)


@pytest.mark.parametrize("metric,seed", [(0, 0), (1, 1), (0, 2)])
def test_enhance_batches_match_the_python_statement(orc, metric, seed):
    rng = np.random.RandomState(seed)
    n, dim, R, kn = 400, 8, 5, 9
    base = synth.gaussian_matrix(40 + seed, n, dim)
    if metric == 1:
        base = synth.normalize_rows(base)
    sign = 1.0 if metric == 0 else -1.0
    st = orc.GraphState(n, R)
    for t in range(8):  # a graph over the first 300 nodes with rows of every fill level
        knn = np.stack([rng.choice(300, 7, replace=False) for _ in range(25)]).astype(np.int32)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=bool(t % 2))
    assert (st.deg[300:] == 0).all() and (st.deg[:300] == R).any() and ((st.deg[:300] > 0) & (st.deg[:300] < R)).any()
    nb, ds, dg = st.nbrs.copy(), st.dists.copy(), st.deg.copy()
    linked = np.where(st.deg > 0)[0]
    for lo in (300, 350):
        iso = np.arange(lo, lo + 50, dtype=np.int32)
        ids = np.empty((50, kn), np.int32)
        dd = np.empty((50, kn), np.float32)
        for i, p in enumerate(iso):  # the exact nearest linked nodes stand in for the search result
            d = np.array([orc.dist(base[p], base[v], metric, SEQ) for v in linked], np.float32)
            o = np.argsort(sign * d, kind="stable")[:kn]
            ids[i], dd[i] = linked[o], d[o]
        ids[3, 6:] = -1
        orc.enhance_batch(base, st, iso, ids, dd, metric=metric)
        py_enhance_batch(orc, base, nb, ds, dg, iso, ids, dd, R, metric)
        assert np.array_equal(st.deg, dg) and np.array_equal(st.nbrs, nb) and st.dists.tobytes() == ds.tobytes()
        linked = np.where(st.deg > 0)[0]
    assert (st.deg[300:] > 0).all()


# ------------------------------------------------------------------ second enhancement phase: the most-hit nodes

def test_top_hit_ids_are_ordered_by_hits_then_id(orc):
    rng = np.random.RandomState(5)
    hits = rng.randint(0, 6, 500).astype(np.uint32)
    want = np.lexsort((np.arange(500), -hits.astype(np.int64)))
    for top_n in (1, 37, 500):
        assert orc.top_hit_ids(hits, top_n).tolist() == want[:top_n].tolist()
    assert orc.top_hit_ids(np.array([0, 3, 3, 1], np.uint32), 3).tolist() == [1, 2, 3]


def test_enhance_top_candidates_are_the_found_list_and_the_current_row(orc):
    #            0    1    2    3     4     5
    base = line([0.0, 1.0, 2.0, 4.0, -1.0, 8.0])
    rows = {0: [(1, 1.0), (3, 16.0)], 1: [(0, 1.0)], 2: [(1, 1.0)], 3: [(2, 4.0)], 4: [(0, 1.0)], 5: [(3, 16.0)]}
    st = state_from_rows(orc, 6, 3, rows)
    # node 0 searched for itself: found 0 (itself, 0), 4 (1), 1 (1), 2 (4)
    knn = np.array([[0, 4, 1, 2]], np.int32)
    kd = np.array([[0.0, 1.0, 1.0, 4.0]], np.float32)
    stats = orc.enhance_top_batch(base, st, [0], knn, kd)
    # reverse edges, found part only (0, 4, 1, 2; never 3, which is only in the current row):
    #   into the row of 0 itself (then overwritten by its rebuilt row), of 4: [0 (1)] -> 0 in front of the equal entry,
    #   of 1: [0 (1)] -> in front, of 2: [1 (1)] -> behind
    assert st.nbrs[4].tolist() == [0, 0, -1] and st.nbrs[1].tolist() == [0, 0, -1] and st.nbrs[2].tolist() == [1, 0, -1]
    assert st.nbrs[3].tolist() == [2, -1, -1]
    assert stats[0] == 4
    # own row from [0 (0), 4 (1), 1 (1), 2 (4)] + current row [1 (1), 3 (16)], sorted, ties in that order:
    #   0 (itself) kept, occludes nobody (its distance to j equals the pivot's); 4 kept; 1: d(4,1)=4 > 1 kept; full.
    assert st.nbrs[0].tolist() == [0, 4, 1] and st.dists[0].tolist() == [0.0, 1.0, 1.0] and st.deg[0] == 3
    # with a wider row the second listing of 1 is dropped, 2 (d(1,2)=1 < 4) and 3 (d(1,3)=9 < 16) are ruled out and
    # fill the row in distance order
    st = state_from_rows(orc, 6, 6, rows)
    orc.enhance_top_batch(base, st, [0], knn, kd)
    assert st.nbrs[0].tolist() == [0, 4, 1, 2, 3, -1] and st.deg[0] == 5


def test_enhance_top_rows_are_read_as_of_before_the_batch(orc):
    #            0    1    2     3
    base = line([0.0, 1.0, 3.0, -2.0])
    rows = {0: [(1, 1.0)], 1: [(0, 1.0)], 2: [(1, 4.0)], 3: [(0, 4.0)]}
    st = state_from_rows(orc, 4, 4, rows)
    # both 0 and 1 are processed in one batch; 0 found 1 and 1 found 0: each gets a reverse edge from the other before
    # its row is rebuilt from (found list + the row of before the batch), which holds the other anyway
    knn = np.array([[0, 1, 3], [1, 0, 2]], np.int32)
    kd = np.array([[0.0, 1.0, 4.0], [0.0, 1.0, 4.0]], np.float32)
    orc.enhance_top_batch(base, st, [0, 1], knn, kd)
    # node 0: [0 (0), 1 (1), 3 (4)] + [1 (1)]: 0 kept, 1 kept, 3: d(1,3)=9 > 4 kept, second 1 dropped
    assert st.nbrs[0].tolist() == [0, 1, 3, -1]
    # node 1: [1 (0), 0 (1), 2 (4)] + [0 (1)]: 1, 0 kept, 2: d(0,2)=9 > 4 kept
    assert st.nbrs[1].tolist() == [1, 0, 2, -1]
    # 3 was claimed by node 0 (first in the batch), 2 by node 1
    assert st.nbrs[3].tolist() == [0, 0, -1, -1] and st.nbrs[2].tolist() == [1, 1, -1, -1]


def py_enhance_top_batch(orc, base, nbrs, dists, deg, top_ids, knn_ids, knn_dists, R, metric):
    k = knn_ids.shape[1]
    lists = []
    for b, t in enumerate(top_ids):  # every list from the rows of before the batch
        found = [(int(v), float(d)) for v, d in zip(knn_ids[b], knn_dists[b])]
        if any(v < 0 for v, _ in found):
            found = found[:[v < 0 for v, _ in found].index(True)]
        lists.append((found, [(int(nbrs[t, j]), float(dists[t, j])) for j in range(deg[t])]))
    rev_ids = np.full((len(top_ids), k), -1, np.int32)
    rev_d = np.zeros((len(top_ids), k), np.float32)
    for b, (found, _) in enumerate(lists):
        for i, (v, d) in enumerate(found):
            rev_ids[b, i], rev_d[b, i] = v, d
    own = {}
    scratch = (nbrs.copy(), dists.copy(), deg.copy())
    py_enhance_batch(orc, base, nbrs, dists, deg, top_ids, rev_ids, rev_d, R, metric)  # reverse edges (+ rows, redone below)
    for b, t in enumerate(top_ids):
        found, row = lists[b]
        own[int(t)] = py_prune(orc, base, [(d, v) for v, d in found + row], R, metric, True)
    for t, row in own.items():
        nbrs[t], dists[t] = -1, 0
        for j, (u, d) in enumerate(row):
            nbrs[t, j], dists[t, j] = u, d
        deg[t] = len(row)
    del scratch


@pytest.mark.parametrize("metric,seed", [(0, 0), (1, 1)])
def test_enhance_top_batches_match_the_python_statement(orc, metric, seed):
    rng = np.random.RandomState(10 + seed)
    n, dim, R, k = 300, 8, 5, 8
    base = synth.gaussian_matrix(60 + seed, n, dim)
    if metric == 1:
        base = synth.normalize_rows(base)
    sign = 1.0 if metric == 0 else -1.0
    st = orc.GraphState(n, R)
    for t in range(10):
        knn = np.stack([rng.choice(n, 7, replace=False) for _ in range(25)]).astype(np.int32)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=bool(t % 2))
    linked = np.where(st.deg > 0)[0]
    nb, ds, dg = st.nbrs.copy(), st.dists.copy(), st.deg.copy()
    for rep in range(2):
        top = rng.choice(linked, 40, replace=False).astype(np.int32)
        ids = np.empty((40, k), np.int32)
        dd = np.empty((40, k), np.float32)
        for i, p in enumerate(top):  # the exact nearest linked nodes (the node itself first) stand in for the search
            d = np.array([orc.dist(base[p], base[v], metric, SEQ) for v in linked], np.float32)
            o = np.argsort(sign * d, kind="stable")[:k]
            ids[i], dd[i] = linked[o], d[o]
        assert (ids[:, 0] == top).all()
        ids[5, 6:] = -1
        orc.enhance_top_batch(base, st, top, ids, dd, metric=metric)
        py_enhance_top_batch(orc, base, nb, ds, dg, top, ids, dd, R, metric)
        assert np.array_equal(st.deg, dg) and np.array_equal(st.nbrs, nb) and st.dists.tobytes() == ds.tobytes()
    # every rebuilt row starts with the node itself (distance 0 sorts first; for IP the self product is the largest)
    assert all(st.nbrs[t, 0] == t for t in top)
