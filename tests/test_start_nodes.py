"""Index maintenance around the search.  Entry-point selection by farthest-point sampling in hop distance
(src/start.cu:10-145): the oracle against hand-computed cases and an all-pairs brute force, the HIP path
against the oracle.  The device-side tombstone marker (src/update.cu:406-412) against the host-built mask."""
import numpy as np
import pytest

from util import ragged


def path_graph(n):
    g = np.full((n, 2), -1, np.int32)
    for i in range(n):
        nb = [j for j in (i - 1, i + 1) if 0 <= j < n]
        g[i, :len(nb)] = nb
    return g


def test_fps_on_a_path_by_hand(orc):
    # 0-1-...-9: from 0 the farthest is 9; then min(d0, d9) peaks at 4 (and 5: lowest id wins);
    # then nodes 2, 6 and 7 are all 2 hops from the chosen set -> 2; then 6 and 7 remain at 2 hops -> 6
    assert orc.fps(path_graph(10), 0, 5).tolist() == [0, 9, 4, 2, 6]
    # a first id in the middle
    assert orc.fps(path_graph(7), 3, 3).tolist() == [3, 0, 6]


def brute_fps(nbrs, first, M):
    n = nbrs.shape[0]
    INF = 10 ** 9
    d = np.full((n, n), INF, np.int64)
    for s in range(n):
        d[s, s] = 0
        frontier = [s]
        while frontier:
            nxt = []
            for u in frontier:
                for v in nbrs[u]:
                    if v < 0:
                        break
                    if d[s, v] == INF:
                        d[s, v] = d[s, u] + 1
                        nxt.append(int(v))
            frontier = nxt
    sel = [first]
    while len(sel) < M:
        m = d[sel].min(axis=0)
        m = np.where(m == INF, -1, m)  # never reached from the chosen set
        sel.append(int(np.argmax(m)))
    return sel


@pytest.mark.parametrize("seed", range(6))
def test_fps_matches_all_pairs_brute_force(orc, seed):
    rng = np.random.RandomState(seed)
    n, R = 120, 4
    g = ragged(rng.randint(0, n, (n, R)).astype(np.int32), seed)
    g[rng.randint(0, n, 10)] = -1  # dead ends; parts of the graph are unreachable
    first = int(np.where(g[:, 0] >= 0)[0][0])
    assert orc.fps(g, first, 8).tolist() == brute_fps(g, first, 8)


@pytest.mark.gpu
@pytest.mark.parametrize("n,R,M,seed", [(5000, 8, 16, 1), (20000, 32, 16, 2), (300, 3, 40, 3), (64, 1, 5, 4)])
def test_gpu_fps_equals_oracle(orc, n, R, M, seed):
    from coral_amd import capi, synth
    rng = np.random.RandomState(seed)
    g = ragged(rng.randint(0, n, (n, R)).astype(np.int32), seed)
    g[rng.randint(0, n, max(1, n // 40))] = -1
    first = int(np.where(g[:, 0] >= 0)[0][seed])
    base = synth.gaussian_matrix(seed, n, 4)
    idx = capi.Index(base, g, np.array([first], np.int32))
    got = idx.start_ids_fps(first, M)
    idx.close()
    assert got.tolist() == orc.fps(g, first, M).tolist()


@pytest.mark.gpu
def test_gpu_mark_deleted_accumulates_like_the_host_mask():
    # src/update.cu:406-412: bit (id & 31) of word (id >> 5), OR-ed in; two batches with repeats
    from coral_amd import capi, synth
    n = 100003
    rng = np.random.RandomState(9)
    idx = capi.Index(synth.gaussian_matrix(1, n, 4), None, None)
    assert not idx.get_deleted().any()
    want = np.zeros((n + 31) // 32, np.uint32)
    for count in (1, 5000, 70000):
        ids = rng.randint(0, n, count).astype(np.int32)
        np.bitwise_or.at(want, ids >> 5, np.uint32(1) << (ids & 31).astype(np.uint32))
        idx.mark_deleted(ids)
        assert np.array_equal(idx.get_deleted(), want)
    idx.mark_deleted(np.zeros(0, np.int32))
    # ids outside the index: reported, the valid ones of the batch still marked
    with pytest.raises(capi.CoralError):
        idx.mark_deleted(np.array([7, n, -1], np.int32))
    want[0] |= np.uint32(1 << 7)
    assert np.array_equal(idx.get_deleted(), want)
    # set_deleted(None) forgets everything
    idx.set_deleted(None)
    assert not idx.get_deleted().any()
    idx.close()


@pytest.mark.gpu
def test_gpu_search_after_mark_deleted_equals_oracle_with_that_mask(orc):
    from coral_amd import capi, synth
    from test_gpu_parity import problem, WAVE64
    from util import make_queries
    n, dim, L, k = 20000, 64, 128, 50
    base, nbrs, starts = problem(n, dim, 32, seed=15)
    q = make_queries(64, dim, 56)
    want = synth.tombstone_mask(n, 77, modulo=4)
    dead_ids = np.where(np.unpackbits(want.view(np.uint8), bitorder="little")[:n])[0].astype(np.int32)
    idx = capi.Index(base, nbrs, starts)
    idx.mark_deleted(dead_ids)
    mask = idx.get_deleted()
    ids, dists, _ = idx.search(q, k, L, policy=0, have_delete=True)
    idx.close()
    assert np.array_equal(mask, want)
    oi, od, _, _ = orc.search_B(orc.Problem(base, nbrs, starts, mask), q, k, L, start_order=WAVE64, nbr_order=WAVE64)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()
