"""Pins the oracle's sorted queue (policy A) against (1) a brute-force model of
what include/efanna2e/neighbor.h:148-237 must hold after any operation sequence
and (2) the reference's own class, compiled in place, bit for bit."""
import numpy as np
import pytest


def model(capacity, ops, dists):
    """Set-based statement of the queue: entries kept sorted by (dist, id); an insert
    is dropped if the id is present, or if the queue is full and the entry sorts after
    the last; otherwise it is placed and the overflow (if any) falls off the end.
    closest_unexpanded flags the first unflagged entry."""
    data = []  # [dist, id, flag]
    popped = []
    for op, d in zip(ops, dists):
        if op >= 0:
            key = (np.float32(d), int(op))
            if len(data) == capacity and (data[-1][0], data[-1][1]) < key:
                continue
            if any(e[1] == op for e in data):
                continue
            data.append([key[0], key[1], 0])
            data.sort(key=lambda e: (e[0], e[1]))
            del data[capacity:]
        else:
            for e in data:
                if not e[2]:
                    e[2] = 1
                    popped.append(e[1])
                    break
    return data, popped


def random_ops(seed, n_ops, id_range, tie_levels):
    rng = np.random.RandomState(seed)
    ops, dists = [], []
    known = {}
    for _ in range(n_ops):
        if rng.rand() < 0.25:
            ops.append(-1)
            dists.append(0.0)
        else:
            i = int(rng.randint(0, id_range))
            # a given id always carries the same distance, as in a search
            if i not in known:
                known[i] = float(rng.randint(0, tie_levels)) if tie_levels else float(rng.rand())
            ops.append(i)
            dists.append(known[i])
    return np.array(ops, np.int32), np.array(dists, np.float32)


@pytest.mark.parametrize("seed", range(30))
@pytest.mark.parametrize("capacity,tie_levels", [(1, 0), (4, 0), (16, 0), (8, 3), (32, 5)])
def test_queue_matches_model(orc, seed, capacity, tie_levels):
    ops, dists = random_ops(seed, 200, 60, tie_levels)
    ids, ds, fl, cur, popped = orc.queue_run(capacity, ops, dists)
    data, mpop = model(capacity, ops, dists)
    assert ids.tolist() == [e[1] for e in data]
    assert ds.tolist() == [float(e[0]) for e in data]
    assert fl.tolist() == [e[2] for e in data]
    assert popped.tolist() == mpop
    first_unflagged = next((i for i, e in enumerate(data) if not e[2]), len(data))
    assert cur == first_unflagged


@pytest.mark.parametrize("seed", range(30))
@pytest.mark.parametrize("capacity,tie_levels", [(1, 0), (4, 0), (16, 0), (8, 3), (32, 5)])
def test_queue_equals_reference_class(orc, ref, seed, capacity, tie_levels):
    ops, dists = random_ops(seed + 1000, 300, 80, tie_levels)
    a = orc.queue_run(capacity, ops, dists)
    b = orc.ref_queue_run(capacity, ops, dists)
    for x, y in zip(a, b):
        assert np.array_equal(np.asarray(x), np.asarray(y))


def test_equal_distance_different_id_order(orc):
    # ties are ordered by id (include/efanna2e/neighbor.h:39-41)
    ids, ds, _, _, _ = orc.queue_run(4, np.array([9, 3, 7, 5, 1], np.int32), np.ones(5, np.float32))
    assert ids.tolist() == [1, 3, 5, 7]


def test_reinsert_of_present_id_is_dropped(orc):
    ops = np.array([5, 6, 5, -1, 5], np.int32)
    d = np.array([2.0, 1.0, 2.0, 0.0, 2.0], np.float32)
    ids, _, fl, cur, popped = orc.queue_run(8, ops, d)
    assert ids.tolist() == [6, 5] and fl.tolist() == [1, 0] and cur == 1 and popped.tolist() == [6]


def test_cursor_moves_back_on_closer_insert(orc):
    ops = np.array([1, 2, -1, -1, 3], np.int32)
    d = np.array([5.0, 6.0, 0, 0, 1.0], np.float32)
    ids, _, fl, cur, _ = orc.queue_run(8, ops, d)
    assert ids.tolist() == [3, 1, 2] and fl.tolist() == [0, 1, 1] and cur == 0
