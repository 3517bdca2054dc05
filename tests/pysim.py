"""An independent, set-based statement of the two traversal policies in plain
Python, written from the algorithm description (not from the C oracle), for
tiny inputs.  Distances are supplied by the caller so that only the traversal
logic is under test."""


def policy_rounds(nbrs, starts, dist, L, k, deleted=frozenset(), trace=None):
    """dist: dict id -> signed distance (smaller is closer).  Returns (ids, hops, expansions, evals).
    trace (a list) receives, per round, (ids expanded in the round, ids in the beam after its merge)."""
    visited = set(starts)
    beam = {s: False for s in starts}  # id -> expanded
    evals = len(starts)
    thr = float("inf")
    hops = expansions = 0
    while True:
        cand = []
        todo = [v for v, ex in beam.items() if not ex]
        for v in todo:
            beam[v] = True
            expansions += 1
            for w in nbrs[v]:
                if w < 0:
                    break
                if w in visited:
                    continue
                visited.add(w)
                evals += 1
                if dist[w] < thr:
                    cand.append(w)
        if not cand:
            break
        hops += len(cand)
        overflow = len(beam) + len(cand) > L
        for w in cand:
            beam[w] = False
        if overflow:
            keep = sorted(beam, key=lambda v: (dist[v], v))[:L]
            beam = {v: beam[v] for v in keep}
            thr = dist[keep[-1]]
        if trace is not None:
            trace.append((frozenset(todo), frozenset(beam)))
    order = sorted(beam, key=lambda v: (dist[v], v))
    live = [v for v in order if v not in deleted][:k]
    return live + [-1] * (k - len(live)), hops, expansions, evals


def policy_best_first(nbrs, starts, dist, L, k, deleted=frozenset(), trace=None):
    """trace (a list) receives, per step, (the id expanded, ids in the beam after the step's inserts)."""
    visited = set()
    beam = {}
    evals = 0

    def insert(v):
        nonlocal beam
        if v in beam:
            return
        beam[v] = False
        if len(beam) > L:
            keep = sorted(beam, key=lambda x: (dist[x], x))[:L]
            beam = {x: beam[x] for x in keep}

    for s in starts:
        insert(s)
        visited.add(s)
        evals += 1
    hops = len(starts)
    expansions = 0
    while True:
        pending = [v for v in sorted(beam, key=lambda x: (dist[x], x)) if not beam[v]]
        if not pending:
            break
        v = pending[0]
        beam[v] = True
        hops += 1
        expansions += 1
        for w in nbrs[v]:
            if w < 0:
                break
            if w in visited:
                continue
            evals += 1
            insert(w)
            visited.add(w)
        if trace is not None:
            trace.append((frozenset([v]), frozenset(beam)))
    order = sorted(beam, key=lambda v: (dist[v], v))
    live = [v for v in order if v not in deleted][:k]
    return live + [-1] * (k - len(live)), hops, expansions, evals
