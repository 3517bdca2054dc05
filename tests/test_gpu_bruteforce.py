"""Exact brute-force kNN on the GPU (the ground-truth / builder-kNN component that replaces
faiss): bit-exact against the oracle's brute force in the same summation order, and within
tolerance of the fp64 closed form."""
import time

import numpy as np
import pytest

from coral_amd import capi, synth, workloads

pytestmark = pytest.mark.gpu
SEQ = 0  # ORDER_GPU_SEQ


def test_comp_gt_tool_and_vectors_only_index(orc, tmp_path):
    """The ground-truth driver: fbin in, gt file out (layout of tests/comp_gt.cpp:142-175)."""
    import os
    import subprocess
    from coral_amd import formats
    n, dim, Q, k = 6000, 100, 50, 20
    base = synth.gaussian_matrix(5, n, dim)
    q = synth.shifted_queries(Q, dim, 6, 7, 8)
    formats.fbin_write(tmp_path / "base.fbin", base)
    formats.fbin_write(tmp_path / "query.fbin", q)
    tool = os.path.join(os.path.dirname(capi.LIB_PATH), "comp_gt")
    for dist, m in (("l2", capi.L2), ("ip", capi.IP)):
        r = subprocess.run([tool, "--base_data_path", str(tmp_path / "base.fbin"), "--query_data_path",
                            str(tmp_path / "query.fbin"), "--gt_save_file", str(tmp_path / "gt.bin"), "--k", str(k),
                            "--nq", "40", "--dist", dist], capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr
        gt = formats.gt_read(tmp_path / "gt.bin")
        assert gt.shape == (40, k)
        b2, q2 = (formats.normalize_l2(base), formats.normalize_l2(q)) if dist == "ip" else (base, q)
        oi, _ = orc.bruteforce(b2, q2[:40], k, m, order=SEQ)
        assert np.array_equal(gt, oi)
    r = subprocess.run([tool, "--dist", "l2"], capture_output=True, text=True)
    assert r.returncode == 255 and "required but missing" in r.stderr
    # a vectors-only index serves brute force and refuses graph search
    idx = capi.Index(base, None, None)
    ids, _, _ = idx.bruteforce(q, k)
    assert np.array_equal(ids, orc.bruteforce(base, q, k, order=SEQ)[0])
    with pytest.raises(capi.CoralError) as e:
        idx.search(q, 5, 16)
    assert e.value.code == capi.ERR_STATE
    idx.close()


def ring(n, R=2):
    g = np.full((n, R), -1, np.int32)
    g[:, 0] = (np.arange(n) + 1) % n
    return g


@pytest.mark.parametrize("n,dim,Q,k,metric,tomb", [
    (3000, 200, 37, 100, "l2", False),
    (3000, 200, 37, 100, "ip", False),
    (5000, 20, 130, 10, "l2", True),
    (777, 132, 5, 129, "l2", False),
    (4097, 4, 257, 1, "ip", True),
    (50, 8, 9, 64, "l2", True),      # fewer live points than k: padded
    (20000, 128, 300, 32, "l2", False),
])
def test_bruteforce_exact_against_oracle(orc, n, dim, Q, k, metric, tomb):
    m = capi.IP if metric == "ip" else capi.L2
    base = synth.gaussian_matrix(n + dim, n, dim)
    q = synth.shifted_queries(Q, dim, 3, 4, 5)
    if metric == "ip":
        base, q = synth.normalize_rows(base), synth.normalize_rows(q)
    mask = synth.tombstone_mask(n, 77, 3) if tomb else None
    idx = capi.Index(base, ring(n), np.array([0], np.int32), m)
    if tomb:
        idx.set_deleted(mask)
    ids, dists, _ = idx.bruteforce(q, k, have_delete=tomb)  # matrix-core screening + exact re-ranking
    redone, fused = idx.bruteforce_last_redone(), idx.bruteforce_last_fused()
    idx.bruteforce_exact_only(2)                            # the screening's candidates from the distance matrix
    ids3, dists3, _ = idx.bruteforce(q, k, have_delete=tomb)
    assert idx.bruteforce_last_fused() == 0 and idx.bruteforce_last_redone() == redone
    assert np.array_equal(ids3, ids) and dists3.tobytes() == dists.tobytes()
    idx.bruteforce_exact_only(True)                         # every pair in the reference's order
    ids2, dists2, _ = idx.bruteforce(q, k, have_delete=tomb)
    assert idx.bruteforce_last_redone() == 0 and idx.bruteforce_last_fused() == 0
    idx.close()
    assert fused == (1 if n >= 8192 else 0)  # 64 tiles of 128 points are what the sample needs
    print("queries that the screening could not vouch for: %d of %d" % (redone, Q), flush=True)
    oi, od = orc.bruteforce(base, q, k, m, deleted=mask, order=SEQ)
    assert np.array_equal(ids, oi)
    assert dists.tobytes() == od.tobytes()
    assert np.array_equal(ids2, oi) and dists2.tobytes() == od.tobytes()
    if n > 2 * (k + 32) and dim >= 20:
        assert redone <= Q // 4  # independent data: the candidates nearly always suffice
    # against the fp64 closed form: same ids except where fp32 rounding reorders near-ties
    ti, td = orc.bruteforce(base, q, k, m, deleted=mask)
    live = ti >= 0
    assert (ids[live] == ti[live]).mean() > 0.98
    assert np.allclose(dists[live], td[live], rtol=1e-5, atol=1e-6)


def test_randomised_knn_problems_equal_the_oracle(orc):
    """Seeded random sizes, k, metrics, tombstones and laws of the data (ties on a lattice, repeated vectors, large
    and small magnitudes, a common offset that makes the screening's error bound bite): the screened path and the
    exact-only path both return the oracle's ids and distance bits; so does the screening with its candidates
    selected from the distance matrix instead of inside the kernel."""
    redone = fused = unfused = 0
    for c in range(80):
        rng = np.random.RandomState(7000 + c)
        n = int(rng.choice([50, 129, 300, 1000, 4097, 10000, 30000]))
        dim = int(rng.choice([4, 8, 12, 20, 32, 64, 100, 128, 200, 256, 512]))
        Q = int(rng.choice([1, 5, 37, 128, 129, 300]))
        k = int(rng.choice([1, 2, 10, 32, 64, 100, 129, 300]))
        metric = capi.IP if rng.rand() < 0.35 else capi.L2
        tomb = rng.rand() < 0.3
        kind = str(rng.choice(["gauss", "lattice", "dups", "big", "tiny", "offset"]))
        while n * dim * Q > 1e9:
            Q = max(1, Q // 2)
        print("case", dict(c=c, n=n, dim=dim, Q=Q, k=k, metric=metric, tomb=tomb, kind=kind), flush=True)
        base = synth.gaussian_matrix(2000 + c, n, dim)
        q = synth.shifted_queries(Q, dim, 3 + c, 4 + c, 5 + c)
        if kind == "lattice":
            base, q = np.round(base), np.round(q)
        elif kind == "dups":
            base[n // 2:] = base[:n - n // 2]
        elif kind == "big":
            base, q = base * 1000.0, q * 1000.0
        elif kind == "tiny":
            base, q = base * 1e-3, q * 1e-3
        elif kind == "offset":
            base, q = base + 50.0, q + 50.0
        base, q = base.astype(np.float32), q.astype(np.float32)
        if metric == capi.IP and kind in ("gauss", "dups"):
            base, q = synth.normalize_rows(base), synth.normalize_rows(q)
        mask = synth.tombstone_mask(n, 77 + c, int(rng.choice([2, 3, 10]))) if tomb else None
        oi, od = orc.bruteforce(base, q, k, metric, deleted=mask, order=SEQ)
        idx = capi.Index(base, None, None, metric)
        if tomb:
            idx.set_deleted(mask)
        for mode in (0, 2, 1):
            idx.bruteforce_exact_only(mode)
            ids, dists, _ = idx.bruteforce(q, k, have_delete=tomb)
            redone += idx.bruteforce_last_redone() if mode == 0 else 0
            if mode == 0 and n >= 8192 and k + 32 <= 1024:
                fused += idx.bruteforce_last_fused()
                unfused += 1 - idx.bruteforce_last_fused()
            else:
                assert idx.bruteforce_last_fused() == 0
            assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes(), "mode %d" % mode
        idx.close()
    print("selection inside the kernel: %d cases, handed to the distance matrix: %d" % (fused, unfused), flush=True)
    assert redone > 0  # some of these queries went through the exact passes after the screening
    assert fused > 0


def test_bruteforce_ties_are_ordered_by_id(orc):
    # integer lattice: many exactly equal distances, including across the k-th place
    side = 7
    grid = np.stack(np.meshgrid(*[np.arange(side)] * 4, indexing="ij"), -1).reshape(-1, 4).astype(np.float32)
    q = np.array([[3, 3, 3, 3], [0, 0, 0, 0], [2.5, 3, 1, 6]], np.float32)
    idx = capi.Index(grid, ring(grid.shape[0]), np.array([0], np.int32))
    redone = 0
    for k in (1, 9, 33, 81, 200):
        ids, dists, _ = idx.bruteforce(q, k)
        redone += idx.bruteforce_last_redone()
        oi, od = orc.bruteforce(grid, q, k, order=SEQ)
        assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()
        d2 = ((grid[ids] - q[:, None, :]) ** 2).sum(-1)
        assert np.array_equal(d2, dists)
        # within equal distances ids ascend
        for r in range(q.shape[0]):
            same = np.diff(dists[r]) == 0
            assert (np.diff(ids[r])[same] > 0).all()
    assert redone > 0  # ties across the last candidate's place: the screening hands those queries over
    idx.close()


def test_bruteforce_rows_with_thousands_of_ties_and_large_k(orc):
    # 30 000 points on a 3 x 3 x 3 x 3 lattice: every distance value is shared by hundreds of points, so the
    # candidates at the selection threshold outgrow the fast path's buffer and the radix path takes the rows;
    # k above 1024 goes to the radix path directly
    rng = np.random.RandomState(3)
    pts = rng.randint(0, 3, (30000, 4)).astype(np.float32)
    q = np.array([[1, 1, 1, 1], [0, 0, 0, 0], [0.5, 2, 1, 0], [7, 7, 7, 7]], np.float32)
    idx = capi.Index(pts, None, None)
    for k in (1, 100, 1000, 1025, 2000):
        ids, dists, _ = idx.bruteforce(q, k)
        oi, od = orc.bruteforce(pts, q, k, order=SEQ)
        assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()
    # a mix in one batch: rows with few ties next to rows with many
    mixed = np.concatenate([pts[:15000], synth.gaussian_matrix(5, 15000, 4)])
    idx2 = capi.Index(mixed, None, None)
    q2 = np.concatenate([q, synth.gaussian_matrix(6, 4, 4)])
    ids, dists, _ = idx2.bruteforce(q2, 64)
    oi, od = orc.bruteforce(mixed, q2, 64, order=SEQ)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()
    idx.close(), idx2.close()


def test_bruteforce_candidate_lists_that_overflow_go_through_the_matrix(orc):
    """The selection inside the matrix-core kernel keeps what does not exceed a bound taken from a sample of the base.
    Where that is more than a list holds -- most of the base at one and the same distance, or a sample that is
    tombstoned away so that no bound exists -- the call falls back to the distance matrix, with the same result."""
    n, dim, k = 20000, 16, 10
    rng = np.random.RandomState(5)
    q = synth.gaussian_matrix(8, 7, dim)
    # (a) all but 50 rows are the same vector: every one of them ties at the bound
    base = np.ones((n, dim), np.float32)
    base[rng.choice(n, 50, replace=False)] = synth.gaussian_matrix(9, 50, dim)
    idx = capi.Index(base, None, None)
    ids, dists, _ = idx.bruteforce(q, k)
    assert idx.bruteforce_last_fused() == 0
    oi, od = orc.bruteforce(base, q, k, order=SEQ)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()
    idx.close()
    # (b) everything but the last 300 ids is tombstoned: the sample holds fewer live points than candidates are kept
    base = synth.gaussian_matrix(10, n, dim)
    mask = np.zeros((n + 31) // 32, np.uint32)
    dead = np.arange(n - 300)
    np.bitwise_or.at(mask, dead >> 5, (np.uint32(1) << (dead & 31).astype(np.uint32)))
    idx = capi.Index(base, None, None)
    idx.set_deleted(mask)
    ids, dists, _ = idx.bruteforce(q, k, have_delete=True)
    assert idx.bruteforce_last_fused() == 0
    oi, od = orc.bruteforce(base, q, k, deleted=mask, order=SEQ)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()
    assert (ids >= n - 300).all()
    idx.close()


def test_bruteforce_segments(orc):
    # more base points than one pass holds (4M): per-segment winners are merged
    n, dim, Q, k = 5 * 1000 * 1000, 8, 40, 50
    base = workloads.gaussian_base(61, n, dim)
    q = synth.shifted_queries(Q, dim, 6, 7, 8)
    idx = capi.Index(base, ring(n), np.array([0], np.int32))
    ids, dists, _ = idx.bruteforce(q, k)
    idx.close()
    oi, od = orc.bruteforce(base, q, k, order=SEQ)
    assert np.array_equal(ids, oi) and dists.tobytes() == od.tobytes()


def test_bruteforce_ground_truth_at_full_size(orc):
    import torch
    n, dim, Q, k = 1000000, 200, 10000, 100
    base = workloads.gaussian_base(2001, n, dim)
    q = synth.shifted_queries(Q, dim, 2002, 2003, 2004)
    idx = capi.Index(base, ring(n), np.array([0], np.int32))
    ids, dists, t = idx.bruteforce(q, k)
    assert idx.bruteforce_last_fused() == 1 and idx.bruteforce_last_redone() == 0
    idx.bruteforce_exact_only(2)
    ids_m, dists_m, t_m = idx.bruteforce(q, k)
    idx.bruteforce_exact_only(0)
    assert np.array_equal(ids_m, ids) and dists_m.tobytes() == dists.tobytes()
    print("candidates selected inside the kernel: %.3f s; from the distance matrix: %.3f s" % (t, t_m), flush=True)
    pairs = float(Q) * n * dim
    print("brute force 10k x 1M x 200: %.3f s, %.2f T pair-dims/s (%.1f TFLOP/s at 3 flop per pair-dim)" %
          (t, pairs / t / 1e12, 3 * pairs / t / 1e12), flush=True)
    assert (np.diff(dists, axis=1) >= 0).all()
    sub = np.arange(0, Q, 313)
    t0 = time.perf_counter()
    oi, od = orc.bruteforce(base, q[sub], k, order=SEQ)
    t_cpu = time.perf_counter() - t0
    print("oracle on %d host threads: %d queries in %.2f s = %.0f queries/s (device: %.0f queries/s)" %
          (orc.max_threads(), len(sub), t_cpu, len(sub) / t_cpu, Q / t), flush=True)
    assert np.array_equal(ids[sub], oi) and dists[sub].tobytes() == od.tobytes()
    # agrees with a matmul-based top-k (|b|^2 - 2 q.b, another arithmetic altogether) up to near-ties
    tb, tq = torch.from_numpy(base).cuda(), torch.from_numpy(q[sub]).cuda()
    gt = torch.topk((tb * tb).sum(1)[None, :] - 2.0 * (tq @ tb.T), k, dim=1, largest=False).indices.cpu().numpy()
    del tb, tq
    agree = np.mean([len(set(a.tolist()) & set(b.tolist())) for a, b in zip(ids[sub], gt)]) / k
    assert agree > 0.999
    # device-pointer entry, and the gt-file layout on disk
    tq = torch.from_numpy(q[:256]).cuda()
    d_ids = torch.empty((256, k), dtype=torch.int32, device="cuda")
    idx.bruteforce_device(tq.data_ptr(), d_ids.data_ptr(), None, 256, k)
    assert np.array_equal(d_ids.cpu().numpy(), ids[:256])
    idx.close()
