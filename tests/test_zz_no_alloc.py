"""The entry point that allocates nothing (coral_search_gpu_noalloc: scratch in a fixed block of device memory
inside the library) against coral_search_gpu on the same inputs: ids and distance bits equal, on two calls in a
row, the second with a smaller input, for both traversal policies, with tombstones, and on a second index that
shares the same block; sizes beyond the block are turned away.  The device's free memory is read around every such
call: it must not move (the first launch of a kernel in a process aside, where the runtime may set up its own
per-queue memory)."""
import numpy as np
import pytest

from coral_amd import capi, synth, workloads
from util import make_queries, ragged

pytestmark = pytest.mark.gpu


def _reference(idx, d_q, Q, k, L, policy, have_delete, torch):
    ids = torch.full((Q, k), -7, dtype=torch.int32, device="cuda")
    dists = torch.full((Q, k), -7.0, dtype=torch.float32, device="cuda")
    idx.prepare(Q, L, policy=policy, best_first_in_lds=True)
    idx.search_device(d_q.data_ptr(), ids.data_ptr(), dists.data_ptr(), Q, k, policy=policy, have_delete=have_delete)
    torch.cuda.synchronize()
    return ids.cpu().numpy(), dists.cpu().numpy()


FREE_MEMORY_MOVED = []  # per coral_search_gpu_noalloc call of this file: free device memory before - after, bytes


def _noalloc(idx, d_q, Q, k, L, policy, have_delete, torch):
    ids = torch.full((Q, k), -7, dtype=torch.int32, device="cuda")
    dists = torch.full((Q, k), -7.0, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    idx.search_device_noalloc(d_q.data_ptr(), ids.data_ptr(), dists.data_ptr(), Q, k, L, policy=policy,
                              have_delete=have_delete)
    torch.cuda.synchronize()  # the call does not wait for its kernels; the index's stream is a blocking stream
    FREE_MEMORY_MOVED.append(free_before - torch.cuda.mem_get_info()[0])
    return ids.cpu().numpy(), dists.cpu().numpy()


def test_no_alloc_entry_point_equals_the_allocating_one():
    import torch
    n, dim, R = 30000, 200, 32
    base = synth.gaussian_matrix(91, n, dim)
    nbrs = ragged(workloads.exact_knn_graph(base, R), 17, keep_min=1)
    starts = np.random.RandomState(5).choice(n, 16, replace=False).astype(np.int32)
    mask = synth.tombstone_mask(n, 77, modulo=7)
    idx = capi.Index(base, nbrs, starts)
    idx.set_deleted(mask)
    q_all = make_queries(700, dim, 901)
    # two calls in a row per setting, the second with a smaller input (fewer queries, shorter beam, smaller k):
    # what the first left in the block must not show in the second.  (The very first call finds no coded copy of the
    # vectors on the index and reads every row in full; the prepare of the comparison leaves one, and every later
    # rounds call screens on it.)
    for policy in (capi.POLICY_ROUNDS, capi.POLICY_BEST_FIRST):
        for have_delete in (False, True):
            for Q, k, L in ((700, 100, 256), (130, 10, 64)):
                print("noalloc case", dict(policy=policy, have_delete=have_delete, Q=Q, k=k, L=L), flush=True)
                d_q = torch.from_numpy(q_all[:Q]).cuda()
                got = _noalloc(idx, d_q, Q, k, L, policy, have_delete, torch)
                want = _reference(idx, d_q, Q, k, L, policy, have_delete, torch)
                assert np.array_equal(got[0], want[0])
                assert got[1].tobytes() == want[1].tobytes()
    # a second index on the same GPU uses the same block.  More nodes than a bitmap in LDS can cover (1.3 M), so the
    # visited set is the table of cells, and at L = 2048 a query outgrows it: ids go to the per-workgroup overflow
    # bitmaps of the block (fewer workgroups than usual, so that each has one) -- and the next, smaller call finds
    # them clean.  (A graph of random neighbours; the check is against coral_search_gpu, no oracle needed.)
    rng = np.random.RandomState(8)
    n3, dim3 = 1300000, 8
    base3 = rng.standard_normal((n3, dim3)).astype(np.float32)
    nbrs3 = rng.randint(0, n3, (n3, 16)).astype(np.int32)
    idx3 = capi.Index(base3, nbrs3, np.array([1, 70000, 1299999], np.int32))
    q3 = make_queries(300, dim3, 903)
    for Q, k, L in ((300, 100, 2048), (16, 5, 32)):
        print("noalloc case on 1.3 M nodes", dict(Q=Q, k=k, L=L), flush=True)
        d_q = torch.from_numpy(q3[:Q]).cuda()
        got = _noalloc(idx3, d_q, Q, k, L, capi.POLICY_ROUNDS, False, torch)
        ids = torch.empty((Q, k), dtype=torch.int32, device="cuda")
        dists = torch.empty((Q, k), dtype=torch.float32, device="cuda")
        idx3.prepare(Q, L)
        st = idx3.search_device(d_q.data_ptr(), ids.data_ptr(), dists.data_ptr(), Q, k)
        torch.cuda.synchronize()
        assert st.spills > 0 if L == 2048 else st.spills == 0
        assert np.array_equal(got[0], ids.cpu().numpy()) and got[1].tobytes() == dists.cpu().numpy().tobytes()
    idx3.close()
    # and a small one
    n2, dim2 = 5000, 64
    base2 = synth.gaussian_matrix(92, n2, dim2)
    nbrs2 = workloads.exact_knn_graph(base2, 16)
    idx2 = capi.Index(base2, nbrs2, np.array([3, 999], np.int32))
    d_q2 = torch.from_numpy(make_queries(50, dim2, 902)).cuda()
    got = _noalloc(idx2, d_q2, 50, 20, 100, capi.POLICY_ROUNDS, False, torch)  # (the first call on a fresh index)
    want = _reference(idx2, d_q2, 50, 20, 100, capi.POLICY_ROUNDS, False, torch)
    assert np.array_equal(got[0], want[0]) and got[1].tobytes() == want[1].tobytes()
    # no call took device memory: the same call again (its launch plan is kept: nothing but two fills and the launch)
    # and all the calls above, the first launches of each kernel form in this process reported apart
    for _ in range(3):
        again = _noalloc(idx2, d_q2, 50, 20, 100, capi.POLICY_ROUNDS, False, torch)
        assert np.array_equal(again[0], want[0]) and again[1].tobytes() == want[1].tobytes()
    print("free device memory moved per call (bytes):", FREE_MEMORY_MOVED, flush=True)
    assert all(d == 0 for d in FREE_MEMORY_MOVED[-3:])
    assert sum(1 for d in FREE_MEMORY_MOVED if d != 0) <= 3, FREE_MEMORY_MOVED  # (three kernel forms: dim 200, 8, 64)
    # beyond the block: clear errors, nothing launched
    d_q = torch.from_numpy(q_all[:8]).cuda()
    out = torch.empty((8, 10), dtype=torch.int32, device="cuda")
    for Q, k, L in ((16385, 10, 64), (8, 10, 4096), (8, 100, 64), (0, 10, 64)):
        with pytest.raises(capi.CoralError) as e:
            idx.search_device_noalloc(d_q.data_ptr(), out.data_ptr(), None, Q, k, L)
        assert e.value.code == capi.ERR_ARG
    idx.set_deleted(None)
    with pytest.raises(capi.CoralError) as e:
        idx.search_device_noalloc(d_q.data_ptr(), out.data_ptr(), None, 8, 10, 64, have_delete=True)
    assert e.value.code == capi.ERR_STATE
    idx2.close()
    idx.close()
