"""Graph construction on the device (src/upd_gpu.cu:12-303, src/enhance.cu:131-208, 334-575, 660-803,
src/index_gpu.cpp:308-580) against the oracle's restatement: rows, per-neighbour distances, degrees and start ids
must be identical, batch by batch and for the whole pipeline."""
import numpy as np
import pytest

from coral_amd import capi, synth
from util import make_queries

pytestmark = pytest.mark.gpu
WAVE64 = 3  # the search kernel's summation order
SEQ = 0  # one thread walks the row: the brute-force kernels and the builder


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_same_state(idx, st):
    nbrs, dists, deg, _ = idx.get_graph(with_build_state=True)
    assert np.array_equal(deg, st.deg)
    assert np.array_equal(nbrs, st.nbrs)
    assert dists.tobytes() == st.dists.tobytes()


def base_of(n, dim, seed, metric):
    base = synth.gaussian_matrix(seed, n, dim)
    return synth.normalize_rows(base) if metric == capi.IP else base


@pytest.mark.parametrize("n,dim,R,kb,batch,metric,need_discard,seed", [
    (3000, 32, 8, 10, 64, capi.L2, 1, 0),
    (3000, 32, 8, 10, 64, capi.L2, 0, 1),
    (4000, 64, 32, 100, 24, capi.L2, 1, 2),
    (4000, 64, 32, 100, 24, capi.IP, 1, 3),
    (2000, 200, 16, 33, 40, capi.L2, 1, 4),
    (2000, 8, 5, 128, 9, capi.IP, 0, 5),
    (500, 4, 3, 2, 300, capi.L2, 1, 6),
    (1500, 16, 6, 12, 50, capi.L2, 2, 7),  # 2: filling and non-filling batches take turns on the same rows
])
def test_nap_batches_equal_the_oracle(orc, n, dim, R, kb, batch, metric, need_discard, seed):
    rng = np.random.RandomState(seed)
    base = base_of(n, dim, 50 + seed, metric)
    if seed == 6:
        base = np.round(base)  # ties and duplicate points
    idx = capi.Index(base, None, None, metric=metric)
    idx.build_begin(R)
    st = orc.GraphState(n, R)
    for it in range(6 if need_discard == 2 else 5):
        if it % 2 == 0:  # clusters of true neighbours: the exact kb-NN of shifted queries
            q = make_queries(batch, dim, 900 + 10 * seed + it, "ip" if metric == capi.IP else "l2")
            knn, _ = orc.bruteforce(base, q, kb, metric, order=SEQ)
        else:  # arbitrary clusters, many ids shared between the clusters of the batch
            pool = rng.choice(n, min(n, 4 * kb + 50), replace=False)
            knn = np.stack([rng.choice(pool, kb, replace=False) for _ in range(batch)]).astype(np.int32)
        t_knn = dev(knn)
        fill = (it + 1) % 2 if need_discard == 2 else need_discard
        idx.build_nap_batch(t_knn.data_ptr(), knn.shape[0], kb, fill)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=fill)
        assert_same_state(idx, st)
    idx.close()


@pytest.mark.parametrize("metric,R,kn,seed", [(capi.L2, 8, 20, 0), (capi.IP, 32, 100, 1), (capi.L2, 5, 9, 2)])
def test_enhance_batches_equal_the_oracle(orc, metric, R, kn, seed):
    rng = np.random.RandomState(seed)
    n, dim, linked_n = 3000, 32, 2400
    base = base_of(n, dim, 70 + seed, metric)
    idx = capi.Index(base, None, None, metric=metric)
    idx.build_begin(R)
    st = orc.GraphState(n, R)
    for it in range(4):  # a graph over the first linked_n nodes, rows of every fill level
        knn = np.stack([rng.choice(linked_n, 12, replace=False) for _ in range(150)]).astype(np.int32)
        t_knn = dev(knn)
        idx.build_nap_batch(t_knn.data_ptr(), 150, 12, it % 2)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=it % 2)
    linked = np.where(st.deg > 0)[0].astype(np.int32)
    sub = base[linked]
    for lo in (linked_n, linked_n + 300):
        iso = np.arange(lo, lo + 300, dtype=np.int32)
        ids, dd = orc.bruteforce(sub, base[iso], kn, metric, order=SEQ)  # the nearest linked nodes stand in for the search
        ids = linked[ids]
        ids[5, kn // 2:] = -1  # a short list
        t_iso, t_ids, t_dd = dev(iso), dev(ids), dev(dd)  # named: the device buffers must outlive the call
        ins, rej = idx.build_enhance_batch(t_iso.data_ptr(), t_ids.data_ptr(), t_dd.data_ptr(), iso.size, kn)
        stats = orc.enhance_batch(base, st, iso, ids, dd, metric=metric)
        assert (ins, rej) == (stats[0], stats[1])
        assert_same_state(idx, st)
        linked = np.where(st.deg > 0)[0].astype(np.int32)
        sub = base[linked]
    assert (st.deg[linked_n:linked_n + 600] > 0).all()
    idx.close()


def test_randomised_shapes_of_both_steps_equal_the_oracle(orc):
    """Seeded random sizes, widths, cluster sizes, metrics and fill modes, small enough for the oracle; each case
    runs a few batch updates and one enhancement batch."""
    rng = np.random.RandomState(2024)
    for case in range(30):
        dim = int(rng.choice([4, 8, 12, 36, 64, 100, 128, 200, 256]))
        R = int(rng.randint(1, 33))
        kb = int(rng.choice([2, 3, 5, 17, 40, 64, 100, 128]))
        n = int(rng.randint(kb + 20, 3000))
        batch = int(rng.randint(1, 80))
        metric = int(rng.randint(0, 2))
        fill = int(rng.randint(0, 2))
        print("case %d: n=%d dim=%d R=%d kb=%d batch=%d metric=%d fill=%d" % (case, n, dim, R, kb, batch, metric, fill),
              flush=True)
        base = base_of(n, dim, 1000 + case, metric)
        if case % 7 == 0:
            base = np.round(base * 2) / 2 if metric == capi.L2 else base  # ties
        linked_n = max(kb + 1, (2 * n) // 3)
        idx = capi.Index(base, None, None, metric=metric)
        idx.build_begin(R)
        st = orc.GraphState(n, R)
        all_knn = []
        for it in range(3):
            knn = np.stack([rng.choice(linked_n, kb, replace=False) for _ in range(batch)]).astype(np.int32)
            all_knn.append(knn)
            t_knn = dev(knn)
            idx.build_nap_batch(t_knn.data_ptr(), batch, kb, fill)
            orc.nap_batch(base, st, knn, metric=metric, need_discard=fill)
            assert_same_state(idx, st)
        linked = np.where(st.deg > 0)[0].astype(np.int32)
        iso = np.where(st.deg == 0)[0].astype(np.int32)[:50]
        kn = int(min(linked.size, rng.choice([1, 7, 33, 100, 160])))
        if iso.size and kn:
            ids, dd = orc.bruteforce(base[linked], base[iso], kn, metric, order=SEQ)
            ids = linked[ids]
            if kn > 2:
                ids[0, kn // 2:] = -1
            t_iso, t_ids, t_dd = dev(iso), dev(ids), dev(dd)
            ins, rej = idx.build_enhance_batch(t_iso.data_ptr(), t_ids.data_ptr(), t_dd.data_ptr(), iso.size, kn)
            stats = orc.enhance_batch(base, st, iso, ids, dd, metric=metric)
            assert (ins, rej) == (stats[0], stats[1])
            assert_same_state(idx, st)
        # the second-phase step over some linked nodes: what is nearest among the linked (themselves first) + own row
        linked = np.where(st.deg > 0)[0].astype(np.int32)
        top = rng.choice(linked, min(40, linked.size), replace=False).astype(np.int32)
        k2 = int(min(linked.size, rng.choice([1, 6, 30, 100, 128])))
        ids, dd = orc.bruteforce(base[linked], base[top], k2, metric, order=SEQ)
        ids = linked[ids]
        if k2 > 2:
            ids[0, k2 // 2:] = -1
        t_top, t_ids, t_dd = dev(top), dev(ids), dev(dd)
        ins, rej = idx.build_enhance_top_batch(t_top.data_ptr(), t_ids.data_ptr(), t_dd.data_ptr(), top.size, k2)
        stats = orc.enhance_top_batch(base, st, top, ids, dd, metric=metric)
        assert (ins, rej) == (stats[0], stats[1])
        assert_same_state(idx, st)
        got_ids, got_hits = idx.build_top_hit_ids(min(n, 50))
        want_hits = np.zeros(n, np.uint32)
        for knn in all_knn:
            np.add.at(want_hits, knn.ravel(), 1)
        assert np.array_equal(got_hits, want_hits) and got_ids.tolist() == orc.top_hit_ids(want_hits, min(n, 50)).tolist()
        idx.close()


def oracle_pipeline(orc, base, aux, metric, p):
    """IndexGPU::BuildGPU composed from the oracle's pieces, in the order coral_build_graph documents."""
    n = base.shape[0]
    st = orc.GraphState(n, p.R)
    hits = np.zeros(n, np.uint32)
    for a0 in range(0, aux.shape[0], p.batch):
        knn, _ = orc.bruteforce(base, aux[a0:a0 + p.batch], p.k_b, metric, order=SEQ)
        np.add.at(hits, knn.ravel(), 1)
        orc.nap_batch(base, st, knn, metric=metric, need_discard=p.need_discard)
    iso = np.where(st.deg == 0)[0].astype(np.int32)
    first = int(np.where(st.deg > 0)[0][0]) if p.first_start_id < 0 else p.first_start_id
    starts = None

    def phase(nodes, step):
        nonlocal starts
        for i in range(0, nodes.size, p.enhance_search_batch):
            part = nodes[i:i + p.enhance_search_batch]
            starts = orc.fps(st.nbrs, first, p.n_start)
            prob = orc.Problem(base, st.nbrs.copy(), starts)
            ids, dd, _, _ = orc.search_B(prob, base[part], p.k_b, p.enhance_L, metric=metric, start_order=WAVE64,
                                         nbr_order=WAVE64)
            for j in range(0, part.size, p.enhance_nap_batch):
                sl = slice(j, j + p.enhance_nap_batch)
                step(base, st, part[sl], ids[sl], dd[sl], metric=metric)

    if p.connect_enhance:
        phase(iso, orc.enhance_batch)
        if p.top_hit_num > iso.size:  # the second phase: the nodes most clusters contain
            phase(orc.top_hit_ids(hits, min(p.top_hit_num - iso.size, n)), orc.enhance_top_batch)
    if starts is None:
        starts = orc.fps(st.nbrs, first, p.n_start)
    return st, starts, iso.size


@pytest.mark.parametrize("metric,ce,seed,top_hit_num", [(capi.L2, 1, 0, 0), (capi.IP, 1, 1, 0), (capi.L2, 0, 2, 0),
                                                        (capi.L2, 1, 3, 9000), (capi.IP, 1, 4, 1000000)])
def test_whole_construction_equals_the_oracle_pipeline(orc, metric, ce, seed, top_hit_num):
    n, dim, A = 12000, 48, 900
    base = base_of(n, dim, 300 + seed, metric)
    aux = make_queries(A, dim, 400 + seed, "ip" if metric == capi.IP else "l2")
    p = capi.build_params(R=16, k_b=24, batch=128, connect_enhance=ce, enhance_search_batch=5000,
                          enhance_nap_batch=700, enhance_L=64, n_start=8, top_hit_num=top_hit_num)
    idx = capi.Index(base, None, None, metric=metric)
    stats = idx.build_graph(aux, p)
    nbrs, dists, deg, starts = idx.get_graph(with_build_state=True)
    st, want_starts, iso_n = oracle_pipeline(orc, base, aux, metric, p)
    assert stats.isolated == iso_n and iso_n > 1000
    assert stats.top_hit_nodes == (min(top_hit_num - iso_n, n) if top_hit_num > iso_n else 0)
    if top_hit_num:
        assert stats.top_hit_nodes > 0 and stats.top_reverse_edges > 0
        print("second phase over %d nodes, %d reverse edges" % (stats.top_hit_nodes, stats.top_reverse_edges), flush=True)
    assert stats.batches == (A + p.batch - 1) // p.batch
    assert np.array_equal(deg, st.deg) and np.array_equal(nbrs, st.nbrs) and dists.tobytes() == st.dists.tobytes()
    assert starts.tolist() == want_starts.tolist()
    assert stats.edges == int(st.deg.sum())
    if ce:
        assert (deg > 0).all()
    # the built index answers searches like an index created from the downloaded rows
    idx.build_end()
    q = make_queries(50, dim, 77, "ip" if metric == capi.IP else "l2")
    ids, dd, _ = idx.search(q, 10, 64)
    idx.close()
    idx2 = capi.Index(base, nbrs, starts, metric=metric)
    ids2, dd2, _ = idx2.search(q, 10, 64)
    idx2.close()
    assert np.array_equal(ids, ids2) and dd.tobytes() == dd2.tobytes()


def test_enhancement_alone_on_a_resumed_build_equals_the_whole_construction():
    """rows, distances and hit counts of a construction without enhancement, handed to a new index
    (coral_build_resume), then coral_build_connect_enhance: the state a construction with enhancement ends in."""
    n, dim, A = 12000, 48, 900
    base = base_of(n, dim, 310, capi.L2)
    aux = make_queries(A, dim, 410)
    kw = dict(R=16, k_b=24, batch=128, enhance_search_batch=5000, enhance_nap_batch=700, enhance_L=64, n_start=8,
              top_hit_num=9000)
    idx = capi.Index(base, None, None)
    idx.build_graph(aux, capi.build_params(connect_enhance=1, **kw))
    want = idx.get_graph(with_build_state=True)
    idx.close()
    idx = capi.Index(base, None, None)
    idx.build_graph(aux, capi.build_params(connect_enhance=0, **kw))
    nbrs, dists, deg, _ = idx.get_graph(with_build_state=True)
    _, hits = idx.build_top_hit_ids(0)
    idx.close()
    assert (deg == 0).sum() > 1000 and hits.sum() == A * 24
    idx = capi.Index(base, None, None)
    idx.build_resume(nbrs, dists, hits)
    got = idx.get_graph(with_build_state=True)
    assert np.array_equal(got[0], nbrs) and got[1].tobytes() == dists.tobytes() and np.array_equal(got[2], deg)
    stats = idx.build_connect_enhance(capi.build_params(connect_enhance=1, **kw))
    got = idx.get_graph(with_build_state=True)
    assert stats.isolated == (deg == 0).sum() and stats.top_hit_nodes == 9000 - stats.isolated
    for g, w in zip(got, want):
        assert g.tobytes() == w.tobytes()
    # rows that no build could have left are turned away, and the index stays as it was
    broken = nbrs.copy()
    broken[5, 3] = n
    with pytest.raises(capi.CoralError) as e:
        idx.build_resume(broken, dists, hits)
    assert e.value.code == 2 and "row 5" in str(e.value)
    broken = nbrs.copy()
    row = int(np.where(deg == 0)[0][0])
    broken[row, 1] = 7  # a neighbour after the end of the row
    with pytest.raises(capi.CoralError) as e:
        idx.build_resume(broken, dists, None)
    assert e.value.code == 2 and "row %d" % row in str(e.value)
    assert np.array_equal(idx.get_graph(with_build_state=True)[0], want[0])
    idx.close()


def test_searches_during_a_build_report_and_change_nothing(orc):
    """GPUFuncs::test_search at the reference's points of a construction (include/gpufuncs.cuh:688-702; every
    test_search_frequency batches src/index_gpu.cpp:525, after the isolated nodes src/enhance.cu:814, after every search
    batch of the most-hit nodes :852, on the finished graph src/index_gpu.cpp:376-378): the watched construction ends
    in the state of the unwatched one, and each report is the search it says it is."""
    import torch
    n, dim, A, Q, k, L = 12000, 48, 900, 64, 10, 64
    base = base_of(n, dim, 311, capi.L2)
    aux = make_queries(A, dim, 411)
    q = make_queries(Q, dim, 511)
    gt, _ = orc.bruteforce(base, q, k)
    kw = dict(R=16, k_b=24, batch=128, enhance_search_batch=2500, enhance_nap_batch=700, enhance_L=64, n_start=8,
              top_hit_num=9000)
    idx = capi.Index(base, None, None)
    idx.build_graph(aux, capi.build_params(**kw))
    want = idx.get_graph(with_build_state=True)
    idx.close()
    mon = capi.Monitor(q, gt, L)
    p = mon.attach(capi.build_params(**kw), every_batches=3)
    idx = capi.Index(base, None, None)
    stats = idx.build_graph(aux, p)
    got = idx.get_graph(with_build_state=True)
    for g, w in zip(got, want):
        assert g.tobytes() == w.tobytes()
    phases = [r[0] for r in mon.reports]
    top_n = 9000 - stats.isolated
    assert stats.batches == 8 and phases[:2] == [capi.MONITOR_BATCHES] * 2  # after the batches numbered 3 and 6
    assert [r[1:3] for r in mon.reports[:2]] == [(512, A), (896, A)]
    assert phases[2] == capi.MONITOR_ISOLATED and mon.reports[2][1:3] == (stats.isolated, stats.isolated)
    tops = [r for r in mon.reports if r[0] == capi.MONITOR_TOP]
    assert [r[1] for r in tops] == list(range(2500, top_n, 2500)) + [top_n] and all(r[2] == top_n for r in tops)
    assert phases[-1] == capi.MONITOR_DONE and len(phases) == 3 + len(tops) + 1
    # the last report against a search of the finished graph by hand, and against the oracle on that graph
    d_q = dev(q)
    d_ids = torch.empty((Q, k), dtype=torch.int32, device="cuda")
    idx.prepare(Q, L)
    st = idx.search_device(d_q.data_ptr(), d_ids.data_ptr(), None, Q, k)
    hits = idx.verify(d_ids.data_ptr(), dev(gt).data_ptr(), Q, k)
    assert mon.reports[-1][3] == hits and mon.reports[-1][4] == st.hops
    oi, _, os_, _ = orc.search_B(orc.Problem(base, got[0], got[3]), q, k, L, start_order=WAVE64, nbr_order=WAVE64)
    assert hits == orc.recall_hits(oi, gt, k) and st.hops == os_[:, 0].sum()
    assert mon.reports[0][3] < mon.reports[2][3] <= Q * k
    # GPUFuncs::test_search by itself: the same search again, reported under the phase the caller names
    idx.build_test_search(p, capi.MONITOR_TOP, 5, 7)
    assert mon.reports[-1][:5] == (capi.MONITOR_TOP, 5, 7, hits, st.hops)
    idx.build_test_search(capi.build_params(**kw))  # no monitor: nothing happens
    assert len(mon.reports) == len(phases) + 1
    # a monitor that cannot be searched for is turned away before the build starts changing rows
    bad = capi.Monitor(q, gt, k - 1)
    with pytest.raises(capi.CoralError) as e:
        idx.build_test_search(bad.attach(capi.build_params(**kw)))
    assert e.value.code == capi.ERR_ARG
    idx.close()
    idx = capi.Index(base, None, None)
    with pytest.raises(capi.CoralError) as e:
        idx.build_graph(aux, bad.attach(capi.build_params(**kw)))
    assert e.value.code == capi.ERR_ARG and not bad.reports
    with pytest.raises(capi.CoralError):  # nothing was begun
        idx.get_graph(with_build_state=True)
    idx.close()
    # without the enhancement there is no closing search (src/index_gpu.cpp:376: CE && test_search)
    mon2 = capi.Monitor(q, gt, L)
    idx = capi.Index(base, None, None)
    idx.build_graph(aux, mon2.attach(capi.build_params(connect_enhance=0, **kw), every_batches=3))
    assert [r[0] for r in mon2.reports] == [capi.MONITOR_BATCHES] * 2
    assert [r[3:5] for r in mon2.reports] == [r[3:5] for r in mon.reports[:2]]
    idx.close()


def test_builder_argument_errors():
    base = synth.gaussian_matrix(1, 100, 8)
    idx = capi.Index(base, None, None)
    knn = dev(np.arange(20, dtype=np.int32).reshape(2, 10))
    with pytest.raises(capi.CoralError):  # not begun
        idx.build_nap_batch(knn.data_ptr(), 2, 10)
    with pytest.raises(capi.CoralError):
        idx.build_begin(33)
    idx.build_begin(4)
    bad = dev(np.array([[1, 2, 100]], np.int32))  # id == n
    with pytest.raises(capi.CoralError) as e:
        idx.build_nap_batch(bad.data_ptr(), 1, 3)
    assert e.value.code == 2
    with pytest.raises(capi.CoralError):
        idx.build_nap_batch(knn.data_ptr(), 2, 129)
    idx.build_nap_batch(knn.data_ptr(), 2, 10)
    nbrs, dists, deg, _ = idx.get_graph(with_build_state=True)
    assert (deg[:20] > 0).all() and (deg[20:] == 0).all()
    with pytest.raises(capi.CoralError) as e:  # rows exist, entry points do not yet
        idx.search(base[:3], 2, 8)
    assert e.value.code == capi.ERR_STATE and "no start ids" in str(e.value)
    idx.build_end()
    with pytest.raises(capi.CoralError):
        idx.get_graph(with_build_state=True)
    idx.close()


def test_build_driver_writes_the_index_directory_the_search_driver_reads(orc, tmp_path):
    """test_build_pipeline -> graph.part0.idx/.data + graph.search_start_ids -> test_search_pipeline."""
    import os
    import subprocess
    from coral_amd import formats
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    n, dim, A, Q, k = 15000, 48, 1100, 100, 10
    base = base_of(n, dim, 500, capi.L2)
    aux = make_queries(A, dim, 600)
    q = make_queries(Q, dim, 700)
    work = tmp_path / "run"
    os.makedirs(work / "cwd")
    formats.fbin_write(work / "base.fbin", base)
    formats.fbin_write(work / "aux.fbin", aux)
    formats.fbin_write(work / "query.fbin", q)
    gt, _ = orc.bruteforce(base, q, k)
    formats.gt_write(work / "gt.bin", gt)
    (work / "config.json").write_text('{"batch": 256, "enhance_nap_batch": 1000, "search_start_nodes_num": 8, '
                                      '"top_hit_num": 20000, "test_search_frequency": 2}')
    cli = os.path.join(root, "coral_amd", "lib", "test_build_pipeline")
    args = [cli, "--data_type", "float", "--dist", "l2", "--dataset", "syn", "--base_data_path", str(work / "base.fbin"),
            "--sampled_query_data_path", str(work / "aux.fbin"), "--M_pjbp", "16", "--k", "24", "--CE", "1",
            "--query_thres", "1.0", "--config_file", str(work / "config.json"), "-T", "8",
            "--query_test_file", str(work / "query.fbin"), "--gt_test_file", str(work / "gt24.bin")]
    gt24, _ = orc.bruteforce(base, q, 24)
    formats.gt_write(work / "gt24.bin", gt24)
    build_args = args
    r = subprocess.run(args, cwd=work / "cwd", capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr + r.stdout
    index_dir = work / "indexes" / "syn_l2_16_1.0_1"  # ../indexes/<dataset>_<dist>_<R>_<thres>_<CE>
    assert "Save index to ../indexes/syn_l2_16_1.0_1" in r.stdout
    nbrs, dists = formats.graph_dir_read(index_dir, n, 16, want_dists=True)
    starts = formats.start_ids_read(index_dir)
    # the same construction through the C ABI
    assert "most-hit nodes rewired: " in r.stdout and "most-hit nodes rewired: 0," not in r.stdout
    p = capi.build_params(R=16, k_b=24, batch=256, enhance_nap_batch=1000, n_start=8, top_hit_num=20000)
    idx = capi.Index(base, None, None)
    idx.build_graph(aux, p)
    want_nbrs, want_dists, deg, want_starts = idx.get_graph(with_build_state=True)
    idx.close()
    assert np.array_equal(nbrs, want_nbrs) and dists.tobytes() == want_dists.tobytes()
    assert starts.tolist() == want_starts.tolist() and len(starts) == 8
    assert (deg > 0).all()
    # the search the build driver ran on the finished graph (test_beam_capacity = 512, k = the cluster size)
    line = [l for l in r.stdout.splitlines() if l.startswith("test search:")][0]
    o24, _, os24, _ = orc.search_B(orc.Problem(base, nbrs, starts), q, 24, 512, start_order=WAVE64, nbr_order=WAVE64)
    assert "L 512, recall@24 " in line
    # the searches of the same test queries while the graph grew (config.json "test_search", on by default; five
    # batches, one search after those numbered 2 and 4): they left the graph as the unwatched construction above
    # made it, and the last of them, on the finished graph, says what the driver's own closing search says
    watch = [l for l in r.stdout.splitlines() if "Testing recall-" in l]
    assert len(watch) == 5 and watch[0].startswith("[batches 768/1100]") and watch[1].startswith("[batches 1100/1100]")
    assert watch[4].startswith("[graph complete 1100/1100]")
    assert watch[2].startswith("[isolated nodes attached ") and watch[3].startswith("[most-hit nodes ")
    recalls = [float(l.split("Testing recall-")[1].split("%")[0]) for l in watch]
    assert recalls[0] < recalls[-1] and recalls[1] < recalls[2]  # (isolated nodes cannot be found before they are attached)
    assert abs(recalls[-1] - float(line.split("recall@24 ")[1].split(" %")[0])) < 1e-3
    assert abs(float(watch[-1].split("avg_hops-")[1].split(",")[0]) - os24[:, 0].sum() / Q) < 1e-2
    assert abs(float(line.split("recall@24 ")[1].split(" %")[0]) - 100.0 * orc.recall_hits(o24, gt24, 24) / (Q * 24)) < 1e-3
    assert abs(float(line.split("avg hops ")[1].split(",")[0]) - os24[:, 0].sum() / Q) < 1e-2
    # and the search driver on that directory
    cli = os.path.join(root, "coral_amd", "lib", "test_search_pipeline")
    args = [cli, "--data_type", "float", "--dist", "l2", "--base_data_path", str(work / "base.fbin"), "--dataset",
            "syn", "--query_path", str(work / "query.fbin"), "--gt_path", str(work / "gt.bin"), "--k", str(k),
            "--max_degree", "16", "--L", "64", "--config_file", str(work / "config.json")]
    r = subprocess.run(args, cwd=work / "cwd", capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    row = [l for l in r.stdout.splitlines() if l.startswith("64\t")][0].split()
    oi, _, _, _ = orc.search_B(orc.Problem(base, nbrs, starts), q, k, 64, start_order=WAVE64, nbr_order=WAVE64)
    assert abs(float(row[3]) - orc.recall_hits(oi, gt, k) / (Q * k)) < 1e-6
    # the same construction from precomputed clusters (--train_gt_file: a ground-truth file of the sampled queries)
    clusters, _ = orc.bruteforce(base, aux, 24, order=SEQ)
    formats.gt_write(work / "clusters.bin", clusters)
    build_cli = os.path.join(root, "coral_amd", "lib", "test_build_pipeline")
    args2 = [build_cli, "--data_type", "float", "--dist", "l2", "--dataset", "syn", "--base_data_path",
             str(work / "base.fbin"), "--sampled_query_data_path", str(work / "aux.fbin"), "--M_pjbp", "16", "--k", "24",
             "--config_file", str(work / "config.json"), "--train_gt_file", str(work / "clusters.bin"), "--index_dir",
             str(work / "from_clusters")]
    r = subprocess.run(args2, cwd=work / "cwd", capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr + r.stdout
    nbrs2, dists2 = formats.graph_dir_read(work / "from_clusters", n, 16, want_dists=True)
    assert np.array_equal(nbrs2, nbrs) and dists2.tobytes() == dists.tobytes()
    assert formats.start_ids_read(work / "from_clusters").tolist() == starts.tolist()
    r = subprocess.run(args2[:-4] + ["--k", "25", "--train_gt_file", str(work / "clusters.bin")], cwd=work / "cwd",
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "expected 25" in r.stderr
    # --CE 0, then --CE 2 (enhancement only) on what it saved: the directory of the --CE 1 run
    staged = ["--index_dir", str(work / "staged")]
    ce_at = build_args.index("--CE") + 1
    for ce in ("0", "2"):
        a = build_args[:ce_at] + [ce] + build_args[ce_at + 1:] + staged
        r = subprocess.run(a, cwd=work / "cwd", capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr + r.stdout
        marks = [l.split("]")[0].split(" ")[0] for l in r.stdout.splitlines() if "Testing recall-" in l]
        assert marks == (["[batches", "[batches"] if ce == "0" else ["[isolated", "[most-hit", "[graph"])
        if ce == "0":
            nbrs0, _ = formats.graph_dir_read(work / "staged", n, 16, want_dists=True)
            assert (nbrs0[:, 0] < 0).sum() > 1000 and not np.array_equal(nbrs0, nbrs)
            hits = formats.hits_read(work / "staged", n)
            assert hits.sum() == A * 24
    nbrs3, dists3 = formats.graph_dir_read(work / "staged", n, 16, want_dists=True)
    assert np.array_equal(nbrs3, nbrs) and dists3.tobytes() == dists.tobytes()
    assert formats.start_ids_read(work / "staged").tolist() == starts.tolist()
    assert np.array_equal(formats.hits_read(work / "staged", n), hits)
    r = subprocess.run(build_args[:ce_at] + ["2"] + build_args[ce_at + 1:] + ["--index_dir", str(work / "nothing_here")],
                       cwd=work / "cwd", capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and "nothing_here" in r.stderr


def test_fewer_reachable_nodes_than_entry_points(orc):
    # one cluster of 5 nodes, no enhancement: the sampling runs out of reachable nodes after 5 ids and repeats
    # itself (as the oracle's does); the index keeps each id once and still searches
    n, dim = 64, 8
    base = synth.gaussian_matrix(3, n, dim)
    p = capi.build_params(R=4, k_b=5, batch=4, connect_enhance=0, n_start=16)
    idx = capi.Index(base, None, None)
    clusters = np.array([[10, 11, 12, 13, 14]], np.int32)
    idx.build_graph_from_clusters(clusters, p)
    nbrs, starts = idx.get_graph()
    want = orc.fps(nbrs, 10, 16)
    assert len(set(want.tolist())) < 16  # repeats in the raw sampling
    assert starts.tolist() == list(dict.fromkeys(want.tolist())) and sorted(starts.tolist()) == [10, 11, 12, 13, 14]
    ids, _, _ = idx.search(base[10:12], 3, 8)
    assert set(ids.ravel().tolist()) <= {10, 11, 12, 13, 14}
    idx.close()
